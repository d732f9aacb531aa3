"""The reference's host loops by their names, for callers that used them as functions of a model
(sampling.py:26-30 `simple_sample`, :108-128 `sample_greedy`). There the loop lives on the host and calls the
model a token at a time; here the engine runs it, so these hand the model's own `sample` the same arguments.
"""
from typing import List, Optional, Tuple, Union

import torch


def simple_sample(model, input_ids, start_ids, sequence_length, eos_token_id=2, top_k=50, streamer=None,
                  output_scores=False) -> Union[torch.Tensor, Tuple[torch.Tensor, List[torch.Tensor]]]:
    """Top-k sampling at temperature 1 that never picks `eos_token_id` (sampling.py:143-151). With
    `output_scores` also the list of the scores each new token was chosen from, `[batch, vocab]` a step, the
    end-of-sequence token at -inf as the loop leaves it (:147-148)."""
    engine = model._need_engine()
    scores: List[torch.Tensor] = []
    hook = engine.logits_hook
    if output_scores:
        def keep(requests, logits):
            order = sorted(range(len(requests)), key=lambda i: requests[i].req_id)
            kept = logits[order].clone()
            kept[:, eos_token_id] = float("-inf")
            scores.append(kept.cpu())
            if hook is not None:
                hook(requests, logits)
        engine.logits_hook = keep
    try:
        tokens = model.sample(input_ids, sequence_length=sequence_length, start_ids=start_ids, top_k=top_k,
                              streamer=streamer, eos_token_id=eos_token_id)
    finally:
        engine.logits_hook = hook
    return (tokens, scores) if output_scores else tokens


def sample_greedy(model, input_ids, start_ids=None, sequence_length=128) -> torch.Tensor:
    """The largest score each time, nothing banned and nothing that stops it (sampling.py:108-128)."""
    from ..config.engine_config import GenerationConfig
    return model.sample(input_ids, sequence_length=sequence_length, start_ids=start_ids,
                        generation_config=GenerationConfig(do_sample=False, top_k=1, eos_token_id=None))
