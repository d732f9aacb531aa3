"""A reduced-precision engine against a float32 one on the same weights, at full depth.

Reference: generation_demo.py:405-443 (`analyze`) loads the logits two runs dumped step by step, takes the
last directory as golden, and for every step checks `allclose(atol=1.0, rtol=0.001)` and that both name the
same token (it assumes greedy generation and stops at the first mismatch). `compare_precisions` is that
check for two engines in one process: both generate greedily through `LLMEngine` from the same prompt, the
second one held to the golden run's tokens so that every later row is comparable, and the logits are taken
where the sampler sees them.
"""
from typing import Dict, List, Sequence

import torch

from ..engine.engine import LLMEngine
from ..sampling.params import SamplingParams


def greedy_logits(engine: LLMEngine, prompt: Sequence[int], steps: int, follow: Sequence[int] = ()):
    """Generate `steps` tokens greedily from `prompt` with one request; returns (tokens, float32 logits
    [steps, vocab] on the host). With `follow`, token n is `follow[n]` whatever the logits say: the logits
    are kept as they came, then the followed token's is raised above all others."""
    rows: List[torch.Tensor] = []

    def hook(requests, logits):
        rows.append(logits[:1].float().cpu().clone())        # (on the host `cpu()` copies nothing)
        if follow:
            logits[0, int(follow[len(rows) - 1])] = float("inf")

    before, engine.logits_hook = engine.logits_hook, hook
    try:
        out = engine.generate([list(prompt)], SamplingParams(max_new_tokens=steps, do_sample=False, ignore_eos=True))[0]
    finally:
        engine.logits_hook = before
    return out, torch.cat(rows)


def compare_logits(candidate: torch.Tensor, golden: torch.Tensor) -> Dict[str, float]:
    """The yardstick of generation_demo.py:437-443 over rows of logits, and the plain distance beside it:
    `allclose_rows`   rows that pass allclose(atol=1.0, rtol=0.001)
    `same_argmax`     rows where both name the same token
    `clear_rows`      rows whose golden winner leads by more than twice the row's largest difference: there a
                      different token would be a fault, not a rounding
    `clear_same`      of these, rows where both name the same token
    `max_abs_diff`, `max_logit`, `rel` = their ratio."""
    n = golden.shape[0]
    diff = (candidate - golden).abs()
    row_err = diff.max(dim=-1).values
    top2 = golden.topk(2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * row_err
    same = candidate.argmax(-1) == golden.argmax(-1)
    close = sum(bool(torch.allclose(candidate[i], golden[i], atol=1.0, rtol=0.001)) for i in range(n))
    scale = float(golden.abs().max())
    return {"rows": n, "allclose_rows": int(close), "same_argmax": int(same.sum()), "clear_rows": int(clear.sum()),
            "clear_same": int((same & clear).sum()), "max_abs_diff": float(diff.max()), "max_logit": scale,
            "rel": float(diff.max()) / scale}


def compare_precisions(golden_engine: LLMEngine, engine: LLMEngine, prompt: Sequence[int], steps: int) -> Dict[str, float]:
    """Both engines generate `steps` tokens greedily from `prompt` (one step over the prompt, then single
    tokens); `engine` is held to the golden engine's tokens. Returns `compare_logits` of the two runs."""
    tokens, golden = greedy_logits(golden_engine, prompt, steps)
    _, got = greedy_logits(engine, prompt, steps, follow=tokens)
    return compare_logits(got, golden)
