"""From logits rows to tokens, one kernel launch for the batch."""
from typing import List

import numpy as np
import torch

from .params import SamplingParams


class Sampler:
    """Greedy rows take the argmax; the others are drawn with their own
    temperature, top-k, top-p and random stream (reference: host loop
    sampling.py:140-157, in-graph form layers/generation.py:137-199)."""

    def __init__(self, ops, device):
        self.ops, self.device = ops, device

    def __call__(self, logits: torch.Tensor, params: List[SamplingParams], draws: List[int]) -> List[int]:
        return self.draw(logits, params, draws).tolist()

    def draw(self, logits: torch.Tensor, params: List[SamplingParams], draws: List[int]) -> torch.Tensor:
        """The chosen tokens, int32 on the logits' device; nothing waits for the device here.
        `draws[i]` is how many tokens request i has drawn before: the counter of its stream."""
        m = logits.shape[0]
        if m != len(params):
            raise ValueError(f"{m} logits rows for {len(params)} requests")
        banned = [p.eos_token_id if (p.ban_eos and p.eos_token_id is not None) else -1 for p in params]
        if any(b >= 0 for b in banned):
            self.ops.ban_tokens(logits, torch.tensor(banned, dtype=torch.int32, device=self.device))
        if all(p.greedy for p in params):
            return self.ops.argmax(logits)
        temp = np.array([0.0 if p.greedy else p.temperature for p in params], dtype=np.float32)
        top_k = np.array([p.top_k for p in params], dtype=np.int32)
        top_p = np.array([p.top_p for p in params], dtype=np.float32)
        seeds = np.array([p.seed for p in params], dtype=np.int64)
        counters = np.array(draws, dtype=np.int64)
        dev = lambda a: torch.from_numpy(a).to(self.device)  # noqa: E731
        return self.ops.sample(logits, dev(temp), dev(top_k), dev(top_p), dev(seeds), dev(counters)).to(self.device)
