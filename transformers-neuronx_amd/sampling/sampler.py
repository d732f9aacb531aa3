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
            if hasattr(self.ops, "send_ints"):
                self.ops.ban_tokens(logits, self.ops.send_ints(np.array(banned, dtype=np.int32)))
            else:
                self.ops.ban_tokens(logits, torch.tensor(banned, dtype=torch.int32, device=self.device))
        if all(p.greedy for p in params):
            return self.ops.argmax(logits)
        temp = np.array([0.0 if p.greedy else p.temperature for p in params], dtype=np.float32)
        top_k = np.array([p.top_k for p in params], dtype=np.int32)
        top_p = np.array([p.top_p for p in params], dtype=np.float32)
        seeds = np.array([p.seed or 0 for p in params], dtype=np.int64)
        counters = np.array([-1 if p.deterministic else n for p, n in zip(params, draws)], dtype=np.int64)
        least = np.array([p.min_tokens_to_keep for p in params], dtype=np.int32)
        if hasattr(self.ops, "send_ints"):
            # one block of integers through pinned memory: nothing here waits for the device
            m2 = m + (m & 1)                                  # the 64-bit pieces start at even places
            flat = np.zeros(3 * m2 + 5 * m, dtype=np.int32)
            flat[0:m] = temp.view(np.int32)
            flat[m2:m2 + m] = top_k
            flat[2 * m2:2 * m2 + m] = top_p.view(np.int32)
            flat[3 * m2:3 * m2 + 2 * m] = seeds.view(np.int32)
            flat[3 * m2 + 2 * m:3 * m2 + 4 * m] = counters.view(np.int32)
            flat[3 * m2 + 4 * m:] = least
            dev = self.ops.send_ints(flat)
            return self.ops.sample(logits, dev[0:m].view(torch.float32), dev[m2:m2 + m],
                                   dev[2 * m2:2 * m2 + m].view(torch.float32),
                                   dev[3 * m2:3 * m2 + 2 * m].view(torch.int64),
                                   dev[3 * m2 + 2 * m:3 * m2 + 4 * m].view(torch.int64), dev[3 * m2 + 4 * m:])
        dev = lambda a: torch.from_numpy(a).to(self.device)  # noqa: E731
        return self.ops.sample(logits, dev(temp), dev(top_k), dev(top_p), dev(seeds), dev(counters),
                               dev(least)).to(self.device)
