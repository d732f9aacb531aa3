"""From logits rows to tokens, one kernel launch for the batch."""
from typing import List, Optional, Sequence

import numpy as np
import torch

from .params import SamplingParams


def banned_ngram_tokens(history: Sequence[int], n: int) -> List[int]:
    """The tokens that would, after `history`, complete a run of `n` tokens that `history` already holds
    (reference: sampling.py:267-300; with n = 1 every token seen so far)."""
    if n <= 0 or len(history) + 1 < n:
        return []
    tail = list(history[len(history) - (n - 1):]) if n > 1 else []
    return [history[i + n - 1] for i in range(len(history) - n + 1) if list(history[i:i + n - 1]) == tail]


class Sampler:
    """Greedy rows take the argmax; the others are drawn with their own
    temperature, top-k, top-p and random stream (reference: host loop
    sampling.py:140-157, in-graph form layers/generation.py:137-199)."""

    def __init__(self, ops, device):
        self.ops, self.device = ops, device

    def __call__(self, logits: torch.Tensor, params: List[SamplingParams], draws: List[int],
                 histories: Optional[List[Sequence[int]]] = None) -> List[int]:
        return self.draw(logits, params, draws, histories).tolist()

    def draw(self, logits: torch.Tensor, params: List[SamplingParams], draws: List[int],
             histories: Optional[List[Sequence[int]]] = None) -> torch.Tensor:
        """The chosen tokens, int32 on the logits' device; nothing waits for the device here.
        `draws[i]` is how many tokens request i has drawn before: the counter of its stream.
        `histories[i]`: the tokens request i holds so far, prompt and all (asked for where a request
        has `no_repeat_ngram_size`)."""
        m = logits.shape[0]
        if m != len(params):
            raise ValueError(f"{m} logits rows for {len(params)} requests")
        # (row, token) pairs that get -inf: every end-of-sequence token of a request that has several and must not
        # choose one, and the tokens that would repeat a run of n
        pairs = [(i, t) for i, p in enumerate(params) if p.ban_eos and len(p.eos_ids) > 1 for t in p.eos_ids]
        for i, p in enumerate(params):
            if p.no_repeat_ngram_size:
                if histories is None or histories[i] is None:
                    raise ValueError("no_repeat_ngram_size needs the tokens a request holds so far")
                pairs += [(i, t) for t in banned_ngram_tokens(histories[i], p.no_repeat_ngram_size)]
        if pairs:
            flat = np.array(pairs, dtype=np.int32).T.copy()            # rows, then tokens
            if hasattr(self.ops, "send_ints"):
                dev = self.ops.send_ints(flat.reshape(-1))
            else:
                dev = torch.from_numpy(flat.reshape(-1)).to(self.device)
            self.ops.ban_pairs(logits, dev[:len(pairs)], dev[len(pairs):])
        banned = [p.eos_ids[0] if (p.ban_eos and len(p.eos_ids) == 1) else -1 for p in params]
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
