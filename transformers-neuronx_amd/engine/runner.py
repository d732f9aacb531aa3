"""The step function: one batch of (request, its next tokens) through the model.

`ModelRunner.step` runs only the tokens it is given, as one batch, from the
cache earlier steps left, and returns the logits at the wanted places. Portions
of prompts stand beside single decoded tokens, cut anywhere. Generation, the
trace replay and the measurement all go through it.

Reference: the OPT path takes either whole prompts or single tokens
(base.py:700-710); the mixed form is the reference's chunked-prefill entry
(base.py:384-408, rows picked at cumsum(query_lens) - 1,
layers/transformer.py:311-317), generalised to any wanted places.
"""
from typing import Dict, Hashable, List, Optional

import torch

from ..cache.manager import CacheManager
from .batch import StepContext, StepEntry, build_context
from .model import DecoderModel


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, ops):
        self.model, self.cache, self.ops = model, cache, ops
        self.vocab = model.spec.vocab_size
        self.max_positions = model.spec.max_positions

    def prepare(self, entries: List[StepEntry]) -> StepContext:
        """Admit new requests, get pages for the step's tokens, lay out the batch."""
        seen = set()
        for e in entries:
            if e.req in seen:
                raise ValueError(f"request {e.req!r} appears twice in one step")
            seen.add(e.req)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req!r} brings no tokens")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= self.vocab:
                raise ValueError(f"request {e.req!r}: token id {lo if lo < 0 else hi} is outside the vocabulary "
                                 f"of {self.vocab}")
        for e in entries:
            if not self.cache.has(e.req):
                self.cache.add_request(e.req)
            new_len = self.cache.num_tokens(e.req) + len(e.tokens)
            if new_len > self.max_positions:
                raise ValueError(f"request {e.req!r} would reach {new_len} tokens; the model has "
                                 f"{self.max_positions} positions")
            self.cache.grow(e.req, new_len)
        reqs = [e.req for e in entries]
        cached = [self.cache.num_tokens(r) for r in reqs]
        slots = [self.cache.slot_of(r) for r in reqs]
        tables = {g: self.cache.block_table(reqs, g) for g in self.cache.groups}
        return build_context(entries, cached, slots, tables, self.cache.page_size, self.model.device)

    @torch.no_grad()
    def step(self, entries: List[StepEntry]) -> Optional[torch.Tensor]:
        """Logits float32 `[wanted, vocab]` in the order of the entries and of
        their `want`; None when nothing is wanted (the step still runs)."""
        if not entries:
            return None
        ctx = self.prepare(entries)
        logits = self.model.forward(ctx, self.cache.caches)
        for e in entries:
            self.cache.advance(e.req, len(e.tokens))
        return logits if ctx.logits_rows.numel() else None

    def finish(self, req: Hashable) -> None:
        """The request is over: its pages and its slot go back."""
        if self.cache.has(req):
            self.cache.free_request(req)
