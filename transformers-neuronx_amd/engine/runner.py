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

import numpy as np

from ..cache.manager import CacheManager
from .. import debug
from .batch import PackedStep, StepContext, StepEntry, context_from, pack_step
from .model import DecoderModel
from .snapshot import snapshots_from_environment


class _Staging:
    """Integers from the host to the device without a wait: two pinned buffers in turn, copied by a kernel
    on the current stream. A pageable copy would hold the host until the device has caught up, and with
    it the start of the next step. A buffer is written again only when the copy that read it has run."""

    def __init__(self, ops, size: int = 0):
        self.ops = ops
        self.buffers = [None, None]
        self.done = [None, None]
        self.turn = 0
        if size:
            self.buffers = [ops.pinned_ints(size), ops.pinned_ints(size)]

    def send(self, flat: np.ndarray, dst: Optional[torch.Tensor] = None, device=None) -> torch.Tensor:
        n = flat.size
        self.turn ^= 1
        i = self.turn
        if self.done[i] is not None:
            self.done[i].synchronize()         # also before a buffer is replaced: its copy may still read it
        if self.buffers[i] is None or self.buffers[i][0].numel() < n:
            self.buffers[i] = self.ops.pinned_ints(max(2 * n, 1024))
        self.buffers[i][0].numpy()[:n] = flat
        if dst is None:
            dst = torch.empty(n, dtype=torch.int32, device=device)
        self.ops.copy_ints(dst, self.buffers[i], n)
        if self.done[i] is None:
            self.done[i] = torch.cuda.Event()
        self.done[i].record()
        return dst


class _RecordedStep:
    """A decode step recorded as a HIP graph: the launches of one step over a fixed number of
    one-token runs, reading their integers from a device buffer that is rewritten before each replay.
    The reference keeps one compiled program per (bucket, batch size) and binds its buffers once
    (decoder.py:2099-2325); this is the counterpart without buckets: what varies between steps is data."""

    def __init__(self, runner: "ModelRunner", packed: PackedStep):
        dev = runner.model.device
        self.layout = packed.layout()
        self.staging = _Staging(runner.ops, packed.flat.size)
        self.static = torch.from_numpy(packed.flat).to(dev)
        self.ctx = context_from(packed, self.static)
        self.ctx.length_bound = packed.length_bound
        self.ctx.kept_tokens = runner.kept_tokens
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):           # once in the open: loads libraries, warms the allocator
            runner.model.forward(self.ctx, runner.cache.caches)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        # Every recording of a runner draws on one pool of memory: recordings are replayed one after the other
        # on one stream, so what a step needs in between may lie where another recording's lay; what a
        # recording hands out (its logits) stays its own for as long as it lives.
        with torch.cuda.graph(self.graph, pool=runner.graph_pool()):
            self.logits = runner.model.forward(self.ctx, runner.cache.caches)

    def replay(self, packed: PackedStep) -> torch.Tensor:
        self.staging.send(packed.flat, self.static)
        # what the context says of the step on the host is this step's too (the launches are the recorded ones)
        self.ctx.plan_host = dict(packed.plan_host)
        self.ctx.run_lens_host, self.ctx.cached_lens_host, self.ctx.slots_host = packed.run_lens, packed.cached, packed.slots
        self.graph.replay()
        return self.logits


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager, ops, use_graphs: bool = False):
        self.model, self.cache, self.ops = model, cache, ops
        self.vocab = model.spec.vocab_size
        self.max_positions = model.spec.max_positions
        # decode-only steps are recorded once per batch size and replayed (HIP kernels only)
        self.use_graphs = use_graphs and getattr(ops, "name", "") == "hip" and model.recordable
        self._recorded: Dict[tuple, _RecordedStep] = {}       # in the order of their last use
        self._graph_pool = None
        self._planners = model.step_planners()
        self.graph_replays = 0
        # The token last chosen for the request in each slot, kept on the device: a step may name a token
        # it brings as -1 - slot, and start before the host has read what the step before it chose.
        self.kept_tokens = torch.zeros(cache.max_seqs, dtype=torch.int32, device=model.device)
        self._last_ctx: Optional[StepContext] = None
        self._staging = _Staging(ops) if hasattr(ops, "pinned_ints") else None
        # steps written to a folder for running them again alone (`engine/snapshot.py`); None: none are
        self.snapshots = snapshots_from_environment()

    # The most recordings kept; the one unused longest goes when another is made. A recording is one batch size
    # and one answer of the parts to `launch_shape` (the decode attention's: how many blocks share a request's
    # keys), and holds its own logits, `[batch, vocabulary]` in float32, beside the pool all of them share.
    max_recordings = 48

    def graph_pool(self):
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        return self._graph_pool

    def _recording(self, packed: PackedStep) -> _RecordedStep:
        key = (packed.layout(), self.model.launch_shape(packed))
        rec = self._recorded.pop(key, None)
        if rec is None:
            while len(self._recorded) >= self.max_recordings:
                self._recorded.pop(next(iter(self._recorded)))
            rec = _RecordedStep(self, packed)
        self._recorded[key] = rec          # the newest at the end
        return rec

    def prepare(self, entries: List[StepEntry], fixed_width: bool = False, kept_allowed: bool = False) -> PackedStep:
        """Admit new requests, get pages for the step's tokens, lay out the batch. With `fixed_width`
        the block tables are as wide as the longest request the model allows, so that every step of
        the same batch size has the same layout. With `kept_allowed` a token id -1 - slot stands for the
        token kept on the device for that slot (`keep_tokens`); otherwise every id is a vocabulary entry."""
        lowest = -self.kept_tokens.numel() if kept_allowed else 0
        seen = set()
        for e in entries:
            if e.req in seen:
                raise ValueError(f"request {e.req!r} appears twice in one step")
            seen.add(e.req)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req!r} brings no tokens")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < lowest or hi >= self.vocab:
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
        if fixed_width:
            full = -(-self.max_positions // self.cache.page_size)
            for g, t in tables.items():
                wide = np.full((t.shape[0], full), -1, dtype=np.int32)
                wide[:, :t.shape[1]] = t
                tables[g] = wide
        packed = pack_step(entries, cached, slots, tables, self.cache.page_size, self._planners)
        if fixed_width:
            packed.length_bound = self.max_positions
        return packed

    @torch.no_grad()
    def step(self, entries: List[StepEntry], kept_allowed: bool = False) -> Optional[torch.Tensor]:
        """Logits float32 `[wanted, vocab]` in the order of the entries and of
        their `want`; None when nothing is wanted (the step still runs)."""
        if not entries:
            return None
        taking = self.snapshots is not None and self.snapshots.wanted()
        recordable = (self.use_graphs and not debug.active() and not taking
                      and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))
        packed = self.prepare(entries, fixed_width=recordable, kept_allowed=kept_allowed)
        if taking:
            self.snapshots.enter(self, entries)
        if recordable:
            rec = self._recording(packed)
            logits = rec.replay(packed)
            self._last_ctx = rec.ctx
            self.graph_replays += 1
        else:
            if self._staging is not None:
                ints = self._staging.send(packed.flat, device=self.model.device)
            else:
                ints = torch.from_numpy(packed.flat).to(self.model.device)
            ctx = context_from(packed, ints)
            ctx.kept_tokens = self.kept_tokens
            if taking:
                with debug.debug_context() as taps:
                    logits = self.model.forward(ctx, self.cache.caches)
                self.snapshots.exit(logits if any(len(e.want) for e in entries) else None, taps)
            else:
                logits = self.model.forward(ctx, self.cache.caches)
            self._last_ctx = ctx
        if self.snapshots is not None:
            self.snapshots.iteration += 1
        for e in entries:
            self.cache.advance(e.req, len(e.tokens))
        return logits if any(len(e.want) for e in entries) else None

    def keep_tokens(self, tokens: torch.Tensor):
        """Leave the tokens chosen from the last step's logits (one per wanted row, on the device) where
        the next step finds them, under the slot of each row's request, and send them to the host.
        Returns what `ops.receive_tokens` turns into a list."""
        return self.ops.send_tokens(tokens, self.kept_tokens, self._last_ctx)

    def finish(self, req: Hashable) -> None:
        """The request is over: its pages and its slot go back."""
        if self.cache.has(req):
            self.cache.free_request(req)
