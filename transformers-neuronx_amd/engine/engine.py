"""The engine: requests in, tokens out. It joins the scheduler, the step
function and the sampler; everything between a request's tokens and its next
token passes through `step()`.
"""
import itertools
import time
from dataclasses import dataclass
from typing import Callable, Dict, Hashable, List, Optional, Sequence

import torch

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import Request, ScheduledRun, Scheduler


@dataclass
class StepOutput:
    req_id: Hashable
    token: int
    finished: bool
    finish_reason: Optional[str]


class LLMEngine:
    def __init__(self, runner: ModelRunner, config: EngineConfig):
        self.runner, self.config = runner, config
        max_len = min(config.max_model_len or runner.max_positions, runner.max_positions)
        self.scheduler = Scheduler(runner.cache, config.max_num_seqs, config.max_num_batched_tokens, max_len,
                                   prompts_first=config.prompts_first)
        self.sampler = Sampler(runner.ops, runner.model.device)
        self.requests: Dict[Hashable, Request] = {}
        self._ids = itertools.count()
        self.timings: List[dict] = []          # one record per step when `record_timings`
        self.record_timings = False
        # called with (requests that sample in this step, their logits [n, vocab] float32) before the draw
        self.logits_hook: Optional[Callable] = None

    # ---------------------------------------------------------------- requests

    def add_request(self, prompt: Sequence[int], params: SamplingParams, req_id: Optional[Hashable] = None):
        if params.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        rid = req_id if req_id is not None else next(self._ids)
        if rid in self.requests and not self.requests[rid].finished:
            raise ValueError(f"request {rid!r} is already live")
        req = Request(rid, [int(t) for t in prompt], params)
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work

    # ---------------------------------------------------------------- one step

    @torch.no_grad()
    def step(self) -> List[StepOutput]:
        """Schedule, run, sample, record: one batch of portions and decoded tokens."""
        runs = self.scheduler.schedule()
        if not runs:
            return []
        t0 = time.perf_counter() if self.record_timings else 0.0
        entries = []
        for run in runs:
            toks = run.request.span(run.start, run.count)
            entries.append(StepEntry(run.request.req_id, toks, [run.count - 1] if run.samples else []))
        logits = self.runner.step(entries)
        sampling = [r for r in runs if r.samples]
        tokens: List[Optional[int]] = [None] * len(runs)
        if sampling:
            if self.logits_hook is not None:
                self.logits_hook([r.request for r in sampling], logits)
            drawn = self.sampler(logits, [r.request.params for r in sampling],
                                 [len(r.request.output) for r in sampling])
            it = iter(drawn)
            tokens = [next(it) if r.samples else None for r in runs]
        self.scheduler.update(runs, tokens)
        if self.record_timings:
            self.runner.ops.synchronize()
            self.timings.append({"seconds": time.perf_counter() - t0, "tokens": sum(r.count for r in runs),
                                 "prefill_tokens": sum(r.count for r in runs if r.count > 1 or not r.samples),
                                 "sampled": len(sampling)})
        return [StepOutput(r.request.req_id, t, r.request.finished, r.request.finish_reason)
                for r, t in zip(runs, tokens) if t is not None]

    def run(self, on_token: Optional[Callable[[StepOutput], None]] = None) -> None:
        """Step until every request has ended."""
        while self.has_work:
            for out in self.step():
                if on_token:
                    on_token(out)

    def generate(self, prompts: Sequence[Sequence[int]], params) -> List[List[int]]:
        """Generated tokens (without the prompts) of a set of prompts; `params` is one
        `SamplingParams` for all or a list with one each."""
        plist = params if isinstance(params, (list, tuple)) else [params] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, plist)]
        self.run()
        return [list(self.requests[i].output) for i in ids]

    def reset(self) -> None:
        """Forget every request and give back all pages (reference: `reset()` zero-fills
        the caches, decoder.py:1957-1969; here nothing needs clearing)."""
        self.scheduler.waiting.clear()
        self.scheduler.running.clear()
        self.runner.cache.reset()
        self.requests.clear()
