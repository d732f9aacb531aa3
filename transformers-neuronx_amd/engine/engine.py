"""The engine: requests in, tokens out. It joins the scheduler, the step
function and the sampler; everything between a request's tokens and its next
token passes through `step()`.
"""
import dataclasses
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
from .scheduler import PENDING, Request, ScheduledRun, Scheduler


@dataclass
class StepOutput:
    req_id: Hashable
    token: int
    finished: bool
    finish_reason: Optional[str]


@dataclass
class _StartedStep:
    """A step whose tokens are chosen on the device and not read yet."""
    runs: List[ScheduledRun]
    sampling: List[ScheduledRun]
    sent: object                         # the tokens on their way to the host (`ops.send_tokens`)
    started: float


class LLMEngine:
    """With `run_ahead` (the default) a call of `step()` starts one step and returns the tokens of the
    step before it: the device chooses a step's tokens and keeps them where the next step's embedding
    finds them, so the host can plan, lay out and start that next step while the device still works,
    and reads the tokens only afterwards. What a request generates is the same either way; a request
    that ends at its end-of-sequence token is found out one step late, and the run it has in the step
    started meanwhile is wasted and dropped."""

    def __init__(self, runner: ModelRunner, config: EngineConfig):
        self.runner, self.config = runner, config
        max_len = min(config.max_model_len or runner.max_positions, runner.max_positions)
        self.scheduler = Scheduler(runner.cache, config.max_num_seqs, config.max_num_batched_tokens, max_len,
                                   max_portion=config.chunk_size, prompts_first=config.prompts_first)
        self.sampler = Sampler(runner.ops, runner.model.device)
        self.requests: Dict[Hashable, Request] = {}
        self._ids = itertools.count()
        self._taken = 0                        # requests taken since the start or the last reset
        self.timings: List[dict] = []          # one record per step when `record_timings`
        self.record_timings = False
        # called with (requests that sample in this step, their logits [n, vocab] float32) before the draw
        self.logits_hook: Optional[Callable] = None
        self.run_ahead = bool(getattr(config, "run_ahead", True))
        self._started: Optional[_StartedStep] = None
        self._planned = False                  # the last call of `step()` found something to run

    # ---------------------------------------------------------------- requests

    def add_request(self, prompt: Sequence[int], params: SamplingParams, req_id: Optional[Hashable] = None):
        if params.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        rid = req_id if req_id is not None else next(self._ids)
        if rid in self.requests and not self.requests[rid].finished:
            raise ValueError(f"request {rid!r} is already live")
        prompt = [int(t) for t in prompt]
        if prompt and not 0 <= min(prompt) <= max(prompt) < self.runner.vocab:
            raise ValueError(f"request {rid!r}: a token id of the prompt is outside the vocabulary of {self.runner.vocab}")
        if params.seed is None:
            # a stream of the request's own, the same whatever else runs beside it
            params = dataclasses.replace(params, seed=int(self.config.seed) + self._taken)
        self._taken += 1
        req = Request(rid, prompt, params)
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    @property
    def has_work(self) -> bool:
        return self.scheduler.has_work or self._started is not None

    # ---------------------------------------------------------------- one step

    def _start(self) -> Optional[_StartedStep]:
        """Plan a step, run it, choose its tokens on the device and record it with the tokens pending."""
        runs = self.scheduler.schedule()
        self._planned = bool(runs)
        if not runs:
            return None
        t0 = time.perf_counter()
        entries = []
        for run in runs:
            toks = run.request.span(run.start, run.count)
            if toks[-1] == PENDING:
                # drawn by the step before this one and not read yet: the device has it under the slot
                toks = toks[:-1] + [-1 - self.runner.cache.slot_of(run.request.req_id)]
            entries.append(StepEntry(run.request.req_id, toks, [run.count - 1] if run.samples else []))
        logits = self.runner.step(entries, kept_allowed=True)
        sampling = [r for r in runs if r.samples]
        sent = None
        if sampling:
            requests = [r.request for r in sampling]
            if self.logits_hook is not None:
                self.logits_hook(requests, logits)
            histories = None
            if any(q.params.no_repeat_ngram_size for q in requests):
                # (such requests never run ahead, see `step`: every token they hold is known here)
                histories = [list(q.prompt) + list(q.output) if q.params.no_repeat_ngram_size else None
                             for q in requests]
            drawn = self.sampler.draw(logits, [q.params for q in requests], [len(q.output) for q in requests],
                                      histories)
            sent = self.runner.keep_tokens(drawn)
        self.scheduler.record(runs)
        return _StartedStep(runs, sampling, sent, t0)

    def _finish(self, step: _StartedStep) -> List[StepOutput]:
        """Read the tokens of a started step and give them to their requests."""
        tokens: List[Optional[int]] = [None] * len(step.runs)
        if step.sampling:
            it = iter(self.runner.ops.receive_tokens(step.sent))
            tokens = [next(it) if r.samples else None for r in step.runs]
        kept = self.scheduler.resolve(step.runs, tokens)
        self.scheduler.finished.clear()        # the engine reports ends through `StepOutput`; nothing piles up
        if self.record_timings:
            self.runner.ops.synchronize()
            self.timings.append({"seconds": time.perf_counter() - step.started,
                                 "tokens": sum(r.count for r in step.runs),
                                 "prefill_tokens": sum(r.count for r in step.runs if r.count > 1 or not r.samples),
                                 "sampled": len(step.sampling)})
        out = []
        for r, t in zip(step.runs, kept):
            if t is not None:
                q = r.request
                last = q.finished and r.out_index == len(q.output) - 1
                out.append(StepOutput(q.req_id, t, last, q.finish_reason if last else None))
        return out

    @torch.no_grad()
    def step(self) -> List[StepOutput]:
        """Schedule, run, sample, record: one batch of portions and decoded tokens. Returns the tokens of
        the step it ran, or with `run_ahead` those of the step started by the call before."""
        # a request that may not repeat its n-grams needs its last token on the host before the next is chosen
        in_step = any(q.params.no_repeat_ngram_size and not q.finished for q in self.requests.values())
        idle = self._started is None
        if not self.run_ahead or self.record_timings or in_step:
            out = self._finish(self._started) if self._started is not None else []
            self._started = None
            started = self._start()
            self._check_progress(idle)
            return out + (self._finish(started) if started is not None else [])
        started = self._start()
        out = self._finish(self._started) if self._started is not None else []
        self._started = started
        self._check_progress(idle)
        return out

    def _check_progress(self, idle: bool) -> None:
        """Requests wait, no step was under way when this call began and the scheduler has planned none: no
        later call would do better (a pool too small for a lone request raises `OutOfPages` where it is
        found; this is what is left, and every loop over `step()` meets it)."""
        if idle and not self._planned and self.scheduler.has_work:
            raise RuntimeError("no progress: requests wait, the scheduler plans no step and none is under way")

    def profile(self, steps: int = 1, work: bool = False):
        """Run `steps` steps with events around every kernel launch (no recording, no running ahead) and
        return ({kernel: (launches, milliseconds)}, the steps' outputs); with `work` the table's entries are
        (launches, milliseconds, bytes, flops), with what the launches said they move and compute, and its
        names carry their sizes. Reference: `profile`, base.py:754-759."""
        from .. import debug
        ahead, self.run_ahead = self.run_ahead, False
        outs: List[StepOutput] = []
        try:
            with debug.kernel_timer() as t:
                for _ in range(steps):
                    if not self.has_work:
                        break
                    outs += self.step()
                table = t.work_table() if work else t.table()
        finally:
            self.run_ahead = ahead
        return table, outs

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
        return [list(self.pop_request(i).output) for i in ids]

    def abort_request(self, req_id: Hashable) -> Request:
        """Stop a request whose caller has gone, between two calls of `step()`: its pages and its slot are
        free for the next step, no further token of it is reported (one that a step already started would
        still deliver is dropped), and the request is handed over with what it has generated so far."""
        req = self.requests[req_id]
        self.scheduler.abort(req)
        self.scheduler.finished.clear()
        return self.requests.pop(req_id)

    def pop_request(self, req_id: Hashable) -> Request:
        """Hand over a request that has ended and forget it. A request stays in `requests`, with its prompt
        and output, until this is called (or `reset`): a caller that drives `step()` itself calls it when it
        has seen the request's last token."""
        req = self.requests[req_id]
        if not req.finished:
            raise ValueError(f"request {req_id!r} has not ended")
        if PENDING in req.output:
            raise ValueError(f"request {req_id!r} has ended, but its last token is in a step under way: "
                             "the next call of step() delivers it")
        return self.requests.pop(req_id)

    def reset(self) -> None:
        """Forget every request and give back all pages (reference: `reset()` zero-fills
        the caches, decoder.py:1957-1969; here nothing needs clearing)."""
        self._started = None
        self.scheduler.reset()
        self.runner.cache.reset()
        self._taken = 0
        self.requests.clear()
