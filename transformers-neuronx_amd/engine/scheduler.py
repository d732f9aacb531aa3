"""The scheduler: admits requests, cuts prompts into portions under a token
budget, lets running requests decode, finishes them and frees what they hold.

The reference has none: `ContinuousBatchingConfig` (config.py:73-103) declares
capacities for a scheduler outside the repository, and its demo drives a fixed
batch in lock-step (generation_demo.py:474-500). The decisions below are ours.

Every decision is a function of arrival order, lengths and capacities only:
  * each step first gives one token to every running request that is decoding,
    then continues prompts in admission order, then admits waiting requests
    while a slot, pages and budget remain; a portion is what is left of the
    prompt, of the portion limit and of the budget, at least one token;
  * when the pool cannot cover a scheduled token, nothing new is admitted and
    the most recently admitted running request is put back: its pages and slot
    are freed, it rejoins the head of the waiting queue and is computed again
    from its first token later, generated tokens included (they are kept). A
    lone request that does not fit raises `OutOfPages`;
  * a request ends at its end-of-sequence token (unless told to ignore it), at
    `max_new_tokens`, or at the length limit, and frees its pages in that step
    (a `max_time`, the one decision that looks at a clock, ends it at the first
    token that comes too late).

A step's outcome may be recorded in two halves, so that the next step can be planned and started
while the device still works on this one: `record` notes what was computed and puts `PENDING` in
the place of every token that was drawn but not read yet (an end by length is known at once);
`resolve` fills in the tokens when the host has them and ends requests at their end-of-sequence
token. A request that is found to have ended this way may already be part of the step that was
started meanwhile: that run's work is wasted and its token is dropped when it is resolved.
`update` does both at once.
"""
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Hashable, List, Optional

from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages
from ..sampling.params import SamplingParams


PENDING = -1              # stands in `Request.output` for a token that is drawn but not read yet


@dataclass(eq=False)      # a request is itself: lists of requests are searched by identity
class Request:
    req_id: Hashable
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    num_computed: int = 0           # tokens whose keys and values are stored
    finished: bool = False
    finish_reason: Optional[str] = None
    preemptions: int = 0
    arrival: int = 0
    taken_in: float = 0.0           # when the scheduler took it in (time.monotonic), for `max_time`

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    def span(self, start: int, count: int) -> List[int]:
        """Tokens start .. start + count - 1 of prompt and output taken as one sequence."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n:start - n + count]
        if start + count <= n:
            return self.prompt[start:start + count]
        return self.prompt[start:] + self.output[:start + count - n]

    @property
    def decoding(self) -> bool:
        """All tokens but the newest are stored: the next step brings that one token."""
        return len(self.output) > 0 and self.num_computed == self.num_tokens - 1


@dataclass(eq=False)
class ScheduledRun:
    request: Request
    start: int                      # first position of the portion
    count: int                      # tokens in the portion
    samples: bool = False           # the portion ends at the request's newest token: its last logits
                                    # pick the next one
    out_index: int = -1             # where in the request's output that token goes

    def __post_init__(self):
        self.samples = self.start + self.count == self.request.num_tokens


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 max_portion: Optional[int] = None, prompts_first: bool = False):
        self.cache = cache
        self.max_num_seqs = min(max_num_seqs, cache.max_seqs)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_model_len = max_model_len
        self.max_portion = max_portion or max_num_batched_tokens
        # prompts_first: while any prompt is waiting or under way, decoding requests wait (all prompts
        # are taken in before the first decode step); otherwise decoding requests go first every step
        self.prompts_first = prompts_first
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []        # in admission order
        self.finished: List[Request] = []
        self._arrivals = 0
        self.num_preemptions = 0
        self._short = False      # pages have run out and no request has ended since

    # ---------------------------------------------------------------- arrivals

    def add(self, request: Request) -> None:
        """Queue a request; one that can never fit the length limit is refused here
        (reference: opt/model.py:50-57 refuses a sequence longer than the position table)."""
        if not request.prompt:
            raise ValueError(f"request {request.req_id!r} has an empty prompt")
        # the last generated token is never fed back, so it needs no position
        need = len(request.prompt) + request.params.max_new_tokens - 1
        if need > self.max_model_len:
            raise ValueError(f"request {request.req_id!r} needs {need} positions "
                             f"({len(request.prompt)} prompt + {request.params.max_new_tokens} new); "
                             f"the limit is {self.max_model_len}")
        request.arrival = self._arrivals
        request.taken_in = time.monotonic()
        self._arrivals += 1
        self.waiting.append(request)

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def reset(self) -> None:
        """Forget every request and every count (the pages are the cache manager's to give back)."""
        self.waiting.clear()
        self.running.clear()
        self.finished.clear()
        self.num_preemptions = 0
        self._short = False

    # ---------------------------------------------------------------- one step's plan

    def _preempt_last(self, keep: Request) -> bool:
        """Put back the most recently admitted running request other than `keep`."""
        for victim in reversed(self.running):
            if victim is not keep:
                self.running.remove(victim)
                self.cache.free_request(victim.req_id)
                victim.num_computed = 0
                victim.preemptions += 1
                self.num_preemptions += 1
                self.waiting.appendleft(victim)
                return True
        return False

    def _reserve(self, req: Request, new_len: int, planned: List[ScheduledRun]) -> bool:
        """Pages for `req` up to `new_len`, putting later requests back if need be.
        False if `req` itself had to give way."""
        while True:
            try:
                self.cache.grow(req.req_id, new_len)
                return True
            except OutOfPages:
                victim_pool = [r for r in self.running if r is not req]
                if not victim_pool:
                    raise OutOfPages(f"request {req.req_id!r} alone does not fit the page pool "
                                     f"({new_len} tokens wanted)")
                victim = self.running[-1]
                if victim is req:
                    # the newest request gives way to the older ones that are already planned
                    self.running.remove(req)
                    self.cache.free_request(req.req_id)
                    req.num_computed = 0
                    req.preemptions += 1
                    self.num_preemptions += 1
                    self.waiting.appendleft(req)
                    return False
                self._preempt_last(req)
                planned[:] = [p for p in planned if p.request is not victim]

    def _plan_decoding(self, planned: List[ScheduledRun], budget: int, before_all: int) -> tuple:
        """One token for every decoding request, oldest first. Returns (budget left, pages ran out)."""
        blocked = False
        for req in list(self.running):
            if (self.num_preemptions != before_all and req not in self.running) or not req.decoding or budget <= 0:
                continue
            before = self.num_preemptions
            if self._reserve(req, req.num_computed + 1, planned):
                planned.append(ScheduledRun(req, req.num_computed, 1))
                budget -= 1
            blocked |= self.num_preemptions != before
        return budget, blocked

    def schedule(self) -> List[ScheduledRun]:
        budget = self.max_num_batched_tokens
        before_all = self.num_preemptions     # a request can have left `running` only if something was put back
        planned: List[ScheduledRun] = []
        blocked = False                       # pages ran out: admit nothing new this step
        # With `prompts_first` decoding requests wait while a prompt is waiting or under way, but only as
        # long as prompts can get on: once pages have run out (`_short`, until a request ends and frees
        # some) the decoding requests go first again, since only they can end and free pages; and a step
        # in which no prompt could be planned (no slot, no page) is given to them too.
        hold = (self.prompts_first and not self._short
                and (bool(self.waiting) or any(not r.decoding for r in self.running)))
        # 1. one token for every decoding request, oldest first
        if not hold:
            budget, blocked = self._plan_decoding(planned, budget, before_all)
        # 2. the next portion of every prompt under way
        planned_ids = {id(p.request) for p in planned}
        for req in list(self.running):
            if (self.num_preemptions != before_all and req not in self.running) or req.decoding or budget <= 0:
                continue
            if id(req) in planned_ids:
                continue
            count = min(req.num_tokens - req.num_computed, self.max_portion, budget)
            before = self.num_preemptions
            if self._reserve(req, req.num_computed + count, planned):
                planned.append(ScheduledRun(req, req.num_computed, count))
                budget -= count
            blocked |= self.num_preemptions != before
        # 3. admissions, in arrival order, while everything they need is there
        while self.waiting and not blocked and budget > 0 and len(self.running) < self.max_num_seqs:
            req = self.waiting[0]
            count = min(req.num_tokens - req.num_computed, self.max_portion, budget)
            if self.cache.slots.num_free == 0:
                break
            self.cache.add_request(req.req_id)
            if not self.cache.can_grow(req.req_id, req.num_computed + count):
                self.cache.free_request(req.req_id)
                if not self.running:
                    raise OutOfPages(f"request {req.req_id!r} alone does not fit the page pool "
                                     f"({req.num_computed + count} tokens wanted)")
                self._short = True
                break
            self.cache.grow(req.req_id, req.num_computed + count)
            self.waiting.popleft()
            self.running.append(req)
            planned.append(ScheduledRun(req, req.num_computed, count))
            budget -= count
        if self.num_preemptions != before_all:
            self._short = True
        if hold and not planned:
            budget, blocked = self._plan_decoding(planned, budget, before_all)
        # a request put back after it was planned is no longer in `running`
        live = {id(r) for r in self.running}
        return [p for p in planned if id(p.request) in live]

    # ---------------------------------------------------------------- after the step

    def _end(self, req: Request, reason: str, ended: List[Request]) -> None:
        req.finish_reason = reason
        if req.finished:
            return
        req.finished = True
        if req in self.running:
            self.running.remove(req)
        elif req in self.waiting:
            self.waiting.remove(req)
        if self.cache.has(req.req_id):
            self.cache.free_request(req.req_id)
        self._short = False
        self.finished.append(req)
        ended.append(req)

    def abort(self, req: Request) -> None:
        """Take a request out, wherever it stands: it ends with the reason "aborted" and gives back what it
        holds. A token that a step under way is still to deliver for it is dropped when it comes (`resolve`
        finds the request shorter than the place the token was meant for)."""
        if PENDING in req.output:          # also of a request that has ended by its length with its last token under way
            del req.output[req.output.index(PENDING):]
        if not req.finished:
            self._end(req, "aborted", [])

    def record(self, runs: List[ScheduledRun]) -> List[Request]:
        """What the step computes, before its tokens are known: every run that samples gets `PENDING` as
        its request's newest token. Requests that reach `max_new_tokens` or the length limit with it end
        here and free what they hold (their last token is still to be resolved)."""
        ended = []
        for run in runs:
            req = run.request
            req.num_computed = run.start + run.count
            if not run.samples:
                continue
            run.out_index = len(req.output)
            req.output.append(PENDING)
            if len(req.output) >= req.params.max_new_tokens:
                self._end(req, "length", ended)
            elif req.num_tokens > self.max_model_len:
                self._end(req, "model_length", ended)
        return ended

    def resolve(self, runs: List[ScheduledRun], sampled: List[Optional[int]]) -> List[Optional[int]]:
        """The tokens of a recorded step (`sampled[i]` is None for runs that do not sample). Returns, run
        by run, the token that the request keeps, or None: for runs that do not sample and for runs of a
        request that had ended at an earlier token when the step was started."""
        kept: List[Optional[int]] = []
        for run, token in zip(runs, sampled):
            req = run.request
            if not run.samples:
                kept.append(None)
                continue
            if token is None:
                raise ValueError(f"request {req.req_id!r} needs a token this step")
            if run.out_index >= len(req.output):        # the request ended before this token
                kept.append(None)
                continue
            req.output[run.out_index] = int(token)
            kept.append(int(token))
            p = req.params
            if not p.ignore_eos and int(token) in p.eos_ids:
                del req.output[run.out_index + 1:]      # what was drawn after it is dropped
                self._end(req, "eos", [])
            elif p.max_time is not None and time.monotonic() - req.taken_in > p.max_time:
                del req.output[run.out_index + 1:]
                self._end(req, "time", [])
        return kept

    def update(self, runs: List[ScheduledRun], sampled: List[Optional[int]]) -> List[Request]:
        """Record what the step computed and the tokens drawn for the runs that
        sample (`sampled[i]` is None for the others). Returns the requests that ended."""
        before = len(self.finished)
        for run, token in zip(runs, sampled):
            if run.samples and token is None:
                raise ValueError(f"request {run.request.req_id!r} needs a token this step")
        self.record(runs)
        self.resolve(runs, sampled)
        return self.finished[before:]
