"""What one step runs on: the tokens it brings, whose they are, and where their
requests' pages lie.

A step is a concatenation of runs, one run per request: a portion of a prompt
of any length, or a single decoded token. This is the one-dimensional form of
the reference's chunked-prefill entry (base.py:384-408: `query_lens`,
`context_lens`, block tables), with a decoded token as a run of length one.
"""
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch


# What a kernel wants to know about a step beyond its tokens, as int32 arrays that travel in the step's one
# buffer of integers: a planner is `fn(run_lens, cached, page_size) -> ({name: int32 array}, {name: host value})`
# under a name; the arrays of all planners are laid out behind the step's own pieces and reach the kernels as
# `ctx.plan[name]`, the host values as `ctx.plan_host[name]`. A part brings its planners with it
# (`Part.step_planners`, which the model collects and the runner hands to `pack_step`); a planner may also be
# registered here for every step of the process.
_PLANNERS: Dict[str, object] = {}


def register_step_planner(name: str, fn) -> None:
    _PLANNERS[name] = fn


def unregister_step_planner(name: str) -> None:
    _PLANNERS.pop(name, None)


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""
    req: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class GroupView:
    """A page group as a step sees it."""
    block_table: torch.Tensor       # int32 [R, width], -1 where no page is held
    page_size: int
    width: int
    token_page: torch.Tensor = None  # int32 [T], the page each token of the step is stored in
    token_offset: torch.Tensor = None  # int32 [T], and its place inside that page


@dataclass
class StepContext:
    num_tokens: int                 # T
    num_requests: int               # R
    token_ids: torch.Tensor         # int32 [T]
    positions: torch.Tensor         # int32 [T], index of each token in its own request
    token_request: torch.Tensor     # int32 [T], run each token belongs to
    run_start: torch.Tensor         # int32 [R+1], first token of each run
    cached_lens: torch.Tensor       # int32 [R], tokens of each request stored before this step
    slots: torch.Tensor             # int32 [R], state slot of each request
    logits_rows: torch.Tensor       # int32 [M], tokens whose logits are wanted
    groups: Dict[str, GroupView]
    plan: Dict[str, torch.Tensor] = field(default_factory=dict)   # int32 arrays of the registered step planners
    plan_host: Dict[str, object] = field(default_factory=dict)    # and what they say on the host
    # int32 [slots]: the token last chosen for the request in each slot, on the device. A token id -1 - s
    # in `token_ids` stands for `kept_tokens[s]`: a step can be started before the host has read the
    # tokens that the step before it chose.
    kept_tokens: Optional[torch.Tensor] = None
    # When a step is recorded for replay, nothing in its launches may depend on the lengths of this
    # particular step: `length_bound` then stands in for them where a launch is sized.
    length_bound: Optional[int] = None
    # The same on the host, for planning launches and for parts written in Python.
    run_lens_host: np.ndarray = None
    cached_lens_host: np.ndarray = None
    slots_host: np.ndarray = None
    plans: Dict = field(default_factory=dict)    # launch plans the kernel backend keeps per step

    @property
    def max_run(self) -> int:
        return int(self.run_lens_host.max())

    @property
    def max_total(self) -> int:
        return int((self.run_lens_host + self.cached_lens_host).max())


@dataclass
class PackedStep:
    """A step's integers in one host array, and where each piece lies."""
    flat: np.ndarray
    offsets: List[int]
    sizes: List[int]
    num_tokens: int
    num_requests: int
    group_names: List[str]
    widths: Dict[str, int]
    page_size: int
    run_lens: np.ndarray
    cached: np.ndarray
    slots: np.ndarray
    plan_names: List[str]
    plan_host: Dict[str, object]
    # set for a step that is replayed from a recording: what stands in for the requests' lengths where a
    # launch is sized (`StepContext.length_bound`)
    length_bound: Optional[int] = None

    def layout(self):
        """What two steps must share for one to reuse the other's device buffer and views."""
        return (tuple(self.offsets), tuple(self.sizes), self.num_tokens, self.num_requests,
                tuple(self.group_names), tuple(sorted(self.widths.items())), self.page_size)


_FIXED_PIECES = 7    # the step's own pieces, before the planners' and the per-group ones, see pack_step


def pack_step(entries: List[StepEntry], cached: List[int], slots: List[int], tables: Dict[str, np.ndarray],
              page_size: int, planners: Optional[Dict[str, object]] = None) -> PackedStep:
    """`planners`: those of the model's parts; the registered ones are added to them."""
    run_lens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
    cached_np = np.array(cached, dtype=np.int32)
    r, t = len(entries), int(run_lens.sum())
    run_start = np.zeros(r + 1, dtype=np.int32)
    np.cumsum(run_lens, out=run_start[1:])
    token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
    token_request = np.repeat(np.arange(r, dtype=np.int32), run_lens)
    positions = (np.arange(t, dtype=np.int32) - run_start[token_request] + cached_np[token_request]).astype(np.int32)
    rows = []
    for i, e in enumerate(entries):
        for w in e.want:
            if not 0 <= w < len(e.tokens):
                raise ValueError(f"request {e.req!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
            rows.append(run_start[i] + w)
    rows = np.array(rows, dtype=np.int32)
    pieces = [token_ids, positions, token_request, run_start, cached_np, np.array(slots, dtype=np.int32), rows]
    assert len(pieces) == _FIXED_PIECES
    plan_names, plan_host = [], {}
    for planner in {**(planners or {}), **_PLANNERS}.values():
        arrays, host = planner(run_lens, cached_np, page_size)
        for name, array in arrays.items():
            if name in plan_names:
                raise ValueError(f"two step planners name an array {name!r}")
            plan_names.append(name)
            pieces.append(np.ascontiguousarray(array, dtype=np.int32).reshape(-1))
        plan_host.update(host)
    names = list(tables)
    pieces += [tables[g].reshape(-1) for g in names]
    for g in names:
        blocks = positions // page_size
        inside = blocks < tables[g].shape[1]
        pieces.append(np.where(inside, tables[g][token_request, np.minimum(blocks, tables[g].shape[1] - 1)], -1)
                      .astype(np.int32))
    pieces.append((positions % page_size).astype(np.int32))
    # each piece starts at a multiple of 4 integers, so that every view is 16-byte aligned
    offsets, total = [], 0
    for p in pieces:
        offsets.append(total)
        total += -(-p.size // 4) * 4
    flat = np.zeros(max(total, 4), dtype=np.int32)
    for off, p in zip(offsets, pieces):
        flat[off:off + p.size] = p
    return PackedStep(flat, offsets, [p.size for p in pieces], t, r, names,
                      {g: tables[g].shape[1] for g in names}, page_size, run_lens, cached_np,
                      np.array(slots, dtype=np.int32), plan_names, plan_host)


def context_from(packed: PackedStep, dev: torch.Tensor) -> StepContext:
    """Views of the device copy `dev` of a packed step."""
    views = [dev[off:off + n] for off, n in zip(packed.offsets, packed.sizes)]
    groups = {}
    n = len(packed.group_names)
    first = _FIXED_PIECES + len(packed.plan_names)        # the per-group pieces follow the planners'
    for i, g in enumerate(packed.group_names):
        width = packed.widths[g]
        groups[g] = GroupView(views[first + i].view(packed.num_requests, width), packed.page_size, width,
                              token_page=views[first + n + i], token_offset=views[first + 2 * n])
    plan = {name: views[_FIXED_PIECES + i] for i, name in enumerate(packed.plan_names)}
    return StepContext(packed.num_tokens, packed.num_requests, views[0], views[1], views[2], views[3], views[4],
                       views[5], views[6], groups, plan=plan, plan_host=dict(packed.plan_host),
                       run_lens_host=packed.run_lens, cached_lens_host=packed.cached, slots_host=packed.slots)


def build_context(entries: List[StepEntry], cached: List[int], slots: List[int],
                  tables: Dict[str, np.ndarray], page_size: int, device, planners=None) -> StepContext:
    """Pack a step's integers into one buffer, copy it once, and slice it."""
    packed = pack_step(entries, cached, slots, tables, page_size, planners)
    return context_from(packed, torch.from_numpy(packed.flat).to(device))
