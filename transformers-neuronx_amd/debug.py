"""Looking inside a step: intermediate tensors by name, and the time of every kernel.

`tap(name, tensor)` is called by the model at fixed places (after the embedding, after every layer call,
inside the block arrangements); it does nothing unless a `debug_context()` is open, in which case a copy
of the tensor is kept under its name (reference: global_debugger.py:27-92, `tap` and `debug_context`,
where a tapped tensor becomes one more output of the compiled graph; here it is simply copied). A step
that runs inside a debug context or under a kernel timer is never replayed from a recording.

`KernelTimer` brackets every launch of the HIP backend with events (reference: base.py:754-759,
`profile`, which asks its runtime for a trace per compiled kernel).
"""
import contextlib
from collections import OrderedDict
from typing import Dict, List, Optional

import torch

_tapped: Optional["OrderedDict[str, torch.Tensor]"] = None
_timer: Optional["KernelTimer"] = None


def active() -> bool:
    return _tapped is not None or _timer is not None


def tapping() -> bool:
    """A debug context is open: every tapped place needs its tensor as such."""
    return _tapped is not None


def tap(name: str, tensor):
    """Keep a copy of `tensor` under `name` if a debug context is open; returns the tensor."""
    if _tapped is not None and tensor is not None:
        key, n = name, 1
        while key in _tapped:               # a name used again (a later step): numbered
            n += 1
            key = f"{name}#{n}"
        _tapped[key] = tensor.detach().clone()
    return tensor


@contextlib.contextmanager
def debug_context():
    """`with debug_context() as tensors:` runs steps with every tapped tensor kept in `tensors`. Inside another
    one, what is tapped goes to the inner one's `tensors` and, when that closes, to the outer one's as well."""
    global _tapped
    outer, mine = _tapped, OrderedDict()
    _tapped = mine
    try:
        yield mine
    finally:
        _tapped = outer
        for name, tensor in mine.items():
            tap(name.split("#")[0], tensor)


class KernelTimer:
    """Events around every launch; `table()` sums them by kernel name after a synchronize. A launch may say what
    it moves and computes (`bytes`, `flops`: what it has to read and write once, and its multiply-adds times
    two); `work_table()` then gives the rates."""

    def __init__(self):
        self.spans: List[tuple] = []

    def start(self, name: str, bytes: float = 0.0, flops: float = 0.0):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        self.spans.append((name, begin, end, float(bytes), float(flops)))
        return end

    def work_table(self) -> Dict[str, tuple]:
        """{name: (calls, milliseconds, bytes, flops)} by falling time."""
        torch.cuda.synchronize()
        out: Dict[str, list] = {}
        for name, begin, end, nbytes, flops in self.spans:
            row = out.setdefault(name, [0, 0.0, 0.0, 0.0])
            row[0] += 1
            row[1] += begin.elapsed_time(end)
            row[2] += nbytes
            row[3] += flops
        return {k: tuple(v) for k, v in sorted(out.items(), key=lambda kv: -kv[1][1])}

    def table(self) -> Dict[str, tuple]:
        return {k: (v[0], v[1]) for k, v in self.work_table().items()}


def timer() -> Optional[KernelTimer]:
    return _timer


@contextlib.contextmanager
def kernel_timer():
    """`with kernel_timer() as t:` times every launch of the HIP backend; `t.table()` is {name: (calls, ms)}."""
    global _timer
    _timer = KernelTimer()
    try:
        yield _timer
    finally:
        _timer = None
