"""Page and slot allocators: host-side bookkeeping only, no tensors.

The reference has no allocator: block tables and slot mappings come from the
caller (base.py:362-365, :386-398) and `kv_cache_manager.py` only moves whole
caches between devices. These are ours.
"""
from typing import Dict, Hashable, List, Optional


class OutOfPages(RuntimeError):
    """The pool cannot cover the request."""


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class PagePool:
    """A fixed number of pages with a LIFO free list, so that a page given back
    is the next one handed out and reuse shows early. Each page knows its holder;
    handing out a held page, or giving back a page twice or by the wrong holder,
    raises."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._holder: List[Optional[Hashable]] = [None] * num_pages
        self._held: List[bool] = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int, holder: Hashable) -> List[int]:
        """`n` pages for `holder`, all or none."""
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} of {self.num_pages} free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            if self._held[p]:
                raise AssertionError(f"page {p} was on the free list while held by {self._holder[p]!r}")
            self._held[p] = True
            self._holder[p] = holder
        return pages

    def free(self, pages: List[int], holder: Hashable) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page {p} is outside the pool")
            if not self._held[p]:
                raise ValueError(f"page {p} is given back twice")
            if self._holder[p] != holder:
                raise ValueError(f"page {p} is held by {self._holder[p]!r}, not by {holder!r}")
        for p in pages:
            self._held[p] = False
            self._holder[p] = None
            self._free.append(p)

    def holder_of(self, page: int):
        return self._holder[page] if self._held[page] else None

    def check(self) -> None:
        """Every page is either free once or held once."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is on the free list twice")
        on_list = set(free)
        for p in range(self.num_pages):
            if self._held[p] == (p in on_list):
                raise AssertionError(f"page {p} is {'both held and free' if self._held[p] else 'lost'}")


class SlotPool:
    """Slots of fixed-size per-request state; a slot index is stable for the
    request's life."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._holder: Dict[int, Hashable] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, holder: Hashable) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.num_slots} request slots are taken")
        s = self._free.pop()
        self._holder[s] = holder
        return s

    def free(self, slot: int, holder: Hashable) -> None:
        if self._holder.get(slot) != holder:
            raise ValueError(f"slot {slot} is not held by {holder!r}")
        del self._holder[slot]
        self._free.append(slot)
