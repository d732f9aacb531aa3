"""The cache manager: pages of keys and values with a block table per request,
one set of pages per group of layers with the same needs, and slots of
fixed-size state.

Storage of a paged cache (one set of tensors per cache id, that is per writing
call of the run order): whatever the mixer's `CacheNeed` names, each tensor with
the page number in front and the page size where the need says "page". Attention
keeps keys `[pages, kv_heads, page_size, head_size]` and values
`[pages, kv_heads, head_size, page_size]` (values are kept transposed inside a
page: the kernels contract over the tokens of a page). Caches of one group share
page numbers, so one block table serves all of them. The reference's paged
layout is `[num_blocks, block_size, n_kv_heads, d_head]` (decoder.py:1777-1780)
with `slot = block * block_size + offset` (hlo.py:3665-3704); the slot rule is
kept, the order inside a page is ours.

Pages are not cleared when they change hands: every read is bounded by the
reader's own length.
"""
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional

import numpy as np
import torch

from ..parts.base import CacheNeed
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool


@dataclass
class LayerCache:
    """What one call of the run order is handed."""
    cache_id: int
    group: Optional[str]            # name of the page group (None for state-only caches)
    writes: bool = True
    pages: Dict[str, torch.Tensor] = field(default_factory=dict)   # name -> [pages, *shape with the page size in it]
    state: Dict[str, torch.Tensor] = field(default_factory=dict)   # name -> [slots, *shape]

    @property
    def k_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("k")

    @property
    def v_pages(self) -> Optional[torch.Tensor]:
        return self.pages.get("v")

    def reader(self) -> "LayerCache":
        return LayerCache(self.cache_id, self.group, False, self.pages, self.state)


@dataclass
class PageGroup:
    name: str
    window: Optional[int]
    page_size: int
    pool: PagePool
    cache_ids: List[int]


@dataclass
class RequestPages:
    slot: int
    num_tokens: int = 0                                  # tokens whose keys/values are stored
    tables: Dict[str, List[int]] = field(default_factory=dict)   # group -> page per position block, -1 once released


class CacheManager:
    """Bookkeeping on the host, tensors on the device.

    needs      {cache id: CacheNeed} of the calls that write a cache
    num_pages  pages per group (an int for all groups, or {group name: int})
    """

    def __init__(self, needs: Dict[int, CacheNeed], page_size: int, num_pages, max_seqs: int,
                 dtype: torch.dtype, device, allocate: bool = True, page_pad_bytes: int = 0):
        """`page_pad_bytes`: memory left between one page and the next in every page tensor (a multiple of 32).
        Pages whose size is a power of two lie at distances that are powers of two, and so do the requests
        that fill them side by side: the kernels that read all requests at once then meet the same memory
        channels at the same time. A few hundred bytes between pages take that regularity away."""
        self.page_size, self.max_seqs, self.dtype, self.device = page_size, max_seqs, dtype, device
        if page_pad_bytes < 0 or page_pad_bytes % 32:
            raise ValueError(f"page_pad_bytes must be a multiple of 32 from 0 up, got {page_pad_bytes}")
        self.page_pad_bytes = page_pad_bytes
        self.slots = SlotPool(max_seqs)
        self.groups: Dict[str, PageGroup] = {}
        self.caches: Dict[int, LayerCache] = {}
        self.requests: Dict[Hashable, RequestPages] = {}
        by_key: Dict[tuple, str] = {}
        for cid in sorted(needs):
            need = needs[cid]
            if need is None:
                self.caches[cid] = LayerCache(cid, None)
                continue
            if need.kind == "paged":
                key = need.group_key()
                if key not in by_key:
                    name = "full" if need.window is None else f"window{need.window}"
                    by_key[key] = name
                    n = num_pages[name] if isinstance(num_pages, dict) else num_pages
                    self.groups[name] = PageGroup(name, need.window, page_size, PagePool(n), [])
                g = self.groups[by_key[key]]
                g.cache_ids.append(cid)
                lc = LayerCache(cid, g.name)
                if allocate:
                    item = torch.empty(0, dtype=dtype).element_size()
                    for name, shape in need.tensors_of_a_page():
                        dims = [page_size if d == "page" else d for d in shape]
                        count = int(np.prod(dims))
                        whole = torch.empty(g.pool.num_pages, count + page_pad_bytes // item, dtype=dtype, device=device)
                        lc.pages[name] = whole[:, :count].view(g.pool.num_pages, *dims)
                self.caches[cid] = lc
            elif need.kind == "state":
                lc = LayerCache(cid, None)
                if allocate:
                    sdt = getattr(torch, need.state_dtype)
                    for name, shape in need.state_shapes:
                        lc.state[name] = torch.zeros(max_seqs, *shape, dtype=sdt, device=device)
                self.caches[cid] = lc
            else:
                raise ValueError(f"unknown cache kind {need.kind!r}")

    # ---------------------------------------------------------------- sizes

    @staticmethod
    def bytes_per_page(needs: Dict[int, CacheNeed], page_size: int, dtype: torch.dtype, page_pad_bytes: int = 0) -> int:
        item = torch.empty(0, dtype=dtype).element_size()
        total = 0
        for n in needs.values():
            if n is None or n.kind != "paged":
                continue
            for _, shape in n.tensors_of_a_page():
                count = 1
                for d in shape:
                    count *= page_size if d == "page" else d
                total += count * item + page_pad_bytes
        return total

    # ---------------------------------------------------------------- requests

    def add_request(self, req: Hashable) -> int:
        if req in self.requests:
            raise ValueError(f"request {req!r} is already live")
        slot = self.slots.allocate(req)
        self.requests[req] = RequestPages(slot, 0, {g: [] for g in self.groups})
        for lc in self.caches.values():
            for t in lc.state.values():
                t[slot].zero_()
        return slot

    def has(self, req: Hashable) -> bool:
        return req in self.requests

    def num_tokens(self, req: Hashable) -> int:
        return self.requests[req].num_tokens

    def _blocks_for(self, length: int) -> int:
        return -(-length // self.page_size)

    def pages_short(self, req: Hashable, new_len: int) -> Dict[str, int]:
        """Pages each group still has to hand out before `req` can hold `new_len` tokens."""
        r = self.requests[req]
        return {g: max(0, self._blocks_for(new_len) - len(r.tables[g])) for g in self.groups}

    def can_grow(self, req: Hashable, new_len: int, reserve: Optional[Dict[str, int]] = None) -> bool:
        short = self.pages_short(req, new_len)
        return all(short[g] + (reserve or {}).get(g, 0) <= self.groups[g].pool.num_free for g in self.groups)

    def grow(self, req: Hashable, new_len: int) -> None:
        """Pages for positions up to `new_len`, in every group or in none."""
        r = self.requests[req]
        short = self.pages_short(req, new_len)
        for g, n in short.items():
            if n > self.groups[g].pool.num_free:
                raise OutOfPages(f"group {g}: {n} pages wanted for request {req!r}, "
                                 f"{self.groups[g].pool.num_free} free")
        for g, n in short.items():
            if n:
                r.tables[g].extend(self.groups[g].pool.allocate(n, req))

    def advance(self, req: Hashable, n_tokens: int) -> None:
        """`n_tokens` more are stored. Pages of a windowed group that no later
        query can reach go back to the pool: a query at position p reads keys
        `j > p - window`, and later queries have `p >= num_tokens`."""
        r = self.requests[req]
        r.num_tokens += n_tokens
        if r.num_tokens > len(next(iter(r.tables.values()), [])) * self.page_size and self.groups:
            raise AssertionError(f"request {req!r} advanced past its pages")
        for g in self.groups.values():
            if g.window is None:
                continue
            first_needed = r.num_tokens - g.window + 1
            table = r.tables[g.name]
            gone = [i for i, p in enumerate(table) if p >= 0 and (i + 1) * self.page_size <= first_needed]
            if gone:
                g.pool.free([table[i] for i in gone], req)
                for i in gone:
                    table[i] = -1

    def free_request(self, req: Hashable) -> None:
        r = self.requests.pop(req)
        for g in self.groups.values():
            g.pool.free([p for p in r.tables[g.name] if p >= 0], req)
        self.slots.free(r.slot, req)

    def reset(self) -> None:
        for req in list(self.requests):
            self.free_request(req)

    # ---------------------------------------------------------------- views

    def slot_of(self, req: Hashable) -> int:
        return self.requests[req].slot

    def block_table(self, reqs: List[Hashable], group: str) -> np.ndarray:
        """int32 `[len(reqs), widest]`, -1 where a request holds no page."""
        tables = [self.requests[r].tables[group] for r in reqs]
        width = max(1, max((len(t) for t in tables), default=1))
        out = np.full((len(reqs), width), -1, dtype=np.int32)
        for i, t in enumerate(tables):
            out[i, :len(t)] = t
        return out

    def check(self) -> None:
        """No page lost, none held twice; tables agree with the pools."""
        for g in self.groups.values():
            g.pool.check()
            seen = set()
            for req, r in self.requests.items():
                for p in r.tables[g.name]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"page {p} of group {g.name} is in two tables")
                    seen.add(p)
                    if g.pool.holder_of(p) != req:
                        raise AssertionError(f"page {p} is in {req!r}'s table but held by {g.pool.holder_of(p)!r}")
            if len(seen) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError(f"group {g.name}: {g.pool.num_pages - len(seen) - g.pool.num_free} pages lost")
