"""The cache manager: pages of keys and values with a block table for each request, and
slots for per-request state of fixed size.

A mixer declares what it keeps (`PagedTensors`: tensors per page and a window, or `FixedState`:
tensors per request); the manager allocates what is declared and knows nothing of what the tensors
mean. Mixers are put into *groups* by their declaration: attention layers that keep every key form one
group, those that keep a window of the same length another. Every group has pages of its own: its own
id pool, for each declared tensor a slab `[mixers of the group, pages + 1, *shape of a page]` (the last
page is a sink that is never handed out: padding rows of a captured decode step write there, as in
worker/src/inference/torch_engine.py:439-446) and, for each request, its own block table. A table is addressed by position: entry i holds the page of positions
i*block_size .. (i+1)*block_size - 1, or -1 once a window has passed that page and it
was given back. Pages are handed out when a step needs them (`reserve`), given back when
a request ends (`release`), is preempted (`reset`), or a window has passed them
(`commit`), and are used again with their stale contents, which no kernel may read.

The reference has one group and Python lists of ids on each sequence
(worker/src/inference/kv_cache.py:61-103, worker/src/inference/scheduler.py:50).

Slots: every live request owns one slot id. A mixer that declares `FixedState` gets, for each
tensor it names, a slab `[slots + 1, *shape]`; a request's rows are zeroed when the slot is
taken. The model of this engine has no such mixer, the slots exist all the same.

A layer may hold several mixers (its block says which, by name): `requirements[l]` maps the name of
each mixer of layer l to its declaration, and `layer(l)[name]` is that mixer's view.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import torch

from ..parts.base import FixedState, PagedTensors
from .block_pool import BlockPool, OutOfBlocks

GONE = -1


def pages_needed(token_count: int, block_size: int) -> int:
    """Pages that hold `token_count` tokens: (0,16)=0, (16,16)=1, (17,16)=2
    (worker/src/inference/kv_cache.py:28-33)."""
    if block_size < 1:
        raise ValueError("block_size must be >= 1")
    return -(-max(0, token_count) // block_size)


class CacheView:
    """What one mixer gets: the tensors it declared, by name (`view["k"]`): for paged tensors its own
    layer's slab `[pages + 1, *page shape]` and the index of its group (whose block table and slots of the
    step are `meta.groups[group]`); for fixed state `[slots + 1, *shape]` (rows by `meta.state_slots`)."""

    def __init__(self, group: int = -1, tensors: Optional[Dict[str, torch.Tensor]] = None) -> None:
        self.group = group
        self.tensors = tensors or {}

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.tensors[name]


class LayerCache:
    """The views of one layer's mixers, by the mixer's name in its block."""

    def __init__(self) -> None:
        self.views: Dict[str, CacheView] = {}

    def __getitem__(self, name: str) -> CacheView:
        return self.views[name]


@dataclass
class CacheGroup:
    requirement: PagedTensors
    members: List[tuple]                  # (layer, mixer name) of every mixer that shares these pages
    pool: BlockPool
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)    # name -> [members, pages + 1, *page shape]
    # The block tables as the kernels read them: int32 [slots + 1, width] on the device, row = a request's state
    # slot (the last row belongs to the padding rows of captured steps and names the sink page). It lives from
    # step to step; `changed` holds the entries that the book-keeping has changed since the last step took them
    # along (flat index -> page), so a step costs the same whether its requests hold ten pages or ten thousand.
    table: Optional[torch.Tensor] = None
    changed: Dict[int, int] = field(default_factory=dict)

    @property
    def layers(self) -> List[int]:
        return [layer for layer, _ in self.members]

    @property
    def sink_page(self) -> int:
        return self.pool.num_blocks


@dataclass
class RequestCache:
    slot: int
    num_cached: int = 0
    tables: List[List[int]] = field(default_factory=list)   # per group, by page index
    passed: List[int] = field(default_factory=list)         # per group: entries before this one are all given back


class CacheManager:
    def __init__(self, requirements: Sequence, block_size: int, num_blocks: int, num_slots: int,
                 device=None, dtype=torch.float32, allocate: bool = True) -> None:
        """`requirements[l]`: what the mixers of layer l keep, `{mixer name: PagedTensors | FixedState |
        None}` (a bare declaration stands for `{"mixer": declaration}`). `dtype`: of paged tensors that
        name none. `allocate=False` makes the book-keeping without the slabs (for tests of decisions)."""
        if block_size < 1 or num_blocks < 1 or num_slots < 1:
            raise ValueError("block_size, num_blocks and num_slots must be >= 1")
        self.block_size = int(block_size)
        self.num_blocks = int(num_blocks)
        self.num_slots = int(num_slots)
        self.device = device
        self.dtype = dtype
        self.groups: List[CacheGroup] = []
        self._layers: List[LayerCache] = []
        self._state_slabs: List[torch.Tensor] = []
        by_need: Dict[PagedTensors, CacheGroup] = {}
        for layer, needs in enumerate(requirements):
            if not isinstance(needs, dict):
                needs = {"mixer": needs}
            views = LayerCache()
            self._layers.append(views)
            for name, need in needs.items():
                if isinstance(need, PagedTensors):
                    if need not in by_need:
                        by_need[need] = CacheGroup(need, [], BlockPool(self.num_blocks))
                        self.groups.append(by_need[need])
                    by_need[need].members.append((layer, name))
                elif isinstance(need, FixedState):
                    slabs = {}
                    for decl in need.tensors:
                        if allocate:
                            slabs[decl.name] = torch.zeros((self.num_slots + 1, *decl.shape),
                                                           dtype=decl.dtype or torch.float32, device=device)
                            self._state_slabs.append(slabs[decl.name])
                    views.views[name] = CacheView(tensors=slabs)
                elif need is None:
                    views.views[name] = CacheView()
                else:
                    raise TypeError(f"layer {layer}, {name}: unknown cache requirement {need!r}")
        for index, group in enumerate(self.groups):
            need = group.requirement
            if allocate:
                for decl in need.tensors:
                    shape = (len(group.members), self.num_blocks + 1) + need.page_shape(decl, self.block_size)
                    group.tensors[decl.name] = torch.zeros(shape, dtype=decl.dtype or dtype, device=device)
            for i, (layer, name) in enumerate(group.members):
                self._layers[layer].views[name] = CacheView(
                    group=index, tensors={n: slab[i] for n, slab in group.tensors.items()})
        self.slots = BlockPool(self.num_slots)
        self._requests: Dict[Hashable, RequestCache] = {}
        self.table_width = 0

    @staticmethod
    def page_bytes(requirements: Sequence, block_size: int, dtype=torch.float32) -> int:
        """What one more page costs, over all layers and tensors (each group holds a page of its own for
        every page of the pool)."""
        total = 0
        for needs in requirements:
            for need in (needs.values() if isinstance(needs, dict) else [needs]):
                if isinstance(need, PagedTensors):
                    for decl in need.tensors:
                        count = 1
                        for size in need.page_shape(decl, block_size):
                            count *= size
                        total += count * torch.empty((), dtype=decl.dtype or dtype).element_size()
        return total

    # ---------------------------------------------------------------- block tables on the device
    def bind_tables(self, width: int) -> None:
        """Make the device tables, `width` entries a request (once; the step function's builder calls this with
        the most pages a request can hold)."""
        if self.table_width:
            if width != self.table_width:
                raise ValueError(f"the block tables are {self.table_width} entries wide, not {width}")
            return
        self.table_width = int(width)
        for group in self.groups:
            table = torch.full((self.num_slots + 1, self.table_width), GONE, dtype=torch.int32)
            table[self.sink_slot, :] = group.sink_page       # every position of a padding request lies in the sink page
            group.table = table.to(self.device) if self.device is not None else table
            group.changed.clear()
            # what requests hold already goes along with the next step
            for entry in self._requests.values():
                g = self.groups.index(group)
                for i, page in enumerate(entry.tables[g]):
                    group.changed[entry.slot * self.table_width + i] = page

    def _note(self, group: CacheGroup, slot: int, index: int, page: int) -> None:
        if self.table_width:
            if index >= self.table_width:
                raise ValueError(f"a request would hold more than {self.table_width} pages")
            group.changed[slot * self.table_width + index] = page

    def take_changes(self, g: int):
        """-> (flat indexes, pages) of group g's table entries that changed since the last call, as lists."""
        changed = self.groups[g].changed
        if not changed:
            return (), ()
        out = (list(changed.keys()), list(changed.values()))
        changed.clear()
        return out

    # ---------------------------------------------------------------- views
    def layer(self, layer: int) -> LayerCache:
        return self._layers[layer]

    @property
    def sink_slot(self) -> int:
        return self.num_slots

    def bytes(self) -> int:
        slabs = [t for group in self.groups for t in group.tensors.values()] + self._state_slabs
        return sum(t.numel() * t.element_size() for t in slabs)

    # ------------------------------------------------------------- requests
    def __contains__(self, request_id) -> bool:
        return request_id in self._requests

    def request(self, request_id) -> RequestCache:
        return self._requests[request_id]

    def live(self) -> List[Hashable]:
        return list(self._requests)

    def add(self, request_id) -> RequestCache:
        """Take a state slot for a new request; zero its state rows."""
        if request_id in self._requests:
            raise ValueError(f"request {request_id!r} is already in the cache")
        try:
            (slot,) = self.slots.allocate(1)
        except OutOfBlocks as exc:
            raise OutOfBlocks(f"no free state slot (all {self.num_slots} in use)") from exc
        for slab in self._state_slabs:
            slab[slot].zero_()
        entry = RequestCache(slot=slot, tables=[[] for _ in self.groups], passed=[0 for _ in self.groups])
        self._requests[request_id] = entry
        return entry

    def _first_needed_page(self, group: CacheGroup, num_cached: int) -> int:
        """Index of the first page a query at position >= num_cached can still read."""
        window = group.requirement.window
        if window is None:
            return 0
        return max(0, num_cached - window + 1) // self.block_size

    def pages_short(self, request_id, num_new: int) -> List[int]:
        """Per group: pages that `reserve(request_id, num_new)` would have to take."""
        entry = self._requests.get(request_id)
        cached = entry.num_cached if entry else 0
        out = []
        for g, group in enumerate(self.groups):
            held = len(entry.tables[g]) if entry else 0
            last = pages_needed(cached + num_new, self.block_size)
            first = max(held, self._first_needed_page(group, cached))
            out.append(max(0, last - first))
        return out

    def _holds(self, entry: Optional[RequestCache], num_new: int) -> bool:
        """The request's tables already reach over its next `num_new` positions (most decoded tokens:
        one in `block_size` needs a page)."""
        if entry is None:
            return False
        last = pages_needed(entry.num_cached + num_new, self.block_size)
        for table in entry.tables:
            if len(table) < last:
                return False
        return True

    def can_reserve(self, request_id, num_new: int, spare: int = 0) -> bool:
        if spare <= 0 and self._holds(self._requests.get(request_id), num_new):
            return True
        return all(short + spare <= group.pool.num_free
                   for short, group in zip(self.pages_short(request_id, num_new), self.groups))

    def reserve(self, request_id, num_new: int) -> None:
        """Pages for the next `num_new` positions of the request, in every group; all or
        nothing (OutOfBlocks leaves every pool and table as it was)."""
        if num_new < 1:
            raise ValueError("num_new must be >= 1")
        entry = self._requests[request_id]
        if self._holds(entry, num_new):
            return
        short = self.pages_short(request_id, num_new)
        for need, group in zip(short, self.groups):
            if need > group.pool.num_free:
                raise OutOfBlocks(
                    f"out of blocks: request {request_id!r} needs {need} pages, {group.pool.num_free} free")
        last = pages_needed(entry.num_cached + num_new, self.block_size)
        for g, (need, group) in enumerate(zip(short, self.groups)):
            table = entry.tables[g]
            # pages the window has already passed are never taken
            while len(table) < last - need:
                self._note(group, entry.slot, len(table), GONE)
                table.append(GONE)
                entry.passed[g] = len(table)
            for page in group.pool.allocate(need):
                self._note(group, entry.slot, len(table), page)
                table.append(page)

    def commit(self, request_id, num_new: int) -> None:
        """The step has written `num_new` more tokens; give back what windows have passed."""
        entry = self._requests[request_id]
        entry.num_cached += num_new
        for g, group in enumerate(self.groups):
            if group.requirement.window is None:
                continue
            table = entry.tables[g]
            stop = min(self._first_needed_page(group, entry.num_cached), len(table))
            begin = entry.passed[g]
            if stop > begin:
                passed = [table[i] for i in range(begin, stop) if table[i] != GONE]
                if passed:
                    group.pool.free(passed)
                for i in range(begin, stop):
                    if table[i] != GONE:
                        table[i] = GONE
                        self._note(group, entry.slot, i, GONE)
                entry.passed[g] = stop

    def _give_back_pages(self, entry: RequestCache) -> None:
        for g, group in enumerate(self.groups):
            held = [b for b in entry.tables[g] if b != GONE]
            if held:
                group.pool.free(held)
            entry.tables[g] = []
            entry.passed[g] = 0
        entry.num_cached = 0

    def reset(self, request_id) -> None:
        """Preemption by recompute: every page back, nothing cached, the slot's state zeroed."""
        entry = self._requests[request_id]
        self._give_back_pages(entry)
        for slab in self._state_slabs:
            slab[entry.slot].zero_()

    def release(self, request_id) -> None:
        """The request is over: pages and slot back."""
        entry = self._requests.pop(request_id)
        self._give_back_pages(entry)
        self.slots.free([entry.slot])

    # ------------------------------------------------------------ accounting
    def free_pages(self) -> List[int]:
        return [group.pool.num_free for group in self.groups]

    def max_request_pages(self, num_tokens: int) -> int:
        """Most pages of one group a request of `num_tokens` can hold at once."""
        return pages_needed(num_tokens, self.block_size)

    def check(self) -> None:
        """Invariants, for tests: every page is free or in exactly one table; counts agree."""
        for g, group in enumerate(self.groups):
            seen = set()
            for rid, entry in self._requests.items():
                for page in entry.tables[g]:
                    if page == GONE:
                        continue
                    if page in seen:
                        raise AssertionError(f"page {page} of group {g} is held twice")
                    if not group.pool.is_held(page):
                        raise AssertionError(f"page {page} of group {g} is in a table but free")
                    seen.add(page)
            if len(seen) != group.pool.num_used:
                raise AssertionError(f"group {g}: {group.pool.num_used} pages in use, {len(seen)} in tables (lost pages)")
        slots = [e.slot for e in self._requests.values()]
        if len(set(slots)) != len(slots) or len(slots) != self.slots.num_used:
            raise AssertionError("state slots are held twice or lost")
