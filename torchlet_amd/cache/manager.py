"""The cache manager: pages, block tables and fixed-size state slots.

What it owns
------------
* **Groups of pages.**  Every run of the layer order that owns a per-token cache declares
  a :class:`~torchlet_amd.parts.base.PagedNeed`.  Runs with equal needs (planes, their heads and
  widths, element type, window) form a *group*: one pool of pages, per plane one tensor
  ``[runs, pages, heads, page_size, width]`` and one block table per request.
  A page id addresses every run and plane of its group, so one table row serves them all.  Page 0
  of every group is a sentinel that is never handed out and never written: empty table entries
  point to it.  A group with a window needs fewer pages than one that keeps everything: when the
  most tokens of a step are known its pool is sized for what its requests can hold at once.
* **Block tables.**  Per request and group, the list of pages in logical order.  A group
  with a window gives pages back as soon as every key in them lies behind the window of
  all future queries; their table entries fall back to the sentinel.
* **Slots.**  A request holds one slot from admission to release.  Runs that declare a
  :class:`~torchlet_amd.parts.base.StateNeed` get a tensor ``[slots + 1, *shape]``; a slot's
  rows are zeroed when it is handed out.  The last row (``pad_slot``) belongs to no request: the
  padding rows of a step of fixed shape read and write it.

Free lists are last-in-first-out (as the reference's, /root/reference/src/torchlet/
v10_triton_paged_gqa/kvcache.py:39-66): pages freed by a finished request are the next to
be reused.  Pages are never cleared; stale contents are hidden by lengths and masks.

All bookkeeping is host-side Python and works without a GPU (``device=None`` allocates no
tensors), which is how the manager is tested on the CPU.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..parts.base import PagedNeed, StateNeed


class CacheError(RuntimeError):
    """Misuse of the manager: unknown request, double release, foreign page."""


class OutOfPages(RuntimeError):
    """A reservation cannot be met from the free pages."""


class PagePool:
    """Free list of the pages ``1 .. num_pages-1`` (page 0 is the sentinel)."""

    def __init__(self, num_pages: int):
        if num_pages < 2:
            raise ValueError("a pool needs the sentinel page and at least one more")
        self.num_pages = num_pages
        self._free = list(range(1, num_pages))
        self._is_free = [True] * num_pages
        self._is_free[0] = False

    @property
    def free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages wanted, {len(self._free)} free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._is_free[p] = False
        return pages

    def give(self, pages) -> None:
        for p in pages:
            if not 0 < p < self.num_pages:
                raise CacheError(f"page {p} does not belong to this pool")
            if self._is_free[p]:
                raise CacheError(f"page {p} freed twice")
            self._is_free[p] = True
            self._free.append(p)

    def reset(self) -> None:
        self._free = list(range(1, self.num_pages))
        self._is_free = [True] * self.num_pages
        self._is_free[0] = False


@dataclass
class LayerCache:
    """What one run of the layer order sees of the cache."""
    group: int | None                 # index into StepContext.block_tables
    planes: tuple                     # per plane a tensor [pages, heads, page_size, width]
    page_size: int
    state: torch.Tensor | None        # [slots, *shape] of the run's StateNeed
    writable: bool                    # False: the run reads another run's cache


class _PageTable:
    """The pages of one request in one group, by logical block (0: none): a growing int32
    array, so that a step copies rows into its block tables without touching every entry."""
    __slots__ = ("_pages", "_n")

    def __init__(self):
        self._pages = np.zeros(16, dtype=np.int32)
        self._n = 0

    def __len__(self) -> int:
        return self._n

    def __getitem__(self, b: int) -> int:
        if not 0 <= b < self._n:
            raise IndexError(b)
        return int(self._pages[b])

    def __setitem__(self, b: int, page: int) -> None:
        if not 0 <= b < self._n:
            raise IndexError(b)
        self._pages[b] = page

    def __iter__(self):
        return iter(self._pages[: self._n].tolist())

    def extend(self, pages) -> None:
        need = self._n + len(pages)
        if need > len(self._pages):
            grown = np.zeros(max(need, 2 * len(self._pages)), dtype=np.int32)
            grown[: self._n] = self._pages[: self._n]
            self._pages = grown
        self._pages[self._n: need] = pages
        self._n = need

    def append(self, page: int) -> None:
        self.extend([page])

    def view(self) -> np.ndarray:
        return self._pages[: self._n]


class _Group:
    def __init__(self, need: PagedNeed, num_pages: int):
        self.need = need
        self.runs: list[int] = []                 # indices into the run order, in order
        self.pool = PagePool(num_pages)
        self.tables: dict[object, _PageTable] = {}  # request -> page of each logical block (0: none)
        self.tensors: list[torch.Tensor] = []     # per plane [runs, pages, heads, page_size, width]


class _Request:
    __slots__ = ("slot", "length")

    def __init__(self, slot: int):
        self.slot = slot
        self.length = 0


class CacheManager:
    """``plan``: per run of the layer order ``(paged_need | None, state_need | None, cache_of | None)``.
    ``num_pages``: pages of a group's pool, the sentinel included.  ``max_step_tokens``: the most tokens a
    request brings in one step, if the caller keeps to one (a scheduler's token budget); the pool of a group
    with a window is then no larger than what ``max_requests`` requests can hold of it at once."""

    def __init__(self, plan, *, page_size: int, num_pages: int, max_requests: int,
                 dtype: torch.dtype = torch.float32, device=None, max_step_tokens: int | None = None):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if max_requests <= 0:
            raise ValueError("max_requests must be positive")
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_requests = max_requests
        self.pad_slot = max_requests             # a state row of its own for the padding rows of fixed-shape steps
        self.max_step_tokens = max_step_tokens
        self.dtype = dtype
        self.device = device
        self.groups: list[_Group] = []
        self._run_group: list[int | None] = []
        self._run_index: list[int] = []          # index of the run inside its group's tensor
        self._run_owner: list[int] = []          # run whose cache this run uses
        self._state_needs: list[StateNeed | None] = []
        self._states: list[torch.Tensor | None] = []
        by_need: dict[PagedNeed, int] = {}
        for i, (paged, state, cache_of) in enumerate(plan):
            owner = i if cache_of is None else cache_of
            self._run_owner.append(owner)
            if cache_of is not None:
                self._run_group.append(self._run_group[owner])
                self._run_index.append(self._run_index[owner])
                self._state_needs.append(None)
                continue
            if paged is None:
                self._run_group.append(None)
                self._run_index.append(-1)
            else:
                g = by_need.get(paged)
                if g is None:
                    g = by_need[paged] = len(self.groups)
                    self.groups.append(_Group(paged, self._pool_size(paged)))
                self._run_group.append(g)
                self._run_index.append(len(self.groups[g].runs))
                self.groups[g].runs.append(i)
            self._state_needs.append(state)
        self._requests: dict[object, _Request] = {}
        self._free_slots = list(range(max_requests - 1, -1, -1))
        if device is not None:
            for g in self.groups:
                g.tensors = [torch.zeros((len(g.runs), g.pool.num_pages, heads, page_size, width),
                                         dtype=g.need.dtype or dtype, device=device)
                             for heads, width in g.need.plane_shapes]
            for s in self._state_needs:
                self._states.append(None if s is None else
                                    torch.zeros((max_requests + 1, *s.shape), dtype=s.dtype, device=device))
        else:
            self._states = [None] * len(self._state_needs)

    def _held_at_most(self, need: PagedNeed) -> int | None:
        """Most pages one request can hold in a group with a window when no step brings more than
        ``max_step_tokens`` tokens: the blocks from the first one a query can still read to the last
        one the step writes.  ``None``: no bound (no window, or steps of any size)."""
        if need.window is None or self.max_step_tokens is None:
            return None
        return (need.window + self.max_step_tokens - 2) // self.page_size + 2

    def _pool_size(self, need: PagedNeed) -> int:
        most = self._held_at_most(need)
        if most is None:
            return self.num_pages
        return max(2, min(self.num_pages, self.max_requests * most + 1))

    # ------------------------------------------------------------------ queries
    def bytes_per_page(self) -> int:
        """Bytes that one more page of ``num_pages`` costs (groups whose pools are capped do not grow with it)."""
        total = 0
        for g in self.groups:
            if self._held_at_most(g.need) is not None and g.pool.num_pages < self.num_pages:
                continue
            size = torch.empty((), dtype=g.need.dtype or self.dtype).element_size()
            total += sum(len(g.runs) * heads * self.page_size * width * size for heads, width in g.need.plane_shapes)
        return total

    def capacity(self) -> list[int]:
        """Per group, the pages that can be handed out (the pool without its sentinel)."""
        return [g.pool.num_pages - 1 for g in self.groups]

    def has(self, req_id) -> bool:
        return req_id in self._requests

    def length(self, req_id) -> int:
        return self._req(req_id).length

    def slot(self, req_id) -> int:
        return self._req(req_id).slot

    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self) -> list[int]:
        return [g.pool.free for g in self.groups]

    def live_requests(self) -> list:
        return list(self._requests)

    def _req(self, req_id) -> _Request:
        r = self._requests.get(req_id)
        if r is None:
            raise CacheError(f"request {req_id!r} is not in the cache")
        return r

    def _first_live_block(self, g: _Group, length: int) -> int:
        """First logical block that a query at position >= ``length`` can still read."""
        if g.need.window is None:
            return 0
        return max(0, length - g.need.window + 1) // self.page_size

    def pages_missing(self, req_id, new_length: int) -> list[int]:
        """Per group, the pages that ``reserve(req_id, new_length)`` would take.  (A request's
        table holds pages exactly from the first block a query at its length can still read to
        the table's end: what is missing is counted, not looked for.)"""
        length = self._requests[req_id].length if req_id in self._requests else 0
        blocks = -(-new_length // self.page_size)
        out = []
        for g in self.groups:
            held_to = len(g.tables.get(req_id, ()))
            first = self._first_live_block(g, length)
            out.append(max(0, blocks - max(first, held_to)))
        return out

    def pages_for(self, length: int) -> list[int]:
        """Per group, the most pages a request holds at once on its way to ``length`` tokens."""
        out = []
        for g in self.groups:
            blocks = -(-length // self.page_size)
            most = self._held_at_most(g.need)
            out.append(blocks if most is None else min(blocks, most))
        return out

    # ------------------------------------------------------------------ lifecycle
    def add_request(self, req_id) -> int:
        if req_id in self._requests:
            raise CacheError(f"request {req_id!r} is already in the cache")
        if not self._free_slots:
            raise OutOfPages("no free slot")
        slot = self._free_slots.pop()
        self._requests[req_id] = _Request(slot)
        for g in self.groups:
            g.tables[req_id] = _PageTable()
        for s in self._states:
            if s is not None:
                s[slot].zero_()
        return slot

    def reserve(self, req_id, new_length: int) -> bool:
        """Make sure pages exist for every position below ``new_length`` that a query of the
        coming step can read.  All or nothing over all groups: ``False`` takes no page."""
        r = self._req(req_id)
        if new_length < r.length:
            raise CacheError(f"request {req_id!r} holds {r.length} tokens; cannot shrink to {new_length}")
        missing = self.pages_missing(req_id, new_length)
        if any(m > g.pool.free for m, g in zip(missing, self.groups)):
            return False
        blocks = -(-new_length // self.page_size)
        for g in self.groups:
            table = g.tables[req_id]
            first = self._first_live_block(g, r.length)
            if len(table) < min(first, blocks):         # blocks no query of the step can read: never held
                table.extend([0] * (min(first, blocks) - len(table)))
            if len(table) < blocks:
                table.extend(g.pool.take(blocks - len(table)))
        return True

    def commit(self, req_id, new_length: int) -> None:
        """The request now holds ``new_length`` tokens; pages that no later query can read
        (behind a group's window) go back to their pool."""
        r = self._req(req_id)
        if new_length < r.length:
            raise CacheError(f"request {req_id!r} holds {r.length} tokens; cannot shrink to {new_length}")
        old_length, r.length = r.length, new_length
        for g in self.groups:
            if g.need.window is None:
                continue
            table = g.tables[req_id]
            first = min(self._first_live_block(g, new_length), len(table))
            was_first = min(self._first_live_block(g, old_length), first)     # blocks below were given back earlier
            dead = [b for b in range(was_first, first) if table[b]]
            g.pool.give([table[b] for b in dead])
            for b in dead:
                table[b] = 0

    def release(self, req_id) -> None:
        r = self._requests.pop(req_id, None)
        if r is None:
            raise CacheError(f"request {req_id!r} released twice or never added")
        for g in self.groups:
            g.pool.give([p for p in g.tables.pop(req_id) if p])
        self._free_slots.append(r.slot)

    def reset(self) -> None:
        self._requests.clear()
        self._free_slots = list(range(self.max_requests - 1, -1, -1))
        for g in self.groups:
            g.tables.clear()
            g.pool.reset()

    # ------------------------------------------------------------------ views
    def block_table(self, group: int, req_ids, width: int | None = None) -> np.ndarray:
        """int32 ``[len(req_ids), width]`` rows of the requests' tables, sentinel-padded."""
        g = self.groups[group]
        tables = [g.tables[r] for r in req_ids]
        if width is None:
            width = max([len(t) for t in tables] + [1])
        out = np.zeros((len(tables), width), dtype=np.int32)
        for i, t in enumerate(tables):
            n = min(len(t), width)
            out[i, :n] = t.view()[:n]
        return out

    def layer_cache(self, run: int) -> LayerCache | None:
        """The cache view of entry ``run`` of the layer order."""
        owner = self._run_owner[run]
        gi = self._run_group[owner]
        state = self._states[owner] if self._states else None
        if gi is None and state is None:
            return None
        planes: tuple = ()
        if gi is not None:
            planes = tuple(t[self._run_index[owner]] for t in self.groups[gi].tensors)
        return LayerCache(group=gi, planes=planes, page_size=self.page_size, state=state, writable=(owner == run))

    def check(self) -> None:
        """Invariant: every page of a group is either free or held by exactly one request."""
        for gi, g in enumerate(self.groups):
            held: dict[int, object] = {}
            for req, table in g.tables.items():
                pages = list(table)
                held_from = next((b for b, p in enumerate(pages) if p), len(pages))
                if not all(pages[held_from:]):
                    raise CacheError(f"group {gi}: request {req!r} has a gap among its held pages")
                for p in table:
                    if p == 0:
                        continue
                    if p in held:
                        raise CacheError(f"group {gi}: page {p} held by {held[p]!r} and {req!r}")
                    if g.pool._is_free[p]:
                        raise CacheError(f"group {gi}: page {p} of {req!r} is also on the free list")
                    held[p] = req
            if len(held) + g.pool.free != g.pool.num_pages - 1:
                raise CacheError(f"group {gi}: {g.pool.num_pages - 1 - len(held) - g.pool.free} page(s) lost")
            if len(set(g.pool._free)) != len(g.pool._free):
                raise CacheError(f"group {gi}: a page is on the free list twice")
