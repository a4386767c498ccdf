"""The cache manager: pages of what mixers keep per position (keys and values, for attention), with
a block table per request, in groups, and slots of fixed-size state.

reference: one request holds one slot, a whole [layers][max positions][kv width] region
(src/cuda/model.cu:262-275, 615-617); `next_positions[slot]` says where its next token goes
(:550-554); on every way a request ends the slot is reset and given back (app/server.cpp:313-329).
Here a request holds pages instead, as many as its length needs, and a request slot that indexes
the fixed-size state areas.

Groups.  Runs of layers whose caches live equally long (every position kept, or a window of w
positions) form a group.  A group has its own allocator and, per request, its own list of pages:
entry b of the list is the page that holds positions b * page_size ... (b + 1) * page_size - 1.
The page number is shared by all runs of the group: each run has its own pool tensor
[pages, *page shape], indexed by the same page number.  What a page looks like (how many planes,
how many values per position, of which type) is the mixer's `CacheNeed`; how positions and values
lie inside it is the mixer's own business, and nothing here knows of keys or values.  A windowed
group gives a page back as soon as every position on it is out of every later token's window.

Nothing is cleared when pages or slots come back: a kernel reads only rows that were written for
the request that now owns the page, so what an earlier owner left cannot reach a result.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable

import torch

from ..errors import EngineError, ErrorCode, invalid_argument, out_of_bounds, out_of_memory
from ..parts.base import Binding, CacheNeed, StateNeed
from .pages import PageAllocator

ABSENT = -1     # in a request's page list: no page (not yet allocated, or given back by a window)


@dataclass
class RunNeed:
    """What one run of a layer needs of the cache manager."""
    cache_of: int                       # the run whose cache this run reads (itself: it owns one)
    cache: CacheNeed | None = None
    state: StateNeed | None = None


@dataclass
class PageGroup:
    window: int | None
    allocator: PageAllocator
    owners: list[int] = field(default_factory=list)      # runs that own a pool in this group


@dataclass
class RequestPages:
    slot: int
    length: int = 0                                        # positions committed so far
    pages: list[list[int]] = field(default_factory=list)   # per group: block index -> page or ABSENT
    serial: int = 0                                        # which admission this is: no two ever share one


class CacheManager:
    @staticmethod
    def page_bytes(needs: list[RunNeed], page_size: int, dtype: torch.dtype) -> int:
        """Bytes that one more page costs over all runs that own a pool.  `dtype`: the type of
        pools whose need names none."""
        def itemsize(need):
            return torch.empty((), dtype=need.dtype or dtype).element_size()
        return sum(page_size * need.cache.values_per_position() * itemsize(need.cache)
                   for run, need in enumerate(needs) if need.cache is not None and need.cache_of == run)

    def __init__(self, needs: list[RunNeed], page_size: int, num_pages: int, max_requests: int,
                 dtype: torch.dtype, device, max_positions: int | None = None, max_bytes: int | None = None):
        """max_bytes: a budget for the pools; more is refused with `out_of_memory` before anything
        is allocated (src/kv_cache.cpp:40-43)."""
        if page_size <= 0 or page_size & (page_size - 1):
            raise invalid_argument("page_size must be a power of two")
        if max_requests <= 0:
            raise invalid_argument("max_requests must be positive")
        if num_pages <= 0:
            raise invalid_argument("the cache needs at least one page")
        if max_bytes is not None and num_pages * self.page_bytes(needs, page_size, dtype) > max_bytes:
            raise out_of_memory(f"cache pools of {num_pages} pages take {num_pages * self.page_bytes(needs, page_size, dtype)} bytes, "
                                f"which exceeds the configured budget of {max_bytes}")
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = device
        self.max_positions = max_positions
        self.groups: list[PageGroup] = []
        self.bindings: list[Binding] = []
        self._requests: dict[Hashable, RequestPages] = {}
        self._free_slots = list(range(max_requests - 1, -1, -1))   # popped from the end: slot 0 first
        self._slot_in_use = bytearray(max_requests)
        self._admissions = 0
        self.state_areas: list[torch.Tensor] = []

        group_of_window: dict[int | None, int] = {}
        pools: dict[int, torch.Tensor] = {}
        group_of_run: dict[int, int] = {}
        for run, need in enumerate(needs):
            if need.cache is not None and need.cache_of == run:
                if need.cache.window not in group_of_window:
                    group_of_window[need.cache.window] = len(self.groups)
                    self.groups.append(PageGroup(need.cache.window, PageAllocator(num_pages)))
                index = group_of_window[need.cache.window]
                self.groups[index].owners.append(run)
                group_of_run[run] = index
                # zeros once, at creation: positions that were never written then hold finite values
                pools[run] = torch.zeros((num_pages, *need.cache.page_shape(page_size)),
                                         dtype=need.cache.dtype or dtype, device=device)
        for run, need in enumerate(needs):
            binding = Binding()
            if need.cache is not None:
                owner = need.cache_of
                if owner not in pools:
                    raise invalid_argument(f"run {run} reads the cache of run {owner}, which owns none")
                owner_need = needs[owner].cache
                if ((owner_need.planes, owner_need.width, owner_need.dtype)
                        != (need.cache.planes, need.cache.width, need.cache.dtype)):
                    raise invalid_argument(f"run {run} reads the cache of run {owner}, whose pages have another shape")
                binding.group, binding.cache, binding.writes = group_of_run[owner], pools[owner], owner == run
            if need.state is not None:
                area = torch.zeros((max_requests, *need.state.shape), dtype=need.state.dtype, device=device)
                self.state_areas.append(area)
                binding.state = area
            self.bindings.append(binding)

    # ---- requests ------------------------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        """Takes a request slot; the request holds no pages yet.  State rows of the slot start
        at zero."""
        if request in self._requests:
            raise invalid_argument(f"request {request!r} is already live")
        if not self._free_slots:
            raise out_of_memory(f"all {self.max_requests} request slots are in use")
        slot = self._free_slots.pop()
        self._slot_in_use[slot] = 1
        for area in self.state_areas:
            area[slot].zero_()
        self._admissions += 1
        self._requests[request] = RequestPages(slot=slot, pages=[[] for _ in self.groups], serial=self._admissions)
        return slot

    def is_live(self, request: Hashable) -> bool:
        return request in self._requests

    def live_requests(self) -> list:
        return list(self._requests)

    def length(self, request: Hashable) -> int:
        return self._entry(request).length

    def slot(self, request: Hashable) -> int:
        return self._entry(request).slot

    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def _entry(self, request: Hashable) -> RequestPages:
        if request not in self._requests:
            raise invalid_argument(f"request {request!r} is not live")
        return self._requests[request]

    # ---- pages ---------------------------------------------------------------------------
    def _blocks_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def pages_needed(self, request: Hashable, count: int) -> list[int]:
        """Per group, how many new pages `count` more positions of the request take."""
        entry = self._entry(request)
        blocks = self._blocks_for(entry.length + count)
        return [max(0, blocks - len(entry.pages[group])) for group in range(len(self.groups))]

    def free_pages(self) -> list[int]:
        return [group.allocator.num_free for group in self.groups]

    def can_reserve(self, wanted: list[tuple[Hashable, int]]) -> bool:
        """Whether the pools hold enough free pages for all of (request, more positions)."""
        totals = [0] * len(self.groups)
        for request, count in wanted:
            for group, pages in enumerate(self.pages_needed(request, count)):
                totals[group] += pages
        return all(total <= group.allocator.num_free for total, group in zip(totals, self.groups))

    def reserve(self, request: Hashable, count: int) -> None:
        """Allocates the pages that positions length .. length + count - 1 fall on, in every
        group, or none at all (`out_of_memory`)."""
        entry = self._entry(request)
        if count <= 0:
            raise invalid_argument("a request needs at least one new position in a step")
        if self.max_positions is not None and entry.length + count > self.max_positions:
            raise out_of_bounds(f"request {request!r} would reach position {entry.length + count - 1}, "
                                f"past the model's {self.max_positions} positions")
        needed = self.pages_needed(request, count)
        if any(pages > group.allocator.num_free for pages, group in zip(needed, self.groups)):
            raise out_of_memory(f"request {request!r} needs {needed} more pages, free are {self.free_pages()}")
        for group_index, group in enumerate(self.groups):
            entry.pages[group_index].extend(group.allocator.alloc(needed[group_index]))

    def reserve_all(self, wanted: list[tuple[Hashable, int]]) -> bool:
        """`reserve` for every (request, more positions) of a step, or for none of them: False when
        the free pages do not cover them all.  One pass over the requests (a decode step of many
        requests spends its host time here)."""
        groups = range(len(self.groups))
        needs, totals = [], [0] * len(self.groups)
        for request, count in wanted:
            entry = self._entry(request)
            if count <= 0:
                raise invalid_argument("a request needs at least one new position in a step")
            if self.max_positions is not None and entry.length + count > self.max_positions:
                raise out_of_bounds(f"request {request!r} would reach position {entry.length + count - 1}, "
                                    f"past the model's {self.max_positions} positions")
            blocks = (entry.length + count + self.page_size - 1) // self.page_size
            for group in groups:
                more = blocks - len(entry.pages[group])
                if more > 0:
                    needs.append((entry, group, more))
                    totals[group] += more
        if any(total > group.allocator.num_free for total, group in zip(totals, self.groups)):
            return False
        for entry, group, more in needs:
            entry.pages[group].extend(self.groups[group].allocator.alloc(more))
        return True

    def unreserve(self, request: Hashable) -> None:
        """Gives back the pages the request holds beyond those its committed length lies on: what a
        step reserved and then did not run."""
        entry = self._entry(request)
        keep = self._blocks_for(entry.length)
        for group_index, group in enumerate(self.groups):
            pages = entry.pages[group_index]
            spare = [page for page in pages[keep:] if page != ABSENT]
            if spare:
                group.allocator.release(spare)
            del pages[keep:]

    def commit(self, request: Hashable, count: int) -> None:
        """The step that wrote `count` more positions is enqueued: the request is that much
        longer; a windowed group gives back pages that no later token can see."""
        entry = self._entry(request)
        if self._blocks_for(entry.length + count) > min((len(pages) for pages in entry.pages), default=1 << 60):
            raise invalid_argument(f"request {request!r} commits positions it has reserved no pages for")
        entry.length += count
        for group_index, group in enumerate(self.groups):
            if group.window is None:
                continue
            # a later token is at position >= length and sees keys > position - window
            dead_blocks = max(0, (entry.length - group.window + 1)) // self.page_size
            pages = entry.pages[group_index]
            gone = [pages[block] for block in range(min(dead_blocks, len(pages))) if pages[block] != ABSENT]
            if gone:
                group.allocator.release(gone)
                for block in range(min(dead_blocks, len(pages))):
                    pages[block] = ABSENT

    def release(self, request: Hashable) -> None:
        """The request ends: all its pages and its slot come back, uncleared."""
        entry = self._entry(request)
        for group_index, group in enumerate(self.groups):
            group.allocator.release([page for page in entry.pages[group_index] if page != ABSENT])
        if not self._slot_in_use[entry.slot]:
            raise invalid_argument(f"request slot {entry.slot} is freed twice")
        self._slot_in_use[entry.slot] = 0
        self._free_slots.append(entry.slot)
        del self._requests[request]

    def page_list(self, request: Hashable, group: int) -> list[int]:
        return self._entry(request).pages[group]

    def held(self, request: Hashable) -> RequestPages:
        """What the request holds (to read, not to change).  Its page lists only ever grow at the
        end or turn entries ABSENT; `serial` tells one admission of a request name from the next."""
        return self._entry(request)

    def rows(self, request: Hashable, group: int, first: int, count: int) -> list[int]:
        """The cache rows (page * page_size + offset) of positions first .. first + count - 1."""
        pages = self._entry(request).pages[group]
        out = []
        for position in range(first, first + count):
            page = pages[position // self.page_size]
            if page == ABSENT:
                raise EngineError(ErrorCode.OUT_OF_BOUNDS, f"position {position} of request {request!r} has no page")
            out.append(page * self.page_size + position % self.page_size)
        return out

    # ---- bookkeeping checks (used by tests and by debug runs) ----------------------------------
    def check(self) -> None:
        """No page lost, none held twice, none both free and held; the same for slots."""
        for group_index, group in enumerate(self.groups):
            held = [page for entry in self._requests.values() for page in entry.pages[group_index] if page != ABSENT]
            free = group.allocator.free_pages()
            if len(set(held)) != len(held):
                raise AssertionError(f"group {group_index}: a page is held twice")
            if set(held) & set(free):
                raise AssertionError(f"group {group_index}: a page is both held and free")
            if len(held) + len(free) != group.allocator.num_pages or len(set(free)) != len(free):
                raise AssertionError(f"group {group_index}: {group.allocator.num_pages - len(held) - len(free)} pages are lost")
            if any(not group.allocator.in_use(page) for page in held):
                raise AssertionError(f"group {group_index}: a held page is not marked in use")
        slots = [entry.slot for entry in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise AssertionError("a request slot is held twice or both held and free")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise AssertionError("a request slot is lost")
