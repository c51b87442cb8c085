"""The cache manager: page groups, block tables per request, state slots.

Layers are grouped by what they need to keep.  Layers whose tokens see every
earlier key form one group, layers with a window of W form another; each
group has a pool of pages of its own and, for every live request, one block
table (logical page -> physical page) that all layers of the group share.
Every layer of a group has key and value storage of its own (its layout is the
storage's matter), addressed through the group's table.  A window group gives a page back as soon as every position on it has
left the window of the request's next token.  Mixers with a state of fixed size get a
slot per request instead of pages.

The reference sizes its sliding layers apart from its global ones too
(v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:3532-3563), as a ring of
``window`` slots; pages that are freed behind the window replace the ring
here, which removes the ring's hazard under portions longer than one token
(v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:296-307).
"""

from __future__ import annotations

import dataclasses
from typing import Hashable, Optional, Sequence

from ..parts.base import KVNeed, StateNeed
from .pages import BlockTable, CacheBookkeepingError, OutOfPages, PagePool, StateSlots


def group_name(window: Optional[int]) -> str:
    return "full" if window is None else f"window{window}"


@dataclasses.dataclass
class RequestCache:
    """What one live request holds."""

    request: Hashable
    length: int = 0  # tokens whose keys are in the cache
    slot: int = -1
    tables: dict = dataclasses.field(default_factory=dict)  # group -> BlockTable


def window_pages_bound(window: int, page_size: int, max_step_tokens: int) -> int:
    """The most pages a request ever holds in a group whose layers see a window
    of ``window`` keys, when a step brings it at most ``max_step_tokens``
    tokens: the window behind the step's first token, the step's tokens, and
    one more page because both ends may lie inside a page.  This is what a ring
    of ``window`` slots per request would reserve, in pages that return to the
    pool as the window passes them (the reference sizes its sliding layers as
    ceil(window / block) blocks: v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:3532-3563)."""
    return -(-(window - 1 + max_step_tokens) // page_size) + 1


class PageGroup:
    def __init__(self, name: str, window: Optional[int], page_size: int, num_pages: int):
        self.name = name
        self.window = window
        self.page_size = page_size
        self.pool = PagePool(name, num_pages)
        self.layers: list[int] = []

    def first_kept_page(self, length: int) -> int:
        """Logical index of the first page that a request of ``length`` tokens
        still needs: the next token, at position ``length``, sees the keys from
        ``length - window + 1`` on."""
        if self.window is None:
            return 0
        return max(0, length - self.window + 1) // self.page_size

    def pages_to_add(self, table, new_length: int) -> int:
        need = -(-new_length // self.page_size)
        return max(0, need - len(table))


class Reservation:
    """The pages that the portions planned for a step will take, summed as
    they are planned, so that asking whether one more fits costs that one's
    own count and not everyone's again.  ``fits`` and then ``add`` say what
    ``CacheManager.can_extend`` says for the whole list so far: the pools are
    read as they are when asked, so pages that a set-back request gave back in
    between count as free.  A request that is not live needs a free slot;
    once planned it is expected to be made live at once (its slot then leaves
    the free ones), so only the one asked about can be new."""

    def __init__(self, cache: "CacheManager"):
        self.cache = cache
        self.pages = {name: 0 for name in cache.groups}
        self._asked = None  # (request, new length, its pages): `add` usually follows `fits` for the same

    def _need(self, request: Hashable, new_length: int) -> dict[str, int]:
        if self._asked is None or self._asked[0] != request or self._asked[1] != new_length:
            self._asked = (request, new_length, self.cache.pages_needed(request, new_length))
        return self._asked[2]

    def fits(self, request: Hashable, new_length: int) -> bool:
        cache = self.cache
        if request not in cache.requests and cache.slots.free_count < 1:
            return False
        need = self._need(request, new_length)
        return all(self.pages[name] + n <= cache.groups[name].pool.free_count for name, n in need.items())

    def add(self, request: Hashable, new_length: int) -> None:
        for name, n in self._need(request, new_length).items():
            self.pages[name] += n
        self._asked = None


class CacheManager:
    def __init__(self, needs: Sequence, page_size: int, num_pages, max_requests: int):
        """``needs[i]`` is layer i's need (KVNeed, StateNeed or None).
        ``num_pages`` is an int (every group gets as many) or a dict by group name."""
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.needs = list(needs)
        self.groups: dict[str, PageGroup] = {}
        self.layer_group: list[Optional[str]] = []
        self.state_layers: list[int] = []
        for i, need in enumerate(self.needs):
            if isinstance(need, KVNeed):
                name = group_name(need.window)
                if name not in self.groups:
                    n = num_pages[name] if isinstance(num_pages, dict) else num_pages
                    self.groups[name] = PageGroup(name, need.window, page_size, int(n))
                self.groups[name].layers.append(i)
                self.layer_group.append(name)
            else:
                self.layer_group.append(None)
                if isinstance(need, StateNeed):
                    self.state_layers.append(i)
        self.slots = StateSlots(max_requests)
        self.requests: dict[Hashable, RequestCache] = {}

    # ---- requests ----------------------------------------------------
    def add_request(self, request: Hashable) -> RequestCache:
        if request in self.requests:
            raise KeyError(f"request {request!r} is already live")
        rc = RequestCache(request, 0, self.slots.take(request), {name: BlockTable() for name in self.groups})
        self.requests[request] = rc
        return rc

    def has_request(self, request: Hashable) -> bool:
        return request in self.requests

    def length(self, request: Hashable) -> int:
        return self.requests[request].length

    def pages_needed(self, request: Hashable, new_length: int) -> dict[str, int]:
        """Pages each group must add so that the request can hold ``new_length`` tokens."""
        rc = self.requests.get(request)
        pages = -(-new_length // self.page_size)  # every group has the manager's page size
        if rc is None:
            return {name: pages for name in self.groups}
        out = {}
        for name, table in rc.tables.items():
            more = pages - len(table)
            out[name] = more if more > 0 else 0
        return out

    def require(self, wanted: Sequence[tuple[Hashable, int]]) -> None:
        """Raises OutOfPages unless all of ``(request, new_length)`` fit at
        once.  A request not yet live counts from an empty table and needs a
        free slot.  Takes nothing."""
        total = {name: 0 for name in self.groups}
        new_requests = 0
        for request, new_length in wanted:
            if request not in self.requests:
                new_requests += 1
            for name, n in self.pages_needed(request, new_length).items():
                total[name] += n
        if new_requests > self.slots.free_count:
            raise OutOfPages("state slots", new_requests, self.slots.free_count)
        for name, g in self.groups.items():
            if total[name] > g.pool.free_count:
                raise OutOfPages(name, total[name], g.pool.free_count)

    def can_extend(self, wanted: Sequence[tuple[Hashable, int]]) -> bool:
        try:
            self.require(wanted)
        except OutOfPages:
            return False
        return True

    def reservation(self) -> "Reservation":
        """An empty tally of what a step's planned portions will take."""
        return Reservation(self)

    def extend(self, request: Hashable, new_length: int) -> None:
        """Give the request pages for the positions up to ``new_length``
        (exclusive).  All groups or none: raises OutOfPages with nothing taken."""
        rc = self.requests[request]
        if new_length < rc.length:
            raise ValueError(f"request {request!r} holds {rc.length} tokens, cannot extend to {new_length}")
        need = self.pages_needed(request, new_length)
        for name, n in need.items():
            if n > self.groups[name].pool.free_count:
                raise OutOfPages(name, n, self.groups[name].pool.free_count)
        for name, n in need.items():
            if n:
                rc.tables[name].extend(self.groups[name].pool.take(request, n))

    def extend_all(self, wanted: Sequence[tuple[Hashable, int]]) -> None:
        """``extend`` for every (live request, new length) of a step: all of
        them get their pages or, with OutOfPages, none does."""
        needs = []
        total = {name: 0 for name in self.groups}
        for request, new_length in wanted:
            rc = self.requests[request]
            if new_length < rc.length:
                raise ValueError(f"request {request!r} holds {rc.length} tokens, cannot extend to {new_length}")
            need = self.pages_needed(request, new_length)
            needs.append((rc, need))
            for name, n in need.items():
                total[name] += n
        for name, g in self.groups.items():
            if total[name] > g.pool.free_count:
                raise OutOfPages(name, total[name], g.pool.free_count)
        for rc, need in needs:
            for name, n in need.items():
                if n:
                    rc.tables[name].extend(self.groups[name].pool.take(rc.request, n))

    def adopt_length_for_measurement(self, request: Hashable, length: int) -> None:
        """Make a fresh request hold ``length`` tokens without running them:
        it gets exactly the pages a request of that length holds (none behind
        a window).  For measurements on a cache filled by hand."""
        rc = self.requests[request]
        if rc.length != 0 or any(len(rc.tables[name]) for name in self.groups):
            raise ValueError("only a fresh request can adopt a length")
        plan = {}
        for name, g in self.groups.items():
            first = g.first_kept_page(length)
            count = -(-length // g.page_size) - first
            if count > g.pool.free_count:
                raise OutOfPages(name, count, g.pool.free_count)
            plan[name] = (first, count)
        for name, (first, count) in plan.items():
            rc.tables[name] = BlockTable([-1] * first + self.groups[name].pool.take(request, count), passed=first)
        rc.length = length

    def commit(self, request: Hashable, new_length: int) -> None:
        """The step that wrote the positions up to ``new_length`` is done:
        record the length and give back the pages the window has passed."""
        rc = self.requests[request]
        if new_length < rc.length:
            raise ValueError("a request's length cannot shrink")
        for name, g in self.groups.items():
            if -(-new_length // g.page_size) > len(rc.tables[name]):
                raise CacheBookkeepingError(f"request {request!r} committed {new_length} tokens without pages for them")
        rc.length = new_length
        for name, g in self.groups.items():
            passed = rc.tables[name].pass_up_to(g.first_kept_page(new_length))
            if passed:
                g.pool.give_back(request, passed)

    def release(self, request: Hashable) -> None:
        """The request is finished (or set back): everything it holds returns."""
        rc = self.requests.pop(request)
        for name, g in self.groups.items():
            g.pool.give_back(request, rc.tables[name].held())
        self.slots.give_back(request, rc.slot)

    # ---- reading -----------------------------------------------------
    def table(self, request: Hashable, group: str) -> BlockTable:
        return self.requests[request].tables[group]

    def slot(self, request: Hashable) -> int:
        return self.requests[request].slot

    def free_pages(self) -> dict[str, int]:
        return {name: g.pool.free_count for name, g in self.groups.items()}

    def check(self) -> None:
        """The books add up: every page free or owned once, every owned page
        in exactly one table of its owner."""
        for name, g in self.groups.items():
            g.pool.check()
            seen: dict[int, Hashable] = {}
            for rc in self.requests.values():
                for p in rc.tables[name]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise CacheBookkeepingError(f"{name}: page {p} in the tables of {seen[p]!r} and {rc.request!r}")
                    seen[p] = rc.request
                    if g.pool.owner_of(p) != rc.request:
                        raise CacheBookkeepingError(f"{name}: page {p} in the table of {rc.request!r} but owned by "
                                                    f"{g.pool.owner_of(p)!r}")
            if len(seen) != g.pool.num_pages - g.pool.free_count:
                raise CacheBookkeepingError(f"{name}: {g.pool.num_pages - g.pool.free_count - len(seen)} owned page(s) "
                                            "in no table")
        self.slots.check()
