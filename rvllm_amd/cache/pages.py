"""Page pools, block tables and state slots: the bookkeeping of the cache.

Nothing here touches the GPU.  A pool hands out page numbers and takes them
back; it knows the owner of every page, so a page can neither be handed out
twice nor given back twice.  The reference declares the pieces (``BlockId``:
v3/crates/rvllm-core/src/ids.rs:41-44; ``KvExhausted``:
v3/crates/rvllm-core/src/error.rs:243) but gives every sequence a fixed range
of blocks (v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:3652-3656,1803-1808);
the allocator is this engine's own.
"""

from __future__ import annotations

from typing import Hashable, Iterable, Optional

import numpy as np


class OutOfPages(RuntimeError):
    """A pool cannot give as many pages as were asked for."""

    def __init__(self, group: str, wanted: int, free: int):
        self.group, self.wanted, self.free = group, wanted, free
        super().__init__(f"page group {group!r}: {wanted} page(s) wanted, {free} free")


class CacheBookkeepingError(AssertionError):
    """The cache's books do not add up: a page freed twice, or not owned."""


class PagePool:
    """``num_pages`` pages, handed out most-recently-freed first, so that a
    page that was just given back is the next to be used again."""

    def __init__(self, name: str, num_pages: int):
        if num_pages < 1:
            raise ValueError(f"page group {name!r} needs at least one page")
        self.name = name
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))  # pop() gives page 0 first
        self._owner: dict[int, Hashable] = {}
        self._held: dict[Hashable, int] = {}  # pages each owner holds now
        self.most_held_by_one = 0  # the most pages any one owner has held at a time
        # With ``keep_history`` every page remembers its owners in order (tests ask whether pages changed hands).
        self.keep_history = False
        self.history: dict[int, list[Hashable]] = {}

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, owner: Hashable, count: int) -> list[int]:
        if count > len(self._free):
            raise OutOfPages(self.name, count, len(self._free))
        pages = [self._free.pop() for _ in range(count)]
        for p in pages:
            if p in self._owner:
                raise CacheBookkeepingError(f"page {p} of {self.name!r} handed out while owned by {self._owner[p]!r}")
            self._owner[p] = owner
            if self.keep_history:
                self.history.setdefault(p, []).append(owner)
        if count:
            held = self._held.get(owner, 0) + count
            self._held[owner] = held
            if held > self.most_held_by_one:
                self.most_held_by_one = held
        return pages

    def give_back(self, owner: Hashable, pages) -> None:
        count = 0
        for p in pages:
            if self._owner.get(p, _NOBODY) != owner:
                raise CacheBookkeepingError(
                    f"page {p} of {self.name!r} given back by {owner!r} but owned by {self._owner.get(p, 'nobody')!r}")
            del self._owner[p]
            self._free.append(p)
            count += 1
        if count:
            left = self._held[owner] - count
            if left:
                self._held[owner] = left
            else:
                del self._held[owner]

    def held_by(self, owner: Hashable) -> int:
        return self._held.get(owner, 0)

    def owner_of(self, page: int) -> Optional[Hashable]:
        return self._owner.get(page)

    def check(self) -> None:
        """Every page is either free or owned, once."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheBookkeepingError(f"{self.name!r}: a page is on the free list twice")
        if free & set(self._owner):
            raise CacheBookkeepingError(f"{self.name!r}: a page is free and owned")
        if len(free) + len(self._owner) != self.num_pages:
            raise CacheBookkeepingError(f"{self.name!r}: {self.num_pages - len(free) - len(self._owner)} page(s) lost")
        if sum(self._held.values()) != len(self._owner):
            raise CacheBookkeepingError(f"{self.name!r}: the owners' counts do not add up to the pages owned")


_NOBODY = object()


class BlockTable:
    """A request's pages in one group by logical index, -1 where it holds none.

    Kept as an array that grows by doubling, so that a step copies a table of
    thousands of pages into its staging buffer as one block; ``passed`` is the
    number of leading entries that a window has already given back, so that
    giving back looks only at what is new.  Reads like a list."""

    def __init__(self, pages: Iterable[int] = (), passed: int = 0):
        pages = list(pages)
        self._pages = np.full(max(16, len(pages)), -1, dtype=np.int32)
        self._pages[: len(pages)] = pages
        self._n = len(pages)
        self.passed = passed

    def __len__(self) -> int:
        return self._n

    def __array__(self, dtype=None, copy=None):
        view = self._pages[: self._n]
        return view if dtype is None or dtype == view.dtype else view.astype(dtype)

    def view(self) -> np.ndarray:
        """The entries, writable, valid until the table grows."""
        return self._pages[: self._n]

    def __iter__(self):
        return iter(self._pages[: self._n].tolist())

    def __getitem__(self, index):
        got = self._pages[: self._n][index]
        return got.tolist() if isinstance(index, slice) else int(got)

    def __eq__(self, other) -> bool:
        return list(self) == list(other)

    def extend(self, pages: Iterable[int]) -> None:
        pages = list(pages)
        need = self._n + len(pages)
        if need > len(self._pages):
            grown = np.full(max(need, 2 * len(self._pages)), -1, dtype=np.int32)
            grown[: self._n] = self._pages[: self._n]
            self._pages = grown
        self._pages[self._n : need] = pages
        self._n = need

    def held(self) -> list[int]:
        """The pages the table still names."""
        live = self._pages[self.passed : self._n]
        return live[live >= 0].tolist()

    def pass_up_to(self, first_kept: int) -> list[int]:
        """Forget the pages before logical index ``first_kept``; returns them."""
        first_kept = min(first_kept, self._n)
        if first_kept <= self.passed:
            return []
        gone = self._pages[self.passed : first_kept]
        pages = gone[gone >= 0].tolist()
        gone[:] = -1
        self.passed = first_kept
        return pages


class StateSlots:
    """Slots of fixed size, one per live request."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._owner: dict[int, Hashable] = {}

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, owner: Hashable) -> int:
        if not self._free:
            raise OutOfPages("state slots", 1, 0)
        slot = self._free.pop()
        self._owner[slot] = owner
        return slot

    def give_back(self, owner: Hashable, slot: int) -> None:
        if self._owner.get(slot, _NOBODY) != owner:
            raise CacheBookkeepingError(f"slot {slot} given back by {owner!r} but owned by "
                                        f"{self._owner.get(slot, 'nobody')!r}")
        del self._owner[slot]
        self._free.append(slot)

    def check(self) -> None:
        if len(set(self._free)) != len(self._free) or set(self._free) & set(self._owner) \
                or len(self._free) + len(self._owner) != self.num_slots:
            raise CacheBookkeepingError("state slots: the books do not add up")
