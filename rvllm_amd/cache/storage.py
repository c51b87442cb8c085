"""Device memory behind the cache manager's books.

Every layer with a key/value need gets one allocation, keys then values (as
in v3/crates/rvllm-mem/src/kv_layout.rs:1-46).  Inside it keys are
``[num_pages, kv_heads, page_size, head_dim]`` and values are transposed
inside groups of 16 slots, ``[num_pages, kv_heads, page_size / 16, head_dim,
16]``: what one key/value head holds on a page is one contiguous block, and
the matrix-core attention kernel reads both operands in the order it sums
them, 16 keys at a time from one run of memory whatever the page size.  Every layer
with a fixed-size state gets ``[max_requests, *shape]``.  Nothing is cleared when pages change
hands: a position that a token may not see is never read, so what an earlier
request left behind is unreachable (the reference relies on the same for its
rejected drafts: v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:4237-4243).
State slots are cleared when handed out, because a state is read whole.
"""

from __future__ import annotations

from typing import Optional

import torch

VALUE_GROUP = 16  # slots whose values of one dimension lie side by side (csrc/kv_layout.h)

from ..parts.base import KVCacheView, KVNeed, StateNeed, StateView
from .manager import CacheManager


class CacheTooLarge(MemoryError):
    pass


def bytes_needed(manager: CacheManager, dtype: torch.dtype) -> int:
    """What ``CacheStorage`` allocates for these books."""
    elem = torch.empty((), dtype=dtype).element_size()
    total = 0
    for i, need in enumerate(manager.needs):
        if isinstance(need, KVNeed):
            g = manager.groups[manager.layer_group[i]]
            total += 2 * g.pool.num_pages * need.num_kv_heads * g.page_size * need.head_dim * elem
        elif isinstance(need, StateNeed):
            count = 1
            for n in need.shape:
                count *= int(n)
            total += manager.max_requests * count * torch.empty((), dtype=need.dtype).element_size()
    return total


class CacheStorage:
    def __init__(self, manager: CacheManager, device, dtype: torch.dtype, held_by_weights: Optional[int] = None):
        """``held_by_weights``: the bytes the model's weights take on the device (for the message, should the cache
        not fit beside them)."""
        self.manager = manager
        self.device = torch.device(device)
        self.dtype = dtype
        self.views: list = []
        self.bytes = 0
        if self.device.type == "cuda":
            # Said before the first allocation, with the numbers: the allocator's own complaint comes at some layer
            # in the middle and names neither the cache's size nor what the weights hold.
            need_bytes = bytes_needed(manager, dtype)
            free, total = torch.cuda.mem_get_info(self.device)
            free += torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
            if need_bytes > free:
                weights = "" if held_by_weights is None else (
                    f"; the weights hold {held_by_weights / 2**30:.1f} GiB (bf16 matrices lie there twice while "
                    f"tiled_weights is on: row by row for the library's products, in tiles for decode steps)")
                raise CacheTooLarge(
                    f"the cache for {manager.max_requests} requests needs {need_bytes / 2**30:.1f} GiB, "
                    f"{free / 2**30:.1f} GiB of {total / 2**30:.1f} GiB are free{weights}; lower max_cache_tokens, "
                    f"max_num_seqs or max_model_len")
        for i, need in enumerate(manager.needs):
            if isinstance(need, KVNeed):
                g = manager.groups[manager.layer_group[i]]
                kv = torch.zeros((2, g.pool.num_pages, need.num_kv_heads, g.page_size * need.head_dim), dtype=dtype,
                                 device=self.device)
                self.bytes += kv.numel() * kv.element_size()
                keys = kv[0].view(g.pool.num_pages, need.num_kv_heads, g.page_size, need.head_dim)
                if g.page_size % VALUE_GROUP:
                    raise ValueError(f"page_size {g.page_size} must be a multiple of {VALUE_GROUP}: the values are "
                                     f"transposed by groups of that many slots")
                values = kv[1].view(g.pool.num_pages, need.num_kv_heads, g.page_size // VALUE_GROUP, need.head_dim,
                                    VALUE_GROUP)
                self.views.append(KVCacheView(keys, values, g.name, g.page_size))
            elif isinstance(need, StateNeed):
                slots = torch.zeros((manager.max_requests, *need.shape), dtype=need.dtype, device=self.device)
                self.bytes += slots.numel() * slots.element_size()
                self.views.append(StateView(slots))
            else:
                self.views.append(None)

    def clear_slot(self, slot: int) -> None:
        for i in self.manager.state_layers:
            self.views[i].slots[slot].zero_()
