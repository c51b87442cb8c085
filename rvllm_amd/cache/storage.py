"""Device memory behind the cache manager's books.

Every layer with a key/value need gets one allocation, keys then values (as
in v3/crates/rvllm-mem/src/kv_layout.rs:1-46).  Inside it keys are
``[num_pages, kv_heads, page_size, head_dim]`` and values are transposed
inside the page, ``[num_pages, kv_heads, head_dim, page_size]``: what one
key/value head holds on a page is one contiguous block, and the matrix-core
attention kernel reads both operands in the order it sums them.  Every layer
with a fixed-size state gets ``[max_requests, *shape]``.  Nothing is cleared when pages change
hands: a position that a token may not see is never read, so what an earlier
request left behind is unreachable (the reference relies on the same for its
rejected drafts: v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:4237-4243).
State slots are cleared when handed out, because a state is read whole.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..parts.base import KVCacheView, KVNeed, StateNeed, StateView
from .manager import CacheManager


class CacheStorage:
    def __init__(self, manager: CacheManager, device, dtype: torch.dtype):
        self.manager = manager
        self.device = torch.device(device)
        self.dtype = dtype
        self.views: list = []
        self.bytes = 0
        for i, need in enumerate(manager.needs):
            if isinstance(need, KVNeed):
                g = manager.groups[manager.layer_group[i]]
                kv = torch.zeros((2, g.pool.num_pages, need.num_kv_heads, g.page_size * need.head_dim), dtype=dtype,
                                 device=self.device)
                self.bytes += kv.numel() * kv.element_size()
                keys = kv[0].view(g.pool.num_pages, need.num_kv_heads, g.page_size, need.head_dim)
                values = kv[1].view(g.pool.num_pages, need.num_kv_heads, need.head_dim, g.page_size)
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
