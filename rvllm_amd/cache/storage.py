"""Device memory behind the cache manager's books.

Every layer with a key/value need gets one tensor
``[2, num_pages, page_size, kv_heads, head_dim]``, keys then values
(v3/crates/rvllm-mem/src/kv_layout.rs:1-46); every layer with a fixed-size
state gets ``[max_requests, *shape]``.  Nothing is cleared when pages change
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
                kv = torch.zeros((2, g.pool.num_pages, g.page_size, need.num_kv_heads, need.head_dim), dtype=dtype,
                                 device=self.device)
                self.bytes += kv.numel() * kv.element_size()
                self.views.append(KVCacheView(kv[0], kv[1], g.name, g.page_size))
            elif isinstance(need, StateNeed):
                slots = torch.zeros((manager.max_requests, *need.shape), dtype=need.dtype, device=self.device)
                self.bytes += slots.numel() * slots.element_size()
                self.views.append(StateView(slots))
            else:
                self.views.append(None)

    def clear_slot(self, slot: int) -> None:
        for i in self.manager.state_layers:
            self.views[i].slots[slot].zero_()
