"""One step's batch: a flat list of tokens from up to B requests.

Each request contributes a portion of ``n >= 1`` consecutive tokens starting
at its current length; a decoded token is a portion of one.  The reference
never mixes the two kinds in a launch (v3/crates/rvllm-runtime/src/scheduler.rs:3-5),
but its kernels' interface already describes several portions at once by
``cu_seqlens_q`` and ``context_lens`` (v3/kernels/paged_attention_sm89.cu:302-368);
this batch is that description, extended by the request of every token so that
token-wise kernels need no search.

All index arrays lie in one packed int32 buffer (the reference's packed
metadata buffer: v3/crates/rvllm-metadata/src/layout.rs:19-78).  The arrays by
token and by request travel to the GPU with one copy; of each block table, as
wide as the longest context the engine allows, only the step's requests by the
pages of the longest of them travel, as one strided copy.
"""

from __future__ import annotations

import dataclasses
from typing import Optional, Sequence

import numpy as np
import torch

from ..kernels import ops


@dataclasses.dataclass
class Portion:
    """The next tokens of one request in this step."""

    request: object  # the cache manager's handle of the request
    tokens: Sequence[int]
    start: int  # position of tokens[0]
    want: Sequence[int] = ()  # places among `tokens` whose logits are wanted


@dataclasses.dataclass
class StepBatch:
    """Device-side description of a step, read by parts and kernels."""

    num_tokens: int
    num_requests: int
    token_ids: torch.Tensor  # [T] int32
    positions: torch.Tensor  # [T] int32
    token_req: torch.Tensor  # [T] int32, row of the token's request in the tables below
    q_start: torch.Tensor  # [B + 1] int32, first token of each portion
    chunk_start: torch.Tensor  # [B] int32, position of the portion's first token
    context_len: torch.Tensor  # [B] int32, tokens held by the request after this step
    state_slot: torch.Tensor  # [B] int32, slot of the request's fixed-size state
    logit_rows: torch.Tensor  # [R] int32, flat indices of the tokens whose logits are wanted
    block_tables: dict  # group name -> [B, width] int32
    # host-side copies for launch decisions
    max_portion: int = 1
    max_context: int = 1
    num_logit_rows: int = 0
    host_q_start: Optional[np.ndarray] = None
    host_chunk_start: Optional[np.ndarray] = None
    # what parts work out once a step and share between layers (keyed by who made it)
    shared: dict = dataclasses.field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_portion == 1


class BatchLayout:
    """Where each array lies in the packed buffer for given capacities.

    The layout depends only on (token capacity, request capacity, table
    widths), so steps of the same capacity reuse the same device addresses,
    which a captured graph needs."""

    def __init__(self, max_tokens: int, max_requests: int, table_widths: dict[str, int]):
        self.max_tokens = max_tokens
        self.max_requests = max_requests
        self.table_widths = dict(table_widths)
        off = 0
        self.offsets: dict[str, tuple[int, int]] = {}

        def add(name: str, n: int):
            nonlocal off
            self.offsets[name] = (off, n)
            off += (n + 15) // 16 * 16  # keep every array 64-byte aligned

        add("token_ids", max_tokens)
        add("positions", max_tokens)
        add("token_req", max_tokens)
        add("logit_rows", max_tokens)
        add("q_start", max_requests + 1)
        add("chunk_start", max_requests)
        add("context_len", max_requests)
        add("state_slot", max_requests)
        self.tables_from = off  # what lies before is copied whole each step
        for name, width in self.table_widths.items():
            add("bt:" + name, max_requests * width)
        self.total = off


class BatchBuilder:
    """Packs portions into the pinned staging buffer and copies it to the GPU."""

    def __init__(self, device: torch.device, max_tokens: int, max_requests: int, table_widths: dict[str, int]):
        self.device = torch.device(device)
        self.layout = BatchLayout(max_tokens, max_requests, table_widths)
        pin = self.device.type == "cuda"
        # Two staging buffers take turns, so that a step can be packed while
        # the copy of the one before may still be under way.
        self._hosts = [torch.zeros(self.layout.total, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._events = [torch.cuda.Event() if pin else None for _ in range(2)]
        self._turn = 0
        self.host = self._hosts[0]
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(self.layout.total, dtype=torch.int32, device=self.device)
        self.dev[self.layout.tables_from :] = -1  # no page anywhere, until a step says otherwise

    def _table(self, buffer: torch.Tensor, name: str) -> torch.Tensor:
        off, cap = self.layout.offsets["bt:" + name]
        return buffer[off : off + cap].view(self.layout.max_requests, self.layout.table_widths[name])

    def _view(self, name: str, n: Optional[int] = None) -> torch.Tensor:
        off, cap = self.layout.offsets[name]
        return self.dev[off : off + (cap if n is None else n)]

    def _host(self, name: str) -> np.ndarray:
        off, cap = self.layout.offsets[name]
        return self.host_np[off : off + cap]

    def build(self, portions: Sequence[Portion], tables: dict[str, Sequence[Sequence[int]]],
              state_slots: Sequence[int]) -> StepBatch:
        """``tables[group][b]`` is the block table row of portion b."""
        lay = self.layout
        self._turn ^= 1
        self.host = self._hosts[self._turn]
        self.host_np = self.host.numpy()
        event = self._events[self._turn]
        if event is not None:
            event.synchronize()  # the copy that last read this buffer is done
        B = len(portions)
        T = sum(len(p.tokens) for p in portions)
        if B > lay.max_requests:
            raise ValueError(f"step has {B} requests, the engine was built for {lay.max_requests}")
        if T > lay.max_tokens:
            raise ValueError(f"step has {T} tokens, the engine was built for {lay.max_tokens}")
        tok, pos, req, rows = (self._host(n) for n in ("token_ids", "positions", "token_req", "logit_rows"))
        qs, cs, cl, ss = (self._host(n) for n in ("q_start", "chunk_start", "context_len", "state_slot"))
        # Whole arrays at a time, not a portion at a time: with 64 decoded tokens a step, a handful of small
        # assignments per portion cost the host more than the step costs the GPU.
        lens = np.fromiter((len(p.tokens) for p in portions), dtype=np.int64, count=B)
        if B and lens.min() < 1:
            raise ValueError("a portion must hold at least one token")
        starts = np.fromiter((p.start for p in portions), dtype=np.int64, count=B)
        first = np.zeros(B + 1, dtype=np.int64)  # first token of each portion
        np.cumsum(lens, out=first[1:])
        tok[:T] = np.concatenate([np.asarray(p.tokens, dtype=np.int32) for p in portions]) if T else 0
        req[:T] = np.repeat(np.arange(B, dtype=np.int32), lens)
        place = np.repeat(starts - first[:B], lens)
        place += np.arange(T, dtype=np.int64)  # in place, as for the tables below
        pos[:T] = place
        qs[: B + 1] = first
        cs[:B] = starts
        cl[:B] = starts + lens
        ss[:B] = np.fromiter(state_slots, dtype=np.int64, count=B)
        wanted = []
        for b, p in enumerate(portions):
            n, t = int(lens[b]), int(first[b])
            for wplace in p.want:
                if not 0 <= wplace < n:
                    raise ValueError(f"wanted place {wplace} outside a portion of {n} tokens")
                wanted.append(t + wplace)
        r = len(wanted)
        rows[:r] = wanted
        max_portion = max(1, int(lens.max())) if B else 1
        max_context = max(1, int((starts + lens).max())) if B else 1
        used = {}  # group -> entries of the step's longest table: what the step's kernels can ask for
        for name, width in lay.table_widths.items():
            off, _ = lay.offsets["bt:" + name]
            dst = self.host_np[off : off + B * width]
            held = [np.asarray(row, dtype=np.int32) for row in tables[name]]
            counts = np.fromiter((len(row) for row in held), dtype=np.int64, count=B)
            if B and counts.max() > width:
                raise ValueError(f"block table of group {name} has {int(counts.max())} entries, width is {width}")
            used[name] = int(counts.max()) if B else 0
            dst.reshape(B, width)[:, : used[name]] = -1
            total = int(counts.sum())
            if total:
                # entry j of row b goes to b * width + j
                row_first = np.zeros(B, dtype=np.int64)
                np.cumsum(counts[:-1], out=row_first[1:])
                # added in place: a sum of two temporaries of 256 KB or more makes numpy look up the call stack
                # to see whether it may reuse one of them, which costs some 100 ms the first time it happens
                where = np.repeat(np.arange(B, dtype=np.int64) * width - row_first, counts)
                where += np.arange(total, dtype=np.int64)
                dst[where] = np.concatenate(held)
        self.dev[: lay.tables_from].copy_(self.host[: lay.tables_from], non_blocking=True)
        tables_dev = {}
        for name in lay.table_widths:
            tables_dev[name] = self._table(self.dev, name)
            # Rows beyond the step's requests and entries beyond its longest table keep what earlier steps left:
            # no kernel looks there, since a request's keys end with its own context.
            if event is not None:
                ops.copy_rows_to_device(tables_dev[name], self._table(self.host, name), B, used[name])
            else:
                tables_dev[name][:B, : used[name]] = self._table(self.host, name)[:B, : used[name]]
        if event is not None:
            event.record()
        return StepBatch(
            num_tokens=T,
            num_requests=B,
            token_ids=self._view("token_ids", T),
            positions=self._view("positions", T),
            token_req=self._view("token_req", T),
            q_start=self._view("q_start", B + 1),
            chunk_start=self._view("chunk_start", B),
            context_len=self._view("context_len", B),
            state_slot=self._view("state_slot", B),
            logit_rows=self._view("logit_rows", r),
            block_tables=tables_dev,
            max_portion=max_portion,
            max_context=max_context,
            num_logit_rows=r,
            host_q_start=qs[: B + 1].copy(),
            host_chunk_start=cs[:B].copy(),
        )
