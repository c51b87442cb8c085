"""Grouped-query attention over the paged cache.

Order of work for the tokens of a step (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28,
steps 2 to 7): one fused projection to q|k|v, per-head RMSNorm of queries and
keys, rotation, write of keys and values into the cache, attention over the
cache, output projection.  The score scale, the window, the head counts and
sizes, the norm's constants and the position encoding are parameters of the
part.  ``window`` None means every earlier key is visible; otherwise a token at
position p sees the keys p - window + 1 .. p.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import KVCacheView, KVNeed, Mixer, ParamSpec
from .linear import decode_weight, linear
from .registry import MIXERS, POSITION_ENCODINGS
from .spec import PartSpec


class PagedAttention(Mixer):
    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.scale = float(spec["scale"])
        window = spec.get("window")
        self.window: Optional[int] = None if window is None else int(window)
        self.qk_norm: Optional[dict] = spec.get("qk_norm")  # {"eps":, "unit_offset":} or None
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} query heads cannot share {self.num_kv_heads} key/value heads")
        pos_spec = spec.get("position") or PartSpec("none")
        self.position = POSITION_ENCODINGS.build(pos_spec, head_dim=self.head_dim)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_qkv = self.w_o = self.q_norm_w = self.k_norm_w = None

    # ---- weights -----------------------------------------------------
    def param_specs(self, prefix: str) -> list[ParamSpec]:
        p = f"{prefix}.self_attn"
        specs = [
            ParamSpec(f"{p}.q_proj.weight", (self.q_size, self.hidden_size)),
            ParamSpec(f"{p}.k_proj.weight", (self.kv_size, self.hidden_size)),
            ParamSpec(f"{p}.v_proj.weight", (self.kv_size, self.hidden_size)),
            ParamSpec(f"{p}.o_proj.weight", (self.hidden_size, self.q_size)),
        ]
        if self.qk_norm is not None:
            specs += [
                ParamSpec(f"{p}.q_norm.weight", (self.head_dim,), init=("normal", 0.1)),
                ParamSpec(f"{p}.k_norm.weight", (self.head_dim,), init=("normal", 0.1)),
            ]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        p = f"{prefix}.self_attn"
        # q, k and v rows are joined into one matrix, as the reference's loader
        # joins them (v3/crates/rvllm-loader/src/gemma4_load.rs:522,621-625).
        parts = [tensors[f"{p}.{n}_proj.weight"] for n in ("q", "k", "v")]
        self.w_qkv = decode_weight(torch.cat([t.to(device=device, dtype=dtype) for t in parts], dim=0).contiguous())
        self.w_o = decode_weight(tensors[f"{p}.o_proj.weight"].to(device=device, dtype=dtype).contiguous())
        if self.qk_norm is not None:
            self.q_norm_w = tensors[f"{p}.q_norm.weight"].to(device).contiguous()
            self.k_norm_w = tensors[f"{p}.k_norm.weight"].to(device).contiguous()
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.k_norm_w = self.k_norm_w.to(self.q_norm_w.dtype)

    # ---- cache -------------------------------------------------------
    def cache_need(self) -> KVNeed:
        return KVNeed(self.num_kv_heads, self.head_dim, self.window)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step, cache: KVCacheView) -> torch.Tensor:
        n = x.shape[0]
        qkv = linear(x, self.w_qkv, sliced_ok=True)
        q = torch.empty((n, self.q_size), dtype=x.dtype, device=x.device)
        table = step.block_tables[cache.group]
        norm = self.qk_norm or {}
        # prompt portions: values go into their pages a page at a time, in wide stores, by blocks of the same launch
        by_page = (cache.writes and isinstance(qkv, torch.Tensor)
                   and step.max_portion >= ops.VALUES_BY_PAGE_MIN_PORTION)
        ops.qk_norm_rope_kv_write(
            qkv, q, self.q_norm_w, self.k_norm_w, float(norm.get("eps", 0.0)),
            1.0 if norm.get("unit_offset", False) else 0.0, self.position.tables(step),
            self.position.rotary_dim, step.positions, step.token_req, table, cache.k_pages, cache.v_pages,
            self.num_heads, self.num_kv_heads, self.head_dim, write_kv=cache.writes,
            values_by_page=step if by_page else None)
        attn = torch.empty_like(q)
        ops.paged_attention(q, cache.k_pages, cache.v_pages, table, step, attn, self.num_heads, self.scale,
                            self.window)
        return linear(attn, self.w_o, sliced_ok=True)


MIXERS.register("attention", PagedAttention)
