"""Grouped-query attention over the paged cache.

Order of work for the tokens of a step (v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28,
steps 2 to 7): one fused projection to q|k|v, per-head RMSNorm of queries and
keys, rotation, write of keys and values into the cache, attention over the
cache, output projection.  The score scale, the window, the head counts and
sizes, the norm's constants and the position encoding are parameters of the
part.  ``window`` None means every earlier key is visible; otherwise a token at
position p sees the keys p - window + 1 .. p.

Where the checkpoint keeps the part's tensors is a parameter too: ``names`` maps a
role (``q``, ``k``, ``v``, ``o``, ``q_norm``, ``k_norm``) to the tensor's name under
the layer's prefix, without ``.weight`` (the Gemma names if absent); a role ``qkv``
names one stored matrix that holds the rows of q, k and v in this order.  ``bias``
lists the projections that have a ``.bias`` beside their ``.weight`` (True: all).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import KVCacheView, KVNeed, Mixer, ParamSpec
from .linear import bias_roles, decode_weight, linear, tensor_names
from .registry import MIXERS, POSITION_ENCODINGS
from .spec import PartSpec


class PagedAttention(Mixer):
    NAMES = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
             "q_norm": "self_attn.q_norm", "k_norm": "self_attn.k_norm"}

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
        self.names = tensor_names(self.NAMES, spec.get("names"))
        # the projections as the checkpoint stores them: role -> rows
        self.stored = ({"qkv": self.q_size + 2 * self.kv_size} if "qkv" in self.names
                       else {"q": self.q_size, "k": self.kv_size, "v": self.kv_size})
        self.bias = bias_roles(spec.get("bias"), [*self.stored, "o"])
        self.w_qkv = self.w_o = self.q_norm_w = self.k_norm_w = self.b_qkv = self.b_o = None

    # ---- weights -----------------------------------------------------
    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        specs = [ParamSpec(f"{at[role]}.weight", (rows, self.hidden_size)) for role, rows in self.stored.items()]
        specs.append(ParamSpec(f"{at['o']}.weight", (self.hidden_size, self.q_size)))
        specs += [ParamSpec(f"{at[role]}.bias", (rows,)) for role, rows in self.stored.items() if role in self.bias]
        if "o" in self.bias:
            specs.append(ParamSpec(f"{at['o']}.bias", (self.hidden_size,)))
        if self.qk_norm is not None:
            specs += [
                ParamSpec(f"{at['q_norm']}.weight", (self.head_dim,), init=("normal", 0.1)),
                ParamSpec(f"{at['k_norm']}.weight", (self.head_dim,), init=("normal", 0.1)),
            ]
        return specs

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        # q, k and v rows are joined into one matrix, as the reference's loader
        # joins them (v3/crates/rvllm-loader/src/gemma4_load.rs:522,621-625).
        parts = [tensors[f"{at[role]}.weight"].to(device=device, dtype=dtype) for role in self.stored]
        self.w_qkv = decode_weight(torch.cat(parts, dim=0).contiguous(), self.tiled_weights)
        self.w_o = decode_weight(tensors[f"{at['o']}.weight"].to(device=device, dtype=dtype).contiguous(),
                                 self.tiled_weights)
        if self.bias & set(self.stored):  # projections without a bias of their own add zeros
            self.b_qkv = torch.cat([
                tensors[f"{at[role]}.bias"].to(device=device, dtype=torch.float32) if role in self.bias
                else torch.zeros(rows, dtype=torch.float32, device=device) for role, rows in self.stored.items()])
        if "o" in self.bias:
            self.b_o = tensors[f"{at['o']}.bias"].to(device=device, dtype=torch.float32).contiguous()
        if self.qk_norm is not None:
            self.q_norm_w = tensors[f"{at['q_norm']}.weight"].to(device).contiguous()
            self.k_norm_w = tensors[f"{at['k_norm']}.weight"].to(device).contiguous()
            if self.q_norm_w.dtype != self.k_norm_w.dtype:
                self.k_norm_w = self.k_norm_w.to(self.q_norm_w.dtype)

    # ---- cache -------------------------------------------------------
    def cache_need(self) -> KVNeed:
        return KVNeed(self.num_kv_heads, self.head_dim, self.window)

    # ---- run ---------------------------------------------------------
    def forward(self, x: torch.Tensor, step, cache: KVCacheView) -> torch.Tensor:
        n = x.shape[0]
        qkv = linear(x, self.w_qkv, sliced_ok=True)
        if self.b_qkv is not None:
            qkv = ops.add_bias(qkv, self.b_qkv)
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
        out = linear(attn, self.w_o, sliced_ok=True)
        return out if self.b_o is None else ops.add_bias(out, self.b_o)


MIXERS.register("attention", PagedAttention)
