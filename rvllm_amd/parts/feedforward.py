"""Dense gated feed-forward: down(act(gate(x)) * up(x)).

gate and up are one product against their joined rows
(v3/crates/rvllm-loader/src/gemma4_load.rs:683-685: gate rows first; here the
rows lie in fours, two gates and then their two ups, so that the product for a
few rows can apply the activation itself); the activation is a parameter
(tanh-form GELU for Gemma: v3/kernels/fused_gelu_mul_f16.cu:20-27).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec
from .linear import decode_weight, linear
from .registry import FEED_FORWARDS
from .spec import PartSpec


class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(spec["intermediate_size"])
        self.activation = str(spec["activation"])
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.w_gate_up = self.w_down = None
        self.fours = False

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        p = f"{prefix}.mlp"
        return [
            ParamSpec(f"{p}.gate_proj.weight", (self.intermediate_size, self.hidden_size)),
            ParamSpec(f"{p}.up_proj.weight", (self.intermediate_size, self.hidden_size)),
            ParamSpec(f"{p}.down_proj.weight", (self.hidden_size, self.intermediate_size)),
        ]

    def bind(self, tensors, prefix, device, dtype) -> None:
        p = f"{prefix}.mlp"
        gate = tensors[f"{p}.gate_proj.weight"].to(device=device, dtype=dtype)
        up = tensors[f"{p}.up_proj.weight"].to(device=device, dtype=dtype)
        # widths that the activation kernel cannot take in fours keep the gates before the ups
        self.fours = self.intermediate_size % ops.FOURS_WIDTH_MULTIPLE == 0
        self.w_gate_up = decode_weight(ops.rows_in_fours(gate, up) if self.fours
                                       else torch.cat([gate, up], dim=0).contiguous())
        self.w_down = decode_weight(tensors[f"{p}.down_proj.weight"].to(device=device, dtype=dtype).contiguous())

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        # a few rows in bf16: the product applies the activation itself where it holds the sums
        act = ops.gemm_bf16_gate_up(x, self.w_gate_up, self.activation) if self.fours and x.is_cuda else None
        if act is None:
            act = ops.gated_act(linear(x, self.w_gate_up, sliced_ok=True), self.activation, fours=self.fours)
        return linear(act, self.w_down, sliced_ok=True)


FEED_FORWARDS.register("gated_mlp", GatedMLP)
