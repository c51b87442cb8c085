"""Dense gated feed-forward: down(act(gate(x)) * up(x)).

gate and up are one product against their joined rows, gate rows first
(v3/crates/rvllm-loader/src/gemma4_load.rs:683-685); the activation is a
parameter (tanh-form GELU for Gemma: v3/kernels/fused_gelu_mul_f16.cu:20-27).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec
from .linear import linear
from .registry import FEED_FORWARDS
from .spec import PartSpec


FUSED_ACTIVATION_MAX_ROWS = 4


class GatedMLP(FeedForward):
    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(spec["intermediate_size"])
        self.activation = str(spec["activation"])
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.w_gate_up = self.w_down = None

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
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors[f"{p}.down_proj.weight"].to(device=device, dtype=dtype).contiguous()

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        gate_up = linear(x, self.w_gate_up, sliced_ok=True)
        # a few rows in bf16: the down product applies the activation itself while it stages its input
        # (measured on MI355X: a gain up to 4 rows, a loss from 8 on, where every block repeats too much of it)
        if x.shape[0] <= FUSED_ACTIVATION_MAX_ROWS:
            fused = ops.gemm_bf16_gated(gate_up, self.w_down, self.activation, sliced_ok=True)
            if fused is not None:
                return fused
        act = ops.gated_act(gate_up, self.activation)
        return linear(act, self.w_down, sliced_ok=True)


FEED_FORWARDS.register("gated_mlp", GatedMLP)
