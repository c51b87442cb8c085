"""Dense gated feed-forward: down(act(gate(x)) * up(x)).

gate and up are one product against their joined rows
(v3/crates/rvllm-loader/src/gemma4_load.rs:683-685: gate rows first; here the
rows lie in fours, two gates and then their two ups, so that the product for a
few rows can apply the activation itself); the activation is a parameter
(tanh-form GELU for Gemma: v3/kernels/fused_gelu_mul_f16.cu:20-27).

``names`` maps a role (``gate``, ``up``, ``down``) to the tensor's name under the
layer's prefix, without ``.weight`` (the Gemma names if absent); a role
``gate_up`` names one stored matrix that holds the gate rows and then the up
rows.  ``bias`` lists the projections that have a ``.bias`` (True: all).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec
from .linear import bias_roles, decode_weight, linear, tensor_names
from .registry import FEED_FORWARDS
from .spec import PartSpec


class GatedMLP(FeedForward):
    NAMES = {"gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj"}

    def __init__(self, spec: PartSpec, *, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(spec["intermediate_size"])
        self.activation = str(spec["activation"])
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.names = tensor_names(self.NAMES, spec.get("names"))
        inter = self.intermediate_size
        self.stored = {"gate_up": 2 * inter} if "gate_up" in self.names else {"gate": inter, "up": inter}
        self.bias = bias_roles(spec.get("bias"), [*self.stored, "down"])
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None
        self.fours = False

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        specs = [ParamSpec(f"{at[role]}.weight", (rows, self.hidden_size)) for role, rows in self.stored.items()]
        specs.append(ParamSpec(f"{at['down']}.weight", (self.hidden_size, self.intermediate_size)))
        specs += [ParamSpec(f"{at[role]}.bias", (rows,)) for role, rows in self.stored.items() if role in self.bias]
        if "down" in self.bias:
            specs.append(ParamSpec(f"{at['down']}.bias", (self.hidden_size,)))
        return specs

    def _gate_and_up(self, tensors, at, suffix, roles, device, dtype):
        """The gate's and the up's tensor named ``suffix`` (``weight`` or ``bias``), each None unless its stored
        role is among ``roles``."""
        inter = self.intermediate_size
        if "gate_up" in self.stored:
            if "gate_up" not in roles:
                return None, None
            both = tensors[f"{at['gate_up']}.{suffix}"].to(device=device, dtype=dtype)
            return both[:inter], both[inter:]
        return tuple(tensors[f"{at[role]}.{suffix}"].to(device=device, dtype=dtype) if role in roles else None
                     for role in ("gate", "up"))

    def bind(self, tensors, prefix, device, dtype) -> None:
        at = {role: f"{prefix}.{name}" for role, name in self.names.items()}
        gate, up = self._gate_and_up(tensors, at, "weight", self.stored, device, dtype)
        # widths that the activation kernel cannot take in fours keep the gates before the ups
        self.fours = self.intermediate_size % ops.FOURS_WIDTH_MULTIPLE == 0
        join = ops.rows_in_fours if self.fours else (lambda g, u: torch.cat([g, u], dim=0).contiguous())
        self.w_gate_up = decode_weight(join(gate, up), self.tiled_weights)
        self.w_down = decode_weight(tensors[f"{at['down']}.weight"].to(device=device, dtype=dtype).contiguous(),
                                    self.tiled_weights)
        if self.bias & set(self.stored):  # laid out as the rows of the joined matrix are; zeros where there is none
            zeros = torch.zeros(self.intermediate_size, dtype=torch.float32, device=device)
            gate_b, up_b = (zeros if b is None else b
                            for b in self._gate_and_up(tensors, at, "bias", self.bias, device, torch.float32))
            self.b_gate_up = join(gate_b[:, None], up_b[:, None]).reshape(-1).contiguous()
        if "down" in self.bias:
            self.b_down = tensors[f"{at['down']}.bias"].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        act = None
        if self.b_gate_up is None and self.fours and x.is_cuda:
            # a few rows in bf16: the product applies the activation itself where it holds the sums
            act = ops.gemm_bf16_gate_up(x, self.w_gate_up, self.activation)
        if act is None:
            gate_up = linear(x, self.w_gate_up, sliced_ok=True)
            if self.b_gate_up is not None:
                gate_up = ops.add_bias(gate_up, self.b_gate_up)
            act = ops.gated_act(gate_up, self.activation, fours=self.fours)
        out = linear(act, self.w_down, sliced_ok=True)
        return out if self.b_down is None else ops.add_bias(out, self.b_down)


FEED_FORWARDS.register("gated_mlp", GatedMLP)
