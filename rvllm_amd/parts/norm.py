"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * (offset + weight).

eps is added to the mean inside the root; sum, root and product are 32-bit
(v3/kernels/rmsnorm_inplace_f16.cu:29-62, v3/crates/rvllm-fused/src/reference.rs:58-76).
``unit_offset`` selects the zero-centred form of the Gemma checkpoints, where
the stored weight is the gain minus one.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Norm, ParamSpec
from .registry import NORMS
from .spec import PartSpec


class RMSNorm(Norm):
    def __init__(self, spec: PartSpec, *, width: int, name: str):
        self.width = int(width)
        self.name = name
        self.eps = float(spec["eps"])
        self.offset = 1.0 if spec.get("unit_offset", False) else 0.0
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [ParamSpec(f"{prefix}.{self.name}.weight", (self.width,), init=("normal", 0.1))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        # The weight keeps the type it was loaded in (bf16, or 32-bit).
        self.weight = tensors[f"{prefix}.{self.name}.weight"].to(device).contiguous()

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.offset, out=out)

    def forward_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.offset, rows=rows)

    def add_into(self, branch, residual, then=None, then_out=None):
        if then is None:
            return ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual)
        if isinstance(then, RMSNorm):
            return ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual, then.weight, then.eps,
                                   then.offset, then_out)
        ops.add_rmsnorm(branch, self.weight, self.eps, self.offset, residual)
        return then.forward(residual, out=then_out)


NORMS.register("rmsnorm", RMSNorm)
