"""Rotary position encoding with split-half pairs and linear scaling.

inv_freq[i] = theta^(-2i/head_dim) / factor for i < rotary_dim/2; the exponent
uses the head size, not the number of rotated dimensions
(v3/crates/rvllm-loader/src/gemma4_load.rs:1168-1179, metal_host.rs:281-289).
Dividing the inverse frequencies by ``factor`` is the linear scaling of the
global layers: the angle of position p becomes that of p / factor.  The table
is computed in 64-bit and rounded to 32-bit once; the angle
``float(pos) * inv_freq[i]`` and its sine and cosine are 32-bit in the kernel
that tabulates them for a step's tokens.
"""

from __future__ import annotations

from typing import Optional

import torch

from .base import PositionEncoding
from .registry import POSITION_ENCODINGS
from .spec import PartSpec


class RotaryEncoding(PositionEncoding):
    def __init__(self, spec: PartSpec, *, head_dim: int):
        self.head_dim = int(head_dim)
        self.theta = float(spec["theta"])
        self.factor = float(spec.get("factor", 1.0))
        self.rotary_dim = int(spec.get("rotary_dim", head_dim))
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self._table: Optional[torch.Tensor] = None

    def inv_freq_host(self) -> torch.Tensor:
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = self.theta ** (-2.0 * i / self.head_dim) / self.factor
        return inv.to(torch.float32)

    def inv_freq(self, device) -> Optional[torch.Tensor]:
        if self.rotary_dim == 0:
            return None
        if self._table is None or self._table.device != torch.device(device):
            self._table = self.inv_freq_host().to(device)
        return self._table


    def tables(self, step):
        """Cosines and sines of this step's tokens, made once a step for all
        the layers with these parameters."""
        if self.rotary_dim == 0:
            return None
        shared = getattr(step, "shared", None)
        key = ("rope", self.theta, self.factor, self.rotary_dim, self.head_dim)
        if shared is not None and key in shared:
            return shared[key]
        from ..kernels import ops

        made = ops.rope_table(self.inv_freq(step.positions.device), step.positions, step.num_tokens)
        if shared is not None:
            shared[key] = made
        return made


class NoPositionEncoding(PositionEncoding):
    """Queries and keys are left as they are."""

    def __init__(self, spec: PartSpec, *, head_dim: int):
        self.rotary_dim = 0


POSITION_ENCODINGS.register("rope", RotaryEncoding)
POSITION_ENCODINGS.register("none", NoPositionEncoding)
