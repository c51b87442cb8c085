"""Token embedding and the language-model head.

Embedding: x[t] = table[id[t]] * scale.  The table stays unscaled in memory
and the scale is applied in 32-bit at the lookup, as the reference's host
decoder does (v3/crates/rvllm-loader/src/metal_host.rs:298,820-839); so the
tied head can read the same tensor (the tied head uses the *unscaled* table:
v3/crates/rvllm-loader/src/gemma4_load.rs:431-457).

Head: logits = x @ W^T in 32-bit, W the embedding table when tied
(v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:4179-4187), then the optional
soft-cap cap * tanh(logits / cap) (v3/kernels/logit_softcap.cu:28).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import ParamSpec, Part
from .linear import linear
from .spec import PartSpec


class ScaledEmbedding(Part):
    def __init__(self, spec: PartSpec, *, hidden_size: int, vocab_size: int):
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.scale = float(spec.get("scale", 1.0))
        self.table: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [ParamSpec(f"{prefix}.embed_tokens.weight", (self.vocab_size, self.hidden_size))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        self.table = tensors[f"{prefix}.embed_tokens.weight"].to(device=device, dtype=dtype).contiguous()

    def forward(self, token_ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        return ops.embed_gather(self.table, token_ids, self.scale, out)


class LMHead(Part):
    def __init__(self, spec: PartSpec, *, hidden_size: int, vocab_size: int, embedding: ScaledEmbedding):
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.tied = bool(spec.get("tied", True))
        cap = spec.get("softcap")
        self.softcap = None if cap is None else float(cap)
        self.embedding = embedding
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        if self.tied:
            return []
        return [ParamSpec("lm_head.weight", (self.vocab_size, self.hidden_size))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        if self.tied:
            self.weight = self.embedding.table
        else:
            self.weight = tensors["lm_head.weight"].to(device=device, dtype=dtype).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = linear(x, self.weight, out_dtype=torch.float32)
        if self.softcap is not None:
            ops.softcap_(logits, self.softcap)
        return logits
