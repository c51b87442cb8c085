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
from .base import Embedding, Head, ParamSpec
from .linear import decode_weight, linear
from .registry import EMBEDDINGS, HEADS
from .spec import PartSpec


class ScaledEmbedding(Embedding):
    """Parameters: ``scale`` (1 if absent) and ``name``, the table's name under
    the model's prefix (``embed_tokens`` if absent)."""

    def __init__(self, spec: PartSpec, *, hidden_size: int, vocab_size: int):
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.scale = float(spec.get("scale", 1.0))
        self.name = str(spec.get("name", "embed_tokens"))
        self.table: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [ParamSpec(f"{prefix}.{self.name}.weight", (self.vocab_size, self.hidden_size))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        self.table = tensors[f"{prefix}.{self.name}.weight"].to(device=device, dtype=dtype).contiguous()

    def forward(self, step, out: torch.Tensor) -> torch.Tensor:
        return ops.embed_gather(self.table, step.token_ids, self.scale, out)


class LMHead(Head):
    """Parameters: ``tied`` (the head reads the embedding's table, which must
    then have a ``table``), ``softcap`` (None: off) and ``weight_name``, the
    whole name of an untied head's matrix (``lm_head.weight`` if absent: the
    reference looks it up under no prefix, gemma4_load.rs:431-436)."""

    def __init__(self, spec: PartSpec, *, hidden_size: int, vocab_size: int, embedding):
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.tied = bool(spec.get("tied", True))
        cap = spec.get("softcap")
        self.softcap = None if cap is None else float(cap)
        self.weight_name = str(spec.get("weight_name", "lm_head.weight"))
        self.embedding = embedding
        self.weight: Optional[torch.Tensor] = None
        if self.tied and not hasattr(embedding, "table"):
            raise ValueError("a tied head needs an embedding that keeps its table as `table`")

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        if self.tied:
            return []
        return [ParamSpec(self.weight_name, (self.vocab_size, self.hidden_size))]

    def bind(self, tensors, prefix, device, dtype) -> None:
        if self.tied:
            self.weight = decode_weight(self.embedding.table, self.tiled_weights)  # the table itself stays row by row for the lookup
        else:
            self.weight = decode_weight(tensors[self.weight_name].to(device=device, dtype=dtype).contiguous(),
                                        self.tiled_weights)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = linear(x, self.weight, out_dtype=torch.float32)
        if self.softcap is not None:
            ops.softcap_(logits, self.softcap)
        return logits


EMBEDDINGS.register("scaled_embedding", ScaledEmbedding)
HEADS.register("lm_head", LMHead)
