"""A decoder built from a ``ModelSpec``: embedding, blocks run in the order
the schedule gives, final norm on the wanted rows, head.

Order inside a step (v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:3764-3960,
4168-4187): embed, every scheduled layer, final norm of the rows whose logits
are wanted, head.  Nothing here knows an architecture.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..parts import embedding as _embedding  # noqa: F401  (registers the embedding and the head)
from ..parts.base import ParamSpec
from ..parts.registry import BLOCKS, EMBEDDINGS, HEADS, NORMS
from ..parts.spec import ModelSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        H, V = spec.hidden_size, spec.vocab_size
        self.embedding = EMBEDDINGS.build(spec.embedding, hidden_size=H, vocab_size=V)
        self.blocks = [BLOCKS.build(layer.block, layer=layer, hidden_size=H) for layer in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm, width=H, name=spec.final_norm_name)
        self.head = HEADS.build(spec.head, hidden_size=H, vocab_size=V, embedding=self.embedding)
        self.device: Optional[torch.device] = None
        self.dtype: Optional[torch.dtype] = None

    # ---- weights -----------------------------------------------------
    def param_specs(self) -> list[ParamSpec]:
        specs = list(self.embedding.param_specs(self.spec.prefix))
        for layer, block in zip(self.spec.layers, self.blocks):
            specs += block.param_specs(layer.prefix)
        specs += self.final_norm.param_specs(self.spec.prefix)
        specs += self.head.param_specs(self.spec.prefix)
        names = [s.name for s in specs]
        if len(set(names)) != len(names):
            dup = sorted({n for n in names if names.count(n) > 1})
            raise ValueError(f"parts ask for the same tensor twice: {dup}")
        return specs

    def all_parts(self):
        """Every part of the model, the blocks and what they hold."""
        yield self.embedding
        for block in self.blocks:
            yield block
            yield from block.parts()
        yield self.final_norm
        yield self.head

    def bind(self, tensors: dict[str, torch.Tensor], device, dtype: torch.dtype, tiled_weights: bool = True) -> None:
        """``tiled_weights``: whether the parts keep their bf16 matrices a second time in tiles for the
        few-row product (``EngineConfig.tiled_weights``); each model carries its own setting."""
        self.device = torch.device(device)
        self.dtype = dtype
        self.tiled_weights = bool(tiled_weights)
        for part in self.all_parts():
            part.tiled_weights = self.tiled_weights
        self.embedding.bind(tensors, self.spec.prefix, self.device, dtype)
        for layer, block in zip(self.spec.layers, self.blocks):
            block.bind(tensors, layer.prefix, self.device, dtype)
        self.final_norm.bind(tensors, self.spec.prefix, self.device, dtype)
        self.head.bind(tensors, self.spec.prefix, self.device, dtype)

    def weight_bytes(self) -> int:
        """Bytes the bound weights take on the device, every allocation counted once (a tied head shares the
        embedding's table; a matrix in tiles counts with the rows kept beside it)."""
        from ..kernels.ops import TiledWeight

        seen: dict[int, int] = {}

        def count(value):
            if isinstance(value, TiledWeight):
                count(value.tiles)
                count(value.rows)
            elif isinstance(value, torch.Tensor) and value.device.type != "cpu":
                storage = value.untyped_storage()
                seen[storage.data_ptr()] = storage.nbytes()
            elif isinstance(value, (list, tuple)):
                for item in value:
                    count(item)

        for part in self.all_parts():
            for value in vars(part).values():
                count(value)
        return sum(seen.values())

    @property
    def capturable(self) -> bool:
        """Whether a step of this model may be recorded into a HIP graph: only if every part may."""
        return all(part.capturable for part in (self.embedding, *self.blocks, self.final_norm, self.head))

    # ---- cache needs ---------------------------------------------------
    def cache_needs(self) -> list:
        """For every layer what its mixer keeps between steps (or None for a
        layer that only ever reads another layer's cache)."""
        owners = {e.layer for e in self.spec.schedule if e.cache_from is None}
        return [block.mixer.cache_need() if i in owners else None for i, block in enumerate(self.blocks)]

    # ---- run ---------------------------------------------------------
    def forward(self, step, caches: list) -> torch.Tensor:
        """Runs the step's tokens; returns float32 logits ``[wanted rows, vocab]``.

        ``caches[i]`` is the cache view of layer i."""
        x = torch.empty((step.num_tokens, self.spec.hidden_size), dtype=self.dtype, device=self.device)
        self.embedding.forward(step, x)
        schedule = self.spec.schedule
        entered = None
        for i, entry in enumerate(schedule):
            block = self.blocks[entry.layer]
            cache = caches[entry.layer] if entry.cache_from is None else caches[entry.cache_from].reader()
            nxt = self.blocks[schedule[i + 1].layer].entry_norm() if i + 1 < len(schedule) else None
            # None means the block did not apply the next entry norm; the next block then does
            entered = block.forward(x, step, cache, entered=entered, then=nxt)
        if step.num_logit_rows == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        normed = self.final_norm.forward_rows(x, step.logit_rows)
        return self.head.forward(normed)
