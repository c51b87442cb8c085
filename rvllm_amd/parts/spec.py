"""The description of a model as data.

A model is an embedding, a list of layers, the order in which the layers run,
a final norm and a head.  Every layer names its parts by registry key and
gives each part its sizes and constants; nothing here knows an architecture.
An architecture module turns its typed configuration into one ``ModelSpec``;
everything below it (weights, cache groups, the step function) reads only the
spec.  The reference passes per-layer sizes and constants to its layer code the
same way, through ``Gemma4LayerDims``
(v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:44-76).
"""

from __future__ import annotations

import dataclasses
from types import MappingProxyType
from typing import Any, Mapping, Optional


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """One part: its registry key and its parameters."""

    kind: str
    params: Mapping[str, Any] = dataclasses.field(default_factory=dict)

    def __post_init__(self):
        object.__setattr__(self, "params", MappingProxyType(dict(self.params)))

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer: the arrangement and the parts it arranges.

    ``prefix`` is the name under which the layer's tensors are stored."""

    prefix: str
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norm: PartSpec


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``cache_from`` names the layer whose cache this
    run reads instead of keeping one of its own."""

    layer: int
    cache_from: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    prefix: str = "model"
    final_norm_name: str = "norm"  # the final norm's tensor is <prefix>.<final_norm_name>.weight

    def __post_init__(self):
        n = len(self.layers)
        owners = set()
        for entry in self.schedule:
            if not 0 <= entry.layer < n:
                raise ValueError(f"schedule names layer {entry.layer}, model has {n}")
            if entry.cache_from is None:
                owners.add(entry.layer)
        for entry in self.schedule:
            if entry.cache_from is not None and entry.cache_from not in owners:
                raise ValueError(
                    f"layer {entry.layer} reads the cache of layer {entry.cache_from}, "
                    "which never runs with a cache of its own"
                )
