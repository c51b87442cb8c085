"""Random weights from a configuration and a seed.

``write_random_model`` writes a model folder (config.json, model.safetensors)
that loads like any checkpoint, so tests exercise the loader;
``random_tensors`` fills tensors directly on a device for sizes where a file
would only cost time.  Matrices are N(0, 0.02), zero-centred norm weights
N(0, 0.1) (each part names the law of its tensors in its ``ParamSpec``).  The
reference has no such mode; its bench runs on zeroed activations
(v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:1782-1786).
"""

from __future__ import annotations

import json
import os
import zlib
from pathlib import Path
from typing import Any, Sequence

import torch

from ..parts.base import ParamSpec
from .safetensors_io import write_safetensors


def _fill(spec: ParamSpec, seed: int, device, dtype: torch.dtype) -> torch.Tensor:
    # One generator per tensor, seeded by (seed, name): a tensor's values do
    # not depend on which other tensors exist or on their order.
    gen = torch.Generator(device=device)
    gen.manual_seed((int(seed) * 1000003 + zlib.crc32(spec.name.encode())) % (1 << 63))
    kind = spec.init[0]
    if kind == "normal":
        t = torch.empty(spec.shape, dtype=torch.float32, device=device)
        t.normal_(0.0, float(spec.init[1]), generator=gen)
        return t.to(dtype)
    if kind == "randint":
        return torch.randint(int(spec.init[1]), int(spec.init[2]), spec.shape, generator=gen, device=device,
                             dtype=torch.int32)
    if kind == "zeros":
        return torch.zeros(spec.shape, dtype=torch.int32 if spec.integer else dtype, device=device)
    raise ValueError(f"unknown init {spec.init!r} for {spec.name}")


def random_tensors(specs: Sequence[ParamSpec], seed: int, device="cpu",
                   dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    return {s.name: _fill(s, seed, device, dtype) for s in specs}


def write_random_model(model_dir: str | os.PathLike, config: Any, seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write config.json and model.safetensors for ``config`` (a typed
    configuration of a registered architecture)."""
    from ..models.model import DecoderModel
    from ..models.registry import get_architecture

    arch = get_architecture(config.architecture)
    model = DecoderModel(arch.build_spec(config))
    tensors = random_tensors(model.param_specs(), seed, "cpu", dtype)
    out = Path(model_dir)
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(arch.write_config(config), indent=2))
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt", "seed": str(seed)})
    return out
