"""Weights by tensor name.

The model says which tensors it wants (name, shape); the loader finds them in
the folder's safetensors files and reports everything that does not fit in one
error: tensors that are missing, tensors nobody asked for, wrong shapes.  The
reference looks tensors up by name and checks every shape the same way
(v3/crates/rvllm-loader/src/gemma4_load.rs:65-104,504-521,1970-1994), one
error at a time.

Types: floating tensors stored in 16 bits are kept as bfloat16; a tensor
stored in 32 bits stays 32-bit; integer tables become int32.  With a 32-bit
engine every floating tensor is widened to float32 (exact).
"""

from __future__ import annotations

import os
import warnings
from pathlib import Path
from typing import Sequence

import torch

from ..parts.base import ParamSpec
from .safetensors_io import SafetensorsError, SafetensorsFile, read_shard_index, resolve_shards

class WeightError(ValueError):
    """Everything that is wrong with a folder's tensors, in one message."""

    def __init__(self, source: str, missing: Sequence[str] = (), unexpected: Sequence[str] = (),
                 wrong_shape: Sequence[tuple[str, tuple, tuple]] = (), other: Sequence[str] = ()):
        self.source = source
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"{source}: the tensors do not fit the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: expected {list(exp)}, got {list(got)}" for n, exp, got in self.wrong_shape))
        for text in self.other:
            lines.append("  " + text)
        super().__init__("\n".join(lines))


def open_model_files(model_dir: str | os.PathLike) -> list[SafetensorsFile]:
    """The folder's safetensors files, opened.  Where an index says which file
    holds which tensor, every tensor must lie in the file the index names."""
    files = [SafetensorsFile(p) for p in resolve_shards(model_dir)]
    weight_map = read_shard_index(model_dir)
    if weight_map is not None:
        root = Path(model_dir).resolve()
        held = {f.path.resolve(): set(f.names()) for f in files}
        astray = [f"{name!r} is not in {fname}" for name, fname in weight_map.items()
                  if name not in held.get((root / fname).resolve(), ())]
        if astray:
            for f in files:
                f.close()
            raise SafetensorsError(f"{model_dir}: the shard index names tensors that their files do not hold: "
                                   + "; ".join(astray[:8]) + (" ..." if len(astray) > 8 else ""))
    return files


def tensor_names(files: Sequence[SafetensorsFile]) -> list[str]:
    return [n for f in files for n in f.names()]


def _keep_dtype(t: torch.Tensor, integer: bool, engine_dtype: torch.dtype) -> torch.Tensor:
    if integer:
        return t.to(torch.int32)
    if engine_dtype == torch.float32:
        return t.to(torch.float32)
    if t.dtype in (torch.float32, torch.float64):
        return t.to(torch.float32)  # stored in 32 bits (or more): stays 32-bit
    return t.to(torch.bfloat16)


def load_tensors(files: Sequence[SafetensorsFile], specs: Sequence[ParamSpec], engine_dtype: torch.dtype,
                 source: str = "model folder", ignore: Sequence[str] = ()) -> dict[str, torch.Tensor]:
    """The tensors the specs name, as CPU tensors.  ``ignore`` lists name
    prefixes of tensors that may be present without being asked for (the
    other parts of a multimodal checkpoint)."""
    where: dict[str, SafetensorsFile] = {}
    dup = []
    for f in files:
        for n in f.names():
            if n in where:
                dup.append(f"tensor {n!r} appears in more than one file")
            where[n] = f
    wanted = {s.name: s for s in specs}
    missing = [n for n in wanted if n not in where]
    unexpected = [n for n in where if n not in wanted and not any(n.startswith(p) for p in ignore)]
    wrong_shape = []
    wrong_kind = []
    for n, s in wanted.items():
        if n in where:
            e = where[n].entries[n]
            if tuple(e.shape) != tuple(s.shape):
                wrong_shape.append((n, tuple(s.shape), tuple(e.shape)))
            is_int = e.dtype_name in ("I64", "I32", "I16", "I8", "U8", "BOOL")
            if is_int != s.integer:
                wrong_kind.append(f"tensor {n!r} is stored as {e.dtype_name}, expected "
                                  + ("an integer table" if s.integer else "floating values"))
    if missing or unexpected or wrong_shape or dup or wrong_kind:
        raise WeightError(source, missing, unexpected, wrong_shape, dup + wrong_kind)
    out = {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", UserWarning)  # the mapping is read-only; nothing writes to it
        for n, s in wanted.items():
            out[n] = _keep_dtype(where[n].tensor(n), s.integer, engine_dtype)
    return out
