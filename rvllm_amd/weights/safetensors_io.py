"""Reader and writer for safetensors files.

A file is ``[u64 little-endian header length][JSON header][payload]``; the
header maps each tensor name to its dtype, shape and byte range in the
payload.  The reader maps the file into memory and hands out tensors without
copying.  The checks are the reference parser's
(v3/crates/rvllm-loader/src/safetensors.rs:117-285): header length and JSON,
duplicate names, known dtypes, rank, ``dtype * shape == byte range``, ranges
inside the file and not overlapping.  A folder may hold one
``model.safetensors`` or several shards listed by
``model.safetensors.index.json`` (safetensors.rs:325-421).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from pathlib import Path
from typing import Iterable, Optional

import torch

MAX_HEADER_BYTES = 100 << 20
MAX_RANK = 16

DTYPES: dict[str, tuple[torch.dtype, int]] = {
    "F64": (torch.float64, 8),
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAME_OF = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    """The file is not a well-formed safetensors file."""


def _no_duplicates(pairs):
    out = {}
    for k, v in pairs:
        if k in out:
            raise SafetensorsError(f"duplicate key {k!r} in header")
        out[k] = v
    return out


class TensorEntry:
    __slots__ = ("name", "dtype_name", "shape", "begin", "end")

    def __init__(self, name, dtype_name, shape, begin, end):
        self.name, self.dtype_name, self.shape, self.begin, self.end = name, dtype_name, shape, begin, end


class SafetensorsFile:
    """One mapped file.  ``tensor(name)`` returns a CPU tensor that shares the
    mapping's memory; copy it (``.to(device)``) before the file is closed."""

    def __init__(self, path: str | os.PathLike):
        self.path = Path(path)
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError(f"{self.path}: shorter than its length field")
        self._fh = open(self.path, "rb")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if hlen > MAX_HEADER_BYTES or 8 + hlen > size:
            raise SafetensorsError(f"{self.path}: header length {hlen} does not fit the file of {size} bytes")
        try:
            header = json.loads(self._map[8 : 8 + hlen].decode("utf-8"), object_pairs_hook=_no_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{self.path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{self.path}: header must be an object")
        self.metadata = header.pop("__metadata__", None)
        self.data_start = 8 + hlen
        payload = size - self.data_start
        self.entries: dict[str, TensorEntry] = {}
        spans = []
        for name, info in header.items():
            if not isinstance(info, dict):
                raise SafetensorsError(f"{self.path}: entry {name!r} is not an object")
            dtype_name = info.get("dtype")
            shape = info.get("shape")
            offsets = info.get("data_offsets")
            if dtype_name not in DTYPES:
                raise SafetensorsError(f"{self.path}: tensor {name!r} has unsupported dtype {dtype_name!r}")
            if not isinstance(shape, list) or len(shape) > MAX_RANK or any(
                    isinstance(d, bool) or not isinstance(d, int) or d < 0 for d in shape):
                raise SafetensorsError(f"{self.path}: tensor {name!r} has a bad shape {shape!r}")
            if (not isinstance(offsets, list) or len(offsets) != 2
                    or any(isinstance(o, bool) or not isinstance(o, int) for o in offsets)):
                raise SafetensorsError(f"{self.path}: tensor {name!r} has bad data_offsets {offsets!r}")
            begin, end = offsets
            count = 1
            for d in shape:
                count *= d
            if not 0 <= begin <= end <= payload:
                raise SafetensorsError(f"{self.path}: tensor {name!r} lies outside the file ({begin}..{end} of {payload})")
            if end - begin != count * DTYPES[dtype_name][1]:
                raise SafetensorsError(
                    f"{self.path}: tensor {name!r}: {dtype_name}{shape} needs {count * DTYPES[dtype_name][1]} bytes, "
                    f"its range holds {end - begin}")
            self.entries[name] = TensorEntry(name, dtype_name, tuple(shape), begin, end)
            if end > begin:
                spans.append((begin, end, name))
        spans.sort()
        for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
            if b1 < e0:
                raise SafetensorsError(f"{self.path}: tensors {n0!r} and {n1!r} overlap")

    def names(self) -> list[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        dtype, _ = DTYPES[e.dtype_name]
        count = 1
        for d in e.shape:
            count *= d
        if count == 0:
            return torch.empty(e.shape, dtype=dtype)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)  # the mapping is read-only and nothing writes to it
            flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self.data_start + e.begin)
        return flat.view(e.shape)

    def close(self) -> None:
        # Tensors handed out keep the mapping alive through the buffer
        # protocol; closing while they live raises BufferError, which is
        # ignored here: the mapping then goes away with its last tensor.
        try:
            self._map.close()
        except BufferError:
            pass
        self._fh.close()


def read_shard_index(model_dir: str | os.PathLike) -> Optional[dict[str, str]]:
    """tensor name -> file name from model.safetensors.index.json, or None when the folder has no index.
    File names must be plain relative paths that stay inside the folder
    (v3/crates/rvllm-loader/src/safetensors.rs:325-421)."""
    root = Path(model_dir).resolve()
    index = root / "model.safetensors.index.json"
    if not index.is_file():
        return None
    try:
        doc = json.loads(index.read_text(), object_pairs_hook=_no_duplicates)
        weight_map = doc["weight_map"]
        assert isinstance(weight_map, dict)
    except (json.JSONDecodeError, KeyError, AssertionError, SafetensorsError) as e:
        raise SafetensorsError(f"{index}: not a valid shard index: {e}") from None
    for name, fname in weight_map.items():
        if not isinstance(fname, str) or not fname:
            raise SafetensorsError(f"{index}: the file of tensor {name!r} is no file name: {fname!r}")
        parts = Path(fname).parts
        if Path(fname).is_absolute() or any(part in ("..", ".") for part in parts) or \
                root not in (root / fname).resolve().parents:
            raise SafetensorsError(f"{index}: shard {fname!r} leaves the model folder")
    return weight_map


def resolve_shards(model_dir: str | os.PathLike) -> list[Path]:
    """The safetensors files of a model folder."""
    root = Path(model_dir).resolve()
    weight_map = read_shard_index(root)
    if weight_map is not None:
        files = []
        for fname in dict.fromkeys(weight_map.values()):
            p = (root / fname).resolve()
            if not p.is_file():
                raise SafetensorsError(f"{root / 'model.safetensors.index.json'}: shard {fname!r} not found")
            files.append(p)
        return files
    single = root / "model.safetensors"
    if single.is_file():
        return [single]
    raise SafetensorsError(f"{root}: neither model.safetensors nor model.safetensors.index.json found")


def write_safetensors(path: str | os.PathLike, tensors: dict[str, torch.Tensor],
                      metadata: Optional[dict[str, str]] = None) -> None:
    header: dict = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _NAME_OF:
            raise SafetensorsError(f"cannot store dtype {t.dtype} of {name!r}")
        t = t.detach().cpu().contiguous()
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAME_OF[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        blobs.append(raw)
        offset += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * (-len(text) % 8)
    tmp = Path(str(path) + ".tmp")
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for raw in blobs:
            f.write(raw)
    os.replace(tmp, path)
