"""The one registry from an architecture's name to its model.

config.json's ``architectures[0]`` picks the entry, as in the reference
(v3/crates/rvllm-core/src/config/model.rs:14-36,71-80).  An entry knows how to
read its configuration, how its checkpoints name their tensors, and how to
turn both into a ``ModelSpec``; everything else is shared.
"""

from __future__ import annotations

import dataclasses
import json
import os
from pathlib import Path
from typing import Any, Callable, Iterable

from ..config.errors import ConfigError, UnknownArchitectureError
from ..parts.spec import ModelSpec

MAX_CONFIG_BYTES = 4 << 20  # v3/crates/rvllm-core/src/config/model.rs:11


def _names_as_written(names: Iterable[str]) -> dict:
    return {}


@dataclasses.dataclass(frozen=True)
class Architecture:
    """``locate_tensors`` looks at the names a checkpoint holds and returns the
    keyword arguments for ``build_spec`` that say where this architecture's
    tensors lie in it (a prefix, the name of an untied head, ...);
    ``ignored_prefixes`` are name prefixes of tensors such a checkpoint may hold
    beside the model's (the other towers of a multimodal one).  The loader and
    the runner know no architecture's names: they ask here."""

    name: str
    read_config: Callable[[dict, str], Any]  # (config.json document, source) -> typed configuration
    build_spec: Callable[..., ModelSpec]  # (typed configuration, **locate_tensors(names)) -> model description
    write_config: Callable[[Any], dict]  # typed configuration -> config.json document
    locate_tensors: Callable[[Iterable[str]], dict] = _names_as_written
    ignored_prefixes: tuple[str, ...] = ()


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise KeyError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def architecture_names() -> list[str]:
    return sorted(_ARCHITECTURES)


def get_architecture(name: str, source: str = "config.json") -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitectureError(
            source, [f"unsupported architecture: {name!r}; supported: {', '.join(architecture_names())}"]
        ) from None


def read_config_file(model_dir: str | os.PathLike) -> tuple[dict, str]:
    """config.json of a model folder as a document, with the checks the
    reference makes on the file (a regular file inside the folder, at most
    4 MiB: v3/crates/rvllm-core/src/config/model.rs:249-282)."""
    root = Path(model_dir).resolve()
    path = (root / "config.json").resolve()
    source = str(path)
    if root not in path.parents:
        raise ConfigError(source, ["config.json leaves the model folder"])
    if not path.is_file():
        raise ConfigError(source, ["config.json not found or not a regular file"])
    if path.stat().st_size > MAX_CONFIG_BYTES:
        raise ConfigError(source, [f"config.json is larger than {MAX_CONFIG_BYTES} bytes"])
    try:
        doc = json.loads(path.read_text())
    except (json.JSONDecodeError, UnicodeDecodeError) as e:
        raise ConfigError(source, [f"not valid JSON: {e}"]) from None
    if not isinstance(doc, dict):
        raise ConfigError(source, ["top level must be a JSON object"])
    return doc, source


def architecture_of(doc: dict, source: str = "config.json") -> Architecture:
    archs = doc.get("architectures")
    if not (isinstance(archs, list) and archs and isinstance(archs[0], str)):
        raise ConfigError(source, ["missing or invalid required field architectures[0]"])
    return get_architecture(archs[0], source)


def load_config(model_dir: str | os.PathLike) -> tuple[Architecture, Any]:
    doc, source = read_config_file(model_dir)
    arch = architecture_of(doc, source)
    return arch, arch.read_config(doc, source)
