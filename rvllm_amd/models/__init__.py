"""Architectures.  Importing the package registers the ones the framework ships."""

from . import gemma3  # noqa: F401  (registers itself)
from .model import DecoderModel
from .registry import (Architecture, architecture_names, architecture_of, get_architecture, load_config,
                       register_architecture, unregister_architecture)

__all__ = ["DecoderModel", "Architecture", "architecture_names", "architecture_of", "get_architecture", "load_config",
           "register_architecture", "unregister_architecture"]
