"""Architectures known to the registry.  Importing this package registers them."""
from . import qwen3  # noqa: F401
from .decoder import DecoderModel, build_model, expected_checkpoint_tensors

__all__ = ["DecoderModel", "build_model", "expected_checkpoint_tensors"]
