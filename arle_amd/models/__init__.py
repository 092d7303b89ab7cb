"""Architectures known to the registry.  Importing this package registers them."""
from . import qwen3  # noqa: F401
from .decoder import (DecoderModel, build_model, declared_cache_needs, expected_checkpoint_tensors,
                      kv_cache_bytes_per_token)

__all__ = ["DecoderModel", "build_model", "declared_cache_needs", "expected_checkpoint_tensors",
           "kv_cache_bytes_per_token"]
