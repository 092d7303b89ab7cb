"""Random weights from a configuration and a seed: in memory, or as a model folder.

Every tensor is drawn from its own generator, seeded by a hash of (seed, tensor name), so
a tensor's values do not depend on which other tensors exist or in which order they are
made.  Matrices are N(0, std); norm weights are 1 + N(0, norm_std) (norm_std 0 gives
exactly 1).  Values are drawn in float32 and stored as bfloat16 (or float32 if asked).
The reference's inference crate has no such mode; its training crate seeds tensors by
name in the same spirit (crates/train/src/qwen3.rs:877-929).
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from ..models.decoder import expected_checkpoint_tensors
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def _init_normal(shape, gen, std, norm_std, device):
    return torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * std


def _init_ones(shape, gen, std, norm_std, device):
    t = torch.ones(shape, dtype=torch.float32, device=device)
    if norm_std:
        t += torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * norm_std
    return t


def _init_zeros(shape, gen, std, norm_std, device):
    return torch.zeros(shape, dtype=torch.float32, device=device)


# WeightDecl.init -> how a random tensor of that kind is filled: f(shape, generator, std, norm_std, device) -> float32
INITS = {"normal": _init_normal, "ones": _init_ones, "zeros": _init_zeros}


def register_init(name: str, fill) -> None:
    """Make `name` usable as WeightDecl.init: fill(shape, generator, std, norm_std, device) -> float32 tensor."""
    INITS[name] = fill


def random_tensor(name: str, decl, seed: int, std: float, norm_std: float, dtype, device="cpu"):
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    try:
        fill = INITS[decl.init]
    except KeyError:
        raise ValueError(f"tensor '{name}': no way to fill a weight of kind {decl.init!r} is registered "
                         f"(known: {', '.join(sorted(INITS))})") from None
    return fill(tuple(decl.shape), gen, std, norm_std, device).to(dtype)


def random_weights(spec, seed: int, std: float = 0.02, norm_std: float = 0.0,
                   dtype=torch.bfloat16, device="cpu") -> dict:
    """name -> tensor for every tensor the model expects.

    Drawn on `device`; values made on the CPU and on the GPU differ (different generators),
    so folders meant to be compared across machines are written from the CPU.
    """
    expected = expected_checkpoint_tensors(spec)
    return {name: random_tensor(name, decl, seed, std, norm_std, dtype, device)
            for name, decl in expected.items()}


def write_random_model(model_dir: str, arch_name: str, config, seed: int, std: float = 0.02,
                       norm_std: float = 0.0, dtype=torch.bfloat16) -> str:
    """Write config.json and model.safetensors for `config` with seeded random weights."""
    from ..config.registry import detect_architecture

    arch = detect_architecture({"architectures": [arch_name]})
    spec = arch.recipe(config, ())
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config.to_dict(), fh, indent=2)
    tensors = random_weights(spec, seed, std, norm_std, dtype, device="cpu")
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed, "std": std, "norm_std": norm_std})
    return model_dir
