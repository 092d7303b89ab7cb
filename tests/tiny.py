"""Tiny Qwen3 configurations for tests, and helpers that make model folders from them.

A and B differ in every size and option: layers, widths (B's are no powers of two), head
counts and group size, head_dim (B's q width differs from its hidden size), vocabulary,
eps, theta, tied or untied head, page size and the spread of the weights.  C has a head_dim
that is a multiple of 16 but no power of two and odd-ish widths.
"""
from __future__ import annotations

import json
import os

import torch

from arle_amd.config import Qwen3Config
from arle_amd.weights import write_random_model

ARCH = "Qwen3ForCausalLM"

TINY_A = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=1024)
TINY_B = dict(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=2,
              head_dim=32, intermediate_size=224, vocab_size=384, rope_theta=1000000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=2048)
TINY_C = dict(num_hidden_layers=2, hidden_size=88, num_attention_heads=3, num_key_value_heads=1,
              head_dim=48, intermediate_size=136, vocab_size=333, rope_theta=50000.0,
              rms_norm_eps=3e-6, tie_word_embeddings=False, max_position_embeddings=1024)

# D: head_dim 64 (the matrix-core kernels with a compile-time head_dim), a group of four, a page of 32 slots;
# E: head_dim 96 (their run-time head_dim variants, three quarters of a 128 tile), two kv heads of three q heads.
TINY_D = dict(num_hidden_layers=2, hidden_size=120, num_attention_heads=8, num_key_value_heads=2,
              head_dim=64, intermediate_size=200, vocab_size=1003, rope_theta=300000.0,
              rms_norm_eps=2e-6, tie_word_embeddings=True, max_position_embeddings=2048)
TINY_E = dict(num_hidden_layers=2, hidden_size=104, num_attention_heads=6, num_key_value_heads=2,
              head_dim=96, intermediate_size=168, vocab_size=517, rope_theta=20000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=1024)

# F: a head_dim that is even but no multiple of 16: the float32 kernels take it, the bfloat16 ones refuse it
TINY_F = dict(num_hidden_layers=2, hidden_size=56, num_attention_heads=4, num_key_value_heads=2,
              head_dim=24, intermediate_size=100, vocab_size=211, rope_theta=30000.0,
              rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=512)

# name -> (config, page size, weight std, norm std, seed)
TINY = {
    "A": (TINY_A, 4, 0.02, 0.02, 11),
    "B": (TINY_B, 8, 0.05, 0.05, 22),
    "C": (TINY_C, 16, 0.08, 0.1, 33),
    "D": (TINY_D, 32, 0.06, 0.05, 44),
    "E": (TINY_E, 16, 0.07, 0.08, 55),
    "F": (TINY_F, 8, 0.07, 0.06, 66),
}


def make_model_dir(tmp_path, name: str, std_scale: float = 1.0) -> str:
    raw, _, std, norm_std, seed = TINY[name]
    config = Qwen3Config.from_dict(raw)
    d = os.path.join(str(tmp_path), f"tiny_{name}")
    write_random_model(d, ARCH, config, seed=seed, std=std * std_scale, norm_std=norm_std)
    return d


def read_folder(model_dir: str):
    """(config dict, {name: float32 CPU tensor}) read straight from the files, with the `safetensors`
    package's reader: the plain side shares no reader with the engine."""
    from safetensors.torch import load_file

    with open(os.path.join(model_dir, "config.json")) as fh:
        cfg = json.load(fh)
    weights = {n: t.to(torch.float32) for n, t in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, weights


def random_tokens(n: int, vocab: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
