"""Sizes that nothing was tuned for: every configuration that the config class accepts either runs right in both
precisions or is refused with an error that says why; it never gives a wrong result.  Groups of q heads larger than a
row tile of the matrix-core attention (32 q heads on one kv head), odd group sizes (5, 7), no grouping at all, head
sizes 80, 112 and 256, widths that are no multiple of 8 (the 16-byte pieces of the bfloat16 kernels), a vocabulary
that is prime, pages of 4 and of 64 tokens."""
import os

import pytest
import torch

import replay
from arle_amd.config import Qwen3Config
from arle_amd.engine import Engine
from arle_amd.kernels.ops import ShapeError
from arle_amd.weights import write_random_model
from tiny import ARCH, random_tokens, read_folder

pytestmark = pytest.mark.gpu


def cfg(layers, hidden, nq, nkv, d, inter, vocab, theta=10000.0, eps=1e-6, tied=True):
    return dict(num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d,
                intermediate_size=inter, vocab_size=vocab, rope_theta=theta, rms_norm_eps=eps, tie_word_embeddings=tied,
                max_position_embeddings=1024)


ODD = {
    "one kv head under 32 q heads": (cfg(2, 96, 32, 1, 16, 136, 257), 4),
    "groups of five": (cfg(2, 80, 10, 2, 32, 104, 311, theta=5e5, tied=False), 8),
    "groups of seven, head_dim 112": (cfg(1, 72, 7, 1, 112, 88, 199, eps=1e-5), 16),
    "no grouping, head_dim 80": (cfg(2, 120, 5, 5, 80, 200, 509, tied=False), 16),
    "head_dim 256": (cfg(1, 64, 2, 1, 256, 96, 131), 64),
    "widths that are no multiple of 8": (cfg(2, 100, 4, 2, 32, 146, 1009, theta=3e4), 8),
    "an odd hidden size": (cfg(1, 67, 2, 2, 16, 45, 97, tied=False), 4),
}


@pytest.mark.parametrize("name", list(ODD))
@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_odd_sizes_run_right_or_are_refused_with_a_reason(tmp_path, name, dtype, tol):
    raw, page = ODD[name]
    d = os.path.join(str(tmp_path), "odd")
    write_random_model(d, ARCH, Qwen3Config.from_dict(raw), seed=3, std=0.08, norm_std=0.05)
    config, weights = read_folder(d)
    reqs = {f"r{i}": random_tokens(n, raw["vocab_size"], 40 + i) for i, n in enumerate([37, 70, 19, 52])}
    try:
        eng = Engine.from_folder(d, dtype=dtype, page_size=page, max_tokens=3 * 128, max_slots=3)
        got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=2))
        got.update(replay.run_steps(eng, replay.prefill_then_decode("w", reqs["r1"], tail=20)))
    except (ShapeError, ValueError) as refusal:
        assert dtype == "bfloat16", f"the float32 path takes every size: {refusal}"
        assert len(str(refusal)) > 20 and any(word in str(refusal) for word in ("multiple", "must", "supported", "takes"))
        return
    reqs["w"] = reqs["r1"]
    replay.compare(got, config, weights, reqs, tol, f"{name}/{dtype}")
    assert all(f == g.pool.num_pages for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
