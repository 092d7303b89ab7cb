"""Qwen3-4B whole: all 36 layers at its real widths, random bfloat16 weights, float32 and bfloat16, four cuttings.

The plain side never holds the model: it takes one layer's tensors at a time from the weights the engine was built
from, widens them to float64 on the CPU and runs `plain_qwen3.decoder_layer` on the hidden states of both requests.
(The reference's witnesses for "a batch equals its requests alone" at full depth: crates/train/src/qwen3.rs:945-981,
infer/tests/greedy_consistency.rs:205-240.)  A tensor's random values depend on the seed and its name only, so the
first k layers of this model are the k-layer model: the plain hidden states after layers 1, 4 and 12 also give the
logits that engines of those depths must produce, which is how the growth of the error with depth is read off."""
import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd.config import Qwen3Config
from arle_amd.config.registry import detect_architecture
from arle_amd.engine import Engine
from arle_amd.weights.random_init import random_weights
from tiny import ARCH, random_tokens

pytestmark = pytest.mark.gpu

QWEN3_4B = dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=True, max_position_embeddings=4096)
# bfloat16: the error against the exact logits grows with depth, since every layer adds two sums of products of
# activations rounded to bfloat16: measured against this file's plain side at depths 1 / 2 / 4 / 8 / 12 / 24 / 36 of
# this model, the worst of all rows and cuttings relative to the largest logit: 0.70 / 0.92 / 1.09 / 1.53 / 1.49 / 2.0 /
# 2.1 e-2 (float32: 0.34 / 0.44 / 0.57 / 0.68 / 0.88 / 0.95 / 1.08 e-5 with one chain of additions over K, and
# 0.19e-5 at depth 36 since the float32 product adds in three levels).  The tolerance of the two- to four-layer tests
# (2e-2) is what depth 36 measures, so this depth has 3e-2: a bound on rounding, not a net for small faults,
# which the float32 engine (the same cache, batching and layout at 1e-5) and the kernels' own tests catch.
TOL = {"float32": 1e-5, "bfloat16": 3e-2}
SEED, STD = 4, 0.02


def spec_of(layers: int):
    raw = dict(QWEN3_4B, num_hidden_layers=layers)
    return raw, detect_architecture({"architectures": [ARCH]}).recipe(Qwen3Config.from_dict(raw), ())


def plain_logits_by_depth(tensors: dict, raw: dict, requests: dict, depths) -> dict:
    """{depth: {request: float64 logits [T, V]}}: the plain implementation layer by layer, one layer's tensors in
    float64 on the CPU at a time; after each depth asked for, the final norm and the (tied) head."""
    wide = lambda name: tensors[name].to("cpu", torch.float64)
    table = wide("model.embed_tokens.weight")
    final = wide("model.norm.weight")
    hidden = {rid: plain.embedding(table, toks) for rid, toks in requests.items()}
    out = {}
    for layer in range(raw["num_hidden_layers"]):
        prefix = f"model.layers.{layer}."
        w = {name: wide(name) for name in tensors if name.startswith(prefix)}
        for rid, toks in requests.items():
            hidden[rid] = plain.decoder_layer(hidden[rid], w, layer, raw, list(range(len(toks))))
        if layer + 1 in depths:
            out[layer + 1] = {rid: plain.linear(plain.rms_norm(h, final, raw["rms_norm_eps"]), table)
                              for rid, h in hidden.items()}
    return out


@pytest.fixture(scope="module")
def model():
    raw, spec = spec_of(36)
    tensors = random_weights(spec, SEED, STD, 0.0, torch.bfloat16, device=torch.device("cuda:0"))
    requests = {"a": random_tokens(41, raw["vocab_size"], 7), "b": random_tokens(23, raw["vocab_size"], 8)}
    reference = plain_logits_by_depth(tensors, raw, requests, {36})[36]
    return spec, tensors, requests, reference


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_cuttings_of_qwen3_4b_at_all_36_layers(model, dtype):
    spec, tensors, requests, reference = model
    act = torch.float32 if dtype == "float32" else torch.bfloat16
    eng = Engine(spec, {k: v.to(act) for k, v in tensors.items()}, dtype=dtype, page_size=16, max_tokens=256, max_slots=4)
    assert len(eng.model.blocks) == 36
    a = {"a": reference["a"]}
    got = replay.run_steps(eng, replay.whole("a", requests["a"]))
    replay.check_rows(got, a, TOL[dtype], f"4B x 36 whole/{dtype}")
    got = replay.run_steps(eng, replay.prefill_then_decode("a", requests["a"], tail=32))
    replay.check_rows(got, a, TOL[dtype], f"4B x 36 prefill then 32 decoded/{dtype}")
    got = replay.run_steps(eng, replay.portions("a", requests["a"], sizes=(17, 2, 5, 1, 9)))
    replay.check_rows(got, a, TOL[dtype], f"4B x 36 portions/{dtype}")
    got = replay.run_steps(eng, replay.mixed(requests, max_live=2, seed=3))
    assert len(got) == sum(len(t) for t in requests.values())
    replay.check_rows(got, reference, TOL[dtype], f"4B x 36 mixed/{dtype}")
    assert all(f == g.pool.num_pages for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
