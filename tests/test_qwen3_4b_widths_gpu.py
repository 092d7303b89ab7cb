"""The widths of Qwen3-4B (hidden 2560, 32/8 heads of 128, intermediate 9728, vocabulary 151936, tied head)
with one layer and random weights: the kernels at the sizes they are tuned for, against the plain
implementation, in the four cuttings.  The tiny configurations never reach these paths (the register-resident
norm of 2560 columns, the few-rows product with K split eight ways, head_dim 128 with the LDS-staged portions)."""
import pytest
import torch

import replay
from arle_amd.config import Qwen3Config
from arle_amd.engine import Engine
from arle_amd.weights import write_random_model
from tiny import ARCH, random_tokens, read_folder

pytestmark = pytest.mark.gpu

WIDTHS = dict(num_hidden_layers=1, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
              intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=True, max_position_embeddings=4096)
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("widths") / "model")
    write_random_model(d, ARCH, Qwen3Config.from_dict(WIDTHS), seed=17, std=0.02, norm_std=0.0)
    cfg, weights = read_folder(d)
    requests = {"a": random_tokens(44, WIDTHS["vocab_size"], 5), "b": random_tokens(25, WIDTHS["vocab_size"], 6)}
    reference = {rid: replay.plain_logits(cfg, weights, toks).float() for rid, toks in requests.items()}
    return d, requests, reference


def _compare(got, requests, reference, tol, what):
    replay.check_rows(got, {rid: reference[rid].double() for rid in requests}, tol, what, need_all=False)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_cuttings_at_the_widths_of_qwen3_4b(folder, dtype):
    d, requests, reference = folder
    eng = Engine.from_folder(d, dtype=dtype, page_size=16, max_tokens=256, max_slots=4)
    a = {"a": requests["a"]}
    got = replay.run_steps(eng, replay.whole("a", requests["a"]))
    assert len(got) == len(requests["a"])
    _compare(got, a, reference, TOL[dtype], f"whole/{dtype}")
    got = replay.run_steps(eng, replay.prefill_then_decode("a", requests["a"], tail=12))
    _compare(got, a, reference, TOL[dtype], f"prefill then decode/{dtype}")
    got = replay.run_steps(eng, replay.portions("a", requests["a"], sizes=(17, 2, 5, 1, 9)))
    _compare(got, a, reference, TOL[dtype], f"portions/{dtype}")
    got = replay.run_steps(eng, replay.mixed(requests, max_live=2, seed=3))
    assert len(got) == sum(len(t) for t in requests.values())
    _compare(got, requests, reference, TOL[dtype], f"mixed/{dtype}")
