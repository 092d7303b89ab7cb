"""Long decoding, the first tokens of a sequence, and faults that random weights would hide."""
import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd.engine import Engine, StepEntry
from tiny import TINY, make_model_dir, random_tokens, read_folder

pytestmark = pytest.mark.gpu
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = make_model_dir(tmp_path_factory.mktemp("long"), "B")
    return (d, *read_folder(d))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_token_by_token(model_b, dtype):
    d, cfg, weights = model_b
    toks = random_tokens(330, cfg["vocab_size"], 9)
    eng = Engine.from_folder(d, dtype=dtype, page_size=TINY["B"][1], max_tokens=384, max_slots=2)
    steps = [{"entries": [("x", toks[:10], list(range(10)))], "end": []}]
    steps += [{"entries": [("x", [t], [0])], "end": []} for t in toks[10:]]
    got = replay.run_steps(eng, steps)
    replay.compare(got, cfg, weights, {"x": toks}, TOL[dtype], f"long decode/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(model_b, dtype):
    d, cfg, weights = model_b
    toks = random_tokens(6, cfg["vocab_size"], 10)
    eng = Engine.from_folder(d, dtype=dtype, page_size=TINY["B"][1], max_tokens=64, max_slots=2)
    got = replay.run_steps(eng, [{"entries": [("x", [t], [0])], "end": []} for t in toks])
    replay.compare(got, cfg, weights, {"x": toks}, TOL[dtype], f"first tokens/{dtype}")
    eng.end_request("x")
    got = replay.run_steps(eng, [{"entries": [("y", toks[:1], [0])], "end": []},
                                 {"entries": [("y", toks[1:3], [0, 1])], "end": []},
                                 {"entries": [("y", toks[3:], [0, 1, 2])], "end": ["y"]}])
    replay.compare(got, cfg, weights, {"y": toks}, TOL[dtype], f"first tokens in portions/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_and_a_page_edge_show_in_the_logits(model_b, dtype, tmp_path):
    """Scale one layer's q and k weights so that attention is sharp: a wrong key (off by one at a
    page's edge, a stale page, a missing far key) then changes the logits far beyond rounding."""
    from arle_amd.weights import write_safetensors
    import json, os

    d, cfg, weights = model_b
    sharp = {k: v.clone() for k, v in weights.items()}
    for name in ("q_norm", "k_norm"):
        sharp[f"model.layers.0.self_attn.{name}.weight"] *= 4.0   # scores x16
    sharp_dir = str(tmp_path / "sharp")
    os.makedirs(sharp_dir)
    json.dump(cfg, open(os.path.join(sharp_dir, "config.json"), "w"))
    write_safetensors(os.path.join(sharp_dir, "model.safetensors"), {k: v.bfloat16() for k, v in sharp.items()})
    cfg2, weights2 = read_folder(sharp_dir)
    toks = random_tokens(200, cfg["vocab_size"], 12)
    eng = Engine.from_folder(sharp_dir, dtype=dtype, page_size=TINY["B"][1], max_tokens=256, max_slots=2)
    got = replay.run_steps(eng, replay.portions("x", toks, sizes=(8, 9, 7, 16, 1, 24, 3)))
    replay.compare(got, cfg2, weights2, {"x": toks}, TOL[dtype] * (1 if dtype == "float32" else 2), f"sharp/{dtype}")
    # the test has teeth: reading one wrong key at a page's edge moves the last logits far beyond the tolerance
    other = list(toks)
    other[TINY["B"][1] - 1] = (other[TINY["B"][1] - 1] + 1) % cfg["vocab_size"]
    ref = plain.forward_logits(weights2, cfg2, toks, dtype=torch.float64)[-1]
    moved = plain.forward_logits(weights2, cfg2, other, dtype=torch.float64)[-1]
    assert float((ref - moved).abs().max() / ref.abs().max()) > 100 * TOL["float32"]


def test_step_refuses_bad_input(model_b):
    from arle_amd.cache import OutOfPages
    from arle_amd.engine import EngineError

    d, cfg, _ = model_b
    eng = Engine.from_folder(d, dtype="float32", page_size=8, max_tokens=32, max_slots=2)
    with pytest.raises(EngineError, match="not live"):
        eng.step([StepEntry("nobody", [1], [0])])
    eng.add_request("a")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.step([StepEntry("a", [cfg["vocab_size"]], [0])])
    with pytest.raises(ValueError, match="outside its"):
        eng.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(ValueError, match="twice"):
        eng.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1] * 33, [0])])
    assert eng.length("a") == 0 and eng.cache.free_pages() == [4]   # nothing was changed
    out = eng.step([StepEntry("a", [1, 2, 3], [])])
    assert out.shape == (0, cfg["vocab_size"]) and eng.length("a") == 3
