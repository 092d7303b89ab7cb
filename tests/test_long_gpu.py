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


def _write_folder(folder, cfg, weights):
    import json, os
    from arle_amd.weights import write_safetensors

    os.makedirs(folder)
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: v.bfloat16() for k, v in weights.items()})
    return read_folder(folder)


def test_sharp_attention_shows_a_wrong_key_in_float32(model_b, tmp_path):
    """Scale one layer's q and k norm weights so that attention is sharp: a wrong key (off by one at a
    page's edge, a stale page, a missing far key) then changes the logits far beyond the float32
    tolerance.  (In bfloat16 sharp but unsaturated scores amplify the rounding of the stored keys just as
    much as they amplify a fault, so that mode is tested with saturated scores below.)"""
    d, cfg, weights = model_b
    sharp = {k: v.clone() for k, v in weights.items()}
    for name in ("q_norm", "k_norm"):
        sharp[f"model.layers.0.self_attn.{name}.weight"] *= 4.0   # scores x16
    cfg2, weights2 = _write_folder(str(tmp_path / "sharp"), cfg, sharp)
    toks = random_tokens(200, cfg["vocab_size"], 12)
    eng = Engine.from_folder(str(tmp_path / "sharp"), dtype="float32", page_size=TINY["B"][1], max_tokens=256, max_slots=2)
    got = replay.run_steps(eng, replay.portions("x", toks, sizes=(8, 9, 7, 16, 1, 24, 3)))
    # scores sixteen times as large amplify rounding unevenly (a row with two near-equal top keys more than one
    # with a clear winner): rows differ by up to five times the median here, where other comparisons stay under three
    replay.compare(got, cfg2, weights2, {"x": toks}, TOL["float32"], "sharp/float32", outlier_tol=10.0)
    # the test has teeth: reading one wrong key at a page's edge moves the last logits far beyond the tolerance
    other = list(toks)
    other[TINY["B"][1] - 1] = (other[TINY["B"][1] - 1] + 1) % cfg["vocab_size"]
    ref = plain.forward_logits(weights2, cfg2, toks, dtype=torch.float64)[-1]
    moved = plain.forward_logits(weights2, cfg2, other, dtype=torch.float64)[-1]
    assert float((ref - moved).abs().max() / ref.abs().max()) > 100 * TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_planted_keys_at_page_edges_and_far_away_decide_the_logits(model_b, dtype, tmp_path):
    """Layer 0 is made to look at one key only, with a margin that rounding cannot close.

    Hidden column 0 is a positive constant in every embedding row and feeds, through q_proj, the
    slowest-rotating dimension of every query head; hidden column 1 is zero except for three planted
    tokens and feeds the same dimension of every key head; the q/k norm weights of that dimension are
    large.  Every query therefore gives all its weight to the strongest planted key so far.  The three
    are placed at position 0 (soon hundreds of keys away), in the last slot of a page and in the first
    slot of a page, so a kernel that drops a far page, a page's last slot, the newest key or a page's
    first slot returns another token's value.  Saturated scores do not amplify rounding, so bfloat16
    keeps its ordinary tolerance."""
    d, cfg, weights = model_b
    P, D, nq, nkv = TINY["B"][1], cfg["head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    w = {k: v.clone() for k, v in weights.items()}
    emb, slow = w["model.embed_tokens.weight"], D // 2 - 1      # NeoX pair (D/2-1, D-1) turns slowest
    planted = {cfg["vocab_size"] - 3: 0.05, cfg["vocab_size"] - 2: 0.10, cfg["vocab_size"] - 1: 0.15}
    emb[:, 0], emb[:, 1] = 0.15, 0.0
    for tok, level in planted.items():
        emb[tok, 1] = level
    pre = "model.layers.0.self_attn."
    for h in range(nq):
        w[pre + "q_proj.weight"][h * D + slow] = 0.0
        w[pre + "q_proj.weight"][h * D + slow, 0] = 2.0
    for h in range(nkv):
        w[pre + "k_proj.weight"][h * D + slow] = 0.0
        w[pre + "k_proj.weight"][h * D + slow, 1] = 2.0
    w[pre + "q_norm.weight"][slow] = 6.0
    w[pre + "k_norm.weight"][slow] = 6.0
    cfg2, weights2 = _write_folder(str(tmp_path / "planted"), cfg, w)

    weak, mid, strong = planted
    toks = [t % (cfg["vocab_size"] - 3) for t in random_tokens(200, cfg["vocab_size"], 14)]
    places = {0: weak, 3 * P - 1: mid, 11 * P: strong}
    for pos, tok in places.items():
        toks[pos] = tok
    eng = Engine.from_folder(str(tmp_path / "planted"), dtype=dtype, page_size=P, max_tokens=256, max_slots=2)
    got = replay.run_steps(eng, replay.portions("x", toks, sizes=(8, 9, 7, 16, 1, 24, 3, 1, 1, 30)))
    replay.compare(got, cfg2, weights2, {"x": toks}, TOL[dtype], f"planted/{dtype}")

    # teeth: were the planted key at a page's edge not seen, the next position's logits would be those of
    # the sequence without it (only attention carries one position's token to another's logits)
    ref = plain.forward_logits(weights2, cfg2, toks, dtype=torch.float64)
    for pos in (3 * P - 1, 11 * P):
        without = list(toks)
        without[pos] = 5
        moved = plain.forward_logits(weights2, cfg2, without, dtype=torch.float64)
        for at in (pos + 1, len(toks) - 1):
            change = float((ref[at] - moved[at]).abs().max() / ref.abs().max())
            assert change > 10 * TOL["bfloat16"], (pos, at, change)


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


def test_a_portion_of_two_thousand_rows_takes_the_many_rows_kernel(tmp_path):
    """A feed-forward wide enough (gate|up of 4,096 rows) and a portion long enough (2,100 tokens) for
    gemm_tiles with the fused activation: the logits of the whole prompt in one step, in portions that the
    library takes, and of the plain implementation agree; a captured replay of the long step gives the same bits."""
    import os
    from arle_amd.config import Qwen3Config
    from arle_amd.kernels import ops
    from arle_amd.weights import write_random_model

    raw = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
               intermediate_size=2048, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=True, max_position_embeddings=4096)
    d = os.path.join(str(tmp_path), "wide_ffn")
    write_random_model(d, "Qwen3ForCausalLM", Qwen3Config.from_dict(raw), seed=5, std=0.03, norm_std=0.02)
    cfg, weights = read_folder(d)
    n = 2100
    assert ops.gemm_tiles_preferred(n, 2 * raw["intermediate_size"], raw["hidden_size"], raw["hidden_size"], fused=True)
    toks = random_tokens(n, raw["vocab_size"], 12)
    want_at = list(range(n))
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=3 * 2176, max_slots=3)
    whole = replay.run_steps(eng, [{"entries": [("w", toks, want_at)], "end": ["w"]}])
    replay.compare(whole, cfg, weights, {"w": toks}, TOL["bfloat16"], "2,100 rows in one step")
    steps, at = [], 0
    for size in (700, 700, 700):
        wanted = [p - at for p in want_at if at <= p < at + size]
        steps.append({"entries": [("p", toks[at:at + size], wanted)], "end": []})
        at += size
    cut = replay.run_steps(eng, steps)
    replay.compare(cut, cfg, weights, {"p": toks}, TOL["bfloat16"], "2,100 rows in portions of 700")
    # the same long step twice more: the third runs from a captured graph
    again = [replay.run_steps(eng, [{"entries": [(f"g{i}", toks, want_at)], "end": [f"g{i}"]}]) for i in range(2)]
    assert eng.graph_replays >= 1
    for i, got in enumerate(again):
        for (_, pos), logits in got.items():
            assert torch.equal(logits, whole[("w", pos)]), (i, pos)


def test_a_step_of_six_thousand_rows_agrees_with_portions_and_the_plain_implementation(tmp_path):
    """The longest portion of one request follows the GPU's memory (16,384 tokens on an MI355X), so a long prompt is
    one step: 6,200 rows (the library's products; 194 row blocks of the portions' attention) against the plain
    implementation at every position, whole and in portions of 4,200 and 2,000 (the first takes the many-rows
    product with its activation: 17 row blocks of 256 and 17 column blocks, so that its workgroups run in patches
    of row and column blocks that end beyond the last block both ways)."""
    import os
    from arle_amd.config import Qwen3Config
    from arle_amd.kernels import ops
    from arle_amd.weights import write_random_model

    raw = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
               intermediate_size=2048 + 80, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=True, max_position_embeddings=8192)
    d = os.path.join(str(tmp_path), "wide_ffn_long")
    write_random_model(d, "Qwen3ForCausalLM", Qwen3Config.from_dict(raw), seed=6, std=0.03, norm_std=0.02)
    cfg, weights = read_folder(d)
    n = 6200
    assert not ops.gemm_tiles_preferred(n, 2 * raw["intermediate_size"], raw["hidden_size"], raw["hidden_size"], fused=True)
    assert ops.gemm_tiles_preferred(4200, 2 * raw["intermediate_size"], raw["hidden_size"], raw["hidden_size"], fused=True)
    toks = random_tokens(n, raw["vocab_size"], 13)
    want_at = list(range(n))
    ref = replay.plain_logits(cfg, weights, toks).double()
    scale = float(ref.abs().max())

    def check(got, what):
        assert len(got) == n
        err = torch.stack([(got[(rid, p)].double() - ref[p]).abs().max() for (rid, p) in got])
        worst = int(err.argmax())
        assert float(err[worst]) / scale <= TOL["bfloat16"], f"{what}: worst at {list(got)[worst]}: {float(err[worst]) / scale:.3e}"

    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=2 * 6208, max_slots=2, max_request_tokens=6208)
    whole = replay.run_steps(eng, [{"entries": [("w", toks, want_at)], "end": ["w"]}])
    check(whole, "6,200 rows in one step")
    steps, at = [], 0
    for size in (4200, 2000):       # the first portion takes the many-rows product with its activation
        wanted = [p - at for p in want_at if at <= p < at + size]
        steps.append({"entries": [("p", toks[at:at + size], wanted)], "end": []})
        at += size
    cut = replay.run_steps(eng, steps)
    check(cut, "6,200 rows in portions of 4,200 and 2,000")
