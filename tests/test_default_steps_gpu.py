"""The steps that the engine takes when nobody tells it otherwise, against the plain implementation.

On an MI355X the longest portion of one request is 16,384 tokens (the reference's server sizes it by the GPU's
memory: infer/src/scheduler/types.rs:251-334), so a long prompt is one step of that many rows: the library's products
beyond the many-rows kernel's range, 512 and more row blocks of the portions' attention, other splits of their keys.
Checked here whole, cut in two, and followed by decoded tokens, at tiny widths in both precisions and at head_dim
128 with groups of four q heads and pages of 16 in bfloat16; and a mixed step whose (row block, segment) pairs no
longer fit the portions kernel's work list."""
import os

import pytest
import torch

import replay
from arle_amd.config import Qwen3Config
from arle_amd.engine import Engine
from arle_amd.engine.scheduler import SchedulerConfig, pick_chunked_prefill_size_for_hbm
from arle_amd.kernels import ops
from arle_amd.weights import write_random_model
from tiny import ARCH, random_tokens, read_folder

pytestmark = pytest.mark.gpu
TOL = {"float32": 1e-5, "bfloat16": 2e-2}
PORTION = 16384

SMALL = dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
             intermediate_size=160, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-6,
             tie_word_embeddings=True, max_position_embeddings=32768)
# the attention of Qwen3-4B (heads of 128, four q heads a kv head) around a narrow model
HEADS128 = dict(num_hidden_layers=2, hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
                intermediate_size=640, vocab_size=300, rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=False, max_position_embeddings=32768)


def _folder(tmp_path, name, raw, seed, std):
    d = os.path.join(str(tmp_path), name)
    write_random_model(d, ARCH, Qwen3Config.from_dict(raw), seed=seed, std=std, norm_std=0.02)
    return (d, *read_folder(d))


def test_the_default_portion_on_this_gpu_is_what_these_tests_run():
    total = torch.cuda.get_device_properties(0).total_memory
    assert pick_chunked_prefill_size_for_hbm(total) == PORTION
    cfg = SchedulerConfig.runtime_defaults(4).resolve_runtime_envelope(total, None, None)
    assert cfg.chunked_prefill_size == PORTION


def _steps_whole_then_decode(rid, toks, head, cuts):
    """The first `head` tokens in portions of `cuts` (which add up to head), the rest one by one; every place wanted."""
    steps, at = [], 0
    for size in cuts:
        steps.append({"entries": [(rid, toks[at:at + size], list(range(size)))], "end": []})
        at += size
    assert at == head
    steps += [{"entries": [(rid, [t], [0])], "end": []} for t in toks[head:]]
    steps[-1]["end"] = [rid]
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_portion_of_16384_tokens_whole_cut_in_two_and_decoded_on(tmp_path, dtype):
    d, cfg, weights = _folder(tmp_path, "small", SMALL, 21, 0.03)
    toks = random_tokens(PORTION + 8, SMALL["vocab_size"], 31)
    reference = {"x": replay.plain_logits(cfg, weights, toks)}
    eng = Engine.from_folder(d, dtype=dtype, page_size=16, max_tokens=PORTION + 64, max_slots=2,
                             max_request_tokens=PORTION + 64)
    got = replay.run_steps(eng, _steps_whole_then_decode("x", toks, PORTION, (PORTION,)))
    assert len(got) == len(toks)
    replay.check_rows(got, reference, TOL[dtype], f"16,384 rows in one step + 8 decoded/{dtype}")
    cut = replay.run_steps(eng, _steps_whole_then_decode("x", toks, PORTION, (12000, 4384)))
    replay.check_rows(cut, reference, TOL[dtype], f"12,000 + 4,384 rows + 8 decoded/{dtype}")
    if dtype == "float32":      # fixed-order kernels: the cut changes no bit
        for key, row in got.items():
            assert torch.equal(row, cut[key]), key


def test_a_portion_of_16384_tokens_at_head_dim_128_in_bfloat16(tmp_path):
    """The portions kernel of head_dim 128 (32 rows a wave, tiles loaded straight into LDS) over 2,048 row blocks a kv
    head, and the second portion of the cut prompt over 12,000 cached keys with its keys in parts."""
    d, cfg, weights = _folder(tmp_path, "heads128", HEADS128, 22, 0.04)
    toks = random_tokens(PORTION + 8, HEADS128["vocab_size"], 32)
    reference = {"x": replay.plain_logits(cfg, weights, toks)}
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=PORTION + 64, max_slots=2,
                             max_request_tokens=PORTION + 64)
    assert ops.attn_mfma_supported(torch.bfloat16, 128, 16)
    got = replay.run_steps(eng, _steps_whole_then_decode("x", toks, PORTION, (PORTION,)))
    replay.check_rows(got, reference, TOL["bfloat16"], "head_dim 128: 16,384 rows in one step + 8 decoded")
    cut = replay.run_steps(eng, _steps_whole_then_decode("x", toks, PORTION, (12000, 4384)))
    replay.check_rows(cut, reference, TOL["bfloat16"], "head_dim 128: 12,000 + 4,384 rows + 8 decoded")


def test_a_portion_of_9000_tokens_beside_60_decoded_tokens(tmp_path):
    """One long portion and sixty requests that decode, in one step: 282 row blocks x 61 segments are more pairs than
    the portions kernel's work list holds (16,384), so it hands out (row block, segment) pairs unlisted, dead ones
    included, while the decoded tokens go to the split-KV kernel on the side stream."""
    d, cfg, weights = _folder(tmp_path, "heads128m", HEADS128, 23, 0.04)
    long_toks = random_tokens(9000 + 3, HEADS128["vocab_size"], 40)
    short = {f"s{i}": random_tokens(18 + (7 * i) % 29, HEADS128["vocab_size"], 50 + i) for i in range(60)}
    group = HEADS128["num_attention_heads"] // HEADS128["num_key_value_heads"]
    assert -(-9000 * group // 128) * 61 > ops._PORTION_LIST_MAX
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=9216 + 61 * 64, max_slots=61,
                             max_request_tokens=9216)
    # every short request's prompt but its last two tokens, all in one step; then the long portion beside one decoded
    # token of each; then one more token of everybody
    steps = [{"entries": [(rid, t[:-2], list(range(len(t) - 2))) for rid, t in short.items()], "end": []},
             {"entries": [("long", long_toks[:9000], list(range(8990, 9000)))]
                         + [(rid, t[-2:-1], [0]) for rid, t in short.items()], "end": []},
             {"entries": [("long", long_toks[9000:9001], [0])] + [(rid, t[-1:], [0]) for rid, t in short.items()],
              "end": list(short)},
             {"entries": [("long", long_toks[9001:], [0, 1])], "end": ["long"]}]
    got = replay.run_steps(eng, steps)
    reference = {rid: replay.plain_logits(cfg, weights, t) for rid, t in short.items()}
    replay.check_rows(got, reference, TOL["bfloat16"], "60 decoding requests beside a portion of 9,000")
    reference = {"long": replay.plain_logits(cfg, weights, long_toks)}
    replay.check_rows(got, reference, TOL["bfloat16"], "a portion of 9,000 beside 60 decoded tokens", need_all=False)
    assert sum(1 for key in got if key[0] == "long") == 13


# ---- contexts of 16 k and 32 k tokens: one layer, so that its keys and values follow from the tokens alone ----------

ONE_LAYER_128 = dict(HEADS128, num_hidden_layers=1, max_position_embeddings=40960)


def _one_layer_plain_rows(cfg, w, toks, rows):
    """float64 logits of the chosen rows of a one-layer model: keys and values of every token (no attention is
    needed for those in the first layer), attention and everything after it for the chosen rows only."""
    import plain_qwen3 as plain

    w = {k: t.double() for k, t in w.items()}
    T, nq, nkv, D, eps = len(toks), cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    p = "model.layers.0."
    h = plain.embedding(w["model.embed_tokens.weight"], toks)
    a = plain.rms_norm(h, w[p + "input_layernorm.weight"], eps)
    cos, sin = plain.rope_cos_sin(list(range(T)), D, cfg["rope_theta"], dtype=torch.float64)
    q = plain.prepare_heads(plain.linear(a, w[p + "self_attn.q_proj.weight"]).reshape(T, nq, D),
                            w[p + "self_attn.q_norm.weight"], eps, cos, sin)
    k = plain.prepare_heads(plain.linear(a, w[p + "self_attn.k_proj.weight"]).reshape(T, nkv, D),
                            w[p + "self_attn.k_norm.weight"], eps, cos, sin)
    v = plain.linear(a, w[p + "self_attn.v_proj.weight"]).reshape(T, nkv, D)
    att = plain.causal_attention(q, k, v, nkv, rows=rows)[rows].reshape(len(rows), nq * D)
    h = h[rows] + plain.linear(att, w[p + "self_attn.o_proj.weight"])
    b = plain.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    h = h + plain.swiglu_mlp(b, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return plain.linear(plain.rms_norm(h, w["model.norm.weight"], eps), head)


def test_decoding_at_32k_and_16k_tokens_of_context_in_one_batch(tmp_path):
    """Four requests that decode side by side 32,760, 16,390, 9,001 and 31 tokens into their contexts (the split-KV
    attention at its most splits, block tables of 2,048 pages, a short request beside long ones), after prompts fed in
    portions of 16,384.  The last rows of the long prompts' second portions (16,376 keys behind them) are looked at too."""
    d, cfg, weights = _folder(tmp_path, "one_layer", ONE_LAYER_128, 24, 0.04)
    lengths = {"a": 32760, "b": 16390, "c": 9001, "d": 31}
    decoded = 6
    reqs = {rid: random_tokens(n + decoded, ONE_LAYER_128["vocab_size"], 60 + i) for i, (rid, n) in enumerate(lengths.items())}
    eng = Engine.from_folder(d, dtype="bfloat16", page_size=16, max_tokens=sum(lengths.values()) + 4 * 64, max_slots=4,
                             max_request_tokens=32768 + 64)
    looked, steps = {rid: [] for rid in reqs}, []
    for rid, n in lengths.items():      # the prompts, one request a step, 16,384 tokens at most a portion
        for at in range(0, n, PORTION):
            size = min(PORTION, n - at)
            want = list(range(max(0, size - 40), size)) if at + size == n else []
            looked[rid] += [at + w for w in want]
            steps.append({"entries": [(rid, reqs[rid][at:at + size], want)], "end": []})
    for i in range(decoded):            # then all four decode together
        steps.append({"entries": [(rid, [reqs[rid][lengths[rid] + i]], [0]) for rid in reqs], "end": []})
        for rid in reqs:
            looked[rid].append(lengths[rid] + i)
    steps[-1]["end"] = list(reqs)
    got = replay.run_steps(eng, steps)
    for rid, toks in reqs.items():
        rows = sorted(looked[rid])
        ref = _one_layer_plain_rows(cfg, weights, toks, rows)
        scale = float(ref.abs().max())
        every = []
        for i, pos in enumerate(rows):
            err, rms = replay.row_errors(got[(rid, pos)], ref[i], scale)
            every.append(rms)
            assert err <= TOL["bfloat16"], f"request {rid} ({lengths[rid]} tokens) position {pos}: {err:.3e}"
        assert max(every) <= 4.0 * sorted(every)[len(every) // 2], (rid, max(every), sorted(every)[len(every) // 2])
    assert eng.cache.free_pages() == [eng.cache.groups[0].pool.num_pages]
