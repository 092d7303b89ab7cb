"""The plain implementation pinned by what fixes it beside the reference's text:
vectors the reference's own tests hold, special cases that reduce to a library routine,
and invariants; each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from tiny import TINY_A, TINY_B

torch.manual_seed(0)


def test_rmsnorm_vector_of_the_reference():
    # infer/src/ops/tests.rs:90-104: x=[1,2,3,4], w=1, eps=1e-6
    x = torch.tensor([1.0, 2.0, 3.0, 4.0])
    want = x / math.sqrt(7.5 + 1e-6)
    assert torch.allclose(plain.rms_norm(x, torch.ones(4), 1e-6), want, atol=1e-7)


def test_rmsnorm_is_library_rms_norm_and_uses_plain_weight():
    x = torch.randn(5, 260)  # 260: the reference's multi-tile width (ops/tests.rs:107-153)
    w = torch.randn(260)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (260,), w, 1e-5), atol=1e-6)
    # weight 0 gives 0: a (1 + w) norm would not
    assert torch.count_nonzero(plain.rms_norm(x, torch.zeros(260), 1e-5)) == 0
    # scale invariance for eps -> 0
    assert torch.allclose(plain.rms_norm(3.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0), atol=1e-5)


def test_linear_vector_of_the_reference():
    # infer/src/ops/tests.rs:52-78
    a = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    assert plain.linear(torch.tensor([1.0, 2.0, 3.0]), a).tolist() == [14.0, 32.0]
    x = torch.randn(4, 7)
    w = torch.randn(5, 7)
    assert torch.allclose(plain.linear(x, w), F.linear(x, w), atol=1e-6)


def test_rope_position_zero_is_identity_and_norm_is_kept():
    x = torch.randn(1, 3, 32)
    cos, sin = plain.rope_cos_sin([0], 32, 1e6)
    assert torch.equal(plain.apply_rope(x, cos, sin), x)
    cos, sin = plain.rope_cos_sin([7], 32, 1e6)
    y = plain.apply_rope(x, cos, sin)
    half = 16
    pair_norm = lambda t: t[..., :half] ** 2 + t[..., half:] ** 2
    assert torch.allclose(pair_norm(x), pair_norm(y), atol=1e-5)
    assert plain.rope_inv_freq(32, 1e6)[0] == 1.0


def test_rope_matches_rotate_half_form():
    x = torch.randn(6, 2, 16)
    cos, sin = plain.rope_cos_sin(range(6), 16, 1e4)
    full_cos = torch.cat([cos, cos], -1)[:, None, :]
    full_sin = torch.cat([sin, sin], -1)[:, None, :]
    rot = torch.cat([-x[..., 8:], x[..., :8]], -1)
    assert torch.allclose(plain.apply_rope(x, cos, sin), x * full_cos + rot * full_sin, atol=1e-6)


def test_rope_scores_depend_only_on_distance():
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)

    def score(m, n):
        cq, sq = plain.rope_cos_sin([m], 32, 1e4, dtype=torch.float64)
        ck, sk = plain.rope_cos_sin([n], 32, 1e4, dtype=torch.float64)
        return (plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum()

    assert abs(score(5, 2) - score(13, 10)) < 1e-5
    assert abs(score(5, 2) - score(2, 5)) > 1e-3  # a wrong sign of the rotation shows here


def test_attention_special_cases():
    # one key: output is v
    q, k, v = torch.randn(1, 4, 16), torch.randn(1, 2, 16), torch.randn(1, 2, 16)
    out = plain.causal_attention(q, k, v, 2)
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 3], v[0, 1])
    # equal scores: mean of the visible values
    q = torch.zeros(3, 2, 16)
    k, v = torch.randn(3, 2, 16), torch.randn(3, 2, 16)
    out = plain.causal_attention(q, k, v, 2)
    assert torch.allclose(out[2, 1], v[:, 1].mean(0), atol=1e-6)
    assert torch.allclose(out[1, 0], v[:2, 0].mean(0), atol=1e-6)


def test_attention_is_library_sdpa_with_grouped_heads_and_head_dim_scale():
    T, nq, nkv, D = 9, 6, 2, 32
    q, k, v = torch.randn(T, nq, D), torch.randn(T, nkv, D), torch.randn(T, nkv, D)
    rep = lambda t: t.repeat_interleave(nq // nkv, dim=1).transpose(0, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), rep(k), rep(v), is_causal=True,
                                          scale=1.0 / math.sqrt(D)).transpose(0, 1)
    assert torch.allclose(plain.causal_attention(q, k, v, nkv), want, atol=1e-5)


def test_attention_rows_ignore_the_future():
    T = 7
    q, k, v = torch.randn(T, 4, 16), torch.randn(T, 2, 16), torch.randn(T, 2, 16)
    a = plain.causal_attention(q, k, v, 2)
    k2, v2 = k.clone(), v.clone()
    k2[5:] += 3.0
    v2[5:] -= 2.0
    b = plain.causal_attention(q, k2, v2, 2)
    assert torch.equal(a[:5], b[:5]) and not torch.allclose(a[5:], b[5:])


def test_swiglu_gate_is_the_operand_of_silu():
    x = torch.randn(3, 8)
    wg, wu, wd = torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain.swiglu_mlp(x, wg, wu, wd), want, atol=1e-5)
    assert not torch.allclose(plain.swiglu_mlp(x, wu, wg, wd), want, atol=1e-3)
    assert torch.count_nonzero(plain.swiglu_mlp(x, torch.zeros(12, 8), wu, wd)) == 0


def _random_weights(cfg, seed, std=0.05):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    r = lambda *s: torch.randn(*s, generator=g) * std
    n = lambda s: 1.0 + torch.randn(s, generator=g) * std
    w = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": n(H)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = r(V, H)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w.update({p + "input_layernorm.weight": n(H), p + "post_attention_layernorm.weight": n(H),
                  p + "self_attn.q_proj.weight": r(nq * D, H), p + "self_attn.k_proj.weight": r(nkv * D, H),
                  p + "self_attn.v_proj.weight": r(nkv * D, H), p + "self_attn.o_proj.weight": r(H, nq * D),
                  p + "self_attn.q_norm.weight": n(D), p + "self_attn.k_norm.weight": n(D),
                  p + "mlp.gate_proj.weight": r(I, H), p + "mlp.up_proj.weight": r(I, H),
                  p + "mlp.down_proj.weight": r(H, I)})
    return w


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_model_prefix_invariance_and_tied_head(cfg):
    w = _random_weights(cfg, 3)
    toks = torch.randint(0, cfg["vocab_size"], (12,), generator=torch.Generator().manual_seed(1)).tolist()
    full = plain.forward_logits(w, cfg, toks, dtype=torch.float64)
    short = plain.forward_logits(w, cfg, toks[:7], dtype=torch.float64)
    assert torch.allclose(full[:7], short, atol=1e-10)  # causal: a prefix does not see what follows
    # untied model with lm_head := embedding equals the tied model
    tied = dict(cfg, tie_word_embeddings=True)
    untied = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    assert torch.allclose(plain.forward_logits(w2, tied, toks), plain.forward_logits(w2, untied, toks))


def test_model_shift_of_all_positions_changes_nothing():
    # only distances count: a wrong pairing or sign in the rotation fails this
    cfg = TINY_B
    w = _random_weights(cfg, 4)
    toks = list(range(3, 14))
    a = plain.forward_logits(w, cfg, toks, dtype=torch.float64)
    b = plain.forward_logits(w, cfg, toks, dtype=torch.float64, first_position=37)
    assert torch.allclose(a, b, atol=1e-4)


def test_rope_frequencies_and_one_rotated_pair_are_the_literal_numbers():
    # The statement of infer/src/ops/tests.rs:1090-1100: inv_freq_i = 1 / theta^(2i/D), angle = pos * inv_freq_i.
    # D=8, theta=1e4: the exponents are 0, 1/4, 1/2, 3/4, so the frequencies are powers of ten.  theta^(-i/D)
    # (half the exponent) would give 1, 0.316, 0.1, 0.0316; 2i/(D/2) would give 1, 0.01, ...
    from arle_amd.parts.position import rope_table

    literal = torch.tensor([1.0, 0.1, 0.01, 0.001])
    assert torch.allclose(plain.rope_inv_freq(8, 1e4), literal, rtol=1e-6)
    # theta=1e6, D=128 (the checkpoints' values): 10^(-6*2i/128), written out
    inv = plain.rope_inv_freq(128, 1e6)
    assert abs(float(inv[1]) / 0.8058421877614819 - 1) < 1e-6      # 10^-0.09375
    assert abs(float(inv[63]) / 1.2409377607517196e-06 - 1) < 1e-5  # 10^-5.90625
    # the engine's table holds the same angles: cos/sin(pos * inv_freq_i) at pos 7, i = 1 and 63
    cos, sin = rope_table(128, 1e6, 8)
    pcos, psin = plain.rope_cos_sin(range(8), 128, 1e6)
    for i, angle in ((1, 7 * 0.8058421877614819), (63, 7 * 1.2409377607517196e-06)):
        for table_c, table_s in ((cos, sin), (pcos, psin)):
            assert abs(float(table_c[7, i]) - math.cos(angle)) < 1e-6
            assert abs(float(table_s[7, i]) - math.sin(angle)) < 1e-6
    ecos, esin = rope_table(8, 1e4, 4)
    assert torch.allclose(torch.atan2(esin[1], ecos[1]), literal, rtol=1e-5)   # pos 1: the angles are inv_freq
    # one pair rotated by hand at pos=3, i=1 of D=8: angle 0.3; x_1 = 1, x_5 = 2
    #   out_1 = cos(0.3) - 2 sin(0.3) = 0.364296075,  out_5 = sin(0.3) + 2 cos(0.3) = 2.206193185
    x = torch.zeros(1, 1, 8)
    x[0, 0, 1], x[0, 0, 5] = 1.0, 2.0
    for c, s in (plain.rope_cos_sin([3], 8, 1e4), (ecos[3:4], esin[3:4])):
        y = plain.apply_rope(x, c, s)
        assert abs(float(y[0, 0, 1]) - 0.364296075) < 1e-6 and abs(float(y[0, 0, 5]) - 2.206193185) < 1e-6
        assert torch.count_nonzero(y[0, 0, [0, 2, 3, 4, 6, 7]]) == 0


def test_scaling_a_query_heads_projection_changes_nothing():
    # the per-head norm removes a head's scale (eps aside): it is per head, and it is there
    cfg = dict(TINY_A, num_hidden_layers=1)
    w = _random_weights(cfg, 5)
    p = "model.layers.0."
    x = torch.randn(6, cfg["hidden_size"], dtype=torch.float64)
    w64 = {k: t.double() for k, t in w.items()}
    base = plain.attention_block(x, w64, p, cfg, list(range(6)))
    w_scaled = dict(w64)
    wq = w64[p + "self_attn.q_proj.weight"].clone()
    wq[:16] *= 7.0
    w_scaled[p + "self_attn.q_proj.weight"] = wq
    assert torch.allclose(plain.attention_block(x, w_scaled, p, cfg, list(range(6))), base, atol=1e-6)
    # ... and scaling one head does change the others' share if the norm ran over all heads at once
    wq2 = w64[p + "self_attn.q_proj.weight"].clone()
    wq2[:16] *= 7.0
    q = (x @ wq2.T).reshape(6, 4, 16)
    over_all = plain.rms_norm(q.reshape(6, 64), torch.ones(64, dtype=torch.float64), 1e-6).reshape(6, 4, 16)
    assert not torch.allclose(over_all[:, 1], plain.qk_norm(q, torch.ones(16, dtype=torch.float64), 1e-6)[:, 1],
                              atol=1e-3)


def test_qk_norm_comes_before_the_rotation():
    # Host statement infer/src/ops/tests.rs:1164-1212, with its own weights (0.9 + (i % 13) * 0.03, :1083-1085)
    # and head (:1074-1076): norm with a weight that differs between i and i + D/2, then the rotation.  With the
    # order swapped the pair (i, i + D/2) would be mixed before its two different weights apply.
    D, half, eps, pos, theta = 32, 16, 1e-6, 5, 1e6
    head = [((i % 19) - 9.0) * 0.25 for i in range(D)]
    weight = [0.9 + (i % 13) * 0.03 for i in range(D)]
    assert weight[3] != weight[3 + half]
    inv_freq = [1.0 / theta ** (i * 2.0 / D) for i in range(half)]

    def norm(h, wt):
        inv = 1.0 / math.sqrt(sum(v * v for v in h) / len(h) + eps)
        return [v * inv * g for v, g in zip(h, wt)]

    def rotate(h):
        out = [0.0] * D
        for i in range(half):
            c, s = math.cos(pos * inv_freq[i]), math.sin(pos * inv_freq[i])
            out[i] = h[i] * c - h[i + half] * s
            out[i + half] = h[i] * s + h[i + half] * c
        return out

    norm_then_rope = torch.tensor(rotate(norm(head, weight)), dtype=torch.float64)
    rope_then_norm = torch.tensor(norm(rotate(head), weight), dtype=torch.float64)
    assert (norm_then_rope - rope_then_norm).abs().max() > 0.05     # the two orders are far apart here
    cos, sin = plain.rope_cos_sin([pos], D, theta, dtype=torch.float64)
    got = plain.prepare_heads(torch.tensor(head, dtype=torch.float64).reshape(1, 1, D),
                              torch.tensor(weight, dtype=torch.float64), eps, cos, sin)[0, 0]
    assert torch.allclose(got, norm_then_rope, atol=1e-6)
    # the whole attention part uses that preparation: with v = identity-like weights its output moves when
    # the norm weights of the two halves are exchanged (a rotation-first order would not care which half)
    cfg = dict(TINY_A, num_hidden_layers=1)
    w = {k: t.double() for k, t in _random_weights(cfg, 6, std=0.3).items()}
    p = "model.layers.0."
    w[p + "self_attn.q_norm.weight"] = torch.tensor([0.9 + (i % 13) * 0.03 for i in range(16)], dtype=torch.float64)
    x = torch.randn(6, cfg["hidden_size"], dtype=torch.float64)
    T, nq, nkv, Dh = 6, 4, 2, 16
    q = plain.linear(x, w[p + "self_attn.q_proj.weight"]).reshape(T, nq, Dh)
    k = plain.linear(x, w[p + "self_attn.k_proj.weight"]).reshape(T, nkv, Dh)
    v = plain.linear(x, w[p + "self_attn.v_proj.weight"]).reshape(T, nkv, Dh)
    c, s = plain.rope_cos_sin(range(T), Dh, cfg["rope_theta"], dtype=torch.float64)
    by_hand = plain.linear(plain.causal_attention(
        plain.apply_rope(plain.rms_norm(q, w[p + "self_attn.q_norm.weight"], cfg["rms_norm_eps"]), c, s),
        plain.apply_rope(plain.rms_norm(k, w[p + "self_attn.k_norm.weight"], cfg["rms_norm_eps"]), c, s),
        v, nkv).reshape(T, nq * Dh), w[p + "self_attn.o_proj.weight"])
    swapped = plain.linear(plain.causal_attention(
        plain.rms_norm(plain.apply_rope(q, c, s), w[p + "self_attn.q_norm.weight"], cfg["rms_norm_eps"]),
        plain.rms_norm(plain.apply_rope(k, c, s), w[p + "self_attn.k_norm.weight"], cfg["rms_norm_eps"]),
        v, nkv).reshape(T, nq * Dh), w[p + "self_attn.o_proj.weight"])
    block = plain.attention_block(x, w, p, cfg, list(range(T)))
    assert torch.allclose(block, by_hand, atol=1e-9)
    assert (block - swapped).abs().max() > 1e-3


def test_sampling_vectors_of_the_reference():
    # infer/src/ops/tests.rs:333-378
    logits = torch.tensor([1.0, 2.0, 10.0, 1.5, 0.5])
    assert plain.sample_token(logits, 0.01, 0.5) == 2
    assert plain.sample_token(logits, 1.0, 0.0) == 0
    assert plain.sample_token(logits, 1.0, 0.9, top_k=1) == 2
    assert plain.sample_token(logits, 0.0, 0.3) == 2
    # inverse CDF in token order
    probs = torch.softmax(logits.double(), 0)
    u = float(probs[:2].sum()) + 1e-6
    assert plain.sample_token(logits, 1.0, u) == 2
    # top-p keeps the smallest head set reaching the mass: here only token 2
    assert plain.sample_token(logits, 1.0, 0.9999, top_p=0.5) == 2


def test_penalties_of_the_reference():
    # infer/src/sampler.rs:100-140
    l = torch.tensor([2.0, -2.0, 1.0])
    out = plain.apply_penalties(l, {0: 2, 1: 1}, repetition=2.0, frequency=0.5, presence=0.25)
    assert torch.allclose(out, torch.tensor([1.0 - 1.0 - 0.25, -4.0 - 0.5 - 0.25, 1.0]))


def test_attention_of_chosen_rows_equals_those_rows_of_the_whole():
    torch.manual_seed(3)
    q, k, v = torch.randn(11, 4, 8, dtype=torch.float64), torch.randn(11, 2, 8, dtype=torch.float64), torch.randn(11, 2, 8, dtype=torch.float64)
    whole = plain.causal_attention(q, k, v, 2)
    some = plain.causal_attention(q, k, v, 2, rows=[0, 4, 10])
    assert torch.allclose(some[[0, 4, 10]], whole[[0, 4, 10]], rtol=0, atol=1e-14) and float(some[[1, 2, 3, 5]].abs().max()) == 0.0
    windowed = plain.causal_attention(q, k, v, 2, window=3)
    assert torch.allclose(plain.causal_attention(q, k, v, 2, window=3, rows=[7])[7], windowed[7], rtol=0, atol=1e-14)
