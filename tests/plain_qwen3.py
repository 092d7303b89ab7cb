"""Plain, slow statement of the Qwen3 dense decoder, used only by tests.

Whole sequences, no cache, no batching, one function per part.  Nothing here is
imported by the engine and nothing of the engine is imported here: the two meet
only in the tests that compare them.  Every function cites the place in the
reference (paths relative to the cklxx/arle checkout) that fixes its formula.

All arithmetic runs in the dtype of the tensors passed in (float32 by default,
float64 when the caller upcasts the weights), on the CPU.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * 1/sqrt(mean(x^2) + eps) * weight, mean over the last axis, plain weight.

    crates/cuda-kernels/csrc/misc/norm.cu:8 (formula), :59 (1/sqrtf(total/n + eps));
    host statement infer/src/ops/tests.rs:13-35 (offset=false branch).
    """
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    inv = 1.0 / torch.sqrt(mean_sq + eps)
    return x * inv * weight


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x . W^T with W stored [out, in]; no bias.

    crates/cuda-kernels/csrc/gemm/gemv.cu:240-330 (Y[T,N] = X[T,K] . W[N,K]^T);
    vector infer/src/ops/tests.rs:52-78 ([[1,2,3],[4,5,6]] . [1,2,3] = [14,32]).
    """
    return x @ weight.T


def embedding(table: torch.Tensor, token_ids) -> torch.Tensor:
    """Row gather, no scaling, no position term.

    crates/cuda-kernels/csrc/misc/elementwise_basic.cu:186-199.
    """
    return torch.stack([table[int(t)] for t in token_ids])


def rope_inv_freq(head_dim: int, theta: float) -> torch.Tensor:
    """inv_freq_i = 1 / theta^(2i/head_dim), i in [0, head_dim/2), in float32.

    infer/src/weight_loader.rs:963-965; crates/train/src/qwen3.rs:845-852.
    """
    half = head_dim // 2
    theta32 = torch.tensor(theta, dtype=torch.float32)
    exps = torch.arange(half, dtype=torch.float32) * 2.0 / float(head_dim)
    return 1.0 / torch.pow(theta32, exps)


def rope_cos_sin(positions, head_dim: int, theta: float, dtype=torch.float32):
    """cos/sin of angle = pos * inv_freq (float32 product), shape [len, head_dim/2].

    infer/src/weight_loader.rs:970-981 (angle in f32); the reference then narrows the
    table to bf16 for its bf16 path, which a 32-bit statement does not do
    (crates/train/src/qwen3.rs:856-862 keeps f32).
    """
    inv = rope_inv_freq(head_dim, theta)
    pos = torch.as_tensor(list(positions), dtype=torch.float32)
    angle = pos[:, None] * inv[None, :]
    return torch.cos(angle).to(dtype), torch.sin(angle).to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split (NeoX) rotation on [T, heads, D]: pairs (i, i + D/2).

    out_i       = x_i cos_i - x_{i+D/2} sin_i
    out_{i+D/2} = x_i sin_i + x_{i+D/2} cos_i
    crates/cuda-kernels/csrc/attention/prefill_attention_paged_prep.cu:60-76;
    host statement infer/src/ops/tests.rs:1174-1186.
    """
    half = x.shape[-1] // 2
    lo, hi = x[..., :half], x[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([lo * c - hi * s, lo * s + hi * c], dim=-1)


def qk_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm over head_dim of every head separately, one weight [D] for all heads.

    crates/cuda-kernels/csrc/attention/prefill_attention_paged_prep.cu:33-56;
    crates/train/src/qwen3.rs:122-123 (before rope).
    """
    return rms_norm(x, weight, eps)


def prepare_heads(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, cos, sin) -> torch.Tensor:
    """What a query or key head goes through before the scores: per-head norm first, rotation second.

    Host statement infer/src/ops/tests.rs:1164-1212 (`apply_rope(&rms_norm(head, weight))` at :1202 and :1210);
    infer/src/model/qwen3/prefill.rs:669-690 (norm and rotation in one kernel, in this order).
    """
    return apply_rope(qk_norm(x, norm_weight, eps), cos, sin)


def causal_attention(q, k, v, num_kv_heads: int, window: int | None = None, rows=None) -> torch.Tensor:
    """softmax(q k^T / sqrt(D) + causal mask) v with grouped heads.

    q [T, nq, D], k/v [T, nkv, D]; q head j uses kv head j // (nq/nkv)
    (crates/cuda-kernels/tools/tilelang/batch_prefill_paged_hd128.py:103);
    scale 1/sqrt(head_dim) (infer/src/ops/attention.rs:636);
    row r sees columns c <= r (crates/autograd/src/ops/attention.rs:52-92).
    `window` (keys c > r - window) is not part of Qwen3; it exists to pin the
    engine's generic attention part in tests.
    `rows`: only these query rows are worked out (the others stay zero), against all
    keys as before: for tests of very long sequences that look at a few rows.
    """
    T, nq, D = q.shape
    group = nq // num_kv_heads
    scale = 1.0 / math.sqrt(D)
    out = torch.zeros_like(q)
    which = list(range(T)) if rows is None else [int(r) for r in rows]
    for h in range(nq):
        kh = h // group
        scores = (q[which, h, :] @ k[:, kh, :].T) * scale
        for i, r in enumerate(which):
            scores[i, r + 1:] = float("-inf")
            if window is not None and r - window >= 0:
                scores[i, : r - window + 1] = float("-inf")
        probs = torch.softmax(scores, dim=-1)
        out[which, h, :] = probs @ v[:, kh, :]
    return out


def silu(z: torch.Tensor) -> torch.Tensor:
    """z / (1 + exp(-z)).  crates/cuda-kernels/csrc/misc/elementwise_basic.cu:18-24."""
    return z / (1.0 + torch.exp(-z))


def swiglu_mlp(x, w_gate, w_up, w_down) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)); gate is silu's operand.

    infer/src/model/qwen3/prefill.rs:291-337; crates/train/src/qwen3.rs:150-155.
    """
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


def attention_block(x, w, prefix, cfg, positions):
    """norm'd input -> q/k/v -> per-head norm -> rope -> causal GQA -> o_proj.

    infer/src/model/qwen3/prefill.rs:652-738; crates/train/src/qwen3.rs:92-145.
    """
    T = x.shape[0]
    nq, nkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    q = linear(x, w[prefix + "self_attn.q_proj.weight"]).reshape(T, nq, D)
    k = linear(x, w[prefix + "self_attn.k_proj.weight"]).reshape(T, nkv, D)
    v = linear(x, w[prefix + "self_attn.v_proj.weight"]).reshape(T, nkv, D)
    cos, sin = rope_cos_sin(positions, D, cfg["rope_theta"], dtype=x.dtype)
    q = prepare_heads(q, w[prefix + "self_attn.q_norm.weight"], eps, cos, sin)
    k = prepare_heads(k, w[prefix + "self_attn.k_norm.weight"], eps, cos, sin)
    a = causal_attention(q, k, v, nkv).reshape(T, nq * D)
    return linear(a, w[prefix + "self_attn.o_proj.weight"])


def decoder_layer(h, w, layer: int, cfg, positions):
    """h += Attn(rms(h)); h += MLP(rms(h)).

    infer/src/model/qwen3/prefill.rs:618-776; crates/train/src/qwen3.rs:91-157.
    """
    p = f"model.layers.{layer}."
    eps = cfg["rms_norm_eps"]
    a = rms_norm(h, w[p + "input_layernorm.weight"], eps)
    h = h + attention_block(a, w, p, cfg, positions)
    b = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    h = h + swiglu_mlp(b, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
    return h


def forward_logits(w: dict, cfg: dict, token_ids, dtype=torch.float32, first_position: int = 0):
    """Logits [T, V] of one whole sequence at every position.

    Embedding -> layers -> final norm -> head; the head is the embedding table when
    tie_word_embeddings is set (infer/src/model/qwen3/weights.rs:305-316;
    crates/qwen3-spec/src/lib.rs:162-168).  `first_position` shifts every position
    (for the invariance test: only distances count).
    """
    w = {k: t.to(dtype) for k, t in w.items()}
    T = len(token_ids)
    positions = [first_position + i for i in range(T)]
    h = embedding(w["model.embed_tokens.weight"], token_ids)
    for layer in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, w, layer, cfg, positions)
    f = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(f, head)


# ---------------------------------------------------------------- sampling


def apply_penalties(logits: torch.Tensor, counts: dict, repetition: float, frequency: float,
                    presence: float) -> torch.Tensor:
    """infer/src/sampler.rs:100-140: l>=0 ? l/rep : l*rep, then - freq*count - presence."""
    out = logits.clone()
    for tok, count in counts.items():
        if count == 0 or tok >= out.numel():
            continue
        l = out[tok]
        if repetition != 1.0:
            l = l / repetition if l >= 0 else l * repetition
        out[tok] = l - frequency * count - presence
    return out


def sample_token(logits: torch.Tensor, temperature: float, u: float, top_k: int = -1,
                 top_p: float = 1.0, min_p: float = 0.0) -> int:
    """Softmax of logits/T, truncations, inverse CDF in token order with uniform u.

    crates/cuda-kernels/csrc/misc/sampling.cu:327-596 (temperature -> softmax ->
    top-k -> renormalise -> top-p -> renormalise -> first index whose running sum
    exceeds u); greedy rule infer/src/sampler.rs:82-84; min_p as stated at
    infer/src/sampler.rs:27-29 (keep p >= min_p * p_max).
    Vectors infer/src/ops/tests.rs:333-378.
    """
    greedy = (temperature <= 0.0 or top_k == 1) and top_p >= 1.0 and min_p <= 0.0
    if greedy:
        return int(torch.argmax(logits))
    t = temperature if temperature > 0.0 else 1.0
    p = torch.softmax(logits.double() / t, dim=-1)
    if min_p > 0.0:
        p = torch.where(p >= min_p * p.max(), p, torch.zeros_like(p))
        p = p / p.sum()
    if 0 < top_k < p.numel():
        kth = torch.sort(p, descending=True).values[top_k - 1]
        p = torch.where(p >= kth, p, torch.zeros_like(p))
        p = p / p.sum()
    if top_p < 1.0:
        vals = torch.sort(p, descending=True).values
        csum = torch.cumsum(vals, 0)
        idx = int((csum >= top_p).nonzero()[0]) if bool((csum >= top_p).any()) else p.numel() - 1
        p = torch.where(p >= vals[idx], p, torch.zeros_like(p))
        p = p / p.sum()
    csum = torch.cumsum(p, 0)
    hit = (csum > u).nonzero()
    if hit.numel() == 0:
        return int((p > 0).nonzero()[-1])
    return int(hit[0])
