"""Grouped-query attention over a paged cache, with optional per-head q/k RMSNorm,
a position encoding of its own choice and an optional window.

Per token row: q, k, v projections (no bias) -> per-head RMSNorm of q and k over head_dim
(one weight [D] for all heads, before the rotation) -> position encoding -> k, v into the
cache at the token's position -> softmax(q k^T / sqrt(D)) v over the request's earlier
keys (all of them, or the last `window`) -> output projection.
infer/src/model/qwen3/prefill.rs:652-738; crates/cuda-kernels/csrc/attention/decode_prep_paged.cu:73-160;
scale infer/src/ops/attention.rs:636; q head j reads kv head j // (nq/nkv).

q, k and v come from one fused [Q+2KV, H] product.  When the schedule says that this layer
reads another layer's cache (`cache_view.writes` False), only q is projected and nothing
is written.
"""
from __future__ import annotations

import math

import torch

from ..cache.manager import PagedNeed
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("mixer", "paged_attention")
class PagedAttention(Part):
    """params: hidden_size, num_q_heads, num_kv_heads, head_dim, qk_norm (bool), eps,
    position (PartSpec), window (int | None), scale (float | None: 1/sqrt(head_dim))."""

    graph_safe = True  # positions, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def declare_weights(cls, params):
        h, d = params["hidden_size"], params["head_dim"]
        nq, nkv = params["num_q_heads"], params["num_kv_heads"]
        decl = {
            "q": WeightDecl((nq * d, h)),
            "k": WeightDecl((nkv * d, h)),
            "v": WeightDecl((nkv * d, h)),
            "o": WeightDecl((h, nq * d)),
        }
        if params.get("qk_norm"):
            decl["q_norm"] = WeightDecl((d,), init="ones")
            decl["k_norm"] = WeightDecl((d,), init="ones")
        return decl

    @classmethod
    def children(cls, params):
        return {"position": ("position", params["position"])}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.nq = int(params["num_q_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.D = int(params["head_dim"])
        if self.nq % self.nkv:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        if not 0 < self.D <= ops.MAX_HEAD_DIM:
            raise ValueError(f"head_dim {self.D} is not supported: the attention kernels take 1..{ops.MAX_HEAD_DIM}")
        if self.D % 16 and not rt.is_f32:
            raise ValueError(f"head_dim {self.D} is not supported in bfloat16: its kernels take multiples of 16 "
                             f"(dtype float32 runs any head_dim up to {ops.MAX_HEAD_DIM})")
        self.eps = float(params.get("eps", 0.0))
        self.window = params.get("window")
        self.scale = float(params["scale"]) if params.get("scale") is not None else 1.0 / math.sqrt(self.D)
        self.position = children["position"]
        self.q_norm = tensors.get("q_norm")
        self.k_norm = tensors.get("k_norm")
        wq, wk, wv = tensors["q"], tensors["k"], tensors["v"]
        if not (wq.dtype == wk.dtype == wv.dtype):
            raise ValueError("q, k and v projections must be stored in one type")
        self.q_width, self.kv_width = self.nq * self.D, self.nkv * self.D
        self.qkv = Linear(torch.cat([wq, wk, wv], dim=0).contiguous(), rt.weight_tiles)
        # for a layer that reads another layer's cache: the q rows of the fused matrix, no copy (head_dim is a
        # multiple of 16, so the q rows are whole operand tiles too)
        self.q_only = Linear(self.qkv.weight[: self.q_width], packed=self.qkv.tiles)
        self.o = Linear(tensors["o"], rt.weight_tiles)
        # steps of single decoded tokens run norm, rotation and cache write inside the attention's kernel where it
        # has that form (ops.attn_decode_prep_supported); params["fold_preparation"] = False keeps the two kernels
        self.folds_preparation = bool(params.get("fold_preparation", True))

    @classmethod
    def declare_cache(cls, params):
        return PagedNeed(num_kv_heads=int(params["num_kv_heads"]), head_dim=int(params["head_dim"]),
                         window=params.get("window"))

    def cache_need(self):
        return self.declare_cache(self.params)

    def products(self):
        if self.qkv.weight.dtype != torch.bfloat16:
            return []
        return [("qkv", self.qkv.out_features, self.qkv.in_features, False, "norm"),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def decode_launch_class(self, rows, max_context):
        # the split-KV factor of the matrix-core kernel is the one launch dimension that follows the context
        if self.rt.is_f32 or self.D % 16 or self.D > ops.MFMA_MAX_HEAD_DIM:
            return None
        return ops.decode_splits(rows, self.nkv, max_context)

    def forward(self, x, batch, cache):
        """x [T, H] -> [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        Q, KV = self.q_width, self.kv_width
        self.position.ensure_positions(batch.max_position + 1)
        cos, sin, rot = self.position.fused_rotary()
        fused = getattr(self.position, "fusable", False)
        nkv = self.nkv if cache.writes else 0   # a layer that reads another layer's cache only needs q
        common = dict(num_q_heads=self.nq, num_kv_heads=nkv, head_dim=self.D, eps=self.eps,
                      positions=batch.positions)
        to_cache = {}
        if cache.writes:
            to_cache = dict(slot_of_token=batch.slot_of_token, block_table=cache.block_table,
                            k_pages=cache.k_pages, v_pages=cache.v_pages, page_size=cache.page_size)
        # the fused preparation kernel can add a stack of partial products itself
        projected = (self.qkv if cache.writes else self.q_only)(x, partials_ok=fused)
        if (fused and cache.writes and batch.max_qlen == 1 and self.folds_preparation
                and (projected.dim() == 3 or projected.dtype == torch.bfloat16)
                and ops.attn_decode_prep_supported(x.dtype, self.D, cache.page_size, self.nq // self.nkv, rot)):
            # single decoded tokens: the attention's kernel sums, norms, rotates and writes to the cache itself
            out = torch.empty((x.shape[0], Q), dtype=x.dtype, device=x.device)
            ops.attn_decode_prep(projected, out, cache.k_pages, cache.v_pages, cache.block_table, batch.seg_row0,
                                 batch.seg_slot, batch.seg_start, max_kv_len=batch.max_position + 1,
                                 num_q_heads=self.nq, num_kv_heads=self.nkv, head_dim=self.D, page_size=cache.page_size,
                                 scale=self.scale, eps=self.eps, q_weight=self.q_norm, k_weight=self.k_norm, cos=cos,
                                 sin=sin, rotary_dim=rot, window=self.window or 0, splits=getattr(batch, "kv_splits", None))
            return self.o(out, partials_ok=True)
        if projected.dim() == 3:
            q = torch.empty((x.shape[0], Q), dtype=x.dtype, device=x.device)
            ops.qk_prep(q, None, None, q_weight=self.q_norm, k_weight=self.k_norm, cos=cos, sin=sin,
                        rotary_dim=rot, parts=projected, **to_cache, **common)
        else:
            if cache.writes:
                q, k, v = projected[:, :Q], projected[:, Q:Q + KV], projected[:, Q + KV:]
            else:
                q = projected
                k = v = projected[:, :0]
            if fused:
                ops.qk_prep(q, k, v, q_weight=self.q_norm, k_weight=self.k_norm, cos=cos, sin=sin,
                            rotary_dim=rot, **to_cache, **common)
            else:
                # a position encoding the fused kernel does not know: norm, encode, then write
                if self.q_norm is not None:
                    ops.qk_prep(q, k, v, q_weight=self.q_norm, k_weight=self.k_norm, **common)
                self.position.apply(q, k, batch.positions, self.nq, nkv)
                if to_cache:
                    ops.qk_prep(q, k, v, **to_cache, **common)
        out = torch.empty((x.shape[0], Q), dtype=q.dtype, device=q.device)
        paged_attention(q, out, cache, batch, num_q_heads=self.nq, num_kv_heads=self.nkv,
                        head_dim=self.D, scale=self.scale, window=self.window or 0)
        return self.o(out, partials_ok=True)


def paged_attention(q, out, cache, batch, *, num_q_heads, num_kv_heads, head_dim, scale, window):
    """Attention of every row of the packed step over its request's cached keys.

    bfloat16 storage runs the matrix-core kernel (split over the keys when the step holds only
    single decoded tokens); float32 storage, and shapes the matrix-core kernel does not take,
    run the fixed-order kernel, which is also the true 32-bit path.
    """
    if ops.attn_mfma_supported(q.dtype, head_dim, cache.page_size):
        ops.attn_paged_mfma(q, out, cache.k_pages, cache.v_pages, cache.block_table, batch.seg_row0,
                            batch.seg_slot, batch.seg_start, max_qlen=batch.max_qlen, min_qlen=batch.min_qlen,
                            max_kv_len=batch.max_position + 1, num_q_heads=num_q_heads,
                            num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=cache.page_size,
                            scale=scale, window=window, splits=getattr(batch, "kv_splits", None),
                            short_segments=getattr(batch, "single_segments", 0) or None,
                            plan_token=getattr(batch, "plan_token", 0),
                            max_portion_kv_len=getattr(batch, "max_portion_kv", 0) or None)
    else:
        ops.attn_paged_simt(q, out, cache.k_pages, cache.v_pages, cache.block_table, batch.positions,
                            batch.slot_of_token, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads,
                            head_dim=head_dim, page_size=cache.page_size, scale=scale, window=window)
