"""Typed Python entry points of the HIP kernels.

Each function checks on the host that the operands have the shapes, dtypes and
layout its kernel assumes (a kernel never sees a shape it was not written for),
then launches on torch's current HIP stream.  There is no CPU path: tensors must
live on the GPU.
"""
from __future__ import annotations

import ctypes
import dataclasses
import functools
import itertools
import math
import os

import torch

from . import lib

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
MAX_HEAD_DIM = 512
_GRID_Y_MAX = 65535


class ShapeError(ValueError):
    """Operands that a kernel was not written for."""


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise ShapeError(f"unsupported element type {t.dtype}; kernels take float32 and bfloat16")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of the current stream of the current device (the raw call is many times cheaper than building a
    Stream object, and this runs once per kernel launch)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ShapeError(msg)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ShapeError("arle_amd kernels run on the GPU only; got a CPU tensor")


def _rows(t: torch.Tensor, name: str) -> None:
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be 2-D with contiguous rows")


def _i32(t, name: str, n: int | None = None) -> None:
    _need(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(), f"{name} must be int32 1-D")
    if n is not None:
        _need(t.numel() == n, f"{name} must have {n} entries, has {t.numel()}")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ------------------------------------------------------------------ embedding


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None):
    """out[t, :] = float32(table[ids[t], :]).  ids must already be checked to lie in range."""
    _gpu(table, ids, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    _i32(ids, "ids")
    tokens, hidden = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (tokens, hidden) and out.is_contiguous(),
          "embed_gather output must be contiguous float32 [T, H]")
    lib.call("arle_embed_gather", table.data_ptr(), _code(table), ids.data_ptr(), out.data_ptr(),
             tokens, hidden, _stream())
    return out


def silu_mul_interleaved(gate_up: torch.Tensor, block: int = 16):
    """out[:, j] = silu(g_j) * u_j for a [T, 2I] buffer whose columns alternate between `block` gate
    columns and the `block` matching up columns."""
    _gpu(gate_up)
    _rows(gate_up, "gate_up")
    tokens, two_i = gate_up.shape
    _need(block > 0 and two_i % (2 * block) == 0, "interleaved gate/up width must be a multiple of 2*block")
    width = two_i // 2
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "silu_mul: width too large")
    out = torch.empty((tokens, width), dtype=gate_up.dtype, device=gate_up.device)
    lib.call("arle_silu_mul", gate_up.data_ptr(), gate_up.data_ptr(), gate_up.stride(0), out.data_ptr(),
             _code(gate_up), tokens, width, int(block), _stream())
    return out


def silu_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor | None = None):
    """out = silu(gate) * up for two [T, I] views with the same row stride."""
    _gpu(gate, up, out)
    _rows(gate, "gate")
    _rows(up, "up")
    _need(gate.shape == up.shape and gate.dtype == up.dtype and gate.stride(0) == up.stride(0),
          "gate and up must agree in shape, dtype and row stride")
    tokens, width = gate.shape
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "silu_mul: width too large")
    if out is None:
        out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    _need(out.shape == (tokens, width) and out.dtype == gate.dtype and out.is_contiguous(),
          "silu_mul output must be contiguous [T, I] of the input type")
    lib.call("arle_silu_mul", gate.data_ptr(), up.data_ptr(), gate.stride(0), out.data_ptr(),
             _code(gate), tokens, width, 0, _stream())
    return out


# ----------------------------------------------------------------------- norms


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: torch.Tensor | None = None, out: torch.Tensor | None = None):
    """out[r] = x[src(r)] / sqrt(mean(x^2) + eps) * weight;  src(r) = rows[r] or r."""
    _gpu(x, weight, rows, out)
    _rows(x, "x")
    width = x.shape[1]
    _need(weight.shape == (width,) and weight.is_contiguous(), "norm weight must be [width]")
    n_rows = x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=x.device)
    _need(out.shape == (n_rows, width) and out.dtype == out_dtype and out.is_contiguous(),
          "rmsnorm output must be contiguous [rows, width]")
    lib.call("arle_rmsnorm", x.data_ptr(), _code(x), x.stride(0), weight.data_ptr(), _code(weight),
             out.data_ptr(), _code(out), _ptr(rows), n_rows, width, float(eps), _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None,
                out: torch.Tensor | None = None):
    """residual += delta (float32, in place unless `rows` is given); out = rmsnorm(residual).

    delta is [T, H], or a stack [S, T, H] of partial sums that are added in the order of the stack
    (what a matrix product with K split over workgroups leaves behind)."""
    _gpu(residual, delta, weight, rows, out)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    _need(delta.dim() in (2, 3) and tuple(delta.shape[-2:]) == tuple(residual.shape) and delta.is_contiguous()
          and delta.dtype in _CODES and (delta.dim() == 2 or delta.shape[0] >= 1),
          "delta must match the residual ([T, H] or a stack [S, T, H])")
    n_delta = delta.shape[0] if delta.dim() == 3 else 1
    width = residual.shape[1]
    _need(weight.shape == (width,) and weight.is_contiguous(), "norm weight must be [width]")
    n_rows = residual.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=residual.device)
    _need(out.shape == (n_rows, width) and out.dtype == out_dtype and out.is_contiguous(),
          "add_rmsnorm output must be contiguous [rows, width]")
    lib.call("arle_add_rmsnorm", residual.data_ptr(), delta.data_ptr(), n_delta, residual.numel(), _code(delta),
             weight.data_ptr(), _code(weight), out.data_ptr(), _code(out), _ptr(rows), n_rows, width,
             float(eps), _stream())
    return out


# ------------------------------------------------------------------- products


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None):
    """out[M, N] = a[M, K] . w[N, K]^T in true float32, fixed k order."""
    _gpu(a, w, out)
    _rows(a, "a")
    _rows(w, "w")
    _need(a.dtype == torch.float32 and w.dtype == torch.float32, "gemm_f32 takes float32 operands")
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_f32: inner sizes differ ({K} vs {w.shape[1]})")
    _need(math.ceil(M / 64) <= _GRID_Y_MAX, "gemm_f32: too many rows for one launch")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    _rows(out, "out")
    _need(out.shape == (M, N) and out.dtype == torch.float32, "gemm_f32 output must be float32 [M, N]")
    lib.call("arle_gemm_f32", a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(),
             out.stride(0), M, N, K, _stream())
    return out


# ------------------------------------------------------ q/k preparation + cache


def qk_prep(q, k, v, *, num_q_heads: int, num_kv_heads: int, head_dim: int, eps: float,
            q_weight=None, k_weight=None, cos=None, sin=None, rotary_dim: int = 0,
            positions=None, slot_of_token=None, block_table=None, k_pages=None, v_pages=None,
            page_size: int = 0, parts=None):
    """Per-head norm + rotation of q and k in place; k and v written to the paged cache.

    q [T, nq*D], k, v [T, nkv*D] (row views of one fused buffer are fine).  With no
    cache given k is rewritten in place and v is left alone.

    parts: float32 [S, T, (nq + 2 nkv) * D], a stack of partial products of the fused q|k|v projection.
    Then the values are the sums over the stack (in order), q is an output only, and k, v are None:
    they go to the cache, which must be given unless num_kv_heads is 0 (a layer that only needs q).
    """
    _gpu(q, k, v, q_weight, k_weight, cos, sin, positions, slot_of_token, block_table, k_pages, v_pages, parts)
    tokens = q.shape[0]
    D = head_dim
    _need(0 < D <= MAX_HEAD_DIM, f"head_dim {D} is outside the supported range 1..{MAX_HEAD_DIM}")
    part_args = (0, 0, 0, 0)
    if parts is not None:
        width = (num_q_heads + 2 * num_kv_heads) * D
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[0] >= 1
              and tuple(parts.shape[1:]) == (tokens, width) and parts.is_contiguous(),
              f"parts must be contiguous float32 [S, {tokens}, {width}]")
        _need(k is None and v is None, "with parts, k and v are not given: they go to the cache")
        _need(num_kv_heads == 0 or k_pages is not None, "with parts, k and v need the cache to go to")
        _rows(q, "q")
        _need(q.shape == (tokens, num_q_heads * D), "q must be [T, heads*D]")
        part_args = (parts.data_ptr(), parts.shape[0], tokens * width, width)
        k = v = q   # never read or written in this mode
    else:
        for name, t, heads in (("q", q, num_q_heads), ("k", k, num_kv_heads), ("v", v, num_kv_heads)):
            _rows(t, name)
            _need(t.shape == (tokens, heads * D), f"{name} must be [T, heads*D]")
            _need(t.dtype == q.dtype, "q, k and v must share one element type")
    _need((q_weight is None) == (k_weight is None), "give both q and k norm weights or neither")
    w_code = F32
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype == k_weight.dtype
              and q_weight.is_contiguous() and k_weight.is_contiguous(),
              "q/k norm weights must be [head_dim] of one type")
        w_code = _code(q_weight)
    _i32(positions, "positions", tokens)
    if rotary_dim:
        _need(rotary_dim % 2 == 0 and rotary_dim <= D, "rotary_dim must be even and <= head_dim")
        _need(cos is not None and sin is not None and cos.dtype == torch.float32
              and sin.dtype == torch.float32 and cos.dim() == 2 and cos.shape == sin.shape
              and cos.shape[1] == rotary_dim // 2 and cos.is_contiguous() and sin.is_contiguous(),
              "cos/sin must be contiguous float32 [positions, rotary_dim/2]")
    table_stride = 0
    if k_pages is not None or v_pages is not None:
        _need(k_pages is not None and v_pages is not None, "give both k and v pages or neither")
        _need(page_size > 0, "page_size must be positive")
        _check_pages(k_pages, v_pages, num_kv_heads, page_size, D, q.dtype)
        _i32(slot_of_token, "slot_of_token", tokens)
        _need(block_table is not None and block_table.dtype == torch.int32 and block_table.dim() == 2
              and block_table.is_contiguous(), "block_table must be contiguous int32 [slots, pages]")
        table_stride = block_table.shape[1]
    heads = num_q_heads + 2 * num_kv_heads
    _need(math.ceil(heads / 4) <= _GRID_Y_MAX, "too many heads")
    lib.call("arle_qk_prep", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(),
             v.stride(0), _code(q), _ptr(q_weight), _ptr(k_weight), w_code, _ptr(cos), _ptr(sin),
             int(rotary_dim), positions.data_ptr(), _ptr(slot_of_token), _ptr(block_table),
             table_stride, _ptr(k_pages), _ptr(v_pages), tokens, num_q_heads, num_kv_heads, D,
             int(page_size), float(eps), *part_args, _stream())


# ------------------------------------------------------------------ attention


def _check_pages(k_pages, v_pages, nkv, page_size, D, dtype):
    """Keys [pages, nkv, page_size, D]; values d-major inside a page [pages, nkv, D, page_size]."""
    _need(k_pages.dim() == 4 and tuple(k_pages.shape[1:]) == (nkv, page_size, D) and k_pages.is_contiguous()
          and k_pages.dtype == dtype, "k_pages must be contiguous [pages, nkv, page_size, D]")
    _need(v_pages.dim() == 4 and tuple(v_pages.shape[1:]) == (nkv, D, page_size) and v_pages.is_contiguous()
          and v_pages.dtype == dtype and v_pages.shape[0] == k_pages.shape[0],
          "v_pages must be contiguous [pages, nkv, D, page_size]")


def _check_paged(q, out, k_pages, v_pages, block_table, positions, slot_of_token, nq, nkv, D,
                 page_size):
    _gpu(q, out, k_pages, v_pages, block_table, positions, slot_of_token)
    tokens = q.shape[0]
    _rows(q, "q")
    _rows(out, "out")
    _need(q.shape == (tokens, nq * D) and out.shape == (tokens, nq * D) and out.dtype == q.dtype,
          "q and out must be [T, nq*D] of one type")
    _need(nkv > 0 and nq % nkv == 0, "number of q heads must be a multiple of the kv heads")
    _check_pages(k_pages, v_pages, nkv, page_size, D, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)


def attn_paged_simt(q, out, k_pages, v_pages, block_table, positions, slot_of_token, *,
                    num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                    scale: float, window: int = 0, row_list=None):
    """Causal attention of every token row (or of `row_list`) over its request's cached keys."""
    _check_paged(q, out, k_pages, v_pages, block_table, positions, slot_of_token, num_q_heads,
                 num_kv_heads, head_dim, page_size)
    _need(0 < head_dim <= MAX_HEAD_DIM, f"head_dim {head_dim} outside 1..{MAX_HEAD_DIM}")
    _need(num_q_heads <= _GRID_Y_MAX, "too many heads")
    n_rows = q.shape[0]
    if row_list is not None:
        _gpu(row_list)
        _i32(row_list, "row_list")
        n_rows = row_list.numel()
    lib.call("arle_attn_paged_simt", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), _code(q), block_table.data_ptr(),
             block_table.shape[1], positions.data_ptr(), slot_of_token.data_ptr(), _ptr(row_list),
             n_rows, num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window),
             _stream())
    return out


MFMA_MAX_HEAD_DIM = 256
_MFMA_TARGET_WAVES = 768    # workgroups wanted for a decode launch: three a compute unit (measured in whole decode steps at batch 4..64; 2,048 gave 3 % less at batch 8, 5 % less at batch 32)


def attn_mfma_supported(dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 0 < head_dim <= MFMA_MAX_HEAD_DIM
            and page_size >= 4 and page_size & (page_size - 1) == 0)


def decode_split_cap(max_kv_len: int) -> int:
    """Most splits worth making for keys up to max_kv_len: at least two 32-key blocks each, at most 64
    (the merge keeps the statistics of one split in each lane of a wave), and a power of two, so that a
    context that grows passes through few different values (a captured decode step is made for one)."""
    most = max(1, min(-(-max_kv_len // 32) // 2, 64))
    return 1 << (most.bit_length() - 1)


_ATTN_ROW_TILE = 16   # rows of the matrix-core tile: a segment with more rows goes to the LDS kernel


def decode_splits(segments: int, num_kv_heads: int, max_kv_len: int) -> int:
    """Split-KV factor of a step of single decoded tokens: enough waves to fill the chip."""
    return max(1, min(-(-_MFMA_TARGET_WAVES // (segments * num_kv_heads)), decode_split_cap(max_kv_len)))


_PORTION_SPLITS_MAX = 8         # parts into which the keys of a portion's row block may be cut
_PORTION_ROWS = 128             # rows of a row block of the portions kernel
_PORTION_LIST_MAX = 16384       # (row block, segment) pairs that its work list holds
_PORTION_WS_BYTES = 256 << 20   # most memory for the parts


@functools.lru_cache(maxsize=None)
def _compute_units(device_index: int) -> int:
    return int(torch.cuda.get_device_properties(device_index).multi_processor_count)


def portion_key_splits(tokens: int, max_qlen: int, long_segments: int, num_q_heads: int, num_kv_heads: int,
                       head_dim: int, max_kv_len: int, device) -> int:
    """Into how many parts the keys of every row block of a prompt portion are cut.

    The portions kernel gives a row block of 128 rows (tokens x q heads of a kv head) to a workgroup.  A short
    portion has fewer row blocks than the chip has compute units, however long its context: then the keys are
    cut too, each part about a thousand keys long at least (the parts are merged by a kernel of its own, which
    writes and reads every part's rows: for a fresh 512-token prompt two parts cost more than they save), and
    the parts are merged afterwards.  The number depends on the shape of the step and on the power-of-two class of
    the longest context only, like the split of decoded tokens, so that a captured step and an eager one choose
    alike.
    """
    group = num_q_heads // num_kv_heads
    blocks = -(-max_qlen * group // _PORTION_ROWS)
    items = blocks * num_kv_heads * max(1, long_segments)
    units = _compute_units(device.index if device.index is not None else torch.cuda.current_device())
    if items >= units or blocks * max(1, long_segments) > _PORTION_LIST_MAX:
        return 1
    most = max(1, (1 << (max(int(max_kv_len), 1).bit_length() - 1)) // 1024)    # 2 from 2,048 keys on, 4 from 4,096, ...
    parts = min(-(-2 * units // items), _PORTION_SPLITS_MAX, most)    # up to two items a compute unit
    while parts > 1 and tokens * num_q_heads * parts * (head_dim + 2) * 4 > _PORTION_WS_BYTES:
        parts -= 1
    return parts


def attn_paged_mfma(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *,
                    max_qlen: int, max_kv_len: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                    page_size: int, scale: float, window: int = 0, splits: int | None = None,
                    min_qlen: int = 1, short_segments: int | None = None, portion_splits: int | None = None,
                    plan_token: int = 0, max_portion_kv_len: int | None = None):
    """Causal attention of a packed step on the matrix cores (bfloat16).

    Segments: rows seg_row0[s]..seg_row0[s+1] belong to block-table row seg_slot[s] and start at
    position seg_start[s].  Segments whose rows (tokens x q heads of a kv head) fit one row tile of 16,
    decoded tokens above all, are split over the keys (split-KV), also beside longer portions in one
    step; `short_segments` says how many there are (default: all), which sets the number of splits.
    Longer portions that are too few to fill the chip have their keys cut into `portion_splits` parts
    (default: portion_key_splits).  `plan_token` (new_plan_token()) names the step: with the same token and the
    same segments the portions kernels list their work once, for the first layer, and not once a layer.
    `max_portion_kv_len`: the longest context among the segments of more than one token (default: max_kv_len); what
    the portions kernels plan by, so that a fresh portion beside requests that decode deep into their contexts is
    not cut into parts for the decoders' sake.
    """
    _gpu(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start)
    tokens = q.shape[0]
    _rows(q, "q")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "the MFMA attention takes bfloat16")
    _need(q.shape == (tokens, num_q_heads * head_dim) and out.shape == q.shape and out.is_contiguous(),
          "q must be [T, nq*D] and out contiguous [T, nq*D]")
    _need(attn_mfma_supported(q.dtype, head_dim, page_size),
          f"the MFMA attention needs head_dim % 16 == 0, head_dim <= {MFMA_MAX_HEAD_DIM} and a power-of-two page_size >= 4 "
          f"(got head_dim {head_dim}, page_size {page_size})")
    _need(q.data_ptr() % 16 == 0 and (q.stride(0) * 2) % 16 == 0, "q rows must be 16-byte aligned")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0, "q heads must be a multiple of kv heads")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    _need(1 <= min_qlen <= max_qlen <= tokens, "need 1 <= min_qlen <= max_qlen <= tokens")
    group = num_q_heads // num_kv_heads
    if min_qlen * group > _ATTN_ROW_TILE:
        splits = 1                      # no segment is short enough for the kernel that splits the keys
    elif splits is None:
        short = segments if short_segments is None else max(1, min(short_segments, segments))
        splits = decode_splits(short, num_kv_heads, max_kv_len)
    _need(segments * splits <= _GRID_Y_MAX and num_kv_heads <= _GRID_Y_MAX, "too many segments for one launch")
    ws_o = ws_ml = None
    if splits > 1:
        ws_rows = segments * max(1, min(max_qlen, _ATTN_ROW_TILE // group))   # arle_attn_ws_rows a segment
        ws_o = torch.empty((ws_rows, num_q_heads, splits, head_dim), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((ws_rows, num_q_heads, splits, 2), dtype=torch.float32, device=q.device)
    if portion_splits is None:
        long_segments = segments if short_segments is None else max(1, segments - short_segments)
        portion_splits = portion_key_splits(tokens, max_qlen, long_segments, num_q_heads, num_kv_heads, head_dim,
                                            max_portion_kv_len or max_kv_len, q.device)
    if max_qlen * group <= _ATTN_ROW_TILE:
        portion_splits = 1              # no portion for the kernel that they are for
    _need(1 <= portion_splits <= _PORTION_SPLITS_MAX, f"portion_splits must be 1..{_PORTION_SPLITS_MAX}")
    pws_o = pws_ml = None
    if portion_splits > 1:
        pws_o = torch.empty((tokens, num_q_heads, portion_splits, head_dim), dtype=torch.float32, device=q.device)
        pws_ml = torch.empty((tokens, num_q_heads, portion_splits, 2), dtype=torch.float32, device=q.device)
    lib.call("arle_attn_paged_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             seg_row0.data_ptr(), seg_slot.data_ptr(), seg_start.data_ptr(), segments, int(max_qlen),
             int(min_qlen), int(max_portion_kv_len or max_kv_len), tokens,
             num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window), int(splits),
             _ptr(ws_o), _ptr(ws_ml), int(portion_splits), _ptr(pws_o), _ptr(pws_ml), int(plan_token), _stream())
    return out


_PREP_HEAD_DIMS = (64, 128)


def attn_decode_prep_supported(dtype, head_dim: int, page_size: int, group: int, rotary_dim: int) -> bool:
    """Whether attn_decode_prep takes these sizes: bfloat16 pages, a head_dim whose kernel is made for it, up to 16
    q heads a kv head, and a rotated width whose halves are whole chunks of 32 columns (or none)."""
    return (attn_mfma_supported(dtype, head_dim, page_size) and head_dim in _PREP_HEAD_DIMS and 1 <= group <= _ATTN_ROW_TILE
            and rotary_dim % 64 == 0 and 0 <= rotary_dim <= head_dim)


def attn_decode_prep(parts, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *, max_kv_len: int,
                     num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int, scale: float, eps: float,
                     q_weight=None, k_weight=None, cos=None, sin=None, rotary_dim: int = 0, window: int = 0,
                     splits: int | None = None):
    """A step of single decoded tokens (segment s is token row s) from the float32 stack of partial products
    [S, T, (nq + 2 nkv) D] of its fused q|k|v projection, or from the projection itself in bfloat16 [T, (nq + 2 nkv) D]:
    what qk_prep and attn_paged_mfma do one after the other, in the attention's own kernel.  Every wave sums, norms and rotates its q heads itself; the wave whose keys end
    with the new token's does the same for the k head, writes key and value into the cache and uses them from its
    registers.  out: bfloat16 [T, nq*D]."""
    _gpu(parts, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, q_weight, k_weight, cos, sin)
    group = num_q_heads // max(num_kv_heads, 1)
    width = (num_q_heads + 2 * num_kv_heads) * head_dim
    whole = parts.dim() == 2     # the projection itself, not a stack of parts
    if whole:
        _rows(parts, "parts")
        _need(parts.dtype == torch.bfloat16 and parts.shape[1] == width and parts.stride(0) % 8 == 0
              and parts.data_ptr() % 16 == 0, f"a whole projection must be bfloat16 [T, {width}] with 16-byte aligned rows")
        n_parts, part_stride, row_stride, tokens = 1, 0, parts.stride(0), parts.shape[0]
    else:
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[0] >= 1 and parts.shape[2] == width
              and parts.is_contiguous(), f"parts must be contiguous float32 [S, T, {width}]")
        n_parts, part_stride, row_stride, tokens = parts.shape[0], parts.stride(0), parts.stride(1), parts.shape[1]
    _need(out.dtype == torch.bfloat16 and out.shape == (tokens, num_q_heads * head_dim) and out.is_contiguous(),
          "out must be contiguous bfloat16 [T, nq*D]")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0, "q heads must be a multiple of kv heads")
    _need(attn_decode_prep_supported(out.dtype, head_dim, page_size, group, rotary_dim),
          f"attn_decode_prep takes head_dim {_PREP_HEAD_DIMS}, up to {_ATTN_ROW_TILE} q heads a kv head and a rotated width "
          f"that is a multiple of 64 (got head_dim {head_dim}, {group} heads, rotary_dim {rotary_dim})")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, out.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _need(segments == tokens, "attn_decode_prep takes one token a segment")
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    _need((q_weight is None) == (k_weight is None), "give both q and k norm weights or neither")
    w_f32 = 0
    if q_weight is not None:
        _need(q_weight.shape == (head_dim,) and k_weight.shape == (head_dim,) and q_weight.dtype == k_weight.dtype
              and q_weight.dtype in (torch.float32, torch.bfloat16) and q_weight.is_contiguous() and k_weight.is_contiguous()
              and q_weight.data_ptr() % 16 == 0 and k_weight.data_ptr() % 16 == 0,
              "q/k norm weights must be 16-byte aligned [head_dim] of one type, float32 or bfloat16")
        w_f32 = int(q_weight.dtype == torch.float32)
    if rotary_dim:
        _need(cos is not None and sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
              and cos.dim() == 2 and cos.shape == sin.shape and cos.shape[1] == rotary_dim // 2 and cos.is_contiguous()
              and sin.is_contiguous() and cos.data_ptr() % 16 == 0 and sin.data_ptr() % 16 == 0,
              "cos/sin must be contiguous 16-byte aligned float32 [positions, rotary_dim/2]")
    if splits is None:
        splits = decode_splits(segments, num_kv_heads, max_kv_len)
    _need(1 <= splits <= 64, "splits must be 1..64")
    _need(segments * splits <= _GRID_Y_MAX and num_kv_heads <= _GRID_Y_MAX, "too many segments for one launch")
    ws_o = ws_ml = None
    if splits > 1:
        ws_o = torch.empty((segments, num_q_heads, splits, head_dim), dtype=torch.float32, device=out.device)
        ws_ml = torch.empty((segments, num_q_heads, splits, 2), dtype=torch.float32, device=out.device)
    lib.call("arle_attn_decode_prep", parts.data_ptr(), int(whole), n_parts, part_stride, row_stride, _ptr(q_weight),
             _ptr(k_weight), w_f32, _ptr(cos), _ptr(sin), int(rotary_dim), float(eps), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], seg_row0.data_ptr(),
             seg_slot.data_ptr(), seg_start.data_ptr(), segments, num_q_heads, num_kv_heads, head_dim, page_size,
             float(scale), int(window), int(splits), _ptr(ws_o), _ptr(ws_ml), _stream())
    return out


_plan_tokens = itertools.count(1)


def new_plan_token() -> int:
    """A number that no other step of this process has (attn_paged_mfma's plan_token)."""
    return next(_plan_tokens)


def attn_decode_static(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *, max_qlen: int,
                       num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int, scale: float,
                       window: int = 0, splits: int = 1):
    """attn_paged_mfma for steps whose every segment fits one row tile of 16, with the split-KV partial results
    in the library's fixed device array: the call allocates nothing (for code under graph capture and other
    callers that cannot allocate).  Steps too large for the array raise with the library's reason; calls that
    overlap on one GPU race on the array."""
    _gpu(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start)
    tokens = q.shape[0]
    _rows(q, "q")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "the MFMA attention takes bfloat16")
    _need(q.shape == (tokens, num_q_heads * head_dim) and out.shape == q.shape and out.is_contiguous(),
          "q must be [T, nq*D] and out contiguous [T, nq*D]")
    _need(q.data_ptr() % 16 == 0 and (q.stride(0) * 2) % 16 == 0, "q rows must be 16-byte aligned")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    status = lib.function("arle_attn_decode_static")(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], seg_row0.data_ptr(), seg_slot.data_ptr(), seg_start.data_ptr(),
        segments, int(max_qlen), num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window), int(splits),
        _stream())
    if status != 0:
        why = lib.function_raw("arle_attn_decode_static_error", ctypes.c_char_p)().decode()
        raise lib.KernelError(why or f"arle_attn_decode_static failed with HIP error {status}")
    return out


# ------------------------------------------------------------------- sampling


def _logits(logits):
    _gpu(logits)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.is_contiguous(),
          "logits must be contiguous float32 [rows, vocab]")
    return logits.shape


@functools.lru_cache(maxsize=None)
def _argmax_chunks(rows: int, vocab: int) -> int:
    """Into how many chunks the argmax kernel cuts each row (it wants scratch for more than one)."""
    return int(lib.function("arle_argmax_chunks")(rows, vocab))


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    rows, vocab = _logits(logits)
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    chunks = _argmax_chunks(rows, vocab)
    parts = torch.empty((rows, chunks, 2), dtype=torch.int32, device=logits.device) if chunks > 1 else None
    lib.call("arle_argmax_rows", logits.data_ptr(), rows, vocab, out.data_ptr(),
             parts.data_ptr() if parts is not None else 0, _stream())
    return out


def token_logprobs(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """float32 [rows]: log softmax(logits[r])[tokens[r]], natural logarithm (tokens int32 [rows])."""
    rows, vocab = _logits(logits)
    _gpu(tokens)
    _i32(tokens, "tokens", rows)
    out = torch.empty((rows,), dtype=torch.float32, device=logits.device)
    lib.call("arle_token_logprobs", logits.data_ptr(), rows, vocab, tokens.data_ptr(), out.data_ptr(), _stream())
    return out


@functools.lru_cache(maxsize=None)
def _sample_scratch_bytes(rows: int, vocab: int) -> int:
    fn = lib.function("arle_sample_scratch_bytes")
    fn.restype = ctypes.c_longlong
    return int(fn(rows, vocab))


def sample_rows(logits, temperature, top_k, top_p, min_p, u, *, use_top_k: bool = True,
                use_top_p: bool = True) -> torch.Tensor:
    """One token id per row; per-row float32 temperature/top_p/min_p/u and int32 top_k.

    use_top_k / use_top_p = False promise that no row has that filter switched on (top_k in 1..vocab-1,
    top_p < 1): the passes over the row that look for its threshold are then not launched.
    """
    rows, vocab = _logits(logits)
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32),
                        ("u", u, torch.float32)):
        _gpu(t)
        _need(t.dtype == dt and t.shape == (rows,) and t.is_contiguous(), f"{name} must be {dt} [rows]")
    probs = torch.empty((rows, vocab), dtype=torch.float32, device=logits.device)
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    words = -(-_sample_scratch_bytes(rows, vocab) // 8)
    scratch = torch.zeros((words,), dtype=torch.int64, device=logits.device)   # histograms start at zero
    lib.call("arle_sample_rows", logits.data_ptr(), rows, vocab, probs.data_ptr(),
             temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), min_p.data_ptr(),
             u.data_ptr(), out.data_ptr(), scratch.data_ptr(), int(bool(use_top_k)), int(bool(use_top_p)),
             _stream())
    return out


def apply_penalties(logits, indptr, tokens, counts, repetition, frequency, presence) -> None:
    """In place: repetition, frequency and presence penalties on the listed (row, token, count)."""
    rows, vocab = _logits(logits)
    _gpu(indptr, tokens, counts, repetition, frequency, presence)
    _i32(indptr, "indptr", rows + 1)
    _i32(tokens, "tokens")
    _i32(counts, "counts", tokens.numel())
    for name, t in (("repetition", repetition), ("frequency", frequency), ("presence", presence)):
        _need(t.dtype == torch.float32 and t.shape == (rows,) and t.is_contiguous(),
              f"{name} must be float32 [rows]")
    lib.call("arle_apply_penalties", logits.data_ptr(), rows, vocab, indptr.data_ptr(),
             tokens.data_ptr(), counts.data_ptr(), repetition.data_ptr(), frequency.data_ptr(),
             presence.data_ptr(), _stream())


# ------------------------------------------------------------ bfloat16 products


ROWS_KERNEL_MAX = 64          # most rows the hand-written few-rows kernel takes
EPI_NONE, EPI_SILU_MUL = 0, 1
# How the few-rows kernel is shaped for a product (measured on MI355X together with the kernel that adds
# the stack of partial products; see the kernel for the variants):
_ROWS_TARGET_WORKGROUPS = 640    # K is split until about this many workgroups stream W
_ROWS_MAX_SPLITS = 4             # ... the consumer pays for every part of the stack (4, 8, 16 measure alike)
_ROWS_PARTIAL_BYTES = 3 << 20    # ... and the float32 partial products stay below this
_ROWS_WIDE_N = 32768             # from here on (an output head) N alone gives enough workgroups
_ROWS_NARROW_N = 4096            # up to here N gives so few that one column tile a workgroup is best
_ROWS_FUSED_MAX = 32             # gate|up with the activation in one go: as many rows as fit into LDS with all of K (27 at K = 2560): 4.20 against 4.41 ms a step at batch 20; more rows: gemm_rows_rounds
_ROWS_PREFERRED = 16             # with more rows the library is at least as fast on MI355X
_V_GENERAL, _V_FUSED_FEW, _V_NARROW, _V_SHARED = 0, 1, 2, 3
ROWS_VARIANTS = 5


def gemm_rows_supported(rows: int, k: int, x_stride: int) -> bool:
    return 0 < rows <= ROWS_KERNEL_MAX and k % 8 == 0 and x_stride % 8 == 0


def _fused_variant(rows: int) -> int:
    return _V_FUSED_FEW if rows <= 4 else _V_SHARED   # 8 rows: 20.7 against 22.3 us for the eight-column-tile workgroups


def gemm_rows_preferred(rows: int, n: int, k: int, x_stride: int, fused: bool = False) -> bool:
    """Whether the hand-written kernel, not the library, should run this product."""
    if fused:   # the activation needs whole sums: the rows of all of K in LDS at once
        return (gemm_rows_supported(rows, k, x_stride) and rows <= _ROWS_FUSED_MAX
                and _rows_min_splits(_fused_variant(rows), rows, k) == 1)
    if not gemm_rows_supported(rows, k, x_stride) or rows > _ROWS_PREFERRED:
        return False
    return True


@functools.lru_cache(maxsize=None)
def _rows_geometry(variant: int):
    """(waves that share a k slice, output columns per workgroup, can apply the fused activation) of a variant."""
    packed = lib.function("arle_gemm_rows_geometry")(variant)
    _need(packed > 0, f"gemm_rows has no variant {variant}")
    return packed >> 20, (packed >> 4) & 0xFFFF, packed & 15


@functools.lru_cache(maxsize=4096)
def _rows_min_splits(variant: int, M: int, K: int) -> int:
    """Fewest k splits with which the X rows of one slice fit into LDS."""
    fn = lib.function("arle_gemm_rows_lds")
    fn.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    cap, steps = cap_fn(), -(-K // 32)
    splits = 1
    while fn(variant, M, -(-steps // splits)) > cap:
        splits += 1
        _need(splits <= steps, f"gemm_rows: {M} rows of one k step do not fit into LDS")
    return splits


@functools.lru_cache(maxsize=4096)
def gemm_rows_plan(M: int, N: int, K: int, fused: bool = False):
    """(variant, splits) for a product: small workgroups, K split across workgroups until enough of them
    stream W, within a budget for the stack of partial products that the consumer has to add."""
    if fused:
        return _fused_variant(M), 1
    if N >= _ROWS_WIDE_N:
        variant, want = (_V_NARROW if M <= 4 else _V_SHARED), 1
    else:
        variant = _V_NARROW if N <= _ROWS_NARROW_N else _V_GENERAL
        _, columns, _ = _rows_geometry(variant)
        groups = -(-N // columns)
        want = min(-(-_ROWS_TARGET_WORKGROUPS // groups), _ROWS_MAX_SPLITS, max(1, _ROWS_PARTIAL_BYTES // (M * N * 4)))
    return variant, max(want, _rows_min_splits(variant, M, K))


def pack_weight_tiles(w: torch.Tensor) -> torch.Tensor:
    """w [N, K] bfloat16 -> [ceil(N/16), ceil(K/32), 512]: the operand tiles that gemm_rows and gemm_stream read
    with one contiguous kilobyte a wave and k step.  Tile (t, s), element 128 g + 8 i + e = w[16 t + i, 32 s + 8 g + e]
    (lane 16 g + i of the wave reads its eight elements); zeros past N and K.  A rearrangement at load time, the
    values are untouched, and the product adds them in the same order as from rows."""
    _need(w.dim() == 2 and w.dtype == torch.bfloat16, "pack_weight_tiles takes a bfloat16 [N, K] matrix")
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        w = torch.nn.functional.pad(w, (0, Kp - K, 0, Np - N))
    return w.reshape(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(Np // 16, Kp // 32, 512)


def _check_tiles(tiles, N: int, K: int) -> None:
    _need(tiles.dtype == torch.bfloat16 and tiles.is_contiguous() and tiles.dim() == 3 and tiles.shape[1:] == (-(-K // 32), 512)
          and tiles.shape[0] >= -(-N // 16) and tiles.data_ptr() % 16 == 0,
          f"operand tiles of a [{N}, {K}] matrix have the shape [{-(-N // 16)}, {-(-K // 32)}, 512], got {tuple(tiles.shape)}")


def gemm_rows(x, w, out_dtype=torch.bfloat16, epilogue: int = EPI_NONE, *, variant: int | None = None,
              splits: int | None = None, tiles: torch.Tensor | None = None):
    """x . w^T for 1..64 rows of x, with x shared through LDS inside a workgroup.

    splits == 1: returns [M, N] (or [M, N/2] with EPI_SILU_MUL) in `out_dtype`.
    splits > 1: K is also split across workgroups; returns float32 [S, M, N] partial products (S <= splits,
    no split is empty) for the consumer to add in the order of S.  With `variant` and `splits` left out
    the shape decides (gemm_rows_plan), so callers must be ready for either form.
    EPI_SILU_MUL: w holds gate and up rows interleaved in blocks of 16; out[m, j] = silu(gate_j) * up_j.
    tiles: pack_weight_tiles(w); the kernel then streams these instead of the rows of w (same sums, bit for bit).
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_rows: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_rows takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_rows writes bfloat16 or float32")
    fused = epilogue == EPI_SILU_MUL
    if variant is None or splits is None:
        plan = gemm_rows_plan(M, N, K, fused)
        variant = plan[0] if variant is None else variant
        splits = plan[1] if splits is None else splits
    _, _, can_fuse = _rows_geometry(variant)
    steps = -(-K // 32)
    per_split = -(-steps // max(1, min(splits, steps)))
    splits = -(-steps // per_split)
    if fused:
        _need(N % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
        _need(can_fuse == 1 and splits == 1,
              "the fused activation needs a variant with an even number of column tiles, and whole sums")
    _need(splits >= _rows_min_splits(variant, M, K),
          f"gemm_rows: {M} rows of {per_split * 32} columns do not fit into LDS; split K further")
    if splits > 1:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        ldo, stride, code = N, M * N, F32
    else:
        out = torch.empty((M, N // 2 if fused else N), dtype=out_dtype, device=x.device)
        ldo, stride, code = out.stride(0), 0, _CODES[out_dtype]
    if tiles is not None:
        _check_tiles(tiles, N, K)
    lib.call("arle_gemm_rows", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), ldo, stride,
             code, M, N, K, int(epilogue), variant, splits, per_split, _stream())
    return out


_ROUNDS_MAX_WORKGROUPS = 256     # one workgroup a compute unit (its x rows take most of a CU's LDS): more would run in two turns
_ROUNDS_TALL_MIN_N = 16384       # 33 to 64 rows (four row tiles a wave): only outputs this wide gain


def gemm_rows_rounds_preferred(rows: int, n: int, k: int, x_stride: int) -> bool:
    """Whether gate|up with its activation should run in the few-rows kernel that walks K in rounds (up to 64
    rows), not as the library's product and the activation kernel.  Measured on MI355X, in us, rounds against
    library, at 28 / 48 / 64 rows: 19,456 x 2,560 (Qwen3-4B) 24.4 / 27.1 / 31.0 against 27.7 / 30.4 / 31.8;
    24,576 x 4,096 (8B) 45.7 / 49.7 / 52.7 against 53.1 / 53.6 / 54.1; 6,144 x 1,024 (0.6B) 8.6 / 11.0 / 12.9
    against 12.1 / 12.8 / 12.6; 12,288 x 2,048 (1.7B, 96 workgroups) 19.9 / 22.6 / 24.9 against 20.5 / 21.4 / 21.8;
    51,200 x 5,120 (32B: 400 workgroups for 256 compute units, two turns) 105.7 / 113.8 / 123.6 against
    100.5 / 104.2 / 110.4.  So: no more workgroups than compute units, and beyond 32 rows a wide output.  Up to 16
    rows the x rows of a round are small enough for several workgroups a compute unit and the kernel is level with
    the library at every width (32B shape, 16 rows: 94 against 94 us), where the product alone without the
    activation, as a stack of parts of K, takes 123 + 5 + 5 us: so rows that the kernel without rounds cannot
    hold (14 to 16 rows at K = 5,120) come here."""
    if not (gemm_rows_supported(rows, k, x_stride) and n % 32 == 0):
        return False
    return rows <= _ROWS_PREFERRED or (-(-n // 128) <= _ROUNDS_MAX_WORKGROUPS and (rows <= 32 or n >= _ROUNDS_TALL_MIN_N))


@functools.lru_cache(maxsize=None)
def _rows_round_steps(rows: int, k: int) -> int:
    """Steps of 32 k whose x rows the fused few-rows kernel can hold in LDS at a time, cut so that the rounds
    that cover K are of one length."""
    steps = -(-k // 32)
    need = lib.function("arle_gemm_rows_lds")
    need.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    most, fit = cap_fn(), steps
    while fit > 1 and need(_V_SHARED, rows, fit) > most:
        fit -= 1
    _need(need(_V_SHARED, rows, fit) <= most, f"gemm_rows_rounds: {rows} rows of 32 columns do not fit into LDS")
    rounds = -(-steps // fit)
    return -(-steps // rounds)


def gemm_rows_rounds(x, w, out_dtype=torch.bfloat16, *, tiles: torch.Tensor | None = None, round_steps: int | None = None):
    """silu(x . gate^T) * (x . up^T) for 1..64 rows of x, w holding gate and up rows interleaved in blocks of 16:
    gemm_rows with the fused activation where the x rows of all of K do not fit into LDS at once (more than 27
    rows at K = 2,560).  K is walked in rounds of `round_steps` steps of 32, the sums stay in registers.
    Returns [M, N/2]."""
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows_rounds takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_rows_rounds: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_rows_rounds takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_rows_rounds writes bfloat16 or float32")
    _need(N % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
    if round_steps is None:
        round_steps = _rows_round_steps(M, K)
    _need(round_steps >= 1, "a round is at least one step of 32")
    round_steps = min(int(round_steps), -(-K // 32))
    need = lib.function("arle_gemm_rows_lds")
    need.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    _need(need(_V_SHARED, M, round_steps) <= cap_fn(),
          f"gemm_rows_rounds: {M} rows of {round_steps * 32} columns do not fit into LDS; take shorter rounds")
    if tiles is not None:
        _check_tiles(tiles, N, K)
    out = torch.empty((M, N // 2), dtype=out_dtype, device=x.device)
    lib.call("arle_gemm_rows_rounds", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), out.stride(0), _CODES[out_dtype], M, N, K, int(round_steps), _stream())
    return out


STREAM_VARIANTS = 5


@functools.lru_cache(maxsize=None)
def _stream_geometry(variant: int):
    """(output columns of a column group, steps of a round) of a variant of the kernel whose workgroups stay."""
    packed = lib.function("arle_gemm_stream_geometry")(variant)
    _need(packed > 0, f"gemm_stream has no variant {variant}")
    return packed >> 8, packed & 255


@functools.lru_cache(maxsize=4096)
def _stream_min_splits(variant: int, M: int, K: int) -> int:
    fn = lib.function("arle_gemm_stream_lds")
    fn.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    cap, steps = cap_fn(), -(-K // 32)
    splits = 1
    while fn(variant, M, -(-steps // splits)) > cap:
        splits += 1
        _need(splits <= steps, f"gemm_stream: {M} rows of one round do not fit into LDS")
    return splits


def gemm_stream(x, w, out_dtype=torch.bfloat16, *, variant: int = 0, splits: int | None = None,
                workgroups: int | None = None, tiles: torch.Tensor | None = None):
    """x . w^T for 1..64 rows of x by workgroups that stay: each stages its slice of x once and walks several
    groups of output columns, so that w alone is streamed (see gemm_stream_kernel).

    Returns [M, N] in `out_dtype` for one k split, else float32 [S, M, N] partial products for the consumer
    to add in the order of S.  `workgroups`: how many of them work on every k split.
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_stream takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_stream: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_stream takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_stream writes bfloat16 or float32")
    columns, _ = _stream_geometry(variant)
    least = _stream_min_splits(variant, M, K)
    steps = -(-K // 32)
    splits = max(least, splits or 1)
    per_split = -(-steps // max(1, min(splits, steps)))
    splits = -(-steps // per_split)
    _need(splits >= least, f"gemm_stream: {M} rows of {per_split * 32} columns do not fit into LDS; split K further")
    groups = -(-N // columns)
    if workgroups is None:
        workgroups = max(1, min(groups, -(-_STREAM_TARGET_WORKGROUPS // splits)))
    if splits > 1:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        ldo, stride, code = N, M * N, F32
    else:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        ldo, stride, code = out.stride(0), 0, _CODES[out_dtype]
    if tiles is not None:
        _check_tiles(tiles, N, K)
    lib.call("arle_gemm_stream", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), ldo, stride,
             code, M, N, K, variant, splits, per_split, int(workgroups), _stream())
    return out


_STREAM_TARGET_WORKGROUPS = 256   # staying workgroups in all: one for every compute unit


# The many-rows kernel that reads operand tiles takes over from the library only where whole prefill steps were
# measured faster with it on MI355X (same machine, both ways, 12 layers): gate|up with the activation fused, a hidden
# size of at most 2,560 and 2,048 to about 6,000 rows.  Qwen3-4B widths: 0.5 to 4.6 % of the step at 2,048 rows (the
# gain differs from machine to machine), 1.8 % at 4,096; hidden sizes 1,024 and 2,048: level; hidden sizes 4,096 and
# 5,120: 9 and 8 % slower, so the library keeps those.  Kernel against kernel with cold weights the library's product
# and the activation kernel take 234-272 us at 2,048 x 19,456 x 2,560 and this kernel 237-255 us; at 8,192 rows the
# library is ahead.  Plain products stay with the library (q|k|v at 2,048 rows: 85 against 60 us).
_TILES_MIN_ROWS = 2048
_TILES_MAX_ROWS = 6144
_TILES_MIN_N = 4096
_TILES_MAX_K = 2560
_TILES_BIG_ROWS = 4096      # from here on workgroups of 256 rows with the pipelined loop


def gemm_tiles_preferred(rows: int, n: int, k: int, x_stride: int, fused: bool = False) -> bool:
    """Whether the many-rows kernel that reads operand tiles, not the library, should run this product."""
    return (fused and _TILES_MIN_ROWS <= rows < _TILES_MAX_ROWS and n >= _TILES_MIN_N and k <= _TILES_MAX_K
            and k % 8 == 0 and x_stride % 8 == 0)


# (row tiles of 32 a workgroup, ring depths W|X; 1xx: the loop with the barrier in mid-step and four LDS stages[,
#  column tiles of 32 a wave: 2 unless given])
TILES_VARIANTS = ((4, 22), (4, 44), (8, 44), (8, 144), (4, 44, 1), (4, 84, 1))


def gemm_tiles(x, tiles, n: int, out_dtype=torch.bfloat16, epilogue: int = EPI_NONE, *, variant=None, splits: int = 1):
    """x [M, K] . W^T for many rows, W [n, K] given as its operand tiles (pack_weight_tiles): workgroups of
    128 or 256 rows x 256 (or 128) columns, W straight from memory into the matrix cores, x through LDS.
    EPI_SILU_MUL: gate and up rows of W interleaved in blocks of 16; returns [M, n/2].
    splits > 1: K cut into that many parts (of whole steps of 32), one workgroup each; returns the float32 stack
    [splits, M, n] for the caller to add in order."""
    _gpu(x, tiles)
    _rows(x, "x")
    _need(x.dtype == torch.bfloat16, "gemm_tiles takes bfloat16 operands")
    M, K = x.shape
    _need(K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "gemm_tiles: K and the row stride of x must be multiples of 8")
    _check_tiles(tiles, n, K)
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_tiles writes bfloat16 or float32")
    fused = epilogue == EPI_SILU_MUL
    _need(not fused or n % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
    if variant is None:
        variant = (8, 144) if M >= _TILES_BIG_ROWS else (4, 44)
    _need(tuple(variant) in TILES_VARIANTS, f"gemm_tiles has no variant {variant}")
    col_tiles = variant[2] if len(variant) > 2 else 2
    steps = -(-K // 32)
    _need(1 <= splits <= steps, f"gemm_tiles cannot cut {steps} steps of K into {splits} parts")
    per = -(-steps // splits)
    splits = -(-steps // per)   # parts of `per` steps cover K; the last one may be shorter
    if splits > 1:
        _need(not fused and out_dtype == torch.float32, "parts of K come back as a float32 stack without an epilogue")
        out = torch.empty((splits, M, n), dtype=torch.float32, device=x.device)
        ldo, stride = out.stride(1), out.stride(0)
    else:
        out = torch.empty((M, n // 2 if fused else n), dtype=out_dtype, device=x.device)
        ldo, stride = out.stride(0), 0
    lib.call("arle_gemm_tiles", x.data_ptr(), x.stride(0), tiles.data_ptr(), out.data_ptr(), ldo,
             _CODES[out_dtype], M, n, K, int(epilogue), variant[0], col_tiles, variant[1], splits, per, stride, _stream())
    return out


def sum_partials(parts: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[S, ...] float32 -> [...]: the stack added in order."""
    _gpu(parts)
    _need(parts.dtype == torch.float32 and parts.dim() >= 2 and parts.is_contiguous() and parts.shape[0] >= 1,
          "sum_partials takes a contiguous float32 stack")
    _need(out_dtype in _CODES, "sum_partials writes bfloat16 or float32")
    out = torch.empty(parts.shape[1:], dtype=out_dtype, device=parts.device)
    lib.call("arle_sum_partials", parts.data_ptr(), parts.shape[0], out.numel(), out.data_ptr(), _CODES[out_dtype],
             out.numel(), _stream())
    return out


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, partials_ok: bool = False,
              tiles: torch.Tensor | None = None):
    """out[M, N] = x[M, K] . w[N, K]^T, bfloat16 operands, float32 accumulation.

    Few rows (decode steps, short portions) run the hand-written weight-streaming kernels.  More rows go
    to the vendor library (hipBLASLt through torch.matmul), the matrix product the reference also leaves
    to a library (crates/cuda-kernels/csrc/gemm/gemv.cu:240-330).  Which kernel it is for a shape is decided in
    one place, `choose_product`: by a measured table where one is loaded for these widths, else by the rules.
    partials_ok: the caller adds a float32 stack [S, M, N] itself (in the order of S) if that is what the
    kernel leaves behind; otherwise the stack is added here by one more small kernel.
    tiles: pack_weight_tiles(w), for the hand-written kernels to stream instead of w.
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_bf16 takes bfloat16 operands")
    _need(x.shape[1] == w.shape[1], f"gemm_bf16: inner sizes differ ({x.shape[1]} vs {w.shape[1]})")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_bf16 writes bfloat16 or float32")
    rows, n, k = x.shape[0], w.shape[0], x.shape[1]
    choice = choose_product(rows, n, k, x.stride(0), tiled=tiles is not None, fused=False, partials_ok=partials_ok,
                            aligned=x.data_ptr() % 16 == 0)
    return run_product(choice, x, w, tiles, out_dtype, partials_ok)


# The library runs a product with a narrow output and a long K (o and down: 2,560 columns) as a few dozen
# workgroups that each walk all of K, and takes as long for 128 rows as for 1,024 (down of the Qwen3-4B shape: 60 us
# at 512 rows, where reading the weights takes 10 and the products 17).  Cut into parts along K, as one batched
# product of the parts, it fills the chip: 33 us at 512 rows, 29 at 128.  The parts come back as a float32 stack
# for the consumer to add in order, like the stacks of the few-rows kernels (added in float32, where the single
# product rounds its sum to bfloat16).  More parts make a larger stack to write and read, so wide outputs and
# rows beyond 1,024 stay whole.  Outputs of 5,120 columns (the 14B and 32B shapes) gain most: down (5,120 x 25,600)
# whole takes 172 / 182 / 261 / 272 / 349 us at 65 / 128 / 256 / 512 / 1,024 rows and 60 / 63 / 79 / 120 / 247 in
# parts; o (5,120 x 8,192) 31 / 46 / 74 / 70 / 94 whole and 31 / 32 / 37 / 48 / 89 in parts.
_LIB_SPLIT_MAX_N = 5120
_LIB_SPLIT_MIN_K = 2048
_LIB_SPLIT_MAX_ROWS = 1024
_LIB_SPLIT_LONG_K = 8192
_LIB_SPLIT_LONG_K_MAX_ROWS = 3072
_BMM_OUT_DTYPE_OK = None


# A product with a narrow output and 65 to 256 rows (o and down of a large decode batch or a short portion) is a
# matter of streaming W, and the library gives it a few dozen workgroups.  gemm_tiles with workgroups of 128 rows x
# 128 columns and K cut into parts, so that about 160 to 200 workgroups stream at once, leaves a float32 stack like
# the few-rows kernels.  Measured on MI355X at the Qwen3-4B shape, in us: o (2,560 x 4,096) at 96 / 128 / 256 rows
# 13.0 / 14.7 / 19.3 against 23.4 / 23.8 / 22.0 for the library's batched parts; down (2,560 x 9,728) at 96 / 128 /
# 192 rows 20.7 / 23.7 / 30.2 against 28.4 / 30.1 / 33.7, and behind at 256 (34.7 against 25.8).  For q|k|v the
# larger stack costs the consumer what the product gains, and gate|up needs whole sums for its activation.
_NARROW_TILES_VARIANT = (4, 44, 1)
_NARROW_TILES_MAX_N = 4096
_NARROW_TILES_MIN_K = 2048
_NARROW_TILES_WORKGROUPS = 200


def narrow_tiles_splits(rows: int, n: int, k: int, x_stride: int) -> int:
    """Into how many parts along K gemm_tiles' narrow workgroups cut such a product; 0: they do not take it."""
    most_rows = 256 if k < 8192 else 192
    if not (ROWS_KERNEL_MAX < rows <= most_rows and n <= _NARROW_TILES_MAX_N and k >= _NARROW_TILES_MIN_K
            and k % 8 == 0 and x_stride % 8 == 0):
        return 0
    blocks = -(-n // 128) * -(-rows // 128)
    splits = 8
    while splits > 1 and (blocks * splits > _NARROW_TILES_WORKGROUPS or k < 320 * splits):
        splits //= 2
    return splits if splits > 1 else 0


def library_k_splits(rows: int, n: int, k: int) -> int:
    """Into how many parts along K the library's product is cut (1: not at all)."""
    if not (ROWS_KERNEL_MAX < rows and n <= _LIB_SPLIT_MAX_N and k >= _LIB_SPLIT_MIN_K):
        return 1
    if rows > _LIB_SPLIT_MAX_ROWS:
        # a very long K still gains from two parts: down of the Qwen3-4B shape 76 / 91 / 126 us at 1,536 / 2,048 /
        # 3,072 rows against 92 / 111 / 146 whole (the consumer pays 6 to 10 us for the stack); at 4,096 whole is ahead
        if not (k >= _LIB_SPLIT_LONG_K and rows <= _LIB_SPLIT_LONG_K_MAX_ROWS):
            return 1
        splits = 2
    elif k >= 8192:
        splits = 8 if rows <= 256 else 4
    else:
        splits = 4 if rows <= 512 else 2
    while splits > 1 and k % (32 * splits):
        splits //= 2
    return splits


def _bmm_takes_out_dtype(device) -> bool:
    """Whether this torch's batched product hands back float32 sums of bfloat16 operands; asked once, on a tiny
    product, so that no failure of a real call (out of memory, say) is taken for the answer."""
    global _BMM_OUT_DTYPE_OK
    if _BMM_OUT_DTYPE_OK is None:
        probe = torch.zeros((2, 16, 32), dtype=torch.bfloat16, device=device)
        try:
            torch.bmm(probe, probe.transpose(1, 2), out_dtype=torch.float32)
            _BMM_OUT_DTYPE_OK = True
        except (TypeError, RuntimeError):
            _BMM_OUT_DTYPE_OK = False
    return _BMM_OUT_DTYPE_OK


def _library_mm_split_k(x, w, splits: int):
    """float32 [splits, M, N]: part s is x[:, s-th part of K] . w[:, s-th part of K]^T; None if this torch cannot
    give a batched product float32 results."""
    if not _bmm_takes_out_dtype(x.device):
        return None
    m, k = x.shape
    n, part = w.shape[0], k // splits
    xs = x.as_strided((splits, m, part), (part, x.stride(0), 1))
    ws = w.as_strided((splits, part, n), (part, 1, w.stride(0)))
    return torch.bmm(xs, ws, out_dtype=torch.float32)


# 17..64 rows: the kernel whose workgroups stay beats the library where the output is narrow and K long (the
# o and down projections: 11 against 15 us and 19 against 29 us at 64 rows of the Qwen3-4B shapes); for wide
# outputs (q|k|v, gate|up) the two are level and the library stays.
_STREAM_VARIANT = 0
_STREAM_SPLITS = 6              # at least so many k splits ...
_STREAM_STEPS_A_SPLIT = 50      # ... and at most so many steps of 32 in one (the 32B shape's down, K = 25600: 16 splits)
_STREAM_MAX_N = 5120            # 60 against the library's 146 us there at 32 rows, 97 against 157 us at 64
_STREAM_MIN_K = 2048


_STREAM_PARTIAL_BYTES = 8 << 20  # a larger stack of partial products is added before it is handed on


# From operand tiles (one contiguous kilobyte a wave and k step) the staying kernel does better still, measured on
# MI355X at the Qwen3-4B shapes: narrow outputs from 9 rows on (down at 16 rows: 12.8 us against 21.1 us of the
# few-rows kernel, which stages x again for every column group); q|k|v (6144 columns) at 17..64 rows with eight
# waves a workgroup and four k splits: 10.1 against the library's 11.9 us at 32 rows, 12.1 against 16.3 us at 64;
# gate|up (19456 columns) stays level with the library, and stays there.
_STREAM_TILED_FROM_ROWS = 8
_STREAM_TILED_MAX_N = 8192
_STREAM_TILED_WIDE = (1, 4)     # (variant, k splits) for outputs wider than _STREAM_MAX_N
_STREAM_TILED_MANY_ROWS = 32    # from here on eight waves a workgroup (variant 1) for the narrow outputs too


def _stream_splits(rows: int, k: int, variant: int = _STREAM_VARIANT) -> int:
    return max(_STREAM_SPLITS, -(-k // (32 * _STREAM_STEPS_A_SPLIT)), _stream_min_splits(variant, rows, k))


def _stream_plan(rows: int, n: int, k: int, tiled: bool):
    """(variant, k splits) of the staying kernel for a product."""
    if tiled and n > _STREAM_MAX_N:
        variant, splits = _STREAM_TILED_WIDE
        return variant, max(splits, _stream_min_splits(variant, rows, k))
    variant = 1 if (tiled and rows > _STREAM_TILED_MANY_ROWS) else _STREAM_VARIANT
    return variant, _stream_splits(rows, k, variant)


def gemm_stream_preferred(rows: int, n: int, k: int, x_stride: int, tiled: bool = False) -> bool:
    """Whether the kernel whose workgroups stay should run this product: a long K, and from rows: 17..64 rows and a
    narrow output; from operand tiles: 9..64 rows and a narrow output, 17..64 rows and a middling one."""
    least = _STREAM_TILED_FROM_ROWS if (tiled and n <= _STREAM_MAX_N) else _ROWS_PREFERRED
    widest = _STREAM_TILED_MAX_N if tiled else _STREAM_MAX_N
    return (least < rows <= ROWS_KERNEL_MAX and n <= widest and k >= _STREAM_MIN_K
            and gemm_rows_supported(rows, k, x_stride))


_MM_OUT_DTYPE_OK = None


def _library_mm_f32out(x, w):
    """bfloat16 x bfloat16 -> float32 through the library.  With a torch that takes `out_dtype` the 32-bit
    accumulators are returned as they are; an older one hands back bfloat16, which is then only widened (the
    result has been rounded once).  Which torch this is, is asked once on a tiny product."""
    global _MM_OUT_DTYPE_OK
    if _MM_OUT_DTYPE_OK is None:
        probe = torch.zeros((16, 32), dtype=torch.bfloat16, device=x.device)
        try:
            torch.mm(probe, probe.t(), out_dtype=torch.float32)
            _MM_OUT_DTYPE_OK = True
        except (TypeError, RuntimeError):
            _MM_OUT_DTYPE_OK = False
    if _MM_OUT_DTYPE_OK:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return torch.matmul(x, w.t()).float()


# ------------------------------------------------------ which kernel runs a product
#
# One place decides.  A choice names a kernel and what it needs to be launched; `product_by_rules` holds the
# thresholds that were measured at the Qwen3-4B, 8B and 32B widths (the constants above, each beside the numbers that
# set it); a table measured for a model's own widths (`arle_amd.kernels.tune`, `bench.py --tune-products`) takes
# their place where one is loaded: {(N, K, fused, tiled): [(most rows, choice), ...]}.  Another width then costs a
# run of the tuner, not a reading of these rules.


@dataclasses.dataclass(frozen=True)
class ProductChoice:
    kernel: str            # "rows", "stream", "rounds", "tiles", "tiles_parts", "library", "library_parts"
    variant: tuple = ()    # the kernel's own variant, where it has several
    splits: int = 0        # parts of K; 0: the kernel's own plan


PRODUCT_KERNELS = ("rows", "stream", "rounds", "tiles", "tiles_parts", "library", "library_parts")
_PRODUCT_TABLE: dict = {}


def product_by_rules(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool, partials_ok: bool,
                     aligned: bool = True) -> ProductChoice:
    """The kernel for x[rows, k] . w[n, k]^T by the measured thresholds.  fused: gate|up with SiLU·mul (w holds
    gate and up rows interleaved in blocks of 16), whose result is the activation [rows, n/2]."""
    if fused:
        if rows and aligned and gemm_rows_preferred(rows, n, k, x_stride, fused=True):
            return ProductChoice("rows", (_fused_variant(rows),), 1)
        if rows and aligned and tiled and gemm_rows_rounds_preferred(rows, n, k, x_stride):
            return ProductChoice("rounds")
        if aligned and tiled and gemm_tiles_preferred(rows, n, k, x_stride, fused=True):
            return ProductChoice("tiles", (8, 144) if rows >= _TILES_BIG_ROWS else (4, 44))
        return ProductChoice("library")
    staying = aligned and gemm_stream_preferred(rows, n, k, x_stride, tiled=tiled)
    if not staying and aligned and gemm_rows_preferred(rows, n, k, x_stride):
        return ProductChoice("rows")
    if staying:
        variant, splits = _stream_plan(rows, n, k, tiled)
        return ProductChoice("stream", (variant,), splits)
    if partials_ok and tiled and aligned:
        splits = narrow_tiles_splits(rows, n, k, x_stride)
        if splits:
            return ProductChoice("tiles_parts", _NARROW_TILES_VARIANT, splits)
    if partials_ok:
        splits = library_k_splits(rows, n, k)
        if splits > 1:
            return ProductChoice("library_parts", (), splits)
    return ProductChoice("library")


_CANDIDATE_STACK_BYTES = 32 << 20     # a candidate may leave a stack of partial products of at most this size


def product_candidates(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool) -> list:
    """Every choice that can run this shape (what a tuner times against each other): the library whole and in parts
    of K, and the hand-written kernels in their variants with several numbers of parts."""
    found = [ProductChoice("library")]
    eight = k % 8 == 0 and x_stride % 8 == 0
    few = gemm_rows_supported(rows, k, x_stride)
    steps = -(-k // 32)
    small = lambda parts: parts * rows * n * 4 <= _CANDIDATE_STACK_BYTES
    if fused:
        if few and n % 32 == 0:
            for variant in (_V_GENERAL, _V_FUSED_FEW, _V_SHARED, 4):
                if _rows_geometry(variant)[2] == 1 and _rows_min_splits(variant, rows, k) == 1:
                    found.append(ProductChoice("rows", (variant,), 1))
            if tiled:
                found.append(ProductChoice("rounds"))
                longest = _rows_round_steps(rows, k)
                for round_steps in (8, 13, 20, 27, 40):       # shorter rounds than the longest that fits
                    if round_steps < longest:
                        found.append(ProductChoice("rounds", (round_steps,)))
        if tiled and eight and n % 32 == 0 and rows > ROWS_KERNEL_MAX:
            found += [ProductChoice("tiles", v) for v in ((4, 44), (8, 144))]
        return found
    if few:
        for variant in range(ROWS_VARIANTS):
            least = _rows_min_splits(variant, rows, k)
            for parts in (1, 2, 3, 4, 6, 8):
                if least <= parts <= steps and small(parts):
                    found.append(ProductChoice("rows", (variant,), parts))
        for variant in range(STREAM_VARIANTS):
            least = _stream_min_splits(variant, rows, k)
            for parts in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16):
                if least <= parts <= steps and small(parts):
                    found.append(ProductChoice("stream", (variant,), parts))
                    if parts in (2, 4, 8):      # and with two workgroups for every compute unit
                        found.append(ProductChoice("stream", (variant, 2 * _STREAM_TARGET_WORKGROUPS // parts), parts))
    if rows > ROWS_KERNEL_MAX // 2:
        for parts in (2, 4, 8):
            if k % (32 * parts) == 0 and small(parts):
                found.append(ProductChoice("library_parts", (), parts))
            if tiled and eight and rows <= 1024 and k >= 320 * parts and small(parts):
                found.append(ProductChoice("tiles_parts", _NARROW_TILES_VARIANT, parts))
    return list(dict.fromkeys(found))


def load_product_table(table) -> None:
    """Take a measured table in: {"N,K,fused,tiled": [[most rows, kernel, variant, splits], ...]} (what the tuner
    writes, or the path of its JSON file).  Entries are looked up by the exact widths; other widths keep the rules."""
    import json

    if isinstance(table, (str, bytes)) or hasattr(table, "__fspath__"):
        with open(table, encoding="utf-8") as fh:
            table = json.load(fh)
    for key, entries in table.items():
        if isinstance(key, str):
            n, k, fused, tiled = key.split(",")
            key = (int(n), int(k), fused.strip() in ("1", "True", "true"), tiled.strip() in ("1", "True", "true"))
        parsed = []
        for most_rows, kernel, variant, splits in entries:
            _need(kernel in PRODUCT_KERNELS, f"a product table names the kernel {kernel!r}; known: {', '.join(PRODUCT_KERNELS)}")
            parsed.append((int(most_rows), ProductChoice(kernel, tuple(variant), int(splits))))
        _PRODUCT_TABLE[key] = sorted(parsed, key=lambda e: e[0])


def clear_product_table() -> None:
    _PRODUCT_TABLE.clear()


def choose_product(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool, partials_ok: bool,
                   aligned: bool = True) -> ProductChoice:
    """The table's entry for these widths and this many rows if there is one (the tables were measured with operands
    on the 16-byte grid: others go by the rules), else `product_by_rules`."""
    on_grid = aligned and k % 8 == 0 and x_stride % 8 == 0
    entries = _PRODUCT_TABLE.get((n, k, fused, tiled)) if on_grid and _PRODUCT_TABLE else None
    if entries:
        for most_rows, choice in entries:
            if rows <= most_rows:
                return choice
    return product_by_rules(rows, n, k, x_stride, tiled=tiled, fused=fused, partials_ok=partials_ok, aligned=aligned)


def run_product(choice: ProductChoice, x, w, tiles, out_dtype, partials_ok: bool, fused: bool = False):
    """Launch what `choice` names.  Plain products come back as [M, N] in out_dtype, or, where the caller said
    partials_ok, possibly as a float32 stack [S, M, N]; fused ones as the activation [M, N/2]."""
    kernel = choice.kernel
    if fused:
        if kernel == "rows":
            return gemm_rows(x, w, x.dtype, EPI_SILU_MUL, variant=choice.variant[0] if choice.variant else None,
                             splits=1 if choice.variant else None, tiles=tiles)
        if kernel == "rounds":
            return gemm_rows_rounds(x, w, x.dtype, tiles=tiles, round_steps=choice.variant[0] if choice.variant else None)
        if kernel == "tiles":
            return gemm_tiles(x, tiles, w.shape[0], x.dtype, EPI_SILU_MUL, variant=choice.variant or None)
        return silu_mul_interleaved(gemm_bf16(x, w, x.dtype, tiles=tiles), 16)
    if kernel == "rows":
        out = gemm_rows(x, w, out_dtype, variant=choice.variant[0] if choice.variant else None,
                        splits=choice.splits or None, tiles=tiles)
    elif kernel == "stream":
        out = gemm_stream(x, w, out_dtype, variant=choice.variant[0] if choice.variant else _STREAM_VARIANT,
                          splits=choice.splits or None, workgroups=choice.variant[1] if len(choice.variant) > 1 else None,
                          tiles=tiles)
    elif kernel == "tiles_parts":
        out = gemm_tiles(x, tiles, w.shape[0], torch.float32, variant=choice.variant or _NARROW_TILES_VARIANT,
                         splits=choice.splits)
    elif kernel == "tiles":
        out = gemm_tiles(x, tiles, w.shape[0], out_dtype, variant=choice.variant or None)
    elif kernel == "library_parts":
        out = _library_mm_split_k(x, w, choice.splits)
        if out is None:
            out = _library_mm_f32out(x, w) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    else:
        out = _library_mm_f32out(x, w) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    # a large stack is added here by many workgroups; the consumer would add it with one workgroup a row
    if out.dim() == 3 and (not partials_ok or (kernel in ("rows", "stream") and out.numel() * 4 > _STREAM_PARTIAL_BYTES)):
        out = sum_partials(out, out_dtype)
    elif out.dim() == 2 and out.dtype != out_dtype:
        out = out.to(out_dtype)
    return out


def gate_up_act(x: torch.Tensor, w: torch.Tensor, tiles: torch.Tensor | None = None) -> torch.Tensor:
    """silu(x . gate^T) * (x . up^T) for w [2I, K] holding gate and up rows interleaved in blocks of 16: [M, I]."""
    _gpu(x, w)
    _rows(x, "x")
    rows, n, k = x.shape[0], w.shape[0], x.shape[1]
    if rows == 0:
        return torch.empty((0, n // 2), dtype=x.dtype, device=x.device)
    choice = choose_product(rows, n, k, x.stride(0), tiled=tiles is not None, fused=True, partials_ok=False,
                            aligned=x.data_ptr() % 16 == 0)
    return run_product(choice, x, w, tiles, x.dtype, False, fused=True)


PRODUCT_TABLE_ENV = "ARLE_AMD_PRODUCT_TABLE"   # the path of a table that is taken in when this module is loaded ("none": no table at all)
PRODUCT_TABLE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tables")


def load_shipped_product_tables() -> int:
    """The tables that come with the package (measured on an MI355X for the widths of Qwen3-4B, 8B and 32B)."""
    count = 0
    if os.path.isdir(PRODUCT_TABLE_DIR):
        for name in sorted(os.listdir(PRODUCT_TABLE_DIR)):
            if name.endswith(".json"):
                load_product_table(os.path.join(PRODUCT_TABLE_DIR, name))
                count += 1
    return count


if os.environ.get(PRODUCT_TABLE_ENV, "") != "none":
    load_shipped_product_tables()
    if os.environ.get(PRODUCT_TABLE_ENV):
        load_product_table(os.environ[PRODUCT_TABLE_ENV])
