"""The decode attention entry point that allocates nothing (`arle_attn_decode_static`), called through
ctypes, against the existing entry point (`arle_attn_paged_mfma`, which takes its split-KV workspace from the
caller): two calls in a row, the second with a smaller input, so that what the first call left in the
library's fixed scratch array must not show.  The file name makes pytest collect it last."""
import ctypes
import math

import pytest
import torch

import plain_qwen3 as plain
from arle_amd.kernels import lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

_p, _i, _ll, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_float


def _entry():
    cdll = lib.library("attention_mfma")      # a ctypes.CDLL of the built library
    fn = cdll.arle_attn_decode_static
    fn.argtypes = [_p, _ll, _p, _ll, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p]
    fn.restype = _i
    err = cdll.arle_attn_decode_static_error
    err.argtypes = []
    err.restype = ctypes.c_char_p
    return fn, err


def _case(nq, nkv, D, P, contexts, seed, qlen=1):
    """Requests that hold `contexts[i]` tokens and bring `qlen` more; pages handed out in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    dt = torch.bfloat16
    lengths = [c + qlen for c in contexts]
    pages_per = [-(-n // P) for n in lengths]
    total = sum(pages_per) + 5
    perm = iter(torch.randperm(total, generator=g).tolist())
    table = torch.zeros(len(lengths), max(pages_per) + 1, dtype=torch.int32)
    k_pages = torch.full((total, nkv, P, D), float("nan"), dtype=dt)     # stale slots hold NaN
    v_pages = torch.full((total, nkv, D, P), float("nan"), dtype=dt)
    qs, wants = [], []
    for s, n in enumerate(lengths):
        for i in range(pages_per[s]):
            table[s, i] = next(perm)
        q, k, v = (torch.randn(n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
        for pos in range(n):
            page = int(table[s, pos // P])
            k_pages[page, :, pos % P] = k[pos]
            v_pages[page, :, :, pos % P] = v[pos]
        qs.append(q[contexts[s]:].reshape(qlen, nq * D))
        wants.append(plain.causal_attention(q.double(), k.double(), v.double(), nkv)[contexts[s]:].reshape(qlen, -1))
    i32 = lambda vals: torch.tensor(vals, dtype=torch.int32, device=DEV)
    return dict(q=torch.cat(qs).to(DEV), k=k_pages.to(DEV), v=v_pages.to(DEV), table=table.to(DEV),
                row0=i32([qlen * s for s in range(len(lengths) + 1)]), slot=i32(list(range(len(lengths)))),
                start=i32(contexts), want=torch.cat(wants), segments=len(lengths), qlen=qlen,
                max_kv=max(lengths), nq=nq, nkv=nkv, D=D, P=P)


def _run_both(c, splits):
    fn, err = _entry()
    scale = 1.0 / math.sqrt(c["D"])
    ref = torch.full_like(c["q"], float("nan"))
    ops.attn_paged_mfma(c["q"], ref, c["k"], c["v"], c["table"], c["row0"], c["slot"], c["start"],
                        max_qlen=c["qlen"], min_qlen=c["qlen"], max_kv_len=c["max_kv"], num_q_heads=c["nq"],
                        num_kv_heads=c["nkv"], head_dim=c["D"], page_size=c["P"], scale=scale, splits=splits)
    out = torch.full_like(c["q"], float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = fn(c["q"].data_ptr(), c["q"].stride(0), out.data_ptr(), out.stride(0), c["k"].data_ptr(), c["v"].data_ptr(),
            c["table"].data_ptr(), c["table"].shape[1], c["row0"].data_ptr(), c["slot"].data_ptr(),
            c["start"].data_ptr(), c["segments"], c["qlen"], c["nq"], c["nkv"], c["D"], c["P"], scale, 0, splits,
            torch.cuda.current_stream().cuda_stream)
    assert rc == 0, err().decode()
    torch.cuda.synchronize()
    return out, ref, free_before, torch.cuda.mem_get_info()[0]


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def test_two_calls_in_a_row_equal_the_entry_point_with_a_workspace():
    print("no-alloc decode attention: first call 6 segments of 32/8 heads x 128, 5 splits", flush=True)
    big = _case(32, 8, 128, 16, [299, 0, 31, 640, 95, 1023], seed=5)
    out, ref, _, _ = _run_both(big, splits=5)
    assert torch.isfinite(out).all()
    assert torch.equal(out, ref)
    assert _rel(out.cpu(), big["want"]) < 8e-3
    print("no-alloc decode attention: second call 3 segments of 4/2 heads x 64, two tokens each, 3 splits", flush=True)
    small = _case(4, 2, 64, 8, [130, 7, 64], seed=6, qlen=2)
    out, ref, free_before, free_after = _run_both(small, splits=3)
    assert torch.isfinite(out).all()
    assert torch.equal(out, ref)
    assert _rel(out.cpu(), small["want"]) < 8e-3
    assert free_after == free_before        # the device's free memory did not move: nothing was allocated
    # and once more without a split: no scratch is used at all
    out, ref, _, _ = _run_both(small, splits=1)
    assert torch.equal(out, ref)


def test_sizes_beyond_the_fixed_array_are_refused_with_a_reason():
    fn, err = _entry()
    c = _case(4, 2, 64, 8, [20], seed=7)
    out = torch.zeros_like(c["q"])
    args = lambda segments, qlen, nq, nkv, D, splits: (
        c["q"].data_ptr(), c["q"].stride(0), out.data_ptr(), out.stride(0), c["k"].data_ptr(), c["v"].data_ptr(),
        c["table"].data_ptr(), c["table"].shape[1], c["row0"].data_ptr(), c["slot"].data_ptr(), c["start"].data_ptr(),
        segments, qlen, nq, nkv, D, 8, 0.125, 0, splits, torch.cuda.current_stream().cuda_stream)
    # refused before anything is launched: 512 segments x 32 heads x 64 splits x 128 floats is far beyond 2 Mi floats
    assert fn(*args(512, 1, 32, 8, 128, 64)) != 0
    assert "partial outputs" in err().decode() and "maximum" in err().decode()
    assert fn(*args(1, 9, 4, 2, 64, 2)) != 0          # 9 tokens x 2 heads a group: more than one row tile
    assert "rows of a segment" in err().decode()
    assert fn(*args(1, 1, 4, 2, 24, 2)) != 0          # head_dim no multiple of 16
    assert "head_dim" in err().decode()
    assert fn(*args(1, 1, 4, 2, 64, 2)) == 0 and err().decode() == ""
    torch.cuda.synchronize()
