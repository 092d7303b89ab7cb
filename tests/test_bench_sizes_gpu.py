"""The attention kernels and the engine at the sizes the benchmark runs (head_dim 128, groups of four, pages of 16,
thousands of keys, page pools of several GiB), against the plain implementation in float64.

The tiny configurations stop at a few hundred keys; these cases reach what only long contexts reach: more than 64
logical pages (the kernels keep 64 page ids in a register and refill it), the split factors that `decode_splits`
picks at 2,048 to 8,192 keys, both settings of the portions kernel that loads tiles straight into LDS, and page
addresses beyond 4 GiB."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
import replay
from arle_amd.config import Qwen3Config
from arle_amd.engine import Engine
from arle_amd.kernels import lib, ops
from arle_amd.weights import write_random_model
from tiny import ARCH, random_tokens, read_folder

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
BF = torch.bfloat16


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _g(seed):
    return torch.Generator().manual_seed(seed)


def _i32(vals):
    return torch.tensor(vals, dtype=torch.int32, device=DEV)


def _tables(lengths, P, total_pages, seed, top=False):
    """Block tables [requests, pages]: shuffled page ids, from anywhere in the pool or from its top."""
    need = [-(-n // P) for n in lengths]
    perm = torch.randperm(total_pages, generator=_g(seed))
    if top:
        perm = total_pages - 1 - torch.randperm(sum(need) + 7, generator=_g(seed))
    table = torch.zeros(len(lengths), max(need) + 1, dtype=torch.int32)
    at = 0
    for s, n in enumerate(need):
        table[s, :n] = perm[at:at + n].to(torch.int32)
        at += n
    return table


def _fill(k_pages, v_pages, table_row, k, v, P):
    """Keys [n, nkv, D] and values into the pages of one request (device tensors, any pool size)."""
    n = k.shape[0]
    pos = torch.arange(n, device=k_pages.device)
    page = table_row.to(k_pages.device).long()[pos // P]
    k_pages[page, :, pos % P] = k.to(k_pages.device)
    v_pages[page, :, :, pos % P] = v.to(k_pages.device)


def _last_rows(q_tail, k, v, nkv):
    """Attention of the last len(q_tail) rows of a sequence, in float64: row i of the tail sees the keys up to its
    own position.  The library routine, which plain.causal_attention reduces to (checked below at a small size)."""
    n, t = k.shape[0], q_tail.shape[0]
    G = q_tail.shape[1] // nkv
    kk = k.double().repeat_interleave(G, dim=1).transpose(0, 1)          # [nq, n, D]
    vv = v.double().repeat_interleave(G, dim=1).transpose(0, 1)
    mask = torch.arange(n)[None, :] <= (n - t + torch.arange(t))[:, None]
    out = F.scaled_dot_product_attention(q_tail.double().transpose(0, 1), kk, vv, attn_mask=mask,
                                         scale=1.0 / math.sqrt(q_tail.shape[-1]))
    return out.transpose(0, 1).reshape(t, -1)


def test_the_reference_of_this_file_is_the_plain_attention():
    q, k, v = (torch.randn(50, h, 32, generator=_g(1)) for h in (6, 2, 2))
    want = plain.causal_attention(q.double(), k.double(), v.double(), 2)
    assert torch.allclose(_last_rows(q[-7:], k, v, 2), want[-7:].reshape(7, -1), atol=1e-12)
    assert torch.allclose(_last_rows(q, k, v, 2), want.reshape(50, -1), atol=1e-12)


def _attention(q, table, k_pages, v_pages, segs, nq, nkv, P, **kw):
    """segs: [(cached, rows)] in the order of `table`'s rows; q [rows of all segments, nq*D] on the GPU."""
    row0 = [0]
    for _, n in segs:
        row0.append(row0[-1] + n)
    out = torch.full_like(q, float("nan"))
    ops.attn_paged_mfma(q, out, k_pages, v_pages, table.to(DEV), _i32(row0), _i32(list(range(len(segs)))),
                        _i32([c for c, _ in segs]), max_qlen=max(n for _, n in segs), min_qlen=min(n for _, n in segs),
                        max_kv_len=max(c + n for c, n in segs), num_q_heads=nq, num_kv_heads=nkv, head_dim=D,
                        page_size=P, scale=1.0 / math.sqrt(D), **kw)
    return out


def _random_case(segs, nq, nkv, P, seed, total_pages=None, top=False, stale=float("nan")):
    lengths = [c + n for c, n in segs]
    total = total_pages or sum(-(-n // P) for n in lengths) + 9
    table = _tables(lengths, P, total, seed, top=top)
    k_pages = torch.full((total, nkv, P, D), stale, dtype=BF, device=DEV)
    v_pages = torch.full((total, nkv, D, P), stale, dtype=BF, device=DEV)
    qs, wants = [], []
    for s, (cached, n) in enumerate(segs):
        g = _g(seed + 1 + s)
        q = torch.randn(n, nq, D, generator=g).to(BF)                     # the rows of the step only
        k, v = (torch.randn(cached + n, nkv, D, generator=g).to(BF) for _ in range(2))
        _fill(k_pages, v_pages, table[s], k, v, P)
        qs.append(q.reshape(n, nq * D))
        wants.append(_last_rows(q, k, v, nkv))
    return torch.cat(qs).to(DEV), table, k_pages, v_pages, torch.cat(wants)


@pytest.mark.parametrize("P", [16, 64])          # tiles that span pages, and tiles that lie in one page
def test_a_prompt_of_2048_tokens_at_the_benchmarks_shape_through_both_portion_kernels(P):
    """32 q heads over 8 kv heads, 2,048 rows: 128 logical pages of 16 (two refills of the page-id register).
    On a 256-unit GPU the launcher takes the kernel that loads tiles straight into LDS for this shape by itself;
    forced to either kernel the result is the plain one."""
    nq, nkv, segs = 32, 8, [(0, 2048)]
    q, table, k_pages, v_pages, want = _random_case(segs, nq, nkv, P, seed=300 + P)
    got = {}
    for variant in (-1, 0, 1):
        lib.function("arle_attn_prefill_variant")(variant)
        try:
            print(f"prefill 2048 rows, page {P}, kernel variant {variant}", flush=True)
            got[variant] = _attention(q, table, k_pages, v_pages, segs, nq, nkv, P)
        finally:
            lib.function("arle_attn_prefill_variant")(-1)
        assert torch.isfinite(got[variant]).all()
        assert _rel(got[variant].cpu(), want) < 8e-3, f"variant {variant}"
    if torch.cuda.get_device_properties(0).multi_processor_count <= 256:
        assert torch.equal(got[-1], got[1])      # 512 items for 512 workgroup slots: the launcher's own choice


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("P", [8, 16])
def test_long_prompts_and_a_portion_behind_a_long_prefix(variant, P):
    """A whole prompt of 2,100 keys and a portion of 900 rows behind 1,200 cached keys (its first tile already
    lies past the first 64 pages), beside a short portion and a decoded token; keys cut into parts or not."""
    nq, nkv = 8, 2
    segs = [(0, 2100), (1200, 900), (700, 1), (40, 70)]
    q, table, k_pages, v_pages, want = _random_case(segs, nq, nkv, P, seed=320 + P)
    for parts in (1, 4):
        lib.function("arle_attn_prefill_variant")(variant)
        try:
            print(f"long prompts, page {P}, kernel variant {variant}, parts {parts}", flush=True)
            got = _attention(q, table, k_pages, v_pages, segs, nq, nkv, P, portion_splits=parts, short_segments=1)
        finally:
            lib.function("arle_attn_prefill_variant")(-1)
        assert torch.isfinite(got).all()
        assert _rel(got.cpu(), want) < 8e-3


@pytest.mark.parametrize("batch,nq,nkv,around", [(8, 32, 8, 2048), (1, 32, 8, 2048), (64, 32, 8, 2048),
                                                   (8, 4, 1, 8192), (8, 32, 8, 8192), (3, 64, 8, 4100)])
def test_decoded_tokens_with_the_splits_the_engine_chooses_at_long_contexts(batch, nq, nkv, around):
    """Steps of single decoded tokens at the benchmark's contexts, split over the keys as `decode_splits` says
    (12, 32 and 2 splits at batch 8, 1 and 64 of the 4B shape; 64 splits for one kv head at 8,192 keys)."""
    P = 16
    contexts = [around - 1 - (37 * i) % 300 for i in range(batch)]
    contexts[0] = around - 1                       # the step's token is the `around`-th key
    if batch > 1:
        contexts[1] = around                       # one key past the page boundary
    segs = [(c, 1) for c in contexts]
    q, table, k_pages, v_pages, want = _random_case(segs, nq, nkv, P, seed=340 + batch + around)
    splits = ops.decode_splits(batch, nkv, around + 1)
    print(f"decode batch {batch} at {around} keys: {splits} splits", flush=True)
    assert splits == max(1, min(-(-768 // (batch * nkv)), 32 if around < 4096 else 64))
    got = _attention(q, table, k_pages, v_pages, segs, nq, nkv, P)          # splits=None: the engine's choice
    assert torch.isfinite(got).all()
    assert _rel(got.cpu(), want) < 8e-3
    forced = _attention(q, table, k_pages, v_pages, segs, nq, nkv, P, splits=splits)
    assert torch.equal(got, forced)


def test_a_far_key_among_8192_is_found_by_every_split():
    """One key near the start carries a score far above the rest: the row's output is that key's value, whatever
    split it falls into."""
    nq, nkv, P, n = 4, 1, 16, 8192
    g = _g(360)
    q = (torch.randn(n, nq, D, generator=g) * 0.05).to(BF)
    k = (torch.randn(n, nkv, D, generator=g) * 0.05).to(BF)
    v = torch.randn(n, nkv, D, generator=g).to(BF)
    far = 1037
    k[far, 0] = (q[n - 1, 2].float() * 600.0).to(BF)
    table = _tables([n], P, n // P + 5, 361)
    k_pages = torch.zeros(n // P + 5, nkv, P, D, dtype=BF, device=DEV)
    v_pages = torch.zeros(n // P + 5, nkv, D, P, dtype=BF, device=DEV)
    _fill(k_pages, v_pages, table[0], k, v, P)
    for splits in (None, 1, 7, 64):
        got = _attention(q[n - 1:].reshape(1, -1).to(DEV), table, k_pages, v_pages, [(n - 1, 1)], nq, nkv, P,
                         splits=splits)
        assert torch.allclose(got.cpu().reshape(nq, D)[2].float(), v[far, 0].float(), atol=2e-2), splits


def test_pages_beyond_4_gib_are_written_and_read():
    """A pool whose key buffer and value buffer each take 4.6 GB, with the requests' pages at its top: page
    offsets beyond 2^31 elements and 2^32 bytes, through the kernel that writes the cache (per-head norm, rotation,
    page write) and through every attention kernel that reads it."""
    nq, nkv, P, eps, theta = 32, 8, 16, 1e-6, 1e6
    pages = 140000                                             # x 8 heads x 16 slots x 128 x 2 bytes = 4.59 GB
    assert pages * nkv * P * D * 2 > 4.5e9
    segs = [(0, 300), (1100, 1), (90, 40)]
    lengths = [c + n for c, n in segs]
    table = _tables(lengths, P, pages, seed=380, top=True)
    assert int(table[table > 0].min()) * nkv * P * D > 2 ** 31        # every page lies beyond 2^31 elements
    print("allocating a pool of 2 x 4.6 GB", flush=True)
    k_pages = torch.empty((pages, nkv, P, D), dtype=BF, device=DEV)
    v_pages = torch.empty((pages, nkv, D, P), dtype=BF, device=DEV)
    top = slice(pages - 200, pages)
    k_pages[top] = float("nan")
    v_pages[top] = float("nan")
    cos, sin = plain.rope_cos_sin(range(max(lengths)), D, theta)
    qw = (1.0 + 0.2 * torch.randn(D, generator=_g(381))).to(BF)
    kw = (1.0 + 0.2 * torch.randn(D, generator=_g(382))).to(BF)
    Q, KV = nq * D, nkv * D
    raw = [torch.randn(n, (nq + 2 * nkv) * D, generator=_g(383 + s)).to(BF) for s, n in enumerate(lengths)]
    # the write kernel, request by request (every token of a request in one call), as a prefill would
    prepared = []
    for s, n in enumerate(lengths):
        x = raw[s].to(DEV).clone()
        print(f"writing {n} tokens into pages near {int(table[s, 0])}", flush=True)
        ops.qk_prep(x[:, :Q], x[:, Q:Q + KV], x[:, Q + KV:], num_q_heads=nq, num_kv_heads=nkv, head_dim=D, eps=eps,
                    q_weight=qw.to(DEV), k_weight=kw.to(DEV), cos=cos.to(DEV), sin=sin.to(DEV), rotary_dim=D,
                    positions=_i32(list(range(n))), slot_of_token=_i32([s] * n), block_table=table.to(DEV),
                    k_pages=k_pages, v_pages=v_pages, page_size=P)
        prepared.append(x[:, :Q].clone())
    torch.cuda.synchronize()
    wants, qs = [], []
    for s, (cached, rows) in enumerate(segs):
        n = lengths[s]
        x = raw[s].double()
        c, sn = plain.rope_cos_sin(range(n), D, theta, dtype=torch.float64)
        q = plain.prepare_heads(x[:, :Q].reshape(n, nq, D), qw.double(), eps, c, sn)
        k = plain.prepare_heads(x[:, Q:Q + KV].reshape(n, nkv, D), kw.double(), eps, c, sn)
        v = x[:, Q + KV:].reshape(n, nkv, D)
        # what landed in the pages is what the plain preparation gives
        pos = torch.arange(n)
        page = table[s].long()[pos // P]
        got_k = k_pages[page.to(DEV), :, (pos % P).to(DEV)].cpu()
        got_v = v_pages[page.to(DEV), :, :, (pos % P).to(DEV)].cpu()
        assert _rel(got_k, k) < 6e-3 and torch.equal(got_v.double(), v)
        assert _rel(prepared[s].cpu().reshape(n, nq, D), q) < 6e-3
        qs.append(prepared[s][cached:])
        wants.append(_last_rows(prepared[s][cached:].cpu().reshape(rows, nq, D), got_k, got_v, nkv))
    q_all, want = torch.cat(qs), torch.cat(wants)
    for variant in (0, 1):
        lib.function("arle_attn_prefill_variant")(variant)
        try:
            print(f"attention over pages beyond 4 GiB, portions kernel variant {variant}", flush=True)
            got = _attention(q_all, table, k_pages, v_pages, segs, nq, nkv, P, short_segments=1)
        finally:
            lib.function("arle_attn_prefill_variant")(-1)
        assert torch.isfinite(got).all()
        assert _rel(got.cpu(), want) < 8e-3
    # the decoded token alone, split over the keys, and through the fixed-order kernel
    one = [segs[1]]
    got = _attention(qs[1], table[1:2], k_pages, v_pages, one, nq, nkv, P)
    assert _rel(got.cpu(), wants[1]) < 8e-3
    out = torch.empty_like(qs[1])
    ops.attn_paged_simt(qs[1], out, k_pages, v_pages, table[1:2].contiguous().to(DEV), _i32([1100]), _i32([0]),
                        num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D))
    assert _rel(out.cpu(), wants[1]) < 8e-3


# ---- the engine with several layers at the widths of Qwen3-4B ------------------------------------------------------

WIDTHS4 = dict(num_hidden_layers=4, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6,
               tie_word_embeddings=True, max_position_embeddings=4096)


@pytest.fixture(scope="module")
def four_layers(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("widths4") / "model")
    print("writing four layers at the widths of Qwen3-4B", flush=True)
    write_random_model(d, ARCH, Qwen3Config.from_dict(WIDTHS4), seed=23, std=0.02, norm_std=0.0)
    cfg, weights = read_folder(d)
    requests = {"a": random_tokens(150, WIDTHS4["vocab_size"], 7), "b": random_tokens(61, WIDTHS4["vocab_size"], 8),
                "c": random_tokens(38, WIDTHS4["vocab_size"], 9)}
    print("plain implementation of three requests", flush=True)
    reference = {rid: replay.plain_logits(cfg, weights, toks).float() for rid, toks in requests.items()}
    return d, requests, reference


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_four_layers_at_the_widths_of_qwen3_4b(four_layers, dtype, tol):
    d, requests, reference = four_layers
    eng = Engine.from_folder(d, dtype=dtype, page_size=16, max_tokens=512, max_slots=4)

    def check(got, what):
        for (rid, p), row in got.items():
            ref = reference[rid].double()
            err = float((row.double() - ref[p]).abs().max()) / float(ref.abs().max())
            assert err <= tol, f"{what}/{dtype}: request {rid} position {p}: relative error {err:.3e} > {tol:.1e}"

    print(f"{dtype}: whole prompt of 150 tokens, then its last 32 one by one", flush=True)
    check(replay.run_steps(eng, replay.whole("a", requests["a"])), "whole")
    check(replay.run_steps(eng, replay.prefill_then_decode("a", requests["a"], tail=32)), "prefill then decode")
    print(f"{dtype}: three requests mixed", flush=True)
    got = replay.run_steps(eng, replay.mixed(requests, max_live=3, seed=5, max_portion=40))
    assert len(got) == sum(len(t) for t in requests.values())
    check(got, "mixed")


def test_bench_sorts_the_kernels_of_real_steps_into_every_part_of_a_layer():
    """`bench.py --parts-only` on two layers of the benchmark's shape: the kernel names that the profiler reports
    today are sorted into all parts of a prefill and of a decode step (a renamed kernel or a changed list of
    template arguments would leave a part empty, which the program refuses)."""
    import json
    import os
    import subprocess
    import sys

    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--parts-only", "--layers", "2", "--batch", "2"],
                         capture_output=True, text=True, timeout=400, cwd=root)
    lines = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
    assert res.returncode == 0 and lines, res.stderr[-2000:]
    line = json.loads(lines[-1])
    for step in ("prefill_parts_us", "decode_parts_us"):
        for part in ("qkv", "o", "gate_up", "down", "head", "attention", "qk_prep", "norm"):
            if (step, part) == ("decode_parts_us", "qk_prep"):
                continue     # single decoded tokens are prepared inside the attention's kernel
            assert line[step][part] > 0, (step, part, line[step])
    assert line["prefill_parts_us"]["gate_up"] > line["prefill_parts_us"]["qkv"] > line["prefill_parts_us"]["head"] / 100
