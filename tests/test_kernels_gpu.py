"""Each HIP kernel alone against its plain reference, at sizes other than the engine's."""
import math

import pytest
import torch

import plain_qwen3 as plain
from arle_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True, scope="module")
def rules_only():
    """This file pins the kernels and the rules that choose between them; the measured tables that come with the
    package (which take the rules' place at the widths they were measured for) are put aside meanwhile."""
    saved = dict(ops._PRODUCT_TABLE)
    ops.clear_product_table()
    yield
    ops._PRODUCT_TABLE.update(saved)


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _g(seed):
    return torch.Generator().manual_seed(seed)


def test_embed_gather():
    table = torch.randn(333, 88, generator=_g(0))
    ids = torch.tensor([0, 332, 5, 5, 17], dtype=torch.int32)
    for dt in (torch.float32, torch.bfloat16):
        out = ops.embed_gather(table.to(dt).to(DEV), ids.to(DEV))
        assert out.dtype == torch.float32
        assert torch.equal(out.cpu(), table.to(dt).float()[ids.long()])


@pytest.mark.parametrize("width", [4, 96, 260, 2044, 2560, 4096, 5120, 6004, 8192, 8196, 9001])
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
def test_rmsnorm_and_fused_add(width, act, wdt):
    x = torch.randn(7, width, generator=_g(1)) * 3.0
    w = (1.0 + 0.3 * torch.randn(width, generator=_g(2))).to(wdt)
    eps = 1e-5
    want = plain.rms_norm(x.double(), w.double(), eps)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, act)
    tol = 1e-6 if act == torch.float32 else 5e-3
    assert got.dtype == act and _rel(got.cpu(), want) < tol
    # rows picked by index
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, act, rows=rows.to(DEV))
    assert _rel(got.cpu(), want[rows.long()]) < tol
    # residual add fused in
    delta = (torch.randn(7, width, generator=_g(3))).to(act)
    res = x.clone().to(DEV)
    got = ops.add_rmsnorm(res, delta.to(DEV), w.to(DEV), eps, act)
    total = x.double() + delta.double()
    assert _rel(res.cpu(), total) < 1e-6  # the residual stream itself stays 32-bit
    assert _rel(got.cpu(), plain.rms_norm(total, w.double(), eps)) < tol
    # with rows the residual is left alone
    res2 = x.clone().to(DEV)
    got = ops.add_rmsnorm(res2, delta.to(DEV), w.to(DEV), eps, act, rows=rows.to(DEV))
    assert torch.equal(res2.cpu(), x)
    assert _rel(got.cpu(), plain.rms_norm(total, w.double(), eps)[rows.long()]) < tol


def test_rmsnorm_vector_of_the_reference_and_zero_weight():
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    got = ops.rmsnorm(x.to(DEV), torch.ones(4, device=DEV), 1e-6, torch.float32).cpu()
    assert torch.allclose(got, x / math.sqrt(7.5 + 1e-6), atol=1e-7)
    got = ops.rmsnorm(x.to(DEV), torch.zeros(4, device=DEV), 1e-6, torch.float32).cpu()
    assert torch.count_nonzero(got) == 0  # plain weight, not (1 + w)


@pytest.mark.parametrize("M,N,K", [(1, 2, 3), (7, 333, 88), (70, 96, 224), (130, 64, 17), (64, 129, 2560)])
def test_gemm_f32(M, N, K):
    a = torch.randn(M, K, generator=_g(4))
    w = torch.randn(N, K, generator=_g(5))
    got = ops.gemm_f32(a.to(DEV), w.to(DEV)).cpu()
    assert _rel(got, a.double() @ w.double().T) < 2e-6
    if (M, N, K) == (1, 2, 3):
        a = torch.tensor([[1.0, 2.0, 3.0]])
        w = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
        assert ops.gemm_f32(a.to(DEV), w.to(DEV)).cpu().tolist() == [[14.0, 32.0]]


def test_gemm_f32_rows_do_not_depend_on_the_batch():
    a = torch.randn(77, 200, generator=_g(6)).to(DEV)
    w = torch.randn(150, 200, generator=_g(7)).to(DEV)
    full = ops.gemm_f32(a, w)
    for r in (0, 13, 76):
        assert torch.equal(ops.gemm_f32(a[r:r + 1], w)[0], full[r])
    assert torch.equal(ops.gemm_f32(a[10:31], w), full[10:31])


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (5, 333, 88), (64, 256, 2560), (300, 224, 96)])
def test_gemm_bf16(M, N, K):
    a = torch.randn(M, K, generator=_g(8)).bfloat16()
    w = (torch.randn(N, K, generator=_g(9)) * 0.1).bfloat16()
    want = a.double() @ w.double().T
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.float32).cpu()
    assert got.dtype == torch.float32 and _rel(got, want) < 1e-3
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.bfloat16).cpu()
    assert got.dtype == torch.bfloat16 and _rel(got, want) < 8e-3


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [136, 132, 9728])      # eight columns a thread in bfloat16, or one by one
def test_silu_mul(dt, width):
    gu = (torch.randn(5, 2 * width, generator=_g(10)) * 3.0).to(dt)
    g, u = gu[:, :width].double(), gu[:, width:].double()
    want = plain.silu(g) * u
    d = gu.to(DEV)
    got = ops.silu_mul(d[:, :width], d[:, width:]).cpu()
    assert _rel(got, want) < (1e-6 if dt == torch.float32 else 5e-3)
    if width % 16 == 0:
        inter = torch.stack([gu[:, :width].view(5, -1, 16), gu[:, width:].view(5, -1, 16)], dim=2).reshape(5, 2 * width)
        got = ops.silu_mul_interleaved(inter.contiguous().to(DEV), 16).cpu()
        assert _rel(got, want) < (1e-6 if dt == torch.float32 else 5e-3)
    z = torch.zeros(2, 8, dtype=dt, device=DEV)
    assert torch.count_nonzero(ops.silu_mul(z, torch.ones_like(z))) == 0


def _paged_setup(lengths, nkv, D, P, dtype, seed, shuffle=True):
    """Block tables with shuffled physical pages for requests of the given lengths."""
    g = _g(seed)
    slots = len(lengths)
    pages_per = [-(-n // P) for n in lengths]
    total = sum(pages_per) + 3
    perm = torch.randperm(total, generator=g).tolist() if shuffle else list(range(total))
    table = torch.zeros(slots, max(pages_per) + 1, dtype=torch.int32)
    it = iter(perm)
    for s, n in enumerate(pages_per):
        for i in range(n):
            table[s, i] = next(it)
    k_pages = torch.zeros(total, nkv, P, D, dtype=dtype)
    v_pages = torch.zeros(total, nkv, D, P, dtype=dtype)   # values are d-major inside a page
    return table, k_pages, v_pages


@pytest.mark.parametrize("nq,nkv,D,P", [(4, 2, 128, 16), (2, 1, 64, 16), (3, 3, 128, 32), (2, 2, 64, 64),
                                         (2, 1, 256, 16), (2, 2, 128, 8)])
def test_qk_prep_runs_of_positions_fill_value_pages(nq, nkv, D, P):
    """Portions of prompts: runs of consecutive positions that start on and off a multiple of 16, one after
    the other in the packed rows, with single decoded tokens between them.  Every value lands in its slot
    and no other slot of the cache changes."""
    dt, eps, theta, rot = torch.bfloat16, 1e-6, 1e4, D
    runs = [(0, 16, 48), (1, 5, 37), (2, 70, 1), (3, 32, 32), (1, 42, 1), (0, 64, 19)]   # (slot, start, count)
    lengths = [83, 43, 71, 64]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 40)
    positions = torch.tensor([s + i for _, s, n in runs for i in range(n)], dtype=torch.int32)
    slots = torch.tensor([r for r, _, n in runs for _ in range(n)], dtype=torch.int32)
    T = positions.numel()
    qkv = torch.randn(T, (nq + 2 * nkv) * D, generator=_g(41)).to(dt)
    qw = (1.0 + 0.2 * torch.randn(D, generator=_g(42))).to(dt)
    kw = (1.0 + 0.2 * torch.randn(D, generator=_g(43))).to(dt)
    cos, sin = plain.rope_cos_sin(range(96), rot, theta)
    d_qkv = qkv.to(DEV)
    Q, KV = nq * D, nkv * D
    dk, dv = k_pages.to(DEV), v_pages.to(DEV)
    ops.qk_prep(d_qkv[:, :Q], d_qkv[:, Q:Q + KV], d_qkv[:, Q + KV:], num_q_heads=nq, num_kv_heads=nkv,
                head_dim=D, eps=eps, q_weight=qw.to(DEV), k_weight=kw.to(DEV), cos=cos.to(DEV), sin=sin.to(DEV),
                rotary_dim=rot, positions=positions.to(DEV), slot_of_token=slots.to(DEV),
                block_table=table.to(DEV), k_pages=dk, v_pages=dv, page_size=P)
    x = qkv.double()
    c, s = plain.rope_cos_sin(positions.tolist(), rot, theta, dtype=torch.float64)
    q = plain.apply_rope(plain.qk_norm(x[:, :Q].reshape(T, nq, D), qw.double(), eps), c, s)
    k = plain.apply_rope(plain.qk_norm(x[:, Q:Q + KV].reshape(T, nkv, D), kw.double(), eps), c, s)
    v = x[:, Q + KV:].reshape(T, nkv, D)
    assert _rel(d_qkv[:, :Q].cpu().reshape(T, nq, D), q) < 6e-3
    dk, dv = dk.cpu(), dv.cpu()
    want_v = torch.zeros_like(dv)
    written = torch.zeros(dk.shape[0], P, dtype=torch.bool)
    for t in range(T):
        page, at = int(table[slots[t], positions[t] // P]), int(positions[t]) % P
        assert _rel(dk[page, :, at], k[t]) < 6e-3
        want_v[page, :, :, at] = v[t].to(dt)
        written[page, at] = True
    assert torch.equal(dv, want_v)
    assert torch.count_nonzero(dk.transpose(1, 2)[~written]) == 0


@pytest.mark.parametrize("nq,nkv,D,rot", [(3, 1, 48, 48), (4, 2, 16, 16), (8, 2, 128, 128), (2, 2, 64, 32),
                                           (5, 5, 32, 0), (2, 1, 256, 64), (3, 3, 64, 0), (32, 8, 128, 128)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_qk_prep_norm_rope_and_cache_write(nq, nkv, D, rot, dt):
    P, eps, theta = 8, 1e-5, 1e4
    lengths = [11, 5]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 20)
    positions = torch.tensor([3, 4, 5, 10, 0, 4], dtype=torch.int32)   # rows of two requests
    slots = torch.tensor([0, 0, 0, 0, 1, 1], dtype=torch.int32)
    T = positions.numel()
    qkv = torch.randn(T, (nq + 2 * nkv) * D, generator=_g(21)).to(dt)
    qw = (1.0 + 0.2 * torch.randn(D, generator=_g(22))).to(dt)
    kw = (1.0 + 0.2 * torch.randn(D, generator=_g(23))).to(dt)
    cos = sin = None
    if rot:
        cos, sin = plain.rope_cos_sin(range(16), rot, theta)
    d_qkv = qkv.to(DEV)
    Q, KV = nq * D, nkv * D
    dk, dv = k_pages.to(DEV), v_pages.to(DEV)
    ops.qk_prep(d_qkv[:, :Q], d_qkv[:, Q:Q + KV], d_qkv[:, Q + KV:], num_q_heads=nq, num_kv_heads=nkv,
                head_dim=D, eps=eps, q_weight=qw.to(DEV), k_weight=kw.to(DEV),
                cos=None if cos is None else cos.to(DEV), sin=None if sin is None else sin.to(DEV),
                rotary_dim=rot, positions=positions.to(DEV), slot_of_token=slots.to(DEV),
                block_table=table.to(DEV), k_pages=dk, v_pages=dv, page_size=P)
    # plain: norm per head, rotate the first `rot` dims, at each row's own position
    x = qkv.double()
    q = plain.qk_norm(x[:, :Q].reshape(T, nq, D), qw.double(), eps)
    k = plain.qk_norm(x[:, Q:Q + KV].reshape(T, nkv, D), kw.double(), eps)
    v = x[:, Q + KV:].reshape(T, nkv, D)
    if rot:
        c, s = plain.rope_cos_sin(positions.tolist(), rot, theta, dtype=torch.float64)
        q = torch.cat([plain.apply_rope(q[..., :rot], c, s), q[..., rot:]], -1)
        k = torch.cat([plain.apply_rope(k[..., :rot], c, s), k[..., rot:]], -1)
    tol = 2e-6 if dt == torch.float32 else 6e-3
    assert _rel(d_qkv[:, :Q].cpu().reshape(T, nq, D), q) < tol
    dk, dv = dk.cpu(), dv.cpu()
    for t in range(T):
        page = int(table[slots[t], positions[t] // P])
        assert _rel(dk[page, :, positions[t] % P], k[t]) < tol
        assert torch.equal(dv[page, :, :, positions[t] % P].double(), v[t])
    # nothing else in the cache was touched
    written = torch.zeros(dk.shape[0], P, dtype=torch.bool)
    for t in range(T):
        written[int(table[slots[t], positions[t] // P]), positions[t] % P] = True
    assert torch.count_nonzero(dk.transpose(1, 2)[~written]) == 0

    # the same projections as a stack of three float32 partial products: same q, same cache
    stack = torch.randn(3, T, (nq + 2 * nkv) * D, generator=_g(24))
    stack[2] = qkv.float() - stack[0] - stack[1]
    x = stack.double().sum(0)
    q = plain.qk_norm(x[:, :Q].reshape(T, nq, D), qw.double(), eps)
    k = plain.qk_norm(x[:, Q:Q + KV].reshape(T, nkv, D), kw.double(), eps)
    v = x[:, Q + KV:].reshape(T, nkv, D)
    if rot:
        q = torch.cat([plain.apply_rope(q[..., :rot], c, s), q[..., rot:]], -1)
        k = torch.cat([plain.apply_rope(k[..., :rot], c, s), k[..., rot:]], -1)
    dq = torch.zeros(T, Q, dtype=dt, device=DEV)
    dk, dv = k_pages.to(DEV), v_pages.to(DEV)
    ops.qk_prep(dq, None, None, num_q_heads=nq, num_kv_heads=nkv, head_dim=D, eps=eps, q_weight=qw.to(DEV),
                k_weight=kw.to(DEV), cos=None if cos is None else cos.to(DEV), sin=None if sin is None else sin.to(DEV),
                rotary_dim=rot, positions=positions.to(DEV), slot_of_token=slots.to(DEV),
                block_table=table.to(DEV), k_pages=dk, v_pages=dv, page_size=P, parts=stack.to(DEV))
    assert _rel(dq.cpu().reshape(T, nq, D), q) < tol
    dk, dv = dk.cpu(), dv.cpu()
    for t in range(T):
        page = int(table[slots[t], positions[t] // P])
        assert _rel(dk[page, :, positions[t] % P], k[t]) < tol
        assert _rel(dv[page, :, :, positions[t] % P], v[t]) < tol
    # only q (a layer that reads another layer's cache)
    dq2 = torch.zeros(T, Q, dtype=dt, device=DEV)
    ops.qk_prep(dq2, None, None, num_q_heads=nq, num_kv_heads=0, head_dim=D, eps=eps, q_weight=qw.to(DEV),
                k_weight=kw.to(DEV), cos=None if cos is None else cos.to(DEV), sin=None if sin is None else sin.to(DEV),
                rotary_dim=rot, positions=positions.to(DEV), parts=stack[:, :, :Q].contiguous().to(DEV))
    assert torch.equal(dq2, dq)


def _fill_cache(table, k_pages, v_pages, slot, k, v, P):
    for pos in range(k.shape[0]):
        page = int(table[slot, pos // P])
        k_pages[page, :, pos % P] = k[pos]
        v_pages[page, :, :, pos % P] = v[pos]


@pytest.mark.parametrize("nq,nkv,D,P", [(3, 1, 48, 16), (4, 2, 16, 4), (8, 2, 128, 16), (6, 2, 32, 8),
                                         (2, 1, 256, 32)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_simt_against_plain(nq, nkv, D, P, dt, window):
    lengths = [150, 70, 1]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 30)
    qs, ks, vs, pos, slots = [], [], [], [], []
    for s, n in enumerate(lengths):
        g = _g(31 + s)
        q = torch.randn(n, nq, D, generator=g).to(dt)
        k = torch.randn(n, nkv, D, generator=g).to(dt)
        v = torch.randn(n, nkv, D, generator=g).to(dt)
        _fill_cache(table, k_pages, v_pages, s, k, v, P)
        qs.append(q), ks.append(k), vs.append(v)
        pos += list(range(n))
        slots += [s] * n
    q_all = torch.cat(qs).reshape(-1, nq * D)
    out = torch.empty_like(q_all).to(DEV)
    ops.attn_paged_simt(q_all.to(DEV), out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV),
                        torch.tensor(pos, dtype=torch.int32, device=DEV),
                        torch.tensor(slots, dtype=torch.int32, device=DEV), num_q_heads=nq,
                        num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D), window=window)
    want = torch.cat([plain.causal_attention(q.double(), k.double(), v.double(), nkv,
                                             window=window or None).reshape(-1, nq * D)
                      for q, k, v in zip(qs, ks, vs)])
    assert _rel(out.cpu(), want) < (3e-6 if dt == torch.float32 else 6e-3)


def test_attention_finds_a_far_key_among_hundreds():
    """One early key is made to stand out for the last query; its value must dominate."""
    nq, nkv, D, P, n = 4, 2, 64, 16, 700
    table, k_pages, v_pages = _paged_setup([n], nkv, D, P, torch.float32, 40)
    g = _g(41)
    q = torch.randn(n, nq, D, generator=g) * 0.1
    k = torch.randn(n, nkv, D, generator=g) * 0.1
    v = torch.randn(n, nkv, D, generator=g)
    far = 3
    k[far, 0] = q[n - 1, 1] * 400.0   # head 1 reads kv head 0
    _fill_cache(table, k_pages, v_pages, 0, k, v, P)
    out = torch.empty(n, nq * D, device=DEV)
    ops.attn_paged_simt(q.reshape(n, -1).to(DEV), out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV),
                        torch.arange(n, dtype=torch.int32, device=DEV),
                        torch.zeros(n, dtype=torch.int32, device=DEV), num_q_heads=nq, num_kv_heads=nkv,
                        head_dim=D, page_size=P, scale=1.0 / math.sqrt(D))
    got = out.cpu().reshape(n, nq, D)
    assert torch.allclose(got[n - 1, 1], v[far, 0], atol=1e-3)
    want = plain.causal_attention(q.double(), k.double(), v.double(), nkv)
    assert _rel(got, want) < 3e-6


def test_argmax_rows_first_maximum_wins():
    x = torch.tensor([[1.0, 9.0, 3.0, 8.0], [2.0, 7.0, 7.0, 1.0]])
    assert ops.argmax_rows(x.to(DEV)).tolist() == [1, 1]   # infer/src/ops/tests.rs:81-87
    big = torch.randn(5, 151936, generator=_g(50))
    big[2, 150000] = 50.0
    big[3, 7] = 60.0
    big[3, 100000] = 60.0
    assert ops.argmax_rows(big.to(DEV)).tolist() == big.argmax(-1).tolist()


@pytest.mark.parametrize("rows,vocab", [(1, 151936), (3, 151937), (8, 32003), (64, 50257), (2, 8192), (7, 8191)])
def test_argmax_rows_cut_into_chunks(rows, vocab):
    """Rows long enough to be cut into chunks, with widths that leave the rows unaligned: the maximum at the
    last place, at the first, twice (the first one wins, also from another chunk), and a row of NaNs."""
    x = torch.randn(rows, vocab, generator=_g(51))
    x[0, vocab - 1] = 40.0
    want = x.argmax(-1).tolist()
    if rows > 1:
        x[1, 0] = 41.0
        want[1] = 0
    if rows > 2:
        x[2, vocab // 2 + 1] = 42.0
        x[2, vocab - 3] = 42.0
        want[2] = vocab // 2 + 1
    if rows > 3:
        x[3] = float("nan")
        want[3] = 0
    if rows > 4:
        x[4] = -5.0                                   # all equal: index 0
        want[4] = 0
    assert ops.argmax_rows(x.to(DEV)).tolist() == want


def _sample(logits, temperature, u, top_k=-1, top_p=1.0, min_p=0.0):
    rows = logits.shape[0]
    f = lambda v: torch.full((rows,), v, dtype=torch.float32, device=DEV)
    return ops.sample_rows(logits.to(DEV), f(temperature), torch.full((rows,), top_k, dtype=torch.int32, device=DEV),
                           f(top_p), f(min_p), torch.as_tensor(u, dtype=torch.float32).expand(rows).contiguous().to(DEV)).tolist()


def test_sampling_vectors_of_the_reference():
    x = torch.tensor([[1.0, 2.0, 10.0, 1.5, 0.5]])  # infer/src/ops/tests.rs:333-378
    assert _sample(x, 0.01, 0.5) == [2]
    assert _sample(x, 1.0, 0.0) == [0]
    assert _sample(x, 1.0, 0.9, top_k=1) == [2]
    assert _sample(x, 0.0, 0.3) == [2]


@pytest.mark.parametrize("rows,vocab", [(1, 151936), (5, 333), (9, 4099), (64, 1031)])
def test_token_logprobs_are_the_log_softmax_of_the_chosen_tokens(rows, vocab):
    # for the largest logit: -log(sum exp(x - max)), crates/cuda-kernels/csrc/misc/sampling.cu:299-316
    g = _g(61)
    x = (torch.randn(rows, vocab, generator=g) * 4.0).contiguous()
    x[0, vocab // 2] = 40.0                       # a row with one dominant logit: its log-probability is about 0
    tokens = torch.randint(0, vocab, (rows,), generator=g).to(torch.int32)
    tokens[0] = vocab // 2
    if rows > 1:
        tokens[1] = int(x[1].argmax())
    got = ops.token_logprobs(x.to(DEV), tokens.to(DEV)).cpu().double()
    want = torch.log_softmax(x.double(), dim=-1)[torch.arange(rows), tokens.long()]
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)
    assert abs(float(got[0])) < 1e-3
    if rows > 1:
        m = x[1].double().max()
        assert abs(float(got[1]) + float(torch.log(torch.exp(x[1].double() - m).sum()))) < 2e-5


@pytest.mark.parametrize("vocab", [5, 333, 4099])
def test_sampling_against_plain_inverse_cdf(vocab):
    g = _g(60)
    logits = torch.randn(6, vocab, generator=g) * 2.0
    cases = [dict(temperature=0.8), dict(temperature=1.3, top_k=7), dict(temperature=1.0, top_p=0.6),
             dict(temperature=0.7, min_p=0.05), dict(temperature=1.1, top_k=20, top_p=0.8, min_p=0.01)]
    for case in cases:
        for u in (0.0, 0.13, 0.5, 0.77, 0.999):
            got = _sample(logits, case["temperature"], u, case.get("top_k", -1), case.get("top_p", 1.0),
                          case.get("min_p", 0.0))
            want = [plain.sample_token(row, case["temperature"], u, case.get("top_k", -1),
                                       case.get("top_p", 1.0), case.get("min_p", 0.0)) for row in logits]
            assert got == want, (case, u)


@pytest.mark.parametrize("rows,vocab", [(3, 151936), (9, 50257), (70, 8200)])
def test_sampling_of_long_rows_cut_into_chunks(rows, vocab):
    """Vocabularies long enough for several workgroups a row, widths that leave rows unaligned, rows that differ
    in every parameter (greedy ones among them), and filters switched off for the whole call."""
    g = _g(61)
    logits = torch.randn(rows, vocab, generator=g) * 2.5
    logits[0, vocab - 1] = 14.0                 # a peaked row: top_p keeps one token
    logits[1, :4] = 9.0                         # ties at the top
    pars = [dict(temperature=0.9, top_k=40, top_p=0.9, min_p=0.02), dict(temperature=1.2, top_k=3),
            dict(temperature=0.0), dict(temperature=0.7, top_p=0.35), dict(temperature=1.0, min_p=0.1),
            dict(temperature=1.5), dict(temperature=0.8, top_k=1), dict(temperature=1.0, top_k=vocab + 5, top_p=0.999),
            dict(temperature=0.6, top_k=500, top_p=0.5)]
    pars = [pars[i % len(pars)] for i in range(rows)]
    f32 = lambda key, default: torch.tensor([p.get(key, default) for p in pars], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([p.get("top_k", -1) for p in pars], dtype=torch.int32, device=DEV)
    check = range(rows) if rows <= 9 else range(0, rows, 7)
    for u in (0.0, 0.31, 0.62, 0.9995):
        us = torch.full((rows,), u, dtype=torch.float32, device=DEV)
        got = ops.sample_rows(logits.to(DEV), f32("temperature", 1.0), top_k, f32("top_p", 1.0), f32("min_p", 0.0),
                              us).tolist()
        for r in check:
            p = pars[r]
            want = plain.sample_token(logits[r], p["temperature"], u, p.get("top_k", -1), p.get("top_p", 1.0),
                                      p.get("min_p", 0.0))
            assert got[r] == want, (r, p, u)
    # no row with top_k or top_p: the passes that look for their thresholds are left out
    plain_rows = [dict(temperature=0.9), dict(temperature=1.1, min_p=0.05), dict(temperature=0.0)]
    pars = [plain_rows[i % 3] for i in range(rows)]
    us = torch.full((rows,), 0.44, dtype=torch.float32, device=DEV)
    got = ops.sample_rows(logits.to(DEV), f32("temperature", 1.0), torch.full((rows,), -1, dtype=torch.int32, device=DEV),
                          f32("top_p", 1.0), f32("min_p", 0.0), us, use_top_k=False, use_top_p=False).tolist()
    for r in check:
        p = pars[r]
        assert got[r] == plain.sample_token(logits[r], p["temperature"], 0.44, -1, 1.0, p.get("min_p", 0.0)), (r, p)


def test_penalties():
    logits = torch.tensor([[2.0, -2.0, 1.0, 0.5], [1.0, 1.0, 1.0, 1.0]])
    d = logits.to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
    ops.apply_penalties(d, i32([0, 2, 3]), i32([0, 1, 3]), i32([2, 1, 4]), f32([2.0, 1.0]), f32([0.5, 0.25]),
                        f32([0.25, 0.0]))
    want0 = plain.apply_penalties(logits[0], {0: 2, 1: 1}, 2.0, 0.5, 0.25)
    want1 = plain.apply_penalties(logits[1], {3: 4}, 1.0, 0.25, 0.0)
    assert torch.allclose(d.cpu(), torch.stack([want0, want1]))


def test_kernels_refuse_what_they_were_not_written_for():
    with pytest.raises(ops.ShapeError):
        ops.gemm_f32(torch.zeros(2, 3, device=DEV), torch.zeros(4, 5, device=DEV))
    with pytest.raises(ops.ShapeError):
        ops.rmsnorm(torch.zeros(2, 3), torch.ones(3), 1e-6, torch.float32)  # CPU tensors
    with pytest.raises(ops.ShapeError):
        ops.embed_gather(torch.zeros(4, 4, device=DEV), torch.zeros(2, dtype=torch.int64, device=DEV))


def _mfma_case(nq, nkv, D, P, segs, window, splits, seed, portion_splits=None, stale_nan=False):
    """segs: [(cached length before the step, rows in the step)].  Returns (got, want) [T, nq*D].
    stale_nan: every slot that no request has written holds NaN."""
    dt = torch.bfloat16
    lengths = [a + b for a, b in segs]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, seed)
    if stale_nan:
        k_pages.fill_(float("nan"))
        v_pages.fill_(float("nan"))
    qs, wants, row0, seg_start = [], [], [0], []
    for s, (cached, n) in enumerate(segs):
        g = _g(seed + 1 + s)
        total = cached + n
        q = torch.randn(total, nq, D, generator=g).to(dt)
        k = torch.randn(total, nkv, D, generator=g).to(dt)
        v = torch.randn(total, nkv, D, generator=g).to(dt)
        _fill_cache(table, k_pages, v_pages, s, k, v, P)
        full = plain.causal_attention(q.double(), k.double(), v.double(), nkv, window=window or None)
        qs.append(q[cached:].reshape(n, nq * D))
        wants.append(full[cached:].reshape(n, nq * D))
        row0.append(row0[-1] + n)
        seg_start.append(cached)
    q_all = torch.cat(qs).to(DEV)
    out = torch.full_like(q_all, float("nan"))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ops.attn_paged_mfma(q_all, out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0),
                        i32(list(range(len(segs)))), i32(seg_start), max_qlen=max(n for _, n in segs), min_qlen=min(n for _, n in segs),
                        max_kv_len=max(lengths), num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P,
                        scale=1.0 / math.sqrt(D), window=window, splits=splits, portion_splits=portion_splits)
    return out.cpu(), torch.cat(wants)


@pytest.mark.parametrize("nq,nkv,D,P", [(4, 2, 16, 4), (6, 2, 32, 8), (3, 1, 48, 16), (32, 8, 128, 16),
                                         (5, 1, 64, 16), (8, 1, 128, 32), (2, 2, 256, 16), (16, 1, 80, 64)])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_mfma_prompt_portions(nq, nkv, D, P, window):
    # portions that start mid-page after a cached prefix, a whole prompt, and a single first token
    got, want = _mfma_case(nq, nkv, D, P, [(0, 70), (45, 39), (0, 1), (130, 2)], window, 1, 70)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3


@pytest.mark.parametrize("nq,nkv,D,P", [(4, 2, 16, 4), (32, 8, 128, 16), (5, 1, 64, 16), (2, 2, 256, 16), (16, 1, 80, 64)])
@pytest.mark.parametrize("parts", [None, 2, 5, 8])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_mfma_portions_with_their_keys_cut_into_parts(nq, nkv, D, P, parts, window):
    """Portions too few to fill the chip: every row block's keys are cut into parts (some of them empty: more
    parts than tiles; parts that lie before a window or after a row's own position) and merged afterwards."""
    got, want = _mfma_case(nq, nkv, D, P, [(300, 70), (45, 39), (0, 1), (130, 2), (0, 200)], window, 1, 75,
                           portion_splits=parts)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3


@pytest.mark.parametrize("nq,nkv,D,P", [(4, 2, 16, 4), (6, 2, 32, 8), (3, 1, 48, 16), (32, 8, 128, 16),
                                         (40, 8, 128, 16), (64, 2, 64, 16)])
@pytest.mark.parametrize("splits", [None, 1, 3, 7])
@pytest.mark.parametrize("window", [0, 50])
def test_attention_mfma_decoded_tokens_split_over_the_keys(nq, nkv, D, P, splits, window):
    got, want = _mfma_case(nq, nkv, D, P, [(299, 1), (0, 1), (31, 1), (32, 1), (95, 1)], window, splits, 80)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3


@pytest.mark.parametrize("nq,nkv,D,P", [(16, 1, 128, 64), (8, 1, 128, 32), (16, 1, 80, 64), (32, 8, 128, 16), (6, 2, 32, 8), (8, 8, 64, 4)])
@pytest.mark.parametrize("window", [1, 2, 3, 5])
@pytest.mark.parametrize("splits", [None, 1, 6])
def test_attention_mfma_windows_of_a_few_keys_beside_stale_slots(nq, nkv, D, P, window, splits):
    """A window of a few keys at the end of requests whose lengths are no multiples of four, every unwritten slot
    NaN: the values that a kernel fetches in place of the keys in front of the window are the window's first four,
    which reach past the last token, and 0 * NaN is NaN.  Decoded tokens (all three kernels' stale-slot handling
    goes by the keys fetched, not by the keys asked for), and portions beside them."""
    got, want = _mfma_case(nq, nkv, D, P, [(294, 1), (309, 1), (400, 1), (518, 1), (141, 1), (2, 1), (0, 1)], window, splits, 95,
                           stale_nan=True)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3
    got, want = _mfma_case(nq, nkv, D, P, [(34, 11), (13, 2), (283, 28), (214, 1), (257, 1), (132, 1), (0, 70), (61, 130)], window,
                           1 if splits is None else splits, 96, stale_nan=True)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3


@pytest.mark.parametrize("nq,nkv,D", [(8, 2, 128), (3, 3, 64), (16, 1, 128)])
@pytest.mark.parametrize("splits", [None, 1, 5])
def test_attention_mfma_mixed_step_and_stale_pages(nq, nkv, D, splits):
    """Decoded tokens and portions of a few tokens (split over the keys) beside longer portions in one
    launch; pages hold NaN bits beyond each request's length, and so does the output before the call."""
    P = 16
    dt = torch.bfloat16
    segs = [(200, 1), (17, 30), (63, 1), (0, 5), (40, 3), (0, 2), (330, 1), (100, 16)]
    lengths = [a + b for a, b in segs]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 90)
    k_pages.fill_(float("nan"))
    v_pages.fill_(float("nan"))
    qs, wants, row0, starts = [], [], [0], []
    for s, (cached, n) in enumerate(segs):
        g = _g(91 + s)
        q, k, v = (torch.randn(cached + n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
        _fill_cache(table, k_pages, v_pages, s, k, v, P)
        qs.append(q[cached:].reshape(n, -1))
        wants.append(plain.causal_attention(q.double(), k.double(), v.double(), nkv)[cached:].reshape(n, -1))
        row0.append(row0[-1] + n)
        starts.append(cached)
    q_all = torch.cat(qs).to(DEV)
    out = torch.full_like(q_all, float("nan"))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ops.attn_paged_mfma(q_all, out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0),
                        i32(list(range(len(segs)))), i32(starts), max_qlen=30, min_qlen=1, max_kv_len=max(lengths),
                        num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D),
                        splits=splits, short_segments=3)
    assert torch.isfinite(out).all()
    assert _rel(out.cpu(), torch.cat(wants)) < 8e-3


def test_attention_mfma_step_too_large_for_the_work_list():
    """More (row block, segment) pairs than the planning kernel lists: the portions kernel then walks all
    pairs itself.  One long portion beside many decoded tokens, against the same segments launched alone
    (listed), which must agree bit for bit, and the decoded tokens against the plain implementation."""
    nq, nkv, D, P = 16, 1, 64, 16
    dt = torch.bfloat16
    long_n, singles = 3400, 40                      # 3400 * 16 rows / 128 = 425 row blocks, * 41 segments > 16384
    segs = [(0, long_n)] + [(20 + 3 * i, 1) for i in range(singles)]
    lengths = [a + b for a, b in segs]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 97)
    qs, row0, starts, wants = [], [0], [], []
    for s, (cached, n) in enumerate(segs):
        g = _g(98 + s)
        q, k, v = (torch.randn(cached + n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
        _fill_cache(table, k_pages, v_pages, s, k, v, P)
        qs.append(q[cached:].reshape(n, -1))
        if s > 0:
            wants.append(plain.causal_attention(q.double(), k.double(), v.double(), nkv)[cached:].reshape(n, -1))
        row0.append(row0[-1] + n)
        starts.append(cached)
    q_all = torch.cat(qs).to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    dk, dv, dtab = k_pages.to(DEV), v_pages.to(DEV), table.to(DEV)
    common = dict(num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D))
    out = torch.full_like(q_all, float("nan"))
    ops.attn_paged_mfma(q_all, out, dk, dv, dtab, i32(row0), i32(list(range(len(segs)))), i32(starts),
                        max_qlen=long_n, min_qlen=1, max_kv_len=max(lengths), short_segments=singles, **common)
    assert torch.isfinite(out).all()
    alone = torch.full_like(q_all[:long_n], float("nan"))
    ops.attn_paged_mfma(q_all[:long_n], alone, dk, dv, dtab, i32([0, long_n]), i32([0]), i32([0]),
                        max_qlen=long_n, min_qlen=long_n, max_kv_len=long_n, **common)
    assert torch.equal(out[:long_n], alone)
    assert _rel(out[long_n:].cpu(), torch.cat(wants)) < 8e-3


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("nq,nkv,P", [(32, 8, 16), (8, 8, 8), (16, 1, 64), (8, 1, 32), (6, 2, 128)])
@pytest.mark.parametrize("parts,window", [(None, 0), (1, 0), (3, 0), (8, 37), (1, 200)])
def test_attention_mfma_both_portion_kernels_at_head_dim_128(variant, nq, nkv, P, parts, window):
    """head_dim 128 has two kernels for prompt portions (16 rows a wave with tiles parked in LDS by the waves; 32
    rows a wave with tiles loaded straight into LDS, by one group of four waves or by two that take every other
    tile of keys each), chosen by the shape of the step; here each is forced in turn: portions that start inside a
    page after a cached prefix, whole prompts of several row blocks, a single first token and decoded tokens
    beside them, windows, and keys cut into parts."""
    from arle_amd.kernels import lib
    lib.function("arle_attn_prefill_variant")(min(variant, 1))
    lib.function("arle_attn_prefill_groups")(variant if variant else -1)
    try:
        got, want = _mfma_case(nq, nkv, 128, P, [(300, 70), (45, 39), (0, 1), (130, 2), (0, 330), (77, 1)], window, 1,
                               175, portion_splits=parts)
    finally:
        lib.function("arle_attn_prefill_variant")(-1)
        lib.function("arle_attn_prefill_groups")(-1)
    assert torch.isfinite(got).all()
    assert _rel(got, want) < 8e-3


@pytest.mark.parametrize("variant", [0, 1])
def test_attention_portions_list_their_work_once_for_calls_that_name_the_same_step(variant):
    """Calls with one plan_token and the same segments (the layers of a step) run the planning kernel once; the
    results are those of calls without a token.  Another step under the same token by mistake (other segments)
    is planned anew, and so is the same step under another token."""
    from arle_amd.kernels import lib
    nq, nkv, D, P = 8, 2, 128, 16
    lib.function("arle_attn_prefill_variant")(variant)
    try:
        def case(segs, seed, token):
            lengths = [a + b for a, b in segs]
            table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, torch.bfloat16, seed)
            qs, wants, row0, starts = [], [], [0], []
            for s_, (cached, n) in enumerate(segs):
                g = _g(seed + 1 + s_)
                q, k, v = (torch.randn(cached + n, h, D, generator=g).to(torch.bfloat16) for h in (nq, nkv, nkv))
                _fill_cache(table, k_pages, v_pages, s_, k, v, P)
                qs.append(q[cached:].reshape(n, -1))
                wants.append(plain.causal_attention(q.double(), k.double(), v.double(), nkv)[cached:].reshape(n, -1))
                row0.append(row0[-1] + n)
                starts.append(cached)
            i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
            args = (torch.cat(qs).to(DEV), k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0),
                    i32(list(range(len(segs)))), i32(starts))
            kw = dict(max_qlen=max(n for _, n in segs), min_qlen=min(n for _, n in segs), max_kv_len=max(lengths),
                      num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D))
            outs = []
            for tok in token:
                out = torch.full_like(args[0], float("nan"))
                ops.attn_paged_mfma(args[0], out, *args[1:], plan_token=tok, **kw)
                outs.append(out.cpu())
            return outs, torch.cat(wants)

        first = ops.new_plan_token()
        outs, want = case([(40, 300), (0, 170), (7, 1)], 300, [0, first, first, first, ops.new_plan_token()])
        for out in outs:
            assert torch.equal(out, outs[0]) and _rel(out, want) < 8e-3
        outs, want = case([(0, 50), (90, 420), (3, 33), (0, 200)], 310, [first, first, 0])   # the old token, other segments
        for out in outs:
            assert torch.equal(out, outs[-1]) and _rel(out, want) < 8e-3
    finally:
        lib.function("arle_attn_prefill_variant")(-1)


PREP_CACHED = None    # other context lengths for the test below, when something else calls it


@pytest.mark.parametrize("nq,nkv,D,rot,P", [(32, 8, 128, 128, 16), (8, 8, 64, 64, 8), (16, 1, 128, 64, 64), (6, 2, 64, 0, 4),
                                            (4, 4, 128, 0, 32), (12, 2, 128, 128, 128)])
@pytest.mark.parametrize("n_parts,splits,window,w_dtype", [(1, 1, 0, torch.bfloat16), (4, None, 0, torch.float32),
                                                           (3, 5, 37, torch.bfloat16), (7, 64, 0, None),
                                                           (2, 3, 0, torch.bfloat16), (5, 2, 37, torch.float32), (1, 4, 0, None),
                                                           (0, None, 0, torch.bfloat16), (0, 3, 37, torch.float32),
                                                           (2, 3, 2, torch.bfloat16), (0, 1, 3, torch.float32), (3, None, 1, None)])
def test_decode_attention_with_the_preparation_folded_in(nq, nkv, D, rot, P, n_parts, splits, window, w_dtype):
    """A step of single decoded tokens from the float32 stack of its q|k|v projection: sum, per-head norm, rotation,
    cache write and attention in one kernel.  Requests whose new token is the first of all, the first or last of
    a page and of a 32-key block, deep in a long context; slots of the cache that hold NaN bits where nothing was
    written yet (the new token's own slot among them).  Against the plain implementation, and against the two
    kernels that it replaces: the same cache to the last bit but one, and nothing else touched."""
    dt, eps, theta = torch.bfloat16, 1e-6, 1e4
    cached = PREP_CACHED or [0, 1, 31, 32, 63, P - 1, P, 700, 1029, 255]     # tokens a request holds before the step
    lengths = [c + 1 for c in cached]
    T = len(cached)
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 500)
    k_pages.fill_(float("nan"))
    v_pages.fill_(float("nan"))
    Q, KV = nq * D, nkv * D
    qw = kw = None
    if w_dtype is not None:
        qw = (1.0 + 0.2 * torch.randn(D, generator=_g(501))).to(w_dtype)
        kw = (1.0 + 0.2 * torch.randn(D, generator=_g(502))).to(w_dtype)
    cos = sin = None
    if rot:
        cos, sin = plain.rope_cos_sin(range(max(lengths) + 1), rot, theta)
    def prepared(x, w, positions):   # [n, heads, D] float64 -> norm, rotation of the first rot columns
        if w is not None:
            x = plain.qk_norm(x, w.double(), eps)
        if rot:
            c, s_ = plain.rope_cos_sin(positions, rot, theta, dtype=torch.float64)
            x = torch.cat([plain.apply_rope(x[..., :rot], c, s_), x[..., rot:]], -1)
        return x
    new_rows, wants = [], []
    for s_, n in enumerate(cached):
        g = _g(510 + s_)
        raw = torch.randn(n + 1, (nq + 2 * nkv) * D, generator=g)
        raw[:n] = raw[:n].to(dt).float()         # earlier tokens were projections in bfloat16
        x = raw.double()
        q = prepared(x[:, :Q].reshape(n + 1, nq, D), qw, list(range(n + 1)))
        k = prepared(x[:, Q:Q + KV].reshape(n + 1, nkv, D), kw, list(range(n + 1))).to(dt)
        v = x[:, Q + KV:].reshape(n + 1, nkv, D).to(dt)
        _fill_cache(table, k_pages, v_pages, s_, k[:n], v[:n], P)
        wants.append(plain.causal_attention(q.to(dt).double(), k.double(), v.double(), nkv, window=window or None,
                                            rows=[n])[n].reshape(-1))
        new_rows.append(raw[n])
    row = torch.stack(new_rows)                                      # [T, width] float32
    if n_parts == 0:       # the projection itself in bfloat16 instead of a stack of its parts
        stack = row.to(dt)
        exact = stack.double()
    else:
        stack = torch.randn(n_parts, T, row.shape[1], generator=_g(503))
        stack[-1] = row - (stack[:-1].double().sum(0)).float() if n_parts > 1 else row
        exact = stack.double().sum(0)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    dev = lambda t: None if t is None else t.to(DEV)
    seg = (i32(list(range(T + 1))), i32(list(range(T))), i32(cached))
    kw_args = dict(num_q_heads=nq, num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D), window=window)
    dk, dv = k_pages.to(DEV), v_pages.to(DEV)
    out = torch.full((T, Q), float("nan"), dtype=dt, device=DEV)
    ops.attn_decode_prep(stack.to(DEV), out, dk, dv, table.to(DEV), *seg, max_kv_len=max(lengths), eps=eps, q_weight=dev(qw),
                         k_weight=dev(kw), cos=dev(cos), sin=dev(sin), rotary_dim=rot, splits=splits, **kw_args)
    assert torch.isfinite(out.float()).all()
    if splits in (2, 3, 4):
        # the splits of a request's keys as the waves of one workgroup that merge in LDS, and as workgroups of their own
        # whose parts a second kernel merges: here both are forced in turn
        from arle_amd.kernels import lib
        both = []
        try:
            for mode in (1, 0):
                lib.function("arle_attn_decode_inwg")(mode)
                o_ = torch.full((T, Q), float("nan"), dtype=dt, device=DEV)
                ops.attn_decode_prep(stack.to(DEV), o_, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), *seg,
                                     max_kv_len=max(lengths), eps=eps, q_weight=dev(qw), k_weight=dev(kw), cos=dev(cos),
                                     sin=dev(sin), rotary_dim=rot, splits=splits, **kw_args)
                both.append(o_.cpu())
        finally:
            lib.function("arle_attn_decode_inwg")(-1)
        for o_ in both:
            assert torch.isfinite(o_.float()).all() and _rel(o_, torch.stack(wants)) < 1e-2
        assert _rel(both[0], both[1]) < 4e-3 and torch.equal(out.cpu(), both[1] if T * nkv < 256 else both[0])
    # the stack's own sum is what the kernel saw: compare with plain values made from it
    for s_, n in enumerate(cached):
        x = exact[s_]
        k_want = prepared(x[Q:Q + KV].reshape(1, nkv, D), kw, [n])[0]
        page, at = int(table[s_, n // P]), n % P
        assert _rel(dk[page, :, at].cpu(), k_want) < 6e-3
        assert _rel(dv[page, :, :, at].cpu(), x[Q + KV:].reshape(nkv, D)) < 6e-3
    assert _rel(out.cpu(), torch.stack(wants)) < 1e-2
    # the two kernels that it stands for
    dk2, dv2 = k_pages.to(DEV), v_pages.to(DEV)
    prep_args = dict(num_q_heads=nq, num_kv_heads=nkv, head_dim=D, eps=eps, q_weight=dev(qw), k_weight=dev(kw), cos=dev(cos),
                     sin=dev(sin), rotary_dim=rot, positions=seg[2], slot_of_token=seg[1], block_table=table.to(DEV),
                     k_pages=dk2, v_pages=dv2, page_size=P)
    if n_parts == 0:
        qkv2 = stack.to(DEV)
        q2 = qkv2[:, :Q]
        ops.qk_prep(q2, qkv2[:, Q:Q + KV], qkv2[:, Q + KV:], **prep_args)
    else:
        q2 = torch.empty((T, Q), dtype=dt, device=DEV)
        ops.qk_prep(q2, None, None, parts=stack.to(DEV), **prep_args)
    out2 = torch.full((T, Q), float("nan"), dtype=dt, device=DEV)
    ops.attn_paged_mfma(q2, out2, dk2, dv2, table.to(DEV), *seg, max_qlen=1, max_kv_len=max(lengths), splits=splits, **kw_args)
    assert _rel(out.cpu(), out2.cpu()) < 4e-3
    # the same cache: every slot but the new tokens' bit for bit as it was, theirs as the two kernels leave them but
    # for the last bits (the parts of the stack and the squares of a head are added in another order)
    ka, kb, va, vb = (t.cpu().view(torch.int16).clone() for t in (dk, dk2, dv, dv2))
    for s_, n in enumerate(cached):
        page, at = int(table[s_, n // P]), n % P
        assert _rel(dk[page, :, at].cpu(), dk2[page, :, at].cpu()) < 8e-3
        assert _rel(dv[page, :, :, at].cpu(), dv2[page, :, :, at].cpu()) < 8e-3
        ka[page, :, at] = kb[page, :, at] = 0
        va[page, :, :, at] = vb[page, :, :, at] = 0
    assert torch.equal(ka, kb) and torch.equal(va, vb)


@pytest.mark.parametrize("variant,groups,heads", [(1, 1, 24), (1, 2, 12), (0, -1, 12)])
@pytest.mark.parametrize("parts", [None, 2])
def test_attention_portions_dealt_out_before_the_launch_or_taken_from_the_counter(variant, groups, heads, parts):
    """Both portions kernels get their (row block, kv head, part) items either from a counter at run time or dealt
    out to and fro over the workgroups before the launch; the list of both is ordered by the keys an entry sees.
    Segments of very different lengths and contexts, more items than workgroups (so that a workgroup gets a second
    and third item); the kernel that parks tiles in LDS, and the one that loads them straight there with one or two
    groups of waves: the same bits either way, and the plain result at rows of every segment."""
    from arle_amd.kernels import lib
    nq = nkv = heads
    D, P, dt = 128, 16, torch.bfloat16
    segs = [(100, 512), (0, 2048), (40, 1), (1500, 256), (700, 128)]
    lengths = [a + b for a, b in segs]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 410)
    qs, row0, starts, checks = [], [0], [], []
    for s_, (cached, n) in enumerate(segs):
        g = _g(411 + s_)
        q, k, v = (torch.randn(cached + n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
        _fill_cache(table, k_pages, v_pages, s_, k, v, P)
        rows = sorted({cached, cached + n // 2, cached + n - 1})
        want = plain.causal_attention(q.double(), k.double(), v.double(), nkv, rows=rows)
        checks += [(row0[-1] + r - cached, want[r].reshape(-1)) for r in rows]
        qs.append(q[cached:].reshape(n, -1))
        row0.append(row0[-1] + n)
        starts.append(cached)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    q_all = torch.cat(qs).to(DEV)
    args = (k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0), i32(list(range(len(segs)))), i32(starts))
    kw = dict(max_qlen=2048, min_qlen=1, max_kv_len=max(lengths), num_q_heads=nq, num_kv_heads=nkv, head_dim=D,
              page_size=P, scale=1.0 / math.sqrt(D), portion_splits=parts)
    lib.function("arle_attn_prefill_variant")(variant)
    lib.function("arle_attn_prefill_groups")(groups)
    outs = {}
    try:
        for rounds in (0, 64, -1, 2):   # never dealt; always; by the launcher's rule; up to two items a workgroup
            lib.function("arle_attn_prefill_fixed_rounds")(rounds)
            out = torch.full_like(q_all, float("nan"))
            ops.attn_paged_mfma(q_all, out, *args, **kw)
            outs[rounds] = out.cpu()
    finally:
        lib.function("arle_attn_prefill_variant")(-1)
        lib.function("arle_attn_prefill_groups")(-1)
        lib.function("arle_attn_prefill_fixed_rounds")(-1)
    for rounds, out in outs.items():
        assert torch.isfinite(out.float()).all()
        assert torch.equal(out, outs[0]), rounds
    for row, want in checks:
        assert _rel(outs[0][row].float(), want) < 8e-3


@pytest.mark.parametrize("P", [16, 64, 128])
def test_attention_mfma_dma_kernel_masks_stale_slots(P):
    """The kernel that loads tiles straight into LDS: pages hold NaN bits in every slot that was never written
    (with pages of 64 keys and more it reads a tile's keys beyond the request as they lie there)."""
    from arle_amd.kernels import lib
    nq, nkv, D = 8, 2, 128
    dt = torch.bfloat16
    segs = [(200, 150), (17, 130), (0, 70)]
    lengths = [a + b for a, b in segs]
    table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 190)
    k_pages.fill_(float("nan"))
    v_pages.fill_(float("nan"))
    qs, wants, row0, starts = [], [], [0], []
    for s, (cached, n) in enumerate(segs):
        g = _g(191 + s)
        q, k, v = (torch.randn(cached + n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
        _fill_cache(table, k_pages, v_pages, s, k, v, P)
        qs.append(q[cached:].reshape(n, -1))
        wants.append(plain.causal_attention(q.double(), k.double(), v.double(), nkv)[cached:].reshape(n, -1))
        row0.append(row0[-1] + n)
        starts.append(cached)
    q_all = torch.cat(qs).to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    lib.function("arle_attn_prefill_variant")(1)
    try:
        for parts, groups in ((1, 1), (2, 1), (1, 2), (2, 2)):
            lib.function("arle_attn_prefill_groups")(groups)
            out = torch.full_like(q_all, float("nan"))
            ops.attn_paged_mfma(q_all, out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0), i32([0, 1, 2]),
                                i32(starts), max_qlen=150, min_qlen=70, max_kv_len=max(lengths), num_q_heads=nq,
                                num_kv_heads=nkv, head_dim=D, page_size=P, scale=1.0 / math.sqrt(D), portion_splits=parts)
            assert torch.isfinite(out).all()
            assert _rel(out.cpu(), torch.cat(wants)) < 8e-3
    finally:
        lib.function("arle_attn_prefill_variant")(-1)
        lib.function("arle_attn_prefill_groups")(-1)


def test_attention_mfma_finds_a_far_key():
    nq, nkv, D, P, n = 4, 2, 64, 16, 900
    dt = torch.bfloat16
    table, k_pages, v_pages = _paged_setup([n], nkv, D, P, dt, 95)
    g = _g(96)
    q = (torch.randn(n, nq, D, generator=g) * 0.1).to(dt)
    k = (torch.randn(n, nkv, D, generator=g) * 0.1).to(dt)
    v = torch.randn(n, nkv, D, generator=g).to(dt)
    far = 5
    k[far, 0] = (q[n - 1, 1].float() * 400.0).to(dt)
    _fill_cache(table, k_pages, v_pages, 0, k, v, P)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for splits in (1, 6):   # as the last row of a portion, and as a decoded token split over the keys
        rows = 40 if splits == 1 else 1
        qq = q[n - rows:].reshape(rows, -1).to(DEV).contiguous()
        out = torch.empty_like(qq)
        ops.attn_paged_mfma(qq, out, k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32([0, rows]), i32([0]),
                            i32([n - rows]), max_qlen=rows, min_qlen=rows, max_kv_len=n, num_q_heads=nq, num_kv_heads=nkv,
                            head_dim=D, page_size=P, scale=1.0 / math.sqrt(D), splits=splits)
        got = out.cpu().reshape(rows, nq, D)
        assert torch.allclose(got[-1, 1].float(), v[far, 0].float(), atol=2e-2)


def test_attention_mfma_refuses_shapes_it_was_not_written_for():
    assert not ops.attn_mfma_supported(torch.bfloat16, 24, 16)
    assert not ops.attn_mfma_supported(torch.bfloat16, 128, 6)
    assert not ops.attn_mfma_supported(torch.bfloat16, 128, 12)   # such pages go to the fixed-order kernel
    assert not ops.attn_mfma_supported(torch.float32, 128, 16)
    assert not ops.attn_mfma_supported(torch.bfloat16, 272, 16)
    q = torch.zeros(2, 2 * 24, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.ShapeError, match="head_dim % 16"):
        ops.attn_paged_mfma(q, torch.empty_like(q), torch.zeros(1, 1, 16, 24, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(1, 1, 24, 16, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                            torch.tensor([0, 2], dtype=torch.int32, device=DEV),
                            torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                            max_qlen=2, max_kv_len=2, num_q_heads=2, num_kv_heads=1, head_dim=24, page_size=16, scale=1.0)


def _whole(out):
    """A product, or the stack of partial products a split K leaves behind, as one float64 matrix."""
    return out.double().sum(0).cpu() if out.dim() == 3 else out.double().cpu()


@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(96, 64), (333, 88), (2560, 4096), (6144, 2560), (40, 8), (2560, 9728)])
def test_gemm_rows_as_planned(M, N, K):
    a = torch.randn(M, K, generator=_g(100)).bfloat16()
    w = (torch.randn(N, K, generator=_g(101)) * 0.1).bfloat16()
    want = a.double() @ w.double().T
    got = ops.gemm_rows(a.to(DEV), w.to(DEV), torch.float32)
    assert _rel(_whole(got), want) < 1e-5          # float32 accumulation of exact bfloat16 products
    # the general entry point always hands back whole sums, in the type asked for
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.bfloat16).cpu()
    assert got.dtype == torch.bfloat16 and got.shape == (M, N) and _rel(got, want) < 5e-3
    # a view with a row stride (rows of a wider buffer)
    wide = torch.randn(M, K + 24, generator=_g(102)).bfloat16().to(DEV)
    got = ops.gemm_rows(wide[:, 8:8 + K], w.to(DEV), torch.float32)
    assert _rel(_whole(got), wide[:, 8:8 + K].double().cpu() @ w.double().T) < 1e-5


@pytest.mark.parametrize("variant", range(ops.STREAM_VARIANTS))
@pytest.mark.parametrize("M,N,K,splits,workgroups", [(5, 333, 88, 1, 2), (16, 96, 1096, 3, 1), (20, 200, 520, 2, 64),
                                                     (64, 72, 2056, 5, 1), (33, 2560, 4096, 6, 11), (64, 1000, 2056, 3, 3),
                                                     (48, 100, 4104, 4, None), (1, 40, 8, 1, 7)])
def test_gemm_stream_workgroups_that_walk_several_column_groups(variant, M, N, K, splits, workgroups):
    """The kernel whose workgroups stay: widths that end inside a column group and inside a k step, slices that
    end inside a round, one workgroup for all groups and more workgroups than groups, LDS beyond 64 KB."""
    a = torch.randn(M, K, generator=_g(105)).bfloat16()
    w = (torch.randn(N, K, generator=_g(106)) * 0.1).bfloat16()
    got = ops.gemm_stream(a.to(DEV), w.to(DEV), torch.float32, variant=variant, splits=splits, workgroups=workgroups)
    assert got.dim() == 2 or got.shape[0] >= splits
    assert _rel(_whole(got), a.double() @ w.double().T) < 1e-5


def test_gemm_bf16_takes_the_staying_kernel_for_narrow_outputs_of_17_to_64_rows():
    for M in (17, 40, 64):
        a = torch.randn(M, 4096, generator=_g(107)).bfloat16()
        w = (torch.randn(2560, 4096, generator=_g(108)) * 0.05).bfloat16()
        assert ops.gemm_stream_preferred(M, 2560, 4096, 4096)
        stack = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.bfloat16, partials_ok=True)
        assert stack.dim() == 3 and stack.dtype == torch.float32
        whole = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.bfloat16)
        assert whole.shape == (M, 2560) and whole.dtype == torch.bfloat16
        want = a.double() @ w.double().T
        assert _rel(stack.double().sum(0).cpu(), want) < 1e-5
        assert _rel(whole.cpu(), want) < 6e-3
    assert not ops.gemm_stream_preferred(64, 19456, 2560, 2560) and not ops.gemm_stream_preferred(16, 2560, 4096, 4096)


@pytest.mark.parametrize("variant", range(ops.ROWS_VARIANTS))
@pytest.mark.parametrize("M,N,K,splits", [(5, 333, 88, 1), (16, 96, 1096, 3), (20, 200, 520, 2), (64, 72, 2056, 5),
                                          (33, 2560, 4096, 16), (64, 72, 2056, 3), (48, 100, 4104, 4)])
def test_gemm_rows_every_variant_and_split(variant, M, N, K, splits):
    a = torch.randn(M, K, generator=_g(103)).bfloat16()
    w = (torch.randn(N, K, generator=_g(104)) * 0.1).bfloat16()
    got = ops.gemm_rows(a.to(DEV), w.to(DEV), torch.float32, variant=variant, splits=splits)
    # a stack of at most `splits` partial products, or whole sums when K holds a single round of this variant
    assert (got.dim() == 2 or 1 < got.shape[0] <= splits) and (splits > 1 or got.dim() == 2)
    assert _rel(_whole(got), a.double() @ w.double().T) < 1e-5
    again = ops.gemm_rows(a.to(DEV), w.to(DEV), torch.float32, variant=variant, splits=splits)
    assert torch.equal(got, again)                 # nothing in the kernel depends on timing


@pytest.mark.parametrize("M", [1, 8, 20, 64])
@pytest.mark.parametrize("inter,K", [(48, 64), (224, 96), (9728, 2560)])
def test_gemm_rows_with_fused_activation(M, inter, K):
    x = torch.randn(M, K, generator=_g(110)).bfloat16()
    gate = (torch.randn(inter, K, generator=_g(111)) * 0.1).bfloat16()
    up = (torch.randn(inter, K, generator=_g(112)) * 0.1).bfloat16()
    fused = torch.stack([gate.view(-1, 16, K), up.view(-1, 16, K)], dim=1).reshape(2 * inter, K).contiguous()
    want = plain.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    for variant in (None, 0, 1, 3, 4):
        planned = ops.gemm_rows_plan(M, 2 * inter, K, True)[0] if variant is None else variant
        if ops._rows_min_splits(planned, M, K) > 1:
            continue      # these rows of all of K do not fit into LDS: no whole sums, no fused activation
        got = ops.gemm_rows(x.to(DEV), fused.to(DEV), torch.float32, ops.EPI_SILU_MUL, variant=variant, splits=1).cpu()
        assert got.shape == (M, inter) and _rel(got, want) < 1e-5
    # the same weights through the library product and the interleaved activation kernel
    gu = (x.double() @ fused.double().T).bfloat16().to(DEV)
    got = ops.silu_mul_interleaved(gu, 16).cpu()
    assert _rel(got, want) < 1e-2


@pytest.mark.parametrize("M,N,K", [(65, 2560, 4096), (200, 333, 2048), (512, 2560, 9728), (1024, 96, 8192), (300, 2560, 2080),
                                   (1500, 160, 8256), (3100, 96, 8192), (1100, 96, 4096), (700, 5120, 8192), (700, 5152, 8192)])
def test_library_product_cut_along_k_for_narrow_outputs(M, N, K):
    """65 to 1,024 rows, a narrow output (up to 5,120 columns) and a long K: the library's product is run as a
    batched product of parts of K, and the parts come back as a float32 stack whose sum, in order, is the product;
    with K of 8,192 and more, two parts up to 3,072 rows."""
    x = torch.randn(M, K, generator=_g(150)).bfloat16()
    w = (torch.randn(N, K, generator=_g(151)) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    splits = ops.library_k_splits(M, N, K)
    if M > 1024:
        assert splits == {(1500, 8256): 2, (3100, 8192): 1, (1100, 4096): 1}[(M, K)]
    elif N > 4096:
        assert splits == (4 if N == 5120 else 1)
    else:
        assert splits == {4096: 4 if M <= 512 else 2, 2048: 4, 9728: 4, 8192: 4, 2080: 1}[K] or (K == 4096 and M == 65 and splits == 4)
    got = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.bfloat16, partials_ok=True)
    if splits > 1:
        assert got.dtype == torch.float32 and got.shape == (splits, M, N)
        part = K // splits
        assert _rel(got[1].cpu(), x[:, part:2 * part].double() @ w[:, part:2 * part].double().T) < 1e-5
        assert _rel(got.sum(0).cpu(), want) < 1e-5           # float32 parts: no rounding to bfloat16 in between
    else:
        assert got.shape == (M, N) and _rel(got.cpu(), want) < 8e-3
    whole = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.bfloat16)           # a caller that cannot add a stack gets none
    assert whole.shape == (M, N) and whole.dtype == torch.bfloat16 and _rel(whole.cpu(), want) < 8e-3
    # a strided x (a view of wider rows)
    wide = torch.randn(M, K + 64, generator=_g(152)).bfloat16().to(DEV)
    got = ops.gemm_bf16(wide[:, :K], w.to(DEV), torch.bfloat16, partials_ok=True)
    got = got.sum(0) if got.dim() == 3 else got
    assert _rel(got.cpu(), wide[:, :K].cpu().double() @ w.double().T) < 8e-3


@pytest.mark.parametrize("M,N,K", [(65, 2560, 4096), (128, 2560, 9728), (200, 333, 2048), (256, 2560, 4096), (96, 136, 2056)])
def test_narrow_products_of_65_to_256_rows_go_to_the_tiles_kernel_when_tiles_are_given(M, N, K):
    """With operand tiles at hand a narrow product of 65 to 256 rows is cut along K for gemm_tiles' workgroups of
    128 x 128: a float32 stack whose parts add up to the product; without tiles, or for a caller that cannot add a
    stack, nothing changes."""
    x = torch.randn(M, K, generator=_g(153)).bfloat16()
    w = (torch.randn(N, K, generator=_g(154)) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    tiles = ops.pack_weight_tiles(w.to(DEV))
    splits = ops.narrow_tiles_splits(M, N, K, K)
    assert splits in (2, 4, 8) and -(-N // 128) * -(-M // 128) * splits <= 200
    got = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.bfloat16, partials_ok=True, tiles=tiles)
    assert got.dtype == torch.float32 and got.dim() == 3 and got.shape[1:] == (M, N) and got.shape[0] <= splits
    assert _rel(got.sum(0).cpu(), want) < 1e-5
    whole = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.bfloat16, tiles=tiles)
    assert whole.shape == (M, N) and whole.dtype == torch.bfloat16 and _rel(whole.cpu(), want) < 8e-3
    assert ops.narrow_tiles_splits(64, N, K, K) == 0 and ops.narrow_tiles_splits(257, N, K, K) == 0
    assert ops.narrow_tiles_splits(M, 6144, K, K) == 0 and ops.narrow_tiles_splits(256, 2560, 9728, 9728) == 0


def test_pack_weight_tiles_layout():
    """Tile (t, s), lane 16 g + i, element e is w[16 t + i, 32 s + 8 g + e]; zeros past the matrix."""
    N, K = 37, 72
    w = torch.arange(N * K, dtype=torch.float32).reshape(N, K).bfloat16()
    tiles = ops.pack_weight_tiles(w.to(DEV)).cpu()
    assert tiles.shape == (3, 3, 512)
    for t, s_, g, i, e in [(0, 0, 0, 0, 0), (0, 0, 1, 0, 0), (0, 0, 0, 1, 0), (1, 2, 0, 3, 7), (2, 1, 3, 4, 5), (2, 2, 1, 4, 0),
                           (2, 0, 0, 5, 0)]:
        n, k = 16 * t + i, 32 * s_ + 8 * g + e
        want = w[n, k] if (n < N and k < K) else torch.tensor(0.0).bfloat16()
        assert tiles[t, s_, (16 * g + i) * 8 + e] == want, (t, s_, g, i, e)


@pytest.mark.parametrize("M,N,K,splits", [(1, 333, 88, 1), (5, 37, 72, 1), (16, 96, 1096, 3), (20, 200, 520, 2), (64, 72, 2056, 5),
                                          (8, 2560, 4096, 4), (33, 1000, 2056, 3)])
def test_gemm_rows_and_stream_from_operand_tiles_equal_rows_bit_for_bit(M, N, K, splits):
    """Widths that end inside a tile of 16 rows and inside a k step of 32; every variant of both kernels."""
    a = torch.randn(M, K, generator=_g(120)).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=_g(121)) * 0.1).bfloat16().to(DEV)
    tiles = ops.pack_weight_tiles(w)
    for variant in range(ops.ROWS_VARIANTS):
        rows = ops.gemm_rows(a, w, torch.float32, variant=variant, splits=splits)
        got = ops.gemm_rows(a, w, torch.float32, variant=variant, splits=splits, tiles=tiles)
        assert torch.equal(rows, got), variant
    assert _rel(_whole(got), a.double().cpu() @ w.double().cpu().T) < 1e-5
    for variant in range(ops.STREAM_VARIANTS):
        rows = ops.gemm_stream(a, w, torch.float32, variant=variant, splits=splits, workgroups=3)
        got = ops.gemm_stream(a, w, torch.float32, variant=variant, splits=splits, workgroups=3, tiles=tiles)
        assert torch.equal(rows, got), variant
    assert _rel(_whole(got), a.double().cpu() @ w.double().cpu().T) < 1e-5
    assert torch.equal(ops.gemm_bf16(a, w, torch.bfloat16), ops.gemm_bf16(a, w, torch.bfloat16, tiles=tiles))
    with pytest.raises(ops.ShapeError, match="operand tiles"):
        ops.gemm_rows(a, w, torch.float32, tiles=tiles[:, :-1].contiguous())


def test_gemm_rows_fused_activation_from_operand_tiles():
    M, inter, K = 8, 224, 96
    x = torch.randn(M, K, generator=_g(122)).bfloat16().to(DEV)
    fused = (torch.randn(2 * inter, K, generator=_g(123)) * 0.1).bfloat16().to(DEV)
    rows = ops.gemm_rows(x, fused, torch.bfloat16, ops.EPI_SILU_MUL)
    assert torch.equal(rows, ops.gemm_rows(x, fused, torch.bfloat16, ops.EPI_SILU_MUL, tiles=ops.pack_weight_tiles(fused)))


@pytest.mark.parametrize("M,inter,K,round_steps", [(64, 224, 2560, None), (40, 48, 200, 3), (28, 160, 1096, 7), (33, 64, 96, 1),
                                                   (5, 32, 72, 2), (17, 96, 2560, 80), (64, 32, 264, 4)])
def test_gemm_rows_fused_activation_with_k_walked_in_rounds(M, inter, K, round_steps):
    """gate|up with the activation for more rows than LDS holds of all of K: rounds of every length (one step, one
    round for all of K, a last round that is shorter, K that ends inside a step), every row-tile count, from rows
    and from operand tiles; where one round holds everything the bits are those of the kernel without rounds."""
    x = torch.randn(M, K, generator=_g(140)).bfloat16()
    gate = (torch.randn(inter, K, generator=_g(141)) * 0.1).bfloat16()
    up = (torch.randn(inter, K, generator=_g(142)) * 0.1).bfloat16()
    fused = torch.stack([gate.view(-1, 16, K), up.view(-1, 16, K)], dim=1).reshape(2 * inter, K).contiguous().to(DEV)
    want = plain.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    xd, tiles = x.to(DEV), ops.pack_weight_tiles(fused)
    got = ops.gemm_rows_rounds(xd, fused, torch.float32, round_steps=round_steps)
    assert got.shape == (M, inter) and _rel(got.cpu(), want) < 1e-5
    assert torch.equal(got, ops.gemm_rows_rounds(xd, fused, torch.float32, tiles=tiles, round_steps=round_steps))
    assert _rel(ops.gemm_rows_rounds(xd, fused, torch.bfloat16, tiles=tiles, round_steps=round_steps).cpu(), want) < 5e-3
    if M <= 16 and K <= 2560:      # fits in one go: the same sums in the same order
        assert torch.equal(got, ops.gemm_rows(xd, fused, torch.float32, ops.EPI_SILU_MUL, variant=3, splits=1))
    with pytest.raises(ops.ShapeError):
        ops.gemm_rows_rounds(xd, fused, round_steps=10 ** 6 if M * K > 60000 else 0)


def test_which_kernel_takes_gate_up_with_its_activation_by_rows_and_shape():
    """The few-rows kernel in one go while the x rows of all of K fit into LDS, then the kernel that walks K in
    rounds where it was measured ahead of the library: up to 16 rows at every width, up to 32 rows where the output
    gives no more workgroups than the chip has compute units, up to 64 rows for a wide output."""
    def taken(rows, n, k):
        if ops.gemm_rows_preferred(rows, n, k, k, fused=True):
            return "one go"
        return "rounds" if ops.gemm_rows_rounds_preferred(rows, n, k, k) else "library"
    assert [taken(r, 19456, 2560) for r in (8, 27, 28, 48, 64, 65)] == ["one go"] * 2 + ["rounds"] * 3 + ["library"]
    assert [taken(r, 51200, 5120) for r in (8, 13, 14, 16, 17, 32)] == ["one go"] * 2 + ["rounds"] * 2 + ["library"] * 2
    assert [taken(r, 12288, 2048) for r in (16, 32, 33, 64)] == ["one go", "one go", "library", "library"]
    assert [taken(r, 24576, 4096) for r in (16, 17, 32, 64)] == ["one go", "rounds", "rounds", "rounds"]


@pytest.mark.parametrize("variant", ops.TILES_VARIANTS)
@pytest.mark.parametrize("M,N,K", [(300, 200, 72), (129, 520, 264), (257, 256, 32), (1, 40, 8), (640, 1000, 1096),
                                   (2300, 4900, 64)])
def test_gemm_tiles_many_rows_from_operand_tiles(variant, M, N, K):
    """Rows, columns and K that end inside a workgroup's block, inside a tile and inside a step of 32; fewer steps
    than a ring holds; every workgroup shape and ring depth."""
    x = torch.randn(M, K, generator=_g(130)).bfloat16()
    w = (torch.randn(N, K, generator=_g(131)) * 0.1).bfloat16()
    tiles = ops.pack_weight_tiles(w.to(DEV))
    want = x.double() @ w.double().T
    got = ops.gemm_tiles(x.to(DEV), tiles, N, torch.float32, variant=variant).cpu()
    assert got.shape == (M, N) and _rel(got, want) < 1e-5
    got = ops.gemm_tiles(x.to(DEV), tiles, N, torch.bfloat16, variant=variant).cpu()
    assert got.dtype == torch.bfloat16 and _rel(got, want) < 5e-3
    # a view with a row stride
    wide = torch.randn(M, K + 24, generator=_g(132)).bfloat16().to(DEV)
    got = ops.gemm_tiles(wide[:, 8:8 + K], tiles, N, torch.float32, variant=variant).cpu()
    assert _rel(got, wide[:, 8:8 + K].double().cpu() @ w.double().T) < 1e-5


@pytest.mark.parametrize("variant", ops.TILES_VARIANTS)
@pytest.mark.parametrize("M,inter,K", [(513, 224, 136), (200, 48, 64), (2048, 1024, 256), (300, 128, 1096)])
def test_gemm_tiles_with_fused_activation(variant, M, inter, K):
    x = torch.randn(M, K, generator=_g(133)).bfloat16()
    gate = (torch.randn(inter, K, generator=_g(134)) * 0.1).bfloat16()
    up = (torch.randn(inter, K, generator=_g(135)) * 0.1).bfloat16()
    fused = torch.stack([gate.view(-1, 16, K), up.view(-1, 16, K)], dim=1).reshape(2 * inter, K).contiguous()
    want = plain.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    tiles = ops.pack_weight_tiles(fused.to(DEV))
    got = ops.gemm_tiles(x.to(DEV), tiles, 2 * inter, torch.float32, ops.EPI_SILU_MUL, variant=variant).cpu()
    assert got.shape == (M, inter) and _rel(got, want) < 1e-5
    got = ops.gemm_tiles(x.to(DEV), tiles, 2 * inter, torch.bfloat16, ops.EPI_SILU_MUL, variant=variant).cpu()
    assert _rel(got, want) < 5e-3


@pytest.mark.parametrize("variant", ops.TILES_VARIANTS)
@pytest.mark.parametrize("M,N,K,splits", [(100, 200, 1096, 3), (129, 136, 264, 9), (65, 2560, 4096, 8), (300, 72, 96, 2)])
def test_gemm_tiles_parts_of_k_as_a_stack(variant, M, N, K, splits):
    """K cut into parts that end inside a step of 32 and inside a ring: part p of the stack is the product over
    the p-th part of K alone, and the parts add up to the product."""
    x = torch.randn(M, K, generator=_g(136)).bfloat16()
    w = (torch.randn(N, K, generator=_g(137)) * 0.1).bfloat16()
    tiles = ops.pack_weight_tiles(w.to(DEV))
    got = ops.gemm_tiles(x.to(DEV), tiles, N, torch.float32, variant=variant, splits=splits).cpu()
    steps = -(-K // 32)
    per = -(-steps // splits)
    assert got.shape == (-(-steps // per), M, N)
    for part in range(got.shape[0]):
        k0, k1 = part * per * 32, min((part + 1) * per * 32, K)
        assert _rel(got[part], x[:, k0:k1].double() @ w[:, k0:k1].double().T) < 1e-5, f"part {part}"
    assert _rel(got.double().sum(0), x.double() @ w.double().T) < 1e-5
    with pytest.raises(ops.ShapeError, match="float32 stack"):
        ops.gemm_tiles(x.to(DEV), tiles, N, torch.bfloat16, variant=variant, splits=splits)


def test_gemm_tiles_patches_of_workgroups_cover_every_tile():
    """However the workgroups that run side by side on an XCD are laid out over the row and column blocks (patches
    that end beyond the last row block, the last column block, or both; one workgroup a patch), every tile is
    computed once, with the same bits."""
    from arle_amd.kernels import lib

    M, N, K = 1100, 2100, 64
    x = torch.randn(M, K, generator=_g(136)).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=_g(137)) * 0.1).bfloat16().to(DEV)
    tiles = ops.pack_weight_tiles(w)
    want = x.double().cpu() @ w.double().cpu().T
    patch = lib.function("arle_gemm_tiles_patch")
    try:
        results = []
        for rows, cols in ((8, 8), (3, 2), (1, 1), (5, 1), (2, 7), (4096, 1)):
            patch(rows, cols)
            for variant in ((4, 44), (8, 144), (4, 44, 1)):
                junk = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
                del junk        # the result takes this memory: a tile left out would show
                out = ops.gemm_tiles(x, tiles, N, torch.float32, variant=variant)
                assert _rel(out.cpu(), want) < 1e-5, (rows, cols, variant)
                results.append(out)
        assert all(torch.equal(results[0], r) for r in results[1:])
    finally:
        patch(8, 8)


def test_gemm_tiles_refuses_what_it_cannot_take():
    x = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(48, 64, dtype=torch.bfloat16, device=DEV)
    tiles = ops.pack_weight_tiles(w)
    with pytest.raises(ops.ShapeError, match="operand tiles"):
        ops.gemm_tiles(x, tiles, 64)                       # tiles of another matrix
    with pytest.raises(ops.ShapeError, match="interleaved"):
        ops.gemm_tiles(x, tiles, 48, epilogue=ops.EPI_SILU_MUL)
    with pytest.raises(ops.ShapeError, match="no variant"):
        ops.gemm_tiles(x, tiles, 48, variant=(3, 3))
    with pytest.raises(ops.ShapeError, match="bfloat16"):
        ops.gemm_tiles(x.float(), tiles, 48)


def test_sum_partials_and_stacked_residual_add():
    parts = torch.randn(5, 7, 88, generator=_g(113))
    want = parts.double().sum(0)
    assert _rel(ops.sum_partials(parts.to(DEV), torch.float32).cpu(), want) < 1e-6
    assert ops.sum_partials(parts.to(DEV), torch.bfloat16).dtype == torch.bfloat16
    for width in (88, 2560, 4100):                  # register-resident kernel, and the general one
        parts = torch.randn(6, 3, width, generator=_g(114))
        res = torch.randn(3, width, generator=_g(115)) * 2.0
        nw = 1.0 + 0.2 * torch.randn(width, generator=_g(116))
        on_gpu = res.clone().to(DEV)
        got = ops.add_rmsnorm(on_gpu, parts.to(DEV), nw.to(DEV), 1e-5, torch.float32).cpu()
        summed = res.double() + parts.double().sum(0)
        assert _rel(on_gpu.cpu(), summed) < 1e-6
        assert _rel(got, plain.rms_norm(summed, nw.double(), 1e-5)) < 1e-5
        # picked rows (the final norm): nothing is written back
        rows = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
        on_gpu = res.clone().to(DEV)
        got = ops.add_rmsnorm(on_gpu, parts.to(DEV), nw.to(DEV), 1e-5, torch.float32, rows=rows).cpu()
        assert torch.equal(on_gpu.cpu(), res)
        assert _rel(got, plain.rms_norm(summed[[2, 0]], nw.double(), 1e-5)) < 1e-5


def test_gemm_rows_refuses_what_it_cannot_take():
    x = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.ShapeError, match="1..64 rows"):
        ops.gemm_rows(x, w)
    with pytest.raises(ops.ShapeError, match="K % 8"):
        ops.gemm_rows(torch.zeros(2, 20, dtype=torch.bfloat16, device=DEV),
                      torch.zeros(4, 20, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ops.ShapeError, match="no variant"):
        ops.gemm_rows(x[:4], w, variant=99, splits=1)
    with pytest.raises(ops.ShapeError, match="even number of column tiles"):
        ops.gemm_rows(x[:4], w, epilogue=ops.EPI_SILU_MUL, variant=2, splits=1)
    with pytest.raises(ops.ShapeError, match="whole sums"):
        ops.gemm_rows(x[:4], w, epilogue=ops.EPI_SILU_MUL, variant=1, splits=2)
    with pytest.raises(ops.ShapeError, match="do not fit into LDS"):
        ops.gemm_rows(torch.zeros(64, 9728, dtype=torch.bfloat16, device=DEV),
                      torch.zeros(32, 9728, dtype=torch.bfloat16, device=DEV), variant=0, splits=2)
    # the general entry point still serves such shapes, through the library
    out = ops.gemm_bf16(torch.ones(2, 20, dtype=torch.bfloat16, device=DEV), torch.ones(4, 20, dtype=torch.bfloat16, device=DEV))
    assert out.shape == (2, 4) and float(out[0, 0]) == 20.0


def test_split_choices_depend_on_shape_and_context_class_only():
    """The split-KV factor of decoded tokens and the key parts of a short portion are functions of the step's shape
    and of the power-of-two class of the longest context, so that a captured step and an eager one choose alike."""
    lengths = (1, 63, 64, 127, 128, 1000, 2048, 4095, 4096, 100000)
    caps = [ops.decode_split_cap(n) for n in lengths]
    assert caps == [1, 1, 1, 2, 2, 16, 32, 64, 64, 64]          # largest power of two <= (blocks of 32 keys) / 2, <= 64
    assert all(c & (c - 1) == 0 for c in caps) and caps == sorted(caps)
    dev = torch.device(DEV)
    args = dict(num_q_heads=32, num_kv_heads=8, head_dim=128, device=dev)
    assert ops.portion_key_splits(2048, 2048, 1, max_kv_len=2048, **args) == 1          # enough row blocks
    few = ops.portion_key_splits(512, 512, 1, max_kv_len=2048, **args)
    assert 2 <= few <= 8 and few == ops.portion_key_splits(512, 512, 1, max_kv_len=3000, **args)
    assert ops.portion_key_splits(128, 128, 1, max_kv_len=200, **args) == 1              # too few keys to cut
    assert ops.portion_key_splits(64, 64, 1, max_kv_len=65536, **args) == 8


def test_measuring_kernels_give_plausible_ceilings():
    """The two kernels behind `bench.py --ceilings`: a read of 256 MB and a short run of matrix-core products
    land between a tenth of the published peaks and the peaks themselves."""
    from arle_amd.kernels import ceilings

    read = ceilings.read_bandwidth(DEV, total_bytes=256 << 20, repeats=2)
    assert 0.8e12 < read["best"] < 8.0e12 and set(read["by_workgroups"]) and read["launches"] == 1
    parts = ceilings.read_bandwidth(DEV, total_bytes=256 << 20, launches=4, repeats=2)
    assert 0.5e12 < parts["best"] < 8.0e12
    for shape in (16, 32):
        for random_operands in (False, True):
            rate = ceilings.mfma_rate(DEV, shape=shape, iters=2000, repeats=1, random_operands=random_operands)
            assert 2.5e14 < rate < 2.6e15


@pytest.mark.parametrize("nq,nkv,D,P,splits", [(32, 8, 128, 16, 3), (4, 2, 16, 4, 1), (6, 2, 64, 8, 2)])
def test_attention_decoded_tokens_on_a_side_branch_give_the_bits_of_one_stream(nq, nkv, D, P, splits):
    """In a mixed step the split-KV kernel of the decoded tokens and its merge run on a second stream beside the
    portions kernel (forked and joined by events).  With the branch and without it the result is the same bit for
    bit and right; a graph captured with the branch in it gives the same again on every replay, with eager calls
    and synchronisations between the replays."""
    from arle_amd.kernels import lib
    segs = [(300, 70), (45, 1), (0, 1), (130, 2), (0, 200), (77, 1), (511, 1)]
    results = {}
    try:
        for side in (0, 1):
            lib.function("arle_attn_side_branch")(side)
            results[side], want = _mfma_case(nq, nkv, D, P, segs, 0, splits, 410)
        assert torch.isfinite(results[1]).all() and _rel(results[1], want) < 8e-3
        assert torch.equal(results[0], results[1])

        # the same call captured with the branch in it
        dt = torch.bfloat16
        lengths = [a + b for a, b in segs]
        table, k_pages, v_pages = _paged_setup(lengths, nkv, D, P, dt, 410)
        qs, row0, starts = [], [0], []
        for s, (cached, n) in enumerate(segs):
            g = _g(411 + s)
            q, k, v = (torch.randn(cached + n, h, D, generator=g).to(dt) for h in (nq, nkv, nkv))
            _fill_cache(table, k_pages, v_pages, s, k, v, P)
            qs.append(q[cached:].reshape(n, nq * D))
            row0.append(row0[-1] + n)
            starts.append(cached)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        q_all, out = torch.cat(qs).to(DEV), None
        fixed = (k_pages.to(DEV), v_pages.to(DEV), table.to(DEV), i32(row0), i32(list(range(len(segs)))), i32(starts))
        kw = dict(max_qlen=200, min_qlen=1, max_kv_len=max(lengths), num_q_heads=nq, num_kv_heads=nkv, head_dim=D,
                  page_size=P, scale=1.0 / math.sqrt(D), splits=splits)
        eager = torch.empty_like(q_all)
        ops.attn_paged_mfma(q_all, eager, *fixed, **kw)          # also makes the side stream, outside the capture
        torch.cuda.synchronize()
        assert torch.equal(eager.cpu(), results[1])
        captured = torch.empty_like(q_all)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            ops.attn_paged_mfma(q_all, captured, *fixed, **kw)
        for rep in range(4):
            captured.fill_(float("nan"))
            graph.replay()
            again = torch.empty_like(q_all)
            ops.attn_paged_mfma(q_all, again, *fixed, **kw)      # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(captured, eager) and torch.equal(again, eager), rep
    finally:
        lib.function("arle_attn_side_branch")(1)
