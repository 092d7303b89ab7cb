"""Which kernel runs a matrix product is a choice made in one place (`ops.choose_product`): by a measured table
where one is loaded for the widths, else by the rules.  Whatever a table may name has to be right: every candidate
of a shape is run here against the float64 product, at widths of Qwen3-4B and at awkward ones."""
import json

import pytest
import torch

import plain_qwen3 as plain
from arle_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _g(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("N,K", [(6144, 2560), (2560, 4096), (2560, 9728), (1000, 1096)])
@pytest.mark.parametrize("M", [1, 7, 16, 17, 33, 64, 100, 300])
def test_every_candidate_of_a_plain_product_is_right(M, N, K):
    x = torch.randn(M, K, generator=_g(1)).bfloat16()
    w = (torch.randn(N, K, generator=_g(2)) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    xd, wd = x.to(DEV), w.to(DEV)
    tiles = ops.pack_weight_tiles(wd)
    seen = set()
    for choice in ops.product_candidates(M, N, K, K, tiled=True, fused=False):
        seen.add(choice.kernel)
        stack = ops.run_product(choice, xd, wd, tiles, torch.bfloat16, partials_ok=True)
        if stack.dim() == 3:        # float32 partial products: exact products, float32 sums
            assert stack.dtype == torch.float32 and _rel(stack.double().sum(0).cpu(), want) < 1e-5, choice
        whole = ops.run_product(choice, xd, wd, tiles, torch.bfloat16, partials_ok=False)
        assert whole.shape == (M, N) and whole.dtype == torch.bfloat16 and _rel(whole.cpu(), want) < 6e-3, choice
        whole32 = ops.run_product(choice, xd, wd, tiles, torch.float32, partials_ok=False)
        assert whole32.dtype == torch.float32 and _rel(whole32.cpu(), want) < 6e-3, choice
    assert "library" in seen and (M > 64 or "stream" in seen) and (M > 16 or "rows" in seen)
    assert M <= 32 or "library_parts" in seen or K % 64


@pytest.mark.parametrize("inter,K", [(9728, 2560), (224, 96), (1200, 1096)])
@pytest.mark.parametrize("M", [1, 5, 16, 27, 28, 64, 100, 300])
def test_every_candidate_of_gate_up_with_its_activation_is_right(M, inter, K):
    x = torch.randn(M, K, generator=_g(3)).bfloat16()
    gate = (torch.randn(inter, K, generator=_g(4)) * 0.1).bfloat16()
    up = (torch.randn(inter, K, generator=_g(5)) * 0.1).bfloat16()
    fused = torch.stack([gate.view(-1, 16, K), up.view(-1, 16, K)], dim=1).reshape(2 * inter, K).contiguous().to(DEV)
    want = plain.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    tiles = ops.pack_weight_tiles(fused)
    for choice in ops.product_candidates(M, 2 * inter, K, K, tiled=True, fused=True):
        got = ops.run_product(choice, x.to(DEV), fused, tiles, torch.bfloat16, False, fused=True)
        # the library's product rounds gate and up to bfloat16 before the activation: two roundings more
        tol = 1.2e-2 if choice.kernel == "library" else 6e-3
        assert got.shape == (M, inter) and got.dtype == torch.bfloat16 and _rel(got.cpu(), want) < tol, choice


def test_a_loaded_table_decides_for_its_widths_and_the_rules_for_all_others(tmp_path):
    saved = dict(ops._PRODUCT_TABLE)
    try:
        ops.clear_product_table()
        N, K = 1000, 1096
        by_rule = ops.choose_product(40, N, K, K, tiled=True, fused=False, partials_ok=True)
        assert by_rule == ops.product_by_rules(40, N, K, K, tiled=True, fused=False, partials_ok=True)
        path = tmp_path / "table.json"
        path.write_text(json.dumps({f"{N},{K},0,1": [[16, "rows", [2], 2], [64, "stream", [3], 5], [512, "library_parts", [], 2]]}))
        ops.load_product_table(str(path))
        pick = lambda rows, **kw: ops.choose_product(rows, N, K, kw.pop("stride", K), tiled=kw.pop("tiled", True), fused=False,
                                                     partials_ok=True, **kw)
        assert pick(9) == ops.ProductChoice("rows", (2,), 2) and pick(16).kernel == "rows"
        assert pick(17) == ops.ProductChoice("stream", (3,), 5) and pick(300) == ops.ProductChoice("library_parts", (), 2)
        assert pick(513) == ops.product_by_rules(513, N, K, K, tiled=True, fused=False, partials_ok=True)   # past the table
        assert pick(40, tiled=False) == ops.product_by_rules(40, N, K, K, tiled=False, fused=False, partials_ok=True)
        assert pick(40, aligned=False).kernel == "library" and pick(40, stride=K + 4).kernel == "library"  # off the 16-byte grid
        other = ops.choose_product(40, N + 16, K, K, tiled=True, fused=False, partials_ok=True)                 # other widths
        assert other == ops.product_by_rules(40, N + 16, K, K, tiled=True, fused=False, partials_ok=True)
        # and the product through the general entry point follows the table, with the same result
        x = torch.randn(40, K, generator=_g(6)).bfloat16().to(DEV)
        w = (torch.randn(N, K, generator=_g(7)) * 0.05).bfloat16().to(DEV)
        stack = ops.gemm_bf16(x, w, torch.bfloat16, partials_ok=True, tiles=ops.pack_weight_tiles(w))
        assert stack.dim() == 3 and stack.shape[0] == 5
        assert _rel(stack.double().sum(0).cpu(), x.double().cpu() @ w.double().cpu().T) < 1e-5
        with pytest.raises(ops.ShapeError, match="names the kernel"):
            ops.load_product_table({"8,8,0,0": [[4, "magic", [], 0]]})
    finally:
        ops.clear_product_table()
        ops._PRODUCT_TABLE.update(saved)


def test_an_engine_tunes_the_products_of_its_own_widths(tmp_path):
    """`Engine.tune_products` asks the model's parts for their products, measures them at the row counts given and
    takes the table in; the engine stays right with whatever the table chose, and a second engine reads the file."""
    import replay
    from arle_amd.engine import Engine
    from tiny import TINY, make_model_dir, random_tokens, read_folder

    saved = dict(ops._PRODUCT_TABLE)
    try:
        d = make_model_dir(tmp_path, "D")
        cfg, weights = read_folder(d)
        eng = Engine.from_folder(d, dtype="bfloat16", page_size=TINY["D"][1], max_tokens=4 * 128, max_slots=4)
        path = str(tmp_path / "table.json")
        table = eng.tune_products(rows=(1, 20, 100), path=path)
        h, q, kv, inter, vocab = cfg["hidden_size"], 8 * 64, 2 * 64, cfg["intermediate_size"], cfg["vocab_size"]
        tiled = int(eng.rt.weight_tiles)
        assert set(table) == {f"{q + 2 * kv},{h},0,{tiled}", f"{h},{q},0,{tiled}", f"{2 * inter},{h},{int(inter % 16 == 0)},{tiled}",
                              f"{h},{inter},0,{tiled}", f"{vocab},{h},0,{tiled}"}
        assert all(rows[-1][0] == 100 for rows in table.values())
        assert (h, inter, False, bool(tiled)) in ops._PRODUCT_TABLE
        reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 70 + i) for i, n in enumerate([40, 90, 23])}
        got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=5))
        replay.compare(got, cfg, weights, reqs, 2e-2, "tuned engine/bfloat16")
        ops.clear_product_table()
        other = Engine.from_folder(d, dtype="bfloat16", page_size=TINY["D"][1], max_tokens=4 * 128, max_slots=4, product_table=path)
        assert (h, inter, False, bool(tiled)) in ops._PRODUCT_TABLE
        got = replay.run_steps(other, replay.whole("w", reqs["r1"]))
        replay.compare(got, cfg, weights, {"w": reqs["r1"]}, 2e-2, "engine with a table from a file/bfloat16")
    finally:
        ops.clear_product_table()
        ops._PRODUCT_TABLE.update(saved)
