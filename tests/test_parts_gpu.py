"""Each part alone, built from a PartSpec as a model would build it, against its plain function."""
import math

import pytest
import torch

import plain_qwen3 as plain
from arle_amd.cache import CacheManager
from arle_amd.engine.batch import StepEntry, build_step_batch
from arle_amd.models import decoder  # noqa: F401  (registers the stock parts)
from arle_amd.parts import PartSpec, Runtime, build_part, lookup

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _rt(dtype):
    return Runtime(device=DEV, act_dtype=dtype)


def _rel(a, b):
    return float((a.double().cpu() - b.double()).abs().max() / b.double().abs().max())


def _delta(d):
    """What a mixer or feed-forward hands to the residual add: [T, H], or a float32 stack to be summed."""
    return d.double().sum(0) if d.dim() == 3 else d


def _tensors(shapes, dtype, seed=0, scale=0.2):
    g = torch.Generator().manual_seed(seed)
    return {k: (torch.randn(*s, generator=g) * scale + (1.0 if len(s) == 1 else 0.0)).to(dtype) for k, s in shapes.items()}


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
def test_norm_part(dtype, tol):
    w = _tensors({"n.weight": (88,)}, dtype)
    part = build_part("norm", PartSpec("rmsnorm", {"width": 88, "eps": 3e-6}, {"weight": "n.weight"}),
                      lambda n: w[n].to(DEV), _rt(dtype))
    x = torch.randn(5, 88)
    assert _rel(part.forward(x.to(DEV)), plain.rms_norm(x.double(), w["n.weight"].double(), 3e-6)) < tol
    delta = torch.randn(5, 88).to(dtype)
    res = x.clone().to(DEV)
    got = part.add_norm(res, delta.to(DEV))
    assert _rel(got, plain.rms_norm(x.double() + delta.double(), w["n.weight"].double(), 3e-6)) < tol
    assert _rel(res, x.double() + delta.double()) < 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1e-2)])
def test_feed_forward_part(dtype, tol):
    w = _tensors({"g": (136, 88), "u": (136, 88), "d": (88, 136)}, dtype)
    part = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": 88, "intermediate_size": 136},
                                               {"gate": "g", "up": "u", "down": "d"}), lambda n: w[n].to(DEV), _rt(dtype))
    x = torch.randn(7, 88).to(dtype)
    want = plain.swiglu_mlp(x.double(), w["g"].double(), w["u"].double(), w["d"].double())
    assert _rel(_delta(part.forward(x.to(DEV))), want) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(dtype):
    w = _tensors({"e": (333, 88)}, dtype)
    sizes = {"vocab_size": 333, "hidden_size": 88}
    fetch = lambda n: w[n].to(DEV)
    emb = build_part("embedding", PartSpec("token_table", sizes, {"table": "e"}), fetch, _rt(dtype))
    head = build_part("head", PartSpec("linear", sizes, {"weight": "e"}), fetch, _rt(dtype))
    ids = torch.tensor([3, 332, 0], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(ids).cpu(), w["e"].float()[[3, 332, 0]])
    x = torch.randn(4, 88).to(dtype)
    logits = head.forward(x.to(DEV))
    assert logits.dtype == torch.float32
    assert _rel(logits, plain.linear(x.double(), w["e"].double())) < (2e-6 if dtype == torch.float32 else 2e-3)


def test_position_part_alone_equals_plain_rope():
    part = build_part("position", PartSpec("rope_neox", {"head_dim": 48, "theta": 5e4, "max_positions": 64}),
                      lambda n: None, _rt(torch.float32))
    q, k = torch.randn(5, 3 * 48), torch.randn(5, 1 * 48)
    pos = torch.tensor([0, 1, 7, 33, 63], dtype=torch.int32)
    dq, dk = q.clone().to(DEV), k.clone().to(DEV)
    part.apply(dq, dk, pos.to(DEV), 3, 1)
    cos, sin = plain.rope_cos_sin(pos.tolist(), 48, 5e4, dtype=torch.float64)
    assert _rel(dq, plain.apply_rope(q.double().reshape(5, 3, 48), cos, sin).reshape(5, -1)) < 2e-6
    assert _rel(dk, plain.apply_rope(k.double().reshape(5, 1, 48), cos, sin).reshape(5, -1)) < 2e-6
    part.ensure_positions(200)       # the table grows when a request runs past it
    assert part.cos.shape[0] >= 200


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-6), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("window", [None, 9])
def test_attention_part_over_its_cache(dtype, tol, window):
    H, nq, nkv, D, P, eps, theta = 88, 6, 2, 32, 8, 1e-5, 1e4
    w = _tensors({"q": (nq * D, H), "k": (nkv * D, H), "v": (nkv * D, H), "o": (H, nq * D), "qn": (D,), "kn": (D,)}, dtype)
    pos_spec = PartSpec("rope_neox", {"head_dim": D, "theta": theta, "max_positions": 128})
    spec = PartSpec("paged_attention",
                    {"hidden_size": H, "num_q_heads": nq, "num_kv_heads": nkv, "head_dim": D, "qk_norm": True,
                     "eps": eps, "position": pos_spec, "window": window},
                    {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "qn", "k_norm": "kn"})
    part = build_part("mixer", spec, lambda n: w[n].to(DEV), _rt(dtype))
    cache = CacheManager([part.cache_need()], page_size=P, num_pages=16, max_slots=2, max_request_tokens=64,
                         device=DEV, dtype=dtype)
    T = 37
    x = torch.randn(T, H).to(dtype)
    cache.admit("r")
    outs = []
    for lo, hi in ((0, 20), (20, 21), (21, 37)):      # a portion, one decoded token, another portion
        batch = build_step_batch([StepEntry("r", [0] * (hi - lo), [])], cache.slot_of.__getitem__, cache.length, 10, DEV)
        cache.append([("r", hi - lo)])
        cache.sync_tables()
        outs.append(_delta(part.forward(x[lo:hi].to(DEV), batch, cache.view(0))).double())
        cache.trim_windows("r")
    got = torch.cat(outs)
    wd = {k: v.double() for k, v in w.items()}
    xd = x.double()
    q = plain.qk_norm(plain.linear(xd, wd["q"]).reshape(T, nq, D), wd["qn"], eps)
    k = plain.qk_norm(plain.linear(xd, wd["k"]).reshape(T, nkv, D), wd["kn"], eps)
    v = plain.linear(xd, wd["v"]).reshape(T, nkv, D)
    cos, sin = plain.rope_cos_sin(range(T), D, theta, dtype=torch.float64)
    att = plain.causal_attention(plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin), v, nkv, window=window)
    assert _rel(got, plain.linear(att.reshape(T, -1), wd["o"])) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-6), (torch.bfloat16, 2e-2)])
def test_block_part_alone_equals_a_plain_decoder_layer(dtype, tol):
    """One pre-norm block built from the recipe of a tiny configuration: residual and pending delta in,
    residual and pending delta out, over a portion of 20 rows, a single row and a portion of 6."""
    from arle_amd.config import Qwen3Config
    from arle_amd.models.qwen3 import qwen3_spec
    from arle_amd.parts import lookup as lookup_part
    from tiny import TINY_C

    cfg = dict(TINY_C, num_hidden_layers=1)
    layer = qwen3_spec(Qwen3Config.from_dict(cfg)).layers[0]
    names = {**layer.mixer.weights, **layer.feed_forward.weights, "n1": layer.norms["mixer_in"].weights["weight"],
             "n2": layer.norms["ffn_in"].weights["weight"]}
    H, nq, nkv, D, I = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["intermediate_size"]
    shapes = {names["q"]: (nq * D, H), names["k"]: (nkv * D, H), names["v"]: (nkv * D, H), names["o"]: (H, nq * D),
              names["q_norm"]: (D,), names["k_norm"]: (D,), names["gate"]: (I, H), names["up"]: (I, H),
              names["down"]: (H, I), names["n1"]: (H,), names["n2"]: (H,)}
    w = _tensors(shapes, dtype, seed=9, scale=0.1)
    fetch = lambda n: w[n].to(DEV)
    rt = _rt(dtype)
    mixer = build_part("mixer", layer.mixer, fetch, rt)
    ffn = build_part("feed_forward", layer.feed_forward, fetch, rt)
    norms = {role: build_part("norm", spec, fetch, rt) for role, spec in layer.norms.items()}
    block = lookup_part("block", layer.block)(mixer, ffn, norms)
    cache = CacheManager([mixer.cache_need()], page_size=16, num_pages=8, max_slots=2, max_request_tokens=64,
                         device=DEV, dtype=dtype)
    T = 27
    h0 = torch.randn(T, H)
    pending = (torch.randn(T, H) * 0.3).to(dtype)     # what the block before this one has not added yet
    cache.admit("r")
    out_rows = []
    for lo, hi in ((0, 20), (20, 21), (21, 27)):
        batch = build_step_batch([StepEntry("r", [0] * (hi - lo), [])], cache.slot_of.__getitem__, cache.length, 10, DEV)
        cache.append([("r", hi - lo)])
        cache.sync_tables()
        residual, delta = block.forward(h0[lo:hi].clone().to(DEV), pending[lo:hi].to(DEV), batch, cache.view(0))
        out_rows.append(residual.double().cpu() + _delta(delta).double().cpu())
    got = torch.cat(out_rows)
    wd = {k: v.double() for k, v in w.items()}
    qw = {"model.layers.0." + k: wd[v] for k, v in (("self_attn.q_proj.weight", names["q"]), ("self_attn.k_proj.weight", names["k"]),
          ("self_attn.v_proj.weight", names["v"]), ("self_attn.o_proj.weight", names["o"]), ("self_attn.q_norm.weight", names["q_norm"]),
          ("self_attn.k_norm.weight", names["k_norm"]), ("mlp.gate_proj.weight", names["gate"]), ("mlp.up_proj.weight", names["up"]),
          ("mlp.down_proj.weight", names["down"]), ("input_layernorm.weight", names["n1"]),
          ("post_attention_layernorm.weight", names["n2"]))}
    want = plain.decoder_layer(h0.double() + pending.double(), qw, 0, cfg, list(range(T)))
    assert _rel(got, want) < tol


def test_unknown_part_and_bad_head_dim_are_refused():
    with pytest.raises(KeyError, match="no mixer part named 'nope'"):
        lookup("mixer", "nope")
    pos_spec = PartSpec("rope_neox", {"head_dim": 24, "theta": 1e4, "max_positions": 16})
    spec = PartSpec("paged_attention", {"hidden_size": 48, "num_q_heads": 2, "num_kv_heads": 1, "head_dim": 24,
                                        "qk_norm": False, "position": pos_spec},
                    {"q": "q", "k": "k", "v": "v", "o": "o"})
    w = _tensors({"q": (48, 48), "k": (24, 48), "v": (24, 48), "o": (48, 48)}, torch.float32)
    build_part("mixer", spec, lambda n: w[n].to(DEV), _rt(torch.float32))     # float32 takes any head_dim
    wb = {k: v.bfloat16() for k, v in w.items()}
    with pytest.raises(ValueError, match="head_dim 24 is not supported in bfloat16"):
        build_part("mixer", spec, lambda n: wb[n].to(DEV), _rt(torch.bfloat16))
    spec.params["head_dim"] = 1024
    with pytest.raises(ValueError, match="head_dim 1024 is not supported"):
        build_part("mixer", spec, lambda n: w[n].to(DEV), _rt(torch.float32))
