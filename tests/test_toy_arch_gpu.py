"""A toy architecture defined here, in the test, and registered without touching the framework:
a mixer with state of its own, attention layers with and without a window, a layer that the
schedule names twice, and a layer that reads another layer's cache.  It never becomes a model of
anyone's; it shows that parts, cache manager, step function and loader are architecture-blind."""
import json
import os
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd.cache import StateNeed
from arle_amd.config import register_architecture
from arle_amd.engine import Engine
from arle_amd.parts import LayerSpec, ModelSpec, Part, PartSpec, ScheduleEntry, WeightDecl, register
from arle_amd.weights import write_random_model
from tiny import random_tokens, read_folder

pytestmark = pytest.mark.gpu


@register("mixer", "toy_decay")
class DecayMixer(Part):
    """s_t = decay * s_{t-1} + W_in x_t;  y_t = W_out s_t.  The state s [width] lives in the
    request's fixed-size slot; rows of one request are consumed in order."""

    @classmethod
    def declare_weights(cls, params):
        return {"w_in": WeightDecl((params["state"], params["hidden_size"])),
                "w_out": WeightDecl((params["hidden_size"], params["state"]))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.w_in, self.w_out = tensors["w_in"].float(), tensors["w_out"].float()
        self.decay, self.width = float(params["decay"]), int(params["state"])

    def cache_need(self):
        return StateNeed((self.width,), torch.float32)

    def forward(self, x, batch, cache):
        u = x.float() @ self.w_in.T
        states = torch.empty_like(u)
        for seg in batch.segments:
            s = cache.state[seg.slot]
            for i in range(seg.row0, seg.row0 + seg.length):
                s = self.decay * s + u[i]
                states[i] = s
            cache.state[seg.slot] = s
        return (states @ self.w_out.T).to(x.dtype)


@dataclass(frozen=True)
class ToyConfig:
    hidden_size: int
    intermediate_size: int
    state: int
    decay: float
    heads: int
    kv_heads: int
    head_dim: int
    window: int
    vocab_size: int
    eps: float
    theta: float
    max_position_embeddings: int = 512

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyStateLM"])


def toy_spec(c: ToyConfig, stop_token_ids=()):
    norm = lambda name: PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.eps}, {"weight": name})
    ffn = lambda p: PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size},
                             {"gate": p + "ffn.gate", "up": p + "ffn.up", "down": p + "ffn.down"})

    def attention(p, window):
        pos = PartSpec("rope_neox", {"head_dim": c.head_dim, "theta": c.theta, "max_positions": c.max_position_embeddings})
        return PartSpec("paged_attention",
                        {"hidden_size": c.hidden_size, "num_q_heads": c.heads, "num_kv_heads": c.kv_heads,
                         "head_dim": c.head_dim, "qk_norm": True, "eps": c.eps, "position": pos, "window": window},
                        {"q": p + "attn.q", "k": p + "attn.k", "v": p + "attn.v", "o": p + "attn.o",
                         "q_norm": p + "attn.q_norm", "k_norm": p + "attn.k_norm"})

    mixers = [PartSpec("toy_decay", {"hidden_size": c.hidden_size, "state": c.state, "decay": c.decay},
                       {"w_in": "l0.mix.w_in", "w_out": "l0.mix.w_out"}),
              attention("l1.", c.window), attention("l2.", None)]
    layers = [LayerSpec("pre_norm", m, ffn(f"l{i}."), {"mixer_in": norm(f"l{i}.n1"), "ffn_in": norm(f"l{i}.n2")})
              for i, m in enumerate(mixers)]
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    # state layer, windowed attention, full attention, the windowed layer again (own cache),
    # and the full-attention layer once more, reading the cache its first run wrote
    schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(1), ScheduleEntry(2, cache_from=2)]
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_positions=c.max_position_embeddings,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}), layers=layers, schedule=schedule,
                     final_norm=norm("final_norm"), head=PartSpec("linear", sizes, {"weight": "head"}),
                     stop_token_ids=tuple(stop_token_ids))


register_architecture("ToyStateLM", ToyConfig, toy_spec)

TOY = ToyConfig(hidden_size=48, intermediate_size=80, state=24, decay=0.8, heads=4, kv_heads=2, head_dim=16,
                window=6, vocab_size=120, eps=1e-5, theta=10000.0)


def toy_plain_logits(c: ToyConfig, w, tokens):
    """Whole sequence, no cache, from the plain parts."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    h = plain.embedding(w["embed"], tokens)
    cos, sin = plain.rope_cos_sin(range(T), c.head_dim, c.theta, dtype=torch.float64)
    kv_of_entry = {}
    for entry, (layer, cache_from) in enumerate([(0, None), (1, None), (2, None), (1, None), (2, 2)]):
        p = f"l{layer}."
        a = plain.rms_norm(h, w[p + "n1"], c.eps)
        if layer == 0:
            s = torch.zeros(c.state, dtype=torch.float64)
            rows = []
            for t in range(T):
                s = c.decay * s + w["l0.mix.w_in"] @ a[t]
                rows.append(w["l0.mix.w_out"] @ s)
            m = torch.stack(rows)
        else:
            q = plain.linear(a, w[p + "attn.q"]).reshape(T, c.heads, c.head_dim)
            q = plain.apply_rope(plain.qk_norm(q, w[p + "attn.q_norm"], c.eps), cos, sin)
            if cache_from is None:
                k = plain.linear(a, w[p + "attn.k"]).reshape(T, c.kv_heads, c.head_dim)
                k = plain.apply_rope(plain.qk_norm(k, w[p + "attn.k_norm"], c.eps), cos, sin)
                v = plain.linear(a, w[p + "attn.v"]).reshape(T, c.kv_heads, c.head_dim)
                kv_of_entry[entry] = (k, v)
            else:
                k, v = kv_of_entry[cache_from]
            window = c.window if layer == 1 else None
            att = plain.causal_attention(q, k, v, c.kv_heads, window=window).reshape(T, -1)
            m = plain.linear(att, w[p + "attn.o"])
        h = h + m
        b = plain.rms_norm(h, w[p + "n2"], c.eps)
        h = h + plain.swiglu_mlp(b, w[p + "ffn.gate"], w[p + "ffn.up"], w[p + "ffn.down"])
    return plain.linear(plain.rms_norm(h, w["final_norm"], c.eps), w["head"])


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("toy") / "toy")
    write_random_model(d, "ToyStateLM", TOY, seed=3, std=0.08, norm_std=0.05)
    return d


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2.5e-2)])
def test_toy_architecture_is_built_and_stepped(toy_folder, dtype, tol):
    _, weights = read_folder(toy_folder)
    eng = Engine.from_folder(toy_folder, dtype=dtype, page_size=4, max_tokens=4 * 64, max_slots=4)
    # groups: the two windowed entries share pages; the full-attention entry has its own; one state need
    assert len(eng.cache.groups) == 2 and len(eng.cache.state_buffers) == 1
    reqs = {f"t{i}": random_tokens(n, TOY.vocab_size, 40 + i) for i, n in enumerate([30, 52, 17, 44, 25])}
    got = replay.run_steps(eng, replay.mixed(reqs, max_live=4, seed=2))
    worst = 0.0
    for rid, toks in reqs.items():
        ref = toy_plain_logits(TOY, weights, toks)
        for p in range(len(toks)):
            err = float((got[(rid, p)].double() - ref[p]).abs().max() / ref.abs().max())
            worst = max(worst, err)
            assert err <= tol, f"{dtype}: request {rid} position {p}: {err:.3e}"
    # the windowed group gave pages back while requests ran; everything is free at the end
    assert all(f == g.pool.num_pages for f, g in zip(eng.cache.free_pages(), eng.cache.groups))


def test_windowed_group_needs_fewer_pages(toy_folder):
    eng = Engine.from_folder(toy_folder, dtype="float32", page_size=4, max_tokens=64, max_slots=2)
    toks = random_tokens(60, TOY.vocab_size, 1)
    replay.run_steps(eng, [{"entries": [("a", toks[i:i + 5], [])], "end": []} for i in range(0, 60, 5)])
    windowed = [g for g in eng.cache.groups if g.window][0]
    full = [g for g in eng.cache.groups if not g.window][0]
    assert full.pool.num_pages - full.pool.free_count == 15
    assert windowed.pool.num_pages - windowed.pool.free_count <= 3


def test_a_failed_step_leaves_state_slots_and_pages_as_they_were(toy_folder):
    """A step that fails after its mixers ran must not leave a request with the state of tokens it does not
    hold: the state blocks of the step's slots are put back, like the lengths and pages."""
    _, weights = read_folder(toy_folder)
    eng = Engine.from_folder(toy_folder, dtype="float32", page_size=4, max_tokens=256, max_slots=2, cuda_graph=False)
    toks = random_tokens(21, TOY.vocab_size, 8)
    other = random_tokens(9, TOY.vocab_size, 9)
    eng.add_request("a")
    eng.add_request("b")
    eng.step([("a", toks[:8], []), ("b", other[:4], [])])
    state_before = {e: buf.clone() for e, buf in eng.cache.state_buffers.items()}
    free_before, len_before = eng.cache.free_pages(), (eng.length("a"), eng.length("b"))
    real_forward = eng.model.forward

    def forward_then_fail(batch, cache):
        real_forward(batch, cache)          # every mixer has run: the state blocks are overwritten
        torch.cuda.synchronize()
        raise RuntimeError("planted failure after the layers")

    eng.model.forward = forward_then_fail
    with pytest.raises(RuntimeError, match="planted"):
        eng.step([("a", toks[8:15], [6]), ("b", other[4:6], [])])
    eng.model.forward = real_forward
    assert (eng.length("a"), eng.length("b")) == len_before and eng.cache.free_pages() == free_before
    for e, buf in eng.cache.state_buffers.items():
        assert torch.equal(buf, state_before[e])
    # the requests go on as if nothing had happened
    got = eng.step([("a", toks[8:], list(range(13))), ("b", other[4:], [4])])
    ref = toy_plain_logits(TOY, weights, toks)
    assert float((got[:13].cpu().double() - ref[8:]).abs().max() / ref.abs().max()) <= 1e-5
    ref_b = toy_plain_logits(TOY, weights, other)
    assert float((got[13].cpu().double() - ref_b[8]).abs().max() / ref_b.abs().max()) <= 1e-5
