"""Toy parts of every other role, defined here and registered without touching the framework:
a feed-forward with routing (top-1 of a few experts), a position encoding the fused kernels do not
know (adjacent-pair rotation with a learned angle table), a norm with a bias, and a block that runs
mixer and feed-forward side by side.  Built from torch operations: they show the interfaces, they
are nobody's model.  The attention layers around them are the stock part, so this also drives its
path for position encodings that are applied between the norm and the cache write."""
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd.config import register_architecture
from arle_amd.engine import Engine
from arle_amd.parts import LayerSpec, ModelSpec, Part, PartSpec, ScheduleEntry, WeightDecl, register
from arle_amd.weights import write_random_model
from tiny import random_tokens, read_folder

pytestmark = pytest.mark.gpu


def _whole(delta):
    """A delta as one tensor: stock parts may hand over a stack of partial sums."""
    return delta.float().sum(0) if delta.dim() == 3 else delta.float()


@register("norm", "toy_biased")
class BiasedNorm(Part):
    """(x - mean) / sqrt(var + eps) * w + b."""

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"],), init="ones"), "bias": WeightDecl((params["width"],))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.w, self.b, self.eps = tensors["weight"].float(), tensors["bias"].float(), float(params["eps"])

    def forward(self, x, rows=None):
        x = x.float() if rows is None else x.float()[rows.long()]
        mu = x.mean(-1, keepdim=True)
        var = (x - mu).pow(2).mean(-1, keepdim=True)
        return ((x - mu) / torch.sqrt(var + self.eps) * self.w + self.b).to(self.rt.act_dtype)

    def add_norm(self, residual, delta, rows=None):
        if delta is not None:
            if rows is None:
                residual += _whole(delta)
            else:
                return self.forward(residual + _whole(delta), rows)
        return self.forward(residual, rows)


@register("position", "toy_pairs")
class PairRotation(Part):
    """Rotates the adjacent pairs (2i, 2i+1) of every head by angle[position, i], a learned table."""

    fusable = False

    @classmethod
    def declare_weights(cls, params):
        return {"angle": WeightDecl((params["max_positions"], params["head_dim"] // 2))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.angle, self.D = tensors["angle"].float(), int(params["head_dim"])

    def ensure_positions(self, n):
        assert n <= self.angle.shape[0], "the learned table is as long as it is"

    def fused_rotary(self):
        return None, None, 0

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        a = self.angle[positions.long()]                     # [T, D/2]
        cos, sin = a.cos()[:, None, :], a.sin()[:, None, :]
        for x, heads in ((q, num_q_heads), (k, num_kv_heads)):
            if heads == 0:
                continue
            v = x.float().reshape(x.shape[0], heads, self.D // 2, 2)
            even, odd = v[..., 0], v[..., 1]
            out = torch.stack([even * cos - odd * sin, even * sin + odd * cos], dim=-1)
            x.copy_(out.reshape(x.shape[0], heads * self.D).to(x.dtype))


@register("feed_forward", "toy_routed")
class RoutedFFN(Part):
    """Every row goes to the one expert with the largest router logit: relu(x W1_e^T) W2_e^T, scaled by the
    softmax weight of that expert.  Router logits and softmax in float32."""

    @classmethod
    def declare_weights(cls, params):
        e, h, i = params["experts"], params["hidden_size"], params["intermediate_size"]
        return {"router": WeightDecl((e, h)), "w1": WeightDecl((e * i, h)), "w2": WeightDecl((e * h, i))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        e, h, i = params["experts"], params["hidden_size"], params["intermediate_size"]
        self.router = tensors["router"].float()
        self.w1, self.w2 = tensors["w1"].float().reshape(e, i, h), tensors["w2"].float().reshape(e, h, i)

    def forward(self, x):
        xf = x.float()
        probs = torch.softmax(xf @ self.router.T, dim=-1)
        weight, expert = probs.max(dim=-1)
        hidden = torch.relu(torch.einsum("th,tih->ti", xf, self.w1[expert]))
        return (torch.einsum("ti,thi->th", hidden, self.w2[expert]) * weight[:, None]).to(x.dtype)


@register("block", "toy_parallel")
class ParallelBlock:
    """h += mixer(norm(h)) + feed_forward(norm(h)): one norm, both branches read it."""

    norm_roles = ("in",)

    def __init__(self, mixer, feed_forward, norms):
        self.mixer, self.feed_forward, self.norm = mixer, feed_forward, norms["in"]

    def forward(self, residual, delta, batch, cache_view):
        a = self.norm.add_norm(residual, delta)
        m = _whole(self.mixer.forward(a, batch, cache_view))
        f = _whole(self.feed_forward.forward(a))
        return residual, m + f


@dataclass(frozen=True)
class ToyPartsConfig:
    hidden_size: int
    intermediate_size: int
    experts: int
    heads: int
    kv_heads: int
    head_dim: int
    vocab_size: int
    eps: float
    layers: int
    max_position_embeddings: int = 128

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyPartsLM"])


def toy_parts_spec(c: ToyPartsConfig, stop_token_ids=()):
    def norm(name):
        return PartSpec("toy_biased", {"width": c.hidden_size, "eps": c.eps}, {"weight": name + ".w", "bias": name + ".b"})

    layers = []
    for i in range(c.layers):
        p = f"l{i}."
        pos = PartSpec("toy_pairs", {"head_dim": c.head_dim, "max_positions": c.max_position_embeddings},
                       {"angle": p + "angle"})
        mixer = PartSpec("paged_attention",
                         {"hidden_size": c.hidden_size, "num_q_heads": c.heads, "num_kv_heads": c.kv_heads,
                          "head_dim": c.head_dim, "qk_norm": i % 2 == 0, "eps": c.eps, "position": pos, "window": None},
                         dict({"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"},
                              **({"q_norm": p + "qn", "k_norm": p + "kn"} if i % 2 == 0 else {})))
        ffn = PartSpec("toy_routed", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size,
                                      "experts": c.experts}, {"router": p + "router", "w1": p + "w1", "w2": p + "w2"})
        layers.append(LayerSpec("toy_parallel", mixer, ffn, {"in": norm(p + "n")}))
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    # the last entry runs layer 0 again on the cache that its first run wrote (only q is projected there)
    schedule = [ScheduleEntry(i) for i in range(c.layers)] + [ScheduleEntry(0, cache_from=0)]
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_positions=c.max_position_embeddings,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}), layers=layers, schedule=schedule,
                     final_norm=norm("final"), head=PartSpec("linear", sizes, {"weight": "head"}),
                     stop_token_ids=tuple(stop_token_ids))


register_architecture("ToyPartsLM", ToyPartsConfig, toy_parts_spec)

TOY = ToyPartsConfig(hidden_size=40, intermediate_size=24, experts=3, heads=3, kv_heads=1, head_dim=16,
                     vocab_size=90, eps=1e-5, layers=2)


def _biased_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt((x - mu).pow(2).mean(-1, keepdim=True) + eps) * w + b


def _pair_rotate(x, angle):
    """x [T, heads, D], angle [T, D/2]."""
    T, H, D = x.shape
    v = x.reshape(T, H, D // 2, 2)
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    return torch.stack([v[..., 0] * c - v[..., 1] * s, v[..., 0] * s + v[..., 1] * c], dim=-1).reshape(T, H, D)


def toy_parts_plain_logits(c: ToyPartsConfig, w, tokens):
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    h = plain.embedding(w["embed"], tokens)
    kv0 = None
    for entry, layer in enumerate(list(range(c.layers)) + [0]):
        p = f"l{layer}."
        a = _biased_norm(h, w[p + "n.w"], w[p + "n.b"], c.eps)
        angle = w[p + "angle"][:T]
        q = plain.linear(a, w[p + "q"]).reshape(T, c.heads, c.head_dim)
        if layer % 2 == 0:
            q = plain.qk_norm(q, w[p + "qn"], c.eps)
        q = _pair_rotate(q, angle)
        if entry < c.layers:
            k = plain.linear(a, w[p + "k"]).reshape(T, c.kv_heads, c.head_dim)
            if layer % 2 == 0:
                k = plain.qk_norm(k, w[p + "kn"], c.eps)
            k = _pair_rotate(k, angle)
            v = plain.linear(a, w[p + "v"]).reshape(T, c.kv_heads, c.head_dim)
            if layer == 0:
                kv0 = (k, v)
        else:
            k, v = kv0
        m = plain.linear(plain.causal_attention(q, k, v, c.kv_heads).reshape(T, -1), w[p + "o"])
        probs = torch.softmax(a @ w[p + "router"].T, dim=-1)
        weight, expert = probs.max(dim=-1)
        w1 = w[p + "w1"].reshape(c.experts, c.intermediate_size, c.hidden_size)
        w2 = w[p + "w2"].reshape(c.experts, c.hidden_size, c.intermediate_size)
        f = torch.stack([w2[e] @ torch.relu(w1[e] @ a[t]) * weight[t] for t, e in enumerate(expert.tolist())])
        h = h + m + f
    return plain.linear(_biased_norm(h, w["final.w"], w["final.b"], c.eps), w["head"])


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("toyparts") / "toy")
    write_random_model(d, "ToyPartsLM", TOY, seed=5, std=0.15, norm_std=0.05)
    return d


def test_toy_parts_are_built_and_stepped(folder):
    """float32: the routed feed-forward switches experts on tiny differences, so only the 32-bit path is
    compared row by row."""
    _, weights = read_folder(folder)
    eng = Engine.from_folder(folder, dtype="float32", page_size=4, max_tokens=4 * 64, max_slots=4)
    reqs = {f"t{i}": random_tokens(n, TOY.vocab_size, 70 + i) for i, n in enumerate([23, 40, 9, 31])}
    got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=4))
    for rid, toks in reqs.items():
        ref = toy_parts_plain_logits(TOY, weights, toks)
        for pos in range(len(toks)):
            err = float((got[(rid, pos)].double() - ref[pos]).abs().max() / ref.abs().max())
            assert err <= 2e-5, f"request {rid} position {pos}: {err:.3e}"
    assert all(f == g.pool.num_pages for f, g in zip(eng.cache.free_pages(), eng.cache.groups))


def test_toy_parts_run_in_bfloat16_too(folder):
    """The stock attention, cache and kernels under the toy parts in bfloat16: finite logits of the right shape,
    equal however the prompt is cut wherever the routing is the same (rounding may flip an expert, so rows are
    compared by their best token against the float32 engine, with most of them required to agree)."""
    toks = random_tokens(36, TOY.vocab_size, 91)
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype=dtype, page_size=4, max_tokens=64, max_slots=2)
        got = replay.run_steps(eng, replay.portions("x", toks, sizes=(5, 1, 9, 2)))
        rows = torch.stack([got[("x", p)] for p in range(len(toks))])
        assert torch.isfinite(rows).all() and rows.shape == (len(toks), TOY.vocab_size)
        outs[dtype] = rows
    agree = (outs["float32"].argmax(-1) == outs["bfloat16"].argmax(-1)).float().mean()
    assert float(agree) >= 0.8


# ---- a mixer whose paged cache is not keys and values ---------------------------------------------------------

from arle_amd.cache import PAGE, PagedNeed, PageTensor  # noqa: E402


@register("mixer", "toy_latent_mean")
class LatentMean(Part):
    """Caches one compressed float32 vector per token, c_t = W_down x_t (in a tensor of its own, float32 even in a
    bfloat16 engine, beside a one-byte tag per token), and returns W_up applied to the mean of c_0..c_t."""

    @classmethod
    def declare_weights(cls, params):
        return {"down": WeightDecl((params["latent"], params["hidden_size"])),
                "up": WeightDecl((params["hidden_size"], params["latent"]))}

    @classmethod
    def declare_cache(cls, params):
        return PagedNeed(tensors=(PageTensor("latent", (PAGE, int(params["latent"])), torch.float32),
                                  PageTensor("tag", (PAGE,), torch.uint8)))

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.down, self.up = tensors["down"].float(), tensors["up"].float()

    def cache_need(self):
        return self.declare_cache(self.params)

    def forward(self, x, batch, cache):
        c = x.float() @ self.down.T
        latent, tag, P = cache.pages["latent"], cache.pages["tag"], cache.page_size
        assert latent.dtype == torch.float32 and tag.dtype == torch.uint8
        out = torch.empty_like(c)
        for seg in batch.segments:
            table = cache.block_table[seg.slot].long()
            pos = torch.arange(seg.start, seg.start + seg.length, device=x.device)
            latent[table[pos // P], pos % P] = c[seg.row0:seg.row0 + seg.length]
            tag[table[pos // P], pos % P] = 1
            every = torch.arange(0, seg.start + seg.length, device=x.device)
            assert bool((tag[table[every // P], every % P] == 1).all())      # every earlier token was written
            sums = latent[table[every // P], every % P].cumsum(0)[seg.start:]
            out[seg.row0:seg.row0 + seg.length] = sums / (pos + 1).float()[:, None]
        return (out @ self.up.T).to(x.dtype)


@dataclass(frozen=True)
class LatentConfig:
    hidden_size: int
    intermediate_size: int
    latent: int
    vocab_size: int
    eps: float
    max_position_embeddings: int = 256

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyLatentLM"])


def latent_spec(c: LatentConfig, stop_token_ids=()):
    norm = lambda name: PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.eps}, {"weight": name})
    layers = [LayerSpec("pre_norm",
                        PartSpec("toy_latent_mean", {"hidden_size": c.hidden_size, "latent": c.latent},
                                 {"down": f"l{i}.down", "up": f"l{i}.up"}),
                        PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size},
                                 {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                        {"mixer_in": norm(f"l{i}.n1"), "ffn_in": norm(f"l{i}.n2")}) for i in range(2)]
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_positions=c.max_position_embeddings,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}), layers=layers,
                     schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn"),
                     head=PartSpec("linear", sizes, {"weight": "embed"}), stop_token_ids=tuple(stop_token_ids))


register_architecture("ToyLatentLM", LatentConfig, latent_spec)
LATENT = LatentConfig(hidden_size=40, intermediate_size=72, latent=12, vocab_size=90, eps=1e-5)


def latent_plain_logits(c, w, tokens):
    w = {k: v.double() for k, v in w.items()}
    h = plain.embedding(w["embed"], tokens)
    for i in range(2):
        a = plain.rms_norm(h, w[f"l{i}.n1"], c.eps)
        lat = a @ w[f"l{i}.down"].T
        mean = lat.cumsum(0) / torch.arange(1, len(tokens) + 1, dtype=torch.float64)[:, None]
        h = h + mean @ w[f"l{i}.up"].T
        b = plain.rms_norm(h, w[f"l{i}.n2"], c.eps)
        h = h + plain.swiglu_mlp(b, w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
    return plain.linear(plain.rms_norm(h, w["fn"], c.eps), w["embed"])


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2.5e-2)])
def test_a_mixer_declares_the_tensors_and_types_of_its_own_paged_cache(tmp_path, dtype, tol):
    d = str(tmp_path / "latent")
    write_random_model(d, "ToyLatentLM", LATENT, seed=5, std=0.1, norm_std=0.05)
    _, weights = read_folder(d)
    eng = Engine.from_folder(d, dtype=dtype, page_size=4, max_tokens=3 * 64, max_slots=4)
    group = eng.cache.page_buffers[0]
    assert set(group) == {"latent", "tag"} and group["latent"].dtype == torch.float32
    assert group["latent"].shape == (2, 48, 4, 12) and group["tag"].shape == (2, 48, 4)
    assert eng.kv_bytes_per_token == 2 * (12 * 4 + 1)
    reqs = {f"q{i}": random_tokens(n, LATENT.vocab_size, 60 + i) for i, n in enumerate([33, 50, 19, 41])}
    got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=4))
    for rid, toks in reqs.items():
        ref = latent_plain_logits(LATENT, weights, toks)
        for p in range(len(toks)):
            err = float((got[(rid, p)].double() - ref[p]).abs().max() / ref.abs().max())
            assert err <= tol, f"{dtype}: request {rid} position {p}: {err:.3e}"
    assert eng.cache.free_pages() == [48]


# ---- an arrangement without a mixer, with a further part of its own, and weights filled in other ways --------------

from arle_amd.weights import register_init  # noqa: E402

register_init("toy_uniform", lambda shape, gen, std, norm_std, device:
              (torch.rand(shape, generator=gen, dtype=torch.float32, device=device) - 0.5) * 4.0 * std)


@register("feed_forward", "toy_biased_linear")
class BiasedLinear(Part):
    """x W^T + b: the bias starts at zero ("zeros"), the matrix is filled uniformly ("toy_uniform")."""

    @classmethod
    def declare_weights(cls, params):
        h = params["hidden_size"]
        return {"w": WeightDecl((h, h), init="toy_uniform"), "b": WeightDecl((h,), init="zeros")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.w, self.b = tensors["w"].float(), tensors["b"].float()

    def forward(self, x):
        return (x.float() @ self.w.T + self.b).to(x.dtype)


@register("block", "toy_two_branches")
class TwoBranches:
    """h += feed_forward(norm(h)) + extra["second"](norm(h)): no mixer, no cache, one further part."""

    def __init__(self, mixer, feed_forward, norms, extra):
        assert mixer is None
        self.mixer, self.feed_forward, self.norms, self.second = None, feed_forward, norms, extra["second"]

    def forward(self, residual, delta, batch, cache_view):
        assert cache_view is None
        a = self.norms["in"].add_norm(residual, delta)
        return residual, _whole(self.feed_forward.forward(a)) + _whole(self.second.forward(a))


@dataclass(frozen=True)
class BranchConfig:
    hidden_size: int
    intermediate_size: int
    vocab_size: int
    eps: float
    max_position_embeddings: int = 64

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyBranchLM"])


def branch_spec(c: BranchConfig, stop_token_ids=()):
    norm = lambda name: PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.eps}, {"weight": name})
    layers = [LayerSpec("toy_two_branches",
                        feed_forward=PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size},
                                              {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                        norms={"in": norm(f"l{i}.n")},
                        parts={"second": ("feed_forward", PartSpec("toy_biased_linear", {"hidden_size": c.hidden_size},
                                                                   {"w": f"l{i}.w", "b": f"l{i}.b"}))})
              for i in range(2)]
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_positions=c.max_position_embeddings,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}), layers=layers,
                     schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn"),
                     head=PartSpec("linear", sizes, {"weight": "head"}), stop_token_ids=tuple(stop_token_ids))


register_architecture("ToyBranchLM", BranchConfig, branch_spec)


def test_an_arrangement_without_a_mixer_with_a_further_part_and_other_weight_fills(tmp_path):
    c = BranchConfig(hidden_size=24, intermediate_size=40, vocab_size=50, eps=1e-5)
    d = str(tmp_path / "branch")
    write_random_model(d, "ToyBranchLM", c, seed=9, std=0.2, norm_std=0.05)
    _, w = read_folder(d)
    assert torch.count_nonzero(w["l0.b"]) == 0 and float(w["l0.w"].abs().max()) <= 0.4 + 1e-3     # the two fills
    assert float(w["l0.w"].abs().max()) > 0.3
    eng = Engine.from_folder(d, dtype="float32", page_size=4, max_tokens=64, max_slots=2)
    assert eng.cache.groups == [] and eng.kv_bytes_per_token == 0                                   # no layer keeps anything
    toks = random_tokens(19, c.vocab_size, 3)
    got = replay.run_steps(eng, replay.portions("x", toks, sizes=(4, 1, 7, 2)))
    wd = {k: v.double() for k, v in w.items()}
    h = plain.embedding(wd["embed"], toks)
    for i in range(2):
        a = plain.rms_norm(h, wd[f"l{i}.n"], c.eps)
        h = h + plain.swiglu_mlp(a, wd[f"l{i}.g"], wd[f"l{i}.u"], wd[f"l{i}.d"]) + a @ wd[f"l{i}.w"].T + wd[f"l{i}.b"]
    ref = plain.linear(plain.rms_norm(h, wd["fn"], c.eps), wd["head"])
    for pos in range(len(toks)):
        assert float((got[("x", pos)].double() - ref[pos]).abs().max() / ref.abs().max()) <= 1e-5
