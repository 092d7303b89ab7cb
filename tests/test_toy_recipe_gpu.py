"""What a recipe may say without a change to the framework's files, shown with a toy architecture whose folder
stores q|k|v and gate|up as one matrix each (the stock attention and feed-forward take their parameters as rows of
them), whose second mixer keeps its paged cache in pages of another length than the engine's, and whose mixers keep a
table per position under a name of their own that the engine has them size before the first step (`Part.prepare`).
Built from torch operations where it is not the stock parts: it shows the interfaces, it is nobody's model."""
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd.cache import PAGE, PagedNeed, PageTensor
from arle_amd.config import register_architecture
from arle_amd.engine import Engine
from arle_amd.models.decoder import expected_checkpoint_tensors
from arle_amd.parts import LayerSpec, ModelSpec, Part, PartSpec, Rows, ScheduleEntry, WeightDecl, register
from arle_amd.weights import write_random_model
from tiny import random_tokens, read_folder

pytestmark = pytest.mark.gpu


@register("mixer", "toy_gained_latent")
class GainedLatent(Part):
    """Caches c_t = gain[t] * W_down x_t, one float32 vector a token, in pages of `page_size` tokens of its own, and
    returns W_up applied to the mean of c_0..c_t.  gain[t] = 1 / (1 + t / 16) lives in a table that is empty until
    `prepare` makes it; a step that finds it too short fails, it never grows it."""

    graph_safe = False

    @classmethod
    def declare_weights(cls, params):
        return {"down": WeightDecl((params["latent"], params["hidden_size"])),
                "up": WeightDecl((params["hidden_size"], params["latent"]))}

    @classmethod
    def declare_cache(cls, params):
        return PagedNeed(tensors=(PageTensor("latent", (PAGE, int(params["latent"])), torch.float32),),
                         page_size=int(params["page_size"]))

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.down, self.up = tensors["down"].float(), tensors["up"].float()
        self.gain = torch.empty(0, device=rt.device)
        self.prepared_for = []

    def prepare(self, max_positions):
        self.prepared_for.append(max_positions)
        self.gain = 1.0 / (1.0 + torch.arange(max_positions, device=self.rt.device, dtype=torch.float32) / 16.0)

    def cache_need(self):
        return self.declare_cache(self.params)

    def forward(self, x, batch, cache):
        if batch.max_position >= self.gain.shape[0]:
            raise AssertionError("the gain table was not prepared for this position")
        latent, P = cache.pages["latent"], cache.page_size
        assert P == self.params["page_size"] and latent.shape[1] == P
        c = (x.float() @ self.down.T) * self.gain[batch.positions.long()][:, None]
        out = torch.empty_like(c)
        for seg in batch.segments:
            table = cache.block_table[seg.slot].long()
            pos = torch.arange(seg.start, seg.start + seg.length, device=x.device)
            latent[table[pos // P], pos % P] = c[seg.row0:seg.row0 + seg.length]
            every = torch.arange(0, seg.start + seg.length, device=x.device)
            sums = latent[table[every // P], every % P].cumsum(0)[seg.start:]
            out[seg.row0:seg.row0 + seg.length] = sums / (pos + 1).float()[:, None]
        return (out @ self.up.T).to(x.dtype)


@dataclass(frozen=True)
class FusedConfig:
    hidden_size: int
    intermediate_size: int
    heads: int
    kv_heads: int
    head_dim: int
    latent: int
    latent_page: int
    vocab_size: int
    eps: float
    theta: float
    max_position_embeddings: int = 256

    @classmethod
    def from_dict(cls, raw):
        return cls(**{k: raw[k] for k in cls.__dataclass_fields__})

    def to_dict(self):
        return dict(asdict(self), architectures=["ToyFusedLM"])


def fused_spec(c: FusedConfig, stop_token_ids=()):
    norm = lambda name: PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.eps}, {"weight": name})
    Q, KV, I = c.heads * c.head_dim, c.kv_heads * c.head_dim, c.intermediate_size

    def ffn(i):
        return PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": I},
                        {"gate": Rows(f"l{i}.gate_up", 0, I, 2 * I), "up": Rows(f"l{i}.gate_up", I, 2 * I, 2 * I),
                         "down": f"l{i}.d"})

    position = PartSpec("rope_neox", {"head_dim": c.head_dim, "rotary_dim": c.head_dim, "theta": c.theta,
                                      "max_positions": c.max_position_embeddings})
    attention = PartSpec("paged_attention",
                         {"hidden_size": c.hidden_size, "num_q_heads": c.heads, "num_kv_heads": c.kv_heads,
                          "head_dim": c.head_dim, "qk_norm": True, "eps": c.eps, "position": position, "window": None},
                         {"q": Rows("l0.qkv", 0, Q, Q + 2 * KV), "k": Rows("l0.qkv", Q, Q + KV, Q + 2 * KV),
                          "v": Rows("l0.qkv", Q + KV, Q + 2 * KV, Q + 2 * KV), "o": "l0.o",
                          "q_norm": "l0.qn", "k_norm": "l0.kn"})
    latent = PartSpec("toy_gained_latent", {"hidden_size": c.hidden_size, "latent": c.latent, "page_size": c.latent_page},
                      {"down": "l1.down", "up": "l1.up"})
    layers = [LayerSpec("pre_norm", attention, ffn(0), {"mixer_in": norm("l0.n1"), "ffn_in": norm("l0.n2")}),
              LayerSpec("pre_norm", latent, ffn(1), {"mixer_in": norm("l1.n1"), "ffn_in": norm("l1.n2")})]
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_positions=c.max_position_embeddings,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}), layers=layers,
                     schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn"),
                     head=PartSpec("linear", sizes, {"weight": "embed"}), stop_token_ids=tuple(stop_token_ids))


register_architecture("ToyFusedLM", FusedConfig, fused_spec)
FUSED = FusedConfig(hidden_size=48, intermediate_size=80, heads=4, kv_heads=2, head_dim=16, latent=10, latent_page=8,
                    vocab_size=101, eps=1e-5, theta=10000.0)


def fused_plain_logits(c, w, tokens):
    """Whole sequence in float64; the fused matrices are cut here by hand, rows q, then k, then v, and gate, then up."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    Q, KV, I = c.heads * c.head_dim, c.kv_heads * c.head_dim, c.intermediate_size
    h = plain.embedding(w["embed"], tokens)
    # layer 0: attention from the fused q|k|v
    a = plain.rms_norm(h, w["l0.n1"], c.eps)
    qkv = plain.linear(a, w["l0.qkv"])
    cos, sin = plain.rope_cos_sin(list(range(T)), c.head_dim, c.theta, dtype=torch.float64)
    q = plain.prepare_heads(qkv[:, :Q].reshape(T, c.heads, c.head_dim), w["l0.qn"], c.eps, cos, sin)
    k = plain.prepare_heads(qkv[:, Q:Q + KV].reshape(T, c.kv_heads, c.head_dim), w["l0.kn"], c.eps, cos, sin)
    v = qkv[:, Q + KV:].reshape(T, c.kv_heads, c.head_dim)
    h = h + plain.linear(plain.causal_attention(q, k, v, c.kv_heads).reshape(T, -1), w["l0.o"])
    b = plain.rms_norm(h, w["l0.n2"], c.eps)
    h = h + plain.swiglu_mlp(b, w["l0.gate_up"][:I], w["l0.gate_up"][I:], w["l0.d"])
    # layer 1: the gained running mean
    a = plain.rms_norm(h, w["l1.n1"], c.eps)
    gain = 1.0 / (1.0 + torch.arange(T, dtype=torch.float64) / 16.0)
    lat = (a @ w["l1.down"].T) * gain[:, None]
    mean = lat.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
    h = h + mean @ w["l1.up"].T
    b = plain.rms_norm(h, w["l1.n2"], c.eps)
    h = h + plain.swiglu_mlp(b, w["l1.gate_up"][:I], w["l1.gate_up"][I:], w["l1.d"])
    return plain.linear(plain.rms_norm(h, w["fn"], c.eps), w["embed"])


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("toyfused") / "toy")
    write_random_model(d, "ToyFusedLM", FUSED, seed=8, std=0.12, norm_std=0.05)
    return d


def test_the_folder_holds_the_fused_tensors_whole(folder):
    c = FUSED
    want = expected_checkpoint_tensors(fused_spec(c))
    Q, KV = c.heads * c.head_dim, c.kv_heads * c.head_dim
    assert tuple(want["l0.qkv"].shape) == (Q + 2 * KV, c.hidden_size)
    assert tuple(want["l1.gate_up"].shape) == (2 * c.intermediate_size, c.hidden_size)
    assert not any(name.endswith((".q", ".k", ".v", ".g", ".u")) for name in want)
    _, weights = read_folder(folder)
    assert set(weights) == set(want) and tuple(weights["l0.qkv"].shape) == (Q + 2 * KV, c.hidden_size)


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2.5e-2)])
def test_rows_of_fused_tensors_pages_of_another_length_and_prepared_tables(folder, dtype, tol):
    c = FUSED
    _, weights = read_folder(folder)
    eng = Engine.from_folder(folder, dtype=dtype, page_size=4, max_tokens=3 * 64, max_slots=4, max_request_tokens=64)
    # two groups: keys and values in the engine's pages of 4, the latent vectors in pages of 8 holding as many tokens
    sizes = [(g.page_size, g.pool.num_pages) for g in eng.cache.groups]
    assert sizes == [(4, 48), (8, 24)]
    assert eng.cache.tables_dev[0].shape == (4, 16) and eng.cache.tables_dev[1].shape == (4, 8)
    assert eng.cache.page_buffers[1]["latent"].shape == (1, 24, 8, c.latent)
    # the engine had every part size its tables for the longest request before any step
    assert eng.model.blocks[1].mixer.prepared_for == [64]
    reqs = {f"r{i}": random_tokens(n, c.vocab_size, 30 + i) for i, n in enumerate([37, 52, 21, 45, 33])}
    got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=6))
    for rid, toks in reqs.items():
        ref = fused_plain_logits(c, weights, toks)
        for p in range(len(toks)):
            err = float((got[(rid, p)].double() - ref[p]).abs().max() / ref.abs().max())
            assert err <= tol, f"{dtype}: request {rid} position {p}: {err:.3e}"
    assert eng.cache.free_pages() == [48, 24]


def test_generation_through_the_scheduler_with_two_page_lengths(folder):
    """Admission and planning count pages group by group: with so few pages that requests wait, everything still
    finishes and equals one request at a time."""
    from arle_amd import LLM

    c = FUSED
    prompts = [random_tokens(n, c.vocab_size, 80 + i) for i, n in enumerate([19, 30, 11, 25])]
    alone = []
    for p in prompts:
        eng = Engine.from_folder(folder, dtype="float32", page_size=4, max_tokens=64, max_slots=1, max_request_tokens=64)
        alone.append(LLM(eng).generate([p], max_tokens=6)[0].response_token_ids)
    eng = Engine.from_folder(folder, dtype="float32", page_size=4, max_tokens=96, max_slots=3, max_request_tokens=64)
    llm = LLM(eng, chunked_prefill_size=8)
    outs = llm.generate(prompts, max_tokens=6)
    assert [o.response_token_ids for o in outs] == alone
    assert eng.cache.free_pages() == [24, 12] and not eng.cache.slot_of
