"""The engine against the plain implementation, in 32-bit and in bfloat16, under every way
of cutting the work: whole, prefill then token by token, portions of changing size, and
mixed batches with so few pages that they are used again."""
import pytest
import torch

import replay
from arle_amd.engine import Engine
from tiny import TINY, make_model_dir, random_tokens, read_folder

pytestmark = pytest.mark.gpu

# max |engine - plain(float64)| / max |plain|
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module", params=["A", "B", "C", "D", "E"])
def model(request, tmp_path_factory):
    name = request.param
    d = make_model_dir(tmp_path_factory.mktemp("models"), name)
    cfg, weights = read_folder(d)
    return name, d, cfg, weights


def _engine(model, dtype, max_tokens, **kw):
    name, d, cfg, _ = model
    return Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=max_tokens,
                              max_slots=4, **kw)


def _requests(cfg, lengths, seed):
    return {f"r{i}": random_tokens(n, cfg["vocab_size"], seed + i) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_requests(model, dtype):
    _, _, cfg, weights = model
    reqs = _requests(cfg, [1, 9, 23, 40, 70], 100)
    eng = _engine(model, dtype, 128)
    got = {}
    for rid, toks in reqs.items():
        got.update(replay.run_steps(eng, replay.whole(rid, toks)))
    replay.compare(got, cfg, weights, reqs, TOL[dtype], f"whole/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_last_32_one_by_one(model, dtype):
    _, _, cfg, weights = model
    reqs = _requests(cfg, [33, 50, 75], 200)
    eng = _engine(model, dtype, 128)
    got = {}
    for rid, toks in reqs.items():
        got.update(replay.run_steps(eng, replay.prefill_then_decode(rid, toks, 32)))
    replay.compare(got, cfg, weights, reqs, TOL[dtype], f"decode/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_changing_size(model, dtype):
    _, _, cfg, weights = model
    reqs = _requests(cfg, [17, 61, 90], 300)
    eng = _engine(model, dtype, 128)
    got = {}
    for rid, toks in reqs.items():
        got.update(replay.run_steps(eng, replay.portions(rid, toks)))
    replay.compare(got, cfg, weights, reqs, TOL[dtype], f"portions/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_with_page_reuse(model, dtype):
    name, _, cfg, weights = model
    reqs = _requests(cfg, [40, 23, 57, 31, 64, 18, 45, 12], 400)
    # room for the four longest neighbours only: later requests get pages that earlier ones used
    eng = _engine(model, dtype, 4 * 64)
    steps = replay.mixed(reqs, max_live=4, seed=7)
    got = replay.run_steps(eng, steps)
    replay.compare(got, cfg, weights, reqs, TOL[dtype], f"mixed/{dtype}")
    assert eng.cache.free_pages()[0] == eng.cache.groups[0].pool.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_schedules_with_page_reuse(model, dtype):
    """Schedules drawn at random: three to nine requests of 2 to 140 tokens, one to four live at a time, portions of
    up to 3 to 90 tokens beside single tokens, a decoded tail of 0 to 40 tokens, and a pool that holds just the
    longest live requests (each rounded up to 64 tokens), so that pages go round."""
    import random

    name, d, cfg, weights = model
    for seed in range(6):
        rng = random.Random(1000 * seed + 17)
        lengths = [rng.randint(2, 140) for _ in range(rng.randint(3, 9))]
        reqs = {f"q{i}": random_tokens(n, cfg["vocab_size"], 5000 + 31 * seed + i) for i, n in enumerate(lengths)}
        live = rng.randint(1, 4)
        room = sum(-(-n // 64) * 64 for n in sorted(lengths)[-live:])
        eng = _engine(model, dtype, room)
        steps = replay.mixed(reqs, max_live=live, seed=seed, decode_tail=rng.randint(0, 40),
                             max_portion=rng.choice([3, 9, 17, 40, 90]))
        got = replay.run_steps(eng, steps)
        replay.compare(got, cfg, weights, reqs, TOL[dtype], f"random schedule {seed}/{dtype}, lengths {lengths}, {live} live")
        assert eng.cache.free_pages()[0] == eng.cache.groups[0].pool.num_pages


def test_float32_is_bit_identical_across_cuttings(model):
    """The 32-bit path fixes the order of every reduction, so cutting changes no bit."""
    _, _, cfg, weights = model
    toks = random_tokens(45, cfg["vocab_size"], 5)
    eng = _engine(model, "float32", 128)
    a = replay.run_steps(eng, replay.whole("x", toks))
    b = replay.run_steps(eng, replay.portions("x", toks))
    c = replay.run_steps(eng, replay.prefill_then_decode("x", toks, 20))
    for key in a:
        assert torch.equal(a[key], b[key]) and torch.equal(a[key], c[key]), key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_eager_ones_on_every_replay(model, dtype):
    """Steps of single decoded tokens are replayed from a HIP graph.  Every replay, with eager
    steps (prompt portions, other batch sizes) and synchronisations in between, must give the
    bits the eager engine gives."""
    name, d, cfg, _ = model
    reqs = _requests(cfg, [70, 41, 55], 900)
    eager = Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=256, max_slots=4, cuda_graph=False)
    graphed = Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=256, max_slots=4, cuda_graph=True)
    assert graphed.use_graphs and not eager.use_graphs
    steps = []
    for rid, toks in reqs.items():                       # prompts first, all but the last 20 tokens
        steps.append({"entries": [(rid, toks[:-20], [len(toks) - 21])], "end": []})
    for i in range(20):                                  # then three decoded tokens a step ...
        entries = [(rid, [toks[len(toks) - 20 + i]], [0]) for rid, toks in reqs.items()]
        if i % 6 == 5:
            entries = entries[:2]                        # ... sometimes two (another graph), the third catches up
            steps.append({"entries": entries, "end": []})
            rid, toks = list(reqs.items())[2]
            steps.append({"entries": [(rid, [toks[len(toks) - 20 + i]], [0])], "end": []})
        else:
            steps.append({"entries": entries, "end": []})
    a = replay.run_steps(eager, steps)
    b = replay.run_steps(graphed, steps)
    assert graphed.graph_replays >= 10
    for key in a:
        assert torch.equal(a[key], b[key]), f"graph replay differs from the eager step at {key}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_borrowed_logits_are_the_copied_ones_until_the_next_step(model, dtype):
    """`step(..., borrow_logits=True)` may hand out the buffer that a captured step writes: read before the next
    step they are the bits that a step without it returns, replay after replay, and the next replay does write
    the same memory (which is why only a caller that is done with them by then may ask for it)."""
    from arle_amd.engine import StepEntry

    name, d, cfg, _ = model
    reqs = _requests(cfg, [33, 47], 700)
    make = lambda: Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=192, max_slots=4)
    copying, borrowing = make(), make()
    for eng in (copying, borrowing):
        for rid, toks in reqs.items():
            eng.add_request(rid)
            eng.step([StepEntry(rid, toks[:20], [])])
    seen = []
    for t in range(20, 33):
        entries = [StepEntry(rid, [toks[t]], [0]) for rid, toks in reqs.items()]
        want = copying.step(entries)
        got = borrowing.step(entries, borrow_logits=True)
        assert torch.equal(got, want), f"token {t}"
        seen.append((got.data_ptr(), want.data_ptr()))
    assert borrowing.graph_replays >= 10
    assert len({a for a, _ in seen}) < len(seen), "replays of one captured step hand out one buffer"
    assert len({b for _, b in seen[-3:]}) == 3 or len({b for _, b in seen}) > 1, "copies are tensors of their own"


def test_weights_held_as_operand_tiles_give_the_same_bits(model):
    """The decode-friendly second copy of the projection weights changes where the few-rows kernels read
    from, not what they add in which order."""
    name, d, cfg, _ = model
    reqs = _requests(cfg, [37, 20], 901)
    steps = []
    for rid, toks in reqs.items():
        steps += replay.prefill_then_decode(rid, toks, 12)
    got = []
    for tiles in (True, False):
        eng = Engine.from_folder(d, dtype="bfloat16", page_size=TINY[name][1], max_tokens=256, max_slots=4, weight_tiles=tiles)
        assert eng.rt.weight_tiles == tiles
        assert (eng.model.head.proj.tiles is not None) == tiles
        got.append(replay.run_steps(eng, steps))
    for key in got[0]:
        assert torch.equal(got[0][key], got[1][key]), key
    # the 32-bit path has no such copy
    assert not Engine.from_folder(d, dtype="float32", page_size=TINY[name][1], max_tokens=64, weight_tiles=True).rt.weight_tiles


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_of_repeated_shapes_equal_eager_ones(model, dtype):
    """A step shape that repeats (equal portions of prompts, the same decoded tokens beside a portion) runs from
    a captured graph from its second occurrence on.  Every replay, with steps of other shapes, requests that
    end (pages used again) and synchronisations in between, must give the bits of the eager engine."""
    name, d, cfg, _ = model
    reqs = _requests(cfg, [90, 61, 75, 48], 950)
    make = lambda graphs: Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=256, max_slots=4,
                                             cuda_graph=graphs)
    eager, graphed = make(False), make(True)
    r = {k: list(v) for k, v in reqs.items()}
    steps = []
    # r0 in portions of 12 (the same shape seven times), logits wanted at every portion's end
    for a in range(0, 84, 12):
        steps.append({"entries": [("r0", r["r0"][a:a + 12], [11])], "end": []})
    # r1 whole, then r0 and r1 decode beside portions of 10 of r2: the shape (1, 1, 10) repeats
    steps.append({"entries": [("r1", r["r1"][:55], [54])], "end": []})
    for i in range(6):
        steps.append({"entries": [("r0", [r["r0"][84 + i]], [0]), ("r1", [r["r1"][55 + i]], [0]),
                                  ("r2", r["r2"][10 * i:10 * i + 10], [3, 9])], "end": []})
    steps[-1]["end"] = ["r0", "r1"]
    # pages of r0 and r1 are used again by r3, in portions of 12 (the first shape, replayed once more)
    for a in range(0, 48, 12):
        steps.append({"entries": [("r3", r["r3"][a:a + 12], [11])], "end": []})
    steps.append({"entries": [("r2", r["r2"][60:75], [14])], "end": ["r2", "r3"]})
    a = replay.run_steps(eager, steps)
    b = replay.run_steps(graphed, steps)
    assert graphed.graph_replays >= 12
    assert set(a) == set(b)
    for key in a:
        assert torch.equal(a[key], b[key]), f"graph replay differs from the eager step at {key}"


def test_captured_steps_are_kept_least_recently_used(model):
    """More step shapes than the engine may keep as graphs: the least recently used goes, and a shape that comes
    back is captured again; the logits stay those of the eager engine."""
    name, d, cfg, _ = model
    make = lambda graphs: Engine.from_folder(d, dtype="float32", page_size=TINY[name][1], max_tokens=256, max_slots=4,
                                             cuda_graph=graphs)
    eager, graphed = make(False), make(True)
    graphed.max_graphs = 2
    toks = random_tokens(120, cfg["vocab_size"], 77)
    steps, at = [], 0
    for n in (5, 5, 7, 7, 9, 9, 5, 5, 7, 1, 1, 1, 9, 9):     # portions of three sizes, and decoded tokens
        steps.append({"entries": [("r", toks[at:at + n], [n - 1])], "end": []})
        at += n
    a = replay.run_steps(eager, steps)
    b = replay.run_steps(graphed, steps)
    assert len(graphed._graphs) <= 2 and graphed.graph_replays >= 4
    for key in a:
        assert torch.equal(a[key], b[key]), key


def test_head_dim_that_is_no_multiple_of_16_runs_in_float32_and_is_refused_in_bfloat16(tmp_path):
    d = make_model_dir(tmp_path, "F")
    cfg, weights = read_folder(d)
    assert cfg["head_dim"] == 24
    reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 900 + i) for i, n in enumerate([40, 23, 57, 31, 18])}
    eng = Engine.from_folder(d, dtype="float32", page_size=TINY["F"][1], max_tokens=3 * 64, max_slots=3)
    got = replay.run_steps(eng, replay.mixed(reqs, max_live=3, seed=11))
    replay.compare(got, cfg, weights, reqs, TOL["float32"], "head_dim 24 / float32")
    with pytest.raises(ValueError, match="multiples of 16"):
        Engine.from_folder(d, dtype="bfloat16", page_size=8, max_tokens=64)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_fed_from_gpu_memory_give_the_bits_of_tokens_fed_from_the_host(model, dtype):
    """An entry's one token may be a DeviceToken, an element of an int32 tensor on the GPU: eager steps, captured
    decode steps and a decoded token beside a prompt portion must give the same logits as with the id itself,
    whatever the order of the rows in the tensor."""
    from arle_amd.engine import DeviceToken, StepEntry

    name, d, cfg, _ = model
    reqs = _requests(cfg, [37, 52, 44], 1200)
    outs = {}
    for fed in (False, True):
        eng = Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=320, max_slots=4)
        got = []
        for rid, toks in reqs.items():
            eng.add_request(rid)
            eng.step([StepEntry(rid, toks[:20], [])])
        for i in range(20, 30):                                     # decode steps of three rows: captured from the second on
            ids = [toks[i] for toks in reqs.values()]
            if fed:
                source = torch.tensor(ids[::-1] + [0], dtype=torch.int32, device=eng.device)    # reversed, and one more
                entries = [StepEntry(rid, [DeviceToken(source, 2 - j)], [0]) for j, rid in enumerate(reqs)]
            else:
                entries = [StepEntry(rid, [t], [0]) for rid, t in zip(reqs, ids)]
            got.append(eng.step(entries).clone())
        rid0, rid1 = list(reqs)[:2]                                # a decoded token beside a portion of another request
        t0 = reqs[rid0][30]
        first = [DeviceToken(torch.tensor([t0], dtype=torch.int32, device=eng.device), 0)] if fed else [t0]
        got.append(eng.step([StepEntry(rid0, first, [0]), StepEntry(rid1, reqs[rid1][30:37], [6])]).clone())
        assert eng.graph_replays >= 8
        outs[fed] = got
    for a, b in zip(outs[False], outs[True]):
        assert torch.equal(a, b)
    eng = Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=64, max_slots=2)
    eng.add_request(0)
    source = torch.zeros(2, dtype=torch.int32, device=eng.device)
    with pytest.raises(ValueError, match="DeviceToken"):
        eng.step([StepEntry(0, [DeviceToken(source, 0), 3], [1])])       # only as the one token of an entry
    with pytest.raises(ValueError, match="outside its tensor"):
        eng.step([StepEntry(0, [DeviceToken(source, 2)], [0])])
    assert eng.length(0) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_up_captures_every_decode_graph_before_the_first_request(model, dtype):
    """After `warm_up` no decode step is run eagerly or captured in mid-serving: every one is a replay, the number of
    graphs does not change, nothing is left in the cache, and the logits are those of an engine that was not warmed
    (infer/src/scheduler/cuda/core/warmup.rs:11-160)."""
    from arle_amd.engine.engine import decode_warmup_sizes

    assert decode_warmup_sizes(4) == [1, 2, 3, 4] and decode_warmup_sizes(100)[-4:] == [64, 80, 96, 100]
    assert decode_warmup_sizes(9) == list(range(1, 10)) and decode_warmup_sizes(70)[-2:] == [64, 70]
    name, d, cfg, _ = model
    make = lambda: Engine.from_folder(d, dtype=dtype, page_size=TINY[name][1], max_tokens=3 * 320, max_slots=3,
                                      max_request_tokens=320)
    cold, warm = make(), make()
    captured = warm.warm_up()
    assert captured == len(warm._graphs) >= 3               # at least one graph a batch size
    assert {rows for rows, _ in warm._graphs} == {1, 2, 3}
    assert not warm.cache.slot_of and warm.cache.free_pages() == cold.cache.free_pages()
    warm.cache.check()
    assert warm.warm_up() == 0                              # all there already
    reqs = {f"w{i}": random_tokens(n, cfg["vocab_size"], 300 + i) for i, n in enumerate([150, 40, 20])}
    steps = [{"entries": [(rid, t[:-12], [len(t) - 13]) for rid, t in reqs.items()], "end": []}]
    for i in range(12, 0, -1):    # three decoding requests, then two, then one, with contexts in several classes
        live = [rid for k, rid in enumerate(reqs) if i > 4 * k]
        steps.append({"entries": [(rid, reqs[rid][-i:len(reqs[rid]) - i + 1], [0]) for rid in live], "end": []})
    graphs_before = len(warm._graphs)
    a = replay.run_steps(cold, steps)
    b = replay.run_steps(warm, steps)
    assert warm.graph_replays == 12 and len(warm._graphs) == graphs_before
    for key in a:
        assert torch.equal(a[key], b[key]), key


def test_decode_steps_with_the_preparation_folded_into_the_attention_and_as_a_kernel_of_its_own(tmp_path):
    """bfloat16 decode steps at a head_dim for which the attention's kernel can prepare q, k and v itself (config D:
    64): with that and with `qk_prep` as a kernel of its own the logits are the plain ones, two requests decoded
    token by token side by side after their prompts."""
    d = make_model_dir(tmp_path, "D")
    cfg, weights = read_folder(d)
    reqs = _requests(cfg, [40, 57], 900)
    for folded in (True, False):
        eng = Engine.from_folder(d, dtype="bfloat16", page_size=TINY["D"][1], max_tokens=192, max_slots=4)
        folds = [p for p in eng.model.parts if hasattr(p, "folds_preparation")]
        assert folds and all(p.folds_preparation for p in folds)
        for p in folds:
            p.folds_preparation = folded
        steps = [{"entries": [(rid, toks[:8], list(range(8))) for rid, toks in reqs.items()], "end": []}]
        for t in range(8, 57):
            steps.append({"entries": [(rid, [toks[t]], [0]) for rid, toks in reqs.items() if t < len(toks)], "end": []})
        got = replay.run_steps(eng, steps)
        assert len(got) == 40 + 57
        replay.compare(got, cfg, weights, reqs, TOL["bfloat16"], f"decode, folded {folded}")
