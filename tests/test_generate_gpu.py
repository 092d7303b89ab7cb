"""Generation through the entry point, the scheduler on the real engine, and bin/trace_run."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import replay
from arle_amd import LLM, SamplingParams
from arle_amd.sampling import uniform
from tiny import TINY, make_model_dir, random_tokens, read_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("gen")
    # a larger weight spread than the default separates the logits, so greedy ties are no issue
    return {name: make_model_dir(base, name, std_scale=6.0) for name in ("A", "B")}


def _plain_greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain.forward_logits(weights, cfg, toks, dtype=torch.float64)[-1].argmax()))
    return toks[len(prompt):]


def test_greedy_generation_equals_the_plain_implementation(folders):
    # configuration A of the task: prompts of 5 / 11 / 17 tokens, 8 greedy tokens each
    cfg, weights = read_folder(folders["A"])
    prompts = [random_tokens(n, cfg["vocab_size"], 70 + n) for n in (5, 11, 17)]
    want = [_plain_greedy(cfg, weights, p, 8) for p in prompts]
    llm = LLM(folders["A"], dtype="float32", page_size=TINY["A"][1], kv_cache_tokens=256, max_seq_len=64)
    outs = llm.generate(prompts, max_tokens=8)
    assert [o.response_token_ids for o in outs] == want
    assert all(o.finish_reason == "length" and o.usage.completion_tokens == 8 for o in outs)
    assert [o.usage.prompt_tokens for o in outs] == [5, 11, 17]
    assert llm.last_stats["steps"]["decode"] > 0


def test_bfloat16_greedy_picks_near_best_tokens(folders):
    cfg, weights = read_folder(folders["A"])
    prompts = [random_tokens(n, cfg["vocab_size"], 80 + n) for n in (5, 11, 17)]
    llm = LLM(folders["A"], dtype="bfloat16", page_size=TINY["A"][1], kv_cache_tokens=256, max_seq_len=64)
    for p, o in zip(prompts, llm.generate(prompts, max_tokens=8)):
        hist = list(p)
        for t in o.response_token_ids:
            logits = plain.forward_logits(weights, cfg, hist, dtype=torch.float64)[-1]
            assert float(logits.max() - logits[t]) <= 0.03 * float(logits.abs().max())
            hist.append(t)


def test_temperature_sampling_with_portions_equals_plain_inverse_cdf(folders):
    # configuration B of the task: prompts of 1 / 9 / 23 / 40, portions of 16, temperature 0.8, 6 tokens
    cfg, weights = read_folder(folders["B"])
    prompts = [random_tokens(n, cfg["vocab_size"], 90 + n) for n in (1, 9, 23, 40)]
    llm = LLM(folders["B"], dtype="float32", page_size=TINY["B"][1], kv_cache_tokens=512, max_seq_len=128,
              chunked_prefill_size=16, seed=7)
    params = SamplingParams(temperature=0.8, seed=1234)
    outs = llm.generate(prompts, max_tokens=6, sampling=params)
    assert llm.last_stats["steps"]["mixed"] > 0          # portions ran beside decoded tokens
    for p, o in zip(prompts, outs):
        hist = list(p)
        for i, t in enumerate(o.response_token_ids):
            logits = plain.forward_logits(weights, cfg, hist, dtype=torch.float64)[-1]
            assert t == plain.sample_token(logits, 0.8, uniform(1234, i)), (len(p), i)
            hist.append(t)
        assert len(o.response_token_ids) == 6
    # the same seed gives the same tokens whatever else is in the batch
    alone = llm.generate([prompts[2]], max_tokens=6, sampling=params)[0]
    assert alone.response_token_ids == outs[2].response_token_ids


def test_sampling_parameters_of_their_own_for_every_prompt(folders):
    """`sampling` as a list: every prompt is sampled by its own parameters, as if it had been generated alone."""
    cfg, _ = read_folder(folders["B"])
    prompts = [random_tokens(n, cfg["vocab_size"], 70 + n) for n in (9, 14, 5)]
    params = [SamplingParams(temperature=0.0, ignore_eos=True), SamplingParams(temperature=0.9, top_p=0.8, seed=3, ignore_eos=True),
              SamplingParams(temperature=0.7, top_k=5, seed=11, ignore_eos=True)]
    llm = LLM(folders["B"], dtype="float32", page_size=TINY["B"][1], kv_cache_tokens=256, max_seq_len=64)
    together = llm.generate(prompts, max_tokens=7, sampling=params)
    for p, sp, got in zip(prompts, params, together):
        alone = llm.generate([p], max_tokens=7, sampling=sp)[0]
        assert got.response_token_ids == alone.response_token_ids and len(got.response_token_ids) == 7
    assert together[0].response_token_ids != together[1].response_token_ids
    with pytest.raises(ValueError):
        llm.generate(prompts, max_tokens=2, sampling=params[:2])


def test_generation_survives_a_pool_that_runs_out(folders):
    cfg, weights = read_folder(folders["A"])
    prompts = [random_tokens(10, cfg["vocab_size"], 60 + k) for k in range(4)]
    want = [_plain_greedy(cfg, weights, p, 24) for p in prompts]
    llm = LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=52, max_seq_len=64)
    outs = llm.generate(prompts, max_tokens=24)
    assert llm.last_stats["preemptions"] > 0
    assert [o.response_token_ids for o in outs] == want
    assert llm.engine.cache.free_pages() == [13] and not llm.engine.cache.slot_of


def test_stop_token_from_generation_config(folders, tmp_path):
    cfg, weights = read_folder(folders["A"])
    prompt = random_tokens(9, cfg["vocab_size"], 5)
    free_run = _plain_greedy(cfg, weights, prompt, 8)
    stop = free_run[4]
    with open(os.path.join(folders["A"], "generation_config.json"), "w") as fh:
        json.dump({"eos_token_id": [stop]}, fh)
    try:
        llm = LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=256, max_seq_len=64)
        out = llm.generate([prompt], max_tokens=8)[0]
        assert out.response_token_ids == free_run[:free_run.index(stop)] and out.finish_reason == "stop"
        out = llm.generate([prompt], max_tokens=8, ignore_eos=True)[0]
        assert out.response_token_ids == free_run and out.finish_reason == "length"
    finally:
        os.remove(os.path.join(folders["A"], "generation_config.json"))


def test_command_line_run(folders):
    cfg, weights = read_folder(folders["A"])
    prompt = random_tokens(7, cfg["vocab_size"], 3)
    want = _plain_greedy(cfg, weights, prompt, 5)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "arle-amd"), "--model-path", folders["A"], "--max-tokens", "5",
           "--dtype", "float32", "--max-seq-len", "64", "run", "--prompt-ids", ",".join(map(str, prompt)), "--json"]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    doc = json.loads(res.stdout.strip().splitlines()[-1])
    assert doc["token_ids"] == want and doc["usage"] == {"prompt_tokens": 7, "completion_tokens": 5, "total_tokens": 12}
    assert "tok/s" in res.stderr and "TTFT" in res.stderr


class TraceRun:
    """bin/trace_run as a child process: one JSON line in, `done <step>` out."""

    def __init__(self, model, dtype, out, max_tokens):
        self.out = out
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", dtype,
             "--out", out, "--max-tokens", str(max_tokens)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)

    def step(self, rec):
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {rec['step']}", f"trace_run said {line!r}"
        path = os.path.join(self.out, f"{rec['step']}.f32")
        return np.fromfile(path, dtype="<f4") if os.path.exists(path) else None

    def close(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=120) == 0


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_trace_run_program(folders, tmp_path, dtype, tol):
    cfg, weights = read_folder(folders["B"])
    vocab = cfg["vocab_size"]
    reqs = {f"q{i}": random_tokens(n, vocab, 500 + i) for i, n in enumerate([37, 64, 20, 51, 45])}
    steps = replay.mixed(reqs, max_live=4, seed=3)
    tr = TraceRun(folders["B"], dtype, str(tmp_path / f"out_{dtype}"), max_tokens=4 * 64)
    got, fed = {}, {r: 0 for r in reqs}
    try:
        for i, st in enumerate(steps):
            rec = {"step": i, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in st["entries"]],
                   "end": st["end"]}
            flat = tr.step(rec)
            where = [(r, fed[r] + k) for r, t, w in st["entries"] for k in w]
            for r, t, _ in st["entries"]:
                fed[r] += len(t)
            if where:
                rows = torch.from_numpy(flat.reshape(len(where), vocab).copy())
                got.update(dict(zip(where, rows)))
        # a step that wants nothing writes no file
        assert tr.step({"step": 9999, "entries": [{"id": "z", "tokens": [1, 2, 3], "want": []}], "end": ["z"]}) is None
    finally:
        tr.close()
    replay.compare(got, cfg, weights, reqs, tol, f"trace_run/{dtype}")


@pytest.mark.parametrize("bad,what", [
    ('{"step": 1, "entries": [{"id": "a", "tokens": [1, 99999], "want": [0]}], "end": []}', "outside the vocabulary"),
    ('{"step": 1, "entries": [{"id": "a", "tokens": [1, 2], "want": [5]}], "end": []}', "wanted place"),
    ('{"step": 1, "entries": [{"id": "b", "tokens": ' + str(list(range(200))) + ', "want": []}], "end": []}', "OutOfPages"),
    ('{"step": 1, "entries": [{"id": "a", "tok', "JSONDecodeError"),
    ('{"entries": [], "end": []}', "KeyError"),
])
def test_trace_run_ends_with_the_line_and_the_reason_when_a_step_cannot_be_run(folders, tmp_path, bad, what):
    """A good step, then one that cannot be read or run: the good step's file is there, its `done` line too, the
    program names the input line and the reason on stderr and ends with 1 (no `done` for the bad step)."""
    good = '{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [2]}], "end": []}'
    out = str(tmp_path / "out")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["B"], "--dtype", "float32",
                        "--out", out, "--max-tokens", "64"], input=good + "\n" + bad + "\n", capture_output=True, text=True,
                       timeout=300)
    assert p.returncode == 1
    assert p.stdout.split() == ["done", "0"] and os.path.exists(os.path.join(out, "0.f32"))
    assert "input line 2" in p.stderr and what in p.stderr
    assert not os.path.exists(os.path.join(out, "1.f32"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_through_the_scheduler_with_and_without_captured_steps(folders, dtype):
    """Thirty requests of random lengths and budgets through few slots, small portions and a pool that runs out now
    and then: prompt portions beside decoded tokens in ever changing shapes, some of which repeat and are captured.
    With captured steps and without, every request must get the same tokens (and in float32 the plain ones)."""
    from arle_amd.engine import Engine

    cfg, weights = read_folder(folders["B"])
    rng = np.random.default_rng(5)
    prompts = [random_tokens(int(n), cfg["vocab_size"], 500 + i) for i, n in enumerate(rng.integers(1, 60, size=30))]
    budgets = [int(b) for b in rng.integers(1, 14, size=30)]
    results = {}
    for graphs in (False, True):
        eng = Engine.from_folder(folders["B"], dtype=dtype, page_size=TINY["B"][1], max_tokens=208, max_slots=5,
                                 max_request_tokens=96, cuda_graph=graphs)
        llm = LLM(eng, num_slots=5, chunked_prefill_size=16, max_num_batched_tokens=48, max_seq_len=96)
        outs = []
        for lo in range(0, 30, 10):     # three waves of ten requests, each wave through one scheduler
            wave = llm.generate(prompts[lo:lo + 10], max_tokens=max(budgets[lo:lo + 10]),
                                sampling=SamplingParams(temperature=0.0, ignore_eos=True))
            outs.extend(o.response_token_ids[:b] for o, b in zip(wave, budgets[lo:lo + 10]))
        results[graphs] = outs
        if graphs:
            assert eng.graph_replays > 20
        assert not eng.cache.slot_of
    assert results[False] == results[True]
    if dtype == "float32":
        for p, b, got in list(zip(prompts, budgets, results[True]))[::5]:
            assert got == _plain_greedy(cfg, weights, p, b)


def test_command_line_run_with_a_text_prompt_and_a_tokenizer(folders, tmp_path):
    """`run --prompt TEXT`: text -> tokenizer.json of the folder -> ids -> generation -> text again.  The test writes a
    small word-level tokenizer (word "t<i>" is id i), so the ids are known."""
    import shutil

    tokenizers = pytest.importorskip("tokenizers")
    cfg, weights = read_folder(folders["A"])
    d = str(tmp_path / "with_tokenizer")
    shutil.copytree(folders["A"], d)
    tok = tokenizers.Tokenizer(tokenizers.models.WordLevel({f"t{i}": i for i in range(cfg["vocab_size"])}, unk_token="t0"))
    tok.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tok.decoder = tokenizers.decoders.WordPiece(prefix="##", cleanup=False)     # joins words with a blank
    tok.save(os.path.join(d, "tokenizer.json"))
    prompt = random_tokens(6, cfg["vocab_size"], 31)
    want = _plain_greedy(cfg, weights, prompt, 4)
    text = " ".join(f"t{t}" for t in prompt)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "arle-amd"), "--model-path", d, "--max-tokens", "4",
           "--dtype", "float32", "--max-seq-len", "64", "run", "--prompt", text, "--json"]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    doc = json.loads(res.stdout.strip().splitlines()[-1])
    assert doc["token_ids"] == want and doc["usage"]["prompt_tokens"] == 6
    assert doc["text"].split() == [f"t{t}" for t in want]
    # the same through --stdin, as plain text on stdout
    cmd = cmd[:-3] + ["--stdin"]
    res = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert res.stdout.strip().splitlines()[-1].split() == [f"t{t}" for t in want]


def test_log_probabilities_of_the_chosen_tokens(folders):
    """token_logprobs = log softmax(logits)[token] of every generated token, greedy and sampled rows in one batch
    (greedy: the reference's -log(sum exp(x - max)), crates/cuda-kernels/csrc/misc/sampling.cu:252-317)."""
    cfg, weights = read_folder(folders["B"])
    prompts = [random_tokens(n, cfg["vocab_size"], 40 + n) for n in (7, 12)]
    llm = LLM(folders["B"], dtype="float32", page_size=TINY["B"][1], kv_cache_tokens=256, max_seq_len=64)
    from arle_amd.engine.scheduler import Scheduler

    sched = Scheduler(llm.engine, llm.sampler, llm.sched_config, seed=3)
    a = sched.submit(prompts[0], SamplingParams(logprobs=True), max_tokens=5)
    b = sched.submit(prompts[1], SamplingParams(temperature=0.9, seed=77, logprobs=True), max_tokens=5)
    c = sched.submit(prompts[1], SamplingParams(), max_tokens=5)
    sched.run_until_done()
    assert sched.finished[c].logprobs == []
    for rid, p in ((a, prompts[0]), (b, prompts[1])):
        r = sched.finished[rid]
        assert len(r.logprobs) == len(r.generated) == 5
        hist = list(p)
        for t, lp in zip(r.generated, r.logprobs):
            ref = torch.log_softmax(plain.forward_logits(weights, cfg, hist, dtype=torch.float64)[-1], dim=-1)
            assert abs(lp - float(ref[t])) < 1e-4
            hist.append(t)
    greedy = sched.finished[a]
    assert all(lp <= 0.0 for lp in greedy.logprobs)
    out = llm.generate([prompts[0]], max_tokens=5, logprobs=True)[0]
    assert out.response_token_ids == greedy.generated and out.token_logprobs == pytest.approx(greedy.logprobs, abs=1e-6)
    assert out.tpot_s is not None and out.tpot_s > 0


def test_abort_on_the_real_engine_gives_pages_back(folders):
    from arle_amd.engine.scheduler import ABORT, Scheduler

    cfg, weights = read_folder(folders["A"])
    llm = LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=256, max_seq_len=64, chunked_prefill_size=8)
    sched = Scheduler(llm.engine, llm.sampler, llm.sched_config, seed=1)
    keep_prompt = random_tokens(9, cfg["vocab_size"], 21)
    keep = sched.submit(keep_prompt, max_tokens=10)
    gone = sched.submit(random_tokens(30, cfg["vocab_size"], 22), max_tokens=10)
    sched.iteration()
    sched.iteration()
    assert sched.abort(gone) and sched.finished[gone].finish_reason == ABORT
    sched.run_until_done()
    assert sched.finished[keep].generated == _plain_greedy(cfg, weights, keep_prompt, 10)
    assert llm.engine.cache.free_pages() == [64] and not llm.engine.cache.slot_of


def test_the_pool_is_sized_from_free_memory_when_no_size_is_given(folders):
    """No kv_cache_tokens: pages for what is free less the headroom, but never more than the slots can fill."""
    cfg, weights = read_folder(folders["A"])
    llm = LLM(folders["A"], dtype="bfloat16", page_size=16, num_slots=3, max_seq_len=200)
    cache = llm.engine.cache
    assert cache.groups[0].pool.num_pages == 3 * 13          # 3 slots x ceil(200 / 16) pages: the cap
    assert llm.engine.kv_bytes_per_token == 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * 2
    out = llm.generate([random_tokens(5, cfg["vocab_size"], 2)], max_tokens=3)[0]
    assert len(out.response_token_ids) == 3
    from arle_amd.engine import Engine
    from arle_amd.engine.engine import EngineError

    with pytest.raises(EngineError, match="no memory for the cache"):
        Engine.from_folder(folders["A"], dtype="bfloat16", mem_fraction_static=1e-6)


@pytest.mark.parametrize("overlap", [True, False])
def test_streamed_deltas_add_up_to_what_generate_returns(folders, overlap):
    """generate_stream hands on what every request has newly produced after each iteration: the tokens and
    log-probabilities of a request's deltas are those of `generate`, a request's last delta alone carries its finish
    reason and usage (without a token when a stop token ended it), requests that wait for a slot start later, and an
    empty prompt ends at once."""
    cfg, _ = read_folder(folders["A"])
    llm = LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=256, max_seq_len=64, num_slots=2,
              async_overlap=overlap)
    prompts = [random_tokens(n, cfg["vocab_size"], 30 + n) for n in (5, 9, 3)] + [[]]
    params = SamplingParams(temperature=0.7, seed=11, logprobs=True, ignore_eos=True)
    whole = llm.generate(prompts, max_tokens=7, sampling=params)
    deltas = list(llm.generate_stream(prompts, max_tokens=7, sampling=params))
    for i, want in enumerate(whole):
        mine = [d for d in deltas if d.index == i]
        assert [t for d in mine for t in d.token_ids] == want.response_token_ids
        assert np.allclose([x for d in mine for x in d.logprobs], want.token_logprobs)
        assert [d.finish_reason for d in mine[:-1]] == [None] * (len(mine) - 1) and mine[-1].finish_reason == want.finish_reason
        assert mine[-1].usage.completion_tokens == len(want.response_token_ids) and all(d.usage is None for d in mine[:-1])
        assert all(d.text_delta is None for d in mine)            # a folder without a tokenizer
    assert len([d for d in deltas if d.index == 3]) == 1          # the empty prompt: one delta, its end
    first_of = {i: next(k for k, d in enumerate(deltas) if d.index == i and d.token_ids) for i in range(3)}
    assert first_of[2] > first_of[0] and first_of[2] > first_of[1]   # two slots: the third request starts when one is free
    assert len([d for d in deltas if d.index == 0]) >= 6           # token by token, not all at the end
    # a request that a stop token ends: its last delta has no token
    stop = whole[0].response_token_ids[3]
    if stop not in whole[0].response_token_ids[:3]:
        cut = SamplingParams(temperature=0.7, seed=11, stop_token_ids=[stop])
        mine = list(llm.generate_stream([prompts[0]], max_tokens=7, sampling=cut))
        assert [t for d in mine for t in d.token_ids] == whole[0].response_token_ids[:3]
        assert mine[-1].finish_reason == "stop" and mine[-1].token_ids == []


@pytest.mark.parametrize("overlap", [True, False])
def test_a_stop_string_ends_a_request_in_front_of_it(folders, tmp_path, overlap):
    """With a tokenizer (one word a token, made here) a stop string that begins in one token and ends in the next
    ends the request: the text stops in front of it, streamed or not, nothing of it was handed on early, the tokens
    are those read up to the one that completed it, and the finish reason is `stop`."""
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers

    cfg, _ = read_folder(folders["A"])
    d = str(tmp_path / "with_tokenizer")
    shutil.copytree(folders["A"], d)
    tok = Tokenizer(models.WordLevel({f"w{i}": i for i in range(cfg["vocab_size"])}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(os.path.join(d, "tokenizer.json"))
    llm = LLM(d, dtype="float32", page_size=4, kv_cache_tokens=256, max_seq_len=64, async_overlap=overlap)
    prompt = random_tokens(6, cfg["vocab_size"], 77)
    params = SamplingParams(temperature=0.9, seed=5, ignore_eos=True)
    whole = llm.generate([prompt, "w3 w4 w5"], max_tokens=10, sampling=params)
    words = [f"w{t}" for t in whole[0].response_token_ids]
    assert whole[0].text == " ".join(words) and whole[1].prompt_token_ids == [3, 4, 5]
    full = " ".join(words)
    # the end of word k, a blank, the head of word k + 1, where that does not occur earlier in the text
    k = next(i for i in range(2, 9)
             if full.find(f"{words[i][1:]} w") == len(" ".join(words[:i + 1])) - len(words[i][1:]))
    stop = f"{words[k][1:]} w"
    want_text = full[:full.find(stop)]
    cut = llm.generate([prompt, "w3 w4 w5"], max_tokens=10, sampling=params, stop=["never", "", stop])
    assert cut[0].text == want_text and cut[0].finish_reason == "stop"
    assert cut[0].response_token_ids == whole[0].response_token_ids[:k + 2]
    assert cut[1].response_token_ids == whole[1].response_token_ids and cut[1].finish_reason == "length"
    deltas = [x for x in llm.generate_stream([prompt], max_tokens=10, sampling=params, stop=[stop]) if x.index == 0]
    assert "".join(x.text_delta for x in deltas) == want_text and deltas[-1].finish_reason == "stop"
    sent = ""
    for x in deltas:        # what has gone out never reaches into the stop string
        sent += x.text_delta
        assert want_text.startswith(sent)
    assert any(x.text_delta for x in deltas[:-1])      # and text does go out before the end
    assert llm.engine.cache.free_pages() == [64] and not llm.engine.cache.slot_of
    with pytest.raises(RuntimeError, match="tokenizer"):
        LLM(llm.engine).generate([prompt], stop=["x"])


def test_slots_left_unset_follow_the_cache(folders):
    """num_slots=None: as many requests of max_seq_len as the cache holds (4 to 128), with a given cache and with one
    sized from the GPU's memory; more prompts than slots still all finish."""
    cfg, _ = read_folder(folders["A"])
    llm = LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=640, max_seq_len=64, num_slots=None)
    assert llm.engine.cache.max_slots == 10 and llm.sched_config.num_slots == 10
    prompts = [random_tokens(3 + i % 5, cfg["vocab_size"], 60 + i) for i in range(14)]
    outs = llm.generate(prompts, max_tokens=4, ignore_eos=True)
    assert [len(o.response_token_ids) for o in outs] == [4] * 14
    assert LLM(folders["A"], dtype="float32", page_size=4, kv_cache_tokens=100, max_seq_len=64,
               num_slots=None).engine.cache.max_slots == 4
    big = LLM(folders["A"], dtype="bfloat16", page_size=16, max_seq_len=200, num_slots=None)    # a tiny model on a large GPU
    assert big.engine.cache.max_slots == 128 and big.engine.cache.groups[0].pool.num_pages == 128 * 13


def test_the_sizes_of_a_step_follow_the_gpus_memory_unless_given(folders):
    """Nothing given: the longest portion of one request is what the GPU's whole memory gives (16,384 tokens from
    90 GiB on), so a 700-token prompt is one step; with chunked_prefill_size=256 it is three, and the tokens are the
    same."""
    from arle_amd.engine.scheduler import pick_chunked_prefill_size_for_hbm

    cfg, _ = read_folder(folders["B"])
    llm = LLM(folders["B"], dtype="float32", page_size=TINY["B"][1], kv_cache_tokens=2048, max_seq_len=1024)
    total = torch.cuda.get_device_properties(llm.engine.device).total_memory
    sc = llm.sched_config
    assert sc.chunked_prefill_size == pick_chunked_prefill_size_for_hbm(total) == 16384
    assert (sc.max_prefill_tokens, sc.long_prefill_token_threshold) == (16384, 4096)
    prompt = random_tokens(700, cfg["vocab_size"], 21)
    whole = llm.generate([prompt], max_tokens=6, ignore_eos=True)[0]
    assert llm.last_stats["steps"]["prefill"] == 1
    cut = LLM(llm.engine, chunked_prefill_size=256, max_prefill_tokens=512, max_seq_len=1024)
    assert (cut.sched_config.chunked_prefill_size, cut.sched_config.max_prefill_tokens,
            cut.sched_config.long_prefill_token_threshold) == (256, 512, 256)
    pieces = cut.generate([prompt], max_tokens=6, ignore_eos=True)[0]
    assert cut.last_stats["steps"]["prefill"] == 3
    assert pieces.response_token_ids == whole.response_token_ids


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_give_the_tokens_of_steps_that_wait(folders, dtype):
    """Decode steps fed from the last step's tokens on the GPU, read back one step late, against steps that
    read every token before they go on: greedy and seeded sampling with log-probabilities, requests that end by
    a stop token (one row runs in vain), by their length, and arrive in waves."""
    from arle_amd.engine import Engine

    cfg, weights = read_folder(folders["B"])
    rng = np.random.default_rng(11)
    prompts = [random_tokens(int(n), cfg["vocab_size"], 700 + i) for i, n in enumerate(rng.integers(2, 40, size=12))]
    free_run = _plain_greedy(cfg, weights, prompts[0], 12) if dtype == "float32" else None
    results = {}
    for overlap in (False, True):
        eng = Engine.from_folder(folders["B"], dtype=dtype, page_size=TINY["B"][1], max_tokens=400, max_slots=4,
                                 max_request_tokens=96)
        llm = LLM(eng, num_slots=4, chunked_prefill_size=16, max_num_batched_tokens=48, max_seq_len=96,
                  async_overlap=overlap)
        greedy = llm.generate(prompts[:6], max_tokens=12, sampling=SamplingParams(temperature=0.0, ignore_eos=True))
        ahead = llm.last_stats.get("steps_ahead", 0)
        drawn = llm.generate(prompts[6:], max_tokens=9, sampling=SamplingParams(temperature=0.8, top_p=0.9, seed=3,
                                                                                 ignore_eos=True, logprobs=True))
        stop = greedy[0].response_token_ids[5]
        stopped = llm.generate(prompts[:3], max_tokens=12, sampling=SamplingParams(stop_token_ids=[stop]))
        results[overlap] = ([o.response_token_ids for o in greedy], [o.response_token_ids for o in drawn],
                            [o.token_logprobs for o in drawn], [(o.response_token_ids, o.finish_reason) for o in stopped])
        assert (ahead >= 8) == overlap and (llm.last_stats.get("steps_ahead", 0) > 0) == overlap
        assert stopped[0].finish_reason == "stop" and stop not in stopped[0].response_token_ids
        assert not eng.cache.slot_of
        for g in eng.cache.groups:
            g.check()
            assert g.pool.free_count == g.pool.num_pages
    assert results[False] == results[True]
    if free_run is not None:
        assert results[True][0][0] == free_run


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_traffic_on_the_real_engine_with_and_without_steps_launched_ahead(folders, seed):
    """Requests of random lengths, budgets, priorities and sampling arriving while others run, through few slots
    and a pool so small that requests give pages back, some meeting stop tokens: with steps launched ahead and
    with steps that wait for their tokens every request ends with the same tokens and reason, and the cache is
    empty and consistent at the end."""
    import random

    from arle_amd.engine import Engine
    from arle_amd.engine.scheduler import Scheduler, SchedulerConfig
    from arle_amd.sampling import Sampler

    cfg, _ = read_folder(folders["B"])
    rng = random.Random(seed)
    arrivals = []
    for i in range(10):
        params = SamplingParams(temperature=rng.choice([0.0, 0.0, 0.9]), top_p=rng.choice([1.0, 0.8]), seed=i,
                                logprobs=rng.random() < 0.3, repetition_penalty=rng.choice([1.0, 1.0, 1.0, 1.2]))
        arrivals.append((rng.randint(0, 18), random_tokens(rng.randint(1, 40), cfg["vocab_size"], 900 + 10 * seed + i),
                         params, rng.randint(1, 14), rng.choice([0, 1, 1, 2])))
    stops = tuple(rng.randrange(cfg["vocab_size"]) for _ in range(12))
    pages = rng.choice([14, 40])
    results = []
    for overlap in (True, False):
        eng = Engine.from_folder(folders["B"], dtype="float32", page_size=TINY["B"][1], num_pages=pages, max_slots=3,
                                 max_request_tokens=96)
        s = Scheduler(eng, Sampler(eng.device), SchedulerConfig(num_slots=3, chunked_prefill_size=16, max_num_batched_tokens=40,
                                                                max_seq_len=96, async_overlap=overlap), stop_token_ids=stops)
        ids, it = {}, 0
        while it < 600 and (s.has_work() or len(ids) < len(arrivals)):
            for j, (when, toks, params, budget, priority) in enumerate(arrivals):
                if when == it:
                    ids[j] = s.submit(toks, params, max_tokens=budget, priority=priority)
            s.iteration()
            it += 1
        assert not s.has_work() and len(ids) == len(arrivals)
        assert not eng.cache.slot_of
        for g in eng.cache.groups:
            g.check()
            assert g.pool.free_count == g.pool.num_pages
        results.append({j: (s.finished[i].generated, s.finished[i].finish_reason) for j, i in ids.items()})
        if overlap:
            assert s.stats.get("steps_ahead", 0) > 5
    assert results[0] == results[1]
