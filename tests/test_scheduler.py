"""The scheduler's decisions, on the CPU, against a fake engine that keeps the real cache
bookkeeping but computes nothing (the reference tests its scheduling logic the same way:
infer/src/scheduler/cuda/execution.rs:829-1075, budget.rs:330-545, decode.rs:940-960)."""
from types import SimpleNamespace

import pytest

from arle_amd.cache import CacheManager, OutOfPages, PagedNeed
from arle_amd.engine.scheduler import (ABORT, LENGTH, STOP, Request, Scheduler, SchedulerConfig, plan_prefill,
                                       retract_victim)
from arle_amd.sampling import SamplingParams

VOCAB = 97


def next_token(history):
    """The fake model: the next token is a function of the whole history, so any token fed
    wrongly, twice or out of order changes everything after it."""
    h = 0
    for t in history:
        h = (h * 31 + t + 1) % 1000003
    return h % VOCAB


class FakeEngine:
    def __init__(self, num_pages=64, page_size=4, slots=4, max_request_tokens=256):
        self.cache = CacheManager([PagedNeed(1, 16)], page_size=page_size, num_pages=num_pages,
                                  max_slots=slots, max_request_tokens=max_request_tokens)
        self.spec = SimpleNamespace(vocab_size=VOCAB, stop_token_ids=())
        self.history = {}
        self.steps = []

    def add_request(self, key):
        self.history[key] = []
        return self.cache.admit(key)

    def end_request(self, key):
        self.cache.release(key)
        del self.history[key]

    def step(self, entries):
        self.cache.append([(e.request, len(e.tokens)) for e in entries])
        self.cache.check()
        rows = []
        for e in entries:
            assert len(self.history[e.request]) + len(e.tokens) == self.cache.length(e.request)
            for i, t in enumerate(e.tokens):
                self.history[e.request].append(t)
                if i in e.want:
                    rows.append(next_token(self.history[e.request]))
        self.steps.append([(e.request, len(e.tokens), list(e.want)) for e in entries])
        return rows


class FakeSampler:
    def sample_with_logprobs(self, logits, rows):
        assert len(logits) == len(rows)
        wanted = any(p.logprobs for p, _, _, _ in rows)
        return list(logits), ([-0.5 - t for t in logits] if wanted else None)


def expected_output(prompt, n):
    hist, out = list(prompt), []
    for _ in range(n):
        out.append(next_token(hist))
        hist.append(out[-1])
    return out


def make(num_pages=64, page_size=4, slots=4, **cfg):
    eng = FakeEngine(num_pages, page_size, slots)
    return eng, Scheduler(eng, FakeSampler(), SchedulerConfig(num_slots=slots, **cfg))


def prompt(n, k=0):
    return [(7 * i + k) % VOCAB for i in range(n)]


def test_one_request_prefill_then_decode():
    eng, s = make()
    rid = s.submit(prompt(10), max_tokens=5)
    s.run_until_done()
    r = s.finished[rid]
    assert r.generated == expected_output(prompt(10), 5) and r.finish_reason == LENGTH
    assert eng.steps[0] == [(rid, 10, [9])]
    assert all(step == [(rid, 1, [0])] for step in eng.steps[1:]) and len(eng.steps) == 5
    assert not eng.cache.slot_of and eng.cache.free_pages() == [64]


def test_prompts_are_cut_into_portions_and_logits_asked_only_at_the_end():
    eng, s = make(chunked_prefill_size=4)
    rid = s.submit(prompt(10), max_tokens=2)
    s.run_until_done()
    assert eng.steps[:3] == [[(rid, 4, [])], [(rid, 4, [])], [(rid, 2, [1])]]
    assert s.finished[rid].generated == expected_output(prompt(10), 2)


def test_continuous_batching_mixes_decode_rows_and_portions_in_one_step():
    eng, s = make(chunked_prefill_size=8)
    a = s.submit(prompt(6, 1), max_tokens=6)
    s.iteration()                       # a's whole prompt
    b = s.submit(prompt(20, 2), max_tokens=3)
    plan = s.iteration()
    assert plan.kind == "mixed"
    assert eng.steps[-1] == [(a, 1, [0]), (b, 8, [])]   # decode rows first, then the portion
    s.run_until_done()
    assert s.finished[a].generated == expected_output(prompt(6, 1), 6)
    assert s.finished[b].generated == expected_output(prompt(20, 2), 3)
    assert s.stats["steps"]["mixed"] >= 2


def test_token_budget_is_never_exceeded_and_decode_rows_come_first():
    eng, s = make(num_pages=400, slots=4, max_num_batched_tokens=12, max_prefill_tokens=10,
                  chunked_prefill_size=6)
    ids = [s.submit(prompt(25, k), max_tokens=8) for k in range(4)]
    s.run_until_done()
    for step in eng.steps:
        decode = sum(n for _, n, _ in step if n == 1)
        assert sum(n for _, n, _ in step) <= 12
        assert sum(n for _, n, _ in step if n > 1) <= min(12 - decode, 10)
    for k, rid in enumerate(ids):
        assert s.finished[rid].generated == expected_output(prompt(25, k), 8)


def _req(i, remaining, generated=0, max_tokens=16, prompt_len=None):
    r = Request(i, prompt(prompt_len or remaining), SamplingParams(), max_tokens, 0)
    r.feed = list(r.prompt)
    r.generated = [1] * generated
    return r


def test_a_portion_that_does_not_fit_is_skipped_whole_not_shrunk():
    cfg = SchedulerConfig(max_num_batched_tokens=100, max_prefill_tokens=10, chunked_prefill_size=8)
    queue = [_req(0, 8), _req(1, 5), _req(2, 2), _req(3, 1)]
    picked = plan_prefill(queue, 0, cfg)
    # 8 fits (2 left); 5 does not and is skipped; 2 fits exactly; nothing left for the last
    assert [(r.id, n) for r, n in picked] == [(0, 8), (2, 2)]
    # FCFS among equals: queue order is the only priority
    picked = plan_prefill([_req(5, 4), _req(4, 4), _req(6, 4)], 0, cfg)
    assert [r.id for r, _ in picked] == [5, 4]
    # decode rows shrink the budget first, and cap portions by the long-prefill threshold
    cfg = SchedulerConfig(max_num_batched_tokens=10, max_prefill_tokens=10, chunked_prefill_size=8,
                          long_prefill_token_threshold=3)
    picked = plan_prefill([_req(0, 8), _req(1, 8)], 4, cfg)
    assert [(r.id, n) for r, n in picked] == [(0, 3), (1, 3)]
    # prefill_max_requests
    cfg = SchedulerConfig(prefill_max_requests=1)
    assert len(plan_prefill([_req(0, 8), _req(1, 8)], 0, cfg)) == 1
    # pages: the finishing portion asks for one token more (the first decoded token)
    asked = []
    plan_prefill([_req(0, 8), _req(1, 600)], 0, SchedulerConfig(), asked=asked)
    assert [(r.id, n) for r, n in asked] == [(0, 9), (1, 504)]     # the cut portion stops where the step has 8 + 504 = 512 rows


def test_retract_victim_is_least_progress_then_longest_prompt():
    a, b, c = _req(0, 1, generated=5, prompt_len=10), _req(1, 1, generated=2, prompt_len=10), _req(2, 1, generated=2, prompt_len=30)
    assert retract_victim([a, b, c]) is c
    assert retract_victim([a, b]) is b


def test_stop_token_is_not_emitted_and_max_tokens_is_exact():
    eng, s = make()
    p = prompt(9)
    out = expected_output(p, 6)
    stop = out[3]
    first = out.index(stop)
    rid = s.submit(p, SamplingParams(stop_token_ids=[stop]), max_tokens=6)
    rid2 = s.submit(p, SamplingParams(stop_token_ids=[stop], ignore_eos=True), max_tokens=6)
    s.run_until_done()
    assert s.finished[rid].generated == out[:first] and s.finished[rid].finish_reason == STOP
    assert s.finished[rid2].generated == out and s.finished[rid2].finish_reason == LENGTH
    # stop ids of the model itself
    eng, s = make()
    s.stop_token_ids = {out[0]}
    rid = s.submit(p, max_tokens=6)
    s.run_until_done()
    assert s.finished[rid].generated == [] and s.finished[rid].finish_reason == STOP


def test_rejections_and_the_length_contract():
    eng, s = make(num_pages=8, page_size=4)           # pool of 32 tokens
    assert s.max_request_len == 31 and s.max_request_input_len == 26
    empty = s.submit([], max_tokens=4)
    long = s.submit(prompt(26), max_tokens=4)
    assert s.finished[empty].finish_reason == LENGTH and s.finished[empty].generated == []
    assert s.finished[long].finish_reason == LENGTH and s.stats["rejected"] == 2
    ok = s.submit(prompt(25), max_tokens=100)          # clamped to 31 - 25 - 1 = 5
    s.run_until_done()
    assert len(s.finished[ok].generated) == 5
    assert not s.has_work() and eng.cache.free_pages() == [8]


def test_admission_needs_a_slot_and_pages_for_prompt_plus_one():
    eng, s = make(num_pages=10, page_size=4, slots=2)  # 40 tokens
    a = s.submit(prompt(20, 1), max_tokens=3)          # 21 tokens -> 6 pages
    b = s.submit(prompt(19, 2), max_tokens=3)          # 20 tokens -> 5 pages: does not fit beside a
    c = s.submit(prompt(10, 3), max_tokens=3)          # 11 tokens -> 3 pages: fits beside a
    s.iteration()
    live = set(eng.cache.slot_of)
    assert live == {a, c} and [r.id for r in s.waiting] == [b]   # b keeps its place in the queue
    s.run_until_done()
    for rid, (n, k) in zip((a, b, c), ((20, 1), (19, 2), (10, 3))):
        assert s.finished[rid].generated == expected_output(prompt(n, k), 3)


def test_when_pages_run_out_a_decoding_request_is_preempted_and_everything_still_finishes():
    # 4 requests of 10-token prompts are admitted against 4 * 11 = 44 tokens, then each wants to
    # grow by 24 more: the pool of 52 tokens cannot hold that
    eng, s = make(num_pages=13, page_size=4, slots=4)
    ids = [s.submit(prompt(10, k), max_tokens=24) for k in range(4)]
    s.run_until_done()
    assert s.stats["preemptions"] > 0
    for k, rid in enumerate(ids):
        r = s.finished[rid]
        # a preempted request keeps what it generated and feeds prompt + generated again
        assert r.generated == expected_output(prompt(10, k), 24) and r.finish_reason == LENGTH
    assert any(s.finished[rid].preemptions for rid in ids)
    assert not s.has_work() and not eng.cache.slot_of and eng.cache.free_pages() == [13]
    eng.cache.check()


def test_a_lone_request_that_cannot_grow_finishes_with_length():
    eng, s = make(num_pages=4, page_size=4, slots=2)    # 16 tokens; contract allows 15
    s.max_request_len, s.max_request_input_len = 100, 95  # lift the contract to reach the pool's edge
    rid = s.submit(prompt(12), max_tokens=50)
    s.run_until_done()
    r = s.finished[rid]
    assert r.finish_reason == LENGTH and len(r.generated) == 5   # 12 + 4 fed tokens fill the 16; the 5th is sampled, not fed
    assert r.generated == expected_output(prompt(12), 5)
    assert eng.cache.free_pages() == [4]


def test_a_lone_decoding_request_takes_pages_back_from_a_prompt_that_is_still_being_fed():
    # 8 pages of 4.  a (prompt 10, 12 to generate: 6 pages in the end) and b (prompt 18) enter together and are fed in
    # portions of 4; once a decodes, its growth is set aside and b, 12 tokens in and holding 3 pages, waits.  When a
    # needs its sixth page nothing is free and a is the only request that decodes: b, which has produced nothing,
    # gives its pages back and goes to the front of the queue, and a is not cut short.
    eng, s = make(num_pages=8, page_size=4, slots=2, chunked_prefill_size=4)
    a = s.submit(prompt(10, 1), max_tokens=12)
    b = s.submit(prompt(18, 2), max_tokens=3)
    s.run_until_done()
    ra, rb = s.finished[a], s.finished[b]
    assert ra.generated == expected_output(prompt(10, 1), 12) and ra.finish_reason == LENGTH
    assert rb.generated == expected_output(prompt(18, 2), 3) and rb.finish_reason == LENGTH
    assert rb.preemptions == 1 and ra.preemptions == 0 and s.stats["preemptions"] == 1
    assert eng.steps[2] == [(a, 2, [1]), (b, 4, [])] and eng.steps[14] == [(b, 4, [])]   # b is fed from its start again
    assert s.stats["tokens_prefilled"] == 10 + 12 + 18
    assert not s.has_work() and not eng.cache.slot_of and eng.cache.free_pages() == [8]
    eng.cache.check()


def test_config_is_validated():
    with pytest.raises(ValueError):
        SchedulerConfig(chunked_prefill_size=0).validate()
    with pytest.raises(ValueError):
        SchedulerConfig(num_slots=8, max_num_batched_tokens=4).validate()


def test_a_serving_scheduler_takes_its_portion_size_from_the_gpus_memory():
    """The vectors of the reference's own tests (infer/src/scheduler/types.rs:788-797,950-1000)."""
    from arle_amd.engine.scheduler import GIB, pick_chunked_prefill_size_for_hbm

    assert [pick_chunked_prefill_size_for_hbm(n * GIB) for n in (0, 22, 48, 80, 140)] == [2048, 2048, 4096, 8192, 16384]
    assert pick_chunked_prefill_size_for_hbm(35 * GIB) == 4096 and pick_chunked_prefill_size_for_hbm(90 * GIB) == 16384
    cfg = SchedulerConfig.runtime_defaults(8)
    assert (cfg.num_slots, cfg.chunked_prefill_size, cfg.max_num_batched_tokens, cfg.max_prefill_tokens,
            cfg.long_prefill_token_threshold, cfg.prefill_max_requests) == (8, 4096, 16384, 16384, 4096, None)
    cfg.validate()
    # nothing given: the portion follows the memory, the prompt tokens of a step the step's budget, and the cap on
    # portions beside decoding requests is no longer than a portion
    cfg = SchedulerConfig.runtime_defaults(8).resolve_runtime_envelope(22 * GIB)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens, cfg.long_prefill_token_threshold) == (2048, 16384, 2048)
    cfg = SchedulerConfig.runtime_defaults(4).resolve_runtime_envelope(288 * GIB)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens, cfg.long_prefill_token_threshold) == (16384, 16384, 4096)
    # what the caller gives stands
    cfg = SchedulerConfig.runtime_defaults(4).resolve_runtime_envelope(22 * GIB, 6144, 12288)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens) == (6144, 12288)
    # a tighter step never starves a long prompt: the portion is at most the step
    cfg = SchedulerConfig.runtime_defaults(4)
    cfg.max_num_batched_tokens = 1024
    cfg.resolve_runtime_envelope(288 * GIB)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens, cfg.long_prefill_token_threshold) == (1024, 1024, 1024)
    cfg.validate()
    cfg = SchedulerConfig.runtime_defaults(8)
    cfg.max_num_batched_tokens = 4096
    cfg.resolve_runtime_envelope(80 * GIB)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens) == (4096, 4096)
    cfg = SchedulerConfig.runtime_defaults(4).resolve_runtime_envelope(22 * GIB, 3072)
    assert (cfg.chunked_prefill_size, cfg.max_prefill_tokens) == (3072, 16384)


def test_sampling_params_greedy_rule():
    # infer/src/sampler.rs:82-84,178-
    assert SamplingParams().is_greedy()
    assert SamplingParams(temperature=0.7, top_k=1).is_greedy()
    assert not SamplingParams(temperature=0.7).is_greedy()
    assert not SamplingParams(temperature=0.0, top_p=0.9).is_greedy()
    assert not SamplingParams(temperature=0.0, min_p=0.1).is_greedy()
    assert SamplingParams(repetition_penalty=1.1).has_penalties() and not SamplingParams().has_penalties()


def test_abort_frees_a_request_in_any_phase():
    # the reference finishes a slot whose client has gone at the next cleanup
    # (infer/src/scheduler/cuda/runtime/scheduler_loop.rs:325-340); here by an explicit call
    eng, s = make(num_pages=64, slots=2, chunked_prefill_size=8)
    a = s.submit(prompt(20), max_tokens=50)          # will be prefilling (three portions)
    b = s.submit(prompt(5, 1), max_tokens=50)        # will be decoding
    c = s.submit(prompt(6, 2), max_tokens=50)        # waits: no slot
    s.iteration()
    assert [r.id for r in s.prefilling] == [a] and [r.id for r in s.decoding] == [b] and [r.id for r in s.waiting] == [c]
    free_before = eng.cache.free_pages()[0]
    assert s.abort(c) and s.finished[c].finish_reason == ABORT and not s.waiting
    assert eng.cache.free_pages()[0] == free_before          # a waiting request held nothing
    assert s.abort(a)                                         # mid-prefill: pages and slot come back
    assert not eng.cache.is_live(a) and s.finished[a].finish_reason == ABORT and not s.prefilling
    assert eng.cache.free_pages()[0] > free_before and eng.cache.free_slot_count == 1
    s.iteration()
    kept = list(s.decoding[0].generated)
    assert s.abort(b)                                         # decoding: what it generated stays on the record
    assert s.finished[b].generated == kept == expected_output(prompt(5, 1), len(kept)) and len(kept) >= 2
    assert not s.abort(b) and not s.abort(12345)              # finished already / never submitted
    eng.cache.check()
    assert eng.cache.free_pages()[0] == 64 and eng.cache.free_slot_count == 2 and not s.has_work()
    assert s.stats["aborted"] == 3
    # the scheduler goes on with new work in the freed slots
    d = s.submit(prompt(9, 3), max_tokens=4)
    s.run_until_done()
    assert s.finished[d].generated == expected_output(prompt(9, 3), 4)


def test_out_of_pages_on_a_prefill_only_step_idles_instead_of_running_an_empty_step():
    eng, s = make(num_pages=64, slots=2)

    calls = {"n": 0}
    real_step = eng.step

    def step(entries):
        calls["n"] += 1
        assert entries, "an empty step was run"
        if calls["n"] == 1:
            raise OutOfPages("the pool disagrees with the plan")
        return real_step(entries)

    eng.step = step
    rid = s.submit(prompt(7), max_tokens=3)
    plan = s.iteration()                      # the step is refused; nothing else to run: the iteration idles
    assert plan.kind == "prefill" and s.stats["steps"]["prefill"] == 0 and s.stats["steps_skipped"] == 1
    assert eng.cache.length(rid) == 0
    s.run_until_done()
    assert s.finished[rid].generated == expected_output(prompt(7), 3)


def test_logprobs_reach_the_request_only_when_asked_for():
    eng, s = make()
    a = s.submit(prompt(6), SamplingParams(logprobs=True), max_tokens=4)
    b = s.submit(prompt(7, 1), SamplingParams(), max_tokens=4)
    s.run_until_done()
    ra, rb = s.finished[a], s.finished[b]
    assert ra.logprobs == [-0.5 - t for t in ra.generated] and rb.logprobs == []
    assert len(ra.t_tokens) == 4 and ra.t_tokens == sorted(ra.t_tokens)


# -- decode steps launched before the last step's tokens are read ---------------------------------------------
from arle_amd.engine.batch import DeviceToken


class LazyChosen:
    """What the GPU sampler's `Chosen` is to the scheduler: tokens that can be fed on without being read."""

    def __init__(self, tokens, logprobs, log):
        self._tokens, self._logprobs, self.log = list(tokens), logprobs, log

    def feed(self, row):
        return DeviceToken(self._tokens, row)

    def tokens(self):
        self.log.append("read")
        return self._tokens

    def logprobs(self):
        return self._logprobs


class LazySampler(FakeSampler):
    def __init__(self):
        self.log = []

    def choose(self, logits, rows):
        self.draw_indices = [idx for _, _, idx, _ in rows]
        return LazyChosen(*self.sample_with_logprobs(logits, rows), self.log)


class LazyEngine(FakeEngine):
    """Takes a DeviceToken where a token id stands, as the real step does."""

    def step(self, entries):
        from arle_amd.engine.batch import StepEntry
        self.sampler_log.append("step")
        plain = [StepEntry(e.request, [t.source[t.row] if isinstance(t, DeviceToken) else t for t in e.tokens], e.want)
                 for e in entries]
        self.fed_from_device = sum(isinstance(e.tokens[0], DeviceToken) for e in entries)
        return super().step(plain)


def make_lazy(num_pages=64, page_size=4, slots=4, stop=(), **cfg):
    eng, sampler = LazyEngine(num_pages, page_size, slots), LazySampler()
    eng.sampler_log = sampler.log
    return eng, Scheduler(eng, sampler, SchedulerConfig(num_slots=slots, **cfg), stop_token_ids=stop), sampler


def run_both(submit, **kw):
    """The same requests with and without steps launched ahead: (records, scheduler) each."""
    out = []
    for overlap in (True, False):
        eng, s, _ = make_lazy(async_overlap=overlap, **kw)
        ids = submit(s)
        s.run_until_done()
        eng.cache.check()
        assert not eng.cache.slot_of and eng.cache.free_pages() == [kw.get("num_pages", 64)]
        out.append(([(s.finished[i].generated, s.finished[i].finish_reason, s.finished[i].logprobs) for i in ids], s))
    return out


def test_steps_launched_ahead_give_the_same_tokens():
    def submit(s):
        return [s.submit(prompt(10, k), SamplingParams(logprobs=k == 1), max_tokens=5 + 3 * k) for k in range(3)]
    (ahead, s_ahead), (plain, s_plain) = run_both(submit)
    assert ahead == plain
    assert [g for g, _, _ in ahead] == [expected_output(prompt(10, k), 5 + 3 * k) for k in range(3)]
    assert s_ahead.stats["steps_ahead"] >= 6 and "steps_ahead" not in s_plain.stats
    # no token is computed twice or in vain when requests end by their length
    assert s_ahead.stats["tokens_decoded"] == s_plain.stats["tokens_decoded"]


def test_a_step_ahead_is_launched_before_the_last_tokens_are_read():
    eng, s, sampler = make_lazy()
    s.submit(prompt(6), max_tokens=6)
    s.iteration()                        # the prompt; its token stays with the sampler
    assert sampler.log == ["step"]
    s.iteration()                        # the first decode step: launched from the token not yet read
    assert sampler.log == ["step", "step", "read"] and eng.fed_from_device == 1
    assert sampler.draw_indices == [1]   # the second draw of the request, though the host knew no token yet
    s.iteration()
    assert sampler.log == ["step", "step", "read", "step", "read"] and eng.fed_from_device == 1
    assert sampler.draw_indices == [2]
    s.run_until_done()
    assert s.finished[0].generated == expected_output(prompt(6), 6)


def test_a_stop_token_one_step_late_wastes_one_row_and_nothing_else():
    full = expected_output(prompt(8, 3), 12)
    stop = full[5]
    assert stop not in full[:5]
    def submit(s):
        return [s.submit(prompt(8, 3), max_tokens=12), s.submit(prompt(9, 1), max_tokens=12)]
    (ahead, s_ahead), (plain, s_plain) = run_both(submit, stop=(stop,))
    assert ahead == plain
    assert ahead[0][0] == full[:5] and ahead[0][1] == STOP      # the stop token is not emitted, nor what came after
    # the row that was launched for the stopped request before its stop token was read
    assert s_ahead.stats["tokens_decoded"] == s_plain.stats["tokens_decoded"] + 1


def test_arrivals_preemptions_and_penalties_fall_back_to_reading_first():
    def submit(s):
        ids = [s.submit(prompt(7, 1), max_tokens=20), s.submit(prompt(5, 2), SamplingParams(repetition_penalty=1.2), max_tokens=6)]
        for _ in range(4):
            s.iteration()
        ids.append(s.submit(prompt(12, 4), max_tokens=9))       # arrives while the others decode
        return ids
    (ahead, s_ahead), (plain, _) = run_both(submit, chunked_prefill_size=8)
    assert ahead == plain
    assert s_ahead.stats["steps_ahead"] > 0
    # a pool so small that decoding requests have to give pages back
    def crowd(s):
        return [s.submit(prompt(6, k), max_tokens=14) for k in range(3)]
    (ahead, s_ahead), (plain, s_plain) = run_both(crowd, num_pages=10, slots=3)
    assert ahead == plain and s_ahead.stats["preemptions"] > 0
    assert [g for g, _, _ in ahead] == [expected_output(prompt(6, k), 14) for k in range(3)]


def test_abort_while_a_step_is_pending():
    eng, s, _ = make_lazy()
    a, b = s.submit(prompt(6, 1), max_tokens=30), s.submit(prompt(7, 2), max_tokens=10)
    for _ in range(5):
        s.iteration()
    assert s.stats["steps_ahead"] >= 2
    kept = list(s.finished.get(a, s.decoding[0]).generated)
    assert s.abort(a)
    assert s.finished[a].generated == kept == expected_output(prompt(6, 1), len(kept))
    s.run_until_done()
    eng.cache.check()
    assert s.finished[b].generated == expected_output(prompt(7, 2), 10)
    assert not eng.cache.slot_of and eng.cache.free_pages() == [64] and not s.has_work()


def test_a_cut_portion_gives_up_the_tokens_that_stand_over_a_multiple_of_128_rows():
    cfg = SchedulerConfig(num_slots=16, chunked_prefill_size=512, long_prefill_token_threshold=512)
    long_one = Request(0, prompt(2000), SamplingParams(), 8, 0, feed=prompt(2000))
    assert plan_prefill([long_one], 8, cfg) == [(long_one, 504)]          # 8 + 504 = 512 rows
    assert plan_prefill([long_one], 0, cfg) == [(long_one, 512)]
    assert plan_prefill([long_one], 130, cfg) == [(long_one, 510)]        # 130 + 510 = 640
    short = Request(1, prompt(300), SamplingParams(), 8, 0, feed=prompt(300))
    assert plan_prefill([short], 8, cfg) == [(short, 300)]                # the end of a prompt is never cut
    # 460 tokens would make 768 rows, but the prompt would then need five steps instead of four
    assert plan_prefill([short, long_one], 8, cfg) == [(short, 300), (long_one, 512)]
    even = Request(2, prompt(2048), SamplingParams(), 8, 0, feed=prompt(2048))
    assert plan_prefill([even], 32, cfg) == [(even, 512)]                # 480 would add a fifth step
    longer = Request(3, prompt(3600), SamplingParams(), 8, 0, feed=prompt(3600))
    assert plan_prefill([short, longer], 8, cfg) == [(short, 300), (longer, 460)]     # 768 rows; eight steps either way
    small = SchedulerConfig(num_slots=16, chunked_prefill_size=200, long_prefill_token_threshold=200)
    assert plan_prefill([long_one], 8, small) == [(long_one, 200)]        # fewer than 128 tokens would stay
    off = SchedulerConfig(num_slots=16, chunked_prefill_size=512, long_prefill_token_threshold=512, step_row_alignment=0)
    assert plan_prefill([long_one], 8, off) == [(long_one, 512)]


@pytest.mark.parametrize("seed", range(12))
def test_random_traffic_gives_the_same_tokens_with_and_without_steps_launched_ahead(seed):
    """Requests of random lengths and budgets arriving while others run, stop tokens that some of them meet, a few
    with penalties, pools from generous to so small that requests are preempted, aborts in between: every request
    ends with the same tokens and reason whether steps are launched ahead or wait for their tokens, nothing is
    held at the end, and the cache's books are right after every iteration."""
    import random

    rng = random.Random(seed)
    slots, page_size = rng.choice([2, 3, 5]), rng.choice([2, 4])
    num_pages = rng.choice([12, 20, 64])
    chunk = rng.choice([3, 8, 16])
    arrivals = []
    for i in range(rng.randint(4, 10)):
        plen, budget = rng.randint(1, 18), rng.randint(1, 12)
        if -(-(plen + budget + 1) // page_size) > num_pages - 1:
            budget = 1
        params = SamplingParams(repetition_penalty=1.3) if rng.random() < 0.15 else SamplingParams(logprobs=rng.random() < 0.3)
        arrivals.append((rng.randint(0, 25), prompt(plen, i), params, budget))
    stops = {next_token(prompt(5, 1) + [3]), rng.randrange(VOCAB), rng.randrange(VOCAB), rng.randrange(VOCAB)}
    abort_at = rng.choice([None, 6, 11])
    results = []
    for overlap in (True, False):
        eng, s, _ = make_lazy(num_pages=num_pages, page_size=page_size, slots=slots, stop=tuple(stops),
                              async_overlap=overlap, chunked_prefill_size=chunk, max_num_batched_tokens=max(24, slots))
        ids, it = {}, 0
        while it < 400 and (s.has_work() or len(ids) < len(arrivals)):
            for j, (when, toks, params, budget) in enumerate(arrivals):
                if when == it:
                    ids[j] = s.submit(toks, params, max_tokens=budget)
            if abort_at == it and ids:
                s.abort(ids[min(ids)])
            s.iteration()
            eng.cache.check()
            it += 1
        assert not s.has_work() and len(ids) == len(arrivals)
        assert not eng.cache.slot_of and eng.cache.free_pages() == [num_pages]
        results.append({j: (s.finished[i].generated, s.finished[i].finish_reason, s.finished[i].logprobs)
                        for j, i in ids.items()})
        if overlap:
            ahead = s.stats.get("steps_ahead", 0)
    # (with steps launched ahead a request's end is found out one iteration late, so an abort may still reach a
    # request that the waiting run had just finished)
    aborted = {j for j in results[1] if ABORT in (results[0][j][1], results[1][j][1])}
    for j in results[1]:
        if j in aborted:     # an abort drops the token that was on its way: a prefix of what the waiting run kept
            a, b = results[0][j][0], results[1][j][0]
            assert a == b[:len(a)] or b == a[:len(b)]
        else:
            assert results[0][j] == results[1][j], j
    assert ahead > 0


def test_waiting_requests_are_ordered_by_priority_then_first_come():
    """infer/src/scheduler/cuda/runtime/tests.rs:172-215: a new request goes behind its equals, a requeued one in
    front of them, both behind every higher priority; here also: the scheduler serves them in that order."""
    from collections import deque
    from arle_amd.engine.scheduler import PRIORITY_HIGH, PRIORITY_LOW, PRIORITY_NORMAL, insert_waiting

    def req(label, priority):
        r = Request(0, [1], SamplingParams(), 1, 0, priority=priority)
        r.label = label
        return r

    waiting = deque([req("high", PRIORITY_HIGH), req("first-normal", PRIORITY_NORMAL)])
    insert_waiting(waiting, req("second-normal", PRIORITY_NORMAL), before_equal=False)
    assert [r.label for r in waiting] == ["high", "first-normal", "second-normal"]
    waiting = deque([req("high", PRIORITY_HIGH), req("queued-normal", PRIORITY_NORMAL)])
    insert_waiting(waiting, req("requeued-normal", PRIORITY_NORMAL), before_equal=True)
    assert [r.label for r in waiting] == ["high", "requeued-normal", "queued-normal"]
    insert_waiting(waiting, req("low", PRIORITY_LOW), before_equal=True)
    insert_waiting(waiting, req("late-high", PRIORITY_HIGH), before_equal=False)
    assert [r.label for r in waiting] == ["high", "late-high", "requeued-normal", "queued-normal", "low"]

    eng, s = make(slots=1)
    low = s.submit(prompt(5, 1), max_tokens=2, priority=PRIORITY_LOW)
    normal = s.submit(prompt(5, 2), max_tokens=2)
    high = s.submit(prompt(5, 3), max_tokens=2, priority=PRIORITY_HIGH)
    s.run_until_done()
    first_steps = [step[0][0] for step in eng.steps if step[0][1] == 5]      # the prompts, in the order they ran
    assert first_steps == [high, normal, low]
    assert all(s.finished[r].generated == expected_output(prompt(5, k), 2) for r, k in ((low, 1), (normal, 2), (high, 3)))
    with pytest.raises(ValueError):
        s.submit(prompt(3), priority=7)


def test_a_full_waiting_queue_refuses_the_next_request():
    """Back-pressure at intake (infer/src/scheduler/types.rs:132-133,598: `max_waiting_requests`, SchedulerFull):
    the request over the limit is refused and takes no id, and room comes back as the queue drains."""
    from arle_amd.engine.scheduler import SchedulerFull

    eng, s = make(slots=2, max_waiting_requests=3)
    ids = [s.submit(prompt(5, k), max_tokens=2) for k in range(3)]
    with pytest.raises(SchedulerFull):
        s.submit(prompt(5, 9), max_tokens=2)
    assert len(s.waiting) == 3 and s._next_id == 3
    s.iteration()                      # two are admitted: one place in the queue is free again
    ids.append(s.submit(prompt(5, 4), max_tokens=2))
    s.run_until_done()
    for k, rid in zip((0, 1, 2, 4), ids):
        assert s.finished[rid].generated == expected_output(prompt(5, k), 2)
    assert not eng.cache.slot_of


def fake_llm(eng, **cfg):
    """An LLM around the fake engine: what `LLM.__init__` sets, without a GPU."""
    from arle_amd.engine.api import LLM

    llm = LLM.__new__(LLM)
    llm.engine, llm.model_dir, llm.seed, llm.tokenizer, llm.last_stats = eng, None, 42, None, {}
    llm.sampler = FakeSampler()
    llm.sched_config = SchedulerConfig(num_slots=eng.cache.max_slots, **cfg)
    return llm


def test_a_stream_that_is_left_early_gives_everything_back():
    """A consumer that stops reading `generate_stream`, or an error inside an iteration, must not leave requests
    live in the engine's cache: the next call's requests start at id 0 again."""
    eng = FakeEngine(slots=2)
    llm = fake_llm(eng, chunked_prefill_size=4)
    stream = llm.generate_stream([prompt(9, 1), prompt(6, 2), prompt(7, 3)], max_tokens=8)
    first = next(stream)
    assert first.token_ids
    assert eng.cache.slot_of                    # requests are live in mid-stream
    stream.close()                              # what `break` in a for loop does
    assert not eng.cache.slot_of and eng.cache.free_pages() == [64]
    eng.cache.check()
    outs = llm.generate([prompt(9, 1), prompt(6, 2)], max_tokens=4)
    assert [o.response_token_ids for o in outs] == [expected_output(prompt(9, 1), 4), expected_output(prompt(6, 2), 4)]

    class Boom(RuntimeError):
        pass

    steps = {"n": 0}
    real_step = eng.step

    def failing_step(entries):
        steps["n"] += 1
        if steps["n"] == 3:
            raise Boom("the engine fails in mid-run")
        return real_step(entries)

    eng.step = failing_step
    with pytest.raises(Boom):
        llm.generate([prompt(9, 1), prompt(6, 2)], max_tokens=6)
    assert not eng.cache.slot_of and eng.cache.free_pages() == [64]
    eng.step = real_step
    outs = llm.generate([prompt(5, 5)], max_tokens=3)
    assert outs[0].response_token_ids == expected_output(prompt(5, 5), 3)


def test_the_native_planner_counts_pages_in_every_group_beside_the_decoders_reservations():
    """`plan_prefill` with a cache: a portion is skipped whole when one group cannot take its pages on top of what the
    decoding requests are reserved and what the portions before it took; a later, smaller one still goes in."""
    cache = CacheManager([PagedNeed(1, 16), PagedNeed(1, 16, page_size=8)], page_size=4, num_pages=16, max_slots=5,
                         max_request_tokens=64)       # 64 tokens in either group: 16 pages of 4, 8 pages of 8
    reqs = [Request(i, prompt(n), SamplingParams(), 8, 0, feed=prompt(n)) for i, n in enumerate([20, 30, 6, 3])]
    for r in reqs:
        cache.admit(r.id)
    decoder = Request(9, prompt(5), SamplingParams(), 40, 0, feed=prompt(5), generated=[1])
    cache.admit(decoder.id)
    cache.append([(decoder.id, 5)])                    # holds 2 pages of 4 and 1 page of 8
    cfg = SchedulerConfig(num_slots=5, step_row_alignment=0)
    asked = []
    picked = plan_prefill(reqs, 1, cfg, cache, growth=[(decoder.id, 11)], asked=asked)
    # the decoder's 11 more tokens: 2 pages of 4, 1 page of 8.  Left: 12 and 6.  20 + 1 tokens take 6 and 3 (left 6 and
    # 3); 30 + 1 would take 8 and 4: skipped whole; 6 + 1 take 2 and 1; 3 + 1 take 1 and 1
    assert [(r.id, n) for r, n in picked] == [(0, 20), (2, 6), (3, 3)]
    assert [(r.id, n) for r, n in asked] == [(0, 21), (2, 7), (3, 4)]
    assert cache.can_append([(decoder.id, 11), (0, 21), (2, 7), (3, 4)]) and not cache.can_append([(decoder.id, 11), (0, 21), (1, 31)])
    # without the reservation the long one fits too (14 and 7 pages free: 6 + 8 and 3 + 4), and nothing is left for the short ones
    picked = plan_prefill(reqs, 1, cfg, cache)
    assert [(r.id, n) for r, n in picked] == [(0, 20), (1, 30)]
    with pytest.raises(KeyError):
        plan_prefill([Request(77, prompt(4), SamplingParams(), 8, 0, feed=prompt(4))], 0, cfg, cache)


def _oracle_aligned(n, remaining, rows_before, align):
    """The rule of `aligned_portion` stated once more: a cut portion stops at the last multiple of `align` rows if at
    least `align` of its tokens stay and the prompt, in portions that short, needs no step more than in portions of n."""
    if align <= 0 or n >= remaining:
        return n
    over = (rows_before + n) % align
    shorter = n - over
    if over == 0 or shorter < align:
        return n
    steps = lambda portion: -(-remaining // portion)
    return shorter if steps(shorter) <= steps(n) else n


def _oracle_plan(queue, decode_rows, cfg, page_sizes, free, held, growth):
    """The planner's rule written out in Python for lists of numbers: held[g][id] pages that a request holds in group
    g with length[id] tokens; returns [(id, tokens, tokens its pages are asked for)]."""
    pages = lambda g, tokens: -(-tokens // page_sizes[g])
    reserved = [sum(max(0, pages(g, length + n) - held[g][rid]) for rid, length, n in growth) for g in range(len(page_sizes))]
    tokens_left = min(max(cfg.max_num_batched_tokens - decode_rows, 0), cfg.max_prefill_tokens)
    requests_left = len(queue) if cfg.prefill_max_requests is None else cfg.prefill_max_requests
    cap = max(1, min(cfg.chunked_prefill_size, cfg.long_prefill_token_threshold) if decode_rows > 0 else cfg.chunked_prefill_size)
    rows, out = decode_rows, []
    for rid, length, remaining, first in queue:
        n = min(remaining, cap)
        if remaining <= 0 or n > tokens_left or requests_left <= 0:
            continue
        n = _oracle_aligned(n, remaining, rows, cfg.step_row_alignment)
        asked = n + (1 if n == remaining and first else 0)
        need = [max(0, pages(g, length + asked) - held[g][rid]) for g in range(len(page_sizes))]
        if any(reserved[g] + need[g] > free[g] for g in range(len(page_sizes))):
            continue
        reserved = [a + b for a, b in zip(reserved, need)]
        out.append((rid, n, asked))
        tokens_left, requests_left, rows = tokens_left - n, requests_left - 1, rows + n
    return out


@pytest.mark.parametrize("seed", range(12))
def test_the_native_planner_and_admission_against_the_rules_written_out(seed):
    """Random queues, budgets, page lengths and pools: what `arle_plan_prefill`, `arle_aligned_portion` and
    `arle_admit` decide is what the rules say (scheduler/cuda/execution.rs:200-330, budget.rs:17-33 of the reference
    for the budget and the pages; the alignment is this engine's own), and a plan never asks for more than the step's
    budget or the pools hold."""
    import random

    from arle_amd.engine.scheduler import admit_waiting, aligned_portion

    rng = random.Random(1000 + seed)
    for _ in range(40):
        n, remaining = rng.randint(1, 700), rng.randint(1, 3000)
        n = min(n, remaining)
        rows, align = rng.randint(0, 300), rng.choice([0, 16, 64, 128])
        assert aligned_portion(n, remaining, rows, align) == _oracle_aligned(n, remaining, rows, align), (n, remaining, rows, align)
    for _ in range(25):
        page_sizes = [rng.choice([4, 8, 16]) for _ in range(rng.randint(1, 2))]
        base = min(page_sizes)
        num_pages = rng.randint(6, 40)
        needs = [PagedNeed(1, 16, page_size=p) for p in page_sizes]
        cache = CacheManager(needs, page_size=base, num_pages=num_pages, max_slots=12, max_request_tokens=base * num_pages)
        page_sizes = [g.page_size for g in cache.groups]   # needs of one kind share a group
        # requests in the middle of their prompts, and decoders
        held = [dict() for _ in page_sizes]
        reqs = []
        for rid in range(rng.randint(1, 6)):
            total = rng.randint(1, 60)
            done = rng.randint(0, total - 1) if rng.random() < 0.5 else 0
            r = Request(rid, prompt(total), SamplingParams(), rng.choice([0, 1, 8]), 0, feed=prompt(total))
            cache.admit(rid)
            try:
                if done:
                    cache.append([(rid, done)])
            except OutOfPages:
                done = 0
            r.fed = done
            reqs.append(r)
        decoders = []
        for rid in range(100, 100 + rng.randint(0, 3)):
            have = rng.randint(1, 20)
            cache.admit(rid)
            try:
                cache.append([(rid, have)])
            except OutOfPages:
                cache.release(rid)
                continue
            decoders.append((rid, have, rng.randint(1, 4)))
        free = cache.free_pages()
        for g, p in enumerate(page_sizes):
            for r in reqs:
                held[g][r.id] = -(-r.fed // p)
            for rid, have, _ in decoders:
                held[g][rid] = -(-have // p)
        cfg = SchedulerConfig(num_slots=12, max_num_batched_tokens=rng.choice([16, 40, 100]), max_prefill_tokens=rng.choice([16, 64, 100]),
                              chunked_prefill_size=rng.choice([8, 16, 48]), long_prefill_token_threshold=rng.choice([8, 16, 48]),
                              prefill_max_requests=rng.choice([None, 1, 2, 5]), step_row_alignment=rng.choice([0, 8, 16]))
        decode_rows = len(decoders)
        asked = []
        picked = plan_prefill(reqs, decode_rows, cfg, cache, growth=[(rid, n) for rid, _, n in decoders], asked=asked)
        want = _oracle_plan([(r.id, r.fed, r.remaining_prompt, r.max_tokens - len(r.generated) > 0) for r in reqs], decode_rows, cfg,
                            page_sizes, free, held, decoders)
        assert [(r.id, n) for r, n in picked] == [(rid, n) for rid, n, _ in want], (seed, cfg)
        assert [(r.id, n) for r, n in asked] == [(rid, a) for rid, _, a in want]
        assert sum(n for _, n in picked) + decode_rows <= max(cfg.max_num_batched_tokens, decode_rows)
        # what the plan asks for is what the cache can take in one go (the decoders' growth with it)
        grow = [(rid, n) for rid, _, n in decoders]
        if cache.can_append(grow):
            assert cache.can_append(grow + [(r.id, a) for r, a in asked])
        # admission: slots and pages for every target after the running requests' own
        running = [(r.fed, len(r.prompt) + 1) for r in reqs] + [(have, have + 6) for _, have, _ in decoders]
        waiting = [rng.randint(2, 80) for _ in range(rng.randint(1, 5))]
        slots = rng.randint(0, 3)
        got = admit_waiting(cache, slots, running, waiting)
        left = [free[g] - sum(max(0, -(-t // p) - -(-h // p)) for h, t in running) for g, p in enumerate(page_sizes)]
        expect = []
        for t in waiting:
            ok = slots > 0 and all(-(-t // p) <= left[g] for g, p in enumerate(page_sizes))
            expect.append(ok)
            if ok:
                slots -= 1
                left = [left[g] - -(-t // p) for g, p in enumerate(page_sizes)]
        assert got == expect, (seed, waiting, running)
