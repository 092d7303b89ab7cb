"""Continuous batching above the step function: admit, cut prompts into portions under a
token budget, decode, finish and free -- and what happens when pages run out.

One `iteration()` does, in the reference's order (infer/src/scheduler/cuda/runtime/scheduler_loop.rs:116-199,
infer/src/scheduler/cuda/execution.rs:385-425,669-800):

0. intake: a request joins the waiting queue behind every request of its own or a higher priority and before
   those of a lower one (infer/src/scheduler/cuda/runtime/helpers.rs:200-266); a preempted request goes back in
   front of its equals.
1. admission: a waiting request enters when a slot is free and the pool has pages for its
   prompt + 1 token after the same target of every running request is set aside; decode
   growth is not reserved (scheduler_loop.rs:202-315, budget.rs:17-33).  A request that does
   not fit stays in the queue, in order; later ones may still enter.
2. decode rows: every decoding request brings its last token.  If the pool cannot take one
   more token of each, the request with the fewest generated tokens (ties: the longest
   prompt) is preempted until it can (decode.rs:16-21,82-116); a lone request that still
   does not fit finishes with `length` (decode.rs:52-73), here only once no prompt that is still
   being fed holds pages either (see below).
3. prompt portions under the token budget min(max_num_batched_tokens - decode rows,
   max_prefill_tokens): per request min(remaining, chunked_prefill_size), also capped by
   long_prefill_token_threshold while rows are decoding; a portion that does not fit the
   remaining budget is skipped whole, not shrunk; queue order is the only priority
   (execution.rs:117-215,265-317, budget.rs:229-264).  Pages: each running decode's remaining
   growth min(max_tokens - generated, 4096) is set aside first (execution.rs:160-168).
4. one `Engine.step` with the decode rows first, then the portions; logits are asked only
   where a token is sampled (the reference computes them for every portion and discards them).
5. sampling and transitions: a stop token ends the request without being emitted
   (prefill.rs:426-479, decode.rs:784-808); `max_tokens` ends it with `length`.
6. finished requests give their pages and slot back.  `abort(id)` ends a request in any phase at once and
   frees what it holds, as the reference does when a client has gone (scheduler_loop.rs:325-340: a closed
   delta channel finishes the slot at the next cleanup); its finish reason here is `abort`.

Kept differently on purpose: a preempted request keeps the tokens it has generated and
feeds prompt + generated again when it re-enters (the reference drops them and generates
anew); decode rows and prompt portions always share one step (the reference's default
runs two forwards, `Split`); and before the only decoding request is cut short for want of a page, the
prompts that are still being fed give theirs back, the one admitted last first: they have produced
nothing yet and wait in front of the queue, where the reference ends the decoding request with `length`
while they keep their pages.
"""
from __future__ import annotations

import ctypes
import inspect

import time
from collections import deque
from dataclasses import dataclass, field

from ..cache import native
from ..cache.pages import OutOfPages
from ..sampling.params import SamplingParams
from .batch import StepEntry

LENGTH, STOP, ABORT = "length", "stop", "abort"
PRIORITY_LOW, PRIORITY_NORMAL, PRIORITY_HIGH = 0, 1, 2   # infer/src/scheduler/types.rs:553-564
REQUEST_INPUT_SLACK_TOKENS = 5      # infer/src/scheduler/types.rs:499
DECODE_RESERVATION_CLIP = 4096      # infer/src/scheduler/cuda/budget.rs:3


GIB = 1 << 30


def pick_chunked_prefill_size_for_hbm(gpu_total_bytes: int) -> int:
    """The longest prompt portion of one request by the GPU's whole memory: the larger the GPU, the larger
    the portion (infer/src/scheduler/types.rs:251-260).  An MI355X (288 GB) takes 16,384 tokens."""
    if gpu_total_bytes < 35 * GIB:
        return 2048
    if gpu_total_bytes < 60 * GIB:
        return 4096
    if gpu_total_bytes < 90 * GIB:
        return 8192
    return 16384


class SchedulerFull(RuntimeError):
    pass


@dataclass
class SchedulerConfig:
    """Names and defaults of infer/src/scheduler/types.rs:63-238 (the flags of `infer`)."""

    num_slots: int = 4
    chunked_prefill_size: int = 512
    max_num_batched_tokens: int = 16384
    max_prefill_tokens: int = 16384
    prefill_max_requests: int | None = None
    long_prefill_token_threshold: int = 512
    max_waiting_requests: int = 256
    max_seq_len: int | None = None
    async_overlap: bool = True   # launch a decode step from the last one's tokens on the GPU, read those back after
    step_row_alignment: int = 128  # a portion that does not end its prompt stops where the step's rows are a multiple
                                   # of this (aligned_portion; 0: portions as the reference cuts them)

    @classmethod
    def runtime_defaults(cls, num_slots: int) -> "SchedulerConfig":
        """What a serving scheduler starts from, before the GPU's memory is known
        (infer/src/scheduler/types.rs:270-278); the plain defaults above are those of the reference's
        accounting layer without a GPU."""
        return cls(num_slots=num_slots, chunked_prefill_size=4096, max_num_batched_tokens=16384,
                   long_prefill_token_threshold=4096)

    def resolve_runtime_envelope(self, gpu_total_bytes: int, chunked_prefill_size: int | None = None,
                                 max_prefill_tokens: int | None = None) -> "SchedulerConfig":
        """Settle the sizes of a step on a given GPU (infer/src/scheduler/types.rs:315-334).  A value that
        the caller gives stands; chunked_prefill_size otherwise follows the GPU's memory and never exceeds
        max_num_batched_tokens, max_prefill_tokens otherwise is the whole step's budget, and
        long_prefill_token_threshold is no longer than a portion."""
        self.chunked_prefill_size = (chunked_prefill_size if chunked_prefill_size is not None
                                     else pick_chunked_prefill_size_for_hbm(gpu_total_bytes))
        if self.max_num_batched_tokens > 0:
            self.chunked_prefill_size = min(self.chunked_prefill_size, self.max_num_batched_tokens)
        self.max_prefill_tokens = max_prefill_tokens if max_prefill_tokens is not None else self.max_num_batched_tokens
        self.long_prefill_token_threshold = min(self.long_prefill_token_threshold, self.chunked_prefill_size)
        return self

    def validate(self) -> None:
        for name in ("num_slots", "chunked_prefill_size", "max_num_batched_tokens",
                     "max_prefill_tokens", "long_prefill_token_threshold", "max_waiting_requests"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive")
        if self.prefill_max_requests is not None and self.prefill_max_requests <= 0:
            raise ValueError("prefill_max_requests must be positive when set")
        if self.max_num_batched_tokens < self.num_slots:
            raise ValueError("max_num_batched_tokens must hold one decode row per slot")


@dataclass
class Request:
    id: int
    prompt: list
    sampling: SamplingParams
    max_tokens: int
    seed: int
    feed: list = field(default_factory=list)       # tokens that have to pass through the model
    fed: int = 0                                   # how many of them have
    generated: list = field(default_factory=list)
    logprobs: list = field(default_factory=list)   # of the generated tokens, when the request asks for them
    phase: str = "waiting"                         # waiting | prefilling | decoding | finished
    finish_reason: str | None = None
    preemptions: int = 0
    t_submit: float = 0.0
    t_first_token: float | None = None
    t_finish: float | None = None
    t_tokens: list = field(default_factory=list)   # when each generated token arrived (for the time per output token)
    pending: int = 0                               # tokens that a launched step has chosen and the host has not read yet
    priority: int = PRIORITY_NORMAL                # a higher one is served first among the waiting

    @property
    def remaining_prompt(self) -> int:
        return len(self.feed) - self.fed


@dataclass
class StepPlan:
    decode: list          # requests that bring one token
    prefill: list         # (request, tokens of this portion)

    @property
    def kind(self) -> str:
        if self.decode and self.prefill:
            return "mixed"
        return "decode" if self.decode else ("prefill" if self.prefill else "idle")


class _ChosenNow:
    """What a sampler that answers at once chose, in the shape of the sampler's `Chosen`."""

    def __init__(self, tokens, logprobs):
        self._tokens, self._logprobs = list(tokens), logprobs

    def tokens(self):
        return self._tokens

    def logprobs(self):
        return self._logprobs


def insert_waiting(waiting: deque, req, before_equal: bool) -> None:
    """Put `req` into the waiting queue: before the first request of a lower priority; among its equals behind
    them (a new request: first come, first served) or in front of them (`before_equal`: a request that was
    running already and gave its pages back).  infer/src/scheduler/cuda/runtime/helpers.rs:200-266; its tests
    runtime/tests.rs:172-215."""
    at = len(waiting)
    for i, queued in enumerate(waiting):
        if req.priority > queued.priority or (before_equal and req.priority == queued.priority):
            at = i
            break
    waiting.insert(at, req)


def retract_victim(decoding: list):
    """Fewest generated tokens first; ties: the longest prompt (decode.rs:16-21).  Decided by the native
    runtime core."""
    n = len(decoding)
    generated = (ctypes.c_int * n)(*[len(r.generated) for r in decoding])
    prompts = (ctypes.c_int * n)(*[len(r.prompt) for r in decoding])
    return decoding[native.lib().arle_retract_victim(n, generated, prompts)]


def aligned_portion(n: int, remaining: int, rows_before: int, align: int) -> int:
    """How many of the n tokens that a prompt with `remaining` tokens could bring to a step of `rows_before` rows it
    brings.  The matrix products of a step run in tiles of 128 and 256 rows: 8 decoded tokens beside a portion of 512
    are 520 rows and cost a tenth more than 512 (measured on MI355X, Qwen3-4B shape: 9.8 against 8.7 ms).  So a
    portion that is cut anyway gives up the few tokens that stand over a multiple of `align` rows, if at least
    `align` tokens stay and the prompt does not need one more step for it (a 2,048-token prompt in portions of 512
    stays at four steps).  Worked out by the native runtime core."""
    return int(native.lib().arle_aligned_portion(int(n), int(remaining), int(rows_before), int(align)))


def plan_prefill(queue, decode_rows: int, cfg: SchedulerConfig, cache=None, growth=(), asked: list | None = None) -> list:
    """Pick portions of queued prompts for this step: [(request, tokens)], by the native runtime core
    (`arle_plan_prefill` in csrc/host/runtime.cpp, which also counts the pages in every group of the cache).

    queue: prefilling requests in queue order.  cache: the CacheManager whose pools have to take the portions
    (None: pages are not looked at); growth: [(request id, tokens)] that the decoding requests are reserved before
    any portion.  asked: a list that receives (request, tokens its pages were asked for) of the picked ones: a
    portion that completes its prompt asks for one token more, the first decoded one.
    """
    n_queue = len(queue)
    if n_queue == 0:
        return []
    groups = list(cache.groups) if cache is not None else []
    n_groups, n_decode = len(groups), len(growth)
    handles = (ctypes.c_void_p * max(n_groups, 1))(*[g._h for g in groups])
    decode_keys = (ctypes.c_longlong * max(n_groups * n_decode, 1))(*[g._ids[key] for g in groups for key, _ in growth])
    decode_growth = (ctypes.c_int * max(n_decode, 1))(*[int(n) for _, n in growth])
    queue_keys = (ctypes.c_longlong * max(n_groups * n_queue, 1))(*[g._ids[r.id] for g in groups for r in queue])
    remaining = (ctypes.c_int * n_queue)(*[int(r.remaining_prompt) for r in queue])
    first = (ctypes.c_int * n_queue)(*[1 if r.max_tokens - len(r.generated) > 0 else 0 for r in queue])
    picked, page_tokens = (ctypes.c_int * n_queue)(), (ctypes.c_int * n_queue)()
    count = native.lib().arle_plan_prefill(
        n_groups, handles, n_decode, decode_keys, decode_growth, n_queue, queue_keys, remaining, first, int(decode_rows),
        int(cfg.max_num_batched_tokens), int(cfg.max_prefill_tokens),
        -1 if cfg.prefill_max_requests is None else int(cfg.prefill_max_requests), int(cfg.chunked_prefill_size),
        int(cfg.long_prefill_token_threshold), int(cfg.step_row_alignment), picked, page_tokens)
    if count < 0:
        raise KeyError("a request of the plan has no block table in the cache")
    out = [(r, picked[j]) for j, r in enumerate(queue) if picked[j] > 0]
    if asked is not None:
        asked.extend((r, page_tokens[j]) for j, r in enumerate(queue) if picked[j] > 0)
    return out


def admit_waiting(cache, free_slots: int, running, waiting) -> list:
    """Which of the waiting requests enter now (a list of booleans, in queue order), by the native runtime core
    (`arle_admit`): a free slot and, in every group, pages for prompt + 1 after the same target of every running
    request is set aside.  running: [(tokens cached, target tokens)]; waiting: [target tokens]."""
    if not waiting:
        return []
    groups = list(cache.groups)
    n_groups = len(groups)
    sizes = (ctypes.c_int * max(n_groups, 1))(*[g.page_size for g in groups])
    free = (ctypes.c_int * max(n_groups, 1))(*cache.free_pages())
    lengths = (ctypes.c_int * max(len(running), 1))(*[int(have) for have, _ in running])
    targets = (ctypes.c_int * max(len(running), 1))(*[int(target) for _, target in running])
    wanted = (ctypes.c_int * len(waiting))(*[int(t) for t in waiting])
    admit = (ctypes.c_int * len(waiting))()
    native.lib().arle_admit(n_groups, sizes, free, int(free_slots), len(running), lengths, targets, len(waiting), wanted, admit)
    return [bool(a) for a in admit]


class Scheduler:
    def __init__(self, engine, sampler, config: SchedulerConfig | None = None, seed: int = 42,
                 stop_token_ids=()):
        self.cfg = config or SchedulerConfig()
        self.cfg.validate()
        self.engine = engine
        # the logits of a step are sampled from before the next step is launched: a captured step need not copy them
        self._step_options = {"borrow_logits": True} if "borrow_logits" in inspect.signature(engine.step).parameters else {}
        self.cache = engine.cache
        self.sampler = sampler
        self.seed = seed
        self.stop_token_ids = set(stop_token_ids)
        self.waiting: deque = deque()
        self.prefilling: list = []
        self.decoding: list = []
        self.finished: dict = {}
        self._next_id = 0
        self._pending = None    # (requests, Chosen) of the step whose tokens have not been read back
        pool_tokens = self.cache.pool_tokens()
        context = self.cfg.max_seq_len or pool_tokens
        context = min(context, self.cache.request_capacity)
        # infer/src/scheduler/types.rs:511-553
        self.max_request_len = min(max(context - 1, 0), max(pool_tokens - 1, 0))
        self.max_request_input_len = max(self.max_request_len - REQUEST_INPUT_SLACK_TOKENS, 0)
        self.stats = {"steps": {"decode": 0, "prefill": 0, "mixed": 0}, "tokens_prefilled": 0,
                      "tokens_decoded": 0, "preemptions": 0, "rejected": 0, "aborted": 0, "pages_high_water": 0}

    # -- intake ---------------------------------------------------------------------------
    def submit(self, prompt_tokens, sampling: SamplingParams | None = None,
               max_tokens: int | None = None, priority: int = PRIORITY_NORMAL) -> int:
        """Queue a request; returns its id.  Rejections finish at once with `length` and no tokens
        (infer/src/scheduler/cuda/runtime/admission.rs:71-120)."""
        sampling = sampling or SamplingParams()
        if len(self.waiting) >= self.cfg.max_waiting_requests:
            raise SchedulerFull(f"{len(self.waiting)} requests are waiting already")
        rid = self._next_id
        self._next_id += 1
        prompt = [int(t) for t in prompt_tokens]
        if max_tokens is None:
            max_tokens = sampling.max_new_tokens if sampling.max_new_tokens is not None else self.max_request_len
        seed = sampling.seed if sampling.seed is not None else (self.seed * 0x9E3779B1 + rid) & ((1 << 63) - 1)
        if priority not in (PRIORITY_LOW, PRIORITY_NORMAL, PRIORITY_HIGH):
            raise ValueError("priority is PRIORITY_LOW, PRIORITY_NORMAL or PRIORITY_HIGH")
        req = Request(rid, prompt, sampling, int(max_tokens), seed, feed=list(prompt), t_submit=time.perf_counter(),
                      priority=int(priority))
        if not prompt or len(prompt) >= self.max_request_input_len or req.max_tokens <= 0:
            self.stats["rejected"] += 1
            self._finish(req, LENGTH)
            self.finished[rid] = req
            return rid
        req.max_tokens = min(req.max_tokens, max(self.max_request_len - len(prompt) - 1, 0))
        insert_waiting(self.waiting, req, before_equal=False)
        return rid

    def abort(self, rid: int, reason: str = ABORT) -> bool:
        """End request `rid` now, whatever its phase: out of the queue, or its pages and slot given back.
        True if it was still running or waiting; False if it had finished already or was never submitted.
        The tokens it has generated so far stay on its record (finish reason `abort`; `stop` when the caller
        has found a stop string in its text, which the scheduler does not see)."""
        for req in self.waiting:
            if req.id == rid:
                self.waiting.remove(req)
                self._finish(req, reason)
                self.finished[rid] = req
                self.stats["aborted"] += reason == ABORT
                return True
        for group in (self.prefilling, self.decoding):
            for req in group:
                if req.id == rid and req.phase != "finished":
                    self._finish(req, reason)
                    self.stats["aborted"] += reason == ABORT
                    self._cleanup()
                    return True
        return False

    def close(self) -> None:
        """End every request that has not finished (finish reason `abort`) and read what is still pending, so that
        no slot or page stays held: what a caller does that walks away from a scheduler in mid-run (a consumer that
        stops reading a stream, an error between two iterations).  Harmless when nothing is left."""
        for req in list(self.waiting) + list(self.prefilling) + list(self.decoding):
            if req.phase != "finished":
                self.abort(req.id)
        try:
            self._settle()
        finally:
            self._cleanup()

    # -- one iteration ------------------------------------------------------------------------
    def has_work(self) -> bool:
        return bool(self.waiting or self.prefilling or self.decoding or self._pending is not None)

    def iteration(self) -> StepPlan:
        """One step.  The tokens that a step chooses stay on the GPU until the next iteration reads them
        (the reference launches in iteration i and reads back in i + 1: infer/src/scheduler/cuda/execution.rs:676-708).
        The next step is planned and launched first, its decode rows fed from the tokens on the GPU, and the last
        step's tokens are read while it runs; a request that met a stop token is found out one step late, and
        the row launched for it has run in vain.  Where the plan needs a token's value or a request's true end
        (a request about to reach its length, pages running out and somebody to preempt, penalties over the
        tokens so far), the tokens are read first and the step follows."""
        if self._pending is not None and not self._can_plan_ahead():
            self._settle()
            self._cleanup()     # what the read tokens finished gives its slot and pages back before the plan
        self._admit()
        plan = self._plan()
        if plan.kind != "idle":
            self._run(plan)     # launches, then reads what was pending before
        else:
            self._settle()
        if not self.cfg.async_overlap or (self._pending is not None and not hasattr(self._pending[1], "feed")):
            self._settle()      # nothing to gain from waiting: the tokens are on the host already
        self._cleanup()
        return plan

    def run_until_done(self, max_iterations: int = 1 << 30) -> None:
        idle = 0
        for _ in range(max_iterations):
            if not self.has_work():
                return
            plan = self.iteration()
            idle = idle + 1 if plan.kind == "idle" else 0
            if idle > 2:
                raise RuntimeError("scheduler makes no progress: a waiting request can never be admitted")

    # -- admission ------------------------------------------------------------------------------
    def _admit(self) -> None:
        if not self.waiting:
            return
        running = [(self.cache.length(r.id), len(r.feed) + 1) for r in self.prefilling + self.decoding]
        waiting = list(self.waiting)
        enters = admit_waiting(self.cache, self.cache.free_slot_count, running, [len(r.feed) + 1 for r in waiting])
        deferred = deque()
        for req, goes_in in zip(waiting, enters):
            if not goes_in:
                deferred.append(req)
                continue
            self.engine.add_request(req.id)
            req.phase = "prefilling"
            req.fed = 0
            self.prefilling.append(req)
        self.waiting = deferred

    # -- planning -------------------------------------------------------------------------------
    def _plan(self) -> StepPlan:
        decode = list(self.decoding)
        # pages run out while decoding: preempt until one more token of each fits
        while decode and not self.cache.can_append([(r.id, 1) for r in decode]):
            if len(decode) == 1:
                # nobody else is decoding.  A prompt that is still being fed has produced nothing yet: the one
                # admitted last gives its pages back and waits, before a request that is generating is cut short.
                holders = [r for r in self.prefilling if r.phase == "prefilling" and self.cache.length(r.id) > 0]
                if holders:
                    self._preempt(holders[-1])
                    continue
                self._finish(decode.pop(), LENGTH)
                break
            victim = retract_victim(decode)
            decode.remove(victim)
            self._preempt(victim)
        growth = [(r.id, min(max(r.max_tokens - len(r.generated), 0), DECODE_RESERVATION_CLIP))
                  for r in decode]
        growth = [(k, n) for k, n in growth if n > 0]

        prefill = plan_prefill(self.prefilling, len(decode), self.cfg, self.cache, growth)
        if not decode and not prefill and self.prefilling:
            # nothing is decoding and no portion fits beside the reservations: the pool is
            # simply too small for the queue's head portion; try it alone against the free pages
            req = self.prefilling[0]
            n = min(req.remaining_prompt, self.cfg.chunked_prefill_size, self.cfg.max_prefill_tokens,
                    self.cfg.max_num_batched_tokens)
            if n > 0 and self.cache.can_append([(req.id, n)]):
                prefill = [(req, n)]
        return StepPlan(decode, prefill)

    # -- execution --------------------------------------------------------------------------------
    def _run(self, plan: StepPlan) -> None:
        entries, sampled = [], []
        before = self._pending
        fed_from = {id(r): i for i, r in enumerate(before[0])} if before is not None else {}
        for r in plan.decode:
            # the request's last token: known, or still on the GPU where the step before chose it
            last = before[1].feed(fed_from[id(r)]) if r.pending else r.generated[-1]
            entries.append(StepEntry(r.id, [last], [0]))
            sampled.append(r)
        for r, n in plan.prefill:
            completes = n == r.remaining_prompt
            entries.append(StepEntry(r.id, r.feed[r.fed:r.fed + n], [n - 1] if completes else []))
            if completes:
                sampled.append(r)
        try:
            logits = self.engine.step(entries, **self._step_options)
        except OutOfPages:
            # planning said it fits; if the pool disagrees, nothing was changed: skip the portions
            if not plan.prefill:
                raise
            if not plan.decode:
                self.stats["steps_skipped"] = self.stats.get("steps_skipped", 0) + 1
                return None      # nothing else to run: this iteration idles, the next one plans anew
            return self._run(StepPlan(plan.decode, []))
        self.stats["steps"][plan.kind] += 1
        self.stats["tokens_decoded"] += len(plan.decode)
        self.stats["tokens_prefilled"] += sum(n for _, n in plan.prefill)
        held = max((g.pool.num_pages - g.pool.free_count for g in self.cache.groups), default=0)
        self.stats["pages_high_water"] = max(self.stats["pages_high_water"], held)
        for r, n in plan.prefill:
            r.fed += n
        if before is not None:
            self.stats["steps_ahead"] = self.stats.get("steps_ahead", 0) + 1
        self._pending = None
        if sampled:
            self._choose(logits, sampled, plan)     # queued behind the step
        if before is not None:                      # the step before: its tokens are there by now
            ahead, self._pending = self._pending, before
            self._settle()
            self._pending = ahead

    def _choose(self, logits, sampled: list, plan: StepPlan) -> None:
        """Queue the sampling of a step's wanted rows; what it chooses is read by `_settle`."""
        rows = [(r.sampling, r.seed, len(r.generated) + r.pending, r.generated) for r in sampled]
        if hasattr(self.sampler, "choose"):
            chosen = self.sampler.choose(logits, rows)
        else:   # a sampler that answers at once
            chosen = _ChosenNow(*self.sampler.sample_with_logprobs(logits, rows))
        for r in sampled:
            r.pending += 1
            if r.phase == "prefilling":     # its prompt is through: the next step decodes it, whatever the token is
                self.prefilling.remove(r)
                r.phase = "decoding"
                self.decoding.append(r)
        self._pending = (sampled, chosen, plan)

    def _settle(self) -> None:
        """Read the pending step's tokens and apply them: a request that has finished meanwhile (a stop token
        one step earlier, an abort) takes none."""
        if self._pending is None:
            return
        sampled, chosen, _ = self._pending
        self._pending = None
        tokens, logprobs = chosen.tokens(), chosen.logprobs()
        now = time.perf_counter()
        for i, (r, tok) in enumerate(zip(sampled, tokens)):
            r.pending -= 1
            if r.phase == "finished":
                continue
            wants = logprobs is not None and r.sampling.logprobs
            self._apply_token(r, int(tok), now, float(logprobs[i]) if wants else None)

    # -- planning before the last step's tokens are known -------------------------------------------
    def _can_plan_ahead(self) -> bool:
        if not self.cfg.async_overlap:
            return False
        sampled, chosen, _ = self._pending
        if not hasattr(chosen, "feed"):
            return False
        for r in sampled:
            if r.phase != "decoding":
                continue
            if r.sampling.has_penalties() or len(r.generated) + r.pending >= r.max_tokens:
                return False    # the token's value is needed, or it is the request's last
        # one more token of every decoding request must fit without anybody giving pages back
        return self.cache.can_append([(r.id, 1) for r in self.decoding if r.phase == "decoding"])

    def _apply_token(self, r: Request, tok: int, now: float, logprob: float | None = None) -> None:
        if r.t_first_token is None:
            r.t_first_token = now
        stops = self.stop_token_ids | set(r.sampling.stop_token_ids)
        if tok in stops and not r.sampling.ignore_eos:
            self._finish(r, STOP)  # the stop token is not emitted
            return
        r.generated.append(tok)
        r.t_tokens.append(now)
        if logprob is not None:
            r.logprobs.append(logprob)
        r.feed.append(tok)
        r.fed = len(r.feed) - 1  # the new token is fed by the next decode row
        if len(r.generated) >= r.max_tokens:
            self._finish(r, LENGTH)

    # -- transitions ------------------------------------------------------------------------------
    def _finish(self, r: Request, reason: str) -> None:
        r.phase = "finished"
        r.finish_reason = reason
        r.t_finish = time.perf_counter()

    def _preempt(self, r: Request) -> None:
        """Give a request's pages back and queue it again, at the front."""
        (self.decoding if r in self.decoding else self.prefilling).remove(r)
        self.engine.end_request(r.id)
        r.phase = "waiting"
        r.fed = 0
        r.preemptions += 1
        self.stats["preemptions"] += 1
        insert_waiting(self.waiting, r, before_equal=True)

    def _cleanup(self) -> None:
        for group in (self.prefilling, self.decoding):
            for r in [r for r in group if r.phase == "finished"]:
                group.remove(r)
                if self.cache.is_live(r.id):
                    self.engine.end_request(r.id)
                self.finished[r.id] = r
