"""The Python entry point: load a model, generate for a list of prompts.

    from arle_amd import LLM
    llm = LLM("path/to/model")                       # config.json + safetensors
    outs = llm.generate([[1, 2, 3]], max_tokens=16)  # greedy
    outs[0].response_token_ids, outs[0].finish_reason, outs[0].usage

Request and result follow the reference's engine facade: `CompletionRequest{prompt,
max_tokens, sampling, ...}` -> `CompletionOutput{text, finish_reason, usage,
prompt_token_ids, response_token_ids}` (infer/src/server_engine/types.rs:10-60,147-185).
Prompts are token ids; text goes through the folder's tokenizer.json when the `tokenizers`
package and the file are there.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field

from ..sampling import Sampler, SamplingParams
from .engine import Engine
from .scheduler import STOP, Scheduler, SchedulerConfig


@dataclass
class TokenUsage:
    prompt_tokens: int
    completion_tokens: int

    @property
    def total_tokens(self) -> int:
        return self.prompt_tokens + self.completion_tokens


@dataclass
class CompletionOutput:
    text: str | None
    finish_reason: str            # "length" | "stop"
    usage: TokenUsage
    prompt_token_ids: list
    response_token_ids: list
    ttft_s: float | None = None   # submit -> first token
    tpot_s: float | None = None   # mean time per output token after the first
    token_logprobs: list = field(default_factory=list)   # log-probability of every generated token, if asked for


def _gpu_total_bytes(device) -> int:
    import torch

    device = torch.device(device)
    return torch.cuda.get_device_properties(device).total_memory if device.type == "cuda" else 0


def check_stop_sequences(text: str, stops) -> tuple:
    """(True, where the stop string begins) for the first of `stops`, in their order, that `text` holds; else
    (False, how much of `text` may be handed on): all but as many bytes at its end as the longest stop string
    has, in case one straddles the end of what is decoded so far (infer/src/scheduler/cuda/request.rs:396-413).
    Positions are in characters; empty stop strings do not count."""
    for stop in stops:
        if stop and stop in text:
            return True, text.index(stop)
    hold = max((len(stop.encode("utf-8")) for stop in stops), default=0)
    raw = text.encode("utf-8")
    safe = raw[:max(0, len(raw) - hold)].decode("utf-8", errors="ignore")   # back to the boundary of a character
    return False, len(safe)


@dataclass
class CompletionStreamDelta:
    """What one request has newly produced (the reference's CompletionStreamDelta,
    infer/src/server_engine/types.rs:68-81): the tokens that the host has read since the last delta, their text
    if there is a tokenizer, their log-probabilities if asked for; the request's last delta carries its finish
    reason and usage (and may carry no token: a stop token is not emitted)."""

    index: int                      # which prompt of the call
    token_ids: list
    text_delta: str | None = None
    logprobs: list = field(default_factory=list)
    finish_reason: str | None = None
    usage: TokenUsage | None = None
    prompt_token_ids: list = field(default_factory=list)   # with the finish reason: the prompt as the engine saw it


class LLM:
    def __init__(self, model, *, dtype="bfloat16", device=None, page_size: int | None = None,
                 kv_cache_tokens: int | None = None, num_slots: int | None = 4, max_seq_len: int | None = None,
                 chunked_prefill_size: int | None = None, max_num_batched_tokens: int = 16384,
                 max_prefill_tokens: int | None = None, prefill_max_requests: int | None = None, seed: int = 42,
                 cuda_graph: bool = True, weight_tiles: bool | None = None, mem_fraction_static: float = 0.85,
                 async_overlap: bool = True, warm_up: bool = False, tune_products: bool | str = False):
        """model: a model folder, or an Engine that is already built.

        kv_cache_tokens: tokens the paged cache holds over all live requests.  Default: sized from the GPU's
        free memory after the weights are loaded, less a headroom of (1 - mem_fraction_static) of its whole
        memory (the reference's --mem-fraction-static, default 0.85), and never more than num_slots requests
        of max_seq_len tokens (default: the model's positions) can fill.
        chunked_prefill_size: the longest prompt portion of one request in a step.  Default: by the GPU's
        whole memory, as the reference's server picks it (2,048 below 35 GiB up to 16,384 from 90 GiB on, so
        16,384 on an MI355X), and at most max_num_batched_tokens.  max_prefill_tokens: the prompt tokens of
        all requests in a step; default max_num_batched_tokens.  While requests are decoding a portion is at
        most 4,096 tokens (long_prefill_token_threshold).
        num_slots: requests that run at a time; None: as many requests of max_seq_len tokens as the cache holds, from 4
        to 128 (the reference's --num-slots left unset).
        cuda_graph, weight_tiles: as for Engine (captured steps; the decode-friendly second copy of the weights).
        async_overlap: decode steps are launched from the last step's tokens on the GPU, and those are read back
        while the new step runs (SchedulerConfig.async_overlap); the tokens are the same either way.
        tune_products: measure which kernel runs each of this model's matrix products fastest at each row count and
        go by that (Engine.tune_products; up to a minute and a half); a string: also write the table there, for
        `Engine(product_table=...)` or ARLE_AMD_PRODUCT_TABLE next time.  The widths of Qwen3-4B, 8B and 32B have
        tables that come with the package.
        warm_up: capture the decode graphs of every batch size up to num_slots now (Engine.warm_up), as the
        reference's scheduler does when it starts; otherwise each is captured at its first step.
        """
        if isinstance(model, Engine):
            self.engine = model
        else:
            from ..config.registry import load_model_config
            from .engine import DEFAULT_PAGE_SIZE
            from .. import models  # noqa: F401

            _, config, _ = load_model_config(model)
            positions = getattr(config, "max_position_embeddings", 4096)
            max_seq_len = min(max_seq_len or positions, positions)
            self.engine = Engine.from_folder(model, dtype=dtype, device=device,
                                             page_size=page_size or DEFAULT_PAGE_SIZE,
                                             max_tokens=kv_cache_tokens, max_slots=num_slots,
                                             max_request_tokens=max_seq_len, cuda_graph=cuda_graph,
                                             weight_tiles=weight_tiles, mem_fraction_static=mem_fraction_static)
        self.model_dir = model if isinstance(model, str) else None
        self.seed = seed
        cfg = SchedulerConfig.runtime_defaults(self.engine.cache.max_slots)
        cfg.max_num_batched_tokens = max_num_batched_tokens
        cfg.prefill_max_requests, cfg.max_seq_len, cfg.async_overlap = prefill_max_requests, max_seq_len, async_overlap
        self.sched_config = cfg.resolve_runtime_envelope(_gpu_total_bytes(self.engine.device), chunked_prefill_size,
                                                         max_prefill_tokens)
        self.sched_config.validate()
        self.sampler = Sampler(self.engine.device)
        if tune_products:
            self.engine.tune_products(path=tune_products if isinstance(tune_products, str) else None)
        if warm_up:
            self.engine.warm_up()
        self.tokenizer = self._load_tokenizer()
        self.last_stats: dict = {}

    def _load_tokenizer(self):
        if not self.model_dir:
            return None
        path = os.path.join(self.model_dir, "tokenizer.json")
        if not os.path.exists(path):
            return None
        try:
            from tokenizers import Tokenizer
        except ImportError:
            return None
        return Tokenizer.from_file(path)

    def tokenize(self, text: str) -> list:
        if self.tokenizer is None:
            raise RuntimeError("this model folder has no tokenizer.json (or the `tokenizers` package is "
                               "missing): give prompts as token ids")
        return self.tokenizer.encode(text).ids

    def generate(self, prompts, max_tokens: int = 16, temperature: float = 0.0, seed: int | None = None,
                 ignore_eos: bool = False, sampling: SamplingParams | None = None, logprobs: bool = False,
                 priorities=None, stop=None) -> list:
        """prompts: a list of token-id lists (or strings, with a tokenizer).  One CompletionOutput each,
        in order.  `sampling` overrides temperature / seed / ignore_eos / logprobs when given: one SamplingParams for
        all prompts, or a list with one a prompt.
        priorities: one of PRIORITY_LOW / NORMAL / HIGH (0, 1, 2) a prompt; the higher is served first.
        stop: strings that end a request where its text first holds one of them (the text stops in front of it,
        the finish reason is `stop`); needs a tokenizer."""
        if stop:
            return self._collect(prompts, self.generate_stream(prompts, max_tokens, temperature, seed, ignore_eos,
                                                               sampling, logprobs, priorities, stop))
        sched, ids = self._submit(prompts, max_tokens, temperature, seed, ignore_eos, sampling, logprobs, priorities)
        try:
            sched.run_until_done()
        finally:
            sched.close()   # after an error no request of this call keeps a slot or pages
        self.last_stats = sched.stats
        outs = []
        for rid in ids:
            r = sched.finished[rid]
            text = self.tokenizer.decode(r.generated) if self.tokenizer is not None else None
            ttft = (r.t_first_token - r.t_submit) if r.t_first_token is not None else None
            tpot = ((r.t_tokens[-1] - r.t_tokens[0]) / (len(r.t_tokens) - 1)) if len(r.t_tokens) > 1 else None
            outs.append(CompletionOutput(text=text, finish_reason=r.finish_reason,
                                         usage=TokenUsage(len(r.prompt), len(r.generated)),
                                         prompt_token_ids=list(r.prompt),
                                         response_token_ids=list(r.generated), ttft_s=ttft, tpot_s=tpot,
                                         token_logprobs=list(r.logprobs)))
        return outs


    def _collect(self, prompts, deltas) -> list:
        """The deltas of a streamed call put together as `generate` returns them."""
        n = len(prompts)
        toks, lps, text, end = [[] for _ in range(n)], [[] for _ in range(n)], [""] * n, [None] * n
        for d in deltas:
            toks[d.index] += d.token_ids
            lps[d.index] += d.logprobs
            text[d.index] += d.text_delta or ""
            if d.finish_reason is not None:
                end[d.index] = d
        return [CompletionOutput(text=text[i] if self.tokenizer is not None else None, finish_reason=end[i].finish_reason,
                                 usage=end[i].usage, prompt_token_ids=list(end[i].prompt_token_ids),
                                 response_token_ids=toks[i], token_logprobs=lps[i]) for i in range(n)]

    def _submit(self, prompts, max_tokens, temperature, seed, ignore_eos, sampling, logprobs, priorities):
        sched = Scheduler(self.engine, self.sampler, self.sched_config, seed=self.seed,
                          stop_token_ids=self.engine.spec.stop_token_ids)
        ids = []
        if priorities is not None and len(priorities) != len(prompts):
            raise ValueError("one priority a prompt")
        each = isinstance(sampling, (list, tuple))
        if each and len(sampling) != len(prompts):
            raise ValueError("one SamplingParams a prompt (or one for all)")
        for i, p in enumerate(prompts):
            toks = self.tokenize(p) if isinstance(p, str) else list(p)
            params = (sampling[i] if each else sampling) or SamplingParams(temperature=temperature, seed=seed,
                                                                            ignore_eos=ignore_eos, logprobs=logprobs)
            ids.append(sched.submit(toks, params, max_tokens, **({} if priorities is None else {"priority": priorities[i]})))
        return sched, ids

    def generate_stream(self, prompts, max_tokens: int = 16, temperature: float = 0.0, seed: int | None = None,
                        ignore_eos: bool = False, sampling: SamplingParams | None = None, logprobs: bool = False,
                        priorities=None, stop=None):
        """`generate` as a generator of CompletionStreamDelta: after every iteration of the scheduler, what each
        request has newly produced, in the order of the prompts; a request's last delta has its finish reason and
        usage.  The tokens of all deltas of a request are `generate`'s response_token_ids.  (With steps launched
        ahead a token is read, and so handed on, one iteration after the step that chose it.)
        stop: as for `generate`; text that may still turn out to be the beginning of a stop string is held back
        (infer/src/scheduler/cuda/request.rs:72-117), and the request ends where one is found."""
        stops = [s for s in (stop or []) if s]
        if stops and self.tokenizer is None:
            raise RuntimeError("stop strings are looked for in the text: this model folder has no tokenizer.json")
        sched, ids = self._submit(prompts, max_tokens, temperature, seed, ignore_eos, sampling, logprobs, priorities)
        index = {rid: i for i, rid in enumerate(ids)}
        sent, text_sent, open_ids = {rid: 0 for rid in ids}, {rid: "" for rid in ids}, set(ids)
        idle = 0
        try:
            while open_ids:
                if sched.has_work():
                    plan = sched.iteration()
                    idle = idle + 1 if plan.kind == "idle" else 0
                    if idle > 2:
                        raise RuntimeError("scheduler makes no progress: a waiting request can never be admitted")
                live = {r.id: r for r in list(sched.waiting) + sched.prefilling + sched.decoding}
                for rid in ids:
                    if rid not in open_ids:
                        continue
                    r = sched.finished.get(rid) or live.get(rid)
                    if r is None:
                        continue
                    done = rid in sched.finished
                    new = r.generated[sent[rid]:]
                    if not new and not done:
                        continue
                    delta = CompletionStreamDelta(index[rid], list(new), logprobs=list(r.logprobs[sent[rid]:sent[rid] + len(new)]))
                    sent[rid] += len(new)
                    if self.tokenizer is not None:
                        text = self.tokenizer.decode(r.generated[:sent[rid]])
                        upto = len(text)
                        if stops:
                            found, upto = check_stop_sequences(text, stops)
                            if found and not done:      # the scheduler does not see the text: the request ends here
                                sched.abort(rid, STOP)
                                done = True
                            elif done and not found:
                                upto = len(text)        # nothing more can come: what was held back goes out
                        elif not done and text.endswith("\ufffd"):
                            upto = len(text_sent[rid])  # a character whose bytes are not all there yet waits
                        upto = max(upto, len(text_sent[rid]))
                        delta.text_delta, text_sent[rid] = text[len(text_sent[rid]):upto], text[:upto]
                    if done:
                        delta.finish_reason = r.finish_reason
                        delta.usage = TokenUsage(len(r.prompt), len(r.generated))
                        delta.prompt_token_ids = list(r.prompt)
                        open_ids.discard(rid)
                    yield delta
        finally:
            # a consumer that stops reading, or an error in an iteration or in the tokenizer: nothing stays held
            sched.close()
        self.last_stats = sched.stats


def generate(model, prompts, max_tokens: int = 16, temperature: float = 0.0, seed: int | None = None,
             ignore_eos: bool = False, **engine_args) -> list:
    """One-shot helper: `LLM(model, **engine_args).generate(...)` as plain dictionaries."""
    llm = model if isinstance(model, LLM) else LLM(model, **engine_args)
    return [{"token_ids": o.response_token_ids, "finish_reason": o.finish_reason,
             "usage": {"prompt_tokens": o.usage.prompt_tokens, "completion_tokens": o.usage.completion_tokens,
                       "total_tokens": o.usage.total_tokens}, "text": o.text}
            for o in llm.generate(prompts, max_tokens, temperature, seed, ignore_eos)]
