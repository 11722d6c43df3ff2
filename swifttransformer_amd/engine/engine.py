"""The generation loop: scheduler -> step function -> sampler, until requests finish.

Counterpart of the reference's example driver ``run_batched_inference``
(src/examples/lib/inference_batch.cc:15-232), which is a static batch: one
prefill of all prompts, then lock-step decoding.  Here requests may arrive at any
time and every step is whatever the scheduler composed."""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

import torch

from ..config.cache_param import CacheParam
from ..models import load_model
from ..models.decoder import DecoderModel
from ..sampling import Sampler, SamplingParams
from ..cache.page_pool import OutOfPages
from ..sampling.sampler import PendingTokens
from .scheduler import RUNNING, Request, Scheduled, Scheduler
from .step import ModelRunner, pages_that_fit  # noqa: F401

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    key = name.lower()
    if key in ("fp16", "float16", "half"):
        raise ValueError("this engine's 16-bit type is bfloat16: pass bf16")
    if key not in _DTYPES:
        raise ValueError(f"precision must be bf16 or fp32, got {name!r}")
    return _DTYPES[key]


@dataclass
class EngineStats:
    steps: int = 0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_time: float = 0.0      # time of steps that held a prompt portion
    decode_time: float = 0.0       # time of steps that held decode tokens only
    preemptions: int = 0
    pages_used_peak: int = 0       # most pages held at once (largest over the paged groups)
    # set to a list to have every step appended as (tokens run, keys read, query-key pairs):
    # what a step's memory and arithmetic floors are computed from
    step_log: Optional[list] = None


@dataclass
class RequestOutput:
    req_id: Hashable
    prompt: List[int]
    output: List[int]
    finish_reason: Optional[str]


@dataclass
class _Launched:
    """A step whose work is queued on the device and whose tokens have not been read yet."""
    scheduled: List[Scheduled]
    sampling: List[Scheduled]          # the entries of ``scheduled`` that yield a token, in row order
    pending: PendingTokens
    t0: float


class Engine:
    def __init__(self, model: Union[str, DecoderModel], *, dtype="bf16", page_size: int = 16,
                 num_pages: int = 1024, max_seqs: int = 64, max_batched_tokens: int = 2048,
                 prefill_chunk: int = 512, device: str = "cuda:0", gpu_mem_fraction: float = 0.0,
                 lookahead: bool = True):
        """``gpu_mem_fraction`` > 0 sizes the cache pool from the device memory that is free
        once the weights are loaded and the step arena is allocated (that fraction of it) instead
        of ``num_pages``.
        ``lookahead``: queue a decode step before the previous step's tokens have reached the
        host whenever the next batch is certain (see ``_launch_ahead``)."""
        dt = parse_dtype(dtype)
        if isinstance(model, str):
            model = load_model(model, dt, device)
        self.model = model
        self.runner = ModelRunner(model, CacheParam(page_size=page_size, num_pages=max(1, num_pages),
                                                    max_seqs=max_seqs), device,
                                  max_batched_tokens=max_batched_tokens, gpu_mem_fraction=gpu_mem_fraction)
        self.scheduler = Scheduler(self.runner.manager, max_batched_tokens=max_batched_tokens,
                                   prefill_chunk=prefill_chunk, max_positions=model.max_positions,
                                   eos_token_id=model.spec.eos_token_id)
        self.sampler = Sampler(device)
        self.stats = EngineStats()
        self._next_id = 0
        self.requests: Dict[Hashable, Request] = {}
        self.lookahead = bool(lookahead)
        self._ahead: Optional[_Launched] = None
        self._last_done = 0.0

    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    req_id: Optional[Hashable] = None) -> Hashable:
        if req_id is None:
            req_id = self._next_id
            self._next_id += 1
        if req_id in self.requests:
            raise KeyError(f"request id {req_id!r} is in use")
        vocab = self.model.vocab_size
        if any((t < 0 or t >= vocab) for t in prompt):
            raise ValueError(f"prompt token outside [0, {vocab})")
        req = Request(req_id, [int(t) for t in prompt], params or SamplingParams())
        self.scheduler.add(req)
        self.requests[req_id] = req
        return req_id

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def warm_up(self, prompt_tokens: Optional[Sequence[int]] = None,
                decode_batches: Optional[Sequence[int]] = None) -> int:
        """Record the steps that serving replays before the first request arrives
        (``ModelRunner.warm_up``).  Defaults: prompt portions of every size the recordings are
        bucketed into up to the scheduler's portion, decode steps of 1, 2, 4, ... requests up to
        ``max_seqs``.  Call it while no request is in the engine."""
        if self.scheduler.has_work():
            raise RuntimeError("warm up before requests are added")
        chunk = min(self.scheduler.prefill_chunk, self.runner.max_batched_tokens)
        if prompt_tokens is None:
            prompt_tokens = [n for n in (8, 16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 768, 1024, 1536, 2048)
                             if n <= chunk]
        if decode_batches is None:
            decode_batches, b = [], 1
            while b <= self.runner.cache_param.max_seqs:
                decode_batches.append(b)
                b *= 2
        return self.runner.warm_up(prompt_tokens, decode_batches)

    # ------------------------------------------------------------------ one step
    def _launch(self) -> Optional["_Launched"]:
        """Schedule a step and queue its work on the device; nothing waits for it."""
        scheduled = self.scheduler.schedule()
        if not scheduled:
            if self.scheduler.has_work():
                raise RuntimeError("the scheduler made no progress: the cache pool is too small "
                                   "for the oldest waiting request's first portion")
            return None
        t0 = time.perf_counter()
        items = [self.runner.item(s.request.req_id, s.start, s.tokens,
                                  [len(s.tokens) - 1] if s.sample else []) for s in scheduled]
        logits = self.runner.run(items)
        sampling = [s for s in scheduled if s.sample]
        pending = self.sampler.sample_pending(logits, [s.request.params for s in sampling],
                                              [len(s.request.output) for s in sampling],
                                              best=self.runner.last_best)
        return _Launched(scheduled, sampling, pending, t0)

    def _launch_ahead(self, cur: "_Launched") -> Optional["_Launched"]:
        """Queue the decode step that follows ``cur`` before ``cur``'s tokens are known on the
        host: the device feeds it the ids it has just sampled, so the host's turn-around between
        two steps (reading the ids, bookkeeping, packing the next batch) overlaps with the
        device's work instead of idling it.  Only taken when the next step is certain to be one
        token for exactly these requests: all of them were sampled, nobody waits, nobody reaches
        a length limit, and their next pages are free.  A request that ends on an end-of-sequence
        token is found out one step late; its extra token is computed and dropped."""
        if not (self.lookahead and self.runner.use_graphs):
            return None
        sched = self.scheduler
        if sched.waiting or len(cur.sampling) != len(cur.scheduled) or \
                len(cur.scheduled) != len(sched.running) or len(cur.scheduled) > self.runner.cache_param.max_seqs:
            return None
        starts = []
        for s in cur.scheduled:
            req = s.request
            n_out = len(req.output) + 1                        # once cur's token is appended
            nxt = s.start + len(s.tokens)                      # position of that token
            if n_out >= req.params.max_new_tokens or len(req.prompt) + n_out > sched.max_positions \
                    or nxt + 1 > sched.max_positions:
                return None
            starts.append(nxt)
        manager = self.runner.manager
        grown = []
        try:
            for s, nxt in zip(cur.scheduled, starts):
                rc = manager.requests[s.request.req_id]
                before = (rc.length, {g: len(rc.tables[g]) for g in self.runner.paged_group_ids})
                manager.release_behind_window(s.request.req_id, nxt)
                manager.extend(s.request.req_id, nxt + 1)
                grown.append((s.request.req_id, before))
        except OutOfPages:
            for req_id, (length, pages) in grown:
                manager.shrink(req_id, length, pages)
            return None                                        # the scheduler will pre-empt someone
        t0 = time.perf_counter()
        logits = self.runner.run_decode_from_device([s.request.req_id for s in cur.scheduled], starts,
                                                    cur.pending.device)
        scheduled = [Scheduled(s.request, nxt, [-1], True) for s, nxt in zip(cur.scheduled, starts)]
        pending = self.sampler.sample_pending(logits, [s.request.params for s in scheduled],
                                              [len(s.request.output) + 1 for s in scheduled],
                                              best=self.runner.last_best)
        return _Launched(scheduled, list(scheduled), pending, t0)

    def step(self) -> List[RequestOutput]:
        """One scheduled step; returns the requests that finished in it."""
        cur = self._ahead or self._launch()
        self._ahead = None
        if cur is None:
            return []
        ahead = self._launch_ahead(cur)
        toks = cur.pending.result()                            # waits for this step's ids only
        # requests that ended while this step was already queued have no use for its token
        live = [(s, t) for s, t in zip(cur.sampling, toks) if s.request.status == RUNNING]
        sampled = {s.request.req_id: t for s, t in live}
        scheduled = [s for s in cur.scheduled if s.request.status == RUNNING]
        finished = self.scheduler.update(scheduled, sampled)
        if ahead is not None and not self.scheduler.running:
            ahead = None                                       # everyone ended: nothing to wait for
        self._ahead = ahead
        now = time.perf_counter()
        dt = now - max(cur.t0, self._last_done)               # a step queued ahead counts from the previous one's end
        self._last_done = now
        st = self.stats
        st.steps += 1
        st.generated_tokens += len(live)
        has_prompt = any(len(s.tokens) > 1 or s.start < len(s.request.prompt) for s in scheduled)
        st.prompt_tokens += sum(max(0, min(len(s.request.prompt), s.start + len(s.tokens)) - s.start)
                                for s in scheduled)
        if has_prompt:
            st.prefill_time += dt
        else:
            st.decode_time += dt
        st.preemptions = self.scheduler.num_preemptions
        for g in self.runner.manager.paged_groups:
            st.pages_used_peak = max(st.pages_used_peak, g.pool.num_pages - g.pool.num_free)
        if st.step_log is not None:
            n_tok = sum(len(s.tokens) for s in cur.scheduled)
            keys = sum(s.start + len(s.tokens) for s in cur.scheduled)
            pairs = sum(len(s.tokens) * s.start + len(s.tokens) * (len(s.tokens) + 1) // 2 for s in cur.scheduled)
            st.step_log.append((n_tok, keys, pairs))
        outs = []
        for r in finished:
            outs.append(RequestOutput(r.req_id, r.prompt, list(r.output), r.finish_reason))
            del self.requests[r.req_id]
        return outs

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[List[int]]:
        """Generated token ids for each prompt, in the order given."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        done: Dict[Hashable, List[int]] = {}
        while self.has_work():
            for out in self.step():
                done[out.req_id] = out.output
        return [done[i] for i in ids]
