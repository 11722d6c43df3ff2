"""Continuous batching: admission, portions of prompts under a token budget,
decoding, finishing, and what happens when pages run out.

The reference has no scheduler; its example driver runs all prompts whole in one
step and then decodes in lock-step (src/examples/lib/inference_batch.cc:110-118,
:163-220), dropping a request at the end token (:199-201) and exiting the process
when blocks run out (:61-64).

Policy here, in the order a step is filled:
  1. every running request that has one token to compute (decoding) gets it;
  2. running requests in the middle of their prompt get their next portion;
  3. waiting requests are admitted, first come first served, while a state slot,
     the token budget and pages for their first portion are there.
A portion is min(tokens left, prefill_chunk, budget left).  When a running
request cannot get the pages for its next tokens, the most recently admitted
running request is pre-empted: its pages and slot are given back and it returns
to the front of the waiting queue, to be recomputed from its prompt plus what it
has generated (its sampler counter goes on, so its output is unchanged).  A
request whose prompt and output could never fit the pool is refused when added.
Scheduling depends only on arrival order and parameters, never on logits' values
beyond the tokens they produce.  Runs on the host alone."""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional

from ..cache.manager import CacheManager
from ..cache.page_pool import OutOfPages
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    req_id: Hashable
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    num_computed: int = 0           # tokens of prompt+output whose keys are in the cache
    status: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.num_computed


@dataclass
class Scheduled:
    request: Request
    start: int
    tokens: List[int]
    sample: bool         # this portion reaches the request's last token: its logits are wanted


class Scheduler:
    def __init__(self, manager: CacheManager, *, max_batched_tokens: int = 2048,
                 prefill_chunk: int = 512, max_positions: int, eos_token_id: Optional[int] = None):
        if max_batched_tokens < 1 or prefill_chunk < 1:
            raise ValueError("token budget and portion size must be positive")
        self.manager = manager
        self.max_batched_tokens = max_batched_tokens
        self.prefill_chunk = prefill_chunk
        self.max_positions = max_positions
        self.eos_token_id = eos_token_id
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.num_preemptions = 0

    # --------------------------------------------------------------- admission
    def add(self, request: Request) -> None:
        n = len(request.prompt)
        if n < 1:
            raise ValueError("a request needs at least one prompt token")
        if n >= self.max_positions + 1:
            raise ValueError(f"a prompt of {n} tokens exceeds the model's {self.max_positions} positions")
        most = min(self.max_positions, n + request.params.max_new_tokens)
        pages = -(-most // self.manager.page_size)
        for g in self.manager.paged_groups:
            cap = g.pool.num_pages
            need = pages
            if g.need.window > 0:
                # a windowed group never holds more than the window plus one portion
                need = min(pages, -(-(g.need.window + self.prefill_chunk) // self.manager.page_size) + 1)
            if need > cap:
                raise ValueError(f"request {request.req_id!r} may need {need} pages of cache group "
                                 f"{g.index}; the pool has {cap}")
        if pages > self.manager.max_pages_per_seq:
            raise ValueError(f"request {request.req_id!r} may need {pages} pages; a request may hold "
                             f"{self.manager.max_pages_per_seq}")
        request.status = WAITING
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---------------------------------------------------------------- one step
    def _preempt_last(self) -> Request:
        victim = self.running.pop()
        self.manager.finish(victim.req_id)
        victim.num_computed = 0
        victim.status = WAITING
        victim.preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        return victim

    def _reserve(self, req: Request, n: int) -> bool:
        """Pages for the next n tokens of a running request, pre-empting later arrivals if
        needed.  False if the request itself was pre-empted."""
        while True:
            try:
                self.manager.release_behind_window(req.req_id, req.num_computed)
                self.manager.extend(req.req_id, req.num_computed + n)
                return True
            except OutOfPages:
                victim = self._preempt_last()
                if victim is req:
                    return False

    def schedule(self) -> List[Scheduled]:
        budget = self.max_batched_tokens
        out: List[Scheduled] = []
        planned = set()
        # 1 and 2: running requests, decoding ones first, each kind in admission order
        order = [r for r in self.running if r.pending == 1] + [r for r in self.running if r.pending > 1]
        for req in order:
            if budget <= 0:
                break
            if req.status != RUNNING:      # pre-empted while serving an earlier request
                continue
            n = min(req.pending, self.prefill_chunk, budget)
            if not self._reserve(req, n):
                continue
            toks = req.tokens[req.num_computed:req.num_computed + n]
            out.append(Scheduled(req, req.num_computed, toks, sample=(n == req.pending)))
            planned.add(id(req))
            budget -= n
        # a request scheduled above may have been pre-empted afterwards by a later one's need
        out = [s for s in out if s.request.status == RUNNING]
        # 3: admit
        while self.waiting and budget > 0 and self.manager.num_free_slots > 0:
            req = self.waiting[0]
            n = min(req.pending, self.prefill_chunk, budget)
            if not self.manager.can_extend(req.req_id, n):
                break
            self.waiting.popleft()
            self.manager.admit(req.req_id)
            self.manager.extend(req.req_id, n)
            req.status = RUNNING
            self.running.append(req)
            toks = req.tokens[:n]
            out.append(Scheduled(req, 0, toks, sample=(n == req.pending)))
            budget -= n
        return out

    # ------------------------------------------------------------- after a step
    def update(self, scheduled: List[Scheduled], sampled: Dict[Hashable, int]) -> List[Request]:
        """Account for a finished step; ``sampled``: request id -> new token for the entries with
        ``sample``.  Returns the requests that finished."""
        finished: List[Request] = []
        for s in scheduled:
            req = s.request
            req.num_computed += len(s.tokens)
            if not s.sample:
                continue
            tok = int(sampled[req.req_id])
            req.output.append(tok)
            eos = req.params.eos_token_id if req.params.eos_token_id is not None else self.eos_token_id
            reason = None
            if not req.params.ignore_eos and eos is not None and tok == eos:
                reason = "eos"
            elif len(req.output) >= req.params.max_new_tokens:
                reason = "length"
            elif len(req.prompt) + len(req.output) > self.max_positions:
                reason = "positions"      # the new token has no position left to be run at
            if reason:
                req.status = FINISHED
                req.finish_reason = reason
                self.running.remove(req)
                self.manager.finish(req.req_id)
                finished.append(req)
        return finished
