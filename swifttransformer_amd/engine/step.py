"""The step function: run a batch of (request, its next tokens) from the cache.

Counterpart of the reference's ``Gpt<T>::forward(input_tokens_batched,
first_token_indexes, k_cache, v_cache, block_table)`` (src/csrc/model/gpt/gpt_base.h:74-83,
src/csrc/model/gpt/gpt.cc:507-657), which accepts whole prompts and single decode
tokens and returns one greedy token per request.  Here a batch may also hold
portions of prompts cut anywhere, the cache pool and block tables are owned by
the runner's cache manager, and float32 logits at the wanted positions come
back; choosing tokens is the sampler's job.

Steps are launch-bound below some hundreds of tokens: some two hundred kernels whose
launches cost the host more than they cost the device.  A step is therefore recorded
once per shape as a HIP graph over fixed index buffers and replayed; the kernels and
the cache are the same as in the unrecorded path.  Steps of single tokens (decoding)
are recorded per batch-size bucket at their first use; steps of any other composition
(prompt portions, alone or beside decode tokens) per (padded token count, lengths of the
parts' work lists) once that shape has come up ``record_after`` times; their final norm
and head run after the replay on the rows that are wanted, so the number of wanted rows
is no part of the shape.
Every tensor a step makes is carved from one arena sized when the runner is built
(``ops/arena.py``), so recordings share their scratch memory and an unrecorded step asks
the allocator for nothing but its logits."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.device import DeviceCache
from ..cache.manager import CacheManager
from ..config.cache_param import CacheParam
from ..models.decoder import DecoderModel
from ..ops import kernels as K
from ..ops.arena import StepArena, using as using_arena
from ..ops.tuning import tuning
from ..parts.base import BatchInfo
from .batch import (DecodeBuffers, StepBuffers, StepContext, StepItem, check_items, pack_batch, run_planners,
                    token_bucket)


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class _RecordedStep:
    """A step as a HIP graph over fixed buffers.  ``logits``: what the recording ends with, the
    logits of a decode step, or the residual stream of a step whose head runs after the replay
    (``arena_state``: where the arena stood when the recording ended)."""

    def __init__(self, buffers, graph, logits: torch.Tensor, arena_state=None, best=None):
        self.buffers = buffers
        self.graph = graph
        self.logits = logits
        self.arena_state = arena_state
        self.best = best            # int32 [rows]: the rows' best tokens (recordings that end with the head)


class ModelRunner:
    def __init__(self, model: DecoderModel, cache_param: CacheParam, device="cuda:0",
                 cache_fill: float = 0.0, use_graphs: bool = True, max_batched_tokens: Optional[int] = None,
                 gpu_mem_fraction: float = 0.0, record_after: Optional[int] = None):
        """``max_batched_tokens``: the most tokens a step is expected to bring (a scheduler's budget);
        the step arena is sized for it (larger steps still run, through the allocator).  Default:
        the model's positions, 2,048 at most, plus a token for every other request.
        ``gpu_mem_fraction`` > 0 sizes the cache pool as that share of the device memory still free
        once the weights are loaded and the arena is allocated, instead of ``cache_param.num_pages``.
        ``record_after``: a step that is not plain decoding is recorded when its shape comes up
        for this many-th time (0: never; default: ``ops.tuning``)."""
        self.model = model
        self.device = torch.device(device)
        max_pages = cache_param.max_pages_per_seq or cache_param.pages_for(model.max_positions)
        self.max_pages_per_seq = max_pages
        self.use_graphs = bool(use_graphs) and model.graph_safe and self.device.type == "cuda"
        self.planners = model.step_planners()
        if max_batched_tokens is None:
            max_batched_tokens = min(model.max_positions, 2048) + max(0, cache_param.max_seqs - 1)
        self.max_batched_tokens = int(max_batched_tokens)
        self.arena = StepArena(self.device)
        if self.device.type == "cuda" and model.weights_loaded:
            self._size_arena(cache_param)
        if gpu_mem_fraction > 0:
            from dataclasses import replace
            cache_param = replace(cache_param, num_pages=pages_that_fit(model, cache_param.page_size,
                                                                        gpu_mem_fraction, self.device))
        self.cache_param = cache_param
        self.manager = CacheManager(model.cache_needs(), cache_param.page_size, cache_param.num_pages,
                                    cache_param.max_seqs, max_pages)
        self.cache = DeviceCache(self.manager, model.dtype, self.device, fill=cache_fill)
        self.paged_group_ids = [g.index for g in self.manager.paged_groups]
        self.steps_run = 0
        self._recorded: Dict[int, _RecordedStep] = {}
        self._recorded_general: Dict[tuple, _RecordedStep] = {}
        self._seen: Dict[tuple, int] = {}
        self.record_after = int(tuning.record_after if record_after is None else record_after)
        self.max_recorded = 256          # recordings of general steps kept; the oldest goes first
        self.tune_up_to = tuning.tune_products_up_to_rows
        self.graph_replays = 0
        # int32 [wanted rows] on the device: the best token of every row of the last step's logits
        # (lowest id on ties), found by the head's own kernel or the arg-max kernel; a greedy sampler
        # needs nothing else.  Like a recorded step's logits it is reused by later steps.
        self.last_best: Optional[torch.Tensor] = None

    def _size_arena(self, cache_param: CacheParam) -> None:
        """Measure what a step of ``max_batched_tokens`` tokens makes per layer (one run through the
        ordinary allocator on a one-page cache of its own: a prompt portion as long as the model
        allows, the rest single tokens), and allocate the arena's two banks for it."""
        T = max(1, self.max_batched_tokens)
        ps = cache_param.page_size
        P = min(self.model.max_positions, self.max_pages_per_seq * ps)
        first = min(T, P)
        singles = min(T - first, max(0, cache_param.max_seqs - 1))
        lens = [first] + [1] * singles
        left = T - first - singles
        while left > 0:
            lens.append(min(left, P))
            left -= lens[-1]
        manager = CacheManager(self.model.cache_needs(), ps, 1, len(lens), self.max_pages_per_seq)
        cache = DeviceCache(manager, self.model.dtype, self.device)
        groups = [g.index for g in manager.paged_groups]
        items = [StepItem(slot=i, start=0, tokens=[0] * n, want=[n - 1],
                          pages={g: [0] * (-(-n // ps)) for g in groups}) for i, n in enumerate(lens)]
        ctx = pack_batch(items, groups, self.max_pages_per_seq, ps, self.device, vocab_size=self.model.vocab_size,
                         max_positions=P, planners=self.planners)
        # every token is written to and read from page 0: in bounds, and nobody's cache
        self.arena.measure = True
        try:
            with using_arena(self.arena):
                self.model.forward(ctx, cache.views)
            torch.cuda.synchronize(self.device)
        finally:
            self.arena.measure = False
        # (the run's logits were a tensor of their own; those of a recorded decode step live in the
        # arena, beside the head's input, for up to max_seqs rows)
        need = self.arena.peak + cache_param.max_seqs * (self.model.vocab_size * 4 + 256)
        del ctx, cache, manager
        torch.cuda.empty_cache()
        self.arena.peak = 0
        self.arena.resize(need + need // 16 + (1 << 16))

    # ----------------------------------------------------------------- requests
    def admit(self, req_id: Hashable) -> None:
        self.manager.admit(req_id)      # the device cache clears the slot's state from the manager's hook

    def finish(self, req_id: Hashable) -> None:
        self.manager.finish(req_id)

    def is_live(self, req_id: Hashable) -> bool:
        return req_id in self.manager.requests

    def cached_length(self, req_id: Hashable) -> int:
        return self.manager.requests[req_id].length

    def warm_up(self, prompt_tokens: Sequence[int] = (), decode_batches: Sequence[int] = ()) -> int:
        """Record ahead of time the steps that serving will replay, so that no request pays for a
        recording (an unrecorded run, the timing of the library's kernels, the capture): one prompt
        portion of each of ``prompt_tokens`` tokens alone, and decode steps of each of
        ``decode_batches`` requests.  Uses the cache like any request and gives everything back;
        call it while the pool is free.  Returns the number of recordings made."""
        if not self.use_graphs:
            return 0
        before = len(self._recorded) + len(self._recorded_general)
        keep, self.record_after = self.record_after, 1
        try:
            for n in prompt_tokens:
                n = min(int(n), self.model.max_positions, self.max_batched_tokens)
                if n < 2:
                    continue
                self.admit(("warm-up", 0))
                try:
                    self.step([StepEntry(("warm-up", 0), [0] * n, [n - 1])])
                finally:
                    self.finish(("warm-up", 0))
            for b in decode_batches:
                b = min(int(b), self.cache_param.max_seqs)
                ids = [("warm-up", i) for i in range(b)]
                done = []
                try:
                    for r in ids:
                        self.admit(r)
                        done.append(r)
                    self.step([StepEntry(r, [0], [0]) for r in ids])
                finally:
                    for r in done:
                        self.finish(r)
        finally:
            self.record_after = keep
        torch.cuda.synchronize(self.device)
        return len(self._recorded) + len(self._recorded_general) - before

    # --------------------------------------------------------------------- step
    def item(self, req_id: Hashable, start: int, tokens: Sequence[int], want: Sequence[int]) -> StepItem:
        """Describe tokens whose cache room has already been reserved (by a scheduler)."""
        rc = self.manager.requests[req_id]
        if start + len(tokens) > rc.length:
            raise ValueError(f"request {req_id!r}: positions up to {start + len(tokens) - 1} are not reserved")
        return StepItem(slot=rc.slot, start=start, tokens=list(tokens), want=list(want),
                        pages={g: rc.tables[g] for g in self.paged_group_ids})

    def prepare(self, entries: Sequence[StepEntry]) -> List[StepItem]:
        """Reserve cache room for every entry (all or nothing) and describe the batch."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        items: List[StepItem] = []
        grown: List[Tuple[Hashable, int, Dict[int, int]]] = []
        try:
            for e in entries:
                rc = self.manager.requests[e.req_id]
                start = rc.length
                before = {g: len(rc.tables[g]) for g in self.paged_group_ids}
                self.manager.release_behind_window(e.req_id, start)
                self.manager.extend(e.req_id, start + len(e.tokens))
                grown.append((e.req_id, start, before))
                items.append(StepItem(slot=rc.slot, start=start, tokens=list(e.tokens),
                                      want=list(e.want),
                                      pages={g: rc.tables[g] for g in self.paged_group_ids}))
        except Exception:
            # give back what this step had taken
            for req_id, start, before in grown:
                self.manager.shrink(req_id, start, before)
            raise
        return items

    def run(self, items: Sequence[StepItem]) -> torch.Tensor:
        """float32 logits [wanted rows, vocab].  The tensor of a recorded step is reused by later
        steps: read it (or copy it) before stepping again."""
        if self.use_graphs:
            if self._is_plain_decode(items):
                return self._run_recorded(items)
            if self.record_after > 0:
                logits = self._run_recorded_general(items)
                if logits is not None:
                    return logits
        ctx = pack_batch(items, self.paged_group_ids, self.max_pages_per_seq, self.cache_param.page_size,
                         self.device, vocab_size=self.model.vocab_size,
                         max_positions=self.model.max_positions, planners=self.planners)
        return self.run_context(ctx)

    def run_context(self, ctx: StepContext) -> torch.Tensor:
        best = torch.empty((ctx.num_wanted,), dtype=torch.int32, device=self.device)
        with using_arena(self.arena):
            logits = self.model.forward(ctx, self.cache.views, best=best)
        self.last_best = best
        self.steps_run += 1
        return logits

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """float32 logits [sum of wanted rows, vocab], in the order of entries and of want."""
        return self.run(self.prepare(entries))

    # ----------------------------------------------------------- recorded steps
    def _is_plain_decode(self, items: Sequence[StepItem]) -> bool:
        if len(items) > self.cache_param.max_seqs:
            return False
        return all(len(it.tokens) == 1 and list(it.want) == [0] for it in items)

    def _bucket(self, n: int) -> int:
        """Rows of the recorded step that serves ``n`` requests: ``n`` itself up to 8, the next even
        number up to 16 (there a product's time grows with its rows: 1 to 1.5 % of a step between
        10 and 14 requests against steps of 16 rows), then the next power of two: the library's
        products and the attention cost the same at 40 rows as at 64, and every size is a
        recording and a timing of the library's kernels of its own."""
        if n <= 8:
            return n
        if n <= 16:
            return min(n + (n & 1), self.cache_param.max_seqs)
        b = 32
        while b < n:
            b <<= 1
        return min(b, self.cache_param.max_seqs)

    def _record(self, capacity: int) -> _RecordedStep:
        buffers = DecodeBuffers(capacity, self.paged_group_ids, self.max_pages_per_seq,
                                self.cache_param.page_size, self.device, self.model.max_positions)
        # one unrecorded run on padding rows first: loads code objects, sizes the allocator, and
        # has the library's products of this row count timed and chosen
        # The rows' best tokens are left where the next step's token ids are read: a step that
        # decodes greedily from what the step before it chose needs no copy between the two.
        rec = self._capture(buffers, tune=True, best=buffers.ctx.token_ids)
        self._recorded[capacity] = rec
        return rec

    def _capture(self, buffers, tune: bool, layers_only: bool = False,
                 best: Optional[torch.Tensor] = None) -> _RecordedStep:
        """Run the step that ``buffers`` describe once unrecorded (code objects, the library's plans
        for these row counts, timed and chosen if ``tune``), then record it.  Both runs carve the
        same tensors from the arena, so the recording's addresses are those of every replay.
        ``layers_only``: the recording ends with the residual stream; norm and head of the wanted
        rows run after each replay."""
        if layers_only:
            best = None
        elif best is None:
            best = torch.empty((buffers.ctx.num_wanted,), dtype=torch.int32, device=self.device)
        if layers_only:
            run = lambda: self.model.forward_layers(buffers.ctx, self.cache.views)
        else:
            run = lambda: self.model.forward(buffers.ctx, self.cache.views, best=best)
        with using_arena(self.arena):
            if tune:
                with K.tuned_products():
                    run()
            else:
                run()
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph), using_arena(self.arena):
            out = run()
            state = self.arena.state()
        return _RecordedStep(buffers, graph, out, state, best)

    # ----------------------------------------- recorded steps of any composition
    def _run_recorded_general(self, items: Sequence[StepItem]) -> Optional[torch.Tensor]:
        """Replay (or record) the step of these items' shape; None when it is to run unrecorded:
        larger than the runner was built for, or a shape not seen often enough yet."""
        B = len(items)
        T = sum(len(it.tokens) for it in items)
        R = sum(len(it.want) for it in items)
        if B > self.cache_param.max_seqs or T > self.max_batched_tokens:
            return None
        check_items(items, self.paged_group_ids, self.cache_param.page_size, self.model.vocab_size,
                    self.model.max_positions)
        planned, extra = run_planners(items, self.planners, BatchInfo(
            page_size=self.cache_param.page_size, max_pages=self.max_pages_per_seq, bucketed=True))
        # (the logits' rows are no part of the shape: norm and head run after the replay, on as
        # many rows as are wanted)
        T_pad = token_bucket(T)
        key = (T_pad, tuple((k, tuple(sorted(plan.host.items())), tuple(a.size for _n, _p, a in named))
                            for k, plan, named in planned))
        rec = self._recorded_general.get(key)
        if rec is None:
            seen = self._seen.get(key, 0) + 1
            if seen < self.record_after:
                if len(self._seen) > 4096:
                    self._seen.clear()
                self._seen[key] = seen
                return None
            self._seen.pop(key, None)
        slots = np.fromiter((it.slot for it in items), dtype=np.int64, count=B)
        tables = {g: self.manager.table_array[g][slots] for g in self.paged_group_ids}
        if rec is None:
            buffers = StepBuffers(T_pad, self.cache_param.max_seqs, T_pad, self.paged_group_ids,
                                  self.max_pages_per_seq, self.cache_param.page_size, self.device,
                                  self.model.max_positions, planned, extra)
            buffers.fill(items, tables, planned)
            # the run before the recording does this batch's own work (its keys and values are
            # written again, with the same values, by the replay below)
            rec = self._capture(buffers, tune=T_pad <= self.tune_up_to, layers_only=True)
            while len(self._recorded_general) >= self.max_recorded:
                self._recorded_general.pop(next(iter(self._recorded_general)))
            self._recorded_general[key] = rec
        else:
            rec.buffers.fill(items, tables, planned)
        rec.graph.replay()
        self.steps_run += 1
        self.graph_replays += 1
        best = torch.empty((R,), dtype=torch.int32, device=self.device)
        with using_arena(self.arena, rec.arena_state):
            logits = self.model.forward_head(rec.logits, rec.buffers.ctx, rec.buffers.ctx.want_rows[:R], keep=True,
                                             best=best)
        self.last_best = best
        return logits

    def run_decode_from_device(self, req_ids: Sequence[Hashable], starts: Sequence[int],
                               tokens_dev: torch.Tensor) -> torch.Tensor:
        """A recorded step of one token per request whose token ids are already on the device
        (``tokens_dev`` [B] int32, e.g. what the previous step sampled): nothing here needs
        their values on the host.  Cache room must be reserved."""
        if not self.use_graphs:
            raise RuntimeError("steps from device tokens are recorded steps")
        B = len(req_ids)
        if B < 1 or B > self.cache_param.max_seqs or tokens_dev.shape != (B,):
            raise ValueError("one device token per request, at most max_seqs requests")
        rcs = [self.manager.requests[r] for r in req_ids]
        for rc, st in zip(rcs, starts):
            if st + 1 > rc.length or st + 1 > self.model.max_positions:
                raise ValueError(f"position {st} is not reserved")
        cap = self._bucket(B)
        rec = self._recorded.get(cap) or self._record(cap)
        slots = np.fromiter((rc.slot for rc in rcs), dtype=np.int64, count=B)
        rec.buffers.fill(None, np.asarray(starts, dtype=np.int32), slots.astype(np.int32),
                         {g: self.manager.table_array[g][slots] for g in self.paged_group_ids})
        ids = rec.buffers.ctx.token_ids
        if tokens_dev.data_ptr() != ids.data_ptr():          # else: the last replay of this recording left them there
            ids[:B].copy_(tokens_dev)
        rec.graph.replay()
        self.steps_run += 1
        self.graph_replays += 1
        self.last_best = rec.best[:B]
        return rec.logits[:B]

    def _run_recorded(self, items: Sequence[StepItem]) -> torch.Tensor:
        check_items(items, self.paged_group_ids, self.cache_param.page_size, self.model.vocab_size,
                    self.model.max_positions)
        B = len(items)
        cap = self._bucket(B)
        rec = self._recorded.get(cap) or self._record(cap)
        slots = np.fromiter((it.slot for it in items), dtype=np.int64, count=B)
        rec.buffers.fill(np.fromiter((it.tokens[0] for it in items), dtype=np.int32, count=B),
                         np.fromiter((it.start for it in items), dtype=np.int32, count=B),
                         slots.astype(np.int32),
                         {g: self.manager.table_array[g][slots] for g in self.paged_group_ids})
        rec.graph.replay()
        self.steps_run += 1
        self.graph_replays += 1
        self.last_best = rec.best[:B]
        return rec.logits[:B]


def pages_that_fit(model: DecoderModel, page_size: int, fraction: float, device) -> int:
    """Pages per cache group such that all paged groups together take ``fraction`` of the
    memory now free on ``device``."""
    if not 0.0 < fraction <= 1.0:
        raise ValueError(f"gpu_mem_fraction is a share of the free memory in (0, 1], not {fraction}")
    free, _total = torch.cuda.mem_get_info(torch.device(device))
    elem = 2 if model.dtype == torch.bfloat16 else 4
    per_page = sum(2 * need.num_kv_heads * need.head_dim * page_size * elem
                   for need in model.cache_needs().values() if need.kind == "paged_kv")
    if per_page == 0:
        return 1
    return max(1, int(free * fraction) // per_page)
