"""The step function: run a batch of (request, its next tokens) from the cache.

Counterpart of the reference's ``Gpt<T>::forward(input_tokens_batched,
first_token_indexes, k_cache, v_cache, block_table)`` (src/csrc/model/gpt/gpt_base.h:74-83,
src/csrc/model/gpt/gpt.cc:507-657), which accepts whole prompts and single decode
tokens and returns one greedy token per request.  Here a batch may also hold
portions of prompts cut anywhere, the cache pool and block tables are owned by
the runner's cache manager, and float32 logits at the wanted positions come
back; choosing tokens is the sampler's job.

Steps that hold single tokens only (decoding) are launch-bound: some two hundred
small kernels.  Such a step is recorded once per batch-size bucket as a HIP graph
over fixed index buffers and replayed; the kernels and the cache are the same as
in the unrecorded path."""
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
from .batch import DecodeBuffers, StepContext, StepItem, check_items, pack_batch


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class _RecordedStep:
    def __init__(self, buffers: DecodeBuffers, graph, logits: torch.Tensor):
        self.buffers = buffers
        self.graph = graph
        self.logits = logits


class ModelRunner:
    def __init__(self, model: DecoderModel, cache_param: CacheParam, device="cuda:0",
                 cache_fill: float = 0.0, use_graphs: bool = True):
        self.model = model
        self.device = torch.device(device)
        self.cache_param = cache_param
        max_pages = cache_param.max_pages_per_seq or cache_param.pages_for(model.max_positions)
        self.max_pages_per_seq = max_pages
        self.manager = CacheManager(model.cache_needs(), cache_param.page_size, cache_param.num_pages,
                                    cache_param.max_seqs, max_pages)
        self.cache = DeviceCache(self.manager, model.dtype, self.device, fill=cache_fill)
        self.paged_group_ids = [g.index for g in self.manager.paged_groups]
        self.planners = model.step_planners()
        self.steps_run = 0
        self.use_graphs = bool(use_graphs) and model.graph_safe and self.device.type == "cuda"
        self._recorded: Dict[int, _RecordedStep] = {}
        self.graph_replays = 0

    # ----------------------------------------------------------------- requests
    def admit(self, req_id: Hashable) -> None:
        self.manager.admit(req_id)      # the device cache clears the slot's state from the manager's hook

    def finish(self, req_id: Hashable) -> None:
        self.manager.finish(req_id)

    def is_live(self, req_id: Hashable) -> bool:
        return req_id in self.manager.requests

    def cached_length(self, req_id: Hashable) -> int:
        return self.manager.requests[req_id].length

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
        """float32 logits [wanted rows, vocab].  The tensor of a decode step is reused by the
        next decode step: read it (or copy it) before stepping again."""
        if self.use_graphs and self._is_plain_decode(items):
            return self._run_recorded(items)
        ctx = pack_batch(items, self.paged_group_ids, self.max_pages_per_seq, self.cache_param.page_size,
                         self.device, vocab_size=self.model.vocab_size,
                         max_positions=self.model.max_positions, planners=self.planners)
        return self.run_context(ctx)

    def run_context(self, ctx: StepContext) -> torch.Tensor:
        logits = self.model.forward(ctx, self.cache.views)
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
        with K.tuned_products():
            self.model.forward(buffers.ctx, self.cache.views)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(buffers.ctx, self.cache.views)
        rec = _RecordedStep(buffers, graph, logits)
        self._recorded[capacity] = rec
        return rec

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
        rec.buffers.fill(np.zeros(B, dtype=np.int32), np.asarray(starts, dtype=np.int32),
                         slots.astype(np.int32),
                         {g: self.manager.table_array[g][slots] for g in self.paged_group_ids})
        rec.buffers.ctx.token_ids[:B].copy_(tokens_dev)      # after the upload, in stream order
        rec.graph.replay()
        self.steps_run += 1
        self.graph_replays += 1
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
        return rec.logits[:B]
