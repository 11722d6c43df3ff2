"""The step function: run a batch of (request, its next tokens) from the cache.

Counterpart of the reference's ``Gpt<T>::forward(input_tokens_batched,
first_token_indexes, k_cache, v_cache, block_table)`` (src/csrc/model/gpt/gpt_base.h:74-83,
src/csrc/model/gpt/gpt.cc:507-657), which accepts whole prompts and single decode
tokens and returns one greedy token per request.  Here a batch may also hold
portions of prompts cut anywhere, the cache pool and block tables are owned by
the runner's cache manager, and float32 logits at the wanted positions come
back; choosing tokens is the sampler's job."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from ..cache.device import DeviceCache
from ..cache.manager import CacheManager
from ..config.cache_param import CacheParam
from ..models.decoder import DecoderModel
from .batch import StepContext, StepItem, pack_batch


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class ModelRunner:
    def __init__(self, model: DecoderModel, cache_param: CacheParam, device="cuda:0",
                 cache_fill: float = 0.0):
        self.model = model
        self.device = torch.device(device)
        self.cache_param = cache_param
        max_pages = cache_param.max_pages_per_seq or cache_param.pages_for(model.max_positions)
        self.max_pages_per_seq = max_pages
        self.manager = CacheManager(model.cache_needs(), cache_param.page_size, cache_param.num_pages,
                                    cache_param.max_seqs, max_pages)
        self.cache = DeviceCache(self.manager, model.dtype, self.device, fill=cache_fill)
        self.paged_group_ids = [g.index for g in self.manager.paged_groups]
        self.tile_min_len = 8
        self.steps_run = 0

    # ----------------------------------------------------------------- requests
    def admit(self, req_id: Hashable) -> None:
        rc = self.manager.admit(req_id)
        self.cache.reset_slot(rc.slot)

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
                rc = self.manager.requests[req_id]
                for g, n in before.items():
                    extra = rc.tables[g][n:]
                    self.manager.groups[g].pool.free([p for p in extra if p >= 0])
                    del rc.tables[g][n:]
                rc.length = start
            raise
        return items

    def run(self, items: Sequence[StepItem]) -> torch.Tensor:
        ctx = pack_batch(items, self.paged_group_ids, self.max_pages_per_seq, self.cache_param.page_size,
                         self.device, vocab_size=self.model.vocab_size,
                         max_positions=self.model.max_positions, tile_min_len=self.tile_min_len)
        return self.run_context(ctx)

    def run_context(self, ctx: StepContext) -> torch.Tensor:
        logits = self.model.forward(ctx, self.cache.views)
        self.steps_run += 1
        return logits

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """float32 logits [sum of wanted rows, vocab], in the order of entries and of want."""
        return self.run(self.prepare(entries))
