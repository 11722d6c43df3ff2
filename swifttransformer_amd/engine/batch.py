"""A step's batch and the device-side description of it.

The reference's ``forward`` takes whole prompts or single tokens plus
``first_token_indexes`` and builds eight index arrays on the host, each copied
with its own blocking memcpy (src/csrc/model/gpt/gpt.cc:87-104, :266-296,
:518-539).  Here an item is (request, start position, tokens, wanted rows) for
any cut of a prompt, and all index arrays travel in one packed int32 buffer.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import BatchInfo, StepPlan


@dataclass
class StepItem:
    """The next tokens of one request.

    ``start`` is the position of ``tokens[0]`` in the request (= number of tokens the
    cache already holds for it); ``want`` lists indices into ``tokens`` whose logits
    are returned; ``slot`` is the request's state slot; ``pages[g]`` is its block table
    in cache group g (it must already cover position start+len(tokens)-1)."""
    slot: int
    start: int
    tokens: Sequence[int]
    want: Sequence[int] = ()
    pages: Dict[int, Sequence[int]] = field(default_factory=dict)


@dataclass
class StepContext:
    """Device tensors (int32) describing the batch, shared by all parts of a step."""
    num_tokens: int
    num_items: int
    num_wanted: int
    page_size: int
    token_ids: torch.Tensor        # [T]
    positions: torch.Tensor        # [T] position of each token in its request (-1: padding)
    token_item: torch.Tensor       # [T] batch item of each token (-1: padding)
    item_start: torch.Tensor       # [B]
    item_len: torch.Tensor         # [B] tokens of the item in this step
    item_tok_off: torch.Tensor     # [B] first batch row of the item
    item_slot: torch.Tensor        # [B] state slot
    want_rows: torch.Tensor        # [R] batch rows whose logits are wanted
    block_tables: Dict[int, torch.Tensor]   # group -> [B, max_pages]
    max_kv_len: int                # longest start+len over the items (host knowledge)
    all_single: bool               # every item has exactly one token
    # host copies for parts that decide on the host
    host_item_start: List[int] = field(default_factory=list)
    host_item_len: List[int] = field(default_factory=list)
    host_item_slot: List[int] = field(default_factory=list)
    # True when the step is recorded once and replayed: nothing may depend on the values
    # of this step (lengths, slots); kernels size their work for `max_kv_len` = the longest
    # sequence the model allows
    static_shapes: bool = False
    # the model's position encoding, for mixers to call its ``rotate`` (set by the model)
    position: Optional[object] = None
    # work lists that parts asked for through their ``step_planner`` (key -> StepPlan); a key is
    # absent when its planner had nothing to say about this batch, and in recorded steps
    plans: Dict[Hashable, "StepPlan"] = field(default_factory=dict)


# A planner looks at the items of a step on the host (and at the page size and table width) and
# returns a StepPlan of numpy int32 arrays (or None: nothing to plan for this batch).
Planner = Callable[[Sequence[StepItem], BatchInfo], Optional[StepPlan]]


class BatchError(ValueError):
    pass


def check_items(items: Sequence[StepItem], groups: Sequence[int], page_size: int,
                vocab_size: int, max_positions: int) -> None:
    if len(items) == 0:
        raise BatchError("a step needs at least one item")
    seen = set()
    for it in items:
        n = len(it.tokens)
        if n < 1:
            raise BatchError("an item needs at least one token")
        if it.slot in seen:
            raise BatchError(f"state slot {it.slot} appears twice in one step")
        seen.add(it.slot)
        if it.start < 0 or it.start + n > max_positions:
            # the reference asserts the last position < max_position_embeddings (gpt.cc:528-534)
            raise BatchError(f"tokens at positions {it.start}..{it.start + n - 1} do not fit "
                             f"the model's {max_positions} positions")
        for w in it.want:
            if not 0 <= w < n:
                raise BatchError(f"wanted index {w} is outside the item's {n} tokens")
        need_pages = -(-(it.start + n) // page_size)
        for g in groups:
            # released pages of a windowed group stay in the table as -1
            if len(it.pages.get(g, ())) < need_pages:
                raise BatchError(f"the block table of group {g} has {len(it.pages.get(g, ()))} "
                                 f"pages; positions up to {it.start + n - 1} need {need_pages}")
        if min(it.tokens) < 0 or max(it.tokens) >= vocab_size:
            raise BatchError(f"token id outside [0, {vocab_size})")


class BatchLayout:
    """Offsets of the index arrays inside the packed int32 buffer."""

    def __init__(self, T: int, B: int, R: int, groups: Sequence[int], max_pages: int,
                 extra: Sequence[Tuple[str, int]] = ()):
        self.T, self.B, self.R, self.max_pages = T, B, R, max_pages
        self.groups = list(groups)
        sizes = [("token_ids", T), ("positions", T), ("token_item", T), ("item_start", B),
                 ("item_len", B), ("item_tok_off", B), ("item_slot", B), ("want_rows", max(R, 1))]
        sizes += [(f"bt{g}", B * max_pages) for g in groups]
        sizes += list(extra)       # planners' arrays, named "plan<i>.<array>"
        self.off = {}
        total = 0
        for name, n in sizes:
            self.off[name] = (total, n)
            total += n
        self.total = total

    def view(self, buf, name: str):
        o, n = self.off[name]
        return buf[o:o + n]

    def has(self, name: str) -> bool:
        return name in self.off and self.off[name][1] > 0

    def context(self, dev: torch.Tensor, page_size: int, **kw) -> StepContext:
        v = lambda n: self.view(dev, n)
        return StepContext(
            num_tokens=self.T, num_items=self.B, num_wanted=self.R, page_size=page_size,
            token_ids=v("token_ids"), positions=v("positions"), token_item=v("token_item"),
            item_start=v("item_start"), item_len=v("item_len"), item_tok_off=v("item_tok_off"),
            item_slot=v("item_slot"), want_rows=v("want_rows")[:self.R],
            block_tables={g: v(f"bt{g}").view(self.B, self.max_pages) for g in self.groups}, **kw)


Planned = List[Tuple[Hashable, StepPlan, List[Tuple[str, str, np.ndarray]]]]


def run_planners(items: Sequence[StepItem], planners: Optional[Dict[Hashable, Planner]],
                 info: BatchInfo) -> Tuple[Planned, List[Tuple[str, int]]]:
    """Ask every planner for its plan of ``items``: (key, plan, [(array name, name in the packed
    buffer, int32 array)]) for the planners that had something to say, and the packed names with
    their lengths."""
    planned: Planned = []
    extra: List[Tuple[str, int]] = []
    for i, (key, planner) in enumerate((planners or {}).items()):
        plan = planner(items, info)
        if plan is None:
            continue
        named = []
        for name, arr in plan.arrays.items():
            arr = np.ascontiguousarray(arr, dtype=np.int32).reshape(-1)
            named.append((name, f"plan{i}.{name}", arr))
            extra.append((f"plan{i}.{name}", arr.size))
        planned.append((key, plan, named))
    return planned, extra


def pack_batch(items: Sequence[StepItem], groups: Sequence[int], max_pages: int, page_size: int,
               device, *, vocab_size: int, max_positions: int,
               planners: Optional[Dict[Hashable, Planner]] = None) -> StepContext:
    """Check a batch and move its description to the device in one copy.

    ``planners``: key -> planner of the parts that want work lists of their own for the step
    (``DecoderModel.step_planners()``); their arrays ride in the same copy and come back as
    ``ctx.plans[key]``."""
    check_items(items, groups, page_size, vocab_size, max_positions)
    B = len(items)
    T = sum(len(it.tokens) for it in items)
    R = sum(len(it.want) for it in items)
    planned, extra = run_planners(items, planners, BatchInfo(page_size=page_size, max_pages=max_pages))
    lay = BatchLayout(T, B, R, groups, max_pages, extra)
    host = np.zeros(lay.total, np.int32)
    hv = lambda n: lay.view(host, n)
    token_ids, positions, token_item = hv("token_ids"), hv("positions"), hv("token_item")
    item_start, item_len, item_tok_off, item_slot = (hv("item_start"), hv("item_len"),
                                                     hv("item_tok_off"), hv("item_slot"))
    want_rows = hv("want_rows")
    bts = {g: hv(f"bt{g}").reshape(B, max_pages) for g in groups}
    for g in groups:
        bts[g].fill(-1)
    t = r = 0
    max_kv = 0
    for b, it in enumerate(items):
        n = len(it.tokens)
        token_ids[t:t + n] = it.tokens
        positions[t:t + n] = np.arange(it.start, it.start + n)
        token_item[t:t + n] = b
        item_start[b], item_len[b], item_tok_off[b], item_slot[b] = it.start, n, t, it.slot
        for w in it.want:
            want_rows[r] = t + w
            r += 1
        for g in groups:
            pg = it.pages.get(g, ())
            if len(pg) > max_pages:
                raise BatchError(f"a block table of {len(pg)} pages exceeds {max_pages}")
            bts[g][b, :len(pg)] = pg
        max_kv = max(max_kv, it.start + n)
        t += n
    for _key, _plan, named in planned:
        for _name, packed, arr in named:
            hv(packed)[:] = arr
    host_t = torch.from_numpy(host)
    if torch.device(device).type == "cuda":
        host_t = host_t.pin_memory()
    dev = host_t.to(device, non_blocking=True)
    ctx = lay.context(
        dev, page_size, max_kv_len=max_kv, all_single=all(len(it.tokens) == 1 for it in items),
        host_item_start=[it.start for it in items], host_item_len=[len(it.tokens) for it in items],
        host_item_slot=[it.slot for it in items])
    for key, plan, named in planned:
        ctx.plans[key] = StepPlan({name: lay.view(dev, packed) for name, packed, _ in named}, dict(plan.host))
    return ctx


class DecodeBuffers:
    """Fixed buffers for batches of up to ``capacity`` single-token items that all want
    their logits: a pinned host buffer, its device twin at a fixed address, and the
    context whose tensors view the device buffer.  A recorded step (HIP graph) reads
    the same addresses at every replay; only the contents change.  Unused rows are
    padding (token_item = -1): kernels skip them."""

    def __init__(self, capacity: int, groups: Sequence[int], max_pages: int, page_size: int, device,
                 max_positions: int):
        self.capacity = capacity
        self.lay = BatchLayout(capacity, capacity, capacity, groups, max_pages)
        self.host = torch.zeros(self.lay.total, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(self.lay.total, dtype=torch.int32, device=device)
        self.groups = list(groups)
        self.max_pages = max_pages
        self.ctx = self.lay.context(self.dev, page_size, max_kv_len=max_positions, all_single=True,
                                    static_shapes=True)
        hv = lambda n: self.lay.view(self.host_np, n)
        self._tok, self._pos, self._item = hv("token_ids"), hv("positions"), hv("token_item")
        self._start, self._len, self._off, self._slot = (hv("item_start"), hv("item_len"),
                                                         hv("item_tok_off"), hv("item_slot"))
        self._bts = {g: hv(f"bt{g}").reshape(capacity, max_pages) for g in groups}
        hv("want_rows")[:] = np.arange(capacity)
        self._off[:] = np.arange(capacity)
        self._copied = torch.cuda.Event() if torch.device(device).type == "cuda" else None
        self.fill_padding()

    def _upload(self, tokens: bool = True) -> None:
        # (the token ids are the buffer's first `capacity` words)
        skip = 0 if tokens else self.capacity
        self.dev[skip:].copy_(self.host[skip:], non_blocking=True)
        if self._copied is not None:
            self._copied.record()

    def _host_is_free(self) -> None:
        # the previous upload must have left the pinned buffer before it is rewritten
        if self._copied is not None:
            self._copied.synchronize()

    def fill_padding(self) -> None:
        self._host_is_free()
        self._tok[:] = 0
        self._pos[:] = -1
        self._item[:] = -1
        self._start[:] = 0
        self._len[:] = 0
        self._slot[:] = -1
        for g in self.groups:
            self._bts[g][:] = -1
        self._upload()

    def fill(self, tokens: Optional[np.ndarray], starts: np.ndarray, slots: np.ndarray,
             tables: Dict[int, np.ndarray]) -> None:
        """tokens/starts/slots: [B]; tables[g]: [B, max_pages] rows of the block tables.
        ``tokens`` None: the token ids are on the device already (or are put there by the
        caller after this): that part of the device buffer is left as it is."""
        B = len(starts)
        self._host_is_free()
        if tokens is not None:
            self._tok[:B] = tokens
        self._pos[:B] = starts
        self._item[:B] = np.arange(B)
        self._start[:B] = starts
        self._len[:B] = 1
        self._slot[:B] = slots
        self._pos[B:] = -1
        self._item[B:] = -1
        self._len[B:] = 0
        self._slot[B:] = -1
        for g in self.groups:
            self._bts[g][:B] = tables[g]
        self._upload(tokens is not None)


def token_bucket(n: int) -> int:
    """Rows of the recorded step that serves a batch of ``n`` tokens which are not all single
    decode tokens: ``n`` itself up to 8, the next even number up to 16, 32, 64, then the next
    multiple of 64 up to 1,024, of 256 up to 4,096, of 1,024 beyond.  The rows a batch does not
    fill are padding that every kernel skips or computes for nothing."""
    if n <= 8:
        return n
    if n <= 16:
        return n + (n & 1)
    if n <= 64:
        return 32 if n <= 32 else 64
    if n <= 1024:
        return -(-n // 64) * 64
    if n <= 4096:
        return -(-n // 256) * 256
    return -(-n // 1024) * 1024


class StepBuffers:
    """Fixed buffers of a recorded step of any composition: ``num_tokens`` rows (prompt portions
    and single tokens, the rest padding), up to ``max_items`` items, ``num_wanted`` rows of logits,
    and the parts' work lists at the lengths their planners gave them.  As with ``DecodeBuffers``
    a pinned host buffer is filled and copied to a device buffer whose address the recording
    holds."""

    def __init__(self, num_tokens: int, max_items: int, num_wanted: int, groups: Sequence[int], max_pages: int,
                 page_size: int, device, max_positions: int, planned: "Planned", extra: List[Tuple[str, int]]):
        self.num_tokens, self.max_items, self.num_wanted = num_tokens, max_items, num_wanted
        self.groups, self.max_pages = list(groups), max_pages
        self.lay = BatchLayout(num_tokens, max_items, num_wanted, groups, max_pages, extra)
        pin = torch.device(device).type == "cuda"
        self.host = torch.zeros(self.lay.total, dtype=torch.int32)
        if pin:
            self.host = self.host.pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(self.lay.total, dtype=torch.int32, device=device)
        self.ctx = self.lay.context(self.dev, page_size, max_kv_len=max_positions, all_single=False,
                                    static_shapes=True)
        for key, plan, named in planned:
            self.ctx.plans[key] = StepPlan({name: self.lay.view(self.dev, packed) for name, packed, _ in named},
                                           dict(plan.host))
        self.plan_names = [packed for _key, _plan, named in planned for _name, packed, _arr in named]
        hv = lambda n: self.lay.view(self.host_np, n)
        self._tok, self._pos, self._item = hv("token_ids"), hv("positions"), hv("token_item")
        self._start, self._len, self._off, self._slot = (hv("item_start"), hv("item_len"),
                                                         hv("item_tok_off"), hv("item_slot"))
        self._want = hv("want_rows")
        self._bts = {g: hv(f"bt{g}").reshape(max_items, max_pages) for g in groups}
        self._plans = {packed: hv(packed) for packed in self.plan_names}
        self._copied = torch.cuda.Event() if pin else None

    def fill(self, items: Sequence[StepItem], tables: Dict[int, np.ndarray], planned: "Planned") -> None:
        """``tables[g]``: [len(items), max_pages] rows of the block tables; ``planned``: this batch's
        plans, of the same keys and lengths as those the buffers were made for."""
        if self._copied is not None:
            self._copied.synchronize()       # the previous upload must have left the pinned buffer
        B = len(items)
        t = r = 0
        for b, it in enumerate(items):
            n = len(it.tokens)
            self._tok[t:t + n] = it.tokens
            self._pos[t:t + n] = np.arange(it.start, it.start + n)
            self._item[t:t + n] = b
            self._start[b], self._len[b], self._off[b], self._slot[b] = it.start, n, t, it.slot
            for w in it.want:
                self._want[r] = t + w
                r += 1
            t += n
        self._tok[t:] = 0
        self._pos[t:] = -1
        self._item[t:] = -1
        self._start[B:] = 0
        self._len[B:] = 0
        self._off[B:] = 0
        self._slot[B:] = -1
        self._want[r:] = 0                   # padding rows of the logits repeat row 0
        for g in self.groups:
            self._bts[g][:B] = tables[g]
            self._bts[g][B:] = -1
        names = []
        for _key, _plan, named in planned:
            for _name, packed, arr in named:
                self._plans[packed][:] = arr
                names.append(packed)
        if names != self.plan_names:
            raise BatchError("the batch's plans differ from those its recorded step was made for")
        self.dev.copy_(self.host, non_blocking=True)
        if self._copied is not None:
            self._copied.record()
