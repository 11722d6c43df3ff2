"""A step's batch and the device-side description of it.

The reference's ``forward`` takes whole prompts or single tokens plus
``first_token_indexes`` and builds eight index arrays on the host, each copied
with its own blocking memcpy (src/csrc/model/gpt/gpt.cc:87-104, :266-296,
:518-539).  Here an item is (request, start position, tokens, wanted rows) for
any cut of a prompt, and all index arrays travel in one packed int32 buffer.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..ops.kernels import PREFILL_TILE


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
    positions: torch.Tensor        # [T] position of each token in its request
    token_item: torch.Tensor       # [T] batch item of each token (-1: padding)
    item_start: torch.Tensor       # [B]
    item_len: torch.Tensor         # [B] tokens of the item in this step
    item_tok_off: torch.Tensor     # [B] first batch row of the item
    item_slot: torch.Tensor        # [B] state slot
    want_rows: torch.Tensor        # [R] batch rows whose logits are wanted
    block_tables: Dict[int, torch.Tensor]   # group -> [B, max_pages]
    # attention work split: rows of short items go to the row kernel, long items to tiles
    short_rows: Optional[torch.Tensor]      # [Ns] batch rows (None: every row is "short")
    num_short_rows: int
    tile_item: Optional[torch.Tensor]       # [Nt]
    tile_q0: Optional[torch.Tensor]         # [Nt]
    num_tiles: int
    max_kv_len: int                # longest start+len over the items (host knowledge)
    all_single: bool               # every item has exactly one token
    # host copies for parts that decide on the host
    host_item_start: List[int] = field(default_factory=list)
    host_item_len: List[int] = field(default_factory=list)
    host_item_slot: List[int] = field(default_factory=list)
    fixed_splits: int = 0          # > 0: the number of key splits is fixed (graph replay)


class BatchError(ValueError):
    pass


def pack_batch(items: Sequence[StepItem], groups: Sequence[int], max_pages: int, page_size: int,
               device, *, vocab_size: int, max_positions: int, tile_min_len: int = 8,
               pad_items: int = 0) -> StepContext:
    """Check a batch and move its description to the device in one copy.

    ``tile_min_len``: items with at least this many tokens are cut into tiles of
    PREFILL_TILE rows for the tiled attention kernel; shorter ones go row by row.
    ``pad_items``: pad a batch of single-token items to this many items (fixed-size
    batches for graph replay); padding rows have token_item = -1."""
    B = len(items)
    if B == 0:
        raise BatchError("a step needs at least one item")
    seen = set()
    T = 0
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
        T += n
    all_single = all(len(it.tokens) == 1 for it in items)
    Bp = max(B, pad_items) if (pad_items and all_single) else B
    Tp = T + (Bp - B)
    R = sum(len(it.want) for it in items)

    short_rows: List[int] = []
    tile_item: List[int] = []
    tile_q0: List[int] = []
    # layout of the packed buffer
    sizes = [("token_ids", Tp), ("positions", Tp), ("token_item", Tp), ("item_start", Bp),
             ("item_len", Bp), ("item_tok_off", Bp), ("item_slot", Bp), ("want_rows", max(R, 1))]
    for g in groups:
        sizes.append((f"bt{g}", Bp * max_pages))
    off = {}
    total = 0
    for name, n in sizes:
        off[name] = (total, n)
        total += n
    # tiles and short rows are appended after counting
    token_ids = np.zeros(Tp, np.int32)
    positions = np.full(Tp, -1, np.int32)
    token_item = np.full(Tp, -1, np.int32)
    item_start = np.zeros(Bp, np.int32)
    item_len = np.zeros(Bp, np.int32)
    item_tok_off = np.zeros(Bp, np.int32)
    item_slot = np.full(Bp, -1, np.int32)
    want_rows = np.zeros(max(R, 1), np.int32)
    bts = {g: np.full((Bp, max_pages), -1, np.int32) for g in groups}
    t = 0
    r = 0
    max_kv = 0
    for b, it in enumerate(items):
        n = len(it.tokens)
        toks = np.asarray(it.tokens, dtype=np.int64)
        if toks.min() < 0 or toks.max() >= vocab_size:
            raise BatchError(f"token id outside [0, {vocab_size})")
        token_ids[t:t + n] = toks
        positions[t:t + n] = np.arange(it.start, it.start + n)
        token_item[t:t + n] = b
        item_start[b] = it.start
        item_len[b] = n
        item_tok_off[b] = t
        item_slot[b] = it.slot
        for w in it.want:
            want_rows[r] = t + w
            r += 1
        for g in groups:
            pg = it.pages.get(g, ())
            if len(pg) > max_pages:
                raise BatchError(f"a block table of {len(pg)} pages exceeds {max_pages}")
            bts[g][b, :len(pg)] = pg
        if n >= tile_min_len:
            for q0 in range(0, n, PREFILL_TILE):
                tile_item.append(b)
                tile_q0.append(q0)
        else:
            short_rows.extend(range(t, t + n))
        max_kv = max(max_kv, it.start + n)
        t += n
    for b in range(B, Bp):   # padding items: one row each, never computed on
        item_tok_off[b] = T + (b - B)
        short_rows.append(T + (b - B))
    every_row_short = len(tile_item) == 0
    parts = [token_ids, positions, token_item, item_start, item_len, item_tok_off, item_slot, want_rows]
    parts += [bts[g].reshape(-1) for g in groups]
    extra = {}
    if not every_row_short:
        for name, arr in (("short_rows", np.asarray(short_rows, np.int32)),
                          ("tile_item", np.asarray(tile_item, np.int32)),
                          ("tile_q0", np.asarray(tile_q0, np.int32))):
            extra[name] = (total, arr.size)
            total += arr.size
            parts.append(arr)
    host = torch.from_numpy(np.concatenate(parts))
    if torch.device(device).type == "cuda":
        host = host.pin_memory()
    dev = host.to(device, non_blocking=True)

    def view(name):
        o, n = off[name]
        return dev[o:o + n]

    def xview(name):
        if name not in extra or extra[name][1] == 0:
            return None
        o, n = extra[name]
        return dev[o:o + n]

    return StepContext(
        num_tokens=Tp, num_items=Bp, num_wanted=R, page_size=page_size,
        token_ids=view("token_ids"), positions=view("positions"), token_item=view("token_item"),
        item_start=view("item_start"), item_len=view("item_len"), item_tok_off=view("item_tok_off"),
        item_slot=view("item_slot"), want_rows=view("want_rows")[:R],
        block_tables={g: view(f"bt{g}").view(Bp, max_pages) for g in groups},
        short_rows=None if every_row_short else xview("short_rows"),
        num_short_rows=Tp if every_row_short else len(short_rows),
        tile_item=xview("tile_item"), tile_q0=xview("tile_q0"), num_tiles=len(tile_item),
        max_kv_len=max_kv, all_single=all_single,
        host_item_start=[it.start for it in items], host_item_len=[len(it.tokens) for it in items],
        host_item_slot=[it.slot for it in items],
    )
