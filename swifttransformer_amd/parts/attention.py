"""Multi-head (or grouped-query) attention over the paged cache.

Order of operations, as in the reference's ``layer::attention``
(src/csrc/layer/attention.cc:102-288): fused QKV product + bias; (rotation hook of
the position encoding, a no-op for learned positions, :133-153); the new tokens'
keys and values go into their pages (:159-177); attention of every new token over
its request's cache; output product + bias, here with the residual added in the
same epilogue (the reference adds it inside the next LayerNorm,
src/csrc/kernel/layernorm.cu:40-45).

One path serves whole prompts, portions of prompts and decode tokens: the
portion's keys are written first, then each of its rows attends over the cached
positions [lo, its own].  Rows of long items are handled in tiles by the
matrix-core kernel (one instance per dtype), all others by the row kernel split over the keys.
Scores are scaled by ``scale`` (head_dim**-0.5 in the reference, attention.cc:91)."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

import numpy as np

from ..ops import kernels as K
from ..ops.tuning import tuning
from ..weights.loader import TensorSpec
from .base import CacheNeed, Mixer, StepPlan, count_bucket

_compute_units: Dict[int, int] = {}


def _target_workgroups() -> int:
    """Compute units of the current device (256 where no GPU is visible: host-only planning)."""
    if not torch.cuda.is_available():
        return 256
    dev = torch.cuda.current_device()
    if dev not in _compute_units:
        _compute_units[dev] = torch.cuda.get_device_properties(dev).multi_processor_count
    return _compute_units[dev]


def plan_tiles(items, tile_min_len: int, tile_rows=None, bucketed: bool = False) -> Optional[StepPlan]:
    """The attention work split of a step: items of at least ``tile_min_len`` tokens are cut into
    tiles of query rows for the matrix-core kernel, the rows of shorter items (decode tokens,
    small portions) go to the row kernel.  ``tile_rows``: rows per tile, or a function of the
    number of rows in the long items that chooses it (K.PREFILL_TILE if None).  None when no item
    is long enough.  ``bucketed``: the two lists are filled up with -1 (entries the kernels skip)
    to lengths that many steps share, and the counts are those lengths."""
    long_rows = sum(len(it.tokens) for it in items if len(it.tokens) >= tile_min_len)
    if long_rows == 0:
        return None
    rows = K.PREFILL_TILE if tile_rows is None else tile_rows(long_rows) if callable(tile_rows) else int(tile_rows)
    short_rows: List[int] = []
    tile_item: List[int] = []
    tile_q0: List[int] = []
    t = 0
    for b, it in enumerate(items):
        n = len(it.tokens)
        if n >= tile_min_len:
            for q0 in range(0, n, rows):
                tile_item.append(b)
                tile_q0.append(q0)
        else:
            short_rows.extend(range(t, t + n))
        t += n
    if len(tile_item) > 2:
        # in order of the keys a tile reads, so that the kernel can deal long and short tiles
        # evenly over the compute units
        order = sorted(range(len(tile_item)), key=lambda i: items[tile_item[i]].start + tile_q0[i])
        tile_item = [tile_item[i] for i in order]
        tile_q0 = [tile_q0[i] for i in order]
    if bucketed:
        # padding tiles come first, where the shortest tiles are
        pad = count_bucket(len(tile_item)) - len(tile_item)
        tile_item, tile_q0 = [-1] * pad + tile_item, [0] * pad + tile_q0
        # (entries of the row list that the kernel skips cost next to nothing: powers of two)
        n_short = 1 << (len(short_rows) - 1).bit_length() if short_rows else 0
        short_rows = short_rows + [-1] * (n_short - len(short_rows))
    return StepPlan({"short_rows": np.asarray(short_rows, np.int32), "tile_item": np.asarray(tile_item, np.int32),
                     "tile_q0": np.asarray(tile_q0, np.int32)},
                    {"num_tiles": len(tile_item), "num_short_rows": len(short_rows), "tile_rows": rows})


class PagedAttention(Mixer):
    """params: num_heads, num_kv_heads, head_dim, scale (float), bias (bool), window (int, 0 = all keys),
    tile_min_len (int, default 8: portions from this many tokens on take the tile kernel)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.num_heads = int(self.param("num_heads"))
        self.num_kv_heads = int(self.param("num_kv_heads", self.num_heads))
        self.head_dim = int(self.param("head_dim"))
        self.scale = float(self.param("scale"))
        self.bias = bool(self.param("bias", True))
        self.window = int(spec.params.get("window", 0) or 0)
        self.tile_min_len = int(spec.params.get("tile_min_len", 8))
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads do not divide into {self.num_kv_heads} key heads")
        if self.head_dim % 16 or self.head_dim > 256:
            raise ValueError(f"head_dim {self.head_dim}: the attention kernels take multiples of 16 up to 256")
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_qkv = self.b_qkv = self.w_out = self.b_out = None
        self.position = None     # the model's position part (use_position)

    def _slopes(self) -> Optional[torch.Tensor]:
        """Per-head slopes of a position encoding that biases scores by distance, or None."""
        if self.position is not None and getattr(self.position, "biases_scores", False):
            return self.position.score_slopes(self.num_heads)
        return None

    # ------------------------------------------------------------------ weights
    def tensor_specs(self) -> List[TensorSpec]:
        H = self.hidden_size
        specs = [TensorSpec(self.name("q.weight"), (self.q_size, H), "matrix"),
                 TensorSpec(self.name("k.weight"), (self.kv_size, H), "matrix"),
                 TensorSpec(self.name("v.weight"), (self.kv_size, H), "matrix"),
                 TensorSpec(self.name("out.weight"), (H, self.q_size), "matrix")]
        if self.bias:
            specs += [TensorSpec(self.name("q.bias"), (self.q_size,), "vector"),
                      TensorSpec(self.name("k.bias"), (self.kv_size,), "vector"),
                      TensorSpec(self.name("v.bias"), (self.kv_size,), "vector"),
                      TensorSpec(self.name("out.bias"), (H,), "vector")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # q | k | v stacked along the output dimension: one product makes all three
        # (the reference's converter fuses them offline, scripts/lib/converter_lib.py:259-262)
        self.w_qkv = torch.cat([tensors[self.name(f"{n}.weight")] for n in "qkv"], dim=0).contiguous()
        self.w_out = tensors[self.name("out.weight")]
        if self.bias:
            self.b_qkv = torch.cat([tensors[self.name(f"{n}.bias")] for n in "qkv"], dim=0).contiguous()
            self.b_out = tensors[self.name("out.bias")]

    def cache_need(self) -> CacheNeed:
        return CacheNeed("paged_kv", num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                         window=self.window)

    def plan_key(self):
        biased = self.position is not None and getattr(self.position, "biases_scores", False)
        return ("attention_tiles", self.tile_min_len, self.num_heads, self.head_dim, self.dtype, biased)

    def step_planner(self):
        """(key, planner): attention layers of one geometry share the tile split of a step."""
        n, heads, hd, dtype = self.tile_min_len, self.num_heads, self.head_dim, self.dtype
        biased = self.position is not None and getattr(self.position, "biases_scores", False)

        def planner(items, info):
            # tiles of 128 rows where the kernels serve them better (large heads, enough rows; the
            # kernel that takes them has no score bias)
            choose = lambda rows: (K.PREFILL_TILE if biased else
                                   K.prefill_tile_rows(hd, info.page_size, info.max_pages, heads, rows, dtype))
            return plan_tiles(items, n, choose, bucketed=info.bucketed)
        return self.plan_key(), planner

    # ------------------------------------------------------------------ forward
    def _shape_row_kernel(self, ctx, rows: int):
        """(key splits, waves per workgroup) of the row kernel.  A workgroup serves one
        (row, head, split); when rows * heads alone does not fill the chip, a row's keys are
        split over workgroups (merged by a second kernel), at least tuning.min_keys_per_split keys
        each.  ctx.max_kv_len is the longest sequence of this step, or, for a recorded step,
        the longest the model allows: then the shape depends on the batch size alone."""
        span = ctx.max_kv_len if self.window <= 0 else min(ctx.max_kv_len, self.window)
        groups = max(1, rows * self.num_heads)
        units = _target_workgroups()
        splits = min(-(-units // groups), max(1, span // tuning.min_keys_per_split), 32)
        if splits == 1 and groups > units and span >= 2 * tuning.min_keys_per_split and (-groups) % units > units // 2:
            # more workgroups than compute units and the last round of them less than half full (9
            # rows of 32 heads on 256 units: 288): the units that get a second workgroup keep the
            # others waiting.  Workgroups of half the keys even that out (batch 10, 11, 17, 18: +2 to
            # 3 % a step; nothing where the last round is fuller).
            splits = 2
        return max(1, splits), 4

    def attend(self, qkv: torch.Tensor, ctx, cache, unmerged_ok: bool = False):
        """Attention of every row of ``qkv`` [T, q+2kv] over ``cache`` (already holding the rows' keys).
        With ``unmerged_ok`` the result may be a ``SplitAttention`` that the output projection merges."""
        T = qkv.shape[0]
        q = qkv[:, :self.q_size]
        bt = ctx.block_tables[cache.group]
        out = K.empty((T, self.q_size), self.dtype, qkv.device)
        slopes = self._slopes()
        plan = ctx.plans.get(self.plan_key())
        if plan is not None and K.prefill_available():
            K.attention_prefill(q, cache.k, cache.v, plan.arrays["tile_item"], plan.arrays["tile_q0"],
                                ctx.item_tok_off, ctx.item_start, ctx.item_len, bt, self.num_heads, self.scale,
                                window=self.window, out=out, tile_rows=plan.host["tile_rows"], head_slopes=slopes)
            if plan.host["num_short_rows"] > 0:
                splits, waves = self._shape_row_kernel(ctx, plan.host["num_short_rows"])
                K.attention_rows(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads,
                                 self.scale, window=self.window, row_ids=plan.arrays["short_rows"],
                                 num_splits=splits, num_waves=waves, out=out, head_slopes=slopes)
        else:
            splits, waves = self._shape_row_kernel(ctx, T)
            if unmerged_ok and splits > 1 and K.can_fuse_merge(T, self.hidden_size, self.q_size, splits,
                                                               self.num_heads, self.head_dim, self.dtype):
                return K.attention_rows(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads,
                                        self.scale, window=self.window, num_splits=splits, num_waves=waves,
                                        merge=False, head_slopes=slopes)
            K.attention_rows(q, cache.k, cache.v, ctx.token_item, ctx.positions, bt, self.num_heads,
                             self.scale, window=self.window, num_splits=splits, num_waves=waves, out=out,
                             head_slopes=slopes)
        return out

    accepts_norm = True     # forward(..., norm=part) normalises residual32 itself

    def forward(self, x_t: Optional[torch.Tensor], residual32: torch.Tensor, ctx, cache, write: bool = True,
                norm=None) -> torch.Tensor:
        """residual32 + mix(x_t).  With ``norm`` (a norm part that offers ``as_input``), the
        mixer's input is norm(residual32), computed inside the QKV product."""
        x_in = norm.as_input(residual32) if norm is not None else x_t
        position = self.position if self.position is not None else getattr(ctx, "position", None)
        if position is not None and getattr(position, "rotates", False):
            # a position encoding that turns queries and keys: product, rotation, then the page write
            qkv = K.gemm(x_in, self.w_qkv, bias=self.b_qkv)
            k_new = qkv[:, self.q_size:self.q_size + self.kv_size]
            position.rotate(qkv[:, :self.q_size], k_new, ctx)
            if write:
                K.kv_write(cache.k, cache.v, k_new, qkv[:, self.q_size + self.kv_size:], ctx.token_item,
                           ctx.positions, ctx.block_tables[cache.group], ctx.page_size)
        else:
            # the new keys and values go to their pages from the product's epilogue
            scatter = K.KvScatter(cache.k, cache.v, ctx.token_item, ctx.positions,
                                  ctx.block_tables[cache.group], self.q_size) if write else None
            qkv = K.gemm(x_in, self.w_qkv, bias=self.b_qkv, kv_scatter=scatter)
        # a decode attention split over the keys is merged by the output projection itself
        o = self.attend(qkv, ctx, cache, unmerged_ok=True)
        return K.gemm(o, self.w_out, bias=self.b_out, residual=residual32, out_f32=True)
