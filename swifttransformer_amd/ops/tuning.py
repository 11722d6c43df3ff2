"""Thresholds that were fitted by measurement, in one place.

None of them decides whether a result is right: each chooses between two kernels, or two shapes
of one kernel, that compute the same thing.  They were fitted on an MI355X (256 compute units)
at the layer sizes named beside them, and a sweep over other sizes has already moved some of
them once; on another device or model family they are the first thing to measure again.  The
parts read them from ``tuning`` when they run, so changing a field takes effect at the next step
(steps recorded before keep the shapes they were recorded with).

The thresholds that live in the kernel library have setters of the same kind:
``ops.kernels.gemm_library_rule`` (from how many rows, and for how large and deep a matrix, a
product goes to the vendor library) and ``ops.kernels.gemm_wide_workgroups``."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class Tuning:
    # A product takes the norm of its input rows as its prologue (instead of a norm kernel before
    # it) up to this many rows and this width.  Every workgroup of such a product normalises all
    # rows again, so the kernel it saves is paid back as rows and width grow.  Recorded decode
    # steps of 24 layers: at width 2048 the fused form wins up to the 16 rows the product kernel
    # takes (14 rows: 6,710 tokens/s against 6,390; 16 rows: 7,150 against 7,050); at width 4096
    # it loses at every row count (a layer at 8 rows: 169 us fused against 155 us).
    fused_norm_max_rows: int = 16
    fused_norm_max_width: int = 2048
    # The decode attention splits a row's keys over workgroups until there is a workgroup for
    # every compute unit, at least this many keys a split (two workgroups a unit were 0-2 %
    # slower at batch 2 to 12, OPT-1.3B sizes).
    min_keys_per_split: int = 256
    # A step that is not plain decoding is recorded when its shape comes up for this many-th time.
    record_after: int = 2
    # Recordings of up to this many rows have the vendor library's kernels timed (20 to 100 ms a
    # product shape, once).  Up to 256 rows the fastest candidate is 10 to 25 % ahead of the
    # library's first suggestion at the OPT-1.3B sizes (a layer's four products: 92 -> 76 us at 256
    # rows) and within 3 % beyond; at the 13B sizes the first suggestion is off at prompt sizes too
    # (FC2 at 512 rows 202 -> 156 us, FC1 at 2,048 rows 465 -> 365 us: a layer 8 to 10 % faster),
    # so every recording times them.
    tune_products_up_to_rows: int = 1 << 20


tuning = Tuning()
