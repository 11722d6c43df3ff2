"""The step packer on the CPU: index arrays of a mixed batch, and the work lists that parts ask
for through their planners (the packer knows nothing of what they mean)."""
import numpy as np
import pytest
import torch

from swifttransformer_amd.engine.batch import BatchError, StepItem, pack_batch
from swifttransformer_amd.parts import BatchInfo, StepPlan


def items():
    return [StepItem(slot=2, start=5, tokens=[7, 8, 9], want=[0, 2], pages={0: [4, 1]}),
            StepItem(slot=0, start=0, tokens=list(range(70)), want=[69], pages={0: list(range(10, 19))}),
            StepItem(slot=1, start=30, tokens=[3], want=[0], pages={0: [5, 6, 7, 8]})]


def test_index_arrays_of_a_mixed_batch():
    ctx = pack_batch(items(), [0], 12, 8, "cpu", vocab_size=100, max_positions=200)
    assert (ctx.num_tokens, ctx.num_items, ctx.num_wanted) == (74, 3, 4)
    assert ctx.token_ids[:3].tolist() == [7, 8, 9] and ctx.positions[:3].tolist() == [5, 6, 7]
    assert ctx.token_item.tolist() == [0] * 3 + [1] * 70 + [2]
    assert ctx.positions[3:73].tolist() == list(range(70)) and ctx.positions[73].item() == 30
    assert ctx.item_start.tolist() == [5, 0, 30] and ctx.item_len.tolist() == [3, 70, 1]
    assert ctx.item_tok_off.tolist() == [0, 3, 73] and ctx.item_slot.tolist() == [2, 0, 1]
    assert ctx.want_rows.tolist() == [0, 2, 72, 73]
    bt = ctx.block_tables[0]
    assert bt.shape == (3, 12) and bt[0, :3].tolist() == [4, 1, -1] and bt[1, :9].tolist() == list(range(10, 19))
    assert ctx.max_kv_len == 70 and not ctx.all_single and ctx.plans == {}


def test_planners_arrays_travel_with_the_batch():
    seen = {}

    def planner(its, info):
        seen["info"] = info
        return StepPlan({"lengths": np.array([len(it.tokens) for it in its]), "empty": np.zeros(0, np.int64)},
                        {"total": sum(len(it.tokens) for it in its)})
    ctx = pack_batch(items(), [0], 12, 8, "cpu", vocab_size=100, max_positions=200,
                     planners={"mine": planner, "silent": lambda its, info: None})
    assert seen["info"] == BatchInfo(page_size=8, max_pages=12)
    assert set(ctx.plans) == {"mine"}
    plan = ctx.plans["mine"]
    assert plan.arrays["lengths"].dtype == torch.int32 and plan.arrays["lengths"].tolist() == [3, 70, 1]
    assert plan.arrays["empty"].numel() == 0 and plan.host == {"total": 74}
    # the batch's own arrays are where they were
    assert ctx.want_rows.tolist() == [0, 2, 72, 73]


def test_attention_planner_cuts_long_items_into_tiles():
    from swifttransformer_amd.parts.attention import plan_tiles
    plan = plan_tiles(items(), tile_min_len=8)
    assert plan.host == {"num_tiles": 2, "num_short_rows": 4, "tile_rows": 64}
    assert plan.arrays["tile_item"].tolist() == [1, 1] and plan.arrays["tile_q0"].tolist() == [0, 64]
    assert plan.arrays["short_rows"].tolist() == [0, 1, 2, 73]
    assert plan_tiles(items(), tile_min_len=100) is None                       # nothing long enough
    wide = plan_tiles(items(), 8, tile_rows=lambda rows: 128 if rows >= 70 else 64)
    assert wide.host["tile_rows"] == 128 and wide.arrays["tile_q0"].tolist() == [0]
    # more than two tiles: ordered by the last key a tile reads
    many = [StepItem(0, 500, list(range(130)), [], {0: []}), StepItem(1, 0, list(range(100)), [], {0: []})]
    plan = plan_tiles(many, 8)
    order = list(zip(plan.arrays["tile_item"].tolist(), plan.arrays["tile_q0"].tolist()))
    assert order == [(1, 0), (1, 64), (0, 0), (0, 64), (0, 128)]


def test_batches_that_cannot_run_are_refused():
    bad = items()
    bad[2] = StepItem(slot=1, start=30, tokens=[3], want=[0], pages={0: [5, 6, 7]})      # position 30 needs 4 pages of 8
    with pytest.raises(BatchError, match="block table"):
        pack_batch(bad, [0], 12, 8, "cpu", vocab_size=100, max_positions=200)
    with pytest.raises(BatchError, match="appears twice"):
        pack_batch([items()[0], items()[0]], [0], 12, 8, "cpu", vocab_size=100, max_positions=200)
    with pytest.raises(BatchError, match="do not fit"):
        pack_batch(items(), [0], 12, 8, "cpu", vocab_size=100, max_positions=60)
    with pytest.raises(BatchError, match="token id"):
        pack_batch(items(), [0], 12, 8, "cpu", vocab_size=50, max_positions=200)
