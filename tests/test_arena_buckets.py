"""The step arena's bookkeeping and the bucket rules of recorded steps, on the CPU."""
import numpy as np
import pytest
import torch

from swifttransformer_amd.engine.batch import StepItem, token_bucket
from swifttransformer_amd.ops import arena as A
from swifttransformer_amd.parts.attention import plan_tiles
from swifttransformer_amd.parts.base import count_bucket


def test_arena_banks_take_turns_and_addresses_repeat():
    arena = A.StepArena("cpu")
    arena.resize(4096)
    assert arena.nbytes() == 8192

    def step():
        with A.using(arena):
            e = A.empty((10, 8), torch.float32, "cpu")          # embedding: bank 1
            A.next_bank()
            a = A.empty((100,), torch.bfloat16, "cpu")          # layer 0: bank 0
            b = A.empty((3, 5), torch.int32, "cpu")
            A.next_bank()
            c = A.empty((64,), torch.float32, "cpu")            # layer 1: bank 1 again, from its start
            A.next_bank()
            d = A.empty((7,), torch.float32, "cpu")             # layer 2: bank 0 again
            return [t.data_ptr() for t in (e, a, b, c, d)], (e, a, b, c, d)

    ptrs, tensors = step()
    base = arena.buffer.data_ptr()
    e, a, b, c, d = ptrs
    assert e == base + 4096 and a == base and b == base + 256 and c == base + 4096 and d == base
    assert all((p - base) % 256 == 0 for p in ptrs)       # (a device buffer itself starts on such a boundary)
    assert tensors[2].shape == (3, 5) and tensors[2].dtype == torch.int32 and tensors[1].dtype == torch.bfloat16
    tensors[1].fill_(1.0)
    tensors[2].fill_(7)
    assert (tensors[1] == 1).all() and (tensors[2] == 7).all()          # neighbours do not overlap
    assert step()[0] == ptrs                                            # the same addresses in every step
    assert arena.overflows == 0 and arena.carved == 10 and arena.peak == 512
    # outside a step, and inside `outside()`, the ordinary allocator serves
    assert A.current() is None
    t = A.empty((4,), torch.float32, "cpu")
    assert not (base <= t.data_ptr() < base + 8192)
    with A.using(arena):
        with A.outside():
            u = A.empty((4,), torch.float32, "cpu")
        v = A.empty((4,), torch.float32, "cpu")
    assert not (base <= u.data_ptr() < base + 8192) and base <= v.data_ptr() < base + 8192


def test_arena_overflow_measure_and_resume():
    arena = A.StepArena("cpu")
    arena.resize(1024)
    with A.using(arena):
        A.next_bank()
        a = A.empty((200,), torch.float32, "cpu")               # 800 bytes -> 1024 with alignment
        b = A.empty((8,), torch.float32, "cpu")                 # does not fit any more
        state = arena.state()
    base = arena.buffer.data_ptr()
    assert base <= a.data_ptr() < base + 2048 and not (base <= b.data_ptr() < base + 2048)
    assert arena.overflows == 1
    # going on from a state: the next bank is the other one, the first stays as it was
    with A.using(arena, state):
        A.next_bank()
        c = A.empty((8,), torch.float32, "cpu")
    assert c.data_ptr() == base + 1024
    # measuring: nothing is carved, the need per bank is recorded
    m = A.StepArena("cpu")
    m.measure = True
    with A.using(m):
        A.empty((100,), torch.float32, "cpu")
        A.next_bank()
        A.empty((1000,), torch.float32, "cpu")
        A.empty((10,), torch.float32, "cpu")
        A.next_bank()
        A.empty((50,), torch.float32, "cpu")
    assert m.peak == 4096 + 256 and m.carved == 0 and m.buffer is None


def test_bucket_rules():
    assert [token_bucket(n) for n in (1, 7, 8, 9, 16, 17, 33, 64, 65, 128, 129, 576, 1000, 1025, 2048, 4097)] == \
        [1, 7, 8, 10, 16, 32, 64, 64, 128, 128, 192, 576, 1024, 1280, 2048, 5120]
    assert [count_bucket(n) for n in (0, 3, 8, 9, 15, 17, 64, 65)] == [0, 3, 8, 10, 16, 24, 64, 96]
    for n in range(1, 5000, 7):
        assert n <= token_bucket(n) <= max(n + 1, int(n * 1.5)) + 31


def test_plans_of_recorded_steps_have_shared_lengths():
    items = [StepItem(slot=0, start=10, tokens=[1] * 100), StepItem(slot=1, start=0, tokens=[2]),
             StepItem(slot=2, start=5, tokens=[3] * 3), StepItem(slot=3, start=300, tokens=[4] * 70)]
    exact = plan_tiles(items, 8, 64)
    assert exact.host == {"num_tiles": 4, "num_short_rows": 4, "tile_rows": 64}
    assert exact.arrays["short_rows"].tolist() == [100, 101, 102, 103]
    padded = plan_tiles(items, 8, 64, bucketed=True)
    assert padded.host == {"num_tiles": 4, "num_short_rows": 4, "tile_rows": 64}
    more = [StepItem(slot=i, start=0, tokens=[1] * 70) for i in range(5)] + [StepItem(slot=9, start=3, tokens=[5] * 5)]
    padded = plan_tiles(more, 8, 64, bucketed=True)
    assert padded.host == {"num_tiles": 10, "num_short_rows": 8, "tile_rows": 64}
    ti, tq, sr = (padded.arrays[k].tolist() for k in ("tile_item", "tile_q0", "short_rows"))
    assert ti.count(-1) == 0 and len(ti) == 10                  # ten tiles are ten: no padding needed
    assert sr == [350, 351, 352, 353, 354, -1, -1, -1]
    odd = [StepItem(slot=i, start=0, tokens=[1] * 70) for i in range(6)] + [StepItem(slot=8, start=0, tokens=[1] * 8)]
    padded = plan_tiles(odd, 8, 64, bucketed=True)              # 13 tiles -> a list of 14, the padding first
    ti = padded.arrays["tile_item"].tolist()
    assert len(ti) == 14 and ti[0] == -1 and ti.count(-1) == 1 and padded.host["num_short_rows"] == 0
    assert plan_tiles([StepItem(slot=0, start=0, tokens=[1])], 8, 64, bucketed=True) is None
