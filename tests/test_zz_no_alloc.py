"""The decode attention entry point that allocates nothing (``st_attn_rows_static``), called
through ``ctypes`` as a caller without torch's faces would, against the existing entry point
with a caller's workspace (``st_attn_rows``): two calls in a row, the second with a smaller
input, so that what the first call left in the library's static scratch is still there."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

_p, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float


def _library():
    from swifttransformer_amd.ops import library
    lib = library.load()
    lib.st_last_error.restype = ctypes.c_char_p
    lib.st_attn_rows_static_capacity.restype = ctypes.c_size_t
    lib.st_attn_rows_static.argtypes = [_p, _p, _i64, _p, _p, _i64, _p, _p, _p, _p, _p] + [_i] * 6 + [_f] + [_i] * 4 + [_p]
    lib.st_attn_rows.argtypes = [_p, _p, _p, _p, _i64, _p, _p, _i64, _p, _p, _p, _p, _p] + [_i] * 6 + [_f] + [_i] * 4 + [_p]
    return lib


def _case(rows, heads, hd, ctx_len, page, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    pages_per = -(-ctx_len // page)
    num_pages = rows * pages_per + 3
    k = torch.randn((num_pages, heads, page, hd), generator=g).to(dtype).to(DEV)
    v = torch.randn((num_pages, heads, page, hd), generator=g).to(dtype).to(DEV)
    q = torch.randn((rows, heads * hd), generator=g).to(dtype).to(DEV)
    perm = torch.randperm(num_pages, generator=g)[:rows * pages_per].to(torch.int32)
    table = perm.view(rows, pages_per).contiguous().to(DEV)
    item = torch.arange(rows, dtype=torch.int32, device=DEV)
    # each row sits at another position: the splits' chunks differ from row to row
    pos = torch.tensor([ctx_len - 1 - 7 * r for r in range(rows)], dtype=torch.int32, device=DEV)
    return q, k, v, table, item, pos


def _run_both(lib, rows, heads, hd, ctx_len, page, splits, dtype, seed):
    q, k, v, table, item, pos = _case(rows, heads, hd, ctx_len, page, dtype, seed)
    code = 0 if dtype == torch.float32 else 1
    stream = torch.cuda.current_stream().cuda_stream
    scale = hd ** -0.5
    tail = (table.shape[1], page, rows, heads, heads, hd, scale, 0, splits, 4, code, stream)
    want = torch.zeros((rows, heads * hd), dtype=dtype, device=DEV)
    work = torch.empty(rows * heads * splits * (hd + 1), dtype=torch.float32, device=DEV)
    n_o = rows * heads * splits * hd
    rc = lib.st_attn_rows(want.data_ptr(), work.data_ptr(), work.data_ptr() + 4 * n_o, q.data_ptr(), q.stride(0),
                          k.data_ptr(), v.data_ptr(), k.stride(0), None, item.data_ptr(), pos.data_ptr(),
                          table.data_ptr(), None, *tail)
    assert rc == 0, lib.st_last_error().decode()
    got = torch.zeros_like(want)
    before = torch.cuda.memory_allocated()
    rc = lib.st_attn_rows_static(got.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0),
                                 None, item.data_ptr(), pos.data_ptr(), table.data_ptr(), None, *tail)
    assert rc == 0, lib.st_last_error().decode()
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, want), f"max difference {(got.float() - want.float()).abs().max().item():.3e}"
    return got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_entry_point_equals_the_workspace_one(dtype):
    lib = _library()
    assert lib.st_attn_rows_static_init() == 0, lib.st_last_error().decode()
    # first a larger call, then a smaller one that finds the first one's partial results in the scratch
    big = _run_both(lib, rows=6, heads=5, hd=64, ctx_len=900, page=16, splits=8, dtype=dtype, seed=1)
    small = _run_both(lib, rows=2, heads=3, hd=32, ctx_len=300, page=8, splits=3, dtype=dtype, seed=2)
    assert big.shape == (6, 320) and small.shape == (2, 96)
    # no split: the scratch is not touched at all
    _run_both(lib, rows=3, heads=2, hd=48, ctx_len=70, page=4, splits=1, dtype=dtype, seed=3)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    lib = _library()
    cap = lib.st_attn_rows_static_capacity()
    assert cap == 4 << 20
    rows, heads, hd, splits = 64, 64, 128, 8          # 64*64*8*129 floats = 16.9 MB
    assert rows * heads * splits * (hd + 1) * 4 > cap
    q, k, v, table, item, pos = _case(1, 1, 16, 16, 16, torch.float32, 0)
    out = torch.zeros(4, device=DEV)
    rc = lib.st_attn_rows_static(out.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0),
                                 None, item.data_ptr(), pos.data_ptr(), table.data_ptr(), None, 1, 16, rows, heads, heads,
                                 hd, 1.0, 0, splits, 4, 0, torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert "static scratch" in lib.st_last_error().decode()
    torch.cuda.synchronize()
