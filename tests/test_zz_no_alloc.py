"""The decode attention entry point that allocates nothing (``st_attn_rows_static``), called
through ``ctypes`` as a caller without torch's faces would: two calls in a row, the second with a
smaller input, so that what the first call left in the library's static scratch is still there.
Its output is compared with dense float64 attention over the gathered pages and with the existing
entry point that takes a caller's workspace (``st_attn_rows``); "allocates nothing" is checked on
the device's own count of free memory and by issuing the call while a stream is being captured,
where an allocation is an error."""
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
    """Host tensors of a paged case (pool NaN where no key was written) and their device copies."""
    g = torch.Generator().manual_seed(seed)
    pages_per = -(-ctx_len // page)
    num_pages = rows * pages_per + 3
    perm = torch.randperm(num_pages, generator=g)[:rows * pages_per].to(torch.int32)
    table = perm.view(rows, pages_per).contiguous()
    # each row sits at another position: the splits' chunks differ from row to row
    pos = torch.tensor([ctx_len - 1 - 7 * r for r in range(rows)], dtype=torch.int32)
    kd = torch.randn((rows, heads, ctx_len, hd), generator=g).to(dtype)
    vd = torch.randn((rows, heads, ctx_len, hd), generator=g).to(dtype)
    kd[:, :, 5] *= 4                                       # a far key that row 0's query looks for
    k = torch.full((num_pages, heads, page, hd), float("nan"), dtype=dtype)
    v = torch.full((num_pages, heads, page, hd), float("nan"), dtype=dtype)
    for r in range(rows):
        for pi in range(pages_per):
            a, b = pi * page, min(int(pos[r]) + 1, (pi + 1) * page)
            if b > a:
                k[table[r, pi], :, :b - a] = kd[r, :, a:b]
                v[table[r, pi], :, :b - a] = vd[r, :, a:b]
    q = torch.randn((rows, heads * hd), generator=g).to(dtype)
    q[0] = (kd[0, :, 5] * 0.5).reshape(-1).to(dtype)
    host = dict(q=q, kd=kd, vd=vd, pos=pos)
    dev = tuple(t.to(DEV) for t in (q, k, v, table, torch.arange(rows, dtype=torch.int32), pos))
    return host, dev


def _dense(host, heads, hd, scale):
    """float64 attention of every row over its request's keys [0, position]."""
    out = []
    for r in range(host["q"].shape[0]):
        n = int(host["pos"][r]) + 1
        q = host["q"][r].double().view(heads, hd)
        k, v = host["kd"][r, :, :n].double(), host["vd"][r, :, :n].double()
        p = torch.softmax(torch.einsum("hd,hnd->hn", q, k) * scale, dim=-1)
        out.append(torch.einsum("hn,hnd->hd", p, v).reshape(-1))
    return torch.stack(out)


def _check(got, ref, dtype, what):
    err = (got.double().cpu() - ref).abs()
    tol = 1e-5 + 1e-5 * ref.abs() if dtype == torch.float32 else 1e-3 + 2.0 ** -8 * ref.abs()
    assert torch.isfinite(got.float()).all() and (err <= tol).all(), f"{what}: max err {err.max():.3e}"


def _static_call(lib, got, dev, tail):
    q, k, v, table, item, pos = dev
    return lib.st_attn_rows_static(got.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0),
                                   None, item.data_ptr(), pos.data_ptr(), table.data_ptr(), None, *tail)


def _run(lib, rows, heads, hd, ctx_len, page, splits, dtype, seed, capture=False):
    host, dev = _case(rows, heads, hd, ctx_len, page, dtype, seed)
    q, k, v, table, item, pos = dev
    code = 0 if dtype == torch.float32 else 1
    scale = hd ** -0.5
    ref = _dense(host, heads, hd, scale)
    tail = lambda stream: (table.shape[1], page, rows, heads, heads, hd, scale, 0, splits, 4, code, stream)
    stream = torch.cuda.current_stream().cuda_stream
    # the existing entry point, with a caller's workspace
    want = torch.zeros((rows, heads * hd), dtype=dtype, device=DEV)
    work = torch.empty(rows * heads * splits * (hd + 1), dtype=torch.float32, device=DEV)
    n_o = rows * heads * splits * hd
    rc = lib.st_attn_rows(want.data_ptr(), work.data_ptr(), work.data_ptr() + 4 * n_o, q.data_ptr(), q.stride(0),
                          k.data_ptr(), v.data_ptr(), k.stride(0), None, item.data_ptr(), pos.data_ptr(),
                          table.data_ptr(), None, *tail(stream))
    assert rc == 0, lib.st_last_error().decode()
    _check(want, ref, dtype, "st_attn_rows against dense attention")
    # the entry point under test: the device's free memory does not move across the call
    got = torch.zeros_like(want)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    rc = _static_call(lib, got, dev, tail(stream))
    assert rc == 0, lib.st_last_error().decode()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory moved by {free_before - free_after} bytes"
    _check(got, ref, dtype, "st_attn_rows_static against dense attention")
    assert torch.equal(got, want), f"max difference {(got.float() - want.float()).abs().max().item():.3e}"
    if capture:
        # issued while the stream is being captured, where an allocation (or a lazy code load) would
        # fail the capture; replayed twice with the output cleared in between
        again = torch.zeros_like(want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rc = _static_call(lib, again, dev, tail(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, lib.st_last_error().decode()
        for _ in range(2):
            again.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(again, want)
    return got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_entry_point_equals_dense_attention(dtype):
    lib = _library()
    assert lib.st_attn_rows_static_init() == 0, lib.st_last_error().decode()
    # first a larger call, then a smaller one that finds the first one's partial results in the scratch
    big = _run(lib, rows=6, heads=5, hd=64, ctx_len=900, page=16, splits=8, dtype=dtype, seed=1)
    small = _run(lib, rows=2, heads=3, hd=32, ctx_len=300, page=8, splits=3, dtype=dtype, seed=2, capture=True)
    assert big.shape == (6, 320) and small.shape == (2, 96)
    # no split: the scratch is not touched at all
    _run(lib, rows=3, heads=2, hd=48, ctx_len=70, page=4, splits=1, dtype=dtype, seed=3)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    lib = _library()
    cap = lib.st_attn_rows_static_capacity()
    assert cap == 4 << 20
    rows, heads, hd, splits = 64, 64, 128, 8          # 64*64*8*129 floats = 16.9 MB
    assert rows * heads * splits * (hd + 1) * 4 > cap
    _host, (q, k, v, table, item, pos) = _case(1, 1, 16, 16, 16, torch.float32, 0)
    out = torch.zeros(4, device=DEV)
    rc = lib.st_attn_rows_static(out.data_ptr(), q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0),
                                 None, item.data_ptr(), pos.data_ptr(), table.data_ptr(), None, 1, 16, rows, heads, heads,
                                 hd, 1.0, 0, splits, 4, 0, torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert "static scratch" in lib.st_last_error().decode()
    torch.cuda.synchronize()
