"""Python faces of the HIP kernels: shape/dtype checks on the host, then one
C call on the current torch stream.  Nothing here computes on the CPU and there
is no alternative implementation behind these functions."""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import arena, library
from .arena import empty

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_f = ctypes.c_float
_c_p = ctypes.c_void_p

_configured = False


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODE[dtype]
    except KeyError:
        raise TypeError(f"the kernels store float32 or bfloat16, not {dtype}") from None


def _lib():
    global _configured
    lib = library.load()
    if not _configured:
        lib.st_last_error.restype = ctypes.c_char_p
        lib.st_hash_uniform.restype = ctypes.c_float
        lib.st_hash_uniform.argtypes = [ctypes.c_uint32] * 4
        lib.st_lookup.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_int, _c_int, _c_p]
        lib.st_layernorm.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_f, _c_int, _c_int, _c_p]
        lib.st_kv_write.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_int,
                                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_cast.argtypes = [_c_p, _c_p, _c_i64, _c_int, _c_int, _c_p]
        lib.st_activation_multiply.argtypes = [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_int, _c_int, _c_int,
                                               _c_int, _c_p]
        lib.st_gemm.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                _c_int, _c_int, _c_p, _c_p]
        lib.st_gemm_path_counts.argtypes = [_c_p, _c_int]
        lib.st_gemm_library_rule.argtypes = [_c_int, _c_i64, _c_int]
        lib.st_gemm_can_fuse_norm.argtypes = [_c_int, _c_int, _c_int, _c_int]
        lib.st_gemm_wide_offered.argtypes = [_c_int, _c_int, _c_int, _c_int]
        lib.st_gemm_can_fuse_merge.argtypes = [_c_int] * 7
        lib.st_gemm_library_tuning.argtypes = [_c_int]
        lib.st_attn_rows.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p,
                                     _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_int,
                                     _c_int, _c_int, _c_p]
        lib.st_attn_prefill.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_int,
                                        _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                        _c_f, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_attn_prefill_tile_rows.argtypes = [_c_int] * 6
        lib.st_probe_read.argtypes = [_c_p, _c_i64, _c_p, _c_int, _c_int, _c_p]
        lib.st_probe_empty.argtypes = [_c_p, _c_p]
        lib.st_probe_fill.argtypes = [_c_p, _c_i64, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_probe_mfma.argtypes = [_c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_sample.argtypes = [_c_p, _c_p, _c_int, _c_int, _c_p, _c_p, _c_p, _c_p]
        if torch.cuda.is_available():
            lib.st_gemm_library_init()  # handle and workspace exist before any stream capture
        _configured = True
    return lib


class KernelError(RuntimeError):
    pass


# A KernelTimer (ops/profile.py) while one is active, else None.  Every face below reports its
# call to it: the timer brackets the call with two events on the current stream.
_timer = None


def _timed(name: str, describe):
    """Decorator of a kernel face: with a timer active, the call is bracketed by events and
    recorded under ``name`` with ``describe(*args, **kwargs)`` (a dict of sizes)."""
    def wrap(fn):
        def face(*args, **kwargs):
            if _timer is None:
                return fn(*args, **kwargs)
            begin = _timer.begin()
            out = fn(*args, **kwargs)
            _timer.end(name, describe(*args, **kwargs), begin)
            return out
        face.__name__, face.__doc__ = fn.__name__, fn.__doc__
        return face
    return wrap


# ST_AMD_DEBUG_SYNC=1: wait for the device after every kernel call and surface its errors there
# (the reference's DEBUG build does the same after every launch, src/csrc/util/cuda_utils.h:19-31)
_DEBUG_SYNC = os.environ.get("ST_AMD_DEBUG_SYNC", "") not in ("", "0")


def _check(rc: int) -> None:
    if rc != 0:
        raise KernelError(_lib().st_last_error().decode("utf-8", "replace"))
    if _DEBUG_SYNC and not torch.cuda.is_current_stream_capturing():
        torch.cuda.synchronize()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: Optional[int] = None


def _stream() -> int:
    """The current HIP stream's handle.  Asked for at every kernel call (a caller may have
    switched streams, e.g. to record a step), so by the cheapest route torch offers."""
    global _device_index
    if _raw_stream is None:
        return torch.cuda.current_stream().cuda_stream
    if _device_index is None:
        _device_index = torch.cuda.current_device()     # one GPU per process
    return _raw_stream(_device_index)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, dtype=None, shape=None, contiguous=True) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must be a GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


# ------------------------------------------------------------------------ lookup
def _d_lookup(ids, table, *, add_ids=None, add_table=None, out_f32=None, out_t=None, **kw):
    ref = table if table is not None else add_table
    idx = ids if ids is not None else add_ids
    n, width = idx.shape[0], ref.shape[1]
    tables = (table is not None) + (add_table is not None)
    return {"rows": n, "width": width,
            "bytes": n * width * (tables * ref.element_size() + 4 * (out_f32 is not None) +
                                  ref.element_size() * (out_t is not None))}


@_timed("lookup", _d_lookup)
def lookup(ids: Optional[torch.Tensor], table: Optional[torch.Tensor], *,
           add_ids: Optional[torch.Tensor] = None, add_offset: int = 0,
           add_table: Optional[torch.Tensor] = None, out_f32: Optional[torch.Tensor] = None,
           out_t: Optional[torch.Tensor] = None, accumulate: bool = False) -> None:
    """out[t] = (out[t] if accumulate) + table[ids[t]] + add_table[add_ids[t] + add_offset];
    an index outside its table adds nothing."""
    ref = table if table is not None else add_table
    if ref is None:
        raise KernelError("lookup needs a table")
    width = ref.shape[1]
    idx = ids if ids is not None else add_ids
    n = idx.shape[0]
    if table is not None:
        _need(table, "table", shape=(table.shape[0], width))
        _need(ids, "ids", torch.int32, (n,))
    if add_table is not None:
        _need(add_table, "add_table", ref.dtype, (add_table.shape[0], width))
        _need(add_ids, "add_ids", torch.int32, (n,))
    if out_f32 is not None:
        _need(out_f32, "out_f32", torch.float32, (n, width))
    if out_t is not None:
        _need(out_t, "out_t", ref.dtype, (n, width))
    _check(_lib().st_lookup(_ptr(out_f32), _ptr(out_t), _ptr(ids), _ptr(table), _ptr(add_ids),
                            int(add_offset), _ptr(add_table),
                            table.shape[0] if table is not None else 0,
                            add_table.shape[0] if add_table is not None else 0, n, width, int(accumulate),
                            dtype_code(ref.dtype), _stream()))


# --------------------------------------------------------------------- LayerNorm
def _d_layernorm(x, gamma, beta, eps, *, rows=None, out_t=None, out_f32=None, center=True):
    n = rows.shape[0] if rows is not None else x.shape[0]
    w = x.shape[-1]
    return {"rows": n, "width": w,
            "bytes": n * w * (4 + (out_t.element_size() if out_t is not None else 0) + 4 * (out_f32 is not None))}


@_timed("layernorm", _d_layernorm)
def layernorm(x: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
              eps: float, *, rows: Optional[torch.Tensor] = None,
              out_t: Optional[torch.Tensor] = None, out_f32: Optional[torch.Tensor] = None,
              center: bool = True) -> None:
    """LayerNorm over the last dimension of float rows; row r reads x[rows[r]] if given.
    ``center=False``: no mean is taken off (root-mean-square norm)."""
    _need(x, "x", torch.float32)
    width = x.shape[-1]
    n = rows.shape[0] if rows is not None else x.shape[0]
    if rows is not None:
        _need(rows, "rows", torch.int32, (n,))
    for name, v in (("gamma", gamma), ("beta", beta)):
        if v is not None:
            _need(v, name, torch.float32, (width,))
    if out_t is None and out_f32 is None:
        raise KernelError("layernorm needs a destination")
    code = F32
    if out_t is not None:
        _need(out_t, "out_t", None, (n, width))
        code = dtype_code(out_t.dtype)
    if out_f32 is not None:
        _need(out_f32, "out_f32", torch.float32, (n, width))
        if rows is not None and out_f32.data_ptr() == x.data_ptr():
            raise KernelError("layernorm: a gathered LayerNorm cannot write over its input")
    _check(_lib().st_layernorm(_ptr(out_t), _ptr(out_f32), _ptr(x), _ptr(rows), _ptr(gamma), _ptr(beta),
                               n, width, float(eps), int(bool(center)), code, _stream()))


# -------------------------------------------------------------------------- GEMM
class _GemmExtras(ctypes.Structure):
    """Mirror of StGemmExtras (csrc/gemm_extras.h)."""
    _fields_ = [("ln_x", _c_p), ("ln_gamma", _c_p), ("ln_beta", _c_p), ("ln_eps", _c_f), ("ln_no_center", _c_int),
                ("k_cache", _c_p), ("v_cache", _c_p), ("page_stride", _c_i64), ("token_item", _c_p),
                ("positions", _c_p), ("block_table", _c_p), ("max_pages", _c_int), ("page_size", _c_int),
                ("q_size", _c_int), ("kv_size", _c_int), ("head_dim", _c_int), ("_pad1", _c_int),
                ("mg_o", _c_p), ("mg_lse", _c_p), ("mg_splits", _c_int), ("mg_heads", _c_int),
                ("mg_head_dim", _c_int), ("_pad2", _c_int),
                ("ln_rows", _c_p), ("best_ids", _c_p), ("best_val", _c_p), ("best_idx", _c_p)]


class KvScatter:
    """Where a fused QKV product also stores the new keys and values: the layer's cache views,
    the step's row -> (item, position) arrays and the block table."""

    def __init__(self, k_cache: torch.Tensor, v_cache: torch.Tensor, token_item: torch.Tensor,
                 positions: torch.Tensor, block_table: torch.Tensor, q_size: int):
        self.k_cache, self.v_cache = k_cache, v_cache
        self.token_item, self.positions, self.block_table = token_item, positions, block_table
        self.q_size = q_size


class NormInput:
    """The input of a product given as (float rows, gain, bias, eps): the product normalises
    the rows itself.  With ``rows`` (int32 [M] on the device) row m of the input is the norm of
    ``x32[rows[m]]`` (where ``wide_offered``).  ``center=False``: the root-mean-square norm (no
    mean is taken off)."""

    def __init__(self, x32: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
                 eps: float, rows: Optional[torch.Tensor] = None, center: bool = True):
        self.x32, self.gamma, self.beta, self.eps, self.rows, self.center = x32, gamma, beta, eps, rows, center


class SplitAttention:
    """The input of a product given as an attention output still split over the keys:
    ``part_o`` [M, heads, splits, head_dim] normalised partial results and ``part_lse``
    [M, heads, splits] their log-sum-exps (``attention_rows(..., merge=False)``).  The product
    merges the splits itself."""

    def __init__(self, part_o: torch.Tensor, part_lse: torch.Tensor):
        self.part_o, self.part_lse = part_o, part_lse


def can_fuse_merge(M: int, N: int, K: int, splits: int, heads: int, head_dim: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm`` takes a ``SplitAttention`` for this shape."""
    return bool(_lib().st_gemm_can_fuse_merge(M, N, K, splits, heads, head_dim, dtype_code(dtype)))


class tuned_products:
    """``with tuned_products():`` the vendor library's candidate kernels are timed for every
    product shape issued inside (outside stream capture) and the fastest kept for that shape from
    then on.  For the preparation of steps that are replayed many times; ~20 ms a shape."""

    def __enter__(self):
        _lib().st_gemm_library_tuning(1)
        return self

    def __exit__(self, *exc):
        torch.cuda.synchronize()
        _lib().st_gemm_library_tuning(0)
        return False


GEMM_PATHS = ("library", "generic_f32", "generic_bf16", "resident", "resident_norm", "resident_merge",
              "resident_staged", "skinny16", "skinny32", "skinny64", "tiled_mfma", "wide")


def gemm_path_counts(reset: bool = False) -> dict:
    """Calls of ``gemm`` per kernel family since the last reset: which dispatch branches ran."""
    n = len(GEMM_PATHS)
    buf = (ctypes.c_uint64 * n)()
    got = _lib().st_gemm_path_counts(buf, int(reset))
    if got != n:
        raise KernelError(f"the library counts {got} product paths, this module names {n}")
    return {name: int(buf[i]) for i, name in enumerate(GEMM_PATHS)}


def gemm_library_rule(min_rows: int = -1, min_weights: int = -1, min_depth: int = -1) -> None:
    """Change when bfloat16 products go to the vendor library (for measurements): from ``min_rows``
    rows on, and below that for matrices of ``min_weights`` elements and ``min_depth`` depth.  -1
    leaves a setting, -2 puts its fitted default back (``gemm_library_rule(-2, -2, -2)``: all of
    them).  A step recorded before the change keeps its kernels."""
    _lib().st_gemm_library_rule(int(min_rows), int(min_weights), int(min_depth))


def gemm_wide_workgroups(mode: int = 3) -> None:
    """Which workgroup shapes a product with the norm prologue may take (for measurements and
    tests): 0 only 16 features a workgroup, 1 also 24 with 8 waves, 3 (the default) 24 or 32 with 16 waves,
    7 the same with 32 tried first; a negative number puts the default back."""
    _lib().st_gemm_wide_workgroups(int(mode))


def can_fuse_norm(M: int, N: int, K: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm`` takes a ``NormInput`` (without a row index) for this shape."""
    return bool(_lib().st_gemm_can_fuse_norm(M, N, K, dtype_code(dtype)))


def wide_offered(M: int, N: int, K: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm(..., out_f32=True)`` runs this plain product in the persistent kernel for few
    rows and a very wide matrix (an output head): the kernel that takes a ``NormInput`` with a row
    index and fills ``best``."""
    return bool(_lib().st_gemm_wide_offered(M, N, K, dtype_code(dtype)))


# functions of the products' epilogues and of ``activation_multiply``, by the C interface's number
# (csrc/activation.h; the names config files use for them)
ACTIVATIONS = {"none": 0, "relu": 1, "silu": 2, "gelu_tanh": 3, "gelu_new": 3}


def _d_gemm(x, w, *, bias=None, residual=None, activation="none", out=None, out_f32=False, algo=0,
            kv_scatter=None, best=None):
    N, K = w.shape
    fused = []
    if isinstance(x, NormInput):
        M = x.rows.shape[0] if x.rows is not None else x.x32.shape[0]
        in_bytes = M * K * 4
        fused.append("norm")
    elif isinstance(x, SplitAttention):
        M, in_bytes = x.part_o.shape[0], x.part_o.numel() * 4
        fused.append("merge")
    else:
        M, in_bytes = x.shape[0], x.shape[0] * K * w.element_size()
    if kv_scatter is not None:
        fused.append("kv")
    if best is not None:
        fused.append("best")
    if activation != "none":
        fused.append(activation)
    if residual is not None:
        fused.append("residual")
    out_elem = 4 if (out_f32 or w.dtype == torch.float32) else w.element_size()
    return {"M": M, "N": N, "K": K, "fused": "+".join(fused), "dtype": str(w.dtype).replace("torch.", ""),
            "bytes": N * K * w.element_size() + in_bytes + M * N * (out_elem + 4 * (residual is not None)),
            "flops": 2 * M * N * K}


@_timed("gemm", _d_gemm)
def gemm(x, w: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
         residual: Optional[torch.Tensor] = None, activation: str = "none",
         out: Optional[torch.Tensor] = None, out_f32: bool = False, algo: int = 0,
         kv_scatter: Optional[KvScatter] = None, best: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M,N] = act(x[M,K] @ w[N,K]^T (+bias)) (+residual); float accumulation.  ``activation``
    is one of ``ACTIVATIONS``.

    ``x`` is a tensor of w's dtype, a ``NormInput`` (where ``can_fuse_norm``) or a
    ``SplitAttention`` (where ``can_fuse_merge``).  With
    ``kv_scatter`` the output features after the first q_size are also written into the
    cache pages (w then is a fused q|k|v matrix).  ``best`` (int32 [M], where ``wide_offered``):
    receives the index of every row's largest output, the lowest on ties."""
    N, K = w.shape
    _need(w, "w", None, (N, K))
    code = dtype_code(w.dtype)
    if activation not in ACTIVATIONS:
        raise KernelError(f"the products' epilogues know {sorted(ACTIVATIONS)}, not {activation!r}")
    ex = None
    keep = []
    if isinstance(x, NormInput):
        M = x.x32.shape[0]
        _need(x.x32, "norm input", torch.float32, (M, K))
        for name, v in (("gamma", x.gamma), ("beta", x.beta)):
            if v is not None:
                _need(v, name, torch.float32, (K,))
        ex = _GemmExtras()
        ex.ln_x, ex.ln_gamma, ex.ln_beta, ex.ln_eps = _ptr(x.x32), _ptr(x.gamma), _ptr(x.beta), float(x.eps)
        ex.ln_no_center = 0 if x.center else 1
        if x.rows is not None:
            M = x.rows.shape[0]
            _need(x.rows, "row index", torch.int32, (M,))
            ex.ln_rows = _ptr(x.rows)
        x_ptr, device = None, x.x32.device
    elif isinstance(x, SplitAttention):
        M, heads, splits, hd = x.part_o.shape
        _need(x.part_o, "partial outputs", torch.float32, (M, heads, splits, hd))
        _need(x.part_lse, "log-sum-exps", torch.float32, (M, heads, splits))
        if heads * hd != K:
            raise KernelError(f"{heads} heads of {hd} do not make the product's {K} inputs")
        ex = _GemmExtras()
        ex.mg_o, ex.mg_lse = _ptr(x.part_o), _ptr(x.part_lse)
        ex.mg_splits, ex.mg_heads, ex.mg_head_dim = splits, heads, hd
        x_ptr, device = None, x.part_o.device
    else:
        M = x.shape[0]
        _need(x, "x", w.dtype, (M, K))
        x_ptr, device = x.data_ptr(), x.device
    odt = torch.float32 if (out_f32 or code == F32) else w.dtype
    if out is None:
        out = empty((M, N), odt, device)
    _need(out, "out", odt, (M, N))
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    if residual is not None:
        _need(residual, "residual", torch.float32, (M, N))
    if kv_scatter is not None:
        ks = kv_scatter
        num_pages, nkv, ps, hd = _check_cache(ks.k_cache, ks.v_cache, out)
        _need(ks.token_item, "token_item", torch.int32, (M,))
        _need(ks.positions, "positions", torch.int32, (M,))
        _need(ks.block_table, "block_table", torch.int32)
        if ex is None:
            ex = _GemmExtras()
        ex.k_cache, ex.v_cache, ex.page_stride = _ptr(ks.k_cache), _ptr(ks.v_cache), ks.k_cache.stride(0)
        ex.token_item, ex.positions, ex.block_table = _ptr(ks.token_item), _ptr(ks.positions), _ptr(ks.block_table)
        ex.max_pages, ex.page_size = ks.block_table.shape[1], ps
        ex.q_size, ex.kv_size, ex.head_dim = ks.q_size, nkv * hd, hd
    if best is not None:
        _need(best, "best", torch.int32, (M,))
        n_scratch = 16 * _lib().st_gemm_wide_groups()
        if ex is None:
            ex = _GemmExtras()
        val = empty((n_scratch,), torch.float32, device)
        idx = empty((n_scratch,), torch.int32, device)
        keep += [val, idx]
        ex.best_ids, ex.best_val, ex.best_idx = _ptr(best), _ptr(val), _ptr(idx)
    _check(_lib().st_gemm(_ptr(out), x_ptr, _ptr(w), _ptr(bias), _ptr(residual), M, N, K, ACTIVATIONS[activation],
                          code, int(odt == torch.float32), int(algo),
                          ctypes.byref(ex) if ex is not None else None, _stream()))
    return out


# ---------------------------------------------------------------------- KV write
def _d_kv_write(k_cache, v_cache, k_src, v_src, *a, **kw):
    return {"rows": k_src.shape[0], "width": k_src.shape[1], "bytes": 4 * k_src.numel() * k_src.element_size()}


@_timed("kv_write", _d_kv_write)
def kv_write(k_cache: torch.Tensor, v_cache: torch.Tensor, k_src: torch.Tensor, v_src: torch.Tensor,
             token_item: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
             page_size: int) -> None:
    """Copy each token's key/value heads into its page.

    k_cache/v_cache: [num_pages, num_kv_heads, page_size, head_dim] views (the page
    dimension may be strided).  k_src/v_src: [T, num_kv_heads*head_dim] views with a
    common row stride (e.g. column slices of the fused QKV output)."""
    num_pages, nkv, ps, hd = k_cache.shape
    if ps != page_size:
        raise KernelError(f"cache pages hold {ps} tokens, the step says {page_size}")
    T = k_src.shape[0]
    for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        _need(c, name, k_cache.dtype, (num_pages, nkv, ps, hd), contiguous=False)
        if c.stride()[1:] != (ps * hd, hd, 1):
            raise KernelError(f"{name}: a page must be contiguous")
    if k_cache.stride(0) != v_cache.stride(0):
        raise KernelError("k_cache and v_cache must share the page stride")
    for name, s in (("k_src", k_src), ("v_src", v_src)):
        _need(s, name, k_cache.dtype, (T, nkv * hd), contiguous=False)
        if s.stride(1) != 1 or s.stride(0) != k_src.stride(0):
            raise KernelError(f"{name}: rows must be dense with a common stride")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    _check(_lib().st_kv_write(_ptr(k_cache), _ptr(v_cache), k_cache.stride(0), _ptr(k_src), _ptr(v_src),
                              k_src.stride(0), _ptr(token_item), _ptr(positions), _ptr(block_table),
                              block_table.shape[1], ps, T, nkv, hd, dtype_code(k_cache.dtype), _stream()))


# --------------------------------------------------------------------- attention
def _check_cache(k_cache, v_cache, q):
    num_pages, nkv, ps, hd = k_cache.shape
    for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        _need(c, name, q.dtype, (num_pages, nkv, ps, hd), contiguous=False)
        if c.stride()[1:] != (ps * hd, hd, 1):
            raise KernelError(f"{name}: a page must be contiguous")
    if k_cache.stride(0) != v_cache.stride(0):
        raise KernelError("k_cache and v_cache must share the page stride")
    return num_pages, nkv, ps, hd


def _d_attention_rows(q, k_cache, v_cache, token_item, positions, block_table, num_q_heads, scale, *,
                      num_splits=1, row_ids=None, merge=True, **kw):
    # how many keys the rows read is on the device only: the caller of the timer knows its workload
    rows = row_ids.shape[0] if row_ids is not None else q.shape[0]
    return {"rows": rows, "heads": num_q_heads, "kv_heads": k_cache.shape[1], "head_dim": k_cache.shape[3],
            "splits": num_splits, "merged": bool(merge), "elem": k_cache.element_size()}


def _d_attention_prefill(q, k_cache, v_cache, tile_item, *a, **kw):
    return {"rows": q.shape[0], "tiles": tile_item.shape[0], "heads": q.shape[1] // k_cache.shape[3],
            "kv_heads": k_cache.shape[1], "head_dim": k_cache.shape[3], "elem": k_cache.element_size()}


@_timed("attention_rows", _d_attention_rows)
def attention_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   token_item: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                   num_q_heads: int, scale: float, *, window: int = 0, num_splits: int = 1,
                   num_waves: int = 4, row_ids: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   workspace: Optional[torch.Tensor] = None, merge: bool = True,
                   head_slopes: Optional[torch.Tensor] = None):
    """Each query row attends over its request's cached keys [lo, position].

    q: [T, num_q_heads*head_dim] view (row stride free).  Returns [T, num_q_heads*head_dim];
    with ``row_ids`` only those batch rows are computed (and written).  ``merge=False`` (with
    num_splits > 1, all rows): the splits are left unmerged and returned as a
    ``SplitAttention`` for a product to merge.  ``head_slopes`` (float32 [num_q_heads]): a head's
    scaled scores get slope * (key position - query position) added."""
    num_pages, nkv, ps, hd = _check_cache(k_cache, v_cache, q)
    T = q.shape[0]
    if head_slopes is not None:
        _need(head_slopes, "head_slopes", torch.float32, (num_q_heads,))
    _need(q, "q", None, (T, num_q_heads * hd), contiguous=False)
    if q.stride(1) != 1:
        raise KernelError("q rows must be dense")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    if not merge and (num_splits < 2 or row_ids is not None or T > 65535 or out is not None):
        raise KernelError("unmerged attention output needs splits, all rows and no destination")
    if merge:
        if out is None:
            out = empty((T, num_q_heads * hd), q.dtype, q.device)
        _need(out, "out", q.dtype, (T, num_q_heads * hd))
    n_rows = T
    if row_ids is not None:
        n_rows = row_ids.shape[0]
        _need(row_ids, "row_ids", torch.int32, (n_rows,))
    part_o = part_lse = None
    if num_splits > 1:
        n_o = min(n_rows, 65535) * num_q_heads * num_splits * hd
        n_l = min(n_rows, 65535) * num_q_heads * num_splits
        if workspace is None:
            workspace = empty((n_o + n_l,), torch.float32, q.device)
        _need(workspace, "workspace", torch.float32)
        if workspace.numel() < n_o + n_l:
            raise KernelError("attention workspace is too small")
        part_o, part_lse = workspace[:n_o], workspace[n_o:n_o + n_l]
    step = 65535
    for r0 in range(0, n_rows, step):
        r1 = min(n_rows, r0 + step)
        if row_ids is not None:
            o_ptr, q_ptr, ti_ptr, po_ptr = out.data_ptr(), q.data_ptr(), token_item.data_ptr(), positions.data_ptr()
            rid_ptr = row_ids[r0:r1].data_ptr()
        else:
            o_ptr, q_ptr = (out[r0:r1].data_ptr() if merge else None), q[r0:r1].data_ptr()
            ti_ptr, po_ptr = token_item[r0:r1].data_ptr(), positions[r0:r1].data_ptr()
            rid_ptr = None
        _check(_lib().st_attn_rows(
            o_ptr, _ptr(part_o), _ptr(part_lse), q_ptr, q.stride(0),
            _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), rid_ptr, ti_ptr, po_ptr,
            _ptr(block_table), _ptr(head_slopes), block_table.shape[1], ps, r1 - r0,
            num_q_heads, nkv, hd, float(scale), int(window), int(num_splits), int(num_waves),
            dtype_code(q.dtype), _stream()))
    if not merge:
        return SplitAttention(part_o.view(T, num_q_heads, num_splits, hd), part_lse.view(T, num_q_heads, num_splits))
    return out


@_timed("attention_prefill", _d_attention_prefill)
def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      tile_item: torch.Tensor, tile_q0: torch.Tensor,
                      item_tok_off: torch.Tensor, item_start: torch.Tensor, item_len: torch.Tensor,
                      block_table: torch.Tensor, num_q_heads: int, scale: float, *,
                      window: int = 0, out: Optional[torch.Tensor] = None, key_split: int = 0,
                      tile_rows: int = 64, algo: int = 0,
                      head_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Tiles of consecutive query rows of prompt portions attend over the cache.

    Tile i covers rows [tile_q0[i], tile_q0[i]+tile_rows) of item tile_item[i]; row r of an
    item sits at batch row item_tok_off[item]+r and at position item_start[item]+r.
    ``key_split``: groups of waves that share a tile's key blocks (1, 2 or 4; 0: chosen from
    the number of tiles).  ``tile_rows``: 64, or 128 where ``prefill_tile_rows`` says so.
    ``algo``: 0 chosen by the library, 1 the kernel that stages key blocks through registers,
    2 the kernel that loads them straight into LDS (it takes no ``head_slopes``, which are as in
    ``attention_rows``)."""
    num_pages, nkv, ps, hd = _check_cache(k_cache, v_cache, q)
    T = q.shape[0]
    _need(q, "q", None, (T, num_q_heads * hd), contiguous=False)
    if q.stride(1) != 1:
        raise KernelError("q rows must be dense")
    nt = tile_item.shape[0]
    _need(tile_item, "tile_item", torch.int32, (nt,))
    _need(tile_q0, "tile_q0", torch.int32, (nt,))
    for name, v in (("item_tok_off", item_tok_off), ("item_start", item_start), ("item_len", item_len)):
        _need(v, name, torch.int32)
    _need(block_table, "block_table", torch.int32)
    if out is None:
        out = empty((T, num_q_heads * hd), q.dtype, q.device)
    _need(out, "out", q.dtype, (T, num_q_heads * hd))
    if head_slopes is not None:
        _need(head_slopes, "head_slopes", torch.float32, (num_q_heads,))
    _check(_lib().st_attn_prefill(
        _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0),
        _ptr(tile_item), _ptr(tile_q0), nt, _ptr(item_tok_off), _ptr(item_start), _ptr(item_len),
        _ptr(block_table), _ptr(head_slopes), block_table.shape[1], ps, num_q_heads, nkv, hd, float(scale), int(window),
        int(key_split), int(tile_rows), int(algo), dtype_code(q.dtype), _stream()))
    return out


PREFILL_TILE = 64   # query rows per tile of attention_prefill unless prefill_tile_rows says 128


def prefill_tile_rows(head_dim: int, page_size: int, max_pages: int, num_q_heads: int, num_rows: int,
                      dtype: torch.dtype) -> int:
    """Rows per tile (64 or 128) that ``attention_prefill`` serves best when ``num_rows`` query rows
    sit in items long enough for tiles."""
    return int(_lib().st_attn_prefill_tile_rows(head_dim, page_size, max_pages, num_q_heads, num_rows,
                                                dtype_code(dtype)))


def prefill_available() -> bool:
    """Whether the library holds the tiled (matrix-core) prompt attention kernel."""
    return bool(_lib().st_has_attn_prefill())


# ---------------------------------------------------------------------- sampling
def _d_sample(logits, **kw):
    return {"rows": logits.shape[0], "width": logits.shape[1], "bytes": logits.numel() * 4}


@_timed("sample", _d_sample)
def sample(logits: torch.Tensor, *, temperature: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, draws: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token ids [R] (int32) from float logits [R,V]; rows with temperature <= 0 (or no
    temperature tensor) take the argmax, lowest index on ties."""
    R, V = logits.shape
    _need(logits, "logits", torch.float32, (R, V))
    if temperature is not None:
        _need(temperature, "temperature", torch.float32, (R,))
        _need(seeds, "seeds", torch.int32, (R, 2))
        _need(draws, "draws", torch.int32, (R,))
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out, "out", torch.int32, (R,))
    _check(_lib().st_sample(_ptr(out), _ptr(logits), R, V, _ptr(temperature), _ptr(seeds), _ptr(draws),
                            _stream()))
    return out


def _d_cast(x, dtype, out=None):
    return {"rows": x.shape[0] if x.dim() else 1, "width": x.numel() // max(1, x.shape[0] if x.dim() else 1),
            "bytes": x.numel() * (x.element_size() + torch.empty((), dtype=dtype).element_size())}


@_timed("cast", _d_cast)
def cast(x: torch.Tensor, dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _need(x, "x")
    if out is None:
        out = empty(tuple(x.shape), dtype, x.device)
    _need(out, "out", dtype, x.shape)
    _check(_lib().st_cast(_ptr(out), _ptr(x), x.numel(), dtype_code(x.dtype), dtype_code(dtype), _stream()))
    return out


def _d_activation_multiply(a, b=None, activation="none", out=None):
    return {"rows": a.shape[0], "width": a.shape[1], "fused": activation,
            "bytes": a.numel() * a.element_size() * (2 + (b is not None))}


@_timed("activation_multiply", _d_activation_multiply)
def activation_multiply(a: torch.Tensor, b: Optional[torch.Tensor] = None, activation: str = "none",
                        out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(a) * b elementwise over [rows, width] (``b`` None: out = act(a)), float arithmetic.
    ``a``, ``b`` and ``out`` may be column slices of wider tensors (dense rows, any row stride), e.g.
    the two halves of one product's output; ``out`` may be ``a``."""
    if activation not in ACTIVATIONS:
        raise KernelError(f"the kernels know the activations {sorted(ACTIVATIONS)}, not {activation!r}")
    if a.dim() != 2:
        raise KernelError("activation_multiply takes [rows, width] tensors")
    rows, width = a.shape
    code = dtype_code(a.dtype)
    if out is None:
        out = empty((rows, width), a.dtype, a.device)
    for name, t in (("a", a), ("b", b), ("out", out)):
        if t is None:
            continue
        _need(t, name, a.dtype, (rows, width), contiguous=False)
        if t.stride(1) != 1 or (rows > 1 and t.stride(0) < width):
            raise KernelError(f"{name}: rows must be dense and must not overlap")
    _check(_lib().st_activation_multiply(_ptr(out), max(out.stride(0), width), _ptr(a), max(a.stride(0), width),
                                         _ptr(b), max(b.stride(0), width) if b is not None else 0, rows, width,
                                         ACTIVATIONS[activation], code, _stream()))
    return out


def activation(x: torch.Tensor, kind: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(x) elementwise."""
    return activation_multiply(x, None, kind, out)


def multiply(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = a * b elementwise."""
    return activation_multiply(a, b, "none", out)


def probe_read(src: torch.Tensor, sink: torch.Tensor, workgroups: int, pattern: int = 0) -> None:
    """Measurement aid: a plain read of all of ``src`` by ``workgroups`` workgroups (``sink``: int32,
    one word a workgroup).  ``pattern``: 0 / 1 the grid strides over the buffer with 4 / 8 loads in
    flight per thread, 2 / 3 tiles of 8 / 16 KB dealt round-robin to the workgroups."""
    _need(src, "src")
    _need(sink, "sink", torch.int32)
    nbytes = src.numel() * src.element_size()
    if nbytes % 16 or sink.numel() < workgroups:
        raise KernelError("probe_read: the source must be a multiple of 16 bytes, the sink one word a workgroup")
    _check(_lib().st_probe_read(_ptr(src), nbytes, _ptr(sink), int(workgroups), int(pattern), _stream()))


def probe_empty(sink: torch.Tensor) -> None:
    """Measurement aid: a kernel of one workgroup that does one store."""
    _need(sink, "sink", torch.int32)
    _check(_lib().st_probe_empty(_ptr(sink), _stream()))


def probe_fill(src: torch.Tensor, region: int, sink: torch.Tensor, workgroups: int, turns: int, to_lds: bool) -> None:
    """Measurement aid: ``workgroups`` workgroups each go ``turns`` times 32 KB round their own
    ``region`` bytes of ``src``, by direct loads into LDS or by loads into registers."""
    _need(src, "src")
    _need(sink, "sink", torch.int32)
    if src.numel() * src.element_size() < workgroups * region or sink.numel() < workgroups:
        raise KernelError("probe_fill: the source holds a region a workgroup, the sink one word a workgroup")
    _check(_lib().st_probe_fill(_ptr(src), int(region), _ptr(sink), int(workgroups), int(turns), int(bool(to_lds)),
                                _stream()))


def probe_mfma(sink: torch.Tensor, workgroups: int, rounds: int, wide: bool) -> None:
    """Measurement aid: ``workgroups`` workgroups of four waves issue 16 * ``rounds`` independent
    matrix-core products a wave (bfloat16, the 32x32x16 form if ``wide``, else 16x16x32)."""
    _need(sink, "sink", torch.int32)
    if sink.numel() < workgroups:
        raise KernelError("probe_mfma: the sink holds one word a workgroup")
    _check(_lib().st_probe_mfma(_ptr(sink), int(workgroups), int(rounds), int(bool(wide)), _stream()))


def hash_uniform(seed_lo: int, seed_hi: int, draw: int, v: int) -> float:
    """Host copy of the sampler's counter-based uniform (for plain references)."""
    return float(_lib().st_hash_uniform(seed_lo & 0xffffffff, seed_hi & 0xffffffff,
                                        draw & 0xffffffff, v & 0xffffffff))
