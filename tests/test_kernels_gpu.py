"""Each kernel alone against a plain float64 reference, at other sizes than the engine's."""
import math

import numpy as np
import pytest
import torch

import plain_opt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def K():
    from swifttransformer_amd.ops import kernels
    return kernels


def close(got, ref, dtype, what, scale=None):
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{what}: {got.shape} vs {ref.shape}"
    if dtype == torch.float32:
        tol = 1e-5 + 1e-5 * ref.abs()
    else:   # one rounding of the result to bfloat16 (2^-9 relative) plus input effects given by `scale`
        tol = (scale if scale is not None else 0.0) + 2.0 ** -8 * ref.abs() + 1e-6
    err = (got - ref).abs()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    assert (err <= tol).all(), f"{what}: max err {err.max():.3e} at {torch.argmax(err - tol)}"


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lookup(dtype):
    k = K()
    table, ptab = rnd(50, 72, dtype=dtype, seed=1), rnd(30, 72, dtype=dtype, seed=2)
    ids = torch.tensor([3, 49, 0, 7, 7], dtype=torch.int32)
    pos = torch.tensor([0, 1, 27, 5, 6], dtype=torch.int32)
    ref = table.double()[ids.long()] + ptab.double()[pos.long() + 2]
    out32 = torch.empty(5, 72, device=DEV)
    outt = torch.empty(5, 72, device=DEV, dtype=dtype)
    k.lookup(ids.to(DEV), table.to(DEV), add_ids=pos.to(DEV), add_offset=2, add_table=ptab.to(DEV),
             out_f32=out32, out_t=outt)
    close(out32, ref, torch.float32, "lookup f32 out")
    close(outt, ref, dtype, "lookup t out")
    k.lookup(None, None, add_ids=pos.to(DEV), add_offset=0, add_table=ptab.to(DEV), out_f32=out32,
             accumulate=True)
    close(out32, ref + ptab.double()[pos.long()], torch.float32, "lookup accumulate")
    # an index outside its table (the padding rows of a recorded step carry position -1, which an
    # offset of 0 leaves negative) adds nothing and reads nothing
    ids2 = torch.tensor([3, -1, 50, 7, 0], dtype=torch.int32)
    pos2 = torch.tensor([-1, 1, 29, 30, -5], dtype=torch.int32)
    k.lookup(ids2.to(DEV), table.to(DEV), add_ids=pos2.to(DEV), add_offset=0, add_table=ptab.to(DEV), out_f32=out32)
    ref2 = torch.zeros(5, 72, dtype=torch.float64)
    for r in range(5):
        if 0 <= ids2[r] < 50:
            ref2[r] += table.double()[ids2[r]]
        if 0 <= pos2[r] < 30:
            ref2[r] += ptab.double()[pos2[r]]
    close(out32, ref2, torch.float32, "lookup with indices outside the tables")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [6, 8, 100, 1000, 8192, 10000])
def test_layernorm(dtype, width):
    k = K()
    # sizes after the reference's own test (259 x 8192, eps 1e-4: src/unittest/kernel/layernorm.cc:24-52)
    x = rnd(37, width, seed=3) * 3 + 5          # a large mean would break E[x^2]-E[x]^2 in float
    g, b = torch.rand(width), torch.rand(width)
    ref = torch.nn.functional.layer_norm(x.double(), (width,), g.double(), b.double(), 1e-4)
    out_t = torch.empty(37, width, device=DEV, dtype=dtype)
    out32 = torch.empty(37, width, device=DEV)
    k.layernorm(x.to(DEV), g.to(DEV), b.to(DEV), 1e-4, out_t=out_t, out_f32=out32)
    close(out32, ref, torch.float32, "layernorm f32")
    close(out_t, ref, dtype, "layernorm t")
    rows = torch.tensor([5, 0, 36, 5], dtype=torch.int32)
    out = torch.empty(4, width, device=DEV, dtype=dtype)
    k.layernorm(x.to(DEV), None, None, 1e-4, rows=rows.to(DEV), out_t=out)
    close(out, torch.nn.functional.layer_norm(x.double()[rows.long()], (width,), None, None, 1e-4), dtype,
          "layernorm gathered, no affine")
    # without the mean taken off: the root-mean-square norm (the mean of 5 makes the two forms differ widely)
    xd = x.double()
    rms = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-4) * g.double()
    k.layernorm(x.to(DEV), g.to(DEV), None, 1e-4, out_t=out_t, out_f32=out32, center=False)
    close(out32, rms, torch.float32, "root-mean-square norm f32")
    close(out_t, rms, dtype, "root-mean-square norm t")
    assert (rms - ref).abs().max() > 0.5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K_", [(61, 29, 124), (1, 1000, 64), (8, 96, 320), (130, 200, 50), (257, 65, 17),
                                    (64, 3072, 768), (2, 50272 // 16, 96)])
def test_gemm_generic_and_best(dtype, M, N, K_):
    k = K()
    x, w = rnd(M, K_, dtype=dtype, seed=4), rnd(N, K_, dtype=dtype, seed=5, scale=0.1)
    bias, res = rnd(N, seed=6), rnd(M, N, seed=7)
    base = x.double() @ w.double().T
    # rounding of the stored result only; products of exactly representable inputs are summed in float
    # 1: generic kernel, 0: whatever the engine would pick, 3: the hand-written matrix-core kernels
    for algo in (1, 0, 3):
        out = k.gemm(x.to(DEV), w.to(DEV), algo=algo)
        close(out, base, dtype, f"gemm algo {algo} plain")
        out = k.gemm(x.to(DEV), w.to(DEV), bias=bias.to(DEV), activation="relu", algo=algo)
        close(out, torch.relu(base + bias.double()), dtype, f"gemm algo {algo} bias relu")
        out = k.gemm(x.to(DEV), w.to(DEV), bias=bias.to(DEV), residual=res.to(DEV), out_f32=True, algo=algo)
        assert out.dtype == torch.float32
        close(out, base + bias.double() + res.double(), torch.float32, f"gemm algo {algo} bias residual f32")


def _plain_activation(kind, v):
    """float64 forms of the functions (the reference's src/csrc/kernel/activations.cuh:8-24)."""
    if kind == "relu":
        return torch.relu(v)
    if kind == "silu":
        return v / (1 + torch.exp(-v))
    if kind == "gelu_tanh":
        return 0.5 * v * (1 + torch.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    return v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["silu", "gelu_tanh", "relu"])
@pytest.mark.parametrize("M,N,K_", [(5, 96, 320), (40, 200, 72), (9, 2048, 512), (150, 129, 50)])
def test_gemm_activation_epilogues(dtype, kind, M, N, K_):
    """Every product path applies the same function between bias and residual: the plain kernel
    (1), the engine's choice (0: resident kernel at few rows, the library's product followed by
    the elementwise kernel from 13 rows and in float32), the matrix-core kernels (3)."""
    k = K()
    x, w = rnd(M, K_, dtype=dtype, seed=24), rnd(N, K_, dtype=dtype, seed=25, scale=0.2)
    bias, res = rnd(N, seed=26), rnd(M, N, seed=27)
    pre = x.double() @ w.double().T + bias.double()
    ref = _plain_activation(kind, pre)
    for algo in (1, 0, 3):
        got = k.gemm(x.to(DEV), w.to(DEV), bias=bias.to(DEV), activation=kind, algo=algo)
        # (a stored bfloat16 result may have been rounded once before the function and once after)
        close(got, ref, dtype, f"gemm {kind} algo {algo}", scale=2.0 ** -8 * pre.abs() if dtype == torch.bfloat16 else None)
        got = k.gemm(x.to(DEV), w.to(DEV), bias=bias.to(DEV), activation=kind, residual=res.to(DEV), out_f32=True,
                     algo=algo)
        close(got, ref + res.double(), torch.float32, f"gemm {kind} + residual algo {algo}")
    assert k.ACTIVATIONS["gelu_new"] == k.ACTIVATIONS["gelu_tanh"]
    with pytest.raises(k.KernelError, match="epilogues know"):
        k.gemm(x.to(DEV), w.to(DEV), activation="swish7")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(7, 96), (3, 50), (33, 1000), (1, 8)])
def test_activation_multiply(dtype, rows, width):
    """out = act(a) * b over dense rows of any stride: the two halves of one wider tensor, a
    destination of its own or in place, vector and element paths (a width of 50 divides by no
    vector)."""
    k = K()
    both = rnd(rows, 2 * width, dtype=dtype, seed=31, scale=2.0).to(DEV)
    a, b = both[:, :width], both[:, width:]
    ad, bd = a.double().cpu(), b.double().cpu()
    for kind in ("none", "relu", "silu", "gelu_tanh"):
        close(k.activation_multiply(a, b, kind), _plain_activation(kind, ad) * bd, dtype, f"{kind}(a) * b")
        close(k.activation(a, kind), _plain_activation(kind, ad), dtype, f"{kind}(a)")
    close(k.multiply(a, b), ad * bd, dtype, "a * b")
    wide = both.clone()
    k.activation_multiply(wide[:, :width], wide[:, width:], "silu", out=wide[:, :width])     # in place, strided
    close(wide[:, :width], _plain_activation("silu", ad) * bd, dtype, "in place")
    assert torch.equal(wide[:, width:], both[:, width:])
    with pytest.raises(k.KernelError, match="activations"):
        k.activation(a, "nope")
    with pytest.raises(k.KernelError, match="must have shape"):
        k.multiply(a, both)


@pytest.mark.parametrize("M,N,K_", [(8, 2048, 2048), (1, 6144, 2048), (64, 8192, 2048), (33, 2048, 8192),
                                    (3, 50272, 2048), (17, 200, 72), (200, 1000, 512), (2048, 6144, 2048),
                                    (130, 200, 72), (129, 50272, 96), (64, 64, 64), (65, 64, 64),
                                    (12, 12288, 4096), (4, 4096, 16384), (16, 7168, 7168), (8, 7168, 28672)])
def test_gemm_bf16_at_model_sizes(M, N, K_):
    """Model-sized products (the widths of OPT-1.3B, 6.7B and 30B among them): the engine's choice
    (0), the plain tiled kernel (1), the vendor library (2) and the hand-written matrix-core
    kernels (3: resident slab, skinny, tiled) against a float64 product of the same bfloat16
    operands on the CPU."""
    k = K()
    x_c = rnd(M, K_, dtype=torch.bfloat16, seed=14)
    w_c = rnd(N, K_, dtype=torch.bfloat16, seed=15, scale=0.05)
    bias_c, res_c = rnd(N, seed=16), rnd(M, N, seed=17)
    base = x_c.double() @ w_c.double().T + bias_c.double()
    mag = x_c.double().abs() @ w_c.double().abs().T          # sum of |products|: scale of the float sum's rounding
    x, w, bias, res = x_c.to(DEV), w_c.to(DEV), bias_c.to(DEV), res_c.to(DEV)
    k.gemm_path_counts(reset=True)
    for algo in (0, 1, 2, 3):
        if algo == 2 and (N % 8 or K_ % 8):
            with pytest.raises(k.KernelError, match="library has no kernel"):
                k.gemm(x, w, algo=2)
            continue
        for rep in range(2):
            try:
                got = k.gemm(x, w, bias=bias, residual=res, out_f32=True, algo=algo)
            except k.KernelError as e:
                if algo == 2 and "library has no kernel" in str(e):
                    break        # the library offers nothing for this shape; the engine then takes its own
                raise
            err = (got.double().cpu() - (base + res_c.double())).abs()
            # exact products summed in float in some order: a few roundings of 2^-24 of the running sum
            assert (err <= 4e-7 * math.sqrt(K_) * mag + 1e-6).all(), f"algo {algo} f32 out, rep {rep}: max err {err.max():.3e}"
            gotb = k.gemm(x, w, bias=bias, activation="relu", algo=algo).double().cpu()
            refb = torch.relu(base)
            assert ((gotb - refb).abs() <= 2.0 ** -8 * refb.abs() + 4e-7 * math.sqrt(K_) * mag + 1e-6).all(), \
                f"algo {algo} bf16 out, rep {rep}"
    paths = k.gemm_path_counts()
    assert paths["generic_bf16"] >= 4            # algo 1, and nothing else fell back to it unnoticed
    if K_ % 8 == 0:
        hand = sum(paths[p] for p in ("resident", "resident_staged", "skinny16", "skinny32", "skinny64", "tiled_mfma"))
        assert hand >= 4 and paths["generic_bf16"] == 4, paths
    if (M, K_) == (8, 28672) or (M, K_) == (4, 16384):
        assert paths["skinny16"] >= 4, paths      # deeper than the resident kernel reaches


def dense_attention(q, kd, vd, scale, pos, window, slopes=None):
    """q [nq, hd]; kd, vd [nkv, n, hd] for positions 0..n-1 (n = pos+1): softmax over [lo, pos].
    slopes [nq]: head h's scores get slopes[h] * (key position - pos) added."""
    nq, nkv = q.shape[0], kd.shape[0]
    lo = max(0, pos + 1 - window) if window > 0 else 0
    out = []
    for h in range(nq):
        kh, vh = kd[h // (nq // nkv)][lo:pos + 1], vd[h // (nq // nkv)][lo:pos + 1]
        s = (kh @ q[h]) * scale
        if slopes is not None:
            s = s + float(slopes[h]) * (torch.arange(lo, pos + 1, dtype=s.dtype) - pos)
        p = torch.softmax(s, dim=0)
        out.append(p @ vh)
    return torch.stack(out)


def head_slopes(nq):
    """Slopes that matter at these lengths: the nearest few dozen keys carry the weight for the
    steepest head, one head has none at all."""
    return torch.tensor([0.0 if h == 1 else 0.25 / (h + 1) for h in range(nq)], dtype=torch.float32)


def build_paged_case(dtype, nq, nkv, hd, ps, lens, seed, spike=False):
    """Requests of the given lengths with shuffled pages in a NaN-filled pool."""
    g = torch.Generator().manual_seed(seed)
    n_pages_needed = sum(-(-n // ps) for n in lens)
    num_pages = n_pages_needed + 5
    perm = torch.randperm(num_pages, generator=g).tolist()
    maxp = max(-(-n // ps) for n in lens) + 2
    bt = torch.full((len(lens), maxp), -1, dtype=torch.int32)
    kd = [rnd(nkv, n, hd, dtype=dtype, seed=seed + 10 + i) for i, n in enumerate(lens)]
    vd = [rnd(nkv, n, hd, dtype=dtype, seed=seed + 50 + i) for i, n in enumerate(lens)]
    if spike:
        for kk in kd:               # one far key that the matching query will score far above the rest
            if kk.shape[1] > 3:
                kk[:, 3, :] = kk[:, 3, :] * 6
    kc = torch.full((num_pages, nkv, ps, hd), float("nan"), dtype=dtype)
    vc = torch.full((num_pages, nkv, ps, hd), float("nan"), dtype=dtype)
    used = 0
    for i, n in enumerate(lens):
        for pi in range(-(-n // ps)):
            page = perm[used]
            used += 1
            bt[i, pi] = page
            a, b = pi * ps, min(n, (pi + 1) * ps)
            kc[page, :, :b - a] = kd[i][:, a:b]
            vc[page, :, :b - a] = vd[i][:, a:b]
    return kc, vc, bt, kd, vd


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,ps", [(4, 4, 16, 4), (3, 3, 32, 8), (6, 2, 64, 16), (2, 1, 80, 32),
                                          (5, 5, 128, 1), (2, 2, 256, 16), (8, 4, 48, 3)])
@pytest.mark.parametrize("window,splits,waves", [(0, 1, 4), (0, 4, 8), (37, 3, 4), (0, 1, 8)])
def test_attention_rows(dtype, nq, nkv, hd, ps, window, splits, waves):
    """Query rows of several requests at arbitrary positions, shuffled pages, unread places NaN.
    Head shapes after src/unittest/kernel/fused_attention.cc:44-61; oracle = gather pages, dense softmax
    (src/unittest/kernel/attention_ref.cc:91-140)."""
    k = K()
    lens = [1, 17, 300, 64, 129]
    kc, vc, bt, kd, vd = build_paged_case(dtype, nq, nkv, hd, ps, lens, seed=hd + ps, spike=True)
    # rows: (item, position); several rows of one item at different positions, as in a prompt portion
    rows = [(0, 0), (1, 16), (2, 299), (2, 150), (2, 3), (3, 63), (4, 128), (4, 127), (1, 0)]
    T = len(rows)
    q = rnd(T, nq * hd, dtype=dtype, seed=99)
    # row 2 looks for the far key 3 of request 2: one score among 300 stands out
    q[2] = (kd[2][:, 3, :].repeat_interleave(nq // nkv, 0) * 0.5).reshape(-1).to(dtype)
    token_item = torch.tensor([r[0] for r in rows], dtype=torch.int32)
    positions = torch.tensor([r[1] for r in rows], dtype=torch.int32)
    scale = 1 / math.sqrt(hd)
    out = k.attention_rows(q.to(DEV), kc.to(DEV), vc.to(DEV), token_item.to(DEV), positions.to(DEV),
                           bt.to(DEV), nq, scale, window=window, num_splits=splits, num_waves=waves)
    ref = torch.stack([dense_attention(q[t].double().view(nq, hd), kd[i].double(), vd[i].double(), scale, p,
                                       window).reshape(-1) for t, (i, p) in enumerate(rows)])
    # bf16: exact inputs, float sums; the stored result is rounded once
    close(out, ref, dtype, f"attention_rows hd={hd} ps={ps} window={window} splits={splits}", scale=1e-3)
    if window == 0:
        # the far key must dominate row 2 (else the test would not see a kernel that drops it)
        p = torch.softmax((kd[2].double()[0] @ q[2].double().view(nq, hd)[0]) * scale, 0)
        assert p[3] > 0.5
    # a position encoding that biases scores by distance (slope per head; a head of slope 0 among them)
    sl = head_slopes(nq)
    out_b = k.attention_rows(q.to(DEV), kc.to(DEV), vc.to(DEV), token_item.to(DEV), positions.to(DEV),
                             bt.to(DEV), nq, scale, window=window, num_splits=splits, num_waves=waves,
                             head_slopes=sl.to(DEV))
    ref_b = torch.stack([dense_attention(q[t].double().view(nq, hd), kd[i].double(), vd[i].double(), scale, p,
                                         window, sl.double()).reshape(-1) for t, (i, p) in enumerate(rows)])
    close(out_b, ref_b, dtype, f"attention_rows with slopes hd={hd} ps={ps} window={window} splits={splits}", scale=1e-3)
    assert (ref_b - ref).abs().max() > 0.05, "the slopes change nothing that this test could see"
    # only some rows through row_ids: the others stay untouched
    sentinel = torch.full_like(out, 7.0)
    ids = torch.tensor([6, 2], dtype=torch.int32)
    k.attention_rows(q.to(DEV), kc.to(DEV), vc.to(DEV), token_item.to(DEV), positions.to(DEV), bt.to(DEV),
                     nq, scale, window=window, num_splits=splits, num_waves=waves, row_ids=ids.to(DEV), out=sentinel)
    close(sentinel[[6, 2]], ref[[6, 2]], dtype, "attention_rows row_ids", scale=1e-3)
    assert (sentinel[[0, 1, 3, 4, 5, 7, 8]] == 7.0).all()


def test_library_products_timed_and_chosen_once():
    """Inside ``tuned_products`` the library's candidates are timed on the caller's operands (a
    plan made in passing before is made again); the product is the same afterwards, also with
    bias, ReLU, and a residual into a float result."""
    k = K()
    M, N, K_ = 24, 320, 192
    x, w = rnd(M, K_, dtype=torch.bfloat16, seed=1).to(DEV), rnd(N, K_, dtype=torch.bfloat16, seed=2, scale=0.05).to(DEV)
    bias, res = rnd(N, seed=3).to(DEV), rnd(M, N, seed=4).to(DEV)
    before = k.gemm(x, w, bias=bias, activation="relu", algo=2)
    before_res = k.gemm(x, w, bias=bias, residual=res, out_f32=True, algo=2)
    with k.tuned_products():
        tuned = k.gemm(x, w, bias=bias, activation="relu", algo=2)
        tuned_res = k.gemm(x, w, bias=bias, residual=res, out_f32=True, algo=2)
    after = k.gemm(x, w, bias=bias, activation="relu", algo=2)
    ref = torch.relu(x.double() @ w.double().T + bias.double())
    for got in (before, tuned, after):
        close(got, ref, torch.bfloat16, "library product", scale=1e-3)
    assert torch.equal(tuned, after)
    ref_res = x.double() @ w.double().T + bias.double() + res.double()
    for got in (before_res, tuned_res):
        assert (got.double() - ref_res).abs().max() <= 1e-4 * ref_res.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kv_write(dtype):
    """Reference: src/unittest/kernel/kvcache_mgmt_ref.cc:9-39 (copy per token, head and slot)."""
    k = K()
    nkv, hd, ps, nq = 3, 32, 8, 6
    num_pages, maxp = 11, 6
    bt = torch.tensor([[4, 9, 1, -1, -1, -1], [7, 0, 2, 10, -1, -1]], dtype=torch.int32)
    token_item = torch.tensor([0, 0, 0, 1, 1, -1], dtype=torch.int32)
    positions = torch.tensor([7, 8, 9, 31, 5, -1], dtype=torch.int32)
    qkv = rnd(6, (nq + 2 * nkv) * hd, dtype=dtype, seed=8)
    # the reference's layout: [num_blocks, num_layers, heads, block, dim]; layer 1 of 2 is written
    kc = torch.zeros(num_pages, 2, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    dq = qkv.to(DEV)
    k.kv_write(kc[:, 1], vc[:, 1], dq[:, nq * hd:(nq + nkv) * hd], dq[:, (nq + nkv) * hd:],
               token_item.to(DEV), positions.to(DEV), bt.to(DEV), ps)
    ek, ev = torch.zeros(num_pages, 2, nkv, ps, hd, dtype=dtype), torch.zeros(num_pages, 2, nkv, ps, hd, dtype=dtype)
    for t in range(5):
        page = bt[token_item[t], positions[t] // ps]
        ek[page, 1, :, positions[t] % ps] = qkv[t, nq * hd:(nq + nkv) * hd].view(nkv, hd)
        ev[page, 1, :, positions[t] % ps] = qkv[t, (nq + nkv) * hd:].view(nkv, hd)
    assert torch.equal(kc.cpu(), ek) and torch.equal(vc.cpu(), ev)


def test_sample_argmax_and_temperature():
    k = K()
    # sizes after src/unittest/kernel/findmax.cc:22-43 (smaller), vocabulary no multiple of 64
    R, V = 37, 2345
    logits = rnd(R, V, seed=9)
    logits[3, 100] = logits[3, 2000] = 50.0        # a tie: the lowest index wins
    logits[4, 0] = 60.0
    logits[5, V - 1] = 60.0
    ids = k.sample(logits.to(DEV)).cpu()
    assert ids.tolist() == torch.argmax(logits, dim=1).tolist()[:3] + [100, 0, V - 1] + \
        torch.argmax(logits, dim=1).tolist()[6:]
    temps = torch.full((R,), 0.8)
    temps[7] = 0.0                                  # a greedy row among sampled ones
    seeds = torch.tensor([[s * 7919 + 1, s] for s in range(R)], dtype=torch.int32)
    draws = torch.arange(R, dtype=torch.int32) * 3
    got = k.sample(logits.to(DEV), temperature=temps.to(DEV), seeds=seeds.to(DEV), draws=draws.to(DEV)).cpu()
    for r in range(R):
        seed = int(seeds[r, 0]) | (int(seeds[r, 1]) << 32)
        if temps[r] == 0:
            assert got[r] == torch.argmax(logits[r])
            continue
        score = plain_opt.perturbed_scores(logits[r].numpy(), 0.8, seed, int(draws[r]))
        best = int(np.argmax(score))
        # equal up to float rounding of the noise: the chosen score is the maximum within 1e-4
        assert got[r] == best or score[best] - score[int(got[r])] < 1e-4, (r, int(got[r]), best)
    # same (seed, draw) gives the same token whatever row it is in
    again = k.sample(logits[10:11].to(DEV), temperature=temps[10:11].to(DEV), seeds=seeds[10:11].to(DEV),
                     draws=draws[10:11].to(DEV)).cpu()
    assert again[0] == got[10]


def test_hash_matches_plain():
    k = K()
    u = plain_opt.hash_uniform((5 << 32) | 77, 9, 50)
    for v in (0, 1, 17, 49):
        assert abs(k.hash_uniform(77, 5, 9, v) - float(u[v])) == 0.0


def test_refusals():
    k = K()
    from swifttransformer_amd.ops.kernels import KernelError
    q = torch.zeros(1, 24, device=DEV)
    kc = torch.zeros(2, 1, 4, 24, device=DEV)
    with pytest.raises(KernelError, match="multiple of 16"):
        k.attention_rows(q, kc, kc, torch.zeros(1, dtype=torch.int32, device=DEV),
                         torch.zeros(1, dtype=torch.int32, device=DEV),
                         torch.zeros(1, 2, dtype=torch.int32, device=DEV), 1, 1.0)
    with pytest.raises(KernelError, match="must have shape"):
        k.gemm(torch.zeros(2, 3, device=DEV), torch.zeros(4, 5, device=DEV))
    with pytest.raises(TypeError):
        k.gemm(torch.zeros(2, 3, device=DEV, dtype=torch.float16), torch.zeros(4, 3, device=DEV, dtype=torch.float16))


@pytest.mark.parametrize("dtype,algo,M", [(torch.float32, 0, 9), (torch.bfloat16, 1, 9), (torch.bfloat16, 0, 9),
                                           (torch.bfloat16, 0, 40), (torch.bfloat16, 0, 150),
                                           (torch.bfloat16, 3, 40), (torch.bfloat16, 3, 150),
                                           (torch.bfloat16, 2, 40), (torch.bfloat16, 2, 150)])
def test_gemm_kv_scatter_epilogue_equals_kv_write(dtype, algo, M):
    """A fused QKV product that also stores keys and values into their pages: the generic kernel,
    the skinny and the tiled matrix-core kernels, and the library product followed by the page
    write, against product + separate page write."""
    k = K()
    nq, nkv, hd, ps, H = 6, 3, 32, 8, 96
    N = (nq + 2 * nkv) * hd
    x, w, bias = rnd(M, H, dtype=dtype, seed=21).to(DEV), rnd(N, H, dtype=dtype, seed=22, scale=0.1).to(DEV), rnd(N, seed=23).to(DEV)
    items = 5
    maxp = -(-200 // ps) + 1
    perm = torch.randperm(items * maxp, generator=torch.Generator().manual_seed(3)).int().view(items, maxp)
    token_item = (torch.arange(M) % items).int()
    positions = (torch.arange(M) // items + 3).int()           # distinct (item, position) pairs
    token_item[M - 1] = -1                                      # a padding row writes nothing
    kc_a = torch.zeros(items * maxp, nkv, ps, hd, dtype=dtype, device=DEV)
    vc_a, kc_b, vc_b = torch.zeros_like(kc_a), torch.zeros_like(kc_a), torch.zeros_like(kc_a)
    ti, po, bt = token_item.to(DEV), positions.to(DEV), perm.to(DEV)
    ref = k.gemm(x, w, bias=bias, algo=algo)
    k.kv_write(kc_a, vc_a, ref[:, nq * hd:(nq + nkv) * hd], ref[:, (nq + nkv) * hd:], ti, po, bt, ps)
    got = k.gemm(x, w, bias=bias, algo=algo, kv_scatter=k.KvScatter(kc_b, vc_b, ti, po, bt, nq * hd))
    assert torch.equal(got, ref)
    assert torch.equal(kc_a, kc_b) and torch.equal(vc_a, vc_b)
    assert kc_a.abs().sum() > 0


@pytest.mark.parametrize("M,N,K_,affine", [(8, 6144, 2048, True), (1, 96, 96, True), (13, 320, 192, False),
                                           (16, 200, 72, True), (16, 8192, 2048, True), (8, 2048, 4096, True),
                                           # 0.75 to 1 workgroup of 32 features a compute unit: those, with 16
                                           # waves (also with a depth that leaves waves without a slab); too
                                           # many rows for their LDS: back to 16 features
                                           (12, 6144, 2048, True), (8, 8192, 2048, True), (7, 6400, 1000, False),
                                           (8, 8192, 4096, True), (12, 8192, 4096, True),
                                           # else between one and two tiles of 16 features a unit:
                                           # workgroups of 24 features (two tiles, the second half full)
                                           (5, 4608, 768, False), (9, 5760, 1536, True)])
def test_gemm_norm_prologue_equals_norm_then_product(M, N, K_, affine):
    k = K()
    x32 = (rnd(M, K_, seed=31) * 2 + 0.5).to(DEV)
    g = (1 + 0.1 * rnd(K_, seed=32)).to(DEV) if affine else None
    b = (0.1 * rnd(K_, seed=33)).to(DEV) if affine else None
    w, bias, res = rnd(N, K_, dtype=torch.bfloat16, seed=34, scale=0.05).to(DEV), rnd(N, seed=35).to(DEV), rnd(M, N, seed=36).to(DEV)
    assert k.can_fuse_norm(M, N, K_, torch.bfloat16)
    assert not k.can_fuse_norm(M, N, K_, torch.float32) and not k.can_fuse_norm(17, N, K_, torch.bfloat16)
    a = torch.empty(M, K_, dtype=torch.bfloat16, device=DEV)
    k.layernorm(x32, g, b, 1e-5, out_t=a)
    ref = k.gemm(a, w, bias=bias, residual=res, out_f32=True)
    got = k.gemm(k.NormInput(x32, g, b, 1e-5), w, bias=bias, residual=res, out_f32=True)
    # the same rounded inputs unless a statistic's last bit moves a value across a rounding boundary
    err = (got - ref).abs().max().item()
    assert err <= 2e-3 * ref.abs().max().item(), err
    refb = k.gemm(a, w, bias=bias, activation="relu").float()
    gotb = k.gemm(k.NormInput(x32, g, b, 1e-5), w, bias=bias, activation="relu").float()
    assert ((gotb - refb).abs() <= 2.0 ** -6 * refb.abs() + 2e-3 * refb.abs().max()).all()
    with pytest.raises(k.KernelError, match="no kernel fuses"):
        k.gemm(k.NormInput(torch.zeros(20, K_, device=DEV), g, b, 1e-5), w)


@pytest.mark.parametrize("M,N,K_", [(8, 8192, 2048), (12, 6144, 2048), (3, 6400, 1000)])
def test_gemm_norm_prologue_workgroup_shapes_agree(M, N, K_):
    """The product with the norm prologue in each of its workgroup shapes (16, 24 and 32 features
    a workgroup; the rule picks one by the matrix and the device) against float64: LayerNorm in
    float64, rounded to bfloat16 as the kernel rounds it, then the product."""
    k = K()
    x32 = (rnd(M, K_, seed=41) * 1.5 - 0.3)
    g, b = 1 + 0.1 * rnd(K_, seed=42), 0.1 * rnd(K_, seed=43)
    w, bias = rnd(N, K_, dtype=torch.bfloat16, seed=44, scale=0.05), rnd(N, seed=45)
    xd = x32.double()
    a = ((xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + 1e-5) * g.double()
         + b.double())
    a_bf = a.float().bfloat16().double()
    ref = a_bf @ w.double().T + bias.double()
    bound = 2.0 ** -7 * (a.abs() @ w.double().abs().T) + 1e-4      # a value rounded the other way, float sums
    outs = []
    try:
        for mode in (0, 1, 3, 7):
            k.gemm_wide_workgroups(mode)
            got = k.gemm(k.NormInput(x32.to(DEV), g.to(DEV), b.to(DEV), 1e-5), w.to(DEV), bias=bias.to(DEV), out_f32=True)
            err = (got.double().cpu() - ref).abs()
            assert (err <= bound).all(), f"mode {mode}: max err {err.max().item():.3e}"
            outs.append(got)
    finally:
        k.gemm_wide_workgroups(-1)      # the default again
    # the shapes differ in how K is split over the waves, so in rounding only
    assert (outs[0] - outs[2]).abs().max().item() <= 1e-3 * ref.abs().max().item()
    assert (outs[0] - outs[3]).abs().max().item() <= 1e-3 * ref.abs().max().item()


@pytest.mark.parametrize("nq,nkv,hd,ps", [(4, 4, 16, 4), (3, 3, 32, 8), (6, 2, 64, 16), (2, 1, 80, 32),
                                          (5, 5, 128, 1), (2, 2, 256, 16), (8, 4, 48, 3),
                                          # so many heads that the tiles are dealt in several rows
                                          (32, 32, 16, 16), (64, 8, 32, 4)])
@pytest.mark.parametrize("window,key_split,dtype", [(0, 0, torch.bfloat16), (37, 0, torch.bfloat16),
                                                    (0, 1, torch.bfloat16), (0, 2, torch.bfloat16),
                                                    (37, 4, torch.bfloat16), (0, 0, torch.float32),
                                                    (37, 0, torch.float32), (130, 0, torch.float32)])
def test_attention_prefill_tiles(nq, nkv, hd, ps, window, key_split, dtype):
    """Portions of prompts (from position 0 and from the middle of a request, lengths that are no
    multiple of the tile) through the tiled matrix-core kernels; shuffled pages, unread places NaN,
    one far key made to stand out.  Oracle as for the row kernel.  The float instance has one
    group of waves and is held to the float tolerance."""
    k = K()
    hdp = (hd + 31) // 32
    if (key_split == 4 and hdp > 2) or (key_split == 2 and hdp > 6):
        # more groups of waves than LDS has room for at this head size
        with pytest.raises(k.KernelError, match="wave groups are not offered"):
            prefill_case(k, nq, nkv, hd, ps, window, dtype, key_split=key_split, algo=1)
        return
    # algo 1: the kernel that stages blocks through registers (the direct-load one has a test of its own)
    algo = 1 if dtype == torch.bfloat16 else 0
    plain = prefill_case(k, nq, nkv, hd, ps, window, dtype, key_split=key_split, algo=algo)
    # scores biased by distance, one slope a head; algo 0 here: the choice must fall on a kernel that has the bias
    biased = prefill_case(k, nq, nkv, hd, ps, window, dtype, key_split=key_split, algo=0, slopes=head_slopes(nq))
    assert (biased.float() - plain.float()).abs().max() > 0.05, "the slopes change nothing that this test could see"


def prefill_case(k, nq, nkv, hd, ps, window, dtype, tile_rows=64, slopes=None, **kw):
    # (cached length before the portion, portion length)
    parts = [(0, 1), (0, 130), (217, 83), (64, 64), (5, 200), (300, 9), (100, 300)]
    lens = [a + b for a, b in parts]
    kc, vc, bt, kd, vd = build_paged_case(dtype, nq, nkv, hd, ps, lens, seed=3 * hd + ps, spike=True)
    T = sum(b for _, b in parts)
    q = rnd(T, nq * hd, dtype=dtype, seed=98)
    tok_off, t = [], 0
    for a, b in parts:
        tok_off.append(t)
        t += b
    # the last row of item 2 looks for the far key 3
    q[tok_off[2] + 82] = (kd[2][:, 3, :].repeat_interleave(nq // nkv, 0) * 0.5).reshape(-1).to(dtype)
    tile_item, tile_q0 = [], []
    for i, (a, b) in enumerate(parts):
        for q0 in range(0, b, tile_rows):
            tile_item.append(i)
            tile_q0.append(q0)
    order = torch.randperm(len(tile_item), generator=torch.Generator().manual_seed(1)).tolist()
    ti = torch.tensor([tile_item[i] for i in order], dtype=torch.int32)
    tq = torch.tensor([tile_q0[i] for i in order], dtype=torch.int32)
    scale = 1 / math.sqrt(hd)
    out = k.attention_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), ti.to(DEV), tq.to(DEV),
                              torch.tensor(tok_off, dtype=torch.int32, device=DEV),
                              torch.tensor([a for a, _ in parts], dtype=torch.int32, device=DEV),
                              torch.tensor([b for _, b in parts], dtype=torch.int32, device=DEV),
                              bt.to(DEV), nq, scale, window=window, tile_rows=tile_rows,
                              head_slopes=None if slopes is None else slopes.to(DEV), **kw)
    ref = []
    for i, (a, b) in enumerate(parts):
        for r in range(b):
            ref.append(dense_attention(q[tok_off[i] + r].double().view(nq, hd), kd[i].double(), vd[i].double(),
                                       scale, a + r, window, None if slopes is None else slopes.double()).reshape(-1))
    ref = torch.stack(ref)
    # probabilities enter the second product rounded to bfloat16 (2^-9 each, averaged over the keys)
    close(out, ref, dtype, f"attention_prefill hd={hd} ps={ps} window={window} tile_rows={tile_rows} "
          f"slopes={slopes is not None} {kw}", scale=4e-3)
    return out


@pytest.mark.parametrize("nq,nkv,hd,ps", [(6, 2, 64, 16), (5, 5, 128, 1), (4, 4, 64, 4), (3, 1, 128, 64),
                                          (32, 32, 64, 16), (40, 8, 128, 8), (2, 2, 64, 128),
                                          # rows of 96 dims in LDS, and head sizes 16 below an instance's
                                          # (the missing chunks of every LDS row stay zero)
                                          (4, 4, 96, 16), (6, 2, 80, 8), (32, 32, 80, 16), (3, 3, 48, 4), (2, 1, 112, 16)])
@pytest.mark.parametrize("window", [0, 37, 130])
@pytest.mark.parametrize("tile_rows,key_split", [(64, 1), (128, 1), (64, 0), (64, 2), (64, 4)])
def test_attention_prefill_direct_load(nq, nkv, hd, ps, window, tile_rows, key_split):
    """The kernel that moves key blocks from memory straight into LDS (swizzled rows, transposing
    reads for the values), with tiles of 64 and of 128 rows and with two or four groups of waves
    sharing a tile's key blocks: same cases and oracle as the staged one."""
    k = K()
    if key_split == 4 and hd > 64:
        with pytest.raises(k.KernelError, match="wave groups are not offered"):      # no room in LDS
            prefill_case(k, nq, nkv, hd, ps, window, torch.bfloat16, tile_rows=tile_rows, algo=2, key_split=4)
        return
    if tile_rows == 128 and hd in (80, 96):
        with pytest.raises(k.KernelError, match="tiles of 128 rows need"):           # no such instance
            prefill_case(k, nq, nkv, hd, ps, window, torch.bfloat16, tile_rows=128, algo=2, key_split=key_split)
        return
    prefill_case(k, nq, nkv, hd, ps, window, torch.bfloat16, tile_rows=tile_rows, algo=2, key_split=key_split)


def test_attention_prefill_direct_load_refuses_other_shapes():
    k = K()
    for nq, nkv, hd, ps, dtype, kw, match in [
            (2, 2, 32, 16, torch.bfloat16, dict(algo=2), "direct-load kernel is not offered"),
            (2, 2, 160, 16, torch.bfloat16, dict(algo=2), "direct-load kernel is not offered"),
            (2, 2, 64, 12, torch.bfloat16, dict(algo=2), "direct-load kernel is not offered"),
            (2, 2, 64, 16, torch.float32, dict(tile_rows=128), "tiles of 128 rows need"),
            (2, 2, 96, 16, torch.bfloat16, dict(tile_rows=128), "tiles of 128 rows need"),
            (2, 2, 64, 16, torch.bfloat16, dict(tile_rows=128, algo=1), "tiles of 128 rows need"),
            (2, 2, 64, 16, torch.bfloat16, dict(tile_rows=96), "tiles of 96 rows"),
            # it has no score bias
            (2, 2, 64, 16, torch.bfloat16, dict(algo=2, slopes=head_slopes(2)), "not offered .* with score slopes"),
            (2, 2, 128, 16, torch.bfloat16, dict(tile_rows=128, slopes=head_slopes(2)), "tiles of 128 rows need")]:
        with pytest.raises(k.KernelError, match=match):
            prefill_case(k, nq, nkv, hd, ps, 0, dtype, **kw)
    assert k.prefill_tile_rows(128, 16, 128, 32, 2048, torch.bfloat16) == 128
    assert k.prefill_tile_rows(128, 16, 128, 32, 512, torch.bfloat16) == 64       # too few tiles to fill the chip
    assert k.prefill_tile_rows(64, 16, 128, 32, 4096, torch.bfloat16) == 64       # small heads: 64 rows are faster
    assert k.prefill_tile_rows(80, 16, 128, 32, 4096, torch.bfloat16) == 64
    assert k.prefill_tile_rows(128, 12, 128, 32, 4096, torch.bfloat16) == 64
    assert k.prefill_tile_rows(128, 16, 128, 32, 4096, torch.float32) == 64


@pytest.mark.parametrize("T,nq,nkv,hd,splits", [(1, 32, 32, 64, 8), (2, 32, 32, 64, 4), (4, 32, 8, 64, 2),
                                                 (3, 6, 3, 32, 3), (7, 4, 4, 16, 5),
                                                 # two splits of more rows: the prologue with more elements a thread
                                                 (8, 32, 32, 64, 2), (5, 32, 32, 64, 2), (16, 32, 8, 64, 2), (12, 6, 3, 32, 2)])
def test_gemm_merges_a_split_attention_output(T, nq, nkv, hd, splits):
    """The output projection takes a decode attention still split over the keys (partial results
    and log-sum-exps) and merges it itself.  Oracle: dense attention over the gathered keys in
    float64 (src/unittest/kernel/attention_ref.cc:91-140), then the product in float64; one key
    far from the query is made to dominate a row, so a split that is dropped or weighted wrongly
    shows."""
    k = K()
    dtype = torch.bfloat16
    ps = 16
    lens = [300 + 37 * i for i in range(T)]
    kc, vc, bt, kd, vd = build_paged_case(dtype, nq, nkv, hd, ps, lens, seed=7 * T + hd, spike=True)
    q = rnd(T, nq * hd, dtype=dtype, seed=5)
    q[0] = (kd[0][:, 3, :].repeat_interleave(nq // nkv, 0) * 0.5).reshape(-1).to(dtype)   # looks for key 3
    scale = 1 / math.sqrt(hd)
    p3 = torch.softmax((kd[0].double()[0] @ q[0].double().view(nq, hd)[0]) * scale, 0)[3]
    assert p3 > 0.5, "the far key does not dominate"
    ti = torch.arange(T, dtype=torch.int32).to(DEV)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32).to(DEV)
    args = (q.to(DEV), kc.to(DEV), vc.to(DEV), ti, pos, bt.to(DEV), nq, scale)
    split = k.attention_rows(*args, num_splits=splits, merge=False)
    assert isinstance(split, k.SplitAttention) and split.part_o.shape == (T, nq, splits, hd)
    N, K_ = 96 if nq * hd < 1024 else 2048, nq * hd
    w = rnd(N, K_, dtype=dtype, seed=8, scale=0.05)
    bias, res = rnd(N, seed=9), rnd(T, N, seed=10)
    assert k.can_fuse_merge(T, N, K_, splits, nq, hd, dtype)
    got = k.gemm(split, w.to(DEV), bias=bias.to(DEV), residual=res.to(DEV), out_f32=True)
    attn = torch.stack([dense_attention(q[t].double().view(nq, hd), kd[t].double(), vd[t].double(), scale,
                                        lens[t] - 1, 0).reshape(-1) for t in range(T)])
    ref = attn @ w.double().T + bias.double() + res.double()
    # the merged attention rows are rounded to bfloat16 (2^-9 relative) before the product's
    # K_ float multiply-adds; the residual and bias are exact
    prod = (attn.abs() @ w.double().abs().T)
    err = (got.double().cpu() - ref).abs()
    assert (err <= 2.0 ** -8 * prod + 1e-5).all(), f"max err {err.max().item():.3e}"
    # and the same rows through the merge kernel and a plain product agree with it to rounding
    merged = k.attention_rows(*args, num_splits=splits)
    two = k.gemm(merged, w.to(DEV), bias=bias.to(DEV), residual=res.to(DEV), out_f32=True)
    assert ((two.double().cpu() - ref).abs() <= 2.0 ** -8 * prod + 1e-5).all()
    assert not k.can_fuse_merge(T, N, K_, 9, nq, hd, dtype) and not k.can_fuse_merge(17, N, K_, splits, nq, hd, dtype)
    assert not k.can_fuse_merge(8, 2048, 2048, 4, 32, 64, dtype)       # too many partial results for a thread's registers
    with pytest.raises(k.KernelError, match="no kernel merges"):
        k.gemm(split, w.to(DEV), algo=3)


@pytest.mark.parametrize("M,N,K_", [(1, 50272, 2048), (8, 20010, 2048), (16, 16400, 1000), (5, 17001, 512), (3, 32768, 64)])
def test_gemm_wide_matrix_norm_of_picked_rows_and_best_outputs(M, N, K_):
    """The persistent kernel for few rows and a very wide matrix (an output head): plain stored rows,
    and LayerNorm of rows picked by an index as its prologue, against float64; and the rows' best
    outputs from its epilogue against the arg-max of its own logits, lowest index on ties (two
    features are given equal weights so that there is a tie at the top of some rows)."""
    k = K()
    if not k.wide_offered(M, N, K_, torch.bfloat16):
        pytest.skip("this device has too many compute units for a matrix of this width")
    w_c = rnd(N, K_, dtype=torch.bfloat16, seed=71, scale=0.05)
    x_c = rnd(M, K_, dtype=torch.bfloat16, seed=72)
    # a tie at the top: feature 7 is made the best of row 0 and feature N - 5 a copy of it
    w_c[7] = (x_c[0].float() * 0.2).bfloat16()
    w_c[N - 5] = w_c[7]
    bias_c = rnd(N, seed=73, scale=0.01)
    bias_c[N - 5] = bias_c[7]
    x, w, bias = x_c.to(DEV), w_c.to(DEV), bias_c.to(DEV)
    k.gemm_path_counts(reset=True)
    best = torch.full((M,), -1, dtype=torch.int32, device=DEV)
    got = k.gemm(x, w, bias=bias, out_f32=True, best=best)
    assert k.gemm_path_counts()["wide"] == 1
    ref = x_c.double() @ w_c.double().T + bias_c.double()
    mag = x_c.double().abs() @ w_c.double().abs().T
    assert ((got.double().cpu() - ref).abs() <= 1e-5 * mag + 1e-6).all()
    own = got.cpu()
    for m in range(M):
        top = own[m].max()
        assert int(best[m]) == int((own[m] == top).nonzero()[0]), f"row {m}"
    assert int(best[0]) == 7 and own[0, 7] == own[0, N - 5]
    # the same through the generic kernel's logits: equal up to the float sum's order
    plain = k.gemm(x, w, bias=bias, out_f32=True, algo=1)
    assert ((plain - got).abs().cpu().double() <= 1e-5 * mag + 1e-6).all()
    # norm prologue over picked rows
    T = 40
    x32 = (rnd(T, K_, seed=74) * 1.7 + 0.4)
    g, b = 1 + 0.1 * rnd(K_, seed=75), 0.1 * rnd(K_, seed=76)
    rows = torch.tensor([(7 * i + 3) % T for i in range(M)], dtype=torch.int32)
    xd = x32.double()[rows.long()]
    a = ((xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + 1e-5) * g.double()
         + b.double())
    ref_n = a.float().bfloat16().double() @ w_c.double().T
    bound = 2.0 ** -7 * (a.abs() @ w_c.double().abs().T) + 1e-4     # a value rounded the other way, float sums
    best_n = torch.full((M,), -1, dtype=torch.int32, device=DEV)
    got_n = k.gemm(k.NormInput(x32.to(DEV), g.to(DEV), b.to(DEV), 1e-5, rows=rows.to(DEV)), w, out_f32=True, best=best_n)
    assert ((got_n.double().cpu() - ref_n).abs() <= bound).all()
    assert torch.equal(best_n.cpu().long(), got_n.cpu().argmax(-1))
    no_affine = k.gemm(k.NormInput(x32.to(DEV), None, None, 1e-5, rows=rows.to(DEV)), w, out_f32=True)
    a0 = (xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + 1e-5)
    assert ((no_affine.double().cpu() - a0.float().bfloat16().double() @ w_c.double().T).abs()
            <= 2.0 ** -7 * (a0.abs() @ w_c.double().abs().T) + 1e-4).all()
    # what the kernel does not offer is refused, not computed wrongly
    with pytest.raises(k.KernelError, match="best outputs"):
        k.gemm(x, w[:4096], out_f32=True, best=best)
    with pytest.raises(k.KernelError, match="picked rows"):
        k.gemm(k.NormInput(x32.to(DEV), None, None, 1e-5, rows=rows.to(DEV)), w[:4096], out_f32=True)


@pytest.mark.parametrize("M,N,K_", [(8, 6144, 2048), (3, 20000, 1000)])
def test_product_prologue_with_the_norm_that_takes_no_mean_off(M, N, K_):
    """The norm prologue of the products by its flag: no mean taken off (root-mean-square norm), in
    the kernel that keeps the slab of W in registers and in the one that walks a very wide matrix."""
    k = K()
    x32 = rnd(M, K_, seed=81) * 1.3 + 0.8
    g = 1 + 0.1 * rnd(K_, seed=82)
    w = rnd(N, K_, dtype=torch.bfloat16, seed=83, scale=0.05)
    xd = x32.double()
    a = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * g.double()
    ref = a.float().bfloat16().double() @ w.double().T
    bound = 2.0 ** -7 * (a.abs() @ w.double().abs().T) + 1e-4
    centred = ((xd - xd.mean(-1, keepdim=True)) / torch.sqrt(xd.var(-1, unbiased=False, keepdim=True) + 1e-5)
               * g.double()) @ w.double().T
    assert (centred - ref).abs().max() > 10 * bound.max()          # the flag matters here
    k.gemm_path_counts(reset=True)
    got = k.gemm(k.NormInput(x32.to(DEV), g.to(DEV), None, 1e-5, center=False), w.to(DEV), out_f32=True)
    paths = k.gemm_path_counts()
    assert paths["resident_norm"] + paths["wide"] == 1, paths
    assert ((got.double().cpu() - ref).abs() <= bound).all()


# ------------------------------------------------------------- measurement kernels
def test_read_probes_read_every_byte_once_in_every_pattern():
    """The streaming-read probe behind the benchmark's floors: every pattern leaves the same sum
    of what it read (each 32-bit word of the buffer once), whatever the number of workgroups."""
    k = K()
    n_bytes = 16 * 16384 * 2                                   # 32 groups of 16 rows of 16 KB, 128 of 4 KB
    src = torch.randint(0, 2 ** 31 - 1, (n_bytes // 4,), dtype=torch.int32, device=DEV)
    words = src.view(-1, 4).cpu().numpy().astype(np.uint32)
    want = int((words[:, 0] ^ words[:, 1] ^ words[:, 2] ^ words[:, 3]).astype(np.uint64).sum() % (1 << 32))
    for pattern in range(6):
        for wgs in (3, 64):
            sink = torch.zeros(wgs, dtype=torch.int32, device=DEV)
            k.probe_read(src, sink, wgs, pattern)
            got = int(sink.cpu().numpy().astype(np.uint32).astype(np.uint64).sum() % (1 << 32))
            assert got == want, (pattern, wgs)
    with pytest.raises(k.KernelError):
        k.probe_read(src[:1024 * 5], torch.zeros(4, dtype=torch.int32, device=DEV), 4, 4)   # not groups of 16 rows


def test_fill_and_matrix_core_probes_run():
    """The other two probes of the floors: a workgroup going round its own region (both ways of
    loading leave the same sums, those of the region's last two turns) and the matrix cores'
    issue loop (its result is the product it repeats: 16 * rounds * 32 * (lane & 3))."""
    k = K()
    wgs, region, turns = 8, 64 << 10, 6
    src = torch.randint(0, 2 ** 31 - 1, (wgs * region // 4,), dtype=torch.int32, device=DEV)
    sinks = []
    for to_lds in (False, True):
        sink = torch.zeros(wgs, dtype=torch.int32, device=DEV)
        k.probe_fill(src, region, sink, wgs, turns, to_lds)
        sinks.append(sink.cpu())
    assert (sinks[0] != 0).any() and (sinks[1] != 0).any()
    for wide in (False, True):
        sink = torch.zeros(4, dtype=torch.int32, device=DEV)
        k.probe_mfma(sink, 4, 3, wide)
        torch.cuda.synchronize()
        # thread 0 of a workgroup: a = 0 in every lane it multiplies with, so its first output is 0
        assert sink.cpu().tolist() == [0, 0, 0, 0]
