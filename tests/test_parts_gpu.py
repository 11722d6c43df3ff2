"""Each part alone against the plain implementation's function for it, and a toy mixer with
state of its own, defined here, registered, built and stepped without touching the engine."""
import math

import pytest
import torch

import plain_opt as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, ref):
    if dtype == torch.float32:
        return 2e-5 + 1e-4 * ref.abs()
    return 0.03 * ref.std() + 0.02 * ref.abs()


def check(got, ref, dtype, what):
    got, ref = got.detach().double().cpu(), ref.double()
    assert got.shape == ref.shape, what
    err = (got - ref).abs()
    assert torch.isfinite(got).all() and (err <= tol(dtype, ref)).all(), f"{what}: max err {err.max():.3e}"


def rand_weights(part, dtype, seed=0):
    from swifttransformer_amd.weights import random_tensors
    t = random_tensors(part.tensor_specs(), seed, dtype, DEV)
    return t, {k: v.double().cpu() for k, v in t.items()}


def ctx_for(items, page_size=8, max_pages=16, vocab=100000, max_positions=4096, parts=()):
    """The step description of ``items``, with the work lists that ``parts`` ask for."""
    from swifttransformer_amd.engine.batch import pack_batch
    planners = dict(p.step_planner() for p in parts if hasattr(p, "step_planner"))
    return pack_batch(items, [0], max_pages, page_size, DEV, vocab_size=vocab, max_positions=max_positions,
                      planners=planners)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from swifttransformer_amd.parts import PartSpec, build_part
    H = 200
    part = build_part("norm", PartSpec("layer_norm", {"eps": 3e-4, "affine": True},
                                       {"weight": "n.weight", "bias": "n.bias"}), H, dtype)
    t, w = rand_weights(part, dtype)
    part.bind(t)
    x = torch.randn(9, H) * 2 + 1
    y_t, y32 = part.forward(x.to(DEV), out_t=True, out_f32=True)
    ref = P.layer_norm(x.double(), w["n.weight"], w["n.bias"], 3e-4)
    check(y32, ref, torch.float32, "norm f32")
    check(y_t, ref, dtype, "norm t")
    assert y_t.dtype == dtype
    plain = build_part("norm", PartSpec("layer_norm", {"eps": 1e-5, "affine": False}), H, dtype)
    assert plain.tensor_specs() == []
    y_t, _ = plain.forward(x.to(DEV))
    check(y_t, P.layer_norm(x.double(), None, None, 1e-5), dtype, "norm without gain")
    # the same part as a root-mean-square norm: a gain, no bias, no mean taken off
    rms = build_part("norm", PartSpec("layer_norm", {"eps": 1e-6, "center": False, "bias": False}, {"weight": "r.weight"}),
                     H, dtype)
    assert [s.name for s in rms.tensor_specs()] == ["r.weight"]
    t, w = rand_weights(rms, dtype)
    rms.bind(t)
    y_t, y32 = rms.forward(x.to(DEV), out_t=True, out_f32=True)
    xd = x.double()
    ref = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * w["r.weight"]
    check(y32, ref, torch.float32, "root-mean-square norm f32")
    check(y_t, ref, dtype, "root-mean-square norm t")
    assert rms.as_input(x.to(DEV)).center is False and rms.as_input(x.to(DEV)).beta is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E", [72, 40])
def test_embedding_position_and_head_parts(dtype, E):
    from swifttransformer_amd.engine.batch import StepItem
    from swifttransformer_amd.parts import PartSpec, build_part
    H, V, Pmax = 72, 333, 50
    emb = build_part("embedding", PartSpec("token", {"vocab_size": V, "embed_dim": E},
                                           {"weight": "tok", "project_in": "pin"}), H, dtype)
    pos = build_part("position", PartSpec("learned", {"max_positions": Pmax, "offset": 2}, {"weight": "pos"}),
                     H, dtype)
    head = build_part("head", PartSpec("linear", {"vocab_size": V, "embed_dim": E, "tied_to": "tok"},
                                       {"weight": "lm", "project_out": "pout"}), H, dtype)
    from swifttransformer_amd.weights import random_tensors
    specs = emb.tensor_specs() + pos.tensor_specs() + head.tensor_specs()
    t = random_tensors(specs, 1, dtype, DEV)             # the optional head tensor is left out: tied
    w = {k: v.double().cpu() for k, v in t.items()}
    for p in (emb, pos, head):
        p.bind(t)
    assert head.weight.data_ptr() == emb.table.data_ptr()
    items = [StepItem(0, 5, [7, 300, 2], [0], {0: [0]}), StepItem(1, 0, [332], [0], {0: [1]})]
    ctx = ctx_for(items, vocab=V, max_positions=Pmax)
    x = emb.forward(ctx, pos)
    ref = P.embed([7, 300, 2, 332], [5, 6, 7, 0], w["tok"], w["pos"], 2, w.get("pin"))
    check(x, ref, dtype if E != H else torch.float32, "embedding")
    # no positions: the table rows alone
    none = build_part("position", PartSpec("none"), H, dtype)
    x0 = emb.forward(ctx, none)
    check(x0, P.embed([7, 300, 2, 332], [0] * 4, w["tok"], torch.zeros_like(w["pos"]), 2, w.get("pin")),
          dtype if E != H else torch.float32, "embedding without positions")
    y = torch.randn(3, H).to(dtype)
    logits = head.forward(y.to(DEV))
    yy = y.double()
    if E != H:
        yy = yy @ w["pout"].T
        if dtype == torch.bfloat16:
            yy = yy.to(torch.bfloat16).double()
    assert logits.dtype == torch.float32
    check(logits, yy @ w["tok"].T, torch.float32 if dtype == torch.float32 else dtype, "head")


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(dtype):
    from swifttransformer_amd.parts import PartSpec, build_part
    H, Fd = 72, 200
    names = {f"{n}.{t}": f"l.{n}.{t}" for n in ("fc1", "fc2") for t in ("weight", "bias")}
    part = build_part("feed_forward", PartSpec("dense", {"inner": Fd, "activation": "relu", "bias": True}, names),
                      H, dtype)
    t, w = rand_weights(part, dtype, seed=2)
    part.bind(t)
    d = torch.randn(11, H).to(dtype)
    res = torch.randn(11, H)
    out = part.forward(d.to(DEV), res.to(DEV), None)
    ref = res.double() + P.feed_forward(d.double(), w, "l", True)
    check(out, ref, dtype, "feed-forward")
    with pytest.raises(ValueError, match="activation"):
        build_part("feed_forward", PartSpec("dense", {"inner": 8, "activation": "gelu"}, names), H, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd", [(3, 3, 32), (4, 2, 16)])
def test_attention_part_chunked_equals_whole(dtype, nh, nkv, hd):
    """The mixer alone: a sequence run whole, then again in portions and single tokens on other
    pages; grouped keys too (the plain attention_layer covers nkv == nh)."""
    from swifttransformer_amd.cache.device import CacheView
    from swifttransformer_amd.engine.batch import StepItem
    from swifttransformer_amd.parts import PartSpec, build_part
    H = nh * hd
    names = {f"{n}.{t}": f"l.self_attn.{n}_proj.{t}" for n in ("q", "k", "v", "out") for t in ("weight", "bias")}
    part = build_part("mixer", PartSpec("paged_attention", {"num_heads": nh, "num_kv_heads": nkv, "head_dim": hd,
                                                            "scale": hd ** -0.5, "bias": True}, names), H, dtype)
    t, w = rand_weights(part, dtype, seed=3)
    for k_ in list(t):      # larger weights so that attention is far from uniform
        if k_.endswith("weight"):
            t[k_] = (t[k_].float() * 8).to(t[k_].dtype)
            w[k_] = t[k_].double().cpu()
    part.bind(t)
    n, ps = 45, 8
    a = torch.randn(n, H).to(dtype)
    res = torch.randn(n, H)
    if nkv == nh:
        ref = res.double() + P.attention_layer(a.double(), w, "l", nh, True)
    else:
        # grouped keys: repeat each key head over its query heads, then the plain layer's maths
        rep = nh // nkv
        w2 = dict(w)
        for nm in ("k", "v"):
            w2[f"l.self_attn.{nm}_proj.weight"] = w[f"l.self_attn.{nm}_proj.weight"].view(nkv, hd, H) \
                .repeat_interleave(rep, 0).reshape(nh * hd, H)
            w2[f"l.self_attn.{nm}_proj.bias"] = w[f"l.self_attn.{nm}_proj.bias"].view(nkv, hd) \
                .repeat_interleave(rep, 0).reshape(nh * hd)
        ref = res.double() + P.attention_layer(a.double(), w2, "l", nh, True)
    kc = torch.full((20, nkv, ps, hd), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full_like(kc, float("nan"))
    cache = CacheView(0, 0, k=kc, v=vc)
    pages_whole, pages_cut = [3, 9, 1, 12, 5, 0], [7, 2, 19, 4, 11, 6]
    ctx = ctx_for([StepItem(0, 0, list(range(n)), [], {0: pages_whole})], page_size=ps, parts=[part])
    out = part.forward(a.to(DEV), res.to(DEV), ctx, cache)
    check(out, ref, dtype, "attention part, whole")
    p = 0
    for c in (5, 2, 17, 1, 1, 9, 10):
        ctx = ctx_for([StepItem(1, p, list(range(c)), [], {0: pages_cut})], page_size=ps, parts=[part])
        out = part.forward(a[p:p + c].to(DEV), res[p:p + c].to(DEV), ctx, cache)
        check(out, ref[p:p + c], dtype, f"attention part, portion at {p}")
        p += c


class RunningMeanMixer:
    """A toy mixer with state of its own: the mean of all inputs of the request so far,
    times a matrix.  Its state (running sum and count) lives in the request's state slot."""
    graph_safe = False

    def __init__(self, spec, hidden_size, dtype):
        self.spec, self.hidden_size, self.dtype = spec, hidden_size, dtype
        self.w = None

    def tensor_specs(self):
        from swifttransformer_amd.weights import TensorSpec
        return [TensorSpec(self.spec.names["weight"], (self.hidden_size, self.hidden_size), "matrix")]

    def bind(self, tensors):
        self.w = tensors[self.spec.names["weight"]]

    def cache_need(self):
        from swifttransformer_amd.parts import CacheNeed
        return CacheNeed("state", state_shape=(self.hidden_size + 1,), state_dtype=torch.float32)

    def forward(self, x_t, residual32, ctx, cache, write=True):
        out = torch.empty_like(residual32)
        off = 0
        for slot, n in zip(ctx.host_item_slot, ctx.host_item_len):
            st = cache.state[slot]
            x = x_t[off:off + n].float()
            sums = torch.cumsum(x, 0) + st[:-1]
            counts = st[-1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            mean = sums / counts[:, None]
            out[off:off + n] = residual32[off:off + n] + mean @ self.w.float().T
            st[:-1] = sums[-1]
            st[-1] = counts[-1]
            off += n
        return out


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_registers_builds_and_steps(dtype):
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part
    from swifttransformer_amd.weights import random_tensors
    register_part("mixer", "running_mean", RunningMeanMixer)
    H, V, Pmax, nh = 64, 97, 80, 2
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    ffn = lambda i: PartSpec("dense", {"inner": 96, "activation": "relu", "bias": False},
                             {"fc1.weight": f"l{i}.fc1", "fc2.weight": f"l{i}.fc2"})
    attn = PartSpec("paged_attention", {"num_heads": nh, "head_dim": 32, "scale": 32 ** -0.5, "bias": False},
                    {f"{n}.weight": f"l1.{n}" for n in ("q", "k", "v", "out")})
    layers = [LayerSpec(PartSpec("pre_norm"), norm("l0.n1"), PartSpec("running_mean", {}, {"weight": "l0.toy"}),
                        norm("l0.n2"), ffn(0)),
              LayerSpec(PartSpec("post_norm"), norm("l1.n1"), attn, norm("l1.n2"), ffn(1))]
    # the toy layer runs twice (two caches, i.e. two states), the attention layer once between them
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("learned", {"max_positions": Pmax, "offset": 0}, {"weight": "pos"}),
                     layers=layers,
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2)],
                     final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    needs = model.cache_needs()
    assert sorted(needs) == [0, 1, 2] and needs[0].kind == "state" and needs[1].kind == "paged_kv"
    model.bind(random_tensors(model.tensor_specs(), 5, dtype, DEV))
    assert not model.graph_safe
    runner = ModelRunner(model, CacheParam(page_size=4, num_pages=40, max_seqs=3), DEV)
    assert [g.need.kind for g in runner.manager.groups] == ["state", "paged_kv"]
    seqs = {"a": torch.randint(0, V, (37,), generator=torch.Generator().manual_seed(1)).tolist(),
            "b": torch.randint(0, V, (22,), generator=torch.Generator().manual_seed(2)).tolist()}
    whole = {}
    for rid, toks in seqs.items():
        runner.admit(rid)
        whole[rid] = runner.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu()
        runner.finish(rid)
    # again, cut into portions and mixed in one batch, in slots that held other state before
    done = {"a": 0, "b": 0}
    for rid in ("b", "a"):
        runner.admit(rid)
    cuts = {"a": [5, 1, 9, 2, 20], "b": [2, 12, 1, 7]}
    got = {"a": [], "b": []}
    while any(cuts.values()):
        entries = []
        for rid in ("a", "b"):
            if cuts[rid]:
                c = cuts[rid].pop(0)
                entries.append(StepEntry(rid, seqs[rid][done[rid]:done[rid] + c], list(range(c))))
        logits = runner.step(entries).cpu()
        r = 0
        for e in entries:
            got[e.req_id].append(logits[r:r + len(e.tokens)])
            r += len(e.tokens)
            done[e.req_id] += len(e.tokens)
    for rid in seqs:
        check(torch.cat(got[rid]), whole[rid], dtype, f"toy model, request {rid} cut vs whole")
    # the first token's logits follow from the definition: mean of one input is the input
    assert torch.isfinite(whole["a"]).all()
    runner.finish("a"), runner.finish("b")
    runner.manager.check_invariants()


def _windowed_reference(x, w, nh, hd, window):
    """Plain attention with keys limited to the last `window` positions (own included)."""
    n, H = x.shape
    q, k, v = (x @ w[f"l.{nm}"].T for nm in "qkv")
    out = torch.zeros(n, nh * hd, dtype=torch.float64)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        s = (q[:, sl] @ k[:, sl].T) / math.sqrt(hd)
        i = torch.arange(n)
        mask = (i[None, :] > i[:, None]) | (i[None, :] <= i[:, None] - window)
        out[:, sl] = torch.softmax(s.masked_fill(mask, float("-inf")), -1) @ v[:, sl]
    return out @ w["l.out"].T


@pytest.mark.parametrize("dtype", DTYPES)
def test_windowed_and_full_attention_groups_release_pages(dtype):
    """A layer whose attention sees a window of 20 keys beside a layer that sees all: two cache
    groups with pages of their own; the windowed group gives pages back while the request runs,
    so a pool far smaller than the sequence suffices, and logits equal the whole-sequence run."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, build_part
    from swifttransformer_amd.weights import random_tensors
    H, V, Pmax, nh, hd, W = 64, 120, 400, 2, 32, 20
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    ffn = lambda i: PartSpec("dense", {"inner": 96, "activation": "relu", "bias": False},
                             {"fc1.weight": f"l{i}.fc1", "fc2.weight": f"l{i}.fc2"})
    attn = lambda i, win: PartSpec("paged_attention", {"num_heads": nh, "head_dim": hd, "scale": hd ** -0.5,
                                                       "bias": False, "window": win},
                                   {f"{n}.weight": f"l{i}.{n}" for n in ("q", "k", "v", "out")})
    layers = [LayerSpec(PartSpec("pre_norm"), norm(f"l{i}.n1"), attn(i, win), norm(f"l{i}.n2"), ffn(i))
              for i, win in enumerate((W, 0, W))]
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("learned", {"max_positions": Pmax, "offset": 0}, {"weight": "pos"}),
                     layers=layers, schedule=[ScheduleEntry(i, i) for i in range(3)], final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    tensors = random_tensors(model.tensor_specs(), 9, dtype, DEV)
    for k_ in tensors:                 # sharper attention, so that a key wrongly kept or dropped shows
        if k_.endswith(".q") or k_.endswith(".k"):
            tensors[k_] = (tensors[k_].float() * 10).to(tensors[k_].dtype)
    model.bind(tensors)
    # the windowed mixer alone against the plain windowed attention
    part = model.layers[0].mixer
    w = {f"l.{n}": tensors[f"l0.{n}"].double().cpu() for n in ("q", "k", "v", "out")}
    ps, n = 8, 150
    # group 0: windowed (layers 0 and 2), group 1: full.  12 windowed pages < the 19 the sequence spans
    runner = ModelRunner(model, CacheParam(page_size=ps, num_pages={0: 12, 1: 40}, max_seqs=2), DEV,
                         cache_fill=float("nan"))
    assert [g.need.window for g in runner.manager.groups] == [W, 0]
    toks = torch.randint(0, V, (n,), generator=torch.Generator().manual_seed(4)).tolist()
    big = ModelRunner(model, CacheParam(page_size=ps, num_pages=40, max_seqs=2), DEV)
    big.admit("w")
    whole = big.step([StepEntry("w", toks, list(range(n)))]).cpu()
    runner.admit("r")
    got, p = [], 0
    cuts = [9, 30, 2, 17, 1, 1, 25, 8, 1, 40, 1, 1, 1, 13]
    assert sum(cuts) == n
    for c in cuts:
        got.append(runner.step([StepEntry("r", toks[p:p + c], list(range(c)))]).cpu().clone())
        p += c
        runner.manager.check_invariants()
    held = sum(pg >= 0 for pg in runner.manager.requests["r"].tables[0])
    assert held <= 12 and runner.manager.requests["r"].tables[0][0] == -1      # early pages were given back
    check(torch.cat(got), whole, dtype, "windowed model: portions with released pages vs whole")
    # and the mixer's maths against the plain windowed formula
    a = torch.randn(40, H).to(dtype)
    from swifttransformer_amd.cache.device import CacheView
    from swifttransformer_amd.engine.batch import StepItem
    kc = torch.full((8, nh, ps, hd), float("nan"), dtype=dtype, device=DEV)
    ctx = ctx_for([StepItem(0, 0, list(range(40)), [], {0: [5, 1, 7, 0, 3]})], page_size=ps, parts=[part])
    out = part.forward(a.to(DEV), torch.zeros(40, H, device=DEV), ctx, CacheView(0, 0, k=kc, v=torch.full_like(kc, float("nan"))))
    check(out, _windowed_reference(a.double(), w, nh, hd, W), dtype, "windowed attention part")


class ToyRotary:
    """A toy position encoding that turns each pair (2i, 2i+1) of every head of the queries and
    keys by the angle position * theta**(-i / (head_dim/2)); nothing is added to the embedding."""
    rotates = True

    def __init__(self, spec, hidden_size, dtype):
        self.head_dim = int(spec.params["head_dim"])
        self.theta = float(spec.params["theta"])

    def tensor_specs(self):
        return []

    def bind(self, tensors):
        pass

    def embedding_addend(self, ctx):
        return None

    def angles(self, positions):
        half = self.head_dim // 2
        inv = self.theta ** (-torch.arange(half, dtype=torch.float64, device=positions.device) / half)
        return positions.double()[:, None] * inv[None, :]

    def turn(self, t, positions):
        """t [T, heads*head_dim] -> rotated copy (float64)."""
        T, half = t.shape[0], self.head_dim // 2
        ang = self.angles(positions)
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        v = t.double().reshape(T, -1, half, 2)
        return torch.stack([v[..., 0] * c - v[..., 1] * s, v[..., 0] * s + v[..., 1] * c], -1).reshape(T, -1)

    def rotate(self, q, k, ctx):
        pos = ctx.positions.clamp(min=0)
        for t in (q, k):
            t.copy_(self.turn(t, pos).to(t.dtype))


class ToyScaleNorm:
    """A toy norm: x / sqrt(mean(x^2) + eps) * gain, in float, with library tensor operations."""

    def __init__(self, spec, hidden_size, dtype):
        self.spec, self.dtype, self.width = spec, dtype, hidden_size
        self.eps = float(spec.params["eps"])

    def tensor_specs(self):
        from swifttransformer_amd.weights import TensorSpec
        return [TensorSpec(self.spec.names["gain"], (self.width,), "vector", init="gain")]

    def bind(self, tensors):
        self.gain = tensors[self.spec.names["gain"]]

    @staticmethod
    def compute(x, gain, eps):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * gain

    def forward(self, x32, *, out_t=True, out_f32=False, rows=None):
        x = x32 if rows is None else x32[rows.long()]
        y = self.compute(x, self.gain, self.eps)
        return (y.to(self.dtype) if out_t else None), (y if out_f32 else None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_rotating_position_encoding(dtype):
    """Another position encoding and another norm, defined here: the attention mixer calls the
    encoding's ``rotate`` between the QKV product and the page write; the norm stands before the
    feed-forward.  Whole prompt against a plain computation (which differs from the same without
    rotation), then portions and single tokens against the whole."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part
    from swifttransformer_amd.weights import random_tensors
    register_part("position", "toy_rotary", ToyRotary)
    register_part("norm", "toy_scale", ToyScaleNorm)
    H, V, Pmax, nh, hd = 64, 89, 96, 2, 32
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    attn = PartSpec("paged_attention", {"num_heads": nh, "head_dim": hd, "scale": hd ** -0.5, "bias": False},
                    {f"{n}.weight": f"l0.{n}" for n in ("q", "k", "v", "out")})
    ffn = PartSpec("dense", {"inner": 80, "activation": "relu", "bias": False},
                   {"fc1.weight": "l0.fc1", "fc2.weight": "l0.fc2"})
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("toy_rotary", {"head_dim": hd, "theta": 100.0}),
                     layers=[LayerSpec(PartSpec("pre_norm"), norm("l0.n1"), attn,
                                       PartSpec("toy_scale", {"eps": 1e-4}, {"gain": "l0.n2.g"}), ffn)],
                     schedule=[ScheduleEntry(0, 0)], final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    tensors = random_tensors(model.tensor_specs(), 11, dtype, DEV)
    # with the small random weights every score is near 0 and the softmax near uniform, whatever
    # is done to queries and keys: larger ones make the scores, and so the rotation, count
    for n in ("l0.q", "l0.k"):
        tensors[n] = (tensors[n].float() * 12).to(dtype)
    model.bind(tensors)
    w = {k: v.double().cpu() for k, v in tensors.items()}
    toks = torch.randint(0, V, (41,), generator=torch.Generator().manual_seed(4)).tolist()

    def plain(rotating):
        rot = ToyRotary(spec.position, H, dtype)
        x = w["tok"][toks]
        a = P.layer_norm(x, w["l0.n1.g"], w["l0.n1.b"], 1e-5)
        q, k, v = (a @ w[f"l0.{n}"].T for n in "qkv")
        if rotating:
            pos = torch.arange(len(toks))
            q, k = rot.turn(q, pos), rot.turn(k, pos)
        heads = [P.causal_attention(q[:, h * hd:(h + 1) * hd], k[:, h * hd:(h + 1) * hd],
                                    v[:, h * hd:(h + 1) * hd], hd ** -0.5) for h in range(nh)]
        r = x + torch.cat(heads, 1) @ w["l0.out"].T
        d = ToyScaleNorm.compute(r, w["l0.n2.g"], 1e-4)
        y = r + torch.relu(d @ w["l0.fc1"].T) @ w["l0.fc2"].T
        return P.layer_norm(y, w["fn.g"], w["fn.b"], 1e-5) @ w["tok"].T

    ref = plain(True)
    assert (ref - plain(False)).abs().max() > 0.05 * ref.std()     # the rotation is no side issue
    runner = ModelRunner(model, CacheParam(page_size=4, num_pages=30, max_seqs=2), DEV, cache_fill=float("nan"))
    runner.admit("w")
    check(runner.step([StepEntry("w", toks, list(range(len(toks))))]), ref, dtype, "rotating positions, whole")
    runner.admit("c")
    p, got = 0, []
    for c in (9, 2, 13, 1, 1, 1, 14):
        got.append(runner.step([StepEntry("c", toks[p:p + c], list(range(c)))]).clone())
        p += c
    check(torch.cat(got), ref, dtype, "rotating positions, portions and single tokens")
    runner.finish("w"), runner.finish("c")
    runner.manager.check_invariants()


class ToyDistanceBias:
    """A toy position encoding that adds nothing to the embedding and turns nothing: head h's
    score of (query at p, key at j) gets -steepness / (h + 1) * (p - j) added."""
    rotates = False
    biases_scores = True

    def __init__(self, spec, hidden_size, dtype):
        self.steepness = float(spec.params["steepness"])
        self._slopes = {}

    def tensor_specs(self):
        return []

    def bind(self, tensors):
        pass

    def embedding_addend(self, ctx):
        return None

    def slopes(self, num_heads):
        return torch.tensor([self.steepness / (h + 1) for h in range(num_heads)], dtype=torch.float32)

    def score_slopes(self, num_heads):
        if num_heads not in self._slopes:
            self._slopes[num_heads] = self.slopes(num_heads).to(DEV)
        return self._slopes[num_heads]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_toy_position_encoding_that_biases_scores(dtype):
    """A position encoding of a third kind (neither added to the embedding nor a rotation): a bias
    on the attention scores that grows with the distance, a slope a head.  Registered from here,
    it reaches the prompt tiles, the decode rows and the recorded decode step through the mixer's
    hook alone; compared with a plain model, whole, in portions and decoded one by one."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part
    from swifttransformer_amd.weights import random_tensors
    register_part("position", "toy_distance_bias", ToyDistanceBias)
    H, V, Pmax, nh, hd = 64, 97, 200, 4, 16
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    attn = PartSpec("paged_attention", {"num_heads": nh, "head_dim": hd, "scale": hd ** -0.5, "bias": False},
                    {f"{n}.weight": f"l0.{n}" for n in ("q", "k", "v", "out")})
    ffn = PartSpec("dense", {"inner": 80, "activation": "relu", "bias": False},
                   {"fc1.weight": "l0.fc1", "fc2.weight": "l0.fc2"})
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("toy_distance_bias", {"steepness": 0.3}),
                     layers=[LayerSpec(PartSpec("pre_norm"), norm("l0.n1"), attn, norm("l0.n2"), ffn)],
                     schedule=[ScheduleEntry(0, 0)], final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    tensors = random_tensors(model.tensor_specs(), 13, dtype, DEV)
    for n in ("l0.q", "l0.k"):               # scores that matter beside the bias
        tensors[n] = (tensors[n].float() * 8).to(dtype)
    model.bind(tensors)
    w = {k: v.double().cpu() for k, v in tensors.items()}
    toks = torch.randint(0, V, (150,), generator=torch.Generator().manual_seed(6)).tolist()
    n = len(toks)

    def plain(steepness):
        x = w["tok"][toks]
        a = P.layer_norm(x, w["l0.n1.g"], w["l0.n1.b"], 1e-5)
        q, k, v = (a @ w[f"l0.{m}"].T for m in "qkv")
        pos = torch.arange(n, dtype=torch.float64)
        dist = pos[None, :] - pos[:, None]                       # key position - query position
        heads = []
        for h in range(nh):
            sl = slice(h * hd, (h + 1) * hd)
            s = (q[:, sl] @ k[:, sl].T) * hd ** -0.5 + steepness / (h + 1) * dist
            s = s.masked_fill(dist > 0, float("-inf"))
            heads.append(torch.softmax(s, -1) @ v[:, sl])
        r = x + torch.cat(heads, 1) @ w["l0.out"].T
        d = P.layer_norm(r, w["l0.n2.g"], w["l0.n2.b"], 1e-5)
        y = r + torch.relu(d @ w["l0.fc1"].T) @ w["l0.fc2"].T
        return P.layer_norm(y, w["fn.g"], w["fn.b"], 1e-5) @ w["tok"].T

    ref = plain(0.3)
    assert (ref - plain(0.0)).abs().max() > 0.05 * ref.std()       # the bias is no side issue
    runner = ModelRunner(model, CacheParam(page_size=4, num_pages=90, max_seqs=2), DEV, cache_fill=float("nan"))
    runner.admit("w")
    check(runner.step([StepEntry("w", toks, list(range(n)))]), ref, dtype, "score bias, whole")
    runner.admit("c")
    p, got = 0, []
    cuts = [9, 2, 70, 1, 1, 1, 30] + [1] * 36
    assert sum(cuts) == n
    replays = runner.graph_replays
    for c in cuts:
        got.append(runner.step([StepEntry("c", toks[p:p + c], list(range(c)))]).clone())
        p += c
    check(torch.cat(got), ref, dtype, "score bias, portions and single tokens")
    assert runner.graph_replays > replays, "no decode step of this test was a recorded one"
    runner.finish("w"), runner.finish("c")
    runner.manager.check_invariants()


class ToyRoutedFeedForward:
    """A toy feed-forward with routing: a router picks one of a few small ReLU experts per token
    (router logits in float); written with library tensor operations, as a part outside the
    package may be."""

    def __init__(self, spec, hidden_size, dtype):
        self.spec, self.hidden_size, self.dtype = spec, hidden_size, dtype
        self.experts, self.inner = int(spec.params["experts"]), int(spec.params["inner"])

    def tensor_specs(self):
        from swifttransformer_amd.weights import TensorSpec
        n, H = self.spec.names, self.hidden_size
        return [TensorSpec(n["router"], (self.experts, H), "matrix"),
                TensorSpec(n["up"], (self.experts * self.inner, H), "matrix"),
                TensorSpec(n["down"], (self.experts * H, self.inner), "matrix")]

    def bind(self, tensors):
        n = self.spec.names
        self.router = tensors[n["router"]].float()
        self.up = tensors[n["up"]].float().view(self.experts, self.inner, self.hidden_size)
        self.down = tensors[n["down"]].float().view(self.experts, self.hidden_size, self.inner)

    @staticmethod
    def compute(x, router, up, down):
        choice = (x @ router.T).argmax(-1)                         # [T]
        hidden = torch.relu(torch.einsum("th,tih->ti", x, up[choice]))
        return torch.einsum("ti,thi->th", hidden, down[choice]), choice

    def forward(self, x_t, residual32, ctx):
        y, _ = self.compute(x_t.float(), self.router, self.up, self.down)
        return residual32 + y


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_feed_forward_with_routing(dtype):
    """A feed-forward with routing, defined here, takes the place of the dense one in one layer of
    a two-layer model (the other keeps the dense one): built from a spec, stepped whole and in
    portions, compared with a plain computation."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part
    from swifttransformer_amd.weights import random_tensors
    register_part("feed_forward", "toy_routed", ToyRoutedFeedForward)
    H, V, Pmax, nh, hd, E, inner = 64, 101, 64, 4, 16, 3, 24
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    attn = lambda i: PartSpec("paged_attention", {"num_heads": nh, "head_dim": hd, "scale": hd ** -0.5, "bias": False},
                              {f"{n}.weight": f"l{i}.{n}" for n in ("q", "k", "v", "out")})
    routed = PartSpec("toy_routed", {"experts": E, "inner": inner},
                      {"router": "l0.router", "up": "l0.up", "down": "l0.down"})
    dense = PartSpec("dense", {"inner": 96, "activation": "relu", "bias": False},
                     {"fc1.weight": "l1.fc1", "fc2.weight": "l1.fc2"})
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("learned", {"max_positions": Pmax, "offset": 0}, {"weight": "pos"}),
                     layers=[LayerSpec(PartSpec("pre_norm"), norm("l0.n1"), attn(0), norm("l0.n2"), routed),
                             LayerSpec(PartSpec("pre_norm"), norm("l1.n1"), attn(1), norm("l1.n2"), dense)],
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1)], final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    tensors = random_tensors(model.tensor_specs(), 21, dtype, DEV)
    tensors["l0.router"] = (tensors["l0.router"].float() * 50).to(dtype)      # clear choices, no near-ties
    model.bind(tensors)
    w = {k: v.double().cpu() for k, v in tensors.items()}
    toks = torch.randint(0, V, (33,), generator=torch.Generator().manual_seed(6)).tolist()

    x = w["tok"][toks] + w["pos"][:len(toks)]
    choices = None
    for i in range(2):
        a = P.layer_norm(x, w[f"l{i}.n1.g"], w[f"l{i}.n1.b"], 1e-5)
        q, k, v = (a @ w[f"l{i}.{n}"].T for n in "qkv")
        heads = [P.causal_attention(q[:, h * hd:(h + 1) * hd], k[:, h * hd:(h + 1) * hd],
                                    v[:, h * hd:(h + 1) * hd], hd ** -0.5) for h in range(nh)]
        r = x + torch.cat(heads, 1) @ w[f"l{i}.out"].T
        d = P.layer_norm(r, w[f"l{i}.n2.g"], w[f"l{i}.n2.b"], 1e-5)
        if i == 0:
            y, choices = ToyRoutedFeedForward.compute(d, w["l0.router"], w["l0.up"].view(E, inner, H),
                                                      w["l0.down"].view(E, H, inner))
        else:
            y = torch.relu(d @ w["l1.fc1"].T) @ w["l1.fc2"].T
        x = r + y
    ref = P.layer_norm(x, w["fn.g"], w["fn.b"], 1e-5) @ w["tok"].T
    assert len(set(choices.tolist())) == E                     # every expert is used

    runner = ModelRunner(model, CacheParam(page_size=8, num_pages=20, max_seqs=2), DEV)
    runner.admit("w")
    check(runner.step([StepEntry("w", toks, list(range(len(toks))))]), ref, dtype, "routed feed-forward, whole")
    runner.admit("c")
    p, got = 0, []
    for c in (4, 11, 1, 1, 16):
        got.append(runner.step([StepEntry("c", toks[p:p + c], list(range(c)))]).clone())
        p += c
    check(torch.cat(got), ref, dtype, "routed feed-forward, portions")
    runner.manager.check_invariants()


class ToyGatedFeedForward:
    """A toy gated feed-forward, y = (silu(x Wg^T) * (x Wu^T)) Wd^T, written from outside the package
    with its kernels: one product for gate and up, the elementwise activation-and-multiply on the
    two halves of its output, one product with the residual sum."""

    def __init__(self, spec, hidden_size, dtype):
        self.spec, self.hidden_size, self.dtype = spec, hidden_size, dtype
        self.inner = int(spec.params["inner"])
        self.activation = str(spec.params.get("activation", "silu"))

    def tensor_specs(self):
        from swifttransformer_amd.weights import TensorSpec
        n, H = self.spec.names, self.hidden_size
        return [TensorSpec(n["gate"], (self.inner, H), "matrix"), TensorSpec(n["up"], (self.inner, H), "matrix"),
                TensorSpec(n["down"], (H, self.inner), "matrix")]

    def bind(self, tensors):
        n = self.spec.names
        self.w_gate_up = torch.cat([tensors[n["gate"]], tensors[n["up"]]], 0).contiguous()
        self.w_down = tensors[n["down"]]

    def forward(self, x_t, residual32, ctx):
        from swifttransformer_amd.ops import kernels as K
        both = K.gemm(x_t, self.w_gate_up)
        gated = K.activation_multiply(both[:, :self.inner], both[:, self.inner:], self.activation)
        return K.gemm(gated, self.w_down, residual=residual32, out_f32=True)


def _gated_model(dtype, seed=23):
    """Two layers: the toy gated feed-forward in the first, the dense one with the tanh-form GELU
    in the second (a function the products' epilogues have and OPT does not use)."""
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part
    from swifttransformer_amd.weights import random_tensors
    register_part("feed_forward", "toy_gated", ToyGatedFeedForward)
    H, V, Pmax, nh, hd, inner = 80, 131, 96, 5, 16, 56
    norm = lambda n: PartSpec("layer_norm", {"eps": 1e-5, "affine": True}, {"weight": f"{n}.g", "bias": f"{n}.b"})
    attn = lambda i: PartSpec("paged_attention", {"num_heads": nh, "head_dim": hd, "scale": hd ** -0.5, "bias": False},
                              {f"{n}.weight": f"l{i}.{n}" for n in ("q", "k", "v", "out")})
    gated = PartSpec("toy_gated", {"inner": inner, "activation": "silu"},
                     {"gate": "l0.gate", "up": "l0.up", "down": "l0.down"})
    dense = PartSpec("dense", {"inner": 112, "activation": "gelu_tanh", "bias": True},
                     {f"{n}.{t}": f"l1.{n}.{t}" for n in ("fc1", "fc2") for t in ("weight", "bias")})
    spec = ModelSpec(hidden_size=H, vocab_size=V, max_positions=Pmax,
                     embedding=PartSpec("token", {"vocab_size": V, "embed_dim": H}, {"weight": "tok"}),
                     position=PartSpec("learned", {"max_positions": Pmax, "offset": 0}, {"weight": "pos"}),
                     layers=[LayerSpec(PartSpec("pre_norm"), norm("l0.n1"), attn(0), norm("l0.n2"), gated),
                             LayerSpec(PartSpec("pre_norm"), norm("l1.n1"), attn(1), norm("l1.n2"), dense)],
                     schedule=[ScheduleEntry(0, 0), ScheduleEntry(1, 1)], final_norm=norm("fn"),
                     head=PartSpec("linear", {"vocab_size": V, "embed_dim": H, "tied_to": "tok"}, {"weight": "lm"}))
    model = DecoderModel(spec, dtype)
    tensors = random_tensors(model.tensor_specs(), seed, dtype, DEV)
    for name in ("l0.gate", "l0.up", "l0.down", "l1.fc1.weight", "l1.fc2.weight"):
        tensors[name] = (tensors[name].float() * 8).to(dtype)       # feed-forwards that matter to the logits
    model.bind(tensors)
    w = {k: v.double().cpu() for k, v in tensors.items()}

    def plain(toks):
        x = w["tok"][toks] + w["pos"][:len(toks)]
        for i in range(2):
            a = P.layer_norm(x, w[f"l{i}.n1.g"], w[f"l{i}.n1.b"], 1e-5)
            q, k, v = (a @ w[f"l{i}.{n}"].T for n in "qkv")
            heads = [P.causal_attention(q[:, h * hd:(h + 1) * hd], k[:, h * hd:(h + 1) * hd],
                                        v[:, h * hd:(h + 1) * hd], hd ** -0.5) for h in range(nh)]
            r = x + torch.cat(heads, 1) @ w[f"l{i}.out"].T
            d = P.layer_norm(r, w[f"l{i}.n2.g"], w[f"l{i}.n2.b"], 1e-5)
            if i == 0:
                g = d @ w["l0.gate"].T
                y = ((g / (1 + torch.exp(-g))) * (d @ w["l0.up"].T)) @ w["l0.down"].T
            else:
                h1 = d @ w["l1.fc1.weight"].T + w["l1.fc1.bias"]
                h1 = 0.5 * h1 * (1 + torch.tanh(0.7978845608028654 * (h1 + 0.044715 * h1 ** 3)))
                y = h1 @ w["l1.fc2.weight"].T + w["l1.fc2.bias"]
            x = r + y
        return P.layer_norm(x, w["fn.g"], w["fn.b"], 1e-5) @ w["tok"].T
    return model, plain, V


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_gated_feed_forward_and_another_activation(dtype):
    """A gated feed-forward defined here (SiLU gate through the package's elementwise kernel) and
    a dense one with another activation than the architecture's own run whole, in portions, as
    recorded decode steps and through ``Engine.generate``, with no change to the package."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.sampling import SamplingParams
    model, plain, V = _gated_model(dtype)
    toks = torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(8)).tolist()
    ref = plain(toks)
    # the two feed-forwards carry weight in the logits: without them the comparison would not see them
    runner = ModelRunner(model, CacheParam(page_size=8, num_pages=24, max_seqs=2), DEV)
    runner.admit("w")
    check(runner.step([StepEntry("w", toks, list(range(len(toks))))]), ref, dtype, "gated feed-forward, whole")
    runner.admit("c")
    p, got = 0, []
    for c in (13, 2, 17, 1, 1, 1, 1, 1, 1, 1, 1):        # 13 and 17 rows: the library's products; then decode steps
        got.append(runner.step([StepEntry("c", toks[p:p + c], list(range(c)))]).clone())
        p += c
    check(torch.cat(got), ref[:p], dtype, "gated feed-forward, portions and decode steps")
    assert runner.graph_replays >= 6
    runner.finish("w"), runner.finish("c")
    if dtype != torch.float32:
        return
    eng = Engine(model, dtype=dtype, page_size=8, num_pages=24, max_seqs=2)
    prompt = toks[:9]
    out = eng.generate([prompt], SamplingParams(max_new_tokens=6, ignore_eos=True))[0]
    seq = list(prompt)
    for t in out:
        assert t == int(plain(seq)[-1].argmax())
        seq.append(t)
