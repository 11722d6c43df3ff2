"""What pins the plain implementation besides the reference's text: library routines it
must reduce to in special cases, and invariants a wrong sign, pairing or norm placement
would break (CPU)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_opt as P
import tiny

torch.manual_seed(0)


def _model(name, tmp_path, seed=0):
    d = tiny.write_model(name, str(tmp_path), seed=seed)
    return P.load_folder(d)


def test_layer_norm_is_the_library_routine():
    # the reference's own test compares with torch::layer_norm (src/unittest/kernel/layernorm.cc:48)
    x = torch.randn(7, 96, dtype=P.DT) * 3 + 1
    g, b = torch.rand(96, dtype=P.DT), torch.rand(96, dtype=P.DT)
    assert torch.allclose(P.layer_norm(x, g, b, 1e-4), F.layer_norm(x, (96,), g, b, 1e-4), atol=1e-12)
    y = P.layer_norm(x, None, None, 1e-5)
    assert torch.allclose(y.mean(-1), torch.zeros(7, dtype=P.DT), atol=1e-12)
    var = x.var(-1, unbiased=False)
    assert torch.allclose(y.var(-1, unbiased=False), var / (var + 1e-5), atol=1e-9)
    const = torch.full((1, 96), 3.25, dtype=P.DT)
    assert torch.allclose(P.layer_norm(const, g, b, 1e-5), b.unsqueeze(0), atol=1e-9)


def test_embedding_uses_rows_after_the_offset():
    tok = torch.randn(50, 8, dtype=P.DT)
    pos = torch.randn(12, 8, dtype=P.DT)
    ids, ps = [3, 7, 7, 49], [0, 1, 2, 9]
    want = F.embedding(torch.tensor(ids), tok) + F.embedding(torch.tensor(ps) + 2, pos)
    assert torch.equal(P.embed(ids, ps, tok, pos, 2, None), want)
    poisoned = pos.clone()
    poisoned[:2] = float("nan")     # the rows the reference's converter drops (converter_lib.py:271)
    assert torch.equal(P.embed(ids, ps, tok, poisoned, 2, None), want)
    # identity projection changes nothing
    assert torch.allclose(P.embed(ids, ps, tok, pos, 2, torch.eye(8, dtype=P.DT)), want)


def test_causal_attention_is_the_library_routine():
    n, hd = 13, 16
    q, k, v = (torch.randn(n, hd, dtype=P.DT) for _ in range(3))
    scale = 1 / math.sqrt(hd)
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, scale=scale)[0]
    assert torch.allclose(P.causal_attention(q, k, v, scale), want, atol=1e-12)
    # zero queries: uniform weights, row i is the mean of v[0..i]
    uni = P.causal_attention(torch.zeros_like(q), k, v, scale)
    means = torch.cumsum(v, 0) / torch.arange(1, n + 1, dtype=P.DT)[:, None]
    assert torch.allclose(uni, means, atol=1e-12)
    assert torch.allclose(P.causal_attention(q[:1], k[:1], v[:1], scale), v[:1])
    # a wrong scale or a missing mask must show
    assert not torch.allclose(P.causal_attention(q, k, v, 1.0), want, atol=1e-6)


def test_attention_layer_split_and_heads(tmp_path):
    cfg, w = _model("A", tmp_path)
    pre = "model.decoder.layers.0"
    H, nh = cfg["hidden_size"], cfg["num_attention_heads"]
    a = torch.randn(9, H, dtype=P.DT)
    # library formulation over all heads at once
    def lin(n):
        return F.linear(a, w[f"{pre}.self_attn.{n}_proj.weight"], w[f"{pre}.self_attn.{n}_proj.bias"])
    q, k, v = (lin(n).view(9, nh, H // nh).transpose(0, 1) for n in "qkv")
    o = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=(H // nh) ** -0.5)
    want = F.linear(o.transpose(0, 1).reshape(9, H), w[f"{pre}.self_attn.out_proj.weight"],
                    w[f"{pre}.self_attn.out_proj.bias"])
    assert torch.allclose(P.attention_layer(a, w, pre, nh, True), want, atol=1e-12)
    # one head over the whole width is a different function (head pairing matters)
    assert not torch.allclose(P.attention_layer(a, w, pre, 1, True), want, atol=1e-6)
    # only the value path non-zero in q/k: uniform attention, so the output is out(mean of v) + b
    w2 = dict(w)
    for n in "qk":
        w2[f"{pre}.self_attn.{n}_proj.weight"] = torch.zeros_like(w[f"{pre}.self_attn.{n}_proj.weight"])
        w2[f"{pre}.self_attn.{n}_proj.bias"] = torch.zeros_like(w[f"{pre}.self_attn.{n}_proj.bias"])
    vv = F.linear(a, w[f"{pre}.self_attn.v_proj.weight"], w[f"{pre}.self_attn.v_proj.bias"])
    means = torch.cumsum(vv, 0) / torch.arange(1, 10, dtype=P.DT)[:, None]
    want2 = F.linear(means, w[f"{pre}.self_attn.out_proj.weight"], w[f"{pre}.self_attn.out_proj.bias"])
    assert torch.allclose(P.attention_layer(a, w2, pre, nh, True), want2, atol=1e-12)


def test_feed_forward_is_the_library_routine(tmp_path):
    cfg, w = _model("A", tmp_path)
    pre = "model.decoder.layers.1"
    d = torch.randn(5, cfg["hidden_size"], dtype=P.DT)
    # src/unittest/layer/parallel_ffn.cc:161-162
    want = F.linear(F.relu(F.linear(d, w[f"{pre}.fc1.weight"], w[f"{pre}.fc1.bias"])),
                    w[f"{pre}.fc2.weight"], w[f"{pre}.fc2.bias"])
    assert torch.allclose(P.feed_forward(d, w, pre, True), want, atol=1e-12)
    w2 = dict(w)
    w2[f"{pre}.fc1.bias"] = torch.full_like(w[f"{pre}.fc1.bias"], -100.0)   # nothing passes the ReLU
    assert torch.allclose(P.feed_forward(d, w2, pre, True), w[f"{pre}.fc2.bias"].expand(5, -1), atol=1e-12)


@pytest.mark.parametrize("name", ["A", "B"])
def test_block_wiring_closed_form(tmp_path, name):
    """With the output matrices of mixer and feed-forward zeroed, a pre-norm block is the
    identity and a post-norm block a chain of two LayerNorms."""
    cfg, w = _model(name, tmp_path)
    w = dict(w)
    L = cfg["num_hidden_layers"]
    for i in range(L):
        p = f"model.decoder.layers.{i}"
        for n in (f"{p}.self_attn.out_proj.weight", f"{p}.fc2.weight", f"{p}.self_attn.out_proj.bias",
                  f"{p}.fc2.bias"):
            if n in w:
                w[n] = torch.zeros_like(w[n])
    toks = tiny.prompt(11, cfg["vocab_size"], 1)
    H, E = cfg["hidden_size"], cfg["word_embed_proj_dim"]
    dec = "model.decoder"
    x = P.embed(toks, range(11), w[f"{dec}.embed_tokens.weight"], w[f"{dec}.embed_positions.weight"], 2,
                w.get(f"{dec}.project_in.weight") if E != H else None)
    if cfg["do_layer_norm_before"]:
        x = F.layer_norm(x, (H,), w[f"{dec}.final_layer_norm.weight"], w[f"{dec}.final_layer_norm.bias"], 1e-5)
    else:
        for i in range(L):
            p = f"{dec}.layers.{i}"
            x = F.layer_norm(x, (H,), w[f"{p}.self_attn_layer_norm.weight"], w[f"{p}.self_attn_layer_norm.bias"], 1e-5)
            x = F.layer_norm(x, (H,), w[f"{p}.final_layer_norm.weight"], w[f"{p}.final_layer_norm.bias"], 1e-5)
    if E != H:
        x = F.linear(x, w[f"{dec}.project_out.weight"])
    want = F.linear(x, w[f"{dec}.embed_tokens.weight"])
    assert torch.allclose(P.forward(cfg, w, toks), want, atol=1e-10)


def _diagonal_block(H=8, heads=2, seed=3):
    """Weights of one block whose mixer and feed-forward are known diagonal maps on a one-token
    sequence: attention of a single token returns its value row, so with Wv = diag(d), Wo = I the
    mixer is x -> d*x; with W1 = I, b1 = 10 (keeps the ReLU linear for normalised inputs),
    W2 = diag(e), b2 = -10 e the feed-forward is x -> e*x."""
    g = torch.Generator().manual_seed(seed)
    d = torch.rand(H, generator=g, dtype=torch.float64) + 0.5
    e = torch.rand(H, generator=g, dtype=torch.float64) * 2 - 1
    p = "blk"
    w = {f"{p}.self_attn.q_proj.weight": torch.randn(H, H, generator=g, dtype=torch.float64),
         f"{p}.self_attn.k_proj.weight": torch.randn(H, H, generator=g, dtype=torch.float64),
         f"{p}.self_attn.v_proj.weight": torch.diag(d), f"{p}.self_attn.out_proj.weight": torch.eye(H, dtype=torch.float64),
         f"{p}.fc1.weight": torch.eye(H, dtype=torch.float64), f"{p}.fc1.bias": torch.full((H,), 10.0, dtype=torch.float64),
         f"{p}.fc2.weight": torch.diag(e), f"{p}.fc2.bias": -10.0 * e}
    for n in ("q", "k", "v", "out"):
        w[f"{p}.self_attn.{n}_proj.bias"] = torch.zeros(H, dtype=torch.float64)
    for n in ("self_attn_layer_norm", "final_layer_norm"):
        w[f"{p}.{n}.weight"] = torch.rand(H, generator=g, dtype=torch.float64) + 0.5
        w[f"{p}.{n}.bias"] = torch.randn(H, generator=g, dtype=torch.float64) * 0.1
    cfg = {"hidden_size": H, "num_attention_heads": heads, "enable_bias": True, "layer_norm_eps": 1e-5}
    x = torch.randn(1, H, generator=g, dtype=torch.float64) * 2 + 0.3
    return cfg, w, p, d, e, x


def test_what_the_parts_of_a_block_read():
    """Which vector the mixer and the feed-forward read, and where the norms sit, in closed form
    with diagonal parts (zeroed parts, as in test_block_wiring_closed_form, cannot see their
    inputs).  Post-norm: both read the un-normed stream and each sum is normalised afterwards;
    pre-norm: both read the normalised stream and add to the un-normed one."""
    cfg, w, p, d, e, x = _diagonal_block()
    H = cfg["hidden_size"]
    n1 = lambda v: F.layer_norm(v, (H,), w[f"{p}.self_attn_layer_norm.weight"], w[f"{p}.self_attn_layer_norm.bias"], 1e-5)
    n2 = lambda v: F.layer_norm(v, (H,), w[f"{p}.final_layer_norm.weight"], w[f"{p}.final_layer_norm.bias"], 1e-5)
    # post-norm
    r = n1(x + d * x)
    want_post = n2(r + e * r)
    got_post = P.block_post_norm(x, w, p, cfg)
    assert torch.allclose(got_post, want_post, atol=1e-12)
    # plausible mistakes give other vectors: the mixer reading the normalised input; the feed-forward
    # reading the un-normed sum; the pre-norm wiring
    s = x + d * x
    for wrong in (n2(n1(x + d * n1(x)) * (1 + e)), n2(n1(s) + e * s)):
        assert not torch.allclose(wrong, want_post, atol=1e-4)
    # pre-norm
    r = x + d * n1(x)
    want_pre = r + e * n2(r)
    got_pre = P.block_pre_norm(x, w, p, cfg)
    assert torch.allclose(got_pre, want_pre, atol=1e-12)
    assert not torch.allclose(want_pre, want_post, atol=1e-4)
    assert not torch.allclose(x + d * x + e * n2(x + d * x), want_pre, atol=1e-4)     # mixer reading x un-normed


def test_order_of_projections_is_fixed_by_the_tensor_shapes():
    """With an embedding width E different from the hidden width H, the model's tensors leave one
    order only: position rows are H wide, so they are added after project_in [H, E]; the final
    norm is H wide, so it acts before project_out [E, H]; the head reads E wide rows, so it comes
    last.  Any other order does not type-check, in the plain model as in the engine."""
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.models.decoder import DecoderModel
    from swifttransformer_amd.models.opt import build_opt_spec
    hp = OptHyperParam(vocab_size=50, max_position_embeddings=20, hidden_size=32, num_hidden_layers=1,
                       num_attention_heads=2, ffn_dim=40, word_embed_proj_dim=24, do_layer_norm_before=True).validate()
    shapes = {s.name: tuple(s.shape) for s in DecoderModel(build_opt_spec(hp), torch.float32).tensor_specs()}
    dec = "model.decoder"
    assert shapes[f"{dec}.embed_tokens.weight"] == (50, 24)
    assert shapes[f"{dec}.project_in.weight"] == (32, 24)
    assert shapes[f"{dec}.embed_positions.weight"] == (22, 32)
    assert shapes[f"{dec}.final_layer_norm.weight"] == (32,)
    assert shapes[f"{dec}.project_out.weight"] == (24, 32)
    assert shapes["lm_head.weight"] == (50, 24)
    # and the plain model follows that order: with project_in = [I; 0] and project_out its transpose
    # the logits are those of positions added to the padded token vector
    g = torch.Generator().manual_seed(0)
    tok = torch.randn(50, 24, generator=g, dtype=torch.float64)
    pos = torch.randn(22, 32, generator=g, dtype=torch.float64)
    pin = torch.zeros(32, 24, dtype=torch.float64)
    pin[:24] = torch.eye(24, dtype=torch.float64)
    x = P.embed([3, 7], [0, 1], tok, pos, 2, pin)
    want = torch.cat([tok[[3, 7]], torch.zeros(2, 8, dtype=torch.float64)], 1) + pos[[2, 3]]
    assert torch.allclose(x, want)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_causality_and_prefix_invariance(tmp_path, name):
    cfg, w = _model(name, tmp_path)
    toks = tiny.prompt(24, cfg["vocab_size"], 2)
    full = P.forward(cfg, w, toks)
    changed = list(toks)
    changed[15] = (changed[15] + 1) % cfg["vocab_size"]
    other = P.forward(cfg, w, changed)
    assert torch.allclose(full[:15], other[:15], atol=1e-12)       # later tokens never reach back
    assert not torch.allclose(full[15:], other[15:], atol=1e-6)
    assert torch.allclose(P.forward(cfg, w, toks[:10]), full[:10], atol=1e-12)


def test_positions_matter(tmp_path):
    """Learned absolute positions: the same token at another position gives other logits."""
    cfg, w = _model("A", tmp_path)
    a = P.forward(cfg, w, [5, 9, 9])
    assert not torch.allclose(a[1], a[2], atol=1e-6)


def test_sampler_noise_distribution():
    """Gumbel-max with the hash noise samples softmax(logits / t): chi-square over many seeds."""
    logits = np.array([0.0, 1.0, -1.0, 2.0, 0.5, 0.5, -3.0, 1.5, 0.2, -0.4, 0.9, 1.1, -2.0, 0.0, 0.3, 0.7])
    t = 0.8
    p = np.exp(logits / t - (logits / t).max())
    p /= p.sum()
    n = 4000
    counts = np.zeros(16)
    for seed in range(n):
        counts[P.choose(logits, t, seed, seed % 7)] += 1
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 45.0, chi2      # 15 degrees of freedom: P(chi2 > 45) < 1e-4
    u = P.hash_uniform(12345, 3, 1000)
    assert 0 < u.min() and u.max() < 1 and abs(u.mean() - 0.5) < 0.05
    assert P.choose(logits, 0.0, 1, 1) == 3
