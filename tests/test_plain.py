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
