"""A plain, slow OPT: whole sequences, no cache, one function per part, float64.

Written from the reference's formulas (file:line of the reference's tree in each
function); it shares no code with the engine.  It reads a model folder with the
``safetensors`` package and ``json`` and returns the logits of every position.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch
from safetensors.torch import load_file

DT = torch.float64


def load_folder(model_dir: str):
    """config.json as a dict and every tensor of model.safetensors as float64."""
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
        cfg = json.load(f)
    raw = load_file(os.path.join(model_dir, "model.safetensors"))
    w = {}
    for k, v in raw.items():
        if not k.startswith("model.") and k != "lm_head.weight":
            k = "model." + k
        w[k] = v.to(DT)
    return cfg, w


# ------------------------------------------------------------------------ parts
def layer_norm(x: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
               eps: float) -> torch.Tensor:
    """y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last dimension, var = E[x^2] - mean^2
    (src/csrc/kernel/layernorm.cu:35-51 sums, :77-82 mean and rsqrt, :86-97 normalise)."""
    mean = x.sum(-1, keepdim=True) / x.shape[-1]
    var = (x * x).sum(-1, keepdim=True) / x.shape[-1] - mean * mean
    y = (x - mean) * torch.rsqrt(var + eps)
    if gamma is not None:
        y = y * gamma
    if beta is not None:
        y = y + beta
    return y


def embed(token_ids: Sequence[int], positions: Sequence[int], tok_table: torch.Tensor,
          pos_table: torch.Tensor, offset: int, project_in: Optional[torch.Tensor]) -> torch.Tensor:
    """x0[t] = Etok[id[t]] + Epos'[pos[t]] (src/csrc/kernel/embedding.cu:25-35) where Epos' is the
    stored table without its first `offset` rows (scripts/lib/converter_lib.py:271), i.e. row
    pos + offset of the stored table; pos[t] = first index + j (src/csrc/model/gpt/gpt.cc:92-102).
    With an input projection the token vector is projected (no bias) before the position is added."""
    tok = tok_table[torch.as_tensor(list(token_ids), dtype=torch.long)]
    if project_in is not None:
        tok = tok @ project_in.T
    pos = pos_table[torch.as_tensor(list(positions), dtype=torch.long) + offset]
    return tok + pos


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """One head, whole sequence: S = q k^T * scale, positions j > i masked, softmax over j, P v
    (oracle src/unittest/kernel/attention_ref.cc:68-84; kernel
    src/csrc/kernel/fused_context_stage_attention.cu:226-293).  The reference masks by adding
    -10000 (:287-291), which underflows to zero weight after the softmax; -inf is used here."""
    n = q.shape[0]
    s = (q @ k.T) * scale
    mask = torch.triu(torch.ones(n, n, dtype=torch.bool), diagonal=1)
    s = s.masked_fill(mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return p @ v


def attention_layer(a: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, num_heads: int,
                    bias: bool) -> torch.Tensor:
    """qkv = a W^T + b split per head (src/csrc/layer/attention.cc:102-130; q heads, then k, then v),
    per-head causal attention with scale 1/sqrt(head_dim) (:91), concatenated heads times the
    output matrix plus bias (:255-264, :279-288)."""
    n, H = a.shape
    hd = H // num_heads

    def lin(name):
        y = a @ w[f"{prefix}.self_attn.{name}_proj.weight"].T
        if bias:
            y = y + w[f"{prefix}.self_attn.{name}_proj.bias"]
        return y

    q, k, v = lin("q"), lin("k"), lin("v")
    heads = []
    for h in range(num_heads):
        sl = slice(h * hd, (h + 1) * hd)
        heads.append(causal_attention(q[:, sl], k[:, sl], v[:, sl], 1.0 / math.sqrt(hd)))
    o = torch.cat(heads, dim=-1)
    y = o @ w[f"{prefix}.self_attn.out_proj.weight"].T
    if bias:
        y = y + w[f"{prefix}.self_attn.out_proj.bias"]
    return y


def feed_forward(d: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, bias: bool) -> torch.Tensor:
    """y = relu(d W1^T + b1) W2^T + b2 (src/csrc/layer/ffn.cc:71-80, :85-92, :96-105, :124;
    ReLU src/csrc/kernel/activations.cuh:12-13)."""
    h = d @ w[f"{prefix}.fc1.weight"].T
    if bias:
        h = h + w[f"{prefix}.fc1.bias"]
    h = torch.clamp_min(h, 0.0)
    y = h @ w[f"{prefix}.fc2.weight"].T
    if bias:
        y = y + w[f"{prefix}.fc2.bias"]
    return y


def _ln(x, w, name, cfg):
    affine = cfg.get("layer_norm_elementwise_affine", True)
    eps = cfg.get("layer_norm_eps", 1e-5)   # 1e-5: src/csrc/model/gpt/gpt_weight.h:63
    return layer_norm(x, w[f"{name}.weight"] if affine else None,
                      w[f"{name}.bias"] if affine else None, eps)


def block_pre_norm(x, w, prefix, cfg):
    """a = LN1(x); r = x + Attn(a); d = LN2(r); x' = r + FFN(d)
    (src/csrc/model/gpt/gpt.cc:325-335, :347-391, :423-436 residual inside LN2, :467-486, :496-501)."""
    bias = cfg.get("enable_bias", True)
    a = _ln(x, w, f"{prefix}.self_attn_layer_norm", cfg)
    r = x + attention_layer(a, w, prefix, cfg["num_attention_heads"], bias)
    d = _ln(r, w, f"{prefix}.final_layer_norm", cfg)
    return r + feed_forward(d, w, prefix, bias)


def block_post_norm(x, w, prefix, cfg):
    """r = LN1(x + Attn(x)); x' = LN2(r + FFN(r)).  The reference refuses this arrangement
    (src/csrc/model/gpt/gpt.cc:238-240); it is the same parts with the norms after the sums."""
    bias = cfg.get("enable_bias", True)
    r = _ln(x + attention_layer(x, w, prefix, cfg["num_attention_heads"], bias), w,
            f"{prefix}.self_attn_layer_norm", cfg)
    return _ln(r + feed_forward(r, w, prefix, bias), w, f"{prefix}.final_layer_norm", cfg)


def forward(cfg: dict, w: Dict[str, torch.Tensor], token_ids: Sequence[int]) -> torch.Tensor:
    """Logits [n, vocab] of a whole sequence from position 0 (src/csrc/model/gpt/gpt.cc:507-657:
    embed, blocks, final norm :614-624, head product :192-201)."""
    H = cfg["hidden_size"]
    E = cfg.get("word_embed_proj_dim") or H
    dec = "model.decoder"
    n = len(token_ids)
    x = embed(token_ids, range(n), w[f"{dec}.embed_tokens.weight"], w[f"{dec}.embed_positions.weight"],
              2, w[f"{dec}.project_in.weight"] if E != H else None)
    pre = cfg.get("do_layer_norm_before", True)
    for i in range(cfg["num_hidden_layers"]):
        blk = block_pre_norm if pre else block_post_norm
        x = blk(x, w, f"{dec}.layers.{i}", cfg)
    if pre and not cfg.get("_remove_final_layer_norm", False):
        x = _ln(x, w, f"{dec}.final_layer_norm", cfg)
    if E != H:
        x = x @ w[f"{dec}.project_out.weight"].T
    head = w["lm_head.weight"] if "lm_head.weight" in w else w[f"{dec}.embed_tokens.weight"]
    return x @ head.T


# --------------------------------------------------------------------- sampling
def _fmix32(h: np.ndarray) -> np.ndarray:
    h = h.astype(np.uint32)
    h ^= h >> np.uint32(16)
    h = (h * np.uint32(0x85ebca6b)).astype(np.uint32)
    h ^= h >> np.uint32(13)
    h = (h * np.uint32(0xc2b2ae35)).astype(np.uint32)
    h ^= h >> np.uint32(16)
    return h


def hash_uniform(seed: int, draw: int, vocab: int) -> np.ndarray:
    """The sampler's noise u_v in (0,1) for v < vocab: four rounds of the 32-bit murmur3 finaliser
    over (seed low, seed high, draw index, v); 24 bits, centred."""
    with np.errstate(over="ignore"):
        lo, hi = np.uint32(seed & 0xffffffff), np.uint32((seed >> 32) & 0xffffffff)
        h = _fmix32(np.array([lo ^ np.uint32(0x9e3779b9)], dtype=np.uint32))
        h = _fmix32(h ^ np.uint32((int(hi) + 0x7f4a7c15) & 0xffffffff))
        h = _fmix32(h ^ np.uint32((draw * 0x85ebca6b + 0xc2b2ae35) & 0xffffffff))
        v = np.arange(vocab, dtype=np.uint64)
        hv = _fmix32((h ^ ((v * 0x27d4eb2f + 0x165667b1) & 0xffffffff).astype(np.uint32)))
    return ((hv >> np.uint32(8)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)


def perturbed_scores(logits: np.ndarray, temperature: float, seed: int, draw: int) -> np.ndarray:
    """logit / temperature + Gumbel noise; its argmax is a sample of softmax(logits / temperature)."""
    u = hash_uniform(seed, draw, logits.shape[-1])
    g = -np.log(-np.log(u.astype(np.float64)))
    return logits.astype(np.float64) / temperature + g


def choose(logits: np.ndarray, temperature: float, seed: int, draw: int) -> int:
    """Greedy for temperature 0 (reference: argmax, src/csrc/kernel/findmax.cu:16-39; lowest index
    on ties here), else the Gumbel-max sample."""
    if temperature <= 0:
        return int(np.argmax(logits))
    return int(np.argmax(perturbed_scores(logits, temperature, seed, draw)))


def generate(cfg, w, prompt: Sequence[int], max_new_tokens: int, temperature: float = 0.0,
             seed: int = 0, eos: Optional[int] = None) -> List[int]:
    """Token by token, recomputing the whole sequence each time."""
    seq = list(prompt)
    out: List[int] = []
    for i in range(max_new_tokens):
        logits = forward(cfg, w, seq)[-1].numpy()
        tok = choose(logits, temperature, seed, i)
        out.append(tok)
        seq.append(tok)
        if eos is not None and tok == eos:
            break
    return out
