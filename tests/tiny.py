"""Tiny OPT configurations for the tests and helpers to write them to a folder.

A and B differ in every size and option: layers, width (B's is no power of two),
heads and head size, feed-forward width, vocabulary, positions, norm placement,
embedding projection, biases, tied head.  C adds a head size of 64, norms without
gain/bias, another eps and an untied head.  D has sizes that no vector load divides (an odd
vocabulary, a feed-forward width of 50), five heads, one layer and pages of two tokens."""
from __future__ import annotations

import os

import torch

from swifttransformer_amd.config import OptHyperParam
from swifttransformer_amd.weights import write_random_model

TINY_A = dict(vocab_size=1000, max_position_embeddings=128, hidden_size=64, num_hidden_layers=2,
              num_attention_heads=4, ffn_dim=256, word_embed_proj_dim=64, do_layer_norm_before=True,
              enable_bias=True, tie_word_embeddings=True)
TINY_B = dict(vocab_size=1536, max_position_embeddings=256, hidden_size=96, num_hidden_layers=3,
              num_attention_heads=3, ffn_dim=320, word_embed_proj_dim=48, do_layer_norm_before=False,
              enable_bias=False, tie_word_embeddings=True)
TINY_C = dict(vocab_size=777, max_position_embeddings=320, hidden_size=192, num_hidden_layers=2,
              num_attention_heads=3, ffn_dim=200, word_embed_proj_dim=192, do_layer_norm_before=True,
              enable_bias=True, tie_word_embeddings=False, layer_norm_elementwise_affine=False,
              layer_norm_eps=1e-3)
TINY_D = dict(vocab_size=1003, max_position_embeddings=160, hidden_size=80, num_hidden_layers=1,
              num_attention_heads=5, ffn_dim=50, word_embed_proj_dim=80, do_layer_norm_before=True,
              enable_bias=False, tie_word_embeddings=True, layer_norm_eps=1e-6)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 2}


def hyper(name: str) -> OptHyperParam:
    return OptHyperParam(**CONFIGS[name]).validate()


def write_model(name: str, folder: str, seed: int = 0, file_dtype=torch.bfloat16) -> str:
    return write_random_model(hyper(name), os.path.join(folder, f"tiny_{name}_{seed}"), seed=seed,
                              file_dtype=file_dtype)


def prompt(length: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()
