"""The figures bench.py divides by: bytes a decode step must read and operations of a prefill,
counted by hand for the OPT-1.3B sizes, and the command line's refusal of more than one GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def hyper_param():
    from swifttransformer_amd.config import OptHyperParam
    return OptHyperParam(vocab_size=50272, max_position_embeddings=2048, hidden_size=2048, num_hidden_layers=24,
                         num_attention_heads=32, ffn_dim=8192, word_embed_proj_dim=2048).validate()


def test_weight_bytes_counts_every_matrix_once():
    import bench
    hp = hyper_param()
    H, F, V, L = 2048, 8192, 50272, 24
    matrices = L * (3 * H * H + H * H + H * F + F * H) + V * H          # QKV, out, FC1, FC2; the tied head once
    vectors = L * (3 * H + H + F + H + 2 * H + 2 * H)                     # biases and the two norms' gains and biases
    assert bench.weight_bytes(hp, 2) == 2 * matrices + 4 * vectors
    assert abs(bench.weight_bytes(hp, 2) / 1e9 - 2.63) < 0.01             # the 2.63 GB the profiles quote
    assert bench.weight_bytes(hp, 4) == 4 * matrices + 4 * vectors


def test_prefill_flops_counts_products_and_causal_attention():
    import bench
    hp = hyper_param()
    H, F, V, L, T = 2048, 8192, 50272, 24, 2048
    linear = 2 * T * L * (4 * H * H + 2 * H * F)
    pairs = T * (T + 1) // 2                                              # (query, key) pairs a causal mask leaves
    attention = L * 2 * (2 * H * pairs)                                   # scores and weighted values, all heads
    head = 2 * H * V                                                      # only the last row goes through the head
    assert bench.prefill_flops(hp, T) == float(linear + attention + head)


def test_more_than_one_gpu_is_refused_with_one_line():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1
