"""Logits at the layer sizes of the models whose throughput is measured (OPT-1.3B, 2.7B, 6.7B,
13B and 30B widths; vocabulary cut to 4,096, one or two layers) against the plain float64 model:
whole prompt, portions, and decoding through recorded steps at batch 1, 5, 8, 10, 24 and 64.  The product
kernels are chosen by shape (rows, depth, size of the matrix), so these widths reach dispatch
branches that tiny models never do; the test reads the product path counters to show which
ones its logits went through.  Head geometries after the reference's own list
(src/unittest/kernel/fused_attention.cc:44-61: 32 x 64, 32 x 80, 32 x 128, 40 x 128, 56 x 128)."""
import numpy as np
import pytest
import torch

import plain_opt
import tiny
from test_engine_gpu import DTYPES, check, make_runner

pytestmark = pytest.mark.gpu

WIDTHS = {
    "1.3b": dict(hidden_size=2048, num_attention_heads=32, ffn_dim=8192, num_hidden_layers=2),
    "2.7b": dict(hidden_size=2560, num_attention_heads=32, ffn_dim=10240, num_hidden_layers=1),
    "6.7b": dict(hidden_size=4096, num_attention_heads=32, ffn_dim=16384, num_hidden_layers=1),
    "13b": dict(hidden_size=5120, num_attention_heads=40, ffn_dim=20480, num_hidden_layers=1),
    "30b": dict(hidden_size=7168, num_attention_heads=56, ffn_dim=28672, num_hidden_layers=1),
}
VOCAB, POSITIONS, PAGE, N_TOKENS, N_DECODE = 4096, 2048, 16, 340, 4


@pytest.fixture(scope="module")
def wide_models(tmp_path_factory):
    """name -> (folder, cfg, base sequences, their plain logits); the float64 weights are dropped
    once the logits are there (the 30B layer alone is 5 GB of them)."""
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.weights import write_random_model
    root = str(tmp_path_factory.mktemp("wide"))
    cache = {}

    def get(name):
        if name not in cache:
            hp = OptHyperParam(vocab_size=VOCAB, max_position_embeddings=POSITIONS,
                               word_embed_proj_dim=WIDTHS[name]["hidden_size"], **WIDTHS[name]).validate()
            d = write_random_model(hp, f"{root}/{name}", seed=21)
            cfg, w = plain_opt.load_folder(d)
            base = [tiny.prompt(N_TOKENS, VOCAB, 900 + i) for i in range(2)]
            refs = [plain_opt.forward(cfg, w, s).numpy() for s in base]
            del w
            cache[name] = (d, cfg, base, refs)
        return cache[name]
    return get


def run_width(wide_models, name, dtype, batches, per_batch=None):
    """Product path counts of the whole run; ``per_batch`` (a dict) receives for every batch size the
    counts of its first decode step alone (for batch 1 that is the one-token portion): the two runs
    that record the step (one timed for the library's kernels, one captured), later steps being
    replays that issue no product."""
    from swifttransformer_amd.engine.step import StepEntry
    from swifttransformer_amd.ops import kernels as K
    d, cfg, base, refs = wide_models(name)
    dt = DTYPES[dtype]
    biggest = max(batches)
    runner = make_runner(d, dt, PAGE, num_pages=(biggest + 2) * (N_TOKENS // PAGE + 1), max_seqs=biggest)
    K.gemm_path_counts(reset=True)
    # whole prompt, every row's logits
    runner.admit("w")
    n = N_TOKENS - N_DECODE
    check(runner.step([StepEntry("w", base[0][:n], list(range(n)))]), refs[0][:n], dt, f"{name} {dtype} whole prompt")
    runner.finish("w")
    # portions of changing size
    runner.admit("p")
    p = 0
    for c in (7, 2, 64, 130, 1, 3, n - 207):
        before = K.gemm_path_counts()
        logits = runner.step([StepEntry("p", base[1][p:p + c], list(range(c)))])
        if c == 1 and per_batch is not None:      # one token that wants its logits: the recorded step of batch 1
            after = K.gemm_path_counts()
            per_batch[1] = {key: after[key] - before[key] for key in after}
        check(logits, refs[1][p:p + c], dt, f"{name} {dtype} portion [{p},{p + c})")
        p += c
    runner.finish("p")
    # decoding through recorded steps
    for batch in batches:
        heads = [n - 3 * i for i in range(batch)]
        for i, h in enumerate(heads):
            runner.admit(i)
            runner.step([StepEntry(i, base[i % 2][:h], [])])
        replays = runner.graph_replays
        for k in range(N_DECODE):
            before = K.gemm_path_counts()
            entries = [StepEntry(i, [base[i % 2][h + k]], [0]) for i, h in enumerate(heads)]
            logits = runner.step(entries)
            if k == 0 and per_batch is not None and batch not in per_batch:
                after = K.gemm_path_counts()
                per_batch[batch] = {key: after[key] - before[key] for key in after}
            ref = np.stack([refs[i % 2][h + k] for i, h in enumerate(heads)])
            check(logits, ref, dt, f"{name} {dtype} batch {batch} decode step {k}")
        assert runner.graph_replays == replays + N_DECODE
        for i in range(batch):
            runner.finish(i)
    runner.manager.check_invariants()
    return K.gemm_path_counts()


def _sides(counts):
    """(products that went to the vendor library, products that took this library's matrix-core
    kernels, products that took the plain kernel) in one run of a step."""
    own = sum(v for k, v in counts.items() if k not in ("library", "generic_f32", "generic_bf16"))
    return counts["library"], own, counts["generic_f32"] + counts["generic_bf16"]


def test_width_of_opt_1_3b_bfloat16(wide_models):
    paths = run_width(wide_models, "1.3b", "bfloat16", (1, 5, 8, 10, 14, 24, 64))
    # up to 16 rows: norms inside the QKV and FC1 products; the split attention merged by the output
    # projection (batch 1) or by its own kernel before a product with staged rows (batch 5);
    # other products from 13 rows, all from 17 rows and for the prompts: the library; batch 10 makes 320
    # attention workgroups for 256 compute units, which are then split in two over the keys
    for p in ("resident_norm", "resident_merge", "resident_staged", "library"):
        assert paths[p] > 0, f"no product took the path {p}: {paths}"
    assert paths["generic_bf16"] == 0 and paths["generic_f32"] == 0, paths


def test_width_of_opt_1_3b_float32(wide_models):
    paths = run_width(wide_models, "1.3b", "float32", (1, 8, 24))
    assert paths["library"] > 0 and paths["generic_f32"] == 0, paths
    assert sum(v for k, v in paths.items() if k != "library") == 0, paths


def test_width_of_opt_6_7b_bfloat16(wide_models):
    paths = run_width(wide_models, "6.7b", "bfloat16", (1, 5, 8, 24, 64))
    # 4,096-wide rows: norm kernel before the products (the fused form loses at this width); the
    # 16,384-deep FC2 is beyond the resident kernel's reach and goes to the library at any row count
    for p in ("resident_merge", "resident_staged", "library"):
        assert paths[p] > 0, f"no product took the path {p}: {paths}"
    assert paths["resident_norm"] == 0 and paths["generic_bf16"] == 0, paths


def test_width_of_opt_30b_bfloat16(wide_models):
    paths = run_width(wide_models, "30b", "bfloat16", (1, 8, 10, 64))
    # 7,168-wide rows do not fit the norm prologue: norm kernel, then large deep products in the library
    # (batch 10: 560 attention workgroups, split in two over the keys and merged by the merge kernel)
    assert paths["resident_norm"] == 0 and paths["library"] > 0, paths
    assert paths["generic_bf16"] == 0, paths


def test_width_of_opt_2_7b_bfloat16(wide_models):
    """2,560 wide, 32 heads of 80, feed-forward 10,240: the two feed-forward matrices (25 Mi weights,
    at least 2,560 deep) are the library's at any row count, the QKV matrix (under 19 Mi), the output
    projection and the head are this library's up to 12 rows; from 13 rows everything is the
    library's.  A step is recorded by two runs of one layer's four products and the head."""
    per_batch = {}
    paths = run_width(wide_models, "2.7b", "bfloat16", (1, 5, 8, 10, 24, 64), per_batch)
    assert paths["generic_bf16"] == 0 and paths["resident_norm"] == 0, paths      # wider than the norm prologue takes
    for batch in (1, 5, 8, 10):
        assert _sides(per_batch[batch]) == (2 * 2, 2 * 3, 0), (batch, per_batch[batch])
    for batch in (24, 64):
        assert _sides(per_batch[batch]) == (2 * 5, 0, 0), (batch, per_batch[batch])
    assert per_batch[1]["resident_merge"] == 2          # batch 1: the output projection merges the key splits


def test_width_of_opt_13b_bfloat16(wide_models):
    """5,120 wide, 40 heads of 128, feed-forward 20,480: all four products of a layer are large and
    deep enough for the library at any row count (the output projection then takes a merged
    attention output); only the head (4,096 x 5,120 here) stays with this library up to 12 rows."""
    per_batch = {}
    paths = run_width(wide_models, "13b", "bfloat16", (1, 5, 8, 10, 24, 64), per_batch)
    assert paths["generic_bf16"] == 0 and paths["resident_norm"] == 0 and paths["resident_merge"] == 0, paths
    for batch in (1, 5, 8, 10):
        assert _sides(per_batch[batch]) == (2 * 4, 2 * 1, 0), (batch, per_batch[batch])
    for batch in (24, 64):
        assert _sides(per_batch[batch]) == (2 * 5, 0, 0), (batch, per_batch[batch])
