"""The engine at contexts up to 2,048 tokens against the plain implementation: what a
benchmark of long decoding runs and short tests do not reach.  The decode attention splits a
row's keys over workgroups only from 512 keys on (and, in a recorded step, by the model's
longest context), the split is merged by a kernel of its own or inside the output projection,
the tile kernel deals 32 tiles an item and shares a late portion's keys between groups of
waves.  Oracle as in the reference's own tests: dense attention over the gathered pages
(src/unittest/kernel/attention_ref.cc:91-140), here the plain float64 model.

Random N(0, 0.02) weights give almost uniform attention, under which a dropped or doubled
range of far keys hardly moves a logit: the query and key matrices of these models are scaled
up until the scores have a spread of about 3, so single far keys carry weight."""
import json
import math
import os

import numpy as np
import pytest
import torch

import plain_opt
import tiny
from test_engine_gpu import DTYPES, check, make_runner

pytestmark = pytest.mark.gpu

# L: head size 16, pre-norm, biases.  M: head size 64 (the benchmark's), three heads, post-norm,
# no biases, embedding projection.
LONG = {
    "L": dict(vocab_size=1000, max_position_embeddings=2048, hidden_size=64, num_hidden_layers=2,
              num_attention_heads=4, ffn_dim=256, word_embed_proj_dim=64, do_layer_norm_before=True,
              enable_bias=True, tie_word_embeddings=True),
    "M": dict(vocab_size=777, max_position_embeddings=2048, hidden_size=192, num_hidden_layers=2,
              num_attention_heads=3, ffn_dim=200, word_embed_proj_dim=96, do_layer_norm_before=False,
              enable_bias=False, tie_word_embeddings=True),
}
PAGE = 16
# key splits of the recorded decode step by (heads of the model, requests in the step), 2,048 positions
# (the runners of that test allow as many requests as the step has, so the step has exactly that many rows)
SPLITS_ON_256_UNITS = {4: {1: 8, 2: 8, 4: 8, 8: 8, 12: 6, 13: 5, 16: 4, 17: 4, 32: 2},
                       3: {1: 8, 2: 8, 4: 8, 8: 8, 12: 8, 13: 7, 16: 6, 17: 6, 32: 3}}


def write_peaked_model(name: str, root: str, seed: int) -> str:
    """A random model folder whose q and k matrices are scaled so that scores spread by ~3."""
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.weights import SafetensorsFile, write_random_model
    from swifttransformer_amd.weights.safetensors_io import save_safetensors
    hp = OptHyperParam(**LONG[name]).validate()
    d = write_random_model(hp, os.path.join(root, f"long_{name}"), seed=seed, file_dtype=torch.bfloat16)
    path = os.path.join(d, "model.safetensors")
    f = SafetensorsFile(path)
    # a score is q.k / sqrt(hd) with q, k elements of spread 0.02 sqrt(H): spread 0.0004 H
    factor = math.sqrt(3.0 / (0.0004 * hp.hidden_size))
    tensors = {}
    for k in f.keys():
        t = f.tensor(k).clone()
        if k.endswith(("q_proj.weight", "k_proj.weight")):
            t = (t.float() * factor).to(t.dtype)
        tensors[k] = t
    f.close()
    save_safetensors(path, tensors, {"format": "pt"})
    return d


@pytest.fixture(scope="module")
def long_models(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("long"))
    out = {}
    for name in LONG:
        d = write_peaked_model(name, root, seed=11)
        cfg, w = plain_opt.load_folder(d)
        base = [tiny.prompt(2048, cfg["vocab_size"], 300 + i) for i in range(4)]
        refs = [plain_opt.forward(cfg, w, s).numpy() for s in base]
        out[name] = (d, cfg, w, base, refs)
    return out


def test_scores_of_the_long_models_are_peaked(long_models):
    """The premise of this file: in these models a single far key can carry a tenth of a row's
    attention, so the logits see which keys were read."""
    d, cfg, w, base, _ = long_models["L"]
    x = plain_opt.embed(base[0][:1024], range(1024), w["model.decoder.embed_tokens.weight"],
                        w["model.decoder.embed_positions.weight"], 2, None)
    p = "model.decoder.layers.0."
    a = plain_opt.layer_norm(x, w[p + "self_attn_layer_norm.weight"], w[p + "self_attn_layer_norm.bias"], 1e-5)
    q = a @ w[p + "self_attn.q_proj.weight"].double().T + w[p + "self_attn.q_proj.bias"].double()
    k = a @ w[p + "self_attn.k_proj.weight"].double().T + w[p + "self_attn.k_proj.bias"].double()
    s = (q[-1, :16] @ k[:, :16].T) / 4.0
    pr = torch.softmax(s, 0)
    assert pr.max() > 20.0 / 1024, "attention is still near uniform"


def scramble_pool(runner, seed: int) -> None:
    """Hand all pages out and take them back in random order, so that later block tables are
    permutations of the physical pages and no request's pages are neighbours."""
    rng = np.random.default_rng(seed)
    m = runner.manager
    n = m.num_free_pages(0)
    ids = []
    per = max(1, min(n // m.max_seqs, m.max_pages_per_seq))
    for i in range(m.max_seqs):
        take = min(per, m.num_free_pages(0))
        if take == 0:
            break
        rid = ("scramble", i)
        m.admit(rid)
        m.extend(rid, take * m.page_size)
        ids.append(rid)
    pool = m.groups[0].pool
    pages = []
    for rid in ids:
        pages.extend(m.requests[rid].tables[0])
        m.requests[rid].tables[0] = []
        m.table_array[0][m.requests[rid].slot, :] = -1
        m.requests[rid].length = 0
        m.finish(rid)
    rng.shuffle(pages)
    pool.free([int(p) for p in pages])
    m.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(LONG))
def test_whole_prompt_of_2048(long_models, name, dtype):
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w, base, refs = long_models[name]
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, PAGE, num_pages=2 * 128 + 5, max_seqs=4)
    scramble_pool(runner, 1)
    runner.admit("r")
    logits = runner.step([StepEntry("r", base[0], list(range(2048)))])
    check(logits, refs[0], dt, f"{name} {dtype} whole prompt of 2,048")
    runner.finish("r")
    runner.manager.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(LONG))
@pytest.mark.parametrize("head,portion", [(1536, 512), (1990, 58), (700, 1300)])
def test_late_portion(long_models, name, dtype, head, portion):
    """A portion at the end of a long request: its tiles read up to 2,048 keys each, most of
    them cached by an earlier step."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w, base, refs = long_models[name]
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, PAGE, num_pages=128 + 9, max_seqs=4)
    scramble_pool(runner, 2)
    runner.admit("r")
    toks = base[1]
    logits = runner.step([StepEntry("r", toks[:head], [head - 1])])
    check(logits, refs[1][head - 1:head], dt, f"{name} {dtype} first {head}")
    logits = runner.step([StepEntry("r", toks[head:head + portion], list(range(portion)))])
    check(logits, refs[1][head:head + portion], dt, f"{name} {dtype} portion of {portion} after {head}")
    runner.finish("r")


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(LONG))
@pytest.mark.parametrize("batch", [1, 2, 4, 8, 12, 13, 16, 17, 32])
def test_recorded_decode_after_long_prompts(long_models, name, dtype, batch):
    """About 1,500 tokens of each request in one step, then 32 tokens one by one, all requests
    in one recorded step per token.  The batch size decides the shape of the decode step: how
    many ways a row's keys are split (8 at batch 1 down to 2 at batch 32 with four heads),
    whether the output projection merges the split, whether the norms run inside the products
    (up to 16 rows at these widths) and whether the other products are the library's (from 13 rows)."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w, base, refs = long_models[name]
    dt = DTYPES[dtype]
    n_decode = 32
    heads = [1500 - 37 * i for i in range(batch)]
    pages = sum(-(-(h + n_decode) // PAGE) for h in heads)
    runner = make_runner(d, dt, PAGE, num_pages=pages + 7, max_seqs=batch)
    scramble_pool(runner, 3 + batch)
    mixer = runner.model.layers[0].mixer
    for i, h in enumerate(heads):
        runner.admit(i)
        toks = base[i % 4]
        logits = runner.step([StepEntry(i, toks[:h], [h - 1])])
        check(logits, refs[i % 4][h - 1:h], dt, f"{name} {dtype} prompt {i}")
    replays = runner.graph_replays
    for k in range(n_decode):
        entries = [StepEntry(i, [base[i % 4][h + k]], [0]) for i, h in enumerate(heads)]
        logits = runner.step(entries)
        ref = np.stack([refs[i % 4][h + k] for i, h in enumerate(heads)])
        check(logits, ref, dt, f"{name} {dtype} batch {batch} decode step {k}")
    assert runner.graph_replays == replays + n_decode, "the decode steps were not recorded steps"
    # the shape the recorded step was given on a device of 256 compute units (an MI355X): the rows'
    # keys are split until rows x heads x splits fills the chip, 256 keys a split at least
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        rec = runner._recorded[runner._bucket(batch)]
        splits, _ = mixer._shape_row_kernel(rec.buffers.ctx, rec.buffers.capacity)
        assert splits == SPLITS_ON_256_UNITS[mixer.num_heads][batch]
    for i in range(batch):
        runner.finish(i)
    runner.manager.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(LONG))
def test_unrecorded_decode_after_long_prompts(long_models, name, dtype):
    """The same decoding without recorded steps: the split then follows the step's own longest
    context, and rows of short portions beside decode tokens take the split row kernel too."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w, base, refs = long_models[name]
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, PAGE, num_pages=3 * 128 + 3, max_seqs=4)
    runner.use_graphs = False
    scramble_pool(runner, 9)
    heads = [1900, 1111, 520]
    for i, h in enumerate(heads):
        runner.admit(i)
        runner.step([StepEntry(i, base[i][:h], [])])
    done = list(heads)
    for k, cuts in enumerate([(1, 1, 1), (1, 3, 1), (2, 1, 5), (1, 1, 1), (7, 1, 2), (1, 1, 1)]):
        entries = [StepEntry(i, base[i][done[i]:done[i] + c], list(range(c))) for i, c in enumerate(cuts)]
        logits = runner.step(entries)
        ref = np.concatenate([refs[i][done[i]:done[i] + c] for i, c in enumerate(cuts)])
        check(logits, ref, dt, f"{name} {dtype} unrecorded step {k}")
        for i, c in enumerate(cuts):
            done[i] += c
    assert runner.graph_replays == 0


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(LONG))
def test_mixed_near_2048_with_page_reuse(long_models, name, dtype):
    """Six requests of 1,700 to 2,048 tokens, four live at a time in a pool that holds four:
    large portions of some beside decode tokens of others; pages of finished requests go to
    later ones."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w, base, refs = long_models[name]
    dt = DTYPES[dtype]
    lens = [2048, 1700, 1999, 1850, 2048, 1733]
    src = [0, 1, 2, 3, 1, 2]
    num_pages = 4 * 128
    runner = make_runner(d, dt, PAGE, num_pages=num_pages, max_seqs=4)
    scramble_pool(runner, 4)
    rng = np.random.default_rng(8)
    waiting = list(range(len(lens)))
    live = {}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 4:
            rid = waiting.pop(0)
            live[rid] = 0
            runner.admit(rid)
        entries, spans = [], []
        for rid, done in list(live.items()):
            if rng.random() < 0.15 and len(live) > 1:
                continue
            remaining = lens[rid] - done
            if remaining > 12:
                c = min(int(rng.choice([2, 9, 64, 200, 333, 512, 700])), remaining - 10)
            else:
                c = 1
            want = [0, c // 2, c - 1] if c > 3 else list(range(c))
            entries.append(StepEntry(rid, base[src[rid]][done:done + c], want))
            spans.append((rid, done, want))
        if not entries:
            continue
        logits = runner.step(entries)
        row = 0
        for rid, done, want in spans:
            ref = refs[src[rid]][[done + x for x in want]]
            check(logits[row:row + len(want)], ref, dt,
                  f"{name} {dtype} step {steps} request {rid} positions {[done + x for x in want]}")
            row += len(want)
        for e in entries:
            live[e.req_id] += len(e.tokens)
            if live[e.req_id] == lens[e.req_id]:
                runner.finish(e.req_id)
                del live[e.req_id]
        runner.manager.check_invariants()
        steps += 1
    assert runner.manager.num_free_pages(0) == num_pages


WIDE_HEAD = dict(vocab_size=512, max_position_embeddings=6400, hidden_size=1024, num_hidden_layers=1,
                 num_attention_heads=8, ffn_dim=512, word_embed_proj_dim=1024, do_layer_norm_before=True,
                 enable_bias=True, tie_word_embeddings=True)


@pytest.fixture(scope="module")
def wide_head_model(tmp_path_factory):
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.weights import write_random_model
    hp = OptHyperParam(**WIDE_HEAD).validate()
    d = write_random_model(hp, str(tmp_path_factory.mktemp("wide_head") / "m"), seed=5)
    cfg, w = plain_opt.load_folder(d)
    toks = tiny.prompt(6400, hp.vocab_size, 77)
    return d, toks, plain_opt.forward(cfg, w, toks).numpy()


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_prompt_of_6144_with_heads_of_128(wide_head_model, dtype):
    """A prompt long enough, with heads large enough, that the attention part's planner asks for
    tiles of 128 rows in bfloat16 (48 tiles x 8 heads fill the chip): whole prompt, a late portion
    and a few decode tokens against the plain model."""
    from swifttransformer_amd.engine.step import StepEntry
    d, toks, ref = wide_head_model
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, PAGE, num_pages=2 * 400 + 3, max_seqs=2)
    scramble_pool(runner, 6)
    key, planner = runner.model.layers[0].mixer.step_planner()
    runner.admit("whole")
    entry = StepEntry("whole", toks[:6144], [0, 63, 64, 127, 128, 3000, 6143])
    items = runner.prepare([entry])
    from swifttransformer_amd.parts import BatchInfo
    plan = planner(items, BatchInfo(page_size=PAGE, max_pages=runner.max_pages_per_seq))
    assert plan.host["tile_rows"] == (128 if dtype == "bfloat16" else 64)
    check(runner.run(items), ref[[0, 63, 64, 127, 128, 3000, 6143]], dt, f"{dtype} prompt of 6,144")
    logits = runner.step([StepEntry("whole", toks[6144:6390], list(range(246)))])      # a late portion: 64-row tiles
    check(logits, ref[6144:6390], dt, f"{dtype} portion after 6,144")
    for p in range(6390, 6400):
        check(runner.step([StepEntry("whole", [toks[p]], [0])]), ref[p:p + 1], dt, f"{dtype} decode at {p}")
    runner.finish("whole")
    runner.manager.check_invariants()
