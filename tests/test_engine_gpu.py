"""The engine against the plain implementation: whole prompts, decoding of the last
32 tokens, portions of changing size, and mixed batches with few pages, in float32
and bfloat16, on the tiny configurations."""
import numpy as np
import pytest
import torch

import plain_opt
import tiny

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def tolerance(dtype, ref: np.ndarray):
    """Allowed |engine - plain| per logit.  float32: rounding of a few hundred float
    operations.  bfloat16: activations are rounded to 8 significant bits at each matrix
    input (unit roundoff 2^-9); a few dozen such roundings per logit, so a few percent of
    the logits' spread at the very most."""
    if dtype == torch.float32:
        return 2e-5 + 1e-4 * np.abs(ref)
    return 0.05 * ref.std() + 0.02 * np.abs(ref)


def check(got: torch.Tensor, ref: np.ndarray, dtype, what: str):
    got = got.detach().float().cpu().numpy()
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    err = np.abs(got - ref)
    tol = tolerance(dtype, ref)
    bad = err > tol
    if bad.any():
        i = np.argwhere(bad)[0]
        raise AssertionError(f"{what}: first wrong logit at row {i[0]} col {i[1]}: got {got[tuple(i)]:.6f} "
                             f"ref {ref[tuple(i)]:.6f}; {bad.sum()} of {bad.size} outside tolerance, "
                             f"max err {err.max():.3e}")


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("models"))
    out = {}
    for name in tiny.CONFIGS:
        d = tiny.write_model(name, root, seed=3)
        cfg, w = plain_opt.load_folder(d)
        out[name] = (d, cfg, w)
    return out


# When a step that is not plain decoding is recorded: at the second sighting of its shape (the
# default: most steps of these tests then run unrecorded), or at the first (every step is then a
# replay of a recording made for it or for an earlier step of its shape)
RECORDING = {"unrecorded": 2, "recorded": 1}


def make_runner(model_dir, dtype, page_size, num_pages, max_seqs=4, nan_fill=True, record_after=2, **kw):
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner
    from swifttransformer_amd.models import load_model
    model = load_model(model_dir, dtype, "cuda:0")
    return ModelRunner(model, CacheParam(page_size=page_size, num_pages=num_pages, max_seqs=max_seqs),
                       "cuda:0", cache_fill=float("nan") if nan_fill else 0.0, record_after=record_after, **kw)


def ref_logits(cfg, w, tokens):
    return plain_opt.forward(cfg, w, tokens).numpy()


@pytest.mark.parametrize("recording", list(RECORDING))
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_whole_prompts(models, name, dtype, recording):
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(d, dt, ps, num_pages=64, record_after=RECORDING[recording])
    for i, n in enumerate((1, 5, 17, 33, 100)):
        toks = tiny.prompt(n, cfg["vocab_size"], i)
        runner.admit(i)
        logits = runner.step([StepEntry(i, toks, list(range(n)))])
        check(logits, ref_logits(cfg, w, toks), dt, f"{name} {dtype} whole prompt of {n}")
        runner.finish(i)
        runner.manager.check_invariants()


@pytest.mark.parametrize("recording", list(RECORDING))
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_tail_decode(models, name, dtype, recording):
    """All but the last 32 tokens in one step, then one token per step."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, tiny.PAGE_SIZE[name], num_pages=64, record_after=RECORDING[recording])
    n = 90
    toks = tiny.prompt(n, cfg["vocab_size"], 7)
    ref = ref_logits(cfg, w, toks)
    runner.admit("r")
    head = n - 32
    logits = runner.step([StepEntry("r", toks[:head], [head - 1])])
    check(logits, ref[head - 1:head], dt, f"{name} {dtype} prefix")
    for p in range(head, n):
        logits = runner.step([StepEntry("r", [toks[p]], [0])])
        check(logits, ref[p:p + 1], dt, f"{name} {dtype} decode position {p}")
    runner.finish("r")
    runner.manager.check_invariants()


@pytest.mark.parametrize("recording", list(RECORDING))
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_ragged_portions(models, name, dtype, recording):
    """A prompt in portions of changing size, down to two tokens (and single ones)."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    runner = make_runner(d, dt, tiny.PAGE_SIZE[name], num_pages=64, record_after=RECORDING[recording])
    n = 120
    toks = tiny.prompt(n, cfg["vocab_size"], 11)
    ref = ref_logits(cfg, w, toks)
    cuts = [7, 2, 16, 3, 2, 1, 31, 9, 2, 40, 5, 2]
    assert sum(cuts) == n
    runner.admit("r")
    p = 0
    for c in cuts:
        logits = runner.step([StepEntry("r", toks[p:p + c], list(range(c)))])
        check(logits, ref[p:p + c], dt, f"{name} {dtype} portion [{p},{p + c})")
        p += c
    runner.finish("r")


@pytest.mark.parametrize("recording", list(RECORDING))
@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_mixed_batches_with_page_reuse(models, name, dtype, recording):
    """Up to four live requests; portions of some beside decode tokens of others; a pool so
    small that finished requests' pages go to later ones."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    ps = tiny.PAGE_SIZE[name]
    V = cfg["vocab_size"]
    lens = [45, 70, 33, 90, 51, 64, 20, 77]
    seqs = [tiny.prompt(n, V, 20 + i) for i, n in enumerate(lens)]
    refs = [ref_logits(cfg, w, s) for s in seqs]
    # room for about four requests at a time
    num_pages = sum(-(-n // ps) for n in sorted(lens)[-4:]) + 1
    runner = make_runner(d, dt, ps, num_pages=num_pages, record_after=RECORDING[recording])
    rng = np.random.default_rng(5)
    waiting = list(range(len(seqs)))
    live = {}            # id -> tokens done
    steps = 0
    while waiting or live:
        while waiting and len(live) < 4:
            rid = waiting[0]
            need = -(-lens[rid] // ps)
            held = sum(-(-lens[r] // ps) for r in live)
            if held + need > num_pages:
                break
            waiting.pop(0)
            live[rid] = 0
            runner.admit(rid)
        entries, spans = [], []
        for rid, done in list(live.items()):
            if rng.random() < 0.2 and len(live) > 1:
                continue          # left out of this step, goes on later
            remaining = lens[rid] - done
            if remaining > 16 and done < lens[rid] - 12:
                c = int(rng.integers(2, 24))
                c = min(c, remaining - 8)
            else:
                c = 1             # decoding
            want = list(range(c)) if c <= 4 else [0, c // 2, c - 1]
            entries.append(StepEntry(rid, seqs[rid][done:done + c], want))
            spans.append((rid, done, want))
        if not entries:
            continue
        logits = runner.step(entries)
        row = 0
        for rid, done, want in spans:
            for wi in want:
                check(logits[row:row + 1], refs[rid][done + wi:done + wi + 1], dt,
                      f"{name} {dtype} step {steps} request {rid} position {done + wi}")
                row += 1
        for e in entries:
            live[e.req_id] += len(e.tokens)
            if live[e.req_id] == lens[e.req_id]:
                runner.finish(e.req_id)
                del live[e.req_id]
        runner.manager.check_invariants()
        steps += 1
    assert runner.manager.num_free_pages(0) == num_pages
    if recording == "recorded":
        assert runner.graph_replays == runner.steps_run, "a step ran unrecorded"


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_recorded_decode_steps_of_24_requests(models, name, dtype):
    """Decode steps of 24 requests at once: more rows than the resident-slab product takes, so
    the products of the recorded step (a HIP graph) run in the vendor library, followed by the
    separate page write.  Every replay is checked against the plain implementation, with
    unrecorded work (a prompt of another request) between the replays."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    n_req, n_decode = 24, 5
    runner = make_runner(d, dt, tiny.PAGE_SIZE[name], num_pages=24 * 12 + 16, max_seqs=32)
    seqs = [tiny.prompt(3 + i + n_decode, cfg["vocab_size"], 50 + i) for i in range(n_req)]
    refs = [ref_logits(cfg, w, s) for s in seqs]
    for i, s in enumerate(seqs):
        runner.admit(i)
        n = len(s) - n_decode
        logits = runner.step([StepEntry(i, s[:n], [n - 1])])
        check(logits, refs[i][n - 1:n], dt, f"{name} {dtype} prompt {i}")
    replays = 0
    for k in range(n_decode):
        entries = [StepEntry(i, [s[len(s) - n_decode + k]], [0]) for i, s in enumerate(seqs)]
        before = runner.graph_replays
        logits = runner.step(entries).clone()
        replays += runner.graph_replays - before
        ref = np.stack([refs[i][len(s) - n_decode + k] for i, s in enumerate(seqs)])
        check(logits, ref, dt, f"{name} {dtype} recorded decode step {k}")
        # other work between two replays (a prompt step, unrecorded or a recording of its own)
        runner.admit("x")
        other = tiny.prompt(9 + k, cfg["vocab_size"], 90 + k)
        check(runner.step([StepEntry("x", other, [len(other) - 1])]), ref_logits(cfg, w, other)[-1:], dt,
              f"{name} {dtype} prompt between replays {k}")
        runner.finish("x")
    assert replays == n_decode, "the decode steps were not replays of a recorded step"
    for i in range(n_req):
        runner.finish(i)
    runner.manager.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", list(tiny.CONFIGS))
def test_portions_beside_many_decode_tokens(models, name, dtype):
    """Steps that hold portions of two prompts beside the decode tokens of 20 other requests (the
    shape of a serving step under load): the portions' tiles and the decode rows are two kernels
    writing rows of one output, and the products see more rows than any other mixed test gives
    them.  Every row of every step is compared with the plain implementation; the portions
    change size from step to step, the order of the entries alternates, and the pages are few."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    V, P = cfg["vocab_size"], cfg["max_position_embeddings"]
    n_dec, n_steps = 20, 6
    deco = [tiny.prompt(5 + 2 * i + n_steps, V, 300 + i) for i in range(n_dec)]
    longs = [tiny.prompt(min(P, 100 + 17 * j), V, 400 + j) for j in range(2)]
    refs_d = [ref_logits(cfg, w, s) for s in deco]
    refs_l = [ref_logits(cfg, w, s) for s in longs]
    ps = tiny.PAGE_SIZE[name]
    pages = sum(-(-len(s) // ps) for s in deco + longs) + 3
    runner = make_runner(d, dt, ps, num_pages=pages, max_seqs=32)
    for i, s in enumerate(deco):
        runner.admit(("d", i))
        runner.step([StepEntry(("d", i), s[:len(s) - n_steps], [])])
    for j in range(2):
        runner.admit(("l", j))
    done = [0, 0]
    cuts = [(9, 30), (40, 8), (1, 25), (23, 23), (8, 2), (19, 12)]
    for k in range(n_steps):
        entries, ref = [], []
        for j in range(2):                               # portions first, decode tokens after them
            c = min(cuts[k][j], len(longs[j]) - done[j])
            if c > 0:
                entries.append(StepEntry(("l", j), longs[j][done[j]:done[j] + c], list(range(c))))
                ref.append(refs_l[j][done[j]:done[j] + c])
                done[j] += c
        for i, s in enumerate(deco):
            p = len(s) - n_steps + k
            entries.append(StepEntry(("d", i), [s[p]], [0]))
            ref.append(refs_d[i][p:p + 1])
        if k % 2:                                        # and the other way round
            entries, ref = entries[::-1], ref[::-1]
        check(runner.step(entries), np.concatenate(ref), dt, f"{name} {dtype} step {k}")
    for i in range(n_dec):
        runner.finish(("d", i))
    for j in range(2):
        runner.finish(("l", j))
    runner.manager.check_invariants()


@pytest.mark.parametrize("dtype", list(DTYPES))
@pytest.mark.parametrize("name", ["A", "B"])
def test_recorded_steps_of_one_shape_are_refilled(models, name, dtype):
    """One recording serves every batch of its shape: portions of 20 to 24 tokens (one padded row
    count, one tile list length) of three requests in turn, at changing offsets, with another number of
    wanted rows inside one bucket, and with unrecorded work, decode replays and steps of other
    shapes between the replays.  Every replay is compared with the plain implementation, and
    what an earlier batch left in the buffers (more items, other pages, other wanted rows) must
    not show."""
    from swifttransformer_amd.engine.step import StepEntry
    d, cfg, w = models[name]
    dt = DTYPES[dtype]
    V = cfg["vocab_size"]
    ps = tiny.PAGE_SIZE[name]
    runner = make_runner(d, dt, ps, num_pages=3 * (-(-120 // ps)) + 8, max_seqs=4)
    seqs = [tiny.prompt(120, V, 600 + i) for i in range(3)]
    refs = [ref_logits(cfg, w, s) for s in seqs]
    done = [0, 0, 0]
    for i in range(3):
        runner.admit(i)
    sizes = [24, 21, 23, 20, 24, 22, 23, 24, 20, 21, 22, 24]
    replays = 0
    for k, c in enumerate(sizes):
        i = k % 3
        want = [0, c - 1] if k % 2 else [c - 1, 3]          # two wanted rows, in either order
        before = runner.graph_replays
        logits = runner.step([StepEntry(i, seqs[i][done[i]:done[i] + c], want)])
        replays += runner.graph_replays - before
        ref = np.stack([refs[i][done[i] + x] for x in want])
        check(logits, ref, dt, f"{name} {dtype} portion {k} of request {i} at {done[i]}")
        done[i] += c
        if k % 4 == 1:       # a step of another shape and a decode replay in between
            j = (i + 1) % 3
            lg = runner.step([StepEntry(j, seqs[j][done[j]:done[j] + 1], [0])])
            check(lg, refs[j][done[j]:done[j] + 1], dt, f"{name} {dtype} decode token between")
            done[j] += 1
            runner.admit("x")
            other = tiny.prompt(5 + k, V, 650 + k)
            check(runner.step([StepEntry("x", other, [len(other) - 1])]), ref_logits(cfg, w, other)[-1:], dt,
                  f"{name} {dtype} prompt between")
            runner.finish("x")
    # 20..24 tokens are one bucket of 32 rows: recorded at the second sighting, replayed from then on
    assert replays == len(sizes) - 1, replays
    assert len(runner._recorded_general) >= 1 and runner.arena.overflows == 0
    for i in range(3):
        runner.finish(i)
    runner.manager.check_invariants()


@pytest.mark.parametrize("n_req,max_seqs", [(14, 16), (48, 64), (100, 128)])
def test_recorded_steps_with_model_sized_products(tmp_path, n_req, max_seqs):
    """A 2,048-wide two-layer model, 14, 48 or 100 requests decoding at once: the recorded step's products
    are the library's kernels for these shapes, chosen by timing while the step is recorded, among
    those that need no workspace (other kernels than on the tiny models).  Every replay is
    compared with the same step run unrecorded on a second runner, and with the plain
    implementation."""
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.engine.step import StepEntry
    from swifttransformer_amd.weights import write_random_model
    hp = OptHyperParam(vocab_size=4096, max_position_embeddings=256, hidden_size=2048, num_hidden_layers=2,
                       num_attention_heads=32, ffn_dim=8192, word_embed_proj_dim=2048).validate()
    d = write_random_model(hp, str(tmp_path / "wide"), seed=9)
    cfg, w = plain_opt.load_folder(d)
    n_decode = 4
    dt = torch.bfloat16
    recorded = make_runner(d, dt, 16, num_pages=n_req * 3, max_seqs=max_seqs)
    eager = make_runner(d, dt, 16, num_pages=n_req * 3, max_seqs=max_seqs)
    eager.use_graphs = False
    seqs = [tiny.prompt(5 + i % 7 + n_decode, hp.vocab_size, 400 + i) for i in range(n_req)]
    for i, s in enumerate(seqs):
        for r in (recorded, eager):
            r.admit(i)
            r.step([StepEntry(i, s[:len(s) - n_decode], [])])
    refs = [ref_logits(cfg, w, s) for s in seqs[:6]]
    replays = recorded.graph_replays         # (prompt steps of a shape seen before are replays too)
    for k in range(n_decode):
        entries = [StepEntry(i, [s[len(s) - n_decode + k]], [0]) for i, s in enumerate(seqs)]
        a = recorded.step(entries).clone()
        b = eager.step(entries)
        # the same kernels on the same inputs, except that the recorded attention is shaped for the
        # longest context the model allows: rounding only
        diff = (a - b).abs().max().item()
        assert diff <= 0.02 * b.std().item(), f"replay {k}: recorded and unrecorded steps differ by {diff}"
        ref = np.stack([refs[i][len(seqs[i]) - n_decode + k] for i in range(6)])
        check(a[:6], ref, dt, f"wide model, recorded decode step {k}")
    assert recorded.graph_replays == replays + n_decode and eager.graph_replays == 0


@pytest.mark.parametrize("seed", [1, 5, 9, 20])
def test_random_configuration_and_trace(seed, tmp_path):
    """A configuration drawn at random (heads, head size in steps of 16, widths and vocabulary that
    are no power of two, norm placement, biases, tied head, embedding projection) and a trace
    drawn at random (up to four live requests, portions from 1 to 130 tokens, requests left out of
    steps, a pool that holds exactly what is live) through the replay loop, in both precisions,
    against the plain implementation."""
    import io
    import json
    import random
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.engine.trace import replay
    from swifttransformer_amd.weights import write_random_model
    rng = random.Random(seed)
    heads, hd = rng.choice([1, 2, 3, 4, 5, 8, 12]), rng.choice([16, 32, 48, 64, 80, 96, 128])
    H = heads * hd
    hp = OptHyperParam(vocab_size=rng.choice([257, 1000, 1003, 4096, 5001]),
                       max_position_embeddings=rng.choice([160, 300, 512]), hidden_size=H,
                       num_hidden_layers=rng.choice([1, 2, 3]), num_attention_heads=heads,
                       ffn_dim=rng.choice([H, 2 * H + 8, 4 * H, 50, 136]),
                       word_embed_proj_dim=rng.choice([H, H, max(16, H // 2)]),
                       do_layer_norm_before=rng.random() < 0.7, enable_bias=rng.random() < 0.7,
                       tie_word_embeddings=rng.random() < 0.7,
                       layer_norm_elementwise_affine=rng.random() < 0.8,
                       layer_norm_eps=rng.choice([1e-5, 1e-6, 1e-3])).validate()
    d = write_random_model(hp, str(tmp_path / "m"), seed=seed)
    cfg, w = plain_opt.load_folder(d)
    lens = [rng.randrange(1, hp.max_position_embeddings + 1) for _ in range(rng.choice([2, 4, 6]))]
    reqs = {f"r{i}": tiny.prompt(n, hp.vocab_size, 700 + 10 * seed + i) for i, n in enumerate(lens)}
    refs = {r: ref_logits(cfg, w, t) for r, t in reqs.items()}
    steps, wanted = [], {}
    pos, waiting, live = {r: 0 for r in reqs}, list(reqs), []
    while waiting or live:
        while waiting and len(live) < 4 and rng.random() < 0.7:
            live.append(waiting.pop(0))
        if not live:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in list(live):
            if rng.random() < 0.25 and len(live) > 1:
                continue
            take = min(len(reqs[r]) - pos[r], rng.choice([1, 1, 1, 2, 2, 3, 5, 8, 9, 16, 17, 31, 64, 65, 130]))
            want = sorted(rng.sample(range(take), min(rng.choice([0, 1, 2, take]), take)))
            entries.append({"id": r, "tokens": reqs[r][pos[r]:pos[r] + take], "want": want})
            wanted.setdefault(len(steps), []).extend((r, pos[r] + x) for x in want)
            pos[r] += take
            if pos[r] == len(reqs[r]):
                end.append(r)
                live.remove(r)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    max_tokens = sum(sorted((-(-n // 64) * 64 for n in lens), reverse=True)[:4])
    for dtype in DTYPES:
        out = tmp_path / dtype
        log = io.StringIO()
        assert replay(d, dtype, str(out), max_tokens, io.StringIO(text), log=log, max_live=4) == 0
        assert log.getvalue().count("done ") == len(steps)
        for s, rows in wanted.items():
            if not rows:
                assert not (out / f"{s}.f32").exists()      # nothing wanted, nothing written
                continue
            got = np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(len(rows), hp.vocab_size)
            ref = np.stack([refs[r][p] for r, p in rows])
            check(torch.from_numpy(got), ref, DTYPES[dtype], f"seed {seed} {dtype} step {s}")


def test_wide_head_with_the_norm_inside_and_the_best_tokens_out(tmp_path):
    """A vocabulary wide enough for the head's persistent kernel (20,000 words): in bfloat16 the final
    norm of the wanted rows runs inside the head's product and the rows' best tokens come out of
    its epilogue, in unrecorded steps, recorded prompt steps and recorded decode steps; in float32
    the norm kernel, the library's product and the arg-max kernel do the same.  Logits against the
    plain implementation, best tokens against the engine's own logits, greedy generation through
    the engine against the plain model's choices."""
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.engine.step import StepEntry
    from swifttransformer_amd.ops import kernels as K
    from swifttransformer_amd.sampling import SamplingParams
    from swifttransformer_amd.weights import write_random_model
    hp = OptHyperParam(vocab_size=20000, max_position_embeddings=96, hidden_size=128, num_hidden_layers=2,
                       num_attention_heads=2, ffn_dim=256, word_embed_proj_dim=128).validate()
    d = write_random_model(hp, str(tmp_path / "wide_vocab"), seed=13)
    cfg, w = plain_opt.load_folder(d)
    seqs = [tiny.prompt(40 + 3 * i, hp.vocab_size, 820 + i) for i in range(5)]
    refs = [ref_logits(cfg, w, s) for s in seqs]
    for dtype in DTYPES:
        dt = DTYPES[dtype]
        runner = make_runner(d, dt, 8, num_pages=80, max_seqs=8, record_after=2)
        K.gemm_path_counts(reset=True)
        n_decode = 4
        for rep in range(2):                 # the second round's prompt steps are recorded ones
            for i, s in enumerate(seqs):
                runner.admit((rep, i))
                n = len(s) - n_decode
                logits = runner.step([StepEntry((rep, i), s[:n], [0, n - 1])])
                check(logits, refs[i][[0, n - 1]], dt, f"{dtype} prompt {i} round {rep}")
                assert torch.equal(runner.last_best.long(), logits.argmax(-1)), f"{dtype} prompt {i} round {rep}"
            for k in range(n_decode):
                entries = [StepEntry((rep, i), [s[len(s) - n_decode + k]], [0]) for i, s in enumerate(seqs)]
                logits = runner.step(entries)
                check(logits, np.stack([refs[i][len(s) - n_decode + k] for i, s in enumerate(seqs)]), dt,
                      f"{dtype} decode step {k} round {rep}")
                assert torch.equal(runner.last_best.long(), logits.argmax(-1))
            for i in range(len(seqs)):
                runner.finish((rep, i))
        assert runner.graph_replays >= 2 * n_decode + 3
        assert (K.gemm_path_counts()["wide"] > 0) == (dt == torch.bfloat16)
    eng = Engine(d, dtype="fp32", page_size=8, num_pages=80, max_seqs=4)
    prompts = [s[:11 + 5 * i] for i, s in enumerate(seqs[:3])]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=6, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain_opt.generate(cfg, w, p, 6)
    eng = Engine(d, dtype="bf16", page_size=8, num_pages=80, max_seqs=4)
    for p, o in zip(prompts, eng.generate(prompts, SamplingParams(max_new_tokens=6, ignore_eos=True))):
        logits = plain_opt.forward(cfg, w, list(p) + list(o)).numpy()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert row.max() - row[tok] <= 0.05 * row.std() + 0.02 * abs(row.max())
