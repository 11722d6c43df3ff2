"""Generation through the entry points: greedy and temperature sampling through the engine
and the scheduler, the command line, the OptOp-style call, trace replay as a program, long
decoding, and the first tokens of a sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_opt
import tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("gen"))
    out = {}
    for name in tiny.CONFIGS:
        d = tiny.write_model(name, root, seed=11)
        cfg, w = plain_opt.load_folder(d)
        out[name] = (d, cfg, w)
    return out


def test_greedy_generation_config_a(models):
    """The workload of tiny A: prompts of 5/17/33 tokens, 16 greedy tokens each, block size 4."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab_size"], i) for i, n in enumerate((5, 17, 33))]
    eng = Engine(d, dtype="fp32", page_size=4, num_pages=64, max_seqs=4)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=16, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain_opt.generate(cfg, w, p, 16)
    eng.runner.manager.check_invariants()
    assert eng.runner.manager.num_free_pages(0) == 64 and eng.stats.generated_tokens == 48


def test_engine_sized_from_free_memory(models):
    """``gpu_mem_fraction``: the cache pool takes that share of the memory that is free once the
    weights are loaded (no page count given), and the engine generates from it as from any pool."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.models import load_model
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["C"]
    model = load_model(d, torch.bfloat16)
    torch.cuda.synchronize()
    free, _ = torch.cuda.mem_get_info()
    fraction = 0.002
    eng = Engine(model, dtype="bf16", page_size=16, max_seqs=3, gpu_mem_fraction=fraction)
    pool_bytes = eng.runner.cache.bytes()
    # keys and values of tiny C's two layers: 2 x 2 x 3 heads x 16 tokens x 64 dims x 2 bytes a page
    per_page = 2 * 2 * 3 * 16 * 64 * 2
    pages = eng.runner.cache_param.num_pages
    assert pool_bytes == pages * per_page
    # (the share is taken of what is free once the step arena stands; the arena of a tiny model
    # and what its sizing run left with the allocator are some tens of megabytes)
    assert fraction * (free - eng.runner.arena.nbytes() - (256 << 20)) - per_page < pool_bytes <= fraction * free
    assert eng.runner.arena.nbytes() > 0
    assert eng.runner.manager.num_free_pages(0) == pages
    prompts = [tiny.prompt(n, cfg["vocab_size"], 70 + i) for i, n in enumerate((3, 50, 21))]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=6, ignore_eos=True))
    for p, o in zip(prompts, outs):
        logits = plain_opt.forward(cfg, w, list(p) + list(o)).numpy()
        for i, tok in enumerate(o):
            row = logits[len(p) - 1 + i]
            assert row.max() - row[tok] <= 0.05 * row.std() + 0.02 * abs(row.max())
    assert eng.runner.manager.num_free_pages(0) == pages
    with pytest.raises(ValueError):
        Engine(model, dtype="bf16", gpu_mem_fraction=1.5)


def test_warm_up_records_the_steps_ahead_of_the_requests(models):
    """``Engine.warm_up``: recordings for prompt portions and decode batches are made on scratch
    requests that give everything back; the first real prompt of a warmed size is then a replay,
    and the tokens are the plain implementation's."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["A"]
    eng = Engine(d, dtype="fp32", page_size=4, num_pages=64, max_seqs=4, prefill_chunk=32, max_batched_tokens=40)
    made = eng.warm_up()
    assert made == 3 + 3                      # portions of 8, 16 and 32 tokens; batches of 1, 2 and 4 requests
    assert eng.runner.manager.num_free_pages(0) == 64 and eng.runner.manager.num_free_slots == 4
    steps, replays = eng.runner.steps_run, eng.runner.graph_replays
    prompts = [tiny.prompt(n, cfg["vocab_size"], 80 + i) for i, n in enumerate((30, 14))]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=5, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == plain_opt.generate(cfg, w, p, 5)
    assert eng.runner.graph_replays - replays >= 4 and eng.runner.steps_run > steps      # the decode steps at least
    eng.add_request(prompts[0])
    with pytest.raises(RuntimeError, match="warm up before"):
        eng.warm_up()


def test_temperature_generation_config_b_chunked(models):
    """The workload of tiny B: prompts of 1/9/40/100 tokens, 12 tokens each at temperature 0.8
    with a seeded sampler, prompt portions of 16, block size 8."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["B"]
    prompts = [tiny.prompt(n, cfg["vocab_size"], 40 + i) for i, n in enumerate((1, 9, 40, 100))]
    params = [SamplingParams(temperature=0.8, seed=1000 + i, max_new_tokens=12, ignore_eos=True)
              for i in range(4)]
    eng = Engine(d, dtype="fp32", page_size=8, num_pages=40, max_seqs=4, prefill_chunk=16,
                 max_batched_tokens=48)
    outs = eng.generate(prompts, params)
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o) == 12
        # follow the engine's tokens and check each choice against the plain scores
        seq = list(p)
        for j, tok in enumerate(o):
            logits = plain_opt.forward(cfg, w, seq)[-1].numpy()
            score = plain_opt.perturbed_scores(logits, 0.8, 1000 + i, j)
            best = int(np.argmax(score))
            assert tok == best or score[best] - score[tok] < 1e-4, (i, j, tok, best)
            seq.append(tok)
    # the same seeds in another batching give the same tokens
    eng2 = Engine(d, dtype="fp32", page_size=8, num_pages=40, max_seqs=2, prefill_chunk=7,
                  max_batched_tokens=20)
    assert eng2.generate(prompts, params) == outs


def test_preemption_does_not_change_output(models):
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab_size"], 60 + i) for i, n in enumerate((30, 26, 21))]
    sp = SamplingParams(max_new_tokens=24, ignore_eos=True)
    roomy = Engine(d, dtype="fp32", page_size=4, num_pages=64, max_seqs=4).generate(prompts, sp)
    tight = Engine(d, dtype="fp32", page_size=4, num_pages=30, max_seqs=4)
    assert tight.generate(prompts, sp) == roomy
    assert tight.stats.preemptions >= 1
    assert tight.runner.manager.num_free_pages(0) == 30


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_long_decoding_and_eos(models, dtype):
    """Decode up to the model's last position; in float32 the tokens are the plain ones."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["A"]
    p = tiny.prompt(6, cfg["vocab_size"], 77)
    eng = Engine(d, dtype=dtype, page_size=4, num_pages=64, max_seqs=2)
    out = eng.generate([p], SamplingParams(max_new_tokens=500, ignore_eos=True))[0]
    assert len(out) == cfg["max_position_embeddings"] - 6 + 1     # every position used, one token beyond
    ref = plain_opt.generate(cfg, w, p, len(out) - 1)
    if dtype == "fp32":
        assert out[:-1] == ref
    else:
        # bfloat16 may leave the plain path at a near-tie; until then the tokens agree
        k = next((i for i, (a, b) in enumerate(zip(out, ref)) if a != b), len(ref))
        assert k >= 8
        seq = p + out[:k]
        lg = plain_opt.forward(cfg, w, seq)[-1].numpy()
        if k < len(ref):
            assert lg[ref[k]] - lg[out[k]] < 0.05 * lg.std()
    # the end token stops a request
    eos = ref[3]
    first = ref.index(eos)
    out2 = Engine(d, dtype="fp32", page_size=4, num_pages=64).generate(
        [p], SamplingParams(max_new_tokens=50, eos_token_id=eos))[0]
    assert out2 == ref[:first + 1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON steps on stdin, <step>.f32 files out."""
    d, cfg, w = models["B"]
    V = cfg["vocab_size"]
    a, b = tiny.prompt(50, V, 90), tiny.prompt(21, V, 91)
    ra, rb = plain_opt.forward(cfg, w, a).numpy(), plain_opt.forward(cfg, w, b).numpy()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[30:32], "want": []},
                                {"id": "b", "tokens": b[:20], "want": [19]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[32:], "want": [17]}], "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": b, "want": [20]}], "end": ["c"]},
    ]
    out = tmp_path / "out"
    env = dict(os.environ)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "128"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    assert not (out / "1.f32").exists() or np.fromfile(out / "1.f32", "<f4").size == V
    want = {0: np.stack([ra[0], ra[29]]), 1: rb[19:20], 2: rb[20:21], 3: ra[49:50], 4: rb[20:21]}
    for s, ref in want.items():
        got = np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, V)
        tol = (2e-5 + 1e-4 * np.abs(ref)) if dtype == "float32" else (0.05 * ref.std() + 0.02 * np.abs(ref))
        assert got.shape == ref.shape and (np.abs(got - ref) <= tol).all(), (s, np.abs(got - ref).max())


def test_first_tokens_of_a_sequence(models):
    """Positions 0, 1, 2 alone and together: the start of a sequence is where an offset or
    an off-by-one in the position table shows."""
    from swifttransformer_amd.engine.step import StepEntry
    from test_engine_gpu import check, make_runner
    for name in ("A", "B"):
        d, cfg, w = models[name]
        toks = tiny.prompt(3, cfg["vocab_size"], 5)
        ref = plain_opt.forward(cfg, w, toks).numpy()
        for dt in (torch.float32, torch.bfloat16):
            runner = make_runner(d, dt, tiny.PAGE_SIZE[name], 8)
            runner.admit(0)
            for p in range(3):
                check(runner.step([StepEntry(0, [toks[p]], [0])]), ref[p:p + 1], dt, f"{name} position {p}")
            runner.finish(0)
            runner.admit(1)
            check(runner.step([StepEntry(1, toks, [0, 1, 2])]), ref, dt, f"{name} first three together")


def test_optop_style_entry(models):
    """The reference-shaped call: caller-owned caches [blocks, layers, heads, block, dim] and
    block tables; whole prompts, then single tokens with first_token_indexes."""
    from swifttransformer_amd.opt_op import OptOp
    d, cfg, w = models["A"]
    hp = tiny.hyper("A")
    op = OptOp(hp.vocab_size, hp.max_position_embeddings, hp.hidden_size, hp.num_hidden_layers,
               hp.num_attention_heads, hp.head_dim, "fp32", 4, 32, [1, 0, 1, 0], ffn_dim=hp.ffn_dim)
    with pytest.raises(RuntimeError, match="load the weight"):
        op.forward([[1]], [0], torch.zeros(1), torch.zeros(1), [[0]])
    op.load_weight(d)
    kc = torch.zeros(40, hp.num_hidden_layers, hp.num_attention_heads, 4, hp.head_dim, device="cuda:0")
    vc = torch.zeros_like(kc)
    prompts = [tiny.prompt(5, hp.vocab_size, 1), tiny.prompt(17, hp.vocab_size, 2)]
    tables = [[1, 2, 3, 4], [10, 11, 12, 13, 14, 15, 16]]
    toks = op.forward(prompts, [0, 0], kc, vc, tables)
    seqs = [p + [t] for p, t in zip(prompts, toks)]
    for _ in range(5):
        nxt = op.forward([[s[-1]] for s in seqs], [len(s) - 1 for s in seqs], kc, vc, tables)
        for s, t in zip(seqs, nxt):
            s.append(t)
    for p, s in zip(prompts, seqs):
        assert s[len(p):] == plain_opt.generate(cfg, w, p, 6)
    assert op.forward([], [], kc, vc, []) == []
    op2 = OptOp(100, 32, 32, 1, 2, 16, "bf16", 4, 8)
    op2.init_dummy_weights()
    k2 = torch.zeros(4, 1, 2, 4, 16, device="cuda:0", dtype=torch.bfloat16)
    assert len(op2.forward([[1, 2, 3]], [0], k2, torch.zeros_like(k2), [[0]])) == 1


def test_command_line(models, tmp_path):
    d, cfg, w = models["A"]
    prompts = [tiny.prompt(n, cfg["vocab_size"], 30 + i) for i, n in enumerate((4, 9))]
    inp = tmp_path / "in.txt"
    inp.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "run_opt"), d, "opt_tiny", "fp32", str(inp),
                        "--max-new-tokens", "5", "--ignore-eos", "--block-size", "4", "--num-blocks", "32"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 2
    for line, p in zip(lines, prompts):
        gen = line.split(")")[1].split("(")[0].split()
        assert [int(t) for t in gen] == plain_opt.generate(cfg, w, p, 5)
        assert "(5 tokens generated)" in line
    assert "Context stage" in r.stdout and "Regression stage" in r.stdout
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "run_opt"), d, "llama2_7b", "fp32", str(inp)],
                         capture_output=True, text=True, timeout=300)
    assert bad.returncode == 1 and "Invalid model name" in bad.stdout


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_steps_queued_ahead_give_the_same_output(models, dtype):
    """The engine queues a decode step before the previous step's tokens have reached the host.
    With an end token that several requests hit at different steps (found out one step late,
    beside requests that go on), with requests arriving while a step is queued ahead and with
    so few pages that some steps cannot be queued ahead, tokens and finish reasons are those of
    an engine that never queues ahead; no page or slot is lost."""
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["A"]
    V = cfg["vocab_size"]
    prompts = [tiny.prompt(3 + 2 * i, V, 300 + i) for i in range(6)]

    def run(lookahead, eos, num_pages=96, late=()):
        eng = Engine(d, dtype=dtype, page_size=4, num_pages=num_pages, max_seqs=8, lookahead=lookahead)
        sp = [SamplingParams(max_new_tokens=30 + i, temperature=0.9, seed=11 + i,
                             eos_token_id=eos, ignore_eos=eos is None) for i in range(len(prompts))]
        ids = [eng.add_request(p, s) for p, s in zip(prompts, sp) if prompts.index(p) not in late]
        done, n = {}, 0
        while eng.has_work() or n < 4:
            if n == 3:                                   # arrivals while a step is queued ahead
                for i in late:
                    eng.add_request(prompts[i], sp[i], req_id=f"late{i}")
            for o in eng.step():
                done[o.req_id] = (o.output, o.finish_reason)
            n += 1
        eng.runner.manager.check_invariants()
        assert eng.runner.manager.num_free_pages() == num_pages and eng.runner.manager.num_free_slots == 8
        return done, eng

    free_run, _ = run(False, None)
    counts = {}
    for out, _reason in free_run.values():
        for t in set(out[2:]):
            counts[t] = counts.get(t, 0) + 1
    eos = max(counts, key=lambda t: (counts[t], -t))     # a token that ends as many requests as possible
    assert counts[eos] >= 2
    plain, _ = run(False, eos)
    ahead, eng = run(True, eos)
    assert ahead == plain
    reasons = sorted(r for _, r in ahead.values())
    assert "eos" in reasons and "length" in reasons
    assert eng.runner.graph_replays > 20                 # the decode steps were recorded steps
    # arrivals in the middle, and a pool so small that requests are pre-empted
    assert run(True, eos, late=(1, 4))[0] == run(False, eos, late=(1, 4))[0]
    tight_a, eng_a = run(True, None, num_pages=40)
    tight_p, eng_p = run(False, None, num_pages=40)
    assert eng_p.stats.preemptions > 0 and eng_a.stats.preemptions > 0
    if dtype == "fp32":
        # a pre-empted request is recomputed as a prompt: other kernels, other rounding, and in
        # bfloat16 a sampled near-tie may then fall the other way; float32 keeps the tokens
        assert tight_a == tight_p == free_run


def test_benchmark_command_line(capsys):
    """benchmark_all_input_same in the reference's manner: named experiments, dummy weights,
    the reference's table of results."""
    from swifttransformer_amd.cli.benchmark_all_input_same import main
    assert main(["opt_125m", "bf16", "smoke", "--layers", "1"]) == 0
    out = capsys.readouterr().out
    assert "Context stage:" in out and "Regression stage:" in out and "(4 tokens generated)" in out
    assert "  block_size   input_len  batch_size decode_step context_t(ms)  decode_t(ms)   total_t(ms)" in out
    assert main(["opt_125m", "bf16", "no_such_experiment"]) == 1
    assert main(["opt_999b", "bf16", "smoke"]) == 1


def test_model_in_memory_on_the_gpu_equals_its_folder(models):
    """``random_model`` draws on the GPU what ``write_random_model`` drew on the CPU: the same
    tensors bit for bit, so the same logits; the model a benchmark runs can be written to a folder
    (and compared with the plain implementation there)."""
    from swifttransformer_amd.config import CacheParam
    from swifttransformer_amd.engine.step import ModelRunner, StepEntry
    from swifttransformer_amd.models import load_model, random_model
    for name in ("A", "B"):
        d, cfg, w = models[name]
        toks = tiny.prompt(29, cfg["vocab_size"], 3)
        for dtype in (torch.bfloat16, torch.float32):
            mem, disk = random_model(tiny.hyper(name), dtype, seed=11), load_model(d, dtype)
            for pm, pd in zip(mem.all_parts(), disk.all_parts()):
                for n, tm in vars(pm).items():
                    if torch.is_tensor(tm):
                        assert tm.is_cuda and torch.equal(tm, getattr(pd, n)), f"{name} {type(pm).__name__}.{n}"
            logits = []
            for model in (mem, disk):
                runner = ModelRunner(model, CacheParam(page_size=tiny.PAGE_SIZE[name], num_pages=40, max_seqs=1))
                runner.admit(0)
                logits.append(runner.step([StepEntry(0, toks, list(range(len(toks))))]).clone())
            assert torch.equal(logits[0], logits[1])
            if dtype == torch.float32:       # and the folder's logits are the plain implementation's
                ref = plain_opt.forward(cfg, w, toks)
                assert (logits[0].double().cpu() - ref).abs().max() <= 2e-5 + 1e-4 * ref.abs().max()


def test_many_requests_arriving_over_time(models):
    """Sixty requests of mixed lengths, sampling settings and end tokens arrive a few at a time
    into an engine with few slots and few pages (so that requests wait, are pre-empted and pages
    are used again and again).  Everything ends, nothing is lost, and in float32 the outputs are
    those of an engine that never queues a step ahead."""
    import random
    from swifttransformer_amd.engine.engine import Engine
    from swifttransformer_amd.sampling import SamplingParams
    d, cfg, w = models["B"]
    V = cfg["vocab_size"]
    rng = random.Random(5)
    reqs = []
    for i in range(60):
        n = rng.choice([1, 2, 5, 9, 17, 40, 70])
        sp = SamplingParams(max_new_tokens=rng.choice([1, 2, 7, 20, 45]), temperature=rng.choice([0.0, 0.7, 1.3]),
                            seed=100 + i, eos_token_id=rng.randrange(V) if i % 3 else None, ignore_eos=(i % 3 == 0))
        reqs.append((tiny.prompt(n, V, 500 + i), sp))

    def run(lookahead):
        eng = Engine(d, dtype="fp32", page_size=8, num_pages=26, max_seqs=6, max_batched_tokens=64,
                     prefill_chunk=24, lookahead=lookahead)
        done, pending, steps = {}, list(enumerate(reqs)), 0
        while pending or eng.has_work():
            if steps % 2 == 0:
                for i, (p, sp) in pending[:3]:
                    eng.add_request(p, sp, req_id=i)
                pending = pending[3:]
            for o in eng.step():
                done[o.req_id] = (o.output, o.finish_reason)
            steps += 1
            assert steps < 5000
        eng.runner.manager.check_invariants()
        assert eng.runner.manager.num_free_pages() == 26 and eng.runner.manager.num_free_slots == 6
        return done, eng.stats

    ahead, stats = run(True)
    assert len(ahead) == 60 and all(1 <= len(o) <= sp.max_new_tokens for (o, _), (_, sp) in
                                    ((ahead[i], reqs[i]) for i in range(60)))
    assert stats.preemptions > 0
    plain, _ = run(False)
    assert ahead == plain
    # one request against the plain implementation, to tie the two to something outside the engine
    i = next(i for i, (p, sp) in enumerate(reqs) if sp.temperature == 0.0 and sp.ignore_eos and sp.max_new_tokens >= 7)
    assert ahead[i][0] == plain_opt.generate(cfg, w, reqs[i][0], len(ahead[i][0]))
