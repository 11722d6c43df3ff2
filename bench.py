#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on OPT-1.3B layer sizes (random weights).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--dtype bf16|fp32]

A step is one decode step of the whole engine loop (scheduler, step function,
sampling, token ids back on the host) with `batch` requests whose prompts hold
1,024 tokens and which decode up to the 2,048-token context.  With the default
K = 1024 the timed steps cover all of that; a smaller K times the K steps in the
middle of it (after untimed steps), so that their mean context is the workload's.
Prints ONE JSON line: decode tokens/s (`value`), a 2,048-token prefill, the decode
step's fraction of the HBM roofline, and decode at batch 1 and 64.
The reference ships a benchmark program with the same shape of workload
(src/examples/benchmark_all_input_same.cc:95-108, :266-296) and no numbers.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBS = 8000.0                       # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# OPT-1.3B layer sizes (src/examples/lib/common_gpt_hyper_params.h:20-28)
MODEL = dict(vocab_size=50272, max_position_embeddings=2048, hidden_size=2048, num_hidden_layers=24,
             num_attention_heads=32, ffn_dim=8192, word_embed_proj_dim=2048, do_layer_norm_before=True,
             enable_bias=True)
PROMPT_LEN = 1024
CONTEXT = 2048
PAGE = 16
# layer sizes of the OPT family (common_gpt_hyper_params.h:10-68)
SHAPES = {
    "125m": dict(hidden_size=768, num_hidden_layers=12, num_attention_heads=12, ffn_dim=3072),
    "1.3b": dict(hidden_size=2048, num_hidden_layers=24, num_attention_heads=32, ffn_dim=8192),
    "2.7b": dict(hidden_size=2560, num_hidden_layers=32, num_attention_heads=32, ffn_dim=10240),
    "6.7b": dict(hidden_size=4096, num_hidden_layers=32, num_attention_heads=32, ffn_dim=16384),
    "13b": dict(hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, ffn_dim=20480),
    "30b": dict(hidden_size=7168, num_hidden_layers=48, num_attention_heads=56, ffn_dim=28672),
}


def build_engine(layers: int, dtype: str, max_seqs: int, num_pages: int, seed: int = 0, shape: str = "1.3b",
                 max_batched_tokens: int = 0, prefill_chunk: int = 2048, gpu_mem_fraction: float = 0.0):
    import torch
    from swifttransformer_amd.config import OptHyperParam
    from swifttransformer_amd.engine.engine import Engine, parse_dtype
    from swifttransformer_amd.models import random_model
    sizes = dict(MODEL, **SHAPES[shape])
    sizes["word_embed_proj_dim"] = sizes["hidden_size"]
    if layers:
        sizes["num_hidden_layers"] = layers
    hp = OptHyperParam(**sizes).validate()
    dt = parse_dtype(dtype)
    model = random_model(hp, dt, seed, "cuda:0")
    # every prompt of a batch is run in one step, so that all requests decode in lock-step
    eng = Engine(model, dtype=dt, page_size=PAGE, num_pages=num_pages, max_seqs=max_seqs,
                 max_batched_tokens=max_batched_tokens or max_seqs * PROMPT_LEN, prefill_chunk=prefill_chunk,
                 gpu_mem_fraction=gpu_mem_fraction)
    return eng, hp


def prompts(batch: int, length: int, vocab: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (batch, length), generator=g).tolist()


def decode_run(eng, batch: int, steps: int, warmup: int, vocab: int, seed: int, centre: bool = True):
    """(seconds, device steps run in them, tokens decoded, context of the first timed step).

    The workload decodes from 1,024-token prompts up to the 2,048-token context; when fewer
    steps are timed than that takes, the timed ones lie in the middle of it (``centre``), after
    untimed decode steps, so that their mean context is the workload's.  Warm-up runs on
    requests of its own.  Steps are counted on the device: the engine queues a step ahead of
    the host, so the prompts and the untimed steps run without that, and exactly the steps
    launched between the two synchronisations are timed."""
    import torch
    from swifttransformer_amd.sampling import SamplingParams

    def start(n_new, sd):
        for p in prompts(batch, PROMPT_LEN, vocab, sd):
            eng.add_request(p, SamplingParams(max_new_tokens=n_new, ignore_eos=True))
        while any(r.pending > 1 for r in eng.requests.values()) or eng.scheduler.waiting:
            eng.step()                       # prompts (untimed here)

    if warmup > 0:
        start(warmup + 1, seed + 1)
        while eng.has_work():
            eng.step()
    skip = max(0, (CONTEXT - PROMPT_LEN - steps) // 2) if centre else 0
    ahead = eng.lookahead
    eng.lookahead = False                    # nothing of the timed steps is queued before t0
    start(skip + steps + 1, seed)            # the prompt step yields the first token
    for _ in range(skip):
        eng.step()
    torch.cuda.synchronize()
    eng.lookahead = ahead
    first = eng.runner.steps_run
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ran = eng.runner.steps_run - first
    while eng.has_work():
        eng.step()
    return dt, ran, ran * batch, PROMPT_LEN + skip


def prefill_run(eng, tokens: int, vocab: int, reps: int = 3):
    import torch
    from swifttransformer_amd.sampling import SamplingParams
    best = None
    for i in range(reps + 1):
        eng.add_request(prompts(1, tokens, vocab, 100 + i)[0], SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        while eng.has_work():
            eng.step()
        if i > 0:                            # the first one warms up
            best = dt if best is None else min(best, dt)
    return best


def weight_bytes(hp, elem: int) -> int:
    H, F, V, L = hp.hidden_size, hp.ffn_dim, hp.vocab_size, hp.num_hidden_layers
    per_layer = (4 * H * H + 2 * H * F) * elem + (4 * H + F + H + 4 * H) * 4
    return L * per_layer + V * hp.word_embed_proj_dim * elem      # every matrix once; the head once


def prefill_flops(hp, T: int) -> float:
    H, F, V, L = hp.hidden_size, hp.ffn_dim, hp.vocab_size, hp.num_hidden_layers
    linear = 2.0 * T * (4 * H * H + 2 * H * F) * L
    attn = 2.0 * 2.0 * H * (T * (T + 1) / 2) * L      # QK^T and PV over the causal half
    return linear + attn + 2.0 * H * V                # one row through the head


def kernel_times(args) -> int:
    """Per-kernel times and roofline fractions of one decode step (batch `--batch`, every request
    at a context of 1,536 tokens) and of the 2,048-token prefill, from event pairs around every
    kernel call of unrecorded steps.  The kernels are the recorded step's; between them the
    device waits for the host here, so the sum of the calls, not the step's wall time, is what
    compares with a recorded step."""
    import torch
    from swifttransformer_amd.engine.step import StepEntry
    from swifttransformer_amd.ops.profile import KernelTimer
    batch, ctx_len = args.batch, 1536
    num_pages = (batch + 1) * (CONTEXT // PAGE) + 8
    eng, hp = build_engine(args.layers, args.dtype, max_seqs=max(batch, 2), num_pages=num_pages)
    runner = eng.runner
    runner.use_graphs = False
    V = hp.vocab_size
    elem = 2 if args.dtype == "bf16" else 4
    toks = prompts(batch + 1, CONTEXT, V, 5)
    for i in range(batch):
        runner.admit(i)
        runner.step([StepEntry(i, toks[i][:ctx_len], [])])
    out = {}

    def attention_cost(keys_read: int, pairs: float):
        def nbytes(name, info):
            if name in ("attention_rows", "attention_prefill"):
                return 2 * keys_read * info["kv_heads"] * info["head_dim"] * info["elem"]
            return None

        def flops(name, info):
            if name in ("attention_rows", "attention_prefill"):
                return 4.0 * pairs * info["heads"] * info["head_dim"]
            return None
        return nbytes, flops

    def run(label, entries_of, reps, keys_read, pairs):
        for k in range(2):
            runner.step(entries_of(k))                       # warm: code objects, library plans
        with KernelTimer() as t:
            for k in range(2, 2 + reps):
                runner.step(entries_of(k))
        rows = t.summary(*attention_cost(keys_read, pairs))
        for r in rows:
            r["calls"] //= reps
            r["us_total"] = round(r["us_total"] / reps, 1)
        out[label] = {"us_sum_of_calls": round(sum(r["us_total"] for r in rows), 1), "kernels": rows}

    # decode: the keys a step reads grow by one per request and step; priced at the middle one
    reps = 8
    run(f"decode_b{batch}_ctx{ctx_len}",
        lambda k: [StepEntry(i, [toks[i][ctx_len + k]], [0]) for i in range(batch)], reps,
        keys_read=batch * (ctx_len + 2 + reps // 2), pairs=batch * (ctx_len + 2 + reps // 2))
    for i in range(batch):
        runner.finish(i)

    def prefill(k):
        if runner.is_live("p"):
            runner.finish("p")
        runner.admit("p")
        return [StepEntry("p", toks[batch], [CONTEXT - 1])]
    run("prefill_2048", prefill, 3, keys_read=CONTEXT, pairs=CONTEXT * (CONTEXT + 1) / 2.0)
    print(json.dumps({"kernel_times": out, "dtype": args.dtype, "layers": hp.num_hidden_layers,
                      "method": "event pairs around kernel calls of unrecorded steps, event overhead taken off"}))
    return 0


def attention_only(args) -> int:
    """The prompt attention kernel alone on the model's geometry (one 2,048-row prompt, keys and
    values of one layer), three calls: for counter runs under the profiler.  `--attention-algo`
    1 is the kernel that stages key blocks through registers, 2 the one that loads them straight
    into LDS, 0 the library's choice."""
    import math
    import torch
    from swifttransformer_amd.ops import kernels as K
    sizes = dict(MODEL, **SHAPES["1.3b"])
    nh, hd, n = sizes["num_attention_heads"], sizes["hidden_size"] // sizes["num_attention_heads"], 2048
    dev = "cuda:0"
    pages = n // PAGE
    g = torch.Generator(device=dev).manual_seed(0)
    kc = torch.randn((pages, nh, PAGE, hd), generator=g, device=dev).bfloat16()
    vc = torch.randn((pages, nh, PAGE, hd), generator=g, device=dev).bfloat16()
    q = torch.randn((n, nh * hd), generator=g, device=dev).bfloat16()
    bt = torch.randperm(pages, generator=g, device=dev).to(torch.int32).view(1, pages)
    rows = K.prefill_tile_rows(hd, PAGE, pages, nh, n, torch.bfloat16) if args.attention_algo != 1 else 64
    tq = torch.arange(0, n, rows, dtype=torch.int32, device=dev)
    ti = torch.zeros_like(tq)
    zero, length = torch.zeros(1, dtype=torch.int32, device=dev), torch.full((1,), n, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    for i in range(3):
        ev[i].record()
        K.attention_prefill(q, kc, vc, ti, tq, zero, zero, length, bt, nh, 1 / math.sqrt(hd), out=out,
                            tile_rows=rows, algo=args.attention_algo)
    ev[3].record()
    torch.cuda.synchronize()
    us = min(ev[i].elapsed_time(ev[i + 1]) for i in range(3)) * 1e3
    flops = 4.0 * hd * nh * n * (n + 1) / 2
    print(json.dumps({"attention_prefill": {"rows": n, "heads": nh, "head_dim": hd, "tile_rows": rows,
                                            "algo": args.attention_algo, "us": round(us, 1),
                                            "TFLOP/s": round(flops / us / 1e6, 1)}}))
    return 0


def mixed_workload(args, shape: str = "6.7b") -> int:
    """64 requests with prompt lengths uniform in [32, 2048), prompt portions of 512 tokens running
    beside decode tokens, 128 output tokens each, at the layer sizes of ``shape`` (the OPT-6.7B
    ones are the configuration's; the 1.3B ones show the same steps where they are short)."""
    import torch
    from swifttransformer_amd.sampling import SamplingParams
    n_req, n_out = 64, 128
    eng, hp = build_engine(args.layers if args.layers != MODEL["num_hidden_layers"] else 0, args.dtype,
                           max_seqs=n_req, num_pages=n_req * (CONTEXT // PAGE), shape=shape,
                           max_batched_tokens=512 + n_req, prefill_chunk=512)
    def run(seed):
        g = torch.Generator().manual_seed(seed)
        lens = torch.randint(32, 2048 - n_out, (n_req,), generator=g).tolist()
        for i, n in enumerate(lens):
            eng.add_request(prompts(1, n, hp.vocab_size, 200 * seed + i)[0],
                            SamplingParams(max_new_tokens=n_out, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.has_work():
            eng.step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    # one full run of other requests first, as the reference's benchmark warms up
    # (src/examples/benchmark_all_input_same.cc:266-296): code objects, recorded decode steps
    run(3)
    eng.stats = type(eng.stats)(step_log=[])
    dt = run(7)
    st = eng.stats
    # floor of every step: its bytes (every weight once, the keys and values of what its requests
    # hold) against the HBM peak, and its arithmetic (the layers' products per token, the
    # attention's query-key pairs, one head row per sampled token, roughly per request and step)
    # against the matrix peak; the larger of the two
    elem = 2 if args.dtype == "bf16" else 4
    H, F, L, V = hp.hidden_size, hp.ffn_dim, hp.num_hidden_layers, hp.vocab_size
    w_bytes = weight_bytes(hp, elem)
    kv_per_token = 2 * L * H * elem
    floor = hbm_s = flop_s = 0.0
    for n_tok, keys, pairs in st.step_log:
        t_b = (w_bytes + keys * kv_per_token) / (HBM_PEAK_GBS * 1e9)
        t_f = (2.0 * n_tok * (4 * H * H + 2 * H * F) * L + 4.0 * pairs * H * L) / PEAK_FLOPS[args.dtype]
        floor += max(t_b, t_f)
        hbm_s += t_b
        flop_s += t_f
    print(json.dumps({
        "metric": f"mixed continuous batch, OPT-{shape.upper()} shape: tokens/s", "value": round((st.prompt_tokens + st.generated_tokens) / dt, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": st.steps, "ms_per_step": round(dt / st.steps * 1e3, 3),
        "dtype": args.dtype, "data": "synthetic",
        "config": {"model": f"opt-{shape} layer sizes, random weights", "layers": hp.num_hidden_layers,
                   "layers_of_config": SHAPES[shape]["num_hidden_layers"], "requests": n_req,
                   "prompt_tokens": st.prompt_tokens, "generated_tokens": st.generated_tokens,
                   "prefill_chunk": 512, "seconds": round(dt, 3), "preemptions": st.preemptions,
                   "generated_per_s": round(st.generated_tokens / dt, 1), "pages_used_peak": st.pages_used_peak},
        "roofline": {"bound": "per step the larger of hbm and matrix", "floor_s": round(floor, 4),
                     "hbm_floor_s": round(hbm_s, 4), "matrix_floor_s": round(flop_s, 4),
                     "frac": round(floor / dt, 4)}}))
    return 0


def ttft(args) -> int:
    """Time to the first token of one prompt of 32, 128, 512 and 2,048 tokens alone in the engine
    (request added -> its first token on the host), best of a few runs after a warm-up of the same
    length, with the floor of such a step: every weight once against the HBM peak, or its
    arithmetic against the matrix peak, whichever is larger."""
    eng, hp = build_engine(args.layers, args.dtype, max_seqs=4, num_pages=4 * (CONTEXT // PAGE))
    elem = 2 if args.dtype == "bf16" else 4
    out = {}
    for n in (32, 128, 512, 2048):
        t = prefill_run(eng, n, hp.vocab_size, reps=5)
        floor = max(weight_bytes(hp, elem) / (HBM_PEAK_GBS * 1e9), prefill_flops(hp, n) / PEAK_FLOPS[args.dtype])
        out[str(n)] = {"ms": round(t * 1e3, 3), "floor_ms": round(floor * 1e3, 3), "frac": round(floor / t, 3)}
    print(json.dumps({"metric": "time to first token of one prompt alone, OPT-1.3B shape", "unit": "ms",
                      "higher_is_better": False, "n_gpus": 1, "dtype": args.dtype, "data": "synthetic",
                      "config": {"model": "opt-1.3b layer sizes, random weights", "layers": hp.num_hidden_layers,
                                 "layers_of_config": MODEL["num_hidden_layers"]},
                      "value": out["128"]["ms"], "prompts": out,
                      "graph_replays": eng.runner.graph_replays, "steps_run": eng.runner.steps_run}))
    return 0


def floors(args) -> int:
    """What the card gives a kernel of this engine at best, measured: the rate of a plain streaming
    read (grid-stride, consecutive lanes read consecutive 16 bytes) of buffers of 32 MB (a layer's
    largest matrix at the OPT-1.3B sizes), 206 MB (its head) and 800 MB (the keys and values a
    batch-64 decode step reads in a layer), each read from memory (a ring of buffers larger than
    the 256 MB cache); and what a kernel costs in a recorded chain of dependent kernels before it
    streams anything: a chain of kernels without work, and the 32 MB read in a chain of its kind
    against the same bytes at the plain rate."""
    import torch
    from swifttransformer_amd.ops import kernels as K
    dev = "cuda:0"
    units = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)

    def timed_graph(build, reps=5):
        build()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            build()
        g.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            g.replay()
            e.record()
            torch.cuda.synchronize()
            t = s.elapsed_time(e) * 1e3
            best = t if best is None else min(best, t)
        return best       # microseconds for the whole chain

    out = {"compute_units": units, "stream": {}, "chain": {}}
    n_chain = 48
    for label, mb in (("32MB", 32), ("206MB", 206), ("800MB", 800)):
        ring = max(2, -(-640 // mb))                      # the ring holds at least 640 MB
        bufs = [torch.empty(mb << 20, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(ring)]
        best = {}
        calls = max(ring, n_chain // max(1, mb // 32))
        for pattern, name in ((0, "stride4"), (1, "stride8"), (2, "tiles8K"), (3, "tiles16K"), (4, "rows4K"), (5, "rows16K")):
            for per_unit in (1, 2, 4, 8):
                wgs = units * per_unit
                us = timed_graph(lambda: [K.probe_read(bufs[i % ring], sink, wgs, pattern) for i in range(calls)])
                best[f"{name}x{per_unit}"] = us / calls
        per_call = min(best.values())
        out["stream"][label] = {"us_per_call_in_chain": round(per_call, 2),
                                "GB/s_in_chain": round((mb << 20) / per_call / 1e3, 1),
                                "best_shape": min(best, key=best.get),
                                "us_by_pattern_x_workgroups_per_unit": {k: round(v, 2) for k, v in best.items()}}
        del bufs
        torch.cuda.empty_cache()
    empty_us = timed_graph(lambda: [K.probe_empty(sink) for _ in range(4 * n_chain)]) / (4 * n_chain)
    out["chain"]["empty_kernel_us"] = round(empty_us, 2)
    # the long read's rate has the chain's per-kernel cost spread thin: take it as the streaming rate
    rate = (800 << 20) / out["stream"]["800MB"]["us_per_call_in_chain"]          # bytes per microsecond
    small = out["stream"]["32MB"]["us_per_call_in_chain"]
    out["chain"]["stream_rate_GB/s"] = round(rate / 1e3, 1)
    out["chain"]["32MB_read_us"] = small
    out["chain"]["32MB_at_stream_rate_us"] = round((32 << 20) / rate, 2)
    out["chain"]["cost_of_a_dependent_kernel_us"] = round(small - (32 << 20) / rate, 2)
    # how fast a compute unit is filled: every workgroup goes round its own region, all regions
    # together within the L2s (64 KB each) or far beyond every cache (4 MB each, two a unit)
    out["fill"] = {}
    for label, region, per_unit, turns in (("from_L2", 64 << 10, 1, 2000), ("from_memory", 4 << 20, 2, 256)):
        wgs = units * per_unit
        src = torch.empty(wgs * region, dtype=torch.uint8, device=dev).random_(0, 255)
        for to_lds in (True, False):
            us = timed_graph(lambda: K.probe_fill(src, region, sink, wgs, turns, to_lds))
            rate = wgs * turns * 32768.0 / us                       # bytes per microsecond, whole device
            out["fill"][f"{label}_{'direct_to_LDS' if to_lds else 'to_registers'}"] = {
                "GB/s_per_unit": round(rate / 1e3 / units, 1), "TB/s_device": round(rate / 1e6, 2)}
        del src
        torch.cuda.empty_cache()
    # the rate at which one or two waves a SIMD issue matrix-core products (bfloat16, no memory traffic)
    out["matrix_core"] = {"peak_TFLOP/s": PEAK_FLOPS["bf16"] / 1e12}
    rounds = 4000
    for wide, name, flops in ((False, "16x16x32", 2.0 * 16 * 16 * 32), (True, "32x32x16", 2.0 * 32 * 32 * 16)):
        for waves in (1, 2):
            wgs = units * waves
            us = timed_graph(lambda: K.probe_mfma(sink, wgs, rounds, wide))
            out["matrix_core"][f"{name}_{waves}_wave{'s' if waves > 1 else ''}_a_SIMD_TFLOP/s"] = round(
                wgs * 4 * rounds * 16 * flops / us / 1e6, 1)
    out["hbm_peak_GB/s"] = HBM_PEAK_GBS
    print(json.dumps({"floors": out}))
    return 0


def decode_30b(args) -> int:
    """OPT-30B shape, decode at batch 1/8/64 after 1,024-token prompts,
    256 output tokens, the cache pool sized from the HBM left after the weights."""
    eng, hp = build_engine(args.layers if args.layers != MODEL["num_hidden_layers"] else 0, args.dtype,
                           max_seqs=64, num_pages=0, shape="30b", gpu_mem_fraction=0.85)
    elem = 2 if args.dtype == "bf16" else 4
    kv_per_token = 2 * hp.num_hidden_layers * hp.hidden_size * elem
    points, fracs = {}, {}
    for b in (1, 8, 64):
        k = min(args.steps, 256)
        dt, ran, n, ctx0 = decode_run(eng, b, k, min(args.warmup, 4), hp.vocab_size, seed=30 + b, centre=False)
        points[f"decode_b{b}"] = round(n / dt, 1)
        step_bytes = weight_bytes(hp, elem) + b * (ctx0 + (ran + 1) / 2.0) * kv_per_token
        fracs[f"hbm_frac_b{b}"] = round(step_bytes / (dt / ran) / 1e9 / HBM_PEAK_GBS, 4)
    print(json.dumps({
        "metric": "decode tok/s at batch 1/8/64, OPT-30B shape", "value": points["decode_b8"], "unit": "tokens/s",
        "n_gpus": 1, "steps": min(args.steps, 256), "dtype": args.dtype, "data": "synthetic",
        "config": {"model": "opt-30b layer sizes, random weights", "layers": hp.num_hidden_layers,
                   "layers_of_config": SHAPES["30b"]["num_hidden_layers"], "prompt_len": PROMPT_LEN,
                   "cache_pages": eng.runner.cache_param.num_pages, "page_size": PAGE},
        "points": points, "roofline": dict(bound="hbm", peak=HBM_PEAK_GBS, unit="GB/s", **fracs)}))
    return 0


def decode_family(args) -> int:
    """Decode at batch 1/8/64 around context 1,536 and a 2,048-token prefill at the layer sizes of
    the OPT family from 125M to 13B (the 30B shape has a workload of its own): how the kernels'
    dispatch rules, fitted at some of these sizes, hold at the others."""
    import torch
    elem = 2 if args.dtype == "bf16" else 4
    sizes = {}
    for shape in ("125m", "1.3b", "2.7b", "6.7b", "13b"):
        row = {}
        for b in (1, 8, 64):
            eng, hp = build_engine(0, args.dtype, max_seqs=b, num_pages=(b + 1) * (CONTEXT // PAGE + 2), shape=shape)
            k = min(args.steps, 96 if b < 64 else 48)
            dt, ran, n, ctx0 = decode_run(eng, b, k, min(args.warmup, 8), hp.vocab_size, seed=40 + b)
            kv = 2 * hp.num_hidden_layers * hp.hidden_size * elem * b * (ctx0 + (ran + 1) / 2.0)
            row[f"decode_b{b}"] = round(n / dt, 1)
            row[f"hbm_frac_b{b}"] = round((weight_bytes(hp, elem) + kv) / (dt / ran) / 1e9 / HBM_PEAK_GBS, 3)
            if b == 8:
                pt = prefill_run(eng, 2048, hp.vocab_size)
                row["prefill_ms"] = round(pt * 1e3, 2)
                row["prefill_frac"] = round(prefill_flops(hp, 2048) / pt / PEAK_FLOPS[args.dtype], 3)
            del eng
            torch.cuda.empty_cache()
        sizes[shape] = row
    print(json.dumps({"metric": "decode tok/s at batch 1/8/64 and 2,048-token prefill, OPT family layer sizes",
                      "unit": "tokens/s", "n_gpus": 1, "dtype": args.dtype, "data": "synthetic", "sizes": sizes}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=MODEL["num_hidden_layers"])
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1/64 and prefill measurements")
    ap.add_argument("--kernel-times", action="store_true",
                    help="per-kernel times and roofline fractions of a decode step and of the prefill; own line")
    ap.add_argument("--attention-only", action="store_true",
                    help="three calls of the prompt attention kernel alone (for counter runs); own line")
    ap.add_argument("--attention-algo", type=int, default=0, choices=[0, 1, 2])
    ap.add_argument("--floors", action="store_true",
                    help="the card's plain streaming read rate and the cost of a kernel in a recorded chain; own line")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill (for profiling); prints its own line")
    ap.add_argument("--workload", default="decode-1.3b",
                    choices=["decode-1.3b", "mixed-6.7b", "mixed-1.3b", "ttft", "decode-30b", "decode-family"],
                    help="decode-1.3b is the contract's line; the others are the other model shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU")
        return 1
    if args.floors:
        return floors(args)
    if args.kernel_times:
        return kernel_times(args)
    if args.attention_only:
        return attention_only(args)
    if args.workload in ("mixed-6.7b", "mixed-1.3b"):
        return mixed_workload(args, args.workload.split("-")[1])
    if args.workload == "ttft":
        return ttft(args)
    if args.workload == "decode-30b":
        return decode_30b(args)
    if args.workload == "decode-family":
        return decode_family(args)
    steps = min(args.steps, CONTEXT - PROMPT_LEN)
    elem = 2 if args.dtype == "bf16" else 4
    biggest = max(args.batch, 1 if (args.no_points or args.prefill_only) else 64)
    num_pages = biggest * (CONTEXT // PAGE) + 2 * (CONTEXT // PAGE)
    eng, hp = build_engine(args.layers, args.dtype, max_seqs=biggest, num_pages=num_pages)
    V = hp.vocab_size
    if args.prefill_only:
        pt = prefill_run(eng, 2048, V)
        print(json.dumps({"prefill": {"value": round(2048 / pt, 1), "tokens": 2048, "ms": round(pt * 1e3, 3),
                                      "frac": round(prefill_flops(hp, 2048) / pt / PEAK_FLOPS[args.dtype], 4)}}))
        return 0

    dt, ran, n, ctx0 = decode_run(eng, args.batch, steps, args.warmup, V, seed=1)
    if ran != steps:
        print(f"bench.py: {ran} decode steps ran in the timed window, {steps} were asked for", file=sys.stderr)
    ms_step = dt / ran * 1e3
    value = n / dt
    kv_per_token = 2 * hp.num_hidden_layers * hp.hidden_size * elem
    mean_ctx = ctx0 + (ran + 1) / 2.0        # keys a timed step reads per request, on average
    step_bytes = weight_bytes(hp, elem) + args.batch * mean_ctx * kv_per_token
    achieved = step_bytes / (dt / ran) / 1e9
    out = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens (OPT-1.3B)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"model": "opt-1.3b layer sizes, random weights", "global_batch": args.batch,
                   "seq_len": CONTEXT, "parallelism": "single-gpu", "layers": args.layers,
                   "layers_of_config": MODEL["num_hidden_layers"], "hidden_size": hp.hidden_size,
                   "heads": hp.num_attention_heads, "head_dim": hp.head_dim, "ffn_dim": hp.ffn_dim,
                   "vocab_size": V, "prompt_len": PROMPT_LEN, "context_first": ctx0,
                   "context_last": ctx0 + ran, "page_size": PAGE, "prefill_tokens": 2048},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        pt = prefill_run(eng, 2048, V)
        fl = prefill_flops(hp, 2048)
        out["prefill"] = {"value": round(2048 / pt, 1), "tokens": 2048, "ms": round(pt * 1e3, 3),
                          "frac": round(fl / pt / PEAK_FLOPS[args.dtype], 4)}
        points = {}
        for b, k in ((1, min(steps, 256)), (64, min(steps, 128))):
            d, _, m, _ = decode_run(eng, b, k, min(args.warmup, 8), V, seed=2 + b)
            points[f"decode_b{b}"] = round(m / d, 1)
        out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
