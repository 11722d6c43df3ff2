"""Benchmark of a static batch whose requests all hold the same input, in the manner of the
reference's ``benchmark_all_input_same``
(src/examples/benchmark_all_input_same.cc:371-386):

    benchmark_all_input_same model_name precision exp_params_name [-m model_path|dummy]

``model_name``: a named size of a registered architecture (opt_125m ... opt_30b); ``precision``: bf16 or fp32;
``exp_params_name``: a named list of experiments, each (input_len, batch_size, block_size,
num_decoding_step) as in the reference (:29-34); ``-m``: a model folder, or ``dummy`` (the
default) for random weights (:233-238).  Every experiment runs all prompts in one context step
and then decodes in lock-step (src/examples/lib/inference_batch.cc:110-118, :163-220), once to
warm up and once timed, and the results are printed as the reference's table (:325-347).
The input is a seeded random token sequence instead of the reference's counting sentence."""
from __future__ import annotations

import argparse
import time
from typing import Dict, List, NamedTuple, Optional


class ExperimentParameters(NamedTuple):
    input_len: int          # tokens of every input sequence
    batch_size: int         # number of input sequences
    block_size: int         # tokens per cache block
    num_decoding_step: int  # tokens generated per sequence


def _sweep(input_len, batch_sizes, block_sizes, steps) -> List[ExperimentParameters]:
    return [ExperimentParameters(input_len, b, bs, steps) for b in batch_sizes for bs in block_sizes]


EXPERIMENTS: Dict[str, List[ExperimentParameters]] = {
    "diff_block_size_small": _sweep(32, [4], [1, 2, 4, 8, 16, 32], 32),
    "diff_block_size_large_batch": _sweep(32, [128], [4, 16, 32], 32),
    "diff_block_size_large_input": _sweep(512, [4], [4, 16, 32], 16),
    "diff_batch_size": _sweep(1024, [1, 2, 4, 8, 16, 32, 64], [16], 128),
    "headline": _sweep(1024, [1, 8, 64], [16], 256),
    "smoke": _sweep(16, [2], [4], 4),
}


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(
        prog="benchmark_all_input_same",
        description="This program runs a static batch of identical inputs through the model "
                    "and reports the time of the context stage and of the decoding stage.")
    ap.add_argument("model_name", help="Name of the model (opt_125m, opt_1.3b, ..., opt_30b)")
    ap.add_argument("precision", help="Precision used for inference (bf16 or fp32)")
    ap.add_argument("exp_params_name", help="Name of the experiment parameters: " + ", ".join(EXPERIMENTS))
    ap.add_argument("-m", "--model_path", default="dummy",
                    help="Path to the model folder, or 'dummy' for random weights")
    ap.add_argument("--layers", type=int, default=0, help="run only this many layers (dummy weights)")
    ap.add_argument("--seed", type=int, default=0)
    return ap


def run_experiment(model, dtype, exp: ExperimentParameters, vocab: int, seed: int):
    """(context stage ms, decoding stage ms, first request's output) of one timed run."""
    import torch
    from ..engine.engine import Engine
    from ..sampling import SamplingParams
    total = exp.input_len + exp.num_decoding_step
    pages_per_req = -(-total // exp.block_size) + 1
    eng = Engine(model, dtype=dtype, page_size=exp.block_size, num_pages=pages_per_req * exp.batch_size + 1,
                 max_seqs=exp.batch_size, max_batched_tokens=exp.batch_size * exp.input_len,
                 prefill_chunk=exp.input_len)
    g = torch.Generator().manual_seed(seed)
    tokens = torch.randint(0, vocab, (exp.input_len,), generator=g).tolist()
    result = None
    # The passes before the timed one see the prompt step and the decode step as often as it takes
    # for both to be recorded (a step's shape is recorded when it comes up again): the timed pass
    # then replays them, as a server in its steady state does.
    warm_ups = max(1, eng.runner.record_after if eng.runner.use_graphs else 1)
    for timed in [False] * warm_ups + [True]:
        ids = [eng.add_request(tokens, SamplingParams(max_new_tokens=exp.num_decoding_step, ignore_eos=True))
               for _ in range(exp.batch_size)]
        torch.cuda.synchronize()
        ahead, eng.lookahead = eng.lookahead, False          # or the first decode step would be queued, and timed, with the prompts
        t0 = time.perf_counter()
        done = {o.req_id: o.output for o in eng.step()}      # all prompts in one step
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        eng.lookahead = ahead
        while eng.has_work():
            for o in eng.step():
                done[o.req_id] = o.output
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if timed:
            result = ((t1 - t0) * 1e3, (t2 - t1) * 1e3, done[ids[0]])
    return result


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from ..config.registry import hyper_param_by_name
    from ..engine.engine import parse_dtype
    from ..models import load_model, random_model
    try:
        dtype = parse_dtype(args.precision)
    except ValueError as e:
        print(f"Invalid precision: {args.precision}\nValid precision: bf16, fp32 ({e})")
        return 1
    if args.exp_params_name not in EXPERIMENTS:
        print(f"Invalid experiment parameters name: {args.exp_params_name}")
        print("Valid experiment parameters name:")
        for name in EXPERIMENTS:
            print(f"\t{name}")
        return 1
    print("Loading model...")
    if args.model_path == "dummy":
        print("No model path specified, using dummy weights")
        try:
            hp = hyper_param_by_name(args.model_name, **({"num_hidden_layers": args.layers} if args.layers else {}))
        except KeyError as e:
            print(f"Invalid number of parameters: {args.model_name}")
            print(e.args[0])
            return 1
        model = random_model(hp, dtype, args.seed, "cuda:0")
    else:
        model = load_model(args.model_path, dtype, "cuda:0")
        hp = model.hyper_param
    results = []
    for exp in EXPERIMENTS[args.exp_params_name]:
        print("--------")
        print("Exp params:")
        print(f"\tinput_len: {exp.input_len}")
        print(f"\tbatch_size: {exp.batch_size}")
        print(f"\tblock_size: {exp.block_size}")
        print(f"\tnum_decoding_step: {exp.num_decoding_step}")
        print("Warming up... Running...")
        context_ms, decode_ms, out = run_experiment(model, dtype, exp, hp.vocab_size, args.seed)
        print("Time usage:")
        print(f"\tContext stage: {context_ms:.2f} ms")
        print(f"\tRegression stage: {decode_ms:.2f} ms")
        print(f"\tTotal: {context_ms + decode_ms:.2f} ms")
        print("Model output:")
        print("(...) " + " ".join(str(t) for t in out[:16]) + f"  ({len(out)} tokens generated)")
        results.append((exp, context_ms, decode_ms))
    print(f"\nExperiment parameters: {args.exp_params_name}")
    print("Results:")
    print("  block_size   input_len  batch_size decode_step context_t(ms)  decode_t(ms)   total_t(ms)")
    for exp, c, d in results:
        print(f"{exp.block_size:12d}{exp.input_len:12d}{exp.batch_size:12d}{exp.num_decoding_step:12d}"
              f"{c:14.2f}{d:14.2f}{c + d:14.2f}")
    print("\nThe following table is formatted with tabs(\\t) for easy copy-paste.")
    for exp, c, d in results:
        print(f"{exp.block_size}\t{exp.input_len}\t{exp.batch_size}\t{exp.num_decoding_step}\t{c:.2f}\t{d:.2f}\t{c + d:.2f}")
    return 0
