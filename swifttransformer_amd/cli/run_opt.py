"""Command line in the manner of the reference's ``run_gpt``
(src/examples/run_gpt.cc:170-188):

    run_opt model_path model_name [-v vocab_json_path] precision input_path [-d]

``model_path`` is a model folder (config.json + safetensors); ``model_name`` is the
reference's family_size name (``opt_1.3b``): only its family is checked against
config.json, because every size comes from config.json here (``auto`` skips the
check); ``precision`` is ``bf16`` or ``fp32`` (the reference: fp16|fp32);
``input_path`` holds one request per line, whitespace-separated token ids
(run_gpt.cc:73-90).  Output follows run_gpt.cc:124-149: one line per request with
the prompt in parentheses and the generated tokens, then the stage times."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import List, Optional


class SimpleVocabDecoder:
    """id -> token text from a vocab.json (token -> id), a leading 'Ġ' shown as a space
    (src/examples/lib/simple_vocab_decoder.h:14-40)."""

    def __init__(self, path: str):
        with open(path, "r", encoding="utf-8") as f:
            self.map = {int(v): k for k, v in json.load(f).items()}

    def decode(self, token: int) -> str:
        s = self.map.get(int(token))
        if s is None:
            return "<UNK>"
        return " " + s[1:] if s.startswith("Ġ") else s


def read_prompts(path: str) -> List[List[int]]:
    prompts = []
    with open(path, "r", encoding="utf-8") as f:
        for line in f:
            line = line.strip()
            if line:
                prompts.append([int(t) for t in line.split()])
    return prompts


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(
        prog="run_opt",
        description="This program loads a model, feeds it with given input sequences, "
                    "and prints the generated tokens.")
    ap.add_argument("model_path", help="Path to the model folder (config.json + safetensors)")
    ap.add_argument("model_name", help="Name of the model (e.g. opt_1.3b, or auto)")
    ap.add_argument("-v", "--vocab_json_path", default="", help="Path to the vocab json file")
    ap.add_argument("precision", help="Precision used for inference (bf16 or fp32)")
    ap.add_argument("input_path", help="Path to the input file")
    ap.add_argument("-d", "--debug", action="store_true", help="Enable debug mode (print every step)")
    ap.add_argument("--max-new-tokens", type=int, default=128, help="decoding steps per request")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    ap.add_argument("--seed", type=int, default=0, help="seed of the sampler (request i uses seed+i)")
    ap.add_argument("--end-token", type=int, default=None, help="default: config.json's eos_token_id")
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache block")
    ap.add_argument("--num-blocks", type=int, default=1024, help="cache blocks in the pool")
    ap.add_argument("--gpu-mem-fraction", type=float, default=0.0,
                    help="size the cache pool as this fraction of the free GPU memory instead of --num-blocks")
    ap.add_argument("--max-seqs", type=int, default=64, help="requests running at a time")
    ap.add_argument("--max-batched-tokens", type=int, default=2048, help="token budget of a step")
    ap.add_argument("--prefill-chunk", type=int, default=512, help="largest prompt portion in a step")
    ap.add_argument("--random-weights", action="store_true",
                    help="write seeded random weights into model_path if it holds only config.json")
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from ..config.registry import hyper_param_from_dir
    from ..engine.engine import Engine, parse_dtype
    from ..sampling import SamplingParams
    try:
        dtype = parse_dtype(args.precision)
    except ValueError as e:
        print(f"Invalid precision: {args.precision}\nValid precision: bf16, fp32 ({e})")
        return 1
    arch, hp = hyper_param_from_dir(args.model_path)
    if args.model_name != "auto":
        family = args.model_name.split("_")[0].lower()
        if arch.short_name and family != arch.short_name:
            print(f"Invalid model name: {args.model_name} (config.json describes {arch.name}; "
                  f"expected {arch.short_name}_<size> or auto)")
            return 1
    if args.random_weights and not any(
            os.path.exists(os.path.join(args.model_path, f))
            for f in ("model.safetensors", "model.safetensors.index.json")):
        from ..weights.random_init import write_random_model
        print("Writing random weights...")
        write_random_model(hp, args.model_path, seed=args.seed)
    print("Reading input tokens...")
    prompts = read_prompts(args.input_path)
    print("Loading model...")
    if args.debug:
        print(hp)
    eng = Engine(args.model_path, dtype=dtype, page_size=args.block_size, num_pages=args.num_blocks,
                 max_seqs=args.max_seqs, max_batched_tokens=args.max_batched_tokens,
                 prefill_chunk=args.prefill_chunk, gpu_mem_fraction=args.gpu_mem_fraction)
    ids = []
    for i, p in enumerate(prompts):
        ids.append(eng.add_request(p, SamplingParams(
            temperature=args.temperature, max_new_tokens=args.max_new_tokens, seed=args.seed + i,
            eos_token_id=args.end_token, ignore_eos=args.ignore_eos)))
    t0 = time.perf_counter()
    done = {}
    while eng.has_work():
        outs = eng.step()
        if args.debug:
            print(f"step {eng.stats.steps}: finished {[o.req_id for o in outs]}")
        for o in outs:
            done[o.req_id] = o.output
    total = time.perf_counter() - t0
    dec = SimpleVocabDecoder(args.vocab_json_path) if args.vocab_json_path else None
    for i, (rid, p) in enumerate(zip(ids, prompts)):
        out = done[rid]
        if dec:
            text = "(" + "".join(dec.decode(t) for t in p) + ")" + "".join(dec.decode(t) for t in out)
        else:
            text = "(" + "".join(f"{t} " for t in p) + ")" + "".join(f"{t} " for t in out)
        print(f"[{i:2d}] {text}  ({len(out)} tokens generated)")
    st = eng.stats
    print("Time usage:")
    print(f"\tContext stage: {st.prefill_time * 1e3:.2f} ms")
    print(f"\tRegression stage: {st.decode_time * 1e3:.2f} ms")
    print(f"\tTotal: {total * 1e3:.2f} ms")
    if st.prefill_time > 0 and st.decode_time > 0:
        print(f"\tPrompt tokens/s: {st.prompt_tokens / st.prefill_time:.1f}; "
              f"generated tokens/s: {st.generated_tokens / (st.prefill_time + st.decode_time):.1f}; "
              f"pre-emptions: {st.preemptions}")
    print("Done!")
    return 0


if __name__ == "__main__":
    sys.exit(main())
