"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and decides nothing: every step of the trace is one call of
the same ``ModelRunner.step`` that generation uses, on the same cache manager and
kernels.  The reference has no such program (its forward never exposes logits,
src/csrc/model/gpt/gpt.cc:598-636).

Beside the ``<step>.f32`` files it writes ``index.json``: for every step that wrote logits, the
(request, position) of each row, in the file's row order, so that a reader needs no copy of the
trace to know what a row is."""
from __future__ import annotations

import json
import os
import sys
from typing import IO, Dict

import numpy as np
import torch

from ..config.cache_param import CacheParam
from ..models import load_model
from .step import ModelRunner, StepEntry

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32}


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines: IO[str],
           log: IO[str] = sys.stdout, page_size: int = 16, max_live: int = 8,
           device: str = "cuda:0") -> int:
    if dtype not in _DTYPES:
        raise ValueError(f"--dtype must be bfloat16 or float32, got {dtype!r}")
    os.makedirs(out_dir, exist_ok=True)
    model = load_model(model_dir, _DTYPES[dtype], device)
    # the pool holds max_tokens tokens; a request's share is counted in whole pages
    num_pages = max(1, -(-max_tokens // page_size))
    runner = ModelRunner(model, CacheParam(page_size=page_size, num_pages=num_pages,
                                           max_seqs=max_live), device,
                         max_batched_tokens=min(max(max_tokens, 1), 4096))
    index: Dict[str, list] = {}
    try:
        _replay_steps(runner, lines, out_dir, log, index)
    finally:
        with open(os.path.join(out_dir, "index.json"), "w", encoding="utf-8") as f:
            json.dump({"model": os.path.abspath(model_dir), "dtype": dtype, "vocab_size": model.vocab_size,
                       "page_size": page_size, "rows": index}, f)
    return 0


def _replay_steps(runner: ModelRunner, lines: IO[str], out_dir: str, log: IO[str], index: Dict[str, list]) -> None:
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for ent in rec.get("entries", []):
            rid = ent["id"]
            if not runner.is_live(rid):
                runner.admit(rid)
            entries.append(StepEntry(rid, [int(t) for t in ent["tokens"]],
                                     [int(w) for w in ent.get("want", [])]))
        if entries:
            # the position of a wanted row: what the request holds before this step, plus its place
            rows = [[e.req_id, runner.cached_length(e.req_id) + w] for e in entries for w in e.want]
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                index[str(step)] = rows
                arr = logits.detach().to("cpu", torch.float32).contiguous().numpy()
                arr.astype("<f4", copy=False).tofile(os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            if runner.is_live(rid):
                runner.finish(rid)
        log.write(f"done {step}\n")
        log.flush()
