"""Loading weights by tensor name, with one error that names everything wrong.

The reference loads each tensor by name and checks its element count and dtype,
one failure at a time (src/csrc/model/gpt/gpt_weight.cc:235-252, :258-326).
Here the model's parts declare the tensors they need (``TensorSpec``); the
loader compares the whole declaration with the file first and raises a single
``WeightError`` listing missing tensors, unexpected tensors and wrong shapes.

Storage types on the device:
  * ``matrix`` and ``table`` tensors (GEMM operands, embedding tables) take the
    engine's dtype (bfloat16 or float32);
  * ``vector`` tensors (biases, norm gains) are held in float32 in either mode:
    a vector stored in 32-bit stays so, and a bfloat16 one is represented
    exactly;
  * ``int`` tensors become int32.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import ModelFiles


@dataclass(frozen=True)
class TensorSpec:
    name: str                       # name in the file
    shape: Tuple[int, ...]
    kind: str = "matrix"            # matrix | table | vector | int
    optional: bool = False          # may be absent (e.g. a tied head)
    alt_names: Tuple[str, ...] = () # other spellings accepted in the file
    init: str = "normal"            # random-weights mode: "normal" N(0, std) | "gain" 1 + N(0, 0.1)


class WeightError(ValueError):
    def __init__(self, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]],
                 wrong_dtype: Sequence[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["the weight file does not match the model that config.json describes:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}):")
            lines += [f"    {n}" for n in self.missing]
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}):")
            lines += [f"    {n}" for n in self.unexpected]
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += [f"    {n}: expected {list(e)}, file has {list(g)}"
                      for n, e, g in self.wrong_shape]
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}):")
            lines += [f"    {n}: {why}" for n, why in self.wrong_dtype]
        super().__init__("\n".join(lines))


def storage_dtype(kind: str, engine_dtype: torch.dtype) -> torch.dtype:
    if kind == "int":
        return torch.int32
    if kind == "vector":
        return torch.float32
    return engine_dtype


def _strip_candidates(name: str) -> List[str]:
    """Spellings of one tensor name: with and without a leading ``model.``."""
    out = [name]
    if name.startswith("model."):
        out.append(name[len("model."):])
    else:
        out.append("model." + name)
    return out


def match_specs(specs: Iterable[TensorSpec], available: Dict[str, Tuple[int, ...]],
                dtypes: Optional[Dict[str, torch.dtype]] = None) -> Dict[str, str]:
    """Check ``specs`` against the names/shapes a file offers.

    Returns {spec name -> name in the file} for the tensors found; raises
    ``WeightError`` if anything required is missing, anything in the file is
    not asked for, or a shape differs."""
    found: Dict[str, str] = {}
    missing, wrong_shape, wrong_dtype = [], [], []
    used = set()
    for spec in specs:
        hit = None
        for cand in [c for n in (spec.name,) + tuple(spec.alt_names) for c in _strip_candidates(n)]:
            if cand in available:
                hit = cand
                break
        if hit is None:
            if not spec.optional:
                missing.append(spec.name)
            continue
        used.add(hit)
        if tuple(available[hit]) != tuple(spec.shape):
            wrong_shape.append((spec.name, tuple(spec.shape), tuple(available[hit])))
            continue
        if dtypes is not None:
            dt = dtypes[hit]
            if spec.kind == "int":
                if dt.is_floating_point:
                    wrong_dtype.append((spec.name, f"an integer table is stored as {dt}"))
                    continue
            elif not dt.is_floating_point:
                wrong_dtype.append((spec.name, f"a floating-point tensor is stored as {dt}"))
                continue
        found[spec.name] = hit
    unexpected = sorted(k for k in available if k not in used)
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(sorted(missing), unexpected, wrong_shape, wrong_dtype)
    return found


def load_tensors(model_dir: str, specs: Sequence[TensorSpec], engine_dtype: torch.dtype,
                 device: torch.device | str) -> Dict[str, torch.Tensor]:
    """Read every tensor ``specs`` names from ``model_dir`` onto ``device``."""
    files = ModelFiles(model_dir)
    available = {k: files.shape(k) for k in files.keys()}
    dtypes = {k: files.dtype(k) for k in files.keys()}
    found = match_specs(specs, available, dtypes)
    by_name = {s.name: s for s in specs}
    out: Dict[str, torch.Tensor] = {}
    for name, in_file in found.items():
        spec = by_name[name]
        t = files.tensor(in_file)
        out[name] = t.to(device=device, dtype=storage_dtype(spec.kind, engine_dtype)).contiguous()
    return out
