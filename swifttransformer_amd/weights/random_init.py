"""Random weights: tensors drawn by name from a seed, and a model folder written
from a configuration.

The reference fills every tensor with U(-1e-3, 1e-3) from ``torch::manual_seed(0)``
(src/csrc/model/gpt/gpt_weight.cc:329-408).  Here matrices, tables and biases are
N(0, 0.02), norm gains 1 + N(0, 0.1).

Element i of the tensor called ``name`` is a function of (seed, name, i) alone: a
64-bit counter hash gives 32 uniform bits, and the inverse normal distribution is
taken from a table of 65,537 quantiles with linear interpolation between neighbours.
Only integer operations, a gather, one float multiply and one float add are involved,
so the device and the CPU produce the same bits: a model built in memory on the GPU
(``random_tensors``) and the folder ``write_random_model`` writes hold equal values
for a seed, whatever the order of generation."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable, Optional

import torch

from .loader import TensorSpec, storage_dtype
from .safetensors_io import save_safetensors

WEIGHT_STD = 0.02
GAIN_STD = 0.1

_DTYPE_NAMES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
_TABLE_SIZE = 1 << 16
# elements generated at a time: on the CPU the temporaries should stay in the caches (fresh 128 MB
# tensors cost more in page faults than the arithmetic), on the GPU a chunk should be worth its launches
_CHUNK = {"cpu": 1 << 16, "cuda": 1 << 24}
_MASK64 = (1 << 64) - 1


def _i64(v: int) -> int:
    """A 64-bit pattern as the signed value an int64 tensor holds."""
    v &= _MASK64
    return v - (1 << 64) if v >= (1 << 63) else v


_GOLDEN, _MIX1, _MIX2 = _i64(0x9E3779B97F4A7C15), _i64(0xBF58476D1CE4E5B9), _i64(0x94D049BB133111EB)

_tables: Dict[str, tuple] = {}


def _quantile_table(device) -> tuple:
    """(q, dq): q[k] = inverse normal distribution at (k + 0.5) / 65537 for k = 0..65535 and
    dq[k] = q[k + 1] - q[k], float32.  Always computed on the CPU in float64 and then moved, so
    every device sees the same float32 numbers."""
    key = str(torch.device(device))
    if key not in _tables:
        p = (torch.arange(_TABLE_SIZE + 1, dtype=torch.float64) + 0.5) / (_TABLE_SIZE + 1)
        q = torch.special.ndtri(p).to(torch.float32)
        _tables[key] = (q[:-1].contiguous().to(device), (q[1:] - q[:-1]).contiguous().to(device))
    return _tables[key]


def _key_for(name: str, seed: int) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return _i64(int.from_bytes(h[:8], "little"))


def _standard_normal(n: int, key: int, device) -> torch.Tensor:
    """float32 [n]: element i from the hash of (key, i)."""
    q, dq = _quantile_table(device)
    out = torch.empty(n, dtype=torch.float32, device=device)
    chunk = _CHUNK.get(torch.device(device).type, 1 << 20)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        z = torch.arange(lo, hi, dtype=torch.int64, device=device)
        z = z * _GOLDEN + key                                   # int64 arithmetic wraps
        z = (z ^ ((z >> 30) & ((1 << 34) - 1))) * _MIX1          # logical shifts: mask the sign's copies
        z = (z ^ ((z >> 27) & ((1 << 37) - 1))) * _MIX2
        z = z ^ ((z >> 31) & ((1 << 33) - 1))
        k = (z >> 48) & 0xFFFF
        frac = ((z >> 32) & 0xFFFF).to(torch.float32) * (1.0 / 65536.0)   # exact
        step = dq[k] * frac                                     # one rounding
        out[lo:hi] = q[k] + step                                # one rounding
    return out


def random_tensor(spec: TensorSpec, seed: int, device="cpu") -> torch.Tensor:
    """float32 values of one tensor."""
    n = 1
    for d in spec.shape:
        n *= int(d)
    t = _standard_normal(n, _key_for(spec.name, seed), device).view(spec.shape)
    if spec.init == "gain":
        return t * GAIN_STD + 1.0
    return t * WEIGHT_STD


def file_dtype_of(hyper_param, file_dtype: Optional[torch.dtype] = None) -> torch.dtype:
    """The type a model folder of ``hyper_param`` stores its tensors in."""
    if file_dtype is not None:
        return file_dtype
    return _DTYPE_NAMES.get(getattr(hyper_param, "torch_dtype", "bfloat16"), torch.bfloat16)


def random_tensors(specs: Iterable[TensorSpec], seed: int, engine_dtype: torch.dtype,
                   device, skip_optional: bool = True,
                   file_dtype: Optional[torch.dtype] = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Tensors for ``DecoderModel.bind`` generated on ``device`` (no file): the values a folder
    written with ``file_dtype`` would hold, in the storage types the loader gives them.
    ``file_dtype`` None: the float32 draws themselves."""
    out = {}
    for s in specs:
        if s.optional and skip_optional:
            continue
        t = random_tensor(s, seed, device)
        if file_dtype is not None:
            t = t.to(file_dtype)
        out[s.name] = t.to(storage_dtype(s.kind, engine_dtype))
    return out


def write_random_model(hyper_param, folder: str, seed: int = 0,
                       file_dtype: Optional[torch.dtype] = None, architecture=None) -> str:
    """Write config.json and model.safetensors for ``hyper_param`` into ``folder``."""
    from ..config.registry import resolve_architecture
    from ..models.decoder import DecoderModel
    arch = architecture or resolve_architecture(hyper_param.architecture)
    file_dtype = file_dtype_of(hyper_param, file_dtype)
    model = DecoderModel(arch.build_spec(hyper_param), torch.float32)
    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for s in model.tensor_specs():
        if s.optional:
            continue   # e.g. a tied head: the file holds the table only
        tensors[s.name] = random_tensor(s, seed).to(file_dtype)
    save_safetensors(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt"})
    cfg = hyper_param.to_config_dict()
    cfg["torch_dtype"] = {v: k for k, v in _DTYPE_NAMES.items()}[file_dtype]
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    return folder
