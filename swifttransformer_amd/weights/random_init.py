"""Random weights: tensors drawn by name from a seed, and a model folder written
from a configuration.

The reference fills every tensor with U(-1e-3, 1e-3) from ``torch::manual_seed(0)``
(src/csrc/model/gpt/gpt_weight.cc:329-408).  Here matrices, tables and biases are
N(0, 0.02), norm gains 1 + N(0, 0.1); each tensor has its own generator seeded from
(seed, name), so the values do not depend on the order of generation."""
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


def _seed_for(name: str, seed: int) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7fffffffffffffff


def random_tensor(spec: TensorSpec, seed: int, device="cpu") -> torch.Tensor:
    """float32 values of one tensor."""
    g = torch.Generator(device=device)
    g.manual_seed(_seed_for(spec.name, seed))
    t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
    if spec.init == "gain":
        return 1.0 + GAIN_STD * t
    return WEIGHT_STD * t


def random_tensors(specs: Iterable[TensorSpec], seed: int, engine_dtype: torch.dtype,
                   device, skip_optional: bool = True) -> Dict[str, torch.Tensor]:
    """Tensors for ``DecoderModel.bind`` generated on ``device`` (no file)."""
    out = {}
    for s in specs:
        if s.optional and skip_optional:
            continue
        t = random_tensor(s, seed, device)
        out[s.name] = t.to(storage_dtype(s.kind, engine_dtype))
    return out


def write_random_model(hyper_param, folder: str, seed: int = 0,
                       file_dtype: Optional[torch.dtype] = None, architecture=None) -> str:
    """Write config.json and model.safetensors for ``hyper_param`` into ``folder``."""
    from ..config.registry import resolve_architecture
    from ..models.decoder import DecoderModel
    arch = architecture or resolve_architecture(hyper_param.architecture)
    names = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
    if file_dtype is None:
        file_dtype = names.get(getattr(hyper_param, "torch_dtype", "bfloat16"), torch.bfloat16)
    model = DecoderModel(arch.build_spec(hyper_param), torch.float32)
    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for s in model.tensor_specs():
        if s.optional:
            continue   # e.g. a tied head: the file holds the table only
        tensors[s.name] = random_tensor(s, seed).to(file_dtype)
    save_safetensors(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt"})
    cfg = hyper_param.to_config_dict()
    cfg["torch_dtype"] = {v: k for k, v in names.items()}[file_dtype]
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    return folder
