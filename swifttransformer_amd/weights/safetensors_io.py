"""A minimal safetensors reader and writer.

File layout: 8 bytes little-endian header length ``n``; ``n`` bytes of JSON
mapping each tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}``
(offsets relative to the first byte after the header, plus an optional
``"__metadata__"`` entry); then the raw little-endian tensor bytes.

The reference reads one TorchScript file per tensor
(src/csrc/model/gpt/gpt_weight.cc:235-252); a model folder with config.json and
safetensors takes that place here.  Files are memory-mapped, so a tensor's bytes
are touched only when it is copied to the device.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One memory-mapped .safetensors file."""

    def __init__(self, path: str):
        self.path = path
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except Exception as e:  # noqa: BLE001
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + n
        self._entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, ent in header.items():
            dt = ent["dtype"]
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt}")
            b, e = ent["data_offsets"]
            shape = tuple(int(s) for s in ent["shape"])
            numel = 1
            for s in shape:
                numel *= s
            want = numel * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if b < 0 or e < b:
                raise SafetensorsError(f"{path}: tensor {name!r} has data offsets [{b}, {e})")
            if e - b != want or self._data_start + e > size:
                raise SafetensorsError(
                    f"{path}: tensor {name!r} claims {e - b} bytes, its shape needs {want}")
            self._entries[name] = (_DTYPES[dt], shape, b, e)
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def keys(self) -> List[str]:
        return list(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return self._entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (read-only: copy before writing)."""
        dtype, shape, b, e = self._entries[name]
        if e == b:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # read-only buffer warning
            flat = torch.frombuffer(self._mm, dtype=dtype, count=(e - b) // _elem(dtype),
                                    offset=self._data_start + b)
        return flat.view(shape)

    def close(self) -> None:
        # tensors handed out view the map; it is released when they are gone
        self._f.close()


def _elem(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class ModelFiles:
    """All tensors of a model folder: ``model.safetensors`` or the shards that
    ``model.safetensors.index.json`` names."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        self._files: List[SafetensorsFile] = []
        self._where: Dict[str, SafetensorsFile] = {}
        if os.path.isfile(single):
            paths = [single]
        elif os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                wm = json.load(f)["weight_map"]
            paths = [os.path.join(model_dir, p) for p in sorted(set(wm.values()))]
        else:
            raise FileNotFoundError(
                f"{model_dir!r} holds neither model.safetensors nor model.safetensors.index.json")
        for p in paths:
            sf = SafetensorsFile(p)
            self._files.append(sf)
            for k in sf.keys():
                self._where[k] = sf

    def keys(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._where[name].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self._where[name].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)


def save_safetensors(path: str, tensors: Dict[str, torch.Tensor],
                     metadata: Dict[str, str] | None = None) -> None:
    """Write ``tensors`` (CPU, any of the supported dtypes) to ``path``."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order: Iterable[str] = sorted(tensors)
    blobs = []
    for name in order:
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for raw in blobs:
            f.write(raw)
    os.replace(tmp, path)
