"""Choosing tokens from logits on the device."""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..ops import kernels as K
from .params import SamplingParams


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               draws: Sequence[int]) -> List[int]:
        """One token per row of ``logits``; ``draws[i]`` is the index of the output token being
        drawn for row i (the sampler's counter)."""
        R = logits.shape[0]
        if R == 0:
            return []
        if len(params) != R or len(draws) != R:
            raise ValueError("one SamplingParams and one draw index per row")
        if all(p.temperature <= 0 for p in params):
            ids = K.sample(logits)
        else:
            host = np.zeros((R, 4), dtype=np.int32)
            temps = np.zeros(R, dtype=np.float32)
            for i, (p, d) in enumerate(zip(params, draws)):
                temps[i] = p.temperature
                host[i, 0] = np.uint32(p.seed & 0xffffffff).astype(np.int32)
                host[i, 1] = np.uint32((p.seed >> 32) & 0xffffffff).astype(np.int32)
                host[i, 2] = np.uint32(d & 0xffffffff).astype(np.int32)
            meta = torch.from_numpy(host).to(self.device)
            ids = K.sample(logits, temperature=torch.from_numpy(temps).to(self.device),
                           seeds=meta[:, 0:2].contiguous(), draws=meta[:, 2].contiguous())
        return ids.cpu().tolist()
