"""Choosing tokens from logits on the device."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops import kernels as K
from .params import SamplingParams


class _Pinned:
    """A pinned host buffer with the event of the last copy that used it."""

    def __init__(self, shape):
        self.host = torch.zeros(shape, dtype=torch.int32).pin_memory()
        self.event = torch.cuda.Event()
        self.busy = False          # a copy is under way or its result has not been read

    def wait(self) -> None:
        if self.busy:
            self.event.synchronize()   # waits for that copy only, not for work queued after it
            self.busy = False


class _Ring:
    """A few pinned buffers used in turn; a buffer still in use when its turn comes again is
    waited for (by then its copy has long been done)."""

    def __init__(self, width: Optional[int], slots: int = 4):
        self.width, self.slots = width, slots
        self.buffers: List[Optional[_Pinned]] = [None] * slots
        self.turn = 0

    def take(self, rows: int) -> _Pinned:
        i = self.turn
        self.turn = (i + 1) % self.slots
        buf = self.buffers[i]
        if buf is None or buf.host.shape[0] < rows:
            n = max(64, rows)
            buf = self.buffers[i] = _Pinned((n,) if self.width is None else (n, self.width))
        buf.wait()
        return buf


class PendingTokens:
    """Token ids chosen on the device and on their way to the host.  ``device`` [R] int32 can
    feed the next step at once; ``result()`` waits for the copy and returns the ids."""

    def __init__(self, device_ids: torch.Tensor, pinned: Optional[_Pinned] = None):
        self.device = device_ids
        self._pinned = pinned
        self._ids: Optional[List[int]] = None
        if pinned is not None:
            pinned.host[:device_ids.shape[0]].copy_(device_ids, non_blocking=True)
            pinned.event.record()
            pinned.busy = True

    def result(self) -> List[int]:
        if self._ids is None:
            if self._pinned is None:
                self._ids = self.device.cpu().tolist()
            else:
                self._pinned.wait()
                self._ids = self._pinned.host[:self.device.shape[0]].tolist()
                self._pinned = None
        return self._ids


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)
        cuda = self.device.type == "cuda"
        self._ids_ring = _Ring(None) if cuda else None      # sampled ids on their way back
        self._meta_ring = _Ring(4) if cuda else None        # seeds, counters, temperatures on their way in

    def sample_pending(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                       draws: Sequence[int], best: Optional[torch.Tensor] = None) -> PendingTokens:
        """One token per row of ``logits``, left on the device with a copy to the host under
        way; ``draws[i]`` is the index of the output token being drawn for row i (the
        sampler's counter).  ``best`` (int32 [rows] on the device): the rows' arg-max where the step
        has found it already (``ModelRunner.last_best``); greedy rows then need no kernel here.
        Nothing here waits for work queued on the device."""
        R = logits.shape[0]
        if len(params) != R or len(draws) != R:
            raise ValueError("one SamplingParams and one draw index per row")
        if R == 0:
            return PendingTokens(torch.empty((0,), dtype=torch.int32))
        if all(p.temperature <= 0 for p in params):
            ids = best if best is not None and best.shape == (R,) else K.sample(logits)
        else:
            host = np.zeros((R, 4), dtype=np.int32)
            for i, (p, d) in enumerate(zip(params, draws)):
                host[i, 0] = np.uint32(p.seed & 0xffffffff).astype(np.int32)
                host[i, 1] = np.uint32((p.seed >> 32) & 0xffffffff).astype(np.int32)
                host[i, 2] = np.uint32(d & 0xffffffff).astype(np.int32)
                host[i, 3] = np.float32(p.temperature).view(np.int32)
            if self._meta_ring is not None:
                buf = self._meta_ring.take(R)
                buf.host[:R] = torch.from_numpy(host)
                meta = buf.host[:R].to(self.device, non_blocking=True)
                buf.event.record()
                buf.busy = True
            else:
                meta = torch.from_numpy(host).to(self.device)
            ids = K.sample(logits, temperature=meta[:, 3].contiguous().view(torch.float32),
                           seeds=meta[:, 0:2].contiguous(), draws=meta[:, 2].contiguous())
        return PendingTokens(ids, self._ids_ring.take(R) if self._ids_ring is not None else None)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               draws: Sequence[int]) -> List[int]:
        """As ``sample_pending``, waiting for the ids."""
        return self.sample_pending(logits, params, draws).result()
