"""Scratch memory of a step: one device buffer, sized once, from which the tensors a step
makes (activations, partial results, logits of recorded steps) are carved by a bump pointer.

The reference keeps grow-only buffers owned by the model and sized from the number of tokens
of the batch (src/csrc/model/gpt/gpt.h:25-54, grown in src/csrc/model/gpt/gpt.cc:253-264).
Here the buffer has two banks that take turns from layer to layer: what a layer makes lives in
its bank, is read by the next layer (which makes its own in the other bank) and is dead when
the layer after that starts over in the first bank.  A step therefore needs the memory of its
two hungriest layers, not of all of them, every tensor has the same address in every step of
the same shape (which is what lets such steps be recorded and replayed), and nothing is asked
of an allocator between steps.

The rule this puts on parts: a tensor made during a layer may be read until the end of the
next layer and no longer; what has to outlive that belongs in the cache manager's per-request
state.  A part that allocates with ``torch.empty`` itself is untouched by all this.

``measure`` mode runs a step through the ordinary allocator and records how much each bank
would have needed; ``ModelRunner`` uses it once, on a step of ``max_batched_tokens`` padding
rows, to size the buffer.  A request that does not fit the bank (a step larger than the
runner was built for) is served by the ordinary allocator and counted in ``overflows``."""
from __future__ import annotations

from contextlib import contextmanager
from typing import Dict, Optional, Sequence

import torch

_ALIGN = 256
_ITEMSIZE = {torch.float32: 4, torch.bfloat16: 2, torch.int32: 4, torch.float16: 2, torch.int64: 8,
             torch.uint8: 1, torch.int8: 1, torch.float64: 8, torch.int16: 2, torch.bool: 1}


class StepArena:
    def __init__(self, device):
        self.device = torch.device(device)
        self.bank_bytes = 0
        self.buffer: Optional[torch.Tensor] = None           # uint8 [2 * bank_bytes]
        self._typed: Dict[torch.dtype, torch.Tensor] = {}     # flat views of the buffer by dtype
        self.bank = 0
        self.used = [0, 0]
        self.measure = False
        self.peak = 0               # largest bank use seen (in measure mode: what a bank would have needed)
        self.overflows = 0          # requests served by the ordinary allocator because the bank was full
        self.carved = 0             # requests served from the buffer

    def resize(self, bank_bytes: int) -> None:
        """(Re)allocate the buffer: two banks of ``bank_bytes``.  Only before any step has been
        recorded against it: recorded steps keep the addresses they were recorded with."""
        bank_bytes = -(-int(bank_bytes) // _ALIGN) * _ALIGN
        self.bank_bytes = bank_bytes
        self._typed = {}
        self.buffer = torch.empty(2 * bank_bytes, dtype=torch.uint8, device=self.device) if bank_bytes else None
        self.begin_step()

    def nbytes(self) -> int:
        return 2 * self.bank_bytes

    def begin_step(self) -> None:
        self.bank = 1               # the embedding's output; the first layer then starts bank 0
        self.used = [0, 0]

    def state(self):
        """Where the bump pointers stand (to go on from there later, see ``using``)."""
        return (self.bank, tuple(self.used))

    def next_bank(self) -> None:
        """A new layer starts: its tensors go to the other bank, from the bank's beginning."""
        self.bank ^= 1
        self.used[self.bank] = 0

    def empty(self, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for d in shape:
            n *= int(d)
        size = _ITEMSIZE[dtype]
        nbytes = -(-(n * size) // _ALIGN) * _ALIGN
        off = self.used[self.bank]
        if self.measure or off + nbytes > self.bank_bytes:
            if self.measure:
                self.used[self.bank] = off + nbytes
                self.peak = max(self.peak, off + nbytes)
            else:
                self.overflows += 1
            return torch.empty(tuple(shape), dtype=dtype, device=self.device)
        self.used[self.bank] = off + nbytes
        if off + nbytes > self.peak:
            self.peak = off + nbytes
        self.carved += 1
        flat = self._typed.get(dtype)
        if flat is None:
            flat = self._typed[dtype] = self.buffer.view(dtype)
        start = (self.bank * self.bank_bytes + off) // size
        return flat[start:start + n].view(tuple(shape))


_current: Optional[StepArena] = None


def current() -> Optional[StepArena]:
    return _current


def empty(shape: Sequence[int], dtype: torch.dtype, device) -> torch.Tensor:
    """An uninitialised tensor for a step's intermediate result: from the step's arena while one
    is in use (``using``), from the ordinary allocator otherwise."""
    a = _current
    if a is None:
        return torch.empty(tuple(shape), dtype=dtype, device=device)
    return a.empty(shape, dtype)


def next_bank() -> None:
    if _current is not None:
        _current.next_bank()


@contextmanager
def using(arena: Optional[StepArena], state=None):
    """Inside: ``empty`` carves from ``arena`` (None: the ordinary allocator), from the start of a
    step, or going on from ``state`` (what ``arena.state()`` returned at the end of a part of the
    step that ran earlier, e.g. as a replayed recording)."""
    global _current
    before, _current = _current, arena
    if arena is not None:
        if state is None:
            arena.begin_step()
        else:
            arena.bank, arena.used = state[0], list(state[1])
    try:
        yield arena
    finally:
        _current = before


@contextmanager
def outside():
    """Inside: ``empty`` uses the ordinary allocator even while an arena is in use (for what must
    outlive the step, like the logits a caller may keep)."""
    global _current
    before, _current = _current, None
    try:
        yield
    finally:
        _current = before
