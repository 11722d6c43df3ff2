"""Token embedding with an optional input projection, and the output head.

x0[t] = Etok[id[t]] (+ position rows), reference src/csrc/kernel/embedding.cu:25-35.
When the embedding width differs from the hidden width, the token vector is
projected first (no bias) and the position rows are added to the projected
vector; the reference has no such model (README.md:42 tells users to avoid it).
The head computes logits = y * Wlm^T in float (src/csrc/model/gpt/gpt.cc:192-201),
after an optional output projection, and falls back to the embedding table when
the file has no separate head tensor (tied weights, scripts/lib/converter_lib.py:272)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part


class TokenEmbedding(Part):
    """params: vocab_size, embed_dim (width of the table; projected to hidden if different)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.vocab_size = int(self.param("vocab_size"))
        self.embed_dim = int(self.param("embed_dim", hidden_size))
        self.projected = self.embed_dim != hidden_size
        self.table = None
        self.w_in = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.name("weight"), (self.vocab_size, self.embed_dim), "table")]
        if self.projected:
            specs.append(TensorSpec(self.name("project_in"), (self.hidden_size, self.embed_dim), "matrix"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name("weight")]
        if self.projected:
            self.w_in = tensors[self.name("project_in")]

    def forward(self, ctx, position) -> torch.Tensor:
        T = ctx.num_tokens
        dev = self.table.device
        addend = position.embedding_addend(ctx) if position is not None else None
        x32 = K.empty((T, self.hidden_size), torch.float32, dev)
        if not self.projected:
            if addend is None:
                K.lookup(ctx.token_ids, self.table, out_f32=x32)
            else:
                ptab, pidx, poff = addend
                K.lookup(ctx.token_ids, self.table, add_ids=pidx, add_offset=poff, add_table=ptab,
                         out_f32=x32)
            return x32
        tok = K.empty((T, self.embed_dim), self.dtype, dev)
        K.lookup(ctx.token_ids, self.table, out_t=tok)
        K.gemm(tok, self.w_in, out=x32, out_f32=True)
        if addend is not None:
            ptab, pidx, poff = addend
            K.lookup(None, None, add_ids=pidx, add_offset=poff, add_table=ptab, out_f32=x32,
                     accumulate=True)
        return x32


class LMHead(Part):
    """params: vocab_size, embed_dim (input width of the head matrix), tied_to (file name of
    the tensor used when the head's own tensor is absent, or None)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.vocab_size = int(self.param("vocab_size"))
        self.embed_dim = int(self.param("embed_dim", hidden_size))
        self.projected = self.embed_dim != hidden_size
        self.tied_to: Optional[str] = spec.params.get("tied_to")
        self.weight = None
        self.w_out = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.name("weight"), (self.vocab_size, self.embed_dim), "matrix",
                            optional=self.tied_to is not None)]
        if self.projected:
            specs.append(TensorSpec(self.name("project_out"), (self.embed_dim, self.hidden_size), "matrix"))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        own = tensors.get(self.name("weight"))
        if own is None:
            if self.tied_to is None or self.tied_to not in tensors:
                raise KeyError("the head has neither its own tensor nor a table to be tied to")
            own = tensors[self.tied_to]
        self.weight = own
        if self.projected:
            self.w_out = tensors[self.name("project_out")]

    def takes_norm(self, rows: int, norm) -> bool:
        """Whether ``forward`` can take ``norm`` (a norm part) of picked rows as its input instead of
        normalised rows, and report the rows' best outputs: the product with the head matrix then
        runs in the kernel that walks a very wide matrix with few rows."""
        return (not self.projected and hasattr(norm, "as_input") and getattr(norm, "width", None) == self.embed_dim
                and K.wide_offered(rows, self.vocab_size, self.embed_dim, self.dtype))

    def forward(self, y_t, best: Optional[torch.Tensor] = None) -> torch.Tensor:
        """float32 logits [rows, vocab] of ``y_t``: normalised rows, or (where ``takes_norm``) what a
        norm's ``as_input`` returned.  ``best`` (int32 [rows], where ``takes_norm``): receives every
        row's best output, the lowest index on ties."""
        if self.projected:
            y_t = K.gemm(y_t, self.w_out)
        return K.gemm(y_t, self.weight, out_f32=True, best=best)
