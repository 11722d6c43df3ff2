"""How a layer's norms, mixer and feed-forward are wired around the residual stream.

pre-norm (reference src/csrc/model/gpt/gpt.cc:325-335, :347-391, :423-436, :467-501):
    a = N1(x); r = x + Mix(a); d = N2(r); x' = r + FFN(d)
post-norm (the reference refuses it, gpt.cc:238-240):
    r = N1(x + Mix(x)); x' = N2(r + FFN(r))
The residual stream is float; parts that multiply matrices take the storage type."""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import Part


def _fuses(part, norm, rows: int) -> bool:
    """A part that accepts a norm and a norm that can be a product's prologue at this size."""
    return (getattr(part, "accepts_norm", False) and hasattr(norm, "fusable")
            and norm.fusable(rows, part.hidden_size))


class PreNorm(Part):
    needs = ("mixer_norm", "ffn_norm", "feed_forward")    # layer slots that must be filled

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True) -> torch.Tensor:
        rows = x32.shape[0]
        if _fuses(layer.mixer, layer.mixer_norm, rows):
            r32 = layer.mixer.forward(None, x32, ctx, cache, write, norm=layer.mixer_norm)
        else:
            a, _ = layer.mixer_norm.forward(x32, out_t=True)
            r32 = layer.mixer.forward(a, x32, ctx, cache, write)
        if _fuses(layer.feed_forward, layer.ffn_norm, rows):
            return layer.feed_forward.forward(None, r32, ctx, norm=layer.ffn_norm)
        d, _ = layer.ffn_norm.forward(r32, out_t=True)
        return layer.feed_forward.forward(d, r32, ctx)


class PostNorm(Part):
    needs = ("mixer_norm", "ffn_norm", "feed_forward")

    def forward(self, x32: torch.Tensor, layer, ctx, cache, write: bool = True) -> torch.Tensor:
        x_t = x32 if self.dtype == torch.float32 else K.cast(x32, self.dtype)
        s32 = layer.mixer.forward(x_t, x32, ctx, cache, write)
        r_t, r32 = layer.mixer_norm.forward(s32, out_t=True, out_f32=True)
        u32 = layer.feed_forward.forward(r_t, r32, ctx)
        _, y32 = layer.ffn_norm.forward(u32, out_t=False, out_f32=True)
        return y32
