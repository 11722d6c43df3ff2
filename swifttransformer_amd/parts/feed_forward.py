"""Dense feed-forward: y = act(x W1^T + b1) W2^T + b2, returned added to the residual.

Reference src/csrc/layer/ffn.cc:71-124: FC1 product, fused bias+activation kernel,
FC2 product, bias kernel; the residual add is a further kernel
(src/csrc/model/gpt/gpt.cc:496-501).  Here bias+ReLU is the FC1 product's epilogue and
bias+residual the FC2 product's."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..ops import kernels as K
from ..weights.loader import TensorSpec
from .base import Part



class DenseFeedForward(Part):
    """params: inner (int), activation (a name the products' epilogues know), bias (bool)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.inner = int(self.param("inner"))
        self.activation = str(self.param("activation", "relu"))
        if self.activation not in K.ACTIVATIONS:
            raise ValueError(f"feed-forward activation {self.activation!r} has no kernel; "
                             f"available: {sorted(K.ACTIVATIONS)}")
        self.bias = bool(self.param("bias", True))
        self.w1 = self.b1 = self.w2 = self.b2 = None

    def tensor_specs(self) -> List[TensorSpec]:
        H, F = self.hidden_size, self.inner
        specs = [TensorSpec(self.name("fc1.weight"), (F, H), "matrix"),
                 TensorSpec(self.name("fc2.weight"), (H, F), "matrix")]
        if self.bias:
            specs += [TensorSpec(self.name("fc1.bias"), (F,), "vector"),
                      TensorSpec(self.name("fc2.bias"), (H,), "vector")]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w1 = tensors[self.name("fc1.weight")]
        self.w2 = tensors[self.name("fc2.weight")]
        if self.bias:
            self.b1 = tensors[self.name("fc1.bias")]
            self.b2 = tensors[self.name("fc2.bias")]

    accepts_norm = True     # forward(..., norm=part) normalises residual32 itself

    def forward(self, x_t, residual32: torch.Tensor, ctx, norm=None) -> torch.Tensor:
        x_in = norm.as_input(residual32) if norm is not None else x_t
        h = K.gemm(x_in, self.w1, bias=self.b1, activation=self.activation)
        return K.gemm(h, self.w2, bias=self.b2, residual=residual32, out_f32=True)
