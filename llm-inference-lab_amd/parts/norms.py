"""Norms."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.loader import TensorSpec, VECTOR, INIT_NORM, INIT_NORMAL
from .base import Norm
from .registry import register_part


class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * w`` with the square, mean, rsqrt and
    both products in float32 and one rounding to the compute dtype at the end.

    Formula: rust/engine/src/runner/model/qwen2/kernels.rs:546-582 (the
    reference rounds once more, before the weight product; in float32 the two
    are the same).  ``size`` and ``eps`` come from the caller.  ``weight_offset``: the stored
    tensor is the scale less this constant (a weight kept around zero has ``weight_offset=1``:
    ``w = 1 + stored``); the sum is taken once, in float32, when the part is bound.  ``scalar``: the
    stored weight is ONE number for all coordinates (a tensor without axes); it is spread over the
    width when the part is bound, so every kernel that takes an RMS norm's weight serves it."""

    folds_pending = True
    keeps_launches = True

    def __init__(self, size: int, eps: float, tensors: Dict[str, str], weight_offset: float = 0.0,
                 scalar: bool = False):
        super().__init__(tensors)
        self.size = int(size)
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.scalar = bool(scalar)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec(() if self.scalar else (self.size,), VECTOR,
                                                        INIT_NORMAL if self.weight_offset else INIT_NORM)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.weight = tensors[self.tensor_names["weight"]].contiguous()
        if self.scalar:
            self.weight = self.weight.reshape(1).expand(self.size).contiguous()
        if self.weight_offset:
            self.weight = (self.weight.float() + self.weight_offset).contiguous()

    def forward(self, x, out, rows=None, pending=None):
        if pending is None:
            self.ops.rmsnorm(x, self.weight, self.eps, out, rows)
        else:
            self.ops.rmsnorm(x, self.weight, self.eps, out, rows, pending=pending)

    def rms_params(self):
        return self.weight, self.eps

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


class LayerNorm(Norm):
    """``y = (x - mean(x)) / sqrt(var(x) + eps) * w`` with ``var`` the mean of the squared
    deviations, a weight and no bias; everything in float32, one rounding at the end.
    ``add_into`` serves blocks that norm a sublayer's OUTPUT: ``stream += norm(y)``."""

    keeps_launches = True

    def __init__(self, size: int, eps: float, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.size = int(size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.size,), VECTOR, INIT_NORM)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.weight = tensors[self.tensor_names["weight"]].contiguous()

    def forward(self, x, out, rows=None):
        self.ops.layernorm(x, self.weight, self.eps, out, rows)

    def add_into(self, y, stream, copy=None):
        """``stream += norm(y)``; ``copy`` (compute dtype) receives the stream's new rows."""
        self.ops.layernorm_add(y, self.weight, self.eps, stream, copy)

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
