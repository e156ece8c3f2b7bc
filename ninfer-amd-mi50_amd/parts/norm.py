"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * gain, in 32-bit; and the layer norm without a
bias, y = (x - mean(x)) * rsqrt(mean((x - mean(x))^2) + eps) * gain (`center`).

Reference: src/ops/kernels.hip:17-41; with the residual sum fused in,
:100-129. The residual stream is kept in 32-bit here (the reference keeps it
in half precision), so the sum is never rounded to the storage type.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import Norm, Part, PendingRows, StepContext, WeightBinder


class RMSNorm(Norm):
    def __init__(self, prefix: str, size: int, eps: float, leaf: str = "weight",
                 single_gain: bool = False, center: bool = False):
        """`leaf`: what follows the prefix in the gain's name ('' when the prefix is the whole
        name). `single_gain`: the checkpoint holds one number (shape []) for all columns.
        `center`: the row's mean is taken off first (a layer norm without a bias)."""
        self.center = bool(center)
        self.prefix = prefix
        self.size = size
        self.eps = eps
        self.leaf = leaf
        self.single_gain = single_gain
        self.gain: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.prefix + self.leaf: TensorSpec(() if self.single_gain else (self.size,), "gain")}

    def bind(self, w: WeightBinder) -> None:
        self.gain = w.float32(self.prefix + self.leaf)
        if self.single_gain:   # the kernel reads one gain per column
            self.gain = self.gain.reshape(1).expand(self.size).contiguous()

    def forward(self, ctx: StepContext, residual, pending):
        out = ctx.empty((residual.shape[0], self.size))
        if isinstance(pending, PendingRows):
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, rows_sum=pending, center=self.center)
        else:
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, delta=pending, center=self.center)
        return out

    def forward_rows(self, ctx: StepContext, residual, rows, pending=None):
        out = ctx.empty((rows.shape[0], self.size))
        if isinstance(pending, PendingRows):
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, rows_sum=pending, rows=rows,
                            center=self.center)
        else:
            ctx.ops.rmsnorm(residual, self.gain, self.eps, out, delta=pending, rows=rows,
                            center=self.center)
        return out


class OutputRMSNorm(Part):
    """The norm of a block that norms what a sublayer gives back, not what it reads:
    residual += y rsqrt(mean(y^2) + eps) gain, in 32-bit, where the gain is one number for
    all columns (`single_gain`, shape []) or one per column. `center`: the layer norm instead
    (y's mean taken off first). `add` takes plain rows, or a `PendingRows` of a sparse
    feed-forward (weights and rows only), whose weighted sum is formed and normed in 32-bit."""

    def __init__(self, tensor: str, size: int, eps: float, single_gain: bool = True,
                 center: bool = False):
        self.center = bool(center)
        self.tensor = tensor
        self.size = size
        self.eps = eps
        self.single_gain = single_gain
        self.gain: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec(() if self.single_gain else (self.size,), "gain")}

    def bind(self, w: WeightBinder) -> None:
        self.gain = w.float32(self.tensor).reshape(-1)

    def add(self, ctx: StepContext, residual: torch.Tensor, y) -> None:
        if isinstance(y, PendingRows):
            if y.shared is not None or y.ids is not None:
                raise ValueError("a norm on a sparse feed-forward's output takes weighted rows only")
            ctx.ops.norm_add(residual, y.y, self.gain, self.eps, center=self.center,
                             weights=y.weights)
        else:
            ctx.ops.norm_add(residual, y, self.gain, self.eps, center=self.center)


class LayerNorm(RMSNorm):
    """(x - mean) rsqrt(variance + eps) gain, the variance the mean of the squared deviations;
    no bias."""

    def __init__(self, prefix: str, size: int, eps: float, leaf: str = "weight"):
        super().__init__(prefix, size, eps, leaf=leaf, center=True)


class OutputLayerNorm(OutputRMSNorm):
    """residual += layer norm of what a sublayer gives back, a gain per column, no bias."""

    def __init__(self, tensor: str, size: int, eps: float):
        super().__init__(tensor, size, eps, single_gain=False, center=True)


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "output_rmsnorm", OutputRMSNorm)
register_part("norm", "layernorm", LayerNorm)
register_part("norm", "output_layernorm", OutputLayerNorm)
