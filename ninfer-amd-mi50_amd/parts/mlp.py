"""Dense SwiGLU feed-forward: (silu(x Wg^T) * (x Wu^T)) Wd^T, no biases.

Gate and up weights are stacked into one [2 I, hidden] matrix, rows [0, I)
gate and [I, 2I) up (reference src/models/model.hip:585-617); the activation
runs in the product's epilogue (the reference does so only for one row,
src/ops/gemv.hip:103-166, and otherwise in a kernel of its own,
src/ops/kernels.hip:131-140).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import FeedForward, StepContext, WeightBinder


class SwiGLU(FeedForward):
    def __init__(self, prefix: str, hidden: int, inner: int, act: str = "silu", bias: bool = False,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"),
                 act_limit: float = 0.0, act_alpha: float = 1.0):
        """`names`: what follows the prefix in the names of the gate's, the other half's and the
        down product's weights. `act` 'clamped_swish': g sigmoid(act_alpha g) (u + 1) with g cut
        at act_limit from above and u to [-act_limit, act_limit]."""
        self.act_limit, self.act_alpha = float(act_limit), float(act_alpha)
        self.prefix = prefix
        self.names = tuple(names)
        self.hidden = hidden
        self.inner = inner
        self.act = act   # the gate's activation: 'silu' | 'gelu_pytorch_tanh' | 'clamped_swish'
        self.bias = bias   # gate_proj.bias, up_proj.bias [inner] and down_proj.bias [hidden] are read
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None
        self.b_gate_up: Optional[torch.Tensor] = None
        self.b_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p = self.prefix
        specs = {p + self.names[0]: TensorSpec((self.inner, self.hidden)),
                 p + self.names[1]: TensorSpec((self.inner, self.hidden)),
                 p + self.names[2]: TensorSpec((self.hidden, self.inner))}
        if self.bias:
            specs[p + "gate_proj.bias"] = TensorSpec((self.inner,), "bias")
            specs[p + "up_proj.bias"] = TensorSpec((self.inner,), "bias")
            specs[p + "down_proj.bias"] = TensorSpec((self.hidden,), "bias")
        return specs

    def bind(self, w: WeightBinder) -> None:
        p = self.prefix
        self.w_gate_up = torch.empty((2 * self.inner, self.hidden), dtype=w.act_dtype,
                                     device=w.device)
        w.matrix_into(p + self.names[0], self.w_gate_up[:self.inner])
        w.matrix_into(p + self.names[1], self.w_gate_up[self.inner:])
        self.w_down = w.matrix(p + self.names[2])
        if self.bias:
            self.b_gate_up = torch.cat([w.float32(p + "gate_proj.bias"), w.float32(p + "up_proj.bias")])
            w.hold(p + "gate_proj.bias", self.b_gate_up[:self.inner])
            w.hold(p + "up_proj.bias", self.b_gate_up[self.inner:])
            self.b_down = w.float32(p + "down_proj.bias")

    def weight_bytes(self) -> int:
        """What one pass over the two weight matrices reads."""
        return 3 * self.inner * self.hidden * self.w_down.element_size()

    def gate_up(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        h = ctx.empty((x.shape[0], self.inner))
        if self.act == "clamped_swish":
            ctx.ops.swiglu_linear(x, self.w_gate_up, h, act=self.act, bias=self.b_gate_up,
                                  limit=self.act_limit, alpha=self.act_alpha)
        else:
            ctx.ops.swiglu_linear(x, self.w_gate_up, h, act=self.act, bias=self.b_gate_up)
        return h

    def down(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        out = ctx.empty((h.shape[0], self.hidden))
        ctx.ops.linear(h, self.w_down, out, bias=self.b_down)
        return out

    def run(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        return self.down(ctx, self.gate_up(ctx, x))

    def forward(self, ctx: StepContext, x, residual):
        return self.run(ctx, x)


register_part("feed_forward", "swiglu", SwiGLU)


class MLP(FeedForward):
    """Dense feed-forward without a gate: act(x Wu^T) Wd^T, no biases. `act`: 'relu2', the
    square of relu. `names`: what follows the prefix in the names of the two weights."""

    ACTS = ("relu2",)

    def __init__(self, prefix: str, hidden: int, inner: int, act: str = "relu2",
                 names=("up", "down")):
        if act not in self.ACTS:
            raise ValueError(f"activation {act!r} is not one of {self.ACTS}")
        self.prefix = prefix
        self.names = tuple(names)
        self.hidden = hidden
        self.inner = inner
        self.act = act
        self.w_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p = self.prefix
        return {p + self.names[0]: TensorSpec((self.inner, self.hidden)),
                p + self.names[1]: TensorSpec((self.hidden, self.inner))}

    def bind(self, w: WeightBinder) -> None:
        self.w_up = w.matrix(self.prefix + self.names[0])
        self.w_down = w.matrix(self.prefix + self.names[1])

    def forward(self, ctx: StepContext, x, residual):
        h = ctx.empty((x.shape[0], self.inner))
        ctx.ops.linear(x, self.w_up, h, act=self.act)
        out = ctx.empty((x.shape[0], self.hidden))
        ctx.ops.linear(h, self.w_down, out)
        return out


register_part("feed_forward", "mlp", MLP)
