"""Gated linear attention: linear attention whose state decays per key channel by a factor
that every token computes for itself.

    q = W_q h dim^(-1/2), k = W_k h   (heads x dim),   v = W_v h   (heads x vdim)
    alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau)        (heads x dim, each in (0, 1))
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t          (per head)
    y = W_o ( concat_heads(rmsnorm_vdim(o_t) * weight) * silu(W_g h) )

The four wide input products are one product over the stacked weight [2 H dim + 2 H vdim,
hidden] (q, k, v, gate). The decay's logits, the decay, the recurrence, its state and the norm
are 32-bit. The state S ([heads, dim, vdim] per request) lives in the request's state slot,
starts at zero, and is carried from step to step: nothing is kept per token, so the mixer asks
for no pages.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CallInfo, Mixer, StepContext, WeightBinder


class GatedLinearAttention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, vdim: int, tau: float,
                 eps: float, rank: Optional[int] = None, q_scale: Optional[float] = None,
                 names=("q", "k", "v", "g", "o", "norm", "a1", "a2", "a2.b")):
        """`tau`: the decay is the tau-th root of a sigmoid. `rank`: the inner size of the
        decay's two-step projection (None: whatever the checkpoint holds). `q_scale`: the
        factor on q (None: dim^(-1/2)). `names`: what follows the prefix in the names of W_q,
        W_k, W_v, W_g, W_o, the norm's weight [vdim], W_a1, W_a2 and its bias."""
        if not tau > 0:
            raise ValueError(f"tau ({tau}) must be positive")
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads, self.dim, self.vdim = hidden, heads, dim, vdim
        self.tau, self.eps, self.rank = float(tau), float(eps), rank
        self.q_scale = float(q_scale) if q_scale is not None else dim ** -0.5
        self.w_in: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.w_a1: Optional[torch.Tensor] = None
        self.w_a2: Optional[torch.Tensor] = None
        self.b_a2: Optional[torch.Tensor] = None
        self.norm_w: Optional[torch.Tensor] = None

    def state_floats(self) -> int:
        return self.heads * self.dim * self.vdim

    def _widths(self):
        qk, v = self.heads * self.dim, self.heads * self.vdim
        return qk, qk, v, v

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, n = self.prefix, self.names
        qk, _, v, _ = self._widths()
        r = self.rank if self.rank is not None else -1   # -1: any size
        return {p + n[0]: TensorSpec((qk, self.hidden)), p + n[1]: TensorSpec((qk, self.hidden)),
                p + n[2]: TensorSpec((v, self.hidden)), p + n[3]: TensorSpec((v, self.hidden)),
                p + n[4]: TensorSpec((self.hidden, v)), p + n[5]: TensorSpec((self.vdim,), "gain"),
                p + n[6]: TensorSpec((r, self.hidden)), p + n[7]: TensorSpec((qk, r)),
                p + n[8]: TensorSpec((qk,), "bias")}

    def bind(self, w: WeightBinder) -> None:
        p, n = self.prefix, self.names
        widths = self._widths()
        self.w_in = torch.empty((sum(widths), self.hidden), dtype=w.act_dtype, device=w.device)
        at = 0
        for name, width in zip(n[:4], widths):
            w.matrix_into(p + name, self.w_in[at:at + width])
            at += width
        self.w_o = w.matrix(p + n[4])
        self.norm_w = w.float32(p + n[5])
        self.w_a1 = w.matrix(p + n[6])
        self.w_a2 = w.matrix(p + n[7])
        self.b_a2 = w.float32(p + n[8])
        if self.w_a1.shape[0] != self.w_a2.shape[1]:
            raise ValueError(f"{p}: the decay's projections do not meet: {tuple(self.w_a1.shape)} "
                             f"and {tuple(self.w_a2.shape)}")

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops = ctx.ops
        qk, _, v, _ = self._widths()
        proj = ctx.empty((ctx.T, 2 * qk + 2 * v))
        ops.linear(x, self.w_in, proj)
        low = ctx.empty((ctx.T, self.w_a1.shape[0]))
        ops.linear(x, self.w_a1, low)
        z = ctx.empty((ctx.T, qk), torch.float32)     # the decay's logits, 32-bit from here on
        ops.linear(low, self.w_a2, z, bias=self.b_a2)
        o = ctx.empty((ctx.T, v), torch.float32)
        # (a step with prompt portions runs in chunks, which keep their scaled rows here)
        wf = ops.gla_work_floats(proj.dtype, ctx, self.heads, self.dim)
        work = ctx.empty((ctx.T, wf), torch.float32) if wf else None
        ops.gated_linear_attention(proj, 0, qk, 2 * qk, z, self.heads, self.dim, self.vdim,
                                   self.tau, self.q_scale, call.state, ctx, o, work=work)
        gated = ctx.empty((ctx.T, v))
        ops.gated_rmsnorm(o, proj[:, 2 * qk + v:], self.norm_w, self.eps, gated, group=self.vdim,
                          gate_act="silu")
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(gated, self.w_o, out)
        return out


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
