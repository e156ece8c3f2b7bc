"""Attention without a softmax, over the paged cache, with grouped key/value heads.

The weight of a visible key is a sigmoid of its score, not a share of a sum over keys:
    w_a(i, j) = sigmoid((q_a,i . k_c(a),j) scale + bias_a)      c(a) = a // (heads / kv_heads)
for key j visible to row i, else 0; weights are not normalised. The heads' weights may then be
mixed, w'_a(i, j) = sum_b M[a, b] w_b(i, j) with a learned [heads, heads] matrix M ("talking
heads"), and head a applies w'_a to the values of its own key/value head; the heads go through
the output projection. Visible: j <= i and, with `chunk`, floor(i / chunk) == floor(j / chunk),
chunks counted from the request's position 0. No rotation: positions enter through the mask
only. Scores, weights and their mixing are 32-bit; the cache holds k [dim] and v [vdim] per
kv head in pools of their own. A layer may read the keys and values another layer's run has
written (`own_kv` False: it has no key/value projections and writes nothing).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CacheNeed, CallInfo, Mixer, PoolSpec, StepContext, WeightBinder


class SigmoidAttention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 scale: float, chunk: Optional[int] = None, head_bias: bool = True,
                 head_mix: bool = True, own_kv: bool = True, page_size: Optional[int] = None,
                 names=("q", "k", "v", "o", "pb", "talk")):
        """`names`: what follows the prefix in the names of the three projections, the output
        projection, the heads' score bias [heads] and the mixing matrix [heads, heads].
        `head_bias` / `head_mix` False: no such tensor (bias 0 / no mixing)."""
        if heads % kv_heads:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if chunk is not None and chunk < 1:
            raise ValueError(f"chunk ({chunk}) must be positive")
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = hidden, heads, kv_heads, dim, vdim
        self.scale, self.chunk = float(scale), chunk
        self.has_bias, self.has_mix, self.own_kv = head_bias, head_mix, own_kv
        self.page_size = page_size
        self.w_in: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.mix: Optional[torch.Tensor] = None

    @property
    def in_width(self) -> int:
        kv = self.kv_heads * (self.dim + self.vdim) if self.own_kv else 0
        return self.heads * self.dim + kv

    def cache_need(self) -> Optional[CacheNeed]:
        if not self.own_kv:
            return None
        return CacheNeed((PoolSpec("k", (self.kv_heads,), (self.dim,)),
                          PoolSpec("v", (self.kv_heads,), (self.vdim,))), None, self.page_size)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, n = self.prefix, self.names
        specs = {p + n[0]: TensorSpec((self.heads * self.dim, self.hidden)),
                 p + n[3]: TensorSpec((self.hidden, self.heads * self.vdim))}
        if self.own_kv:
            specs[p + n[1]] = TensorSpec((self.kv_heads * self.dim, self.hidden))
            specs[p + n[2]] = TensorSpec((self.kv_heads * self.vdim, self.hidden))
        if self.has_bias:
            specs[p + n[4]] = TensorSpec((self.heads,), "bias")
        if self.has_mix:
            specs[p + n[5]] = TensorSpec((self.heads, self.heads), "bias")
        return specs

    def bind(self, w: WeightBinder) -> None:
        p, n = self.prefix, self.names
        nq, nk = self.heads * self.dim, self.kv_heads * self.dim
        self.w_in = torch.empty((self.in_width, self.hidden), dtype=w.act_dtype, device=w.device)
        w.matrix_into(p + n[0], self.w_in[:nq])
        if self.own_kv:
            w.matrix_into(p + n[1], self.w_in[nq:nq + nk])
            w.matrix_into(p + n[2], self.w_in[nq + nk:])
        self.w_o = w.matrix(p + n[3])
        self.bias = w.float32(p + n[4]) if self.has_bias else None
        self.mix = w.float32(p + n[5]) if self.has_mix else None

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops, cache = ctx.ops, call.cache
        if call.writes_cache != self.own_kv:
            raise ValueError(f"{self.prefix}: a layer with key/value projections writes a cache of "
                             f"its own, one without reads another's")
        qkv = ctx.empty((ctx.T, self.in_width))
        ops.linear(x, self.w_in, qkv)
        attn = ctx.empty((ctx.T, self.heads * self.vdim))
        ops.sigmoid_attention(qkv, cache["k"], cache["v"], cache.block_table, ctx, self.heads,
                              self.kv_heads, self.dim, self.vdim, cache.page_size, self.scale,
                              self.chunk or 0, self.bias, self.mix, attn, write_kv=self.own_kv)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(attn, self.w_o, out)
        return out


register_part("mixer", "sigmoid_attention", SigmoidAttention)
