"""Grouped-query attention over the paged cache.

q, k, v = x W^T (+ b) as one fused product over the stacked weight
[(Hq + 2 Hkv) D, hidden] (the reference fuses the same way,
src/models/model.hip:529-558, but has no bias); q and k are rotated, k and v
are written into the request's pages, and every row attends to the keys of
its request at positions <= its own (reference src/ops/attention.hip:216),
within `window` positions if the layer has one. Query head h reads kv head
h // (Hq / Hkv) (src/ops/attention.hip:27-28); scale 1/sqrt(D)
(src/models/model.hip:285). The output projection has no bias.

Parameters beyond the reference's layer: values of another size than keys (`vdim`); a short
causal convolution over time on every channel of the projected q, k and v (`conv_taps`, the
last taps - 1 projected rows of a request being per-request state); a softmax with a sink
(`sink`: one more term exp(0) in the denominator, so that a row may attend to nothing); and
a layer without key and value projections that reads the keys and values another layer's
run has cached (`own_kv` False), with queries, window and everything else of its own.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CacheNeed, CallInfo, Mixer, Part, PositionEncoding, StepContext, WeightBinder


class Attention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, kv_heads: int, head_dim: int,
                 position: PositionEncoding, qkv_bias: bool = True,
                 window: Optional[int] = None, scale: Optional[float] = None,
                 score_slopes: Optional[Sequence[float]] = None,
                 qk_norm_eps: Optional[float] = None, page_size: Optional[int] = None,
                 vdim: Optional[int] = None, conv_taps: int = 0, sink: bool = False,
                 own_kv: bool = True, names=None, cache_window="same"):
        """`score_slopes` [heads]: a distance-based position bias, slope * (key's position -
        query's position) added to head h's scaled scores before the softmax (None: none).
        It is a parameter of the attention kernels, beside or instead of the rotation that
        `position` describes. `qk_norm_eps`: every query and key head is normed over its dims
        (x rsqrt(mean(x^2) + eps) gain, gains `q_norm.weight` and `k_norm.weight` [head_dim] of the
        checkpoint) after the bias and before it turns; None: no such norm. `page_size`: tokens
        in a page of this layer's keys and values (None: the engine's). `vdim`: numbers of a
        value head (None: head_dim). `conv_taps` > 0: the projected q, k and v pass a causal
        convolution over time, channel by channel (weights `<projection>.conv` [channels,
        taps], no bias), before norm and rotation. `sink`: see above. `own_kv` False: no key
        and value tensors; the layer's plan entry names the cache it reads. `names`: what
        follows the prefix in the tensors' names, a dict with any of the keys q, k, v, o,
        q_norm, k_norm, conv (the suffix of a projection's convolution). `cache_window`: the
        span of positions whose keys and values the cache keeps, when it differs from this
        layer's own window (None: all; other layers with wider windows read this cache)."""
        self.cache_window = window if cache_window == "same" else cache_window
        self.vdim = head_dim if vdim is None else int(vdim)
        self.conv_taps, self.sink, self.own_kv = int(conv_taps), bool(sink), bool(own_kv)
        if self.conv_taps < 0:
            raise ValueError(f"conv_taps ({conv_taps}) must be >= 0")
        self.names = dict({"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight",
                           "o": "o_proj.weight", "q_norm": "q_norm.weight",
                           "k_norm": "k_norm.weight", "conv": ".conv"}, **(names or {}))
        # the fused product + rotation + cache write serves the plain layer; everything else
        # (values of their own size, a convolution, another layer's cache) goes the general way
        self.general = self.vdim != head_dim or self.conv_taps > 0 or not self.own_kv
        if self.general and qkv_bias:
            raise ValueError("q/k/v biases beside a convolution, values of their own size or "
                             "another layer's cache are not built")
        self.w_conv: Optional[torch.Tensor] = None     # [channels, taps], as the checkpoint has it
        self.w_conv_t: Optional[torch.Tensor] = None   # [taps, channels]: a tap's weights side by side
        if heads % kv_heads:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if score_slopes is not None and len(score_slopes) != heads:
            raise ValueError(f"score_slopes has {len(score_slopes)} entries for {heads} heads")
        self.prefix = prefix
        self.hidden = hidden
        self.heads = heads
        self.kv_heads = kv_heads
        self.head_dim = head_dim
        self.position = position
        self.qkv_bias = qkv_bias
        self.window = window
        self.scale = scale if scale is not None else 1.0 / math.sqrt(head_dim)
        self.score_slopes = None if score_slopes is None else [float(x) for x in score_slopes]
        self.slopes: Optional[torch.Tensor] = None   # the same on the device (32-bit)
        self.qk_norm_eps = qk_norm_eps
        self.page_size = page_size
        self.q_norm: Optional[torch.Tensor] = None
        self.k_norm: Optional[torch.Tensor] = None
        self.w_qkv: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    @property
    def qkv_width(self) -> int:
        kv = self.kv_heads * (self.head_dim + self.vdim) if self.own_kv else 0
        return self.heads * self.head_dim + kv

    def cache_need(self) -> Optional[CacheNeed]:
        if not self.own_kv:
            return None
        return CacheNeed.keys_values(self.kv_heads, self.head_dim, self.cache_window,
                                     self.page_size, vdim=self.vdim)

    def state_floats(self) -> int:
        """The last conv_taps - 1 projected rows of a request."""
        return max(self.conv_taps - 1, 0) * self.qkv_width

    def children(self) -> List[Part]:
        return [self.position]

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, d, n = self.prefix, self.head_dim, self.names
        specs = {p + n["q"]: TensorSpec((self.heads * d, self.hidden)),
                 p + n["o"]: TensorSpec((self.hidden, self.heads * self.vdim))}
        if self.own_kv:
            specs[p + n["k"]] = TensorSpec((self.kv_heads * d, self.hidden))
            specs[p + n["v"]] = TensorSpec((self.kv_heads * self.vdim, self.hidden))
        if self.conv_taps:
            for key, width in (("q", self.heads * d), ("k", self.kv_heads * d),
                               ("v", self.kv_heads * self.vdim)):
                if key == "q" or self.own_kv:
                    specs[p + n[key] + n["conv"]] = TensorSpec((width, self.conv_taps), "gain")
        if self.qkv_bias:
            specs[p + "q_proj.bias"] = TensorSpec((self.heads * d,), "bias")
            specs[p + "k_proj.bias"] = TensorSpec((self.kv_heads * d,), "bias")
            specs[p + "v_proj.bias"] = TensorSpec((self.kv_heads * d,), "bias")
        if self.qk_norm_eps is not None:
            specs[p + n["q_norm"]] = TensorSpec((d,), "gain")
            if self.own_kv:
                specs[p + n["k_norm"]] = TensorSpec((d,), "gain")
        return specs

    def unused_tensor_specs(self) -> Dict[str, TensorSpec]:
        # older checkpoints store the rotation's frequency table, which is computed here
        if self.position.rot_dim > 0:
            return {self.prefix + "rotary_emb.inv_freq": TensorSpec((self.position.rot_dim // 2,))}
        return {}

    def bind(self, w: WeightBinder) -> None:
        p, d, n = self.prefix, self.head_dim, self.names
        nq, nk = self.heads * d, self.kv_heads * d
        if self.score_slopes is not None:
            self.slopes = torch.tensor(self.score_slopes, dtype=torch.float32, device=w.device)
        if self.qk_norm_eps is not None:
            self.q_norm = w.float32(p + n["q_norm"])
            self.k_norm = w.float32(p + n["k_norm"]) if self.own_kv else None
        self.w_qkv = torch.empty((self.qkv_width, self.hidden), dtype=w.act_dtype, device=w.device)
        w.matrix_into(p + n["q"], self.w_qkv[:nq])
        if self.own_kv:
            w.matrix_into(p + n["k"], self.w_qkv[nq:nq + nk])
            w.matrix_into(p + n["v"], self.w_qkv[nq + nk:])
        if self.conv_taps:
            keys = ("q", "k", "v") if self.own_kv else ("q",)
            parts = [w.float32(p + n[key] + n["conv"]) for key in keys]
            self.w_conv = torch.cat(parts).contiguous()
            self.w_conv_t = self.w_conv.t().contiguous()
            o = 0
            for key, part in zip(keys, parts):
                w.hold(p + n[key] + n["conv"], self.w_conv[o:o + part.shape[0]])
                o += part.shape[0]
        if self.qkv_bias:
            self.b_qkv = torch.cat([w.float32(p + "q_proj.bias"), w.float32(p + "k_proj.bias"),
                                    w.float32(p + "v_proj.bias")])
            w.hold(p + "q_proj.bias", self.b_qkv[:nq])
            w.hold(p + "k_proj.bias", self.b_qkv[nq:nq + nk])
            w.hold(p + "v_proj.bias", self.b_qkv[nq + nk:])
        self.w_o = w.matrix(p + n["o"])

    def _forward_general(self, ctx: StepContext, x, call: CallInfo):
        """Product, then one kernel for convolution, head norms, rotation and the cache write,
        then attention over keys and values of sizes of their own."""
        ops, cache = ctx.ops, call.cache
        if call.writes_cache != self.own_kv:
            raise ValueError(f"{self.prefix}: a layer with key/value projections writes a cache of "
                             f"its own, one without reads another's")
        u = ctx.empty((ctx.T, self.qkv_width))
        ops.linear(x, self.w_qkv, u)
        q = ctx.empty((ctx.T, self.heads * self.head_dim))
        ops.qkv_conv(u, self.w_conv, call.state, ctx, q, self.heads,
                     self.kv_heads if self.own_kv else 0, self.head_dim, self.vdim, cache["k"],
                     cache["v"], cache.block_table, cache.page_size, q_norm=self.q_norm,
                     k_norm=self.k_norm, norm_eps=self.qk_norm_eps or 0.0,
                     inv_freq=self.position.table(), rot_dim=self.position.rot_dim,
                     interleaved=self.position.pairing == "interleaved", w_conv_t=self.w_conv_t)
        attn = ctx.empty((ctx.T, self.heads * self.vdim))
        ops.paged_attention(q, cache["k"], cache["v"], cache.block_table, ctx, self.heads,
                            self.kv_heads, self.head_dim, cache.page_size, self.window, self.scale,
                            attn, slopes=self.slopes, vdim=self.vdim, sink=self.sink)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(attn, self.w_o, out)
        return out

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        if self.general:
            return self._forward_general(ctx, x, call)
        ops = ctx.ops
        cache = call.cache
        qkv = ctx.empty((ctx.T, self.qkv_width))
        # the product, then bias, rotation of q and k, and the write of k, v into pages
        ops.qkv_rope(x, self.w_qkv, self.b_qkv, qkv, ctx.positions, ctx.row_seq,
                     self.position.table(), self.position.rot_dim, self.heads, self.kv_heads,
                     self.head_dim, cache["k"], cache["v"], cache.block_table,
                     cache.page_size, write_kv=call.writes_cache,
                     interleaved=self.position.pairing == "interleaved",
                     q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps or 0.0)
        attn = ctx.empty((ctx.T, self.heads * self.head_dim))
        ops.paged_attention(qkv, cache["k"], cache["v"], cache.block_table, ctx,
                            self.heads, self.kv_heads, self.head_dim,
                            cache.page_size, self.window, self.scale, attn, slopes=self.slopes,
                            sink=self.sink)
        out = ctx.empty((ctx.T, self.hidden))
        ops.linear(attn, self.w_o, out)
        return out


register_part("mixer", "attention", Attention)
