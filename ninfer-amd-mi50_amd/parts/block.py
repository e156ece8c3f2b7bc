"""Pre-norm residual block: x += mixer(norm1(x)); x += feed_forward(norm2(x)).

Reference order: src/models/model.hip:206-444 (layer_start, layer_mid,
end_layer). A part's output is not added at once: it is handed on as
`pending` and summed into the 32-bit residual by the next norm's kernel (the
reference fuses the same sum with the post-attention norm only,
src/ops/kernels.hip:100-129).
"""
from __future__ import annotations

from typing import List, Optional

from ..registry import register_part
import torch

from ..weights.source import TensorSpec
from .base import (Block, CallInfo, FeedForward, Mixer, Norm, Part, PendingRows, StepContext,
                   WeightBinder, settle)


class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ff_norm: Norm, feed_forward: FeedForward):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ff_norm = ff_norm
        self.feed_forward = feed_forward

    def children(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def forward(self, ctx: StepContext, residual, pending, call: CallInfo):
        a = self.mixer_norm.forward(ctx, residual, pending)
        pending = self.mixer.forward(ctx, a, residual, call)
        m = self.ff_norm.forward(ctx, residual, pending)
        return self.feed_forward.forward(ctx, m, residual)


register_part("block", "pre_norm", PreNormBlock)


class OutputNormBlock(Block):
    """A block whose norms sit on the sublayers' outputs: x += norm1(mixer(in1(x))), then
    x += norm2(feed_forward(in2(x))). The sublayers read the 32-bit residual itself, through an
    optional input part each (`mixer_input`, `ff_input`: e.g. a short convolution with state of
    its own); `feed_forward` may be None (a layer with a mixer only). The block adds into the
    residual itself and hands nothing on. Its per-request state holds, in this order, the
    mixer input's, the mixer's and the feed-forward input's."""

    def __init__(self, mixer: Mixer, mixer_norm: Part, feed_forward: Optional[FeedForward] = None,
                 ff_norm: Optional[Part] = None, mixer_input: Optional[Part] = None,
                 ff_input: Optional[Part] = None):
        if (feed_forward is None) != (ff_norm is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.mixer = mixer
        self.mixer_norm = mixer_norm
        self.feed_forward = feed_forward
        self.ff_norm = ff_norm
        self.mixer_input = mixer_input
        self.ff_input = ff_input if feed_forward is not None else None

    def children(self) -> List[Part]:
        return [p for p in (self.mixer_input, self.mixer, self.mixer_norm, self.ff_input,
                            self.feed_forward, self.ff_norm) if p is not None]

    def _state_parts(self):
        a = self.mixer_input.state_floats() if self.mixer_input is not None else 0
        b = self.mixer.state_floats()
        c = self.ff_input.state_floats() if self.ff_input is not None else 0
        return a, b, c

    def state_floats(self) -> int:
        return sum(self._state_parts())

    def _read(self, ctx: StepContext, residual, part, state):
        if part is not None:
            return part.forward(ctx, residual, state)
        if residual.dtype == ctx.act_dtype:
            return residual
        return residual.to(ctx.act_dtype)

    def forward(self, ctx: StepContext, residual, pending, call: CallInfo):
        settled = settle(ctx, residual, pending)
        if settled is not None:
            residual.add_(settled)
        a, b, c = self._state_parts()
        st = call.state
        h = self._read(ctx, residual, self.mixer_input, st[:, :a] if a else None)
        inner = CallInfo(cache=call.cache, writes_cache=call.writes_cache,
                         state=st[:, a:a + b] if b else None)
        self.mixer_norm.add(ctx, residual, self.mixer.forward(ctx, h, residual, inner))
        if self.feed_forward is not None:
            h = self._read(ctx, residual, self.ff_input, st[:, a + b:a + b + c] if c else None)
            y = settle(ctx, residual, self.feed_forward.forward(ctx, h, residual))
            self.ff_norm.add(ctx, residual, y)
        return None


register_part("block", "output_norm", OutputNormBlock)


class SandwichBlock(Block):
    """A block with a norm before and after each sublayer: x += post1(mixer(pre1(x))), then
    x += post2(feed_forward(pre2(x))). The norms before are `Norm`s of the residual, those after
    parts with `add(ctx, residual, y)` (they norm y and add it into the 32-bit residual; a
    sparse feed-forward's weighted rows are summed by the same kernel). `feed_forward` may be
    None (a layer with a mixer only)."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_out_norm: Part,
                 ff_norm: Optional[Norm] = None, feed_forward: Optional[FeedForward] = None,
                 ff_out_norm: Optional[Part] = None):
        if (feed_forward is None) != (ff_norm is None) or (feed_forward is None) != (ff_out_norm is None):
            raise ValueError("a feed-forward and its two norms come together or not at all")
        self.mixer_norm, self.mixer, self.mixer_out_norm = mixer_norm, mixer, mixer_out_norm
        self.ff_norm, self.feed_forward, self.ff_out_norm = ff_norm, feed_forward, ff_out_norm

    def children(self) -> List[Part]:
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_out_norm, self.ff_norm,
                            self.feed_forward, self.ff_out_norm) if p is not None]

    def forward(self, ctx: StepContext, residual, pending, call: CallInfo):
        h = self.mixer_norm.forward(ctx, residual, pending)
        self.mixer_out_norm.add(ctx, residual, self.mixer.forward(ctx, h, residual, call))
        if self.feed_forward is not None:
            h = self.ff_norm.forward(ctx, residual, None)
            y = self.feed_forward.forward(ctx, h, residual)
            if y is None:
                raise ValueError("a feed-forward between two norms hands its rows back")
            self.ff_out_norm.add(ctx, residual, y)
        return None


register_part("block", "sandwich", SandwichBlock)


class ParallelBlock(Block):
    """A block whose sublayers run side by side on the same residual: h = norm(x), then
    x += mult (c1 mixer(h) + c2 feed_forward(h2)), where h2 = h, or ff_norm(x) when the block
    has a second norm of the same x (`ff_norm`), and c1, c2 are per-column factors:
    a learned factor per column (`mixer_scale`, `ff_scale`: tensor names, None for no factor),
    or a gate computed from the sublayer's own input, c = sigmoid(W h + b) per row and column
    (`mixer_gate`, `ff_gate`: the name of W [size, size]; its bias is that name + ".b").
    `feed_forward` may be None. The sum is formed in 32-bit by one kernel, which also adds up
    a sparse feed-forward's weighted rows."""

    def __init__(self, norm: Norm, mixer: Mixer, feed_forward: Optional[FeedForward] = None,
                 mixer_scale: Optional[str] = None, ff_scale: Optional[str] = None, size: int = 0,
                 ff_norm: Optional[Norm] = None, mult: float = 1.0,
                 mixer_gate: Optional[str] = None, ff_gate: Optional[str] = None):
        if (mixer_scale and mixer_gate) or (ff_scale and ff_gate):
            raise ValueError("a sublayer has a learned factor or a gate, not both")
        self.norm = norm
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.ff_norm = ff_norm if feed_forward is not None else None
        self.spare_norm = ff_norm if feed_forward is None else None
        self.mult = float(mult)
        self.mixer_scale_name = mixer_scale
        self.ff_scale_name = ff_scale if feed_forward is not None else None
        self.spare_scale_name = ff_scale if feed_forward is None else None
        self.mixer_gate_name = mixer_gate
        self.ff_gate_name = ff_gate if feed_forward is not None else None
        self.spare_gate_name = ff_gate if feed_forward is None else None
        self.size = size
        self.mixer_scale: Optional[torch.Tensor] = None
        self.ff_scale: Optional[torch.Tensor] = None
        self.mixer_gate = self.mixer_gate_bias = self.ff_gate = self.ff_gate_bias = None

    def children(self) -> List[Part]:
        return [p for p in (self.norm, self.mixer, self.ff_norm, self.feed_forward) if p is not None]

    def tensor_specs(self):
        specs = {n: TensorSpec((self.size,), "gain")
                 for n in (self.mixer_scale_name, self.ff_scale_name) if n}
        for n in (self.mixer_gate_name, self.ff_gate_name):
            if n:
                specs[n] = TensorSpec((self.size, self.size))
                specs[n + ".b"] = TensorSpec((self.size,), "bias")
        return specs

    def unused_tensor_specs(self):
        # a layer without a feed-forward may still carry what belongs to one
        out = {}
        if self.spare_scale_name:
            out[self.spare_scale_name] = TensorSpec((self.size,), "gain")
        if self.spare_gate_name:
            out[self.spare_gate_name] = TensorSpec((self.size, self.size))
            out[self.spare_gate_name + ".b"] = TensorSpec((self.size,), "bias")
        if self.spare_norm is not None:
            out.update(self.spare_norm.all_tensor_specs())
        return out

    def bind(self, w: WeightBinder) -> None:
        if self.mixer_scale_name:
            self.mixer_scale = w.float32(self.mixer_scale_name)
        if self.ff_scale_name:
            self.ff_scale = w.float32(self.ff_scale_name)
        if self.mixer_gate_name:
            self.mixer_gate = w.matrix(self.mixer_gate_name)
            self.mixer_gate_bias = w.float32(self.mixer_gate_name + ".b")
        if self.ff_gate_name:
            self.ff_gate = w.matrix(self.ff_gate_name)
            self.ff_gate_bias = w.float32(self.ff_gate_name + ".b")

    def _gate(self, ctx: StepContext, h, weight):
        if weight is None:
            return None
        g = ctx.empty((h.shape[0], self.size))
        ctx.ops.linear(h, weight, g)
        return g

    def forward(self, ctx: StepContext, residual, pending, call: CallInfo):
        h = self.norm.forward(ctx, residual, pending)
        h2 = h
        if self.ff_norm is not None:
            h2 = self.ff_norm.forward(ctx, residual, None)
        a = self.mixer.forward(ctx, h, residual, call)
        f = self.feed_forward.forward(ctx, h2, residual) if self.feed_forward is not None else None
        if self.mixer_gate is None and self.ff_gate is None and self.mult == 1.0:
            ctx.ops.scaled_sum_add(residual, a, self.mixer_scale, f, self.ff_scale)
            return None
        if self.mixer_scale is not None or self.ff_scale is not None:
            raise ValueError("learned column factors beside gates or a multiplier are not built")
        ctx.ops.gated_sum_add(residual, a, self._gate(ctx, h, self.mixer_gate), self.mixer_gate_bias,
                              f, self._gate(ctx, h2, self.ff_gate), self.ff_gate_bias, self.mult)
        return None


register_part("block", "parallel", ParallelBlock)
