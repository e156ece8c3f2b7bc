"""Attention over a cached low-rank latent (multi-head latent attention).

    q = W_q h                      per head [dim unrotated | rot_dim rotated]
    [c' | r] = W_dkv h             c = rmsnorm(c') * weight  (kv_rank),  r: rot_dim numbers
    k_h = [W_uk,h c | turn(r)],    v_h = W_uv,h c
    score = (q_unrot . W_uk,h c + turn(q_rot) . turn(r)) * scale,   causal softmax
    y = W_o concat_h( sigmoid(W_g h)_h * sum_j p_j v_h,j )

Only c and turn(r) are cached, one row of kv_rank + rot_dim numbers per token for all heads
(pool 'latent'). The heads' keys and values are never formed: the query goes into the
latent's space, q'_h = W_uk,h^T q_unrot (a product per head), the attention kernel scores
q' and the rotated part against the cached rows and sums the latents, and the head's value
is W_uv,h applied to that sum (another product per head). The gate, one number per head and
row, scales the head's output in the attention kernel. `position` turns the first
`position.rot_dim` of the rot_dim rotated numbers (half-split pairs or neighbours, as its
`pairing` says) with its table and magnitude. Norm, angles, scores and softmax are 32-bit;
q' is kept in 32-bit. With `q_rank` the queries pass a latent of their own first:
c_q = rmsnorm(W_dq h) * weight (q_rank numbers, normed in 32-bit), q = W_uq c_q.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..registry import register_part
from ..weights.source import TensorSpec
from .base import CacheNeed, CallInfo, Mixer, Part, PoolSpec, PositionEncoding, StepContext, WeightBinder


class LatentAttention(Mixer):
    def __init__(self, prefix: str, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int,
                 kv_rank: int, scale: float, eps: float, position: PositionEncoding,
                 output_gate: bool = True, window: Optional[int] = None,
                 page_size: Optional[int] = None,
                 names=("q", "dkv", "dkv.norm", "uk", "uv", "g", "o"),
                 q_rank: Optional[int] = None, q_names=("dq", "dq.norm", "uq")):
        """`q_rank`: size of the queries' latent (None: none, `names[0]` projects the queries
        from the layer's input); `q_names`: what follows the prefix in the names of the down
        projection, its norm's weight and the up projection of the queries' latent."""
        if position.rot_dim > rot_dim:
            raise ValueError(f"the rotation turns {position.rot_dim} numbers of {rot_dim}")
        self.q_rank = q_rank
        self.q_names = tuple(q_names)
        self.w_dq: Optional[torch.Tensor] = None
        self.q_norm_w: Optional[torch.Tensor] = None
        if not scale > 0:
            raise ValueError(f"scale must be > 0, got {scale}")
        self.prefix = prefix
        self.hidden = hidden
        self.heads = heads
        self.dim = dim
        self.rot_dim = rot_dim
        self.vdim = vdim
        self.kv_rank = kv_rank
        self.scale = float(scale)
        self.eps = eps
        self.position = position
        self.output_gate = output_gate
        self.window = window
        self.page_size = page_size
        self.names = tuple(names)
        self.w_q: Optional[torch.Tensor] = None
        self.w_dkv_g: Optional[torch.Tensor] = None   # W_dkv, then W_g
        self.norm_w: Optional[torch.Tensor] = None
        self.w_absorb: Optional[torch.Tensor] = None  # [heads, kv_rank, dim]: W_uk,h transposed
        self.w_uv: Optional[torch.Tensor] = None      # [heads, vdim, kv_rank]
        self.w_o: Optional[torch.Tensor] = None

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed((PoolSpec("latent", (), (self.kv_rank + self.rot_dim,)),), self.window,
                         self.page_size)

    def children(self) -> List[Part]:
        return [self.position]

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        p, n = self.prefix, self.names
        qn = self.q_names
        specs = {
            p + n[1]: TensorSpec((self.kv_rank + self.rot_dim, self.hidden)),
            p + n[2]: TensorSpec((self.kv_rank,), "gain"),
            p + n[3]: TensorSpec((self.heads * self.dim, self.kv_rank)),
            p + n[4]: TensorSpec((self.heads * self.vdim, self.kv_rank)),
            p + n[6]: TensorSpec((self.hidden, self.heads * self.vdim)),
        }
        if self.output_gate:
            specs[p + n[5]] = TensorSpec((self.heads, self.hidden))
        q_width = self.heads * (self.dim + self.rot_dim)
        if self.q_rank is None:
            specs[p + n[0]] = TensorSpec((q_width, self.hidden))
        else:
            specs[p + qn[0]] = TensorSpec((self.q_rank, self.hidden))
            specs[p + qn[1]] = TensorSpec((self.q_rank,), "gain")
            specs[p + qn[2]] = TensorSpec((q_width, self.q_rank))
        return specs

    def bind(self, w: WeightBinder) -> None:
        p, n = self.prefix, self.names
        lat = self.kv_rank + self.rot_dim
        if self.q_rank is None:
            self.w_q = w.matrix(p + n[0])
        else:
            self.w_dq = w.matrix(p + self.q_names[0])
            self.q_norm_w = w.float32(p + self.q_names[1])
            self.w_q = w.matrix(p + self.q_names[2])
        self.w_dkv_g = torch.empty((lat + (self.heads if self.output_gate else 0), self.hidden),
                                   dtype=w.act_dtype, device=w.device)
        w.matrix_into(p + n[1], self.w_dkv_g[:lat])
        if self.output_gate:
            w.matrix_into(p + n[5], self.w_dkv_g[lat:])
        self.norm_w = w.float32(p + n[2])
        uk = w.matrix(p + n[3])
        # q'_h = W_uk,h^T q: as a product x w^T, w is W_uk,h transposed, [kv_rank, dim]
        self.w_absorb = uk.view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = w.matrix(p + n[4]).view(self.heads, self.vdim, self.kv_rank)
        self.w_o = w.matrix(p + n[6])

    def forward(self, ctx: StepContext, x, residual, call: CallInfo):
        ops = ctx.ops
        cache = call.cache
        T, H, R, rd = ctx.T, self.heads, self.kv_rank, self.rot_dim
        q = ctx.empty((T, H * (self.dim + rd)))
        if self.q_rank is None:
            ops.linear(x, self.w_q, q)
        else:   # the queries' latent: projected into 32-bit, normed there, then up
            cq32 = ctx.empty((T, self.q_rank), torch.float32)
            ops.linear(x, self.w_dq, cq32)
            cq = ctx.empty((T, self.q_rank))
            ops.rmsnorm(cq32, self.q_norm_w, self.eps, cq)
            ops.linear(cq, self.w_q, q)
        dkv_g = ctx.empty((T, self.w_dkv_g.shape[0]))
        ops.linear(x, self.w_dkv_g, dkv_g)
        q_abs = ctx.empty((T, H, R + rd), torch.float32)
        ops.latent_kv_write(dkv_g, q, q_abs, cache["latent"], cache.block_table, ctx, H, self.dim,
                            R, rd, self.norm_w, self.eps, self.position.table(),
                            self.position.rot_dim, getattr(self.position, "magnitude", 1.0),
                            cache.page_size, write_kv=call.writes_cache,
                            interleaved=self.position.pairing == "interleaved")
        ops.per_head_linear(q.view(T, H, self.dim + rd), self.w_absorb, q_abs, ctx, self.dim, R)
        mixed = ctx.empty((T, H * R))
        ops.latent_attention(q_abs, cache["latent"], cache.block_table, ctx, H, R, rd,
                             cache.page_size, self.scale, mixed,
                             gate=dkv_g[:, R + rd:] if self.output_gate else None,
                             window=self.window)
        heads_out = ctx.empty((T, H, self.vdim))
        ops.per_head_linear(mixed.view(T, H, R), self.w_uv, heads_out, ctx, R, self.vdim)
        out = ctx.empty((T, self.hidden))
        ops.linear(heads_out.view(T, H * self.vdim), self.w_o, out)
        return out


register_part("mixer", "latent_attention", LatentAttention)
