"""A plain PyTorch twin of every kernel of the HIP library, with the same call
signatures, computing in 32-bit with elementary torch operations.

Used two ways: on the GPU, each HIP kernel is compared with its twin here on
random inputs; on the CPU, the engine's host logic (batch building, cache
manager, block tables, plan, scheduler) is run end to end with these twins in
place of the kernels, which have no CPU form. Formula sources are the same
reference lines that tests/plain_model.py cites.
"""
from __future__ import annotations

import contextlib
import math

import torch


def _f(t):
    return t.to(torch.float32)


class PlainOps:
    force_generic = False

    def together(self):
        """Independent products: nothing to gain here, they run as they are called."""
        return contextlib.nullcontext()

    beside_min_rows = 8   # low, so that the host tests walk the many-row branch too

    def wants_beside(self, rows, weight_bytes=0):
        return rows >= self.beside_min_rows

    def beside(self):
        """Work for a second stream: here it simply runs where it is called."""
        return contextlib.nullcontext()

    def join(self):
        pass

    def fill_nan_pages(self, pool, pages):
        pool.index_fill_(0, pages.long(), float("nan"))

    def embed(self, tokens, table, out, positions=None, pos_table=None):
        x = _f(table[tokens.long()])
        if pos_table is not None:
            x = x + _f(pos_table[positions.long()])
        out.copy_(x)

    def rmsnorm(self, x, gain, eps, out, delta=None, rows=None, rows_sum=None, center=False):
        extra = None
        if delta is not None:
            extra = _f(delta)
        if rows_sum is not None:
            add = torch.zeros_like(x)
            self.moe_combine(add, rows_sum.y, rows_sum.weights, rows_sum.shared, rows_sum.gate)
            extra = add if extra is None else extra + add
        if rows is None:
            if extra is not None:
                x += extra
            v = x
        else:
            v = x[rows.long()]
            if extra is not None:
                v = v + extra[rows.long()]
        if center:
            v = v - v.mean(-1, keepdim=True)
        ms = (v * v).sum(-1, keepdim=True) / v.shape[-1]
        out.copy_((v * torch.rsqrt(ms + eps) * gain).to(out.dtype))

    def norm_add(self, residual, y, gain, eps, center=False, weights=None):
        v = _f(y)
        if weights is not None:
            t, k = weights.shape
            v = (v.view(t, k, -1) * weights[:, :, None]).sum(1)
        if center:
            v = v - v.mean(-1, keepdim=True)
        residual += v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * gain

    @staticmethod
    def _turn(x, positions, inv_freq, rot_dim, interleaved):
        """x [T, heads, d]: the first rot_dim numbers of every head turned by pos * inv_freq."""
        if not rot_dim:
            return x
        phi = positions.to(torch.float32)[:, None] * inv_freq[None, :]
        c, s = torch.cos(phi)[:, None, :], torch.sin(phi)[:, None, :]
        x = x.clone()
        if interleaved:
            a, b = x[..., 0:rot_dim:2].clone(), x[..., 1:rot_dim:2].clone()
            x[..., 0:rot_dim:2] = a * c - b * s
            x[..., 1:rot_dim:2] = b * c + a * s
        else:
            half = rot_dim // 2
            a, b = x[..., :half].clone(), x[..., half:rot_dim].clone()
            x[..., :half] = a * c - b * s
            x[..., half:rot_dim] = b * c + a * s
        return x

    def qkv_conv(self, u, w_conv, state, ctx, q_out, heads, kv_heads, dim, vdim, k_pool, v_pool,
                 block_table, page_size, q_norm=None, k_norm=None, norm_eps=0.0, inv_freq=None,
                 rot_dim=0, interleaved=False, w_conv_t=None):
        t, ch = u.shape
        y = _f(u).clone()
        if w_conv is not None:
            taps = w_conv.shape[1]
            start, slots = ctx.seq_row_start.tolist(), ctx.seq_slots.tolist()
            for s in range(ctx.S):
                rows = _f(u[start[s]:start[s + 1]])
                if taps > 1:
                    held = state[slots[s], :(taps - 1) * ch].view(taps - 1, ch)
                    ext = torch.cat([held, rows], 0)
                    state[slots[s], :(taps - 1) * ch] = ext[ext.shape[0] - (taps - 1):].reshape(-1)
                else:
                    ext = rows
                n = rows.shape[0]
                acc = torch.zeros_like(rows)
                for j in range(taps):
                    acc += w_conv[:, j][None, :] * ext[j:j + n]
                y[start[s]:start[s + 1]] = acc
        nq, nk = heads * dim, kv_heads * dim

        def normed(x, gain):
            if gain is None:
                return x
            return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + norm_eps) * gain
        q = self._turn(normed(y[:, :nq].view(t, heads, dim), q_norm), ctx.positions, inv_freq,
                       rot_dim, interleaved)
        q_out.copy_(q.reshape(t, nq).to(q_out.dtype))
        if not kv_heads:
            return
        k = self._turn(normed(y[:, nq:nq + nk].view(t, kv_heads, dim), k_norm), ctx.positions,
                       inv_freq, rot_dim, interleaved)
        v = y[:, nq + nk:].view(t, kv_heads, vdim)
        pos = ctx.positions.long()
        page = block_table[ctx.row_seq.long(), pos // page_size].long()
        assert (page >= 0).all(), "write into a page that is not held"
        k_pool[page, :, pos % page_size, :] = k.to(k_pool.dtype)
        v_pool[page, :, pos % page_size, :] = v.to(v_pool.dtype)

    def latent_kv_write(self, dkv, q, q_abs, pool, block_table, ctx, heads, dim, rank, rot_dim,
                        norm_w, eps, freq, rot_n, magnitude, page_size, write_kv=True,
                        interleaved=False):
        assert magnitude == 1.0, "the stand-in turns without a magnitude"
        t = ctx.T
        c = _f(dkv[:, :rank])
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w
        kr = self._turn(_f(dkv[:, rank:rank + rot_dim]).view(t, 1, rot_dim), ctx.positions, freq,
                        rot_n, interleaved)[:, 0]
        if write_kv:
            pos = ctx.positions.long()
            page = block_table[ctx.row_seq.long(), pos // page_size].long()
            assert (page >= 0).all(), "write into a page that is not held"
            pool[page, pos % page_size, :] = torch.cat([c, kr], -1).to(pool.dtype)
        qr = self._turn(_f(q).view(t, heads, dim + rot_dim)[:, :, dim:], ctx.positions, freq, rot_n,
                        interleaved)
        q_abs[:, :, rank:] = qr

    def head_index(self, ctx, heads):
        return None, None

    def per_head_linear(self, x, w, out, ctx, k, n):
        out[:, :, :n] = torch.einsum("thk,hnk->thn", _f(x[:, :, :k]), _f(w)).to(out.dtype)

    def latent_attention(self, q_abs, pool, block_table, ctx, heads, rank, rot_dim, page_size,
                         scale, out, gate=None, window=None):
        pos, seq = ctx.positions.tolist(), ctx.row_seq.tolist()
        for r in range(ctx.T):
            lo = max(0, pos[r] - window + 1) if window else 0
            js = torch.arange(lo, pos[r] + 1)
            pages = block_table[seq[r], js // page_size].long()
            assert (pages >= 0).all(), "read of a page that is not held"
            rows = _f(pool[pages, js % page_size, :])          # [n, rank + rot_dim]
            p = torch.softmax(rows @ q_abs[r].T * scale, 0)     # [n, heads]
            o = p.T @ rows[:, :rank]
            if gate is not None:
                o = o * torch.sigmoid(_f(gate[r]))[:, None]
            out[r] = o.reshape(-1).to(out.dtype)

    def qkv_rope(self, x, w_qkv, bias, qkv, positions, row_seq, inv_freq, rot_dim, n_q, n_kv,
                 head_dim, k_pool, v_pool, block_table, page_size, write_kv=True,
                 interleaved=False, q_norm=None, k_norm=None, norm_eps=0.0):
        self.linear(x, w_qkv, qkv)
        self.rope_kv_write(qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv, head_dim,
                           k_pool, v_pool, block_table, page_size, write_kv, interleaved,
                           q_norm, k_norm, norm_eps)

    def rope_kv_write(self, qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv, head_dim,
                      k_pool, v_pool, block_table, page_size, write_kv=True, interleaved=False,
                      q_norm=None, k_norm=None, norm_eps=0.0):
        t = qkv.shape[0]
        x = _f(qkv)
        if bias is not None:
            x = x + bias
        x = x.view(t, n_q + 2 * n_kv, head_dim).clone()
        if q_norm is not None:   # query and key heads normed over their dims before they turn
            for lo, hi, gain in ((0, n_q, q_norm), (n_q, n_q + n_kv, k_norm)):
                part = x[:, lo:hi]
                x[:, lo:hi] = part * torch.rsqrt((part * part).mean(-1, keepdim=True) + norm_eps) * gain
        if rot_dim:
            half = rot_dim // 2
            phi = positions.to(torch.float32)[:, None] * inv_freq[None, :]
            c, s = torch.cos(phi)[:, None, :], torch.sin(phi)[:, None, :]
            qk = x[:, :n_q + n_kv, :]
            if interleaved:   # pair i is dims (2i, 2i + 1)
                x1, x2 = qk[..., 0:rot_dim:2].clone(), qk[..., 1:rot_dim:2].clone()
                qk[..., 0:rot_dim:2] = x1 * c - x2 * s
                qk[..., 1:rot_dim:2] = x1 * s + x2 * c
            else:             # pair i is dims (i, i + rot_dim / 2)
                x1, x2 = qk[..., :half].clone(), qk[..., half:rot_dim].clone()
                qk[..., :half] = x1 * c - x2 * s
                qk[..., half:rot_dim] = x1 * s + x2 * c
        qkv.view(t, n_q + 2 * n_kv, head_dim)[:, :n_q] = x[:, :n_q].to(qkv.dtype)
        if not write_kv:
            return
        pos = positions.long()
        page = block_table[row_seq.long(), pos // page_size].long()
        assert (page >= 0).all(), "write into a page that is not held"
        slot = pos % page_size
        k_pool[page, :, slot, :] = x[:, n_q:n_q + n_kv].to(k_pool.dtype)
        v_pool[page, :, slot, :] = x[:, n_q + n_kv:].to(v_pool.dtype)

    def moe_combine(self, residual, y, wts, shared=None, gate=None):
        t, h = residual.shape
        k = wts.shape[1]
        acc = (_f(y).view(t, k, h) * wts[:, :, None]).sum(1)
        if shared is not None:
            g = torch.sigmoid(gate.reshape(t, 1)) if gate is not None else 1.0
            acc = acc + g * _f(shared)
        residual += acc

    def linear(self, x, w, out, bias=None, act=None):
        r = _f(x) @ _f(w).T
        if bias is not None:
            r = r + bias
        if act is not None:
            assert act == "relu2", act
            r = torch.relu(r) ** 2
        out.copy_(r.to(out.dtype))

    @staticmethod
    def _gated(g, u, act, limit=0.0, alpha=1.0):
        if act == "clamped_swish":
            g = torch.clamp(g, max=limit)
            return g / (1 + torch.exp(-alpha * g)) * (torch.clamp(u, -limit, limit) + 1)
        return PlainOps._act(g, act) * u

    @staticmethod
    def _act(g, act):
        if act == "silu":
            return g / (1 + torch.exp(-g))
        assert act == "gelu_pytorch_tanh", act
        return 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))

    def swiglu_linear(self, x, w_gate_up, out, act="silu", bias=None, limit=0.0, alpha=1.0):
        inner = w_gate_up.shape[0] // 2
        g = _f(x) @ _f(w_gate_up[:inner]).T
        u = _f(x) @ _f(w_gate_up[inner:]).T
        if bias is not None:
            g, u = g + bias[:inner], u + bias[inner:]
        out.copy_(self._gated(g, u, act, limit, alpha).to(out.dtype))

    def grouped_swiglu(self, x, w_gate_up, offsets, order, top_k, out, tiles=None, act="silu",
                       limit=0.0, alpha=1.0):
        e, two_i, _ = w_gate_up.shape
        inner = two_i // 2
        off = offsets.tolist()
        for g in range(e):
            rows = order[off[g]:off[g + 1]].long()
            if rows.numel() == 0:
                continue
            xs = _f(x[rows // top_k])
            gg = xs @ _f(w_gate_up[g, :inner]).T
            uu = xs @ _f(w_gate_up[g, inner:]).T
            out[off[g]:off[g + 1]] = self._gated(gg, uu, act, limit, alpha).to(out.dtype)

    def grouped_down(self, h, w_down, offsets, order, out, tiles=None):
        e = w_down.shape[0]
        off = offsets.tolist()
        for g in range(e):
            rows = order[off[g]:off[g + 1]].long()
            if rows.numel() == 0:
                continue
            out[rows] = (_f(h[off[g]:off[g + 1]]) @ _f(w_down[g]).T).to(out.dtype)

    def router_topk(self, logits, experts, top_k, renorm, ids, wts, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0, group_top=1,
                    renorm_eps=0.0):
        l = logits[:, :experts]
        if score == "sigmoid":
            p = 1 / (1 + torch.exp(-l))
        else:
            p = torch.exp(l - l.max(-1, keepdim=True).values)
            p = p / p.sum(-1, keepdim=True)
        work = p.clone() if choice_bias is None else p + choice_bias[None, :]
        rows = torch.arange(work.shape[0])
        if n_group > 1 and topk_group < n_group:
            # group-limited: the groups by their best score, a stable sort (ties: lower group)
            per = experts // n_group
            # (a group's score: its best, or the sum of its group_top best)
            best_of = work.view(-1, n_group, per).topk(max(1, group_top), -1).values.sum(-1)
            keep = torch.sort(best_of, dim=-1, descending=True, stable=True).indices[:, :topk_group]
            is_open = torch.zeros_like(best_of, dtype=torch.bool)
            is_open.scatter_(1, keep, True)
            work = work.masked_fill(~is_open.repeat_interleave(per, dim=1), -float("inf"))
        for j in range(top_k):
            best = work.max(-1).values
            # lowest index among the maxima
            idx = torch.argmax((work == best[:, None]).to(torch.int32), dim=-1)
            ids[:, j] = idx.to(torch.int32)
            wts[:, j] = p[rows, idx]
            work[rows, idx] = -float("inf")
        if renorm:
            wts /= wts.sum(-1, keepdim=True) + renorm_eps
        wts *= scale

    def moe_align(self, ids, experts, offsets, order, tiles=None, weightless=0):
        flat = ids.reshape(-1).long()
        counts = torch.bincount(flat, minlength=experts)
        offsets[0] = 0
        offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
        order.copy_(torch.sort(flat, stable=True).indices.to(torch.int32))
        if tiles is not None and tiles.tiles16 is not None:
            off = offsets.tolist()
            for size, out in ((16, tiles.tiles16), (256, tiles.tiles_big)):
                lst = [[e, r, off[e + 1], 0] for e in range(experts - weightless)
                       for r in range(off[e], off[e + 1], size)]
                if lst:
                    out[:len(lst)] = torch.tensor(lst, dtype=torch.int32, device=out.device)
                tiles.tile_counts[0 if size == 16 else 1] = len(lst)

    def moe_route(self, logits, experts, top_k, renorm, r, score="softmax", choice_bias=None,
                  scale=1.0, n_group=0, topk_group=0, group_top=1, renorm_eps=0.0, weightless=0):
        self.router_topk(logits, experts, top_k, renorm, r.ids, r.weights, score, choice_bias,
                         scale, n_group, topk_group, group_top, renorm_eps)
        self.moe_align(r.ids, experts, r.offsets, r.order, tiles=r, weightless=weightless)

    def paged_attention(self, qkv, k_pool, v_pool, block_table, ctx, n_q, n_kv, head_dim,
                        page_size, window, scale, out, slopes=None, vdim=None, sink=False):
        t = qkv.shape[0]
        vdim = head_dim if vdim is None else vdim
        q = _f(qkv[:, :n_q * head_dim]).view(t, n_q, head_dim)
        group = n_q // n_kv
        pos = ctx.positions.tolist()
        seq = ctx.row_seq.tolist()
        for r in range(t):
            lo = max(0, pos[r] - window + 1) if window else 0
            js = torch.arange(lo, pos[r] + 1)
            pages = block_table[seq[r], js // page_size].long()
            assert (pages >= 0).all(), "read of a page that is not held"
            k = _f(k_pool[pages, :, js % page_size, :])  # [n, n_kv, D]
            v = _f(v_pool[pages, :, js % page_size, :])
            for h in range(n_q):
                g = h // group
                s = (k[:, g, :] @ q[r, h]) * scale
                if slopes is not None:
                    s = s + float(slopes[h]) * (js - pos[r]).float().to(s.device)
                top = torch.clamp(s.max(), min=0.0) if sink else s.max()
                p = torch.exp(s - top)
                p = p / (p.sum() + (torch.exp(-top) if sink else 0.0))
                out[r, h * vdim:(h + 1) * vdim] = (p @ v[:, g, :]).to(out.dtype)

    # ---- parallel sublayers, hashed pairs, differential attention ------------------------------
    def embed_pairs(self, ctx, table, out, scale=1.0, pair_table=None, buckets=0, mul_prev=0,
                    mul_cur=0, state=None):
        toks = ctx.tokens.tolist()
        x = _f(table[ctx.tokens.long()]) * scale
        if pair_table is not None:
            start, slots = ctx.seq_row_start.tolist(), ctx.seq_slots.tolist()
            held = state.view(torch.int32)
            for s in range(ctx.S):
                prev = int(held[slots[s], 0]) - 1
                for t in range(start[s], start[s + 1]):
                    row = buckets if prev < 0 else (prev * mul_prev + toks[t] * mul_cur) % buckets
                    x[t] += _f(pair_table[row])
                    prev = toks[t]
                held[slots[s], 0] = prev + 1
        out.copy_(x)

    def concat_rows(self, a, b, out):
        out.copy_(torch.cat([a, b], -1).to(out.dtype))

    def scaled_sum_add(self, residual, a, s1, f, s2):
        if a is not None:
            residual += _f(a) * (s1 if s1 is not None else 1.0)
        if f is None:
            return
        if hasattr(f, "weights"):
            add = torch.zeros_like(residual)
            self.moe_combine(add, f.y, f.weights, f.shared, f.gate)
        else:
            add = _f(f)
        residual += add * (s2 if s2 is not None else 1.0)

    def gated_sum_add(self, residual, a, g1, b1, f, g2, b2, mult=1.0):
        def gate(g, b):
            if g is None:
                return 1.0
            return torch.sigmoid(_f(g) + (b if b is not None else 0.0))
        total = torch.zeros_like(residual)
        if a is not None:
            total += _f(a) * gate(g1, b1)
        if f is not None and hasattr(f, "weights"):
            t, h = residual.shape
            k = f.weights.shape[1]
            y = _f(f.y).view(t, k, h)
            if getattr(f, "ids", None) is not None:
                back = (f.ids >= f.real)[:, :, None]
                y = torch.where(back, _f(f.rows)[:, None, :].expand(t, k, h), y)
            total += (y * f.weights[:, :, None]).sum(1) * gate(g2, b2)
        elif f is not None:
            total += _f(f) * gate(g2, b2)
        residual += mult * total

    def gated_rmsnorm(self, o, gate, weight, eps, out, group=0, gate_act="sigmoid"):
        t, n = o.shape
        g = group or n
        x = o.view(t, n // g, g)
        x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * weight
        z = _f(gate)
        f = torch.sigmoid(z) * (z if gate_act == "silu" else 1.0)
        out.copy_((x.reshape(t, n) * f).to(out.dtype))

    def gla_work_floats(self, qkv_dtype, ctx, heads, dim):
        return 0

    def gated_linear_attention(self, qkv, q_off, k_off, v_off, z, heads, dim, vdim, tau, q_scale,
                               state, ctx, out, work=None):
        starts, slots = ctx.seq_row_start.tolist(), ctx.seq_slots.tolist()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(-1, heads, dim)
        for s, slot in enumerate(slots):
            st = state[slot, :heads * dim * vdim].view(heads, dim, vdim)
            for r in range(starts[s], starts[s + 1]):
                q = _f(qkv[r, q_off:q_off + heads * dim]).view(heads, dim) * q_scale
                k = _f(qkv[r, k_off:k_off + heads * dim]).view(heads, dim)
                v = _f(qkv[r, v_off:v_off + heads * vdim]).view(heads, vdim)
                st.copy_(alpha[r][:, :, None] * st + k[:, :, None] * v[:, None, :])
                out[r] = torch.einsum("hd,hdv->hv", q, st).reshape(-1)

    def sigmoid_attention(self, qkv, k_pool, v_pool, block_table, ctx, heads, kv_heads, dim, vdim,
                          page_size, scale, chunk, head_bias, mix, out, write_kv=True):
        t = qkv.shape[0]
        nq, nk = heads * dim, kv_heads * dim
        pos, seq = ctx.positions.tolist(), ctx.row_seq.tolist()
        if write_kv:
            for r in range(t):
                page = int(block_table[seq[r], pos[r] // page_size])
                assert page >= 0, "write into a page that is not held"
                k_pool[page, :, pos[r] % page_size] = qkv[r, nq:nq + nk].view(kv_heads, dim)
                v_pool[page, :, pos[r] % page_size] = qkv[r, nq + nk:].view(kv_heads, vdim)
        q = _f(qkv[:, :nq]).view(t, heads, dim)
        per = heads // kv_heads
        for r in range(t):
            first = pos[r] // chunk * chunk if chunk else 0
            js = torch.arange(first, pos[r] + 1)
            pages = block_table[seq[r], js // page_size].long()
            assert (pages >= 0).all(), "read of a page that is not held"
            k = _f(k_pool[pages, :, js % page_size])      # [n, kv_heads, dim]
            v = _f(v_pool[pages, :, js % page_size])
            w = torch.stack([k[:, h // per] @ q[r, h] for h in range(heads)]) * scale
            if head_bias is not None:
                w = w + head_bias[:, None]
            w = torch.sigmoid(w)
            if mix is not None:
                w = mix @ w
            for h in range(heads):
                out[r, h * vdim:(h + 1) * vdim] = (w[h] @ v[:, h // per]).to(out.dtype)

    def tanh_cap(self, x, cap):
        x.copy_(cap * torch.tanh(x / cap))

    def relu_square(self, x):
        x.copy_((torch.relu(_f(x)) ** 2).to(x.dtype))

    def diff_attention(self, qkv, k_pool, v_pool, block_table, ctx, heads, kv_heads, dim, vdim,
                       page_size, scale, cap, temp_coef, temp_every, lam, eps, out_scale, out,
                       write_kv=True):
        t = qkv.shape[0]
        nq, nk = heads * 2 * dim, kv_heads * 2 * dim
        pos, seq = ctx.positions.tolist(), ctx.row_seq.tolist()
        if write_kv:
            for r in range(t):
                page = int(block_table[seq[r], pos[r] // page_size])
                assert page >= 0, "write into a page that is not held"
                k_pool[page, :, pos[r] % page_size] = qkv[r, nq:nq + nk].view(kv_heads, 2 * dim)
                v_pool[page, :, pos[r] % page_size] = qkv[r, nq + nk:].view(kv_heads, vdim)
        q = _f(qkv[:, :nq]).view(t, heads, 2, dim)
        for r in range(t):
            js = torch.arange(0, pos[r] + 1)
            pages = block_table[seq[r], js // page_size].long()
            assert (pages >= 0).all(), "read of a page that is not held"
            k = _f(k_pool[pages, :, js % page_size]).view(-1, kv_heads, 2, dim)
            v = _f(v_pool[pages, :, js % page_size])
            temp = 1.0 + temp_coef * math.log((pos[r] + 1) // temp_every + 1) if temp_coef else 1.0
            for h in range(heads):
                g = h // (heads // kv_heads)
                maps = []
                for i in range(2):
                    s = (k[:, g, i] @ q[r, h, i]) * (scale * temp)
                    if cap > 0:
                        s = cap * torch.tanh(s / cap)
                    p = torch.exp(s - s.max())
                    maps.append((p / p.sum()) @ v[:, g])
                o = maps[0] - lam * maps[1]
                if eps >= 0:
                    o = o / torch.sqrt((o * o).mean() + eps)
                out[r, h * vdim:(h + 1) * vdim] = (o * out_scale).to(out.dtype)

    def sample(self, logits, temperature, uniform, out, top_k=None, top_p=None, rep_penalty=None,
               pen_tokens=None, pen_counts=None, pen_offsets=None):
        from plain_model import sample_distribution
        r, v = logits.shape
        for i in range(r):
            recent = []
            if pen_offsets is not None:
                for e in range(int(pen_offsets[i]), int(pen_offsets[i + 1])):
                    recent += [int(pen_tokens[e])] * int(pen_counts[e])
            p = sample_distribution(
                logits[i].cpu(), float(temperature[i]), int(top_k[i]) if top_k is not None else 0,
                float(top_p[i]) if top_p is not None else 1.0,
                float(rep_penalty[i]) if rep_penalty is not None else 1.0, recent)
            cdf = torch.cumsum(p.double(), 0)
            idx = int(torch.searchsorted(cdf, torch.tensor(float(uniform[i]) * float(cdf[-1]),
                                                           dtype=torch.float64), right=True))
            out[i] = min(idx, v - 1)
