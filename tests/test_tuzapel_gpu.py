"""Tuzapel on the GPU against the plain implementation: every mechanism alone through its
kernel, then whole models (three small configurations, in 32-bit and in bfloat16) layer by
layer, whole, decoded token by token, in portions down to two tokens, in mixed batches with
pages and state slots that are given back and used again, from a captured graph, generated
greedily through the scheduler, through the trace replay program, and configurations drawn at
random. bfloat16 is compared with the plain implementation on the bfloat16-rounded weights.
Prompts are chosen so that no routing decision of the plain implementation is a close call."""
import json
import math
import os
import random
import subprocess
import sys

import pytest
import torch

import plain_tuzapel as plain
import tuzapel_cases
import util

pytestmark = pytest.mark.gpu
DEV = "cuda"
STD = 0.25
D = torch.float64


@pytest.fixture(scope="module")
def ops():
    from ninfer_amd.kernels import load_ops
    return load_ops()


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def _cut(n, sizes, tail):
    """n rows as portions of the given sizes in turn, the last `tail` one by one."""
    out, i, j = [], 0, 0
    while i < n - tail:
        s = min(sizes[j % len(sizes)], n - tail - i)
        out.append(s)
        i += s
        j += 1
    return out + [1] * tail


def _steps(ops, dtype, cuts, slots):
    """StepContexts for requests that go on from step to step; cuts[r]: request r's portions.
    Requests that bring one row come first in a step, as the engine orders them."""
    done = [0] * len(cuts)
    for i in range(max(len(c) for c in cuts)):
        who = [r for r, c in enumerate(cuts) if i < len(c)]
        who.sort(key=lambda r: cuts[r][i] != 1)
        ctx = util.make_context(ops, dtype, [(done[r], cuts[r][i]) for r in who])
        ctx.seq_slots = torch.tensor([slots[r] for r in who], dtype=torch.int32, device=DEV)
        ctx.single_rows = sum(1 for r in who if cuts[r][i] == 1)
        yield ctx, who, [done[r] for r in who], [cuts[r][i] for r in who]
        for r in who:
            done[r] += cuts[r][i]


# ---- mechanisms alone ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 256, 1100, 5000])
def test_layer_norms(ops, dtype, width):
    """The norm in front of a sublayer (of the residual, of the residual plus rows, of chosen
    rows) and the norm behind it (of plain rows and of a weighted sum of an expert's rows),
    with a mean that is far from zero."""
    g = torch.Generator().manual_seed(width)
    t, k = 19, 3
    x = torch.randn(t, width, generator=g) * 2 + 3
    delta = (torch.randn(t, width, generator=g) + 1).to(dtype)
    gain = 1 + 0.3 * torch.randn(width, generator=g)
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    out = torch.empty(t, width, dtype=dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), gain.to(DEV), 1e-5, out, center=True)
    assert rel_err(out, plain.layer_norm(x.double(), gain, 1e-5)) < tol
    xs = x.to(DEV)
    ops.rmsnorm(xs, gain.to(DEV), 1e-5, out, delta=delta.to(DEV), center=True)
    assert rel_err(out, plain.layer_norm(x.double() + delta.double(), gain, 1e-5)) < tol
    assert rel_err(xs, x.double() + delta.double()) < 1e-6     # the sum is kept, uncentred
    rows = torch.tensor([4, 0, 18], dtype=torch.int32, device=DEV)
    few = torch.empty(3, width, dtype=dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), gain.to(DEV), 1e-5, few, rows=rows, center=True)
    assert rel_err(few, plain.layer_norm(x.double()[[4, 0, 18]], gain, 1e-5)) < tol
    # behind a sublayer: residual += ln(y) gain
    y = (torch.randn(t, width, generator=g) * 0.5 - 2).to(dtype)
    res = x.clone().to(DEV)
    ops.norm_add(res, y.to(DEV), gain.to(DEV), 1e-5, center=True)
    assert rel_err(res, x.double() + plain.layer_norm(y.double(), gain, 1e-5)) < 2e-6
    ys = (torch.randn(t * k, width, generator=g) + 0.5).to(dtype)
    wts = torch.rand(t, k, generator=g)
    want = (ys.double().view(t, k, width) * wts.double()[:, :, None]).sum(1)
    res = x.clone().to(DEV)
    ops.norm_add(res, ys.to(DEV), gain.to(DEV), 1e-5, center=True, weights=wts.to(DEV))
    assert rel_err(res, x.double() + plain.layer_norm(want, gain, 1e-5)) < 2e-6
    res = x.clone().to(DEV)     # and without the mean taken off, as other designs use it
    ops.norm_add(res, y.to(DEV), gain.to(DEV), 1e-5)
    assert rel_err(res, x.double() + plain.rms_norm(y.double(), gain, 1e-5)) < 2e-6


def _gather(pool, table, n, page_size):
    """Rows 0 .. n - 1 of a request from its pages: [n, heads, numbers]."""
    js = torch.arange(n)
    pages = table[js // page_size].long()
    return pool[pages, :, js % page_size, :]


@pytest.mark.parametrize("dtype,plain_kernel", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("heads,kv,dim,vdim,taps,rot,pairing", [
    (6, 3, 20, 12, 4, 10, "half"), (4, 2, 64, 32, 3, 64, "half"), (2, 1, 88, 72, 2, 40, "interleaved"),
    (3, 0, 24, 8, 5, 24, "half"), (2, 2, 16, 16, 1, 0, "half"), (1, 1, 8, 40, 0, 8, "half"),
    (16, 4, 128, 128, 4, 64, "half")])
def test_projected_rows_on_their_way_to_attention(ops, dtype, plain_kernel, heads, kv, dim, vdim, taps, rot, pairing):
    """Convolution, head norms, rotation and the cache write in one kernel (a wave per head, or
    for bfloat16 heads of whole pieces of 8 a thread per piece): three requests in slots 2, 0
    and 3 of a wider state tensor, cut into portions down to two rows and single rows (the
    taps - 1 rows before a portion come from the state), against the plain convolution of the
    whole request followed by norm and rotation. kv 0: queries only."""
    ops.force_generic = plain_kernel
    ops.conv_pieces_always = not plain_kernel     # (the steps here have few rows)
    try:
        _projected_rows(ops, dtype, heads, kv, dim, vdim, taps, rot, pairing)
    finally:
        ops.force_generic = False
        ops.conv_pieces_always = False


def _projected_rows(ops, dtype, heads, kv, dim, vdim, taps, rot, pairing):
    g = torch.Generator().manual_seed(dim + taps)
    lens, ps, eps = [45, 7, 30], 8, 1e-5
    ch = heads * dim + kv * (dim + vdim)
    rows = [torch.randn(n, ch, generator=g).to(dtype) for n in lens]
    w_conv = (torch.randn(ch, taps, generator=g) * 0.6) if taps else None
    qn, kn = 1 + 0.3 * torch.randn(dim, generator=g), 1 + 0.3 * torch.randn(dim, generator=g)
    rot_cfg = {"base": 300.0, "dims": rot, "scaling": {"factor": 2.0, "low": 1.0, "high": 8.0, "original": 40}}
    freq = plain.frequencies(rot_cfg).float().to(DEV) if rot else None
    floats = max(taps - 1, 0) * ch
    state = torch.full((4, floats + 9), 7.0, device=DEV)
    state[:, 4:4 + floats] = 0
    view = state[:, 4:4 + floats] if floats else None
    n_pages = sum(-(-n // ps) for n in lens)
    perm = torch.randperm(n_pages, generator=g).tolist()
    tables = []
    for n in lens:
        tables.append([perm.pop() for _ in range(-(-n // ps))])
    width = max(len(t) for t in tables)
    k_pool = torch.zeros(n_pages, max(kv, 1), ps, dim, dtype=dtype, device=DEV)
    v_pool = torch.zeros(n_pages, max(kv, 1), ps, vdim, dtype=dtype, device=DEV)
    got_q = [torch.zeros(n, heads * dim) for n in lens]
    cuts = [_cut(45, [13, 2, 9, 3], 6), _cut(7, [3, 2], 2), _cut(30, [2, 11, 1, 8], 4)]
    for ctx, who, starts, counts in _steps(ops, dtype, cuts, [2, 0, 3]):
        u = torch.cat([rows[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
        bt = torch.tensor([tables[r] + [-1] * (width - len(tables[r])) for r in who], dtype=torch.int32, device=DEV)
        q = torch.empty(ctx.T, heads * dim, dtype=dtype, device=DEV)
        ops.qkv_conv(u, w_conv.to(DEV) if taps else None, view, ctx, q, heads, kv, dim, vdim, k_pool, v_pool, bt,
                     ps, q_norm=qn.to(DEV), k_norm=kn.to(DEV) if kv else None, norm_eps=eps, inv_freq=freq,
                     rot_dim=rot, interleaved=pairing == "interleaved",
                     w_conv_t=w_conv.t().contiguous().to(DEV) if taps else None)
        o = 0
        for r, s, n in zip(who, starts, counts):
            got_q[r][s:s + n] = q[o:o + n].float().cpu()
            o += n
    tol = 3e-6 if dtype == torch.float32 else 6e-3
    for r, n in enumerate(lens):
        y = plain.short_conv(rows[r].double(), w_conv) if taps else rows[r].double()
        pos = torch.arange(n)
        q = plain.rotate(plain.rms_norm(y[:, :heads * dim].reshape(n, heads, dim), qn, eps), pos, rot_cfg, pairing)
        assert rel_err(got_q[r], q.reshape(n, -1)) < tol
        if kv:
            nk = heads * dim
            k = plain.rotate(plain.rms_norm(y[:, nk:nk + kv * dim].reshape(n, kv, dim), kn, eps), pos, rot_cfg, pairing)
            table = torch.tensor(tables[r])
            assert rel_err(_gather(k_pool.cpu(), table, n, ps), k) < tol
            assert rel_err(_gather(v_pool.cpu(), table, n, ps), y[:, nk + kv * dim:].reshape(n, kv, vdim)) < tol
    if floats:
        assert (state[:, :4] == 7).all() and (state[:, 4 + floats:] == 7).all() and (state[1, 4:4 + floats] == 0).all()
        last = rows[0][45 - (taps - 1):].float().reshape(-1)
        assert torch.equal(state[2, 4:4 + floats].cpu(), last)


def _dense_attention(q, k, v, heads, kv, window, sink, scale, first):
    """q [n_q, heads, d] for positions first .. of a request whose keys k [n, kv, d] and values
    v [n, kv, dv] are all there: the plain softmax, row by row."""
    n_q, n = q.shape[0], k.shape[0]
    vis = plain.visible(n, window)[first:first + n_q]
    per = heads // kv
    out = torch.zeros(n_q, heads, v.shape[-1], dtype=D)
    for a in range(heads):
        s = q[:, a].double() @ k[:, a // per].double().T * scale
        out[:, a] = plain.softmax_rows(s, vis, sink) @ v[:, a // per].double()
    return out


class _Cached:
    """Keys and values of a few requests laid into shuffled pages."""

    def __init__(self, lens, kv, dim, vdim, ps, dtype, g, spare=3):
        self.ps, self.lens = ps, lens
        n_pages = sum(-(-n // ps) for n in lens) + spare
        perm = torch.randperm(n_pages, generator=g).tolist()
        self.k = [torch.randn(n, kv, dim, generator=g).to(dtype) for n in lens]
        self.v = [torch.randn(n, kv, vdim, generator=g).to(dtype) for n in lens]
        self.tables = [[perm.pop() for _ in range(-(-n // ps))] for n in lens]
        self.k_pool = torch.full((n_pages, kv, ps, dim), float("nan"), dtype=dtype)
        self.v_pool = torch.full((n_pages, kv, ps, vdim), float("nan"), dtype=dtype)

    def lay(self):
        for r, n in enumerate(self.lens):
            js = torch.arange(n)
            pages = torch.tensor(self.tables[r])[js // self.ps]
            self.k_pool[pages, :, js % self.ps] = self.k[r]
            self.v_pool[pages, :, js % self.ps] = self.v[r]
        return self.k_pool.to(DEV), self.v_pool.to(DEV)

    def table(self, who, lo=None):
        """Block table rows of the requests `who`; with `lo` the pages wholly before position
        lo[i] are given as -1, as a window's cache gives them back."""
        width = max(len(t) for t in self.tables)
        rows = []
        for i, r in enumerate(who):
            t = list(self.tables[r]) + [-1] * (width - len(self.tables[r]))
            if lo is not None:
                for p in range(max(lo[i], 0) // self.ps):
                    t[p] = -1
            rows.append(t)
        return torch.tensor(rows, dtype=torch.int32, device=DEV)


SHAPES = [  # heads, kv, dim, vdim, window, page
    (6, 3, 20, 12, 10, 4), (8, 2, 64, 32, 32, 16), (4, 4, 32, 96, 48, 8), (6, 2, 88, 72, 52, 16),
    (16, 2, 64, 32, 16, 16), (3, 1, 128, 128, 70, 32), (2, 2, 8, 24, None, 8), (5, 5, 40, 8, 1, 2),
    (40, 1, 16, 16, 9, 4)]


@pytest.mark.parametrize("dtype,plain_kernel", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("sink", [True, False])
@pytest.mark.parametrize("heads,kv,dim,vdim,window,ps", SHAPES)
def test_attention_with_window_sink_and_value_size(ops, dtype, plain_kernel, sink, heads, kv, dim, vdim, window, ps):
    """Three requests: whole prompts in one step, then a step that mixes single rows with a
    portion, then single rows alone (the kernels for prompt tiles and for single rows, and the
    plain kernel), pages before the window given back; against the plain softmax."""
    g = torch.Generator().manual_seed(heads * dim + (window or 0))
    lens = [150, 37, 70]
    c = _Cached(lens, kv, dim, vdim, ps, dtype, g)
    k_pool, v_pool = c.lay()
    q = [torch.randn(n, heads, dim, generator=g).to(dtype) for n in lens]
    scale = 0.9 / math.sqrt(dim)
    want = [_dense_attention(q[r], c.k[r], c.v[r], heads, kv, window, sink, scale, 0) for r in range(3)]
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    ops.force_generic = plain_kernel
    try:
        # (request, first row, rows) of every step; single rows first
        for step in ([(0, 0, 150), (1, 0, 37), (2, 0, 70)], [(1, 36, 1), (2, 69, 1), (0, 97, 53)],
                     [(0, 149, 1), (1, 20, 1), (2, 64, 1)], [(2, 3, 2), (0, 60, 33)]):
            ctx = util.make_context(ops, dtype, [(s, n) for _, s, n in step])
            ctx.single_rows = sum(1 for _, _, n in step if n == 1) if step[0][2] == 1 else 0
            who = [r for r, _, _ in step]
            bt = c.table(who, lo=[s - window + 1 for _, s, _ in step] if window else None)
            rows = torch.cat([q[r][s:s + n] for r, s, n in step]).reshape(ctx.T, heads * dim).to(DEV)
            out = torch.full((ctx.T, heads * vdim), float("nan"), dtype=dtype, device=DEV)
            ops.paged_attention(rows, k_pool, v_pool, bt, ctx, heads, kv, dim, ps, window, scale, out,
                                vdim=vdim, sink=sink)
            ref = torch.cat([want[r][s:s + n] for r, s, n in step]).reshape(ctx.T, -1)
            assert torch.isfinite(out).all()
            assert rel_err(out, ref) < tol, step
    finally:
        ops.force_generic = False


@pytest.mark.parametrize("dtype,plain_kernel", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("window,ps", [(44, 16), (64, 16), (17, 8), (1, 4), (None, 16)])
def test_one_loud_key_at_the_windows_edges(ops, dtype, plain_kernel, window, ps):
    """Among hundreds of quiet keys one key whose score stands out, with a value no other key
    has: just inside the window (the row's output is that value), just outside (nothing of
    it), at a page's border, at a tile's border, and far back when there is no window; for a
    row inside a prompt portion and for a row decoded alone. With a sink and quiet keys only,
    the output is close to nothing."""
    heads, kv, dim, vdim, n = 4, 2, 32, 16, 300
    g = torch.Generator().manual_seed(7)
    rows = [299, 256, 255, 191, 130, 64] + ([48] if (window or 99) <= 44 else [])
    dist_in = (window - 1) if window else None
    for row in rows:
        far = [row - dist_in] if window else [0, 3, row - row % ps, row - 64 - row % 64]
        for j, seen in [(x, True) for x in far] + ([(row - window, False)] if window and row >= window else []):
            if j < 0:
                continue
            c = _Cached([n], kv, dim, vdim, ps, dtype, g)
            c.k[0] *= 0.05
            c.v[0] *= 0.1
            c.k[0][j, :, 0] = 30.0
            c.v[0][j] = 5.0
            q = (torch.randn(n, heads, dim, generator=g) * 0.05).to(dtype)
            q[row, :, 0] = 30.0
            k_pool, v_pool = c.lay()
            ops.force_generic = plain_kernel
            try:
                for first, count in ((row - min(row, 37), min(row, 37) + 1), (row, 1)):
                    ctx = util.make_context(ops, dtype, [(first, count)])
                    ctx.single_rows = 1 if count == 1 else 0
                    bt = c.table([0], lo=[first - window + 1] if window else None)
                    out = torch.empty(count, heads * vdim, dtype=dtype, device=DEV)
                    ops.paged_attention(q[first:first + count].reshape(count, -1).to(DEV), k_pool, v_pool, bt, ctx,
                                        heads, kv, dim, ps, window, 0.2, out, vdim=vdim, sink=True)
                    last = out[-1].float().cpu()
                    if seen:
                        assert (last - 5.0).abs().max() < 0.05, (row, j, count)
                    else:
                        assert last.abs().max() < 0.2, (row, j, count)
            finally:
                ops.force_generic = False


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_rows_turn_in_neighbouring_pairs(ops, dtype):
    """The cache write of latent attention with pairs (2i, 2i + 1): the normed latent and the
    turned shared key part in the page, the turned part of every query head behind its latent."""
    g = torch.Generator().manual_seed(3)
    heads, dim, rank, rd, ps, eps = 3, 12, 40, 6, 4, 1e-5
    seqs = [(5, 9), (0, 3)]
    ctx = util.make_context(ops, dtype, seqs)
    dkv = torch.randn(ctx.T, rank + rd + 5, generator=g).to(dtype)
    q = torch.randn(ctx.T, heads * (dim + rd), generator=g).to(dtype)
    nw = 1 + 0.3 * torch.randn(rank, generator=g)
    rot = {"base": 50.0, "dims": rd}
    pool = torch.zeros(8, ps, rank + rd, dtype=dtype, device=DEV)
    bt = torch.tensor([[6, 2, 5, 0], [3, -1, -1, -1]], dtype=torch.int32, device=DEV)
    q_abs = torch.zeros(ctx.T, heads, rank + rd, device=DEV)
    ops.latent_kv_write(dkv.to(DEV)[:, :rank + rd + 5], q.to(DEV), q_abs, pool, bt, ctx, heads, dim, rank, rd,
                        nw.to(DEV), eps, plain.frequencies(rot).float().to(DEV), rd, 1.0, ps, interleaved=True)
    pos = ctx.positions.cpu()
    tol = 3e-6 if dtype == torch.float32 else 6e-3
    want_q = plain.rotate(q.double().view(ctx.T, heads, dim + rd)[..., dim:], pos, rot, "interleaved")
    assert rel_err(q_abs[..., rank:], want_q) < 3e-6
    want_c = plain.rms_norm(dkv.double()[:, :rank], nw, eps)
    want_r = plain.rotate(dkv.double()[:, None, rank:rank + rd], pos, rot, "interleaved")[:, 0]
    table = bt.cpu()
    for t in range(ctx.T):
        s = 0 if t < 9 else 1
        row = pool[table[s, int(pos[t]) // ps], int(pos[t]) % ps].cpu()
        assert rel_err(row[:rank], want_c[t]) < tol and rel_err(row[rank:], want_r[t]) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 20, 70, 300])
def test_feed_forwards(ops, dtype, rows):
    """The clamped gated product, dense and as routed experts whose logits carry a bias and
    whose weights are the softmax over the chosen logits, at every row count (few-row, tile
    and plain product kernels) against the plain feed-forward."""
    from ninfer_amd.parts import SparseMoE, SwiGLU, WeightBinder
    hidden, inner, experts, top = 128, 64, 7, 3
    g = torch.Generator().manual_seed(rows)
    moe = SparseMoE("m.", hidden, experts, top, inner, renorm=True, act="clamped_swish", act_limit=0.8,
                    act_alpha=1.702, router={"logit_bias_leaf": "router.b"},
                    names={"router": "", "router_leaf": "router", "experts": "e", "expert_leaves": ("gate", "up", "down")})
    dense = SwiGLU("d.", hidden, inner, act="clamped_swish", act_limit=0.8, act_alpha=1.702, names=("gate", "up", "down"))
    w = {}
    for part, seed in ((moe, 5), (dense, 6)):
        w.update({k: v.to(dtype).float() for k, v in util.random_part_weights(part, seed, std=0.3).items()})
    w["m.router.b"] = torch.tensor([0.0, -9.0, 0.5, 0.0, -0.5, 0.0, 9.0])     # a bias that decides choices
    binder = WeightBinder(util.DictSource(w), torch.device(DEV), dtype)
    moe.bind_all(binder)
    dense.bind_all(binder)
    mlp = {"kind": "moe", "expert": {"ff": inner, "limit": 0.8}, "router": {"experts": experts, "top": top}}
    x = torch.randn(rows * 3, hidden, generator=g).to(dtype)
    ids, _, margin = plain.route(w, "m.", mlp, x.double())
    keep = (margin > 0.05).nonzero()[:rows, 0]
    assert len(keep) == rows
    x = x[keep]
    assert (ids[keep] == 6).any(-1).float().mean() > 0.7 and (ids[keep] == 1).any(-1).float().mean() < 0.3
    ctx = util.make_context(ops, dtype, [(0, rows)])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    res = torch.zeros(rows, hidden, device=DEV)
    y = moe.forward(ctx, x.to(DEV), res)
    gain = torch.ones(hidden, device=DEV)
    ops.norm_add(res, y.y, gain, 1e-5, center=True, weights=y.weights)
    want = plain.feed_forward(w, "m.", mlp, x.double())[0]
    assert rel_err(res, plain.layer_norm(want, gain.cpu(), 1e-5)) < tol
    got = dense.forward(ctx, x.to(DEV), res)
    assert rel_err(got, plain.expert(w, "d.", 0.8, x.double())) < tol


# ---- whole models ----------------------------------------------------------------------------

PROMPT_LENGTHS = [70, 1, 23, 97, 40, 64]


def safe_prompt(w, cfg, n, seed, rel_margin=0.3):
    """n tokens drawn so that every routing decision of the plain implementation is clear by
    `rel_margin` in the router's logits, which are a few units large (a close call may fall the
    other way under rounding, which no test is about)."""
    rng = random.Random(seed)
    toks = []
    tries = 0
    while len(toks) < n:
        cand = rng.randrange(cfg["vocab"])
        margin = plain.forward(cfg, w, toks + [cand])[2]
        tries += 1
        if float(margin[-1]) >= rel_margin:
            toks.append(cand)
        elif tries % (10 * n + 50) == 0:
            rel_margin /= 2
            if rel_margin < 5e-3:
                raise RuntimeError("no prompt with clear routing found")
    return toks


def row_errors(got, ref):
    d = (got - ref).double()
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / ref.double().std()


def noise_of(cfg, w, toks, ref):
    """How far the plain implementation's logits move when every weight is disturbed by one
    part in 2^9 (what rounding to bfloat16 does to a number): median, ninth decile and largest
    of the rows' errors. The comparisons' bounds come from the model at hand."""
    g = torch.Generator().manual_seed(len(toks))
    w2 = {k: v * (1 + torch.randn(v.shape, generator=g) * 2.0 ** -9) if v.is_floating_point() else v
          for k, v in w.items()}
    e = row_errors(plain.forward(cfg, w2, toks)[0], ref)
    return e.median().item(), e.kthvalue(max(1, int(0.9 * len(e)))).values.item(), e.max().item()


@pytest.fixture(scope="module", params=list(tuzapel_cases.CASES))
def case(request, tmp_path_factory):
    import ninfer_amd
    name = request.param
    make, seed = tuzapel_cases.CASES[name]
    raw = make()
    out = {"name": name, "cfg": raw, "dirs": {}, "ref": {}, "reqs": {}, "noise": {}}
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"tuzapel_{name}_{dtype}"))
        ninfer_amd.write_random_model(d, raw, seed, dtype=dtype, std=STD)
        out["dirs"][dtype] = d
    cfg, w = util.read_folder(out["dirs"]["bfloat16"])
    for i, n in enumerate(PROMPT_LENGTHS):
        out["reqs"][f"r{i}"] = safe_prompt(w, cfg, n, 50 + i)
    for dtype in ("float32", "bfloat16"):
        cfg, w = util.read_folder(out["dirs"][dtype])
        out["ref"][dtype] = {k: plain.forward(cfg, w, v)[0] for k, v in out["reqs"].items()}
        out["noise"][dtype] = {k: noise_of(cfg, w, v, out["ref"][dtype][k]) for k, v in out["reqs"].items()}
    return out


def make_runner(case, dtype, page_size=8, num_pages=40, seqs=4, **more):
    from ninfer_amd import EngineOptions, load_model
    opt = EngineOptions(dtype=dtype, max_context=128, num_sequences=seqs, page_size=page_size,
                        num_pages=num_pages, check_pages=True, poison_freed_pages=True, **more)
    return load_model(case["dirs"][dtype], opt)


def check_logits(case, dtype, got, what):
    for rid, g in got.items():
        ref = case["ref"][dtype][rid]
        who = f"{case['name']} {rid} {what}"
        assert g.shape == ref.shape, who
        assert torch.isfinite(g).all(), f"{who}: not finite"
        err = row_errors(g, ref)
        n50, n90, nmax = case["noise"][dtype][rid]
        f50, f90, fmax, floor = (3, 3, 3, 0.03) if dtype == "bfloat16" else \
            (8 * 2.0 ** -15, 8 * 2.0 ** -15, 16 * 2.0 ** -15, 3e-6)
        e50 = err.median().item()
        e90 = err.kthvalue(max(1, int(0.9 * len(err)))).values.item()
        if len(err) >= 20:
            assert e50 <= max(f50 * n50, floor), f"{who}: median row error {e50:.2e} (disturbance {n50:.2e})"
            assert e90 <= max(f90 * n90, floor), f"{who}: ninth decile {e90:.2e} (disturbance {n90:.2e})"
        assert err.max().item() <= max(fmax * nmax, 4 * floor), \
            f"{who}: row {err.argmax()} is off by {err.max():.2e} (disturbance {nmax:.2e})"


def test_layer_by_layer(case):
    """The 32-bit residual stream after every layer, for a prompt in one step and in portions."""
    from ninfer_amd.engine import Chunk
    cfg, w = util.read_folder(case["dirs"]["float32"])
    toks = case["reqs"]["r4"]
    streams = plain.forward(cfg, w, toks)[1]
    runner = make_runner(case, "float32")
    assert len(runner.spec.plan) == len(streams)
    for cuts in ([len(toks)], [17, 2, len(toks) - 19]):
        slot = runner.open()
        got = [[] for _ in streams]
        runner.tap = lambda i, residual, pending: got[i].append(residual.cpu().clone())
        o = 0
        for n in cuts:
            runner.step([Chunk(slot, toks[o:o + n], [])])
            o += n
        runner.tap = None
        runner.close(slot)
        for i, want in enumerate(streams):
            g = torch.cat(got[i]).double()
            assert (g - want).abs().max() <= 2e-5 * max(1.0, want.abs().max().item()), f"layer {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_portions(case, dtype):
    runner = make_runner(case, dtype)
    for rid, toks in case["reqs"].items():
        for what, sched in (("whole", util.schedule_whole(rid, toks)),
                            ("tail", util.schedule_tail(rid, toks, 48)),
                            ("portions", util.schedule_portions(rid, toks, seed=len(toks)))):
            if what == "tail" and len(toks) == 1:
                continue
            check_logits(case, dtype, util.run_schedule(runner, sched), what)
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_cut_does_not_matter_in_32_bit(case):
    """Every way of cutting a request gives the same logits to the bit in 32-bit: all kernels
    of that path sum in an order that depends on the row alone."""
    runner = make_runner(case, "float32")
    toks = case["reqs"]["r3"]
    whole = util.run_schedule(runner, util.schedule_whole("a", toks))["a"]
    for sched in (util.schedule_tail("a", toks, 40), util.schedule_portions("a", toks, seed=3)):
        assert torch.equal(util.run_schedule(runner, sched)["a"], whole)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(case, dtype):
    """Up to four live requests, prompt portions beside single tokens, in a pool so small that
    pages are used again (freed pages are filled with NaN) and with four state slots for twelve
    requests, then schedules drawn at random; every request's logits equal those of the
    request alone."""
    runner = make_runner(case, dtype, page_size=8, num_pages=34)
    reqs = dict(case["reqs"])
    reqs.update({k + "again": v for k, v in case["reqs"].items()})
    ref = {**case["ref"][dtype], **{k + "again": v for k, v in case["ref"][dtype].items()}}
    noise = {**case["noise"][dtype], **{k + "again": v for k, v in case["noise"][dtype].items()}}
    sub = {"name": case["name"], "ref": {dtype: ref}, "noise": {dtype: noise}}
    check_logits(sub, dtype, util.run_schedule(runner, util.schedule_mixed(reqs, seed=1)), "mixed")
    for seed in (2, 3):
        steps = util.schedule_random(reqs, seed)
        got = util.run_schedule(runner, steps)
        wanted = {}
        for entries, _ in steps:
            for rid, toks, want in entries:
                wanted.setdefault(rid, [0, []])
                wanted[rid][1] += [wanted[rid][0] + w_ for w_ in want]
                wanted[rid][0] += len(toks)
        part = {"name": case["name"], "noise": {dtype: noise},
                "ref": {dtype: {rid: ref[rid][rows] for rid, (_, rows) in wanted.items() if rows}}}
        check_logits(part, dtype, got, f"random {seed}")
    assert runner.cache.pages_reused() > 0
    runner.cache.check()


def test_a_slot_used_again_starts_empty(case):
    """One state slot: every request gets the slot the last one left, with that request's
    last projected rows still in it unless it is cleared."""
    runner = make_runner(case, "float32", seqs=1)
    for rid in ("r3", "r0", "r1", "r2"):
        toks = case["reqs"][rid]
        sched = util.schedule_tail(rid, toks, 5) if len(toks) > 1 else util.schedule_whole(rid, toks)
        check_logits(case, "float32", util.run_schedule(runner, sched), "slot used again")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(case, dtype):
    """A few tokens of prompt, then hundreds of single steps: across pages, with every window
    passing over decoded tokens many times and giving its pages back, across the attention
    kernels' tiles, with the convolutions' state carried on."""
    if case["name"] == "ones" and dtype == "bfloat16":
        pytest.skip("covered by the other two")
    from ninfer_amd import EngineOptions, load_model
    n = 230
    cfg, w = util.read_folder(case["dirs"][dtype])
    toks = safe_prompt(w, cfg, n, 9)
    ref = plain.forward(cfg, w, toks)[0]
    runner = load_model(case["dirs"][dtype], EngineOptions(
        dtype=dtype, max_context=256, num_sequences=2, page_size=16, num_pages=18, check_pages=True,
        poison_freed_pages=True))
    got = util.run_schedule(runner, util.schedule_tail("x", toks, n - 3))["x"]
    sub = {"name": case["name"], "ref": {dtype: {"x": ref}}, "noise": {dtype: {"x": noise_of(cfg, w, toks, ref)}}}
    check_logits(sub, dtype, {"x": got}, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt(case, dtype):
    """Hundreds of tokens in one step and in two portions (the kernels that many rows choose),
    with keys far back for the layers that see them all."""
    if case["name"] == "ones":
        pytest.skip("covered by the other two")
    from ninfer_amd import EngineOptions, load_model
    n = 300
    cfg, w = util.read_folder(case["dirs"][dtype])
    toks = safe_prompt(w, cfg, n, 19)
    ref = plain.forward(cfg, w, toks)[0]
    sub = {"name": case["name"], "ref": {dtype: {"x": ref}}, "noise": {dtype: {"x": noise_of(cfg, w, toks, ref)}}}
    runner = load_model(case["dirs"][dtype], EngineOptions(
        dtype=dtype, max_context=320, prefill_chunk=320, num_sequences=2, page_size=16, num_pages=24,
        check_pages=True, poison_freed_pages=True))
    check_logits(sub, dtype, util.run_schedule(runner, util.schedule_whole("x", toks)), "whole")
    steps = [([("x", toks[:257], list(range(257)))], []), ([("x", toks[257:], list(range(n - 257)))], ["x"])]
    check_logits(sub, dtype, util.run_schedule(runner, steps), "two portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_from_a_captured_graph(case, dtype):
    """Decode-only steps replayed from a HIP graph (the first step of a shape runs eagerly, the
    second is captured, the rest are replays), two requests side by side, every replay against
    the plain implementation: the convolutions' state travels in the memory the graph reads
    and writes."""
    runner = make_runner(case, dtype, use_graph=True)
    reqs = {k: case["reqs"][k] for k in ("r0", "r4")}
    from ninfer_amd.engine import Chunk
    slots = {k: runner.open() for k in reqs}
    heads = {k: len(v) - 30 for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    logits = runner.step([Chunk(slots[k], reqs[k][:heads[k]], list(range(heads[k]))) for k in reqs])
    o = 0
    for k in reqs:
        got[k].append(logits[o:o + heads[k]].float().cpu())
        o += heads[k]
    for i in range(30):
        logits = runner.step([Chunk(slots[k], [reqs[k][heads[k] + i]], [0]) for k in reqs])
        for j, k in enumerate(reqs):
            got[k].append(logits[j:j + 1].float().cpu().clone())
    assert len(runner._graphs) >= 1
    for k in reqs:
        runner.close(slots[k])
    check_logits(case, dtype, {k: torch.cat(v) for k, v in got.items()}, "graph replay")


@pytest.mark.parametrize("seed", list(range(8)))
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random (sizes, head counts, kinds and order of layers, windows,
    taps, what is absent), in both precisions: whole, in portions and in a mixed batch."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    raw = tuzapel_cases.random_config(seed)
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path / dtype)
        ninfer_amd.write_random_model(d, raw, 100 + seed, dtype=dtype, std=STD)
        cfg, w = util.read_folder(d)
        if dtype == "float32":
            reqs = {f"q{i}": safe_prompt(w, cfg, n, 7 * seed + i) for i, n in enumerate([33, 1, 14, 50])}
        ref = {k: plain.forward(cfg, w, v)[0] for k, v in reqs.items()}
        sub = {"name": f"random {seed}", "ref": {dtype: ref},
               "noise": {dtype: {k: noise_of(cfg, w, v, ref[k]) for k, v in reqs.items()}}}
        runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3, page_size=8,
                                             num_pages=20, check_pages=True, poison_freed_pages=True))
        for k, v in reqs.items():
            check_logits(sub, dtype, util.run_schedule(runner, util.schedule_whole(k, v)), "whole")
            check_logits(sub, dtype, util.run_schedule(runner, util.schedule_portions(k, v, seed=seed)), "portions")
        check_logits(sub, dtype, util.run_schedule(runner, util.schedule_mixed(reqs, seed=seed, max_live=3)), "mixed")
        runner.release()


def test_greedy_generation_through_the_scheduler(case):
    """The framework's own entry point: prompts of unequal length generated greedily by the
    scheduler (admission, portions under a token budget, batched decoding, sampling kernel),
    token for token what the plain implementation chooses."""
    from ninfer_amd import Ninfer, SamplingParams
    cfg, w = util.read_folder(case["dirs"]["float32"])
    prompts = [case["reqs"][k][:n] for k, n in (("r0", 19), ("r2", 3), ("r3", 41))]
    new = 10
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            z, _, margin = plain.forward(cfg, w, toks)
            top = torch.topk(z[-1], 2).values
            if top[0] - top[1] < 1e-3 or float(margin.min()) < 1e-3:
                break   # too close to call: the comparison ends here for this prompt
            toks.append(int(z[-1].argmax()))
        want.append(toks[len(p):])
    eng = Ninfer(case["dirs"]["float32"], max_context=128, prefill_chunk=16, num_sequences=2,
                 dtype="float32", page_size=8, num_pages=30)
    got = eng.generate(prompts, SamplingParams.greedy(new), stop_ids=[])
    eng.close()
    assert sum(len(x) for x in want) >= new
    assert [g[:len(x)] for g, x in zip(got, want)] == want


def test_command_line_and_trace_replay(case, tmp_path):
    """bin/trace_run on a model folder (a mixed schedule as JSON lines, the logits files
    against the plain implementation) and bin/ninfer generating greedily from it."""
    if case["name"] != "odd":
        pytest.skip("one configuration is enough for the programs")
    reqs = {k: case["reqs"][k] for k in ("r0", "r2", "r4", "r1")}
    steps = util.schedule_mixed(reqs, seed=4)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out_dir = str(tmp_path / "out")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
                        case["dirs"]["float32"], "--dtype", "float32", "--out", out_dir,
                        "--max-tokens", "256"], input=util.write_trace(steps), text=True,
                       capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    got = util.read_trace_output(out_dir, steps, case["cfg"]["vocab"])
    check_logits(case, "float32", got, "trace_run")
    stats = json.load(open(os.path.join(out_dir, "stats.json")))
    assert all(g["in_use"] == 0 for g in stats["groups"]) and any(g["window_freed"] > 0 for g in stats["groups"])
    prompt = case["reqs"]["r2"][:9]
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "ninfer"), case["dirs"]["float32"], "--dtype",
                        "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new", "4", "--temperature",
                        "0", "--max-context", "64"], text=True, capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    cfg, w = util.read_folder(case["dirs"]["float32"])
    first = int(plain.forward(cfg, w, prompt)[0][-1].argmax())
    assert str(first) in p.stdout
