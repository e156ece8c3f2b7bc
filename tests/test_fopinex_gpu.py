"""Fopinex on the GPU against the plain implementation: every mechanism alone through its
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

import fopinex_cases
import plain_fopinex as plain
import util

pytestmark = pytest.mark.gpu
DEV = "cuda"
STD = 0.25


@pytest.fixture(scope="module")
def ops():
    from ninfer_amd.kernels import load_ops
    return load_ops()


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def _steps(ops, dtype, lengths_by_step, slots):
    """StepContexts for requests that go on from step to step: lengths_by_step[i][r] rows of
    request r in step i (0: left out)."""
    done = [0] * len(slots)
    for lengths in lengths_by_step:
        seqs, who = [], []
        for r, n in enumerate(lengths):
            if n:
                seqs.append((done[r], n))
                who.append(r)
        ctx = util.make_context(ops, dtype, seqs)
        ctx.seq_slots = torch.tensor([slots[r] for r in who], dtype=torch.int32, device=DEV)
        yield ctx, who, [done[r] for r in who], [lengths[r] for r in who]
        for r, n in enumerate(lengths):
            done[r] += n


def _cut(n, sizes, tail):
    """n rows as portions of the given sizes in turn, the last `tail` one by one."""
    out, i, j = [], 0, 0
    while i < n - tail:
        s = min(sizes[j % len(sizes)], n - tail - i)
        out.append(s)
        i += s
        j += 1
    return out + [1] * tail


def _as_steps(cuts):
    n_steps = max(len(c) for c in cuts)
    return [[c[i] if i < len(c) else 0 for c in cuts] for i in range(n_steps)]


# ---- mechanisms alone ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 256, 1100])
def test_gated_sum_add(ops, dtype, width):
    """residual += mult (sigmoid(g1 + b1) a + sigmoid(g2 + b2) f): f dense, a weighted sum of
    rows in which some choices stand for experts that hand their input back, or absent."""
    g = torch.Generator().manual_seed(width)
    t, k, real = 37, 3, 4
    rnd = lambda *s: torch.randn(*s, generator=g)
    res = rnd(t, width)
    a, g1, g2, x, dense = (rnd(t, width).to(dtype) for _ in range(5))
    b1, b2 = rnd(width), rnd(width)
    y = rnd(t * k, width).to(dtype)
    wts = torch.rand(t, k, generator=g)
    ids = torch.randint(0, real + 2, (t, k), generator=g, dtype=torch.int32)
    y.view(t, k, width)[ids >= real] = float("nan")      # what no product has written

    class Rows:
        pass
    rows = Rows()
    rows.y, rows.weights, rows.ids, rows.real, rows.rows, rows.shared = y.to(DEV), wts.to(DEV), ids.to(DEV), real, x.to(DEV), None
    sig = lambda z, b: torch.sigmoid(z.double() + b.double())
    yy = torch.where((ids >= real)[:, :, None], x.double()[:, None, :], y.double().view(t, k, width).nan_to_num())
    sparse = (yy * wts.double()[:, :, None]).sum(1)
    for f_dev, f_ref, gate2 in ((dense.to(DEV), dense.double(), True), (rows, sparse, True), (rows, sparse, False),
                                (None, None, False)):
        want = res.double() + 0.6 * (a.double() * sig(g1, b1) +
                                     (0 if f_ref is None else f_ref * (sig(g2, b2) if gate2 else 1.0)))
        got = res.clone().to(DEV)
        ops.gated_sum_add(got, a.to(DEV), g1.to(DEV), b1.to(DEV), f_dev, g2.to(DEV) if gate2 else None,
                          b2.to(DEV) if gate2 else None, 0.6)
        assert rel_err(got, want) < 1e-6
    got = res.clone().to(DEV)       # no mixer rows, no gates, no biases
    ops.gated_sum_add(got, None, None, None, rows, g2.to(DEV), None, 1.0)
    assert rel_err(got, res.double() + sparse * torch.sigmoid(g2.double())) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("groups,group", [(3, 20), (1, 64), (4, 128), (5, 8)])
def test_norm_per_head_with_a_silu_gate(ops, dtype, groups, group):
    g = torch.Generator().manual_seed(group)
    t, n = 9, groups * group
    o = torch.randn(t, n, generator=g) * 3
    wide = torch.randn(t, n + 24, generator=g).to(dtype)
    w = 1 + 0.3 * torch.randn(group, generator=g)
    z = wide[:, 24:].double()
    want = plain.rms(o.double().view(t, groups, group), 1e-5) * w.double()
    want = want.reshape(t, n) * z * torch.sigmoid(z)
    out = torch.empty(t, n, dtype=dtype, device=DEV)
    ops.gated_rmsnorm(o.to(DEV), wide.to(DEV)[:, 24:], w.to(DEV), 1e-5, out, group=group, gate_act="silu")
    assert rel_err(out, want) < (1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 20, 70, 300])
def test_experts_with_clamped_gate_and_identity_experts(ops, dtype, rows):
    """Routing over experts and identity experts, the grouped products with the clamped gate
    at every row count (few-row, tile and plain kernels), the sum with the identity terms:
    against the plain feed-forward."""
    from ninfer_amd.parts import SparseMoE
    hidden, inner, experts, identity, top = 128, 64, 6, 3, 3
    mlp = {"expert": {"ff": inner, "limit": 1.1}, "router": {"experts": experts, "identity": identity, "top": top,
                                                           "groups": {"count": 3, "keep": 2}}}
    part = SparseMoE("m.", hidden, experts, top, inner, renorm=False, act="clamped_swish", act_limit=1.1,
                     act_alpha=1.702, identity=identity,
                     router={"choice_bias": True, "choice_bias_leaf": "correction", "n_group": 3, "topk_group": 2},
                     names={"router": "", "router_leaf": "router", "experts": "e", "expert_leaves": ("gate", "up", "down")})
    w = {k: v.to(dtype).float() for k, v in util.random_part_weights(part, 5, std=0.3).items()}
    w["m.correction"] = w["m.correction"] * 0.2
    from ninfer_amd.parts import WeightBinder
    part.bind_all(WeightBinder(util.DictSource(w), torch.device(DEV), dtype))
    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, hidden, generator=g).to(dtype)
    margins = []
    want = plain.moe(w, "m.", mlp, x.double(), margins)
    clear = margins[0] > 1e-3
    for generic in (False, True):
        ops.force_generic = generic
        try:
            ctx = util.make_context(ops, dtype, [(0, rows)])
            pending = part.forward(ctx, x.to(DEV), None)
            got = torch.zeros(rows, hidden, device=DEV)
            pending.add_to(ctx, got)
        finally:
            ops.force_generic = False
        if rows >= 20:
            assert (pending.ids >= experts).any() and (pending.ids < experts).any()
        assert rel_err(got.cpu()[clear], want[clear]) < (2e-5 if dtype == torch.float32 else 1.5e-2)


class _Paged:
    """A cache of keys and values for requests that go on from step to step, with pages dealt
    out of order, fed through the mixer's own kernels (write and attention)."""

    def __init__(self, ops, dtype, heads, kv_heads, dim, vdim, page_size, lens, seed):
        self.ops, self.dtype = ops, dtype
        self.H, self.G, self.d, self.vd, self.ps = heads, kv_heads, dim, vdim, page_size
        g = torch.Generator().manual_seed(seed)
        per = [-(-n // page_size) for n in lens]
        pages = sum(per) + 3
        perm = torch.randperm(pages, generator=g)
        self.table = torch.full((len(lens), max(per)), -1, dtype=torch.int32)
        at = 0
        for r, n in enumerate(per):
            self.table[r, :n] = perm[at:at + n]
            at += n
        nan = float("nan")   # what is not written is not to be read
        self.k = torch.full((pages, kv_heads, page_size, dim), nan, dtype=dtype, device=DEV)
        self.v = torch.full((pages, kv_heads, page_size, vdim), nan, dtype=dtype, device=DEV)
        width = (heads + kv_heads) * dim + kv_heads * vdim
        self.rows = [(torch.randn(n, width, generator=g)).to(dtype) for n in lens]
        self.bias = torch.randn(heads, generator=g)
        self.mix = torch.randn(heads, heads, generator=g) / math.sqrt(heads) + torch.eye(heads)

    def run(self, steps, scale, chunk, force_plain=False, mix=True, bias=True):
        got = [torch.zeros(r.shape[0], self.H * self.vd) for r in self.rows]
        self.ops.force_generic = force_plain
        try:
            for ctx, who, starts, counts in _steps(self.ops, self.dtype, steps, list(range(len(self.rows)))):
                qkv = torch.cat([self.rows[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
                out = torch.empty(ctx.T, self.H * self.vd, dtype=self.dtype, device=DEV)
                self.ops.sigmoid_attention(qkv, self.k, self.v, self.table[who].contiguous().to(DEV), ctx,
                                           self.H, self.G, self.d, self.vd, self.ps, scale, chunk or 0,
                                           self.bias.to(DEV) if bias else None,
                                           self.mix.to(DEV) if mix else None, out)
                o = 0
                for r, s, n in zip(who, starts, counts):
                    got[r][s:s + n] = out[o:o + n].float().cpu()
                    o += n
        finally:
            self.ops.force_generic = False
        return got

    def plain(self, scale, chunk, mix=True, bias=True):
        """The oracle's attention on these rows (identity projections: the rows are q, k, v)."""
        out = []
        nq, nk = self.H * self.d, self.G * self.d
        m = {"heads": self.H, "kv_heads": self.G, "dim": self.d, "vdim": self.vd, "scale": scale,
             "mask": {"size": chunk} if chunk else None}
        for r in self.rows:
            x = r.double()
            n = x.shape[0]
            w = {"q": torch.eye(nq, dtype=torch.float64), "o": torch.eye(self.H * self.vd, dtype=torch.float64),
                 "pb": self.bias if bias else torch.zeros(self.H),
                 "talk": self.mix if mix else torch.eye(self.H)}
            kv = (x[:, nq:nq + nk].view(n, self.G, self.d).transpose(0, 1),
                  x[:, nq + nk:].view(n, self.G, self.vd).transpose(0, 1))
            out.append(plain.sigmoid_attention(w, "", m, x[:, :nq], kv))
        return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,ps,chunk", [
    (6, 3, 12, 20, 8, 10), (4, 1, 32, 64, 16, 64), (2, 2, 16, 32, 4, None), (4, 2, 64, 128, 16, 96),
    (16, 4, 128, 128, 16, 100), (1, 1, 128, 8, 16, 33), (8, 2, 24, 96, 2, 1), (12, 4, 40, 72, 32, 70),
    (16, 2, 64, 64, 8, 32), (3, 1, 136, 160, 8, 50), (20, 20, 8, 16, 16, 17)])
def test_attention_without_softmax_in_portions(ops, dtype, heads, kv_heads, dim, vdim, ps, chunk):
    """Three requests of unequal length side by side: portions that end before, at and after
    the borders of pages, of chunks and of the kernels' tiles of keys, down to two rows, then
    rows one by one; against the plain implementation, and the plain kernel against the others."""
    lens = [200, 67, 331]
    scale = 0.9 / math.sqrt(dim)
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, lens, seed=dim + vdim)
    steps = _as_steps([_cut(200, [63, 2, 64, 5], 30), _cut(67, [3, 61], 3), _cut(331, [128, 2, 65, 100], 20)])
    want = cache.plain(scale, chunk)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    for force_plain in (False, True):
        got = cache.run(steps, scale, chunk, force_plain)
        for g, w_ in zip(got, want):
            assert torch.isfinite(g).all()
            assert rel_err(g, w_) < tol
    # without the mixing matrix and the bias
    got = cache.run(steps, scale, chunk, mix=False, bias=False)
    for g, w_ in zip(got, cache.plain(scale, chunk, mix=False, bias=False)):
        assert rel_err(g, w_) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_whole_against_rows(ops, dtype):
    """A whole prompt in one step, and the same rows one by one: the 32-bit sums depend on the
    row alone."""
    heads, kv_heads, dim, vdim, ps, n, chunk = 4, 2, 32, 64, 16, 700, 300
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, [n], seed=8)
    want = cache.plain(0.2, chunk)[0]
    whole = cache.run([[n]], 0.2, chunk)[0]
    rows = cache.run([[n - 150]] + [[1]] * 150, 0.2, chunk)[0]
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    assert rel_err(whole, want) < tol and rel_err(rows, want) < tol
    if dtype == torch.float32:
        assert torch.equal(whole, rows)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,key,seen", [
    (96, 576, True), (96, 575, False), (96, 643, True), (96, 600, True), (100, 600, True), (100, 599, False),
    (None, 0, True), (None, 1, True), (None, 300, True), (None, 15, True), (None, 16, True), (700, 0, True),
    (64, 640, True), (64, 639, False), (32, 641, True), (32, 639, False), (644, 0, True), (643, 0, False)])
def test_one_loud_key_at_the_chunk_edges(ops, dtype, chunk, key, seen):
    """All scores far below zero (weights near 0) but one key's, whose weight is near 1: the
    result is that key's value when the key lies in the row's chunk and nothing when it lies
    just outside, for the last row of a prompt portion and for a single row."""
    heads, kv_heads, dim, vdim, ps, n = 2, 1, 16, 32, 16, 644
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, [n], seed=key + 7 * (chunk or 0))
    rows = cache.rows[0].float()
    nq = heads * dim
    rows[:, :nq + dim] *= 0.02                           # quiet queries and keys everywhere
    q = 3.0 * torch.sign(torch.randn(dim))
    for r in (n - 3, n - 1):
        rows[r, :dim] = q
        rows[r, dim:nq] = q
    rows[key, nq:nq + dim] = q * 2                       # score 96 dim / 16 at `key`
    cache.rows[0] = rows.to(dtype)
    cache.bias = torch.full((heads,), -14.0)
    cache.mix = torch.tensor([[1.0, 0.0], [0.5, 0.5]])
    want = cache.plain(1.0 / 4, chunk)[0]
    v = cache.rows[0].double()[key, nq + dim:]
    tol = 1e-4 if dtype == torch.float32 else 1.5e-2
    for steps in ([[n]], [[n - 2], [1], [1]]):
        got = cache.run(steps, 1.0 / 4, chunk)[0]
        for r in (n - 3, n - 1):
            assert (got[r] - want[r].float()).norm() < tol * max(1.0, want[r].norm().item())
        head0 = got[n - 1].view(heads, vdim)[0].double()
        if seen:
            assert rel_err(head0, v) < 0.02
        else:
            assert head0.norm() < 0.01 * v.norm()


def _gla_rows(heads, dim, vdim, lens, seed, dtype, z_scale=3.0):
    g = torch.Generator().manual_seed(seed)
    width = 5 + 2 * heads * dim + heads * vdim
    rows = [torch.randn(n, width, generator=g).to(dtype) for n in lens]
    z = [torch.randn(n, heads * dim, generator=g) * z_scale + 2.0 for n in lens]
    return rows, z


def _gla_plain(rows, z, heads, dim, vdim, tau, q_scale):
    out = []
    for x, zz in zip(rows, z):
        x, n = x.double(), x.shape[0]
        q = x[:, 5:5 + heads * dim].view(n, heads, dim) * q_scale
        k = x[:, 5 + heads * dim:5 + 2 * heads * dim].view(n, heads, dim)
        v = x[:, 5 + 2 * heads * dim:].view(n, heads, vdim)
        alpha = torch.exp(torch.nn.functional.logsigmoid(zz.double()) / tau).view(n, heads, dim)
        s = torch.zeros(heads, dim, vdim, dtype=torch.float64)
        o = torch.zeros(n, heads * vdim, dtype=torch.float64)
        for t in range(n):
            s = alpha[t][:, :, None] * s + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hd,hdv->hv", q[t], s).reshape(-1)
        out.append(o)
    return out


@pytest.mark.parametrize("dtype,chunks", [(torch.float32, False), (torch.bfloat16, False),
                                          (torch.bfloat16, True)])
@pytest.mark.parametrize("heads,dim,vdim,tau", [(3, 10, 12, 5.0), (2, 64, 64, 16.0), (1, 128, 32, 1.0),
                                                (4, 16, 100, 2.0), (2, 200, 24, 8.0), (5, 33, 17, 0.5),
                                                (3, 12, 20, 5.0), (2, 40, 130, 0.5), (1, 4, 1, 1.0)])
def test_gated_linear_attention_in_portions(ops, dtype, chunks, heads, dim, vdim, tau):
    """Three requests in slots 2, 0 and 3 of a wider state tensor, cut into portions down to
    two rows and single rows, with logits that drive some decays to 0 and some to 1; token by
    token, and with the workspace that lets steps with longer portions run in chunks (sizes
    that the chunks refuse fall back by themselves)."""
    lens = [150, 9, 77]
    rows, z = _gla_rows(heads, dim, vdim, lens, dim * vdim, dtype)
    z[0][:, :3] = 40.0          # decay 1: a channel that never forgets
    z[0][:, 3:5] = -60.0        # decay (nearly) 0
    want = _gla_plain(rows, z, heads, dim, vdim, tau, dim ** -0.5)
    slots = [2, 0, 3]
    floats = heads * dim * vdim
    state = torch.full((4, floats + 11), 7.0, device=DEV)
    state[:, 3:3 + floats] = 0
    view = state[:, 3:3 + floats]
    steps = _as_steps([_cut(150, [63, 2, 64, 5], 8), _cut(9, [3, 2], 2), _cut(77, [2, 30, 1, 17], 5)])
    got = [torch.zeros(n, heads * vdim) for n in lens]
    for ctx, who, starts, counts in _steps(ops, dtype, steps, slots):
        x = torch.cat([rows[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
        zz = torch.cat([z[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
        out = torch.empty(ctx.T, heads * vdim, device=DEV)
        wf = ops.gla_work_floats(dtype, ctx, heads, dim) if chunks else 0
        work = torch.full((ctx.T, wf), float("nan"), device=DEV) if wf else None
        ops.gated_linear_attention(x, 5, 5 + heads * dim, 5 + 2 * heads * dim, zz, heads, dim, vdim, tau,
                                   dim ** -0.5, view, ctx, out, work=work)
        o = 0
        for r, s, n in zip(who, starts, counts):
            got[r][s:s + n] = out[o:o + n].cpu()
            o += n
    for g, w_ in zip(got, want):
        assert rel_err(g, w_) < 3e-5
    assert (state[:, :3] == 7).all() and (state[:, 3 + floats:] == 7).all() and (state[1] [3:3 + floats] == 0).all()


# ---- whole models ----------------------------------------------------------------------------

PROMPT_LENGTHS = [70, 1, 23, 97, 40, 64]


def safe_prompt(w, cfg, n, seed, rel_margin=0.02):
    """n tokens drawn so that every routing decision of the plain implementation is clear by
    `rel_margin` (a close call may fall the other way under rounding, which no test is about)."""
    rng = random.Random(seed)
    toks = []
    tries = 0
    while len(toks) < n:
        cand = rng.randrange(cfg["vocab"])
        margins = []
        plain.forward(cfg, w, toks + [cand], margins=margins)
        tries += 1
        if all(float(m[-1]) >= rel_margin for m in margins):
            toks.append(cand)
        elif tries % (10 * n + 50) == 0:
            rel_margin /= 2
            if rel_margin < 5e-4:
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


@pytest.fixture(scope="module", params=list(fopinex_cases.CASES))
def case(request, tmp_path_factory):
    import ninfer_amd
    name = request.param
    make, seed = fopinex_cases.CASES[name]
    raw = make()
    out = {"name": name, "cfg": raw, "dirs": {}, "ref": {}, "reqs": {}, "noise": {}}
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"fopinex_{name}_{dtype}"))
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
    recurrent state still in it unless it is cleared."""
    runner = make_runner(case, "float32", seqs=1)
    for rid in ("r3", "r0", "r1", "r2"):
        toks = case["reqs"][rid]
        sched = util.schedule_tail(rid, toks, 5) if len(toks) > 1 else util.schedule_whole(rid, toks)
        check_logits(case, "float32", util.run_schedule(runner, sched), "slot used again")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(case, dtype):
    """A few tokens of prompt, then hundreds of single steps: across pages, across many chunks
    of the mask, across the attention kernels' tiles, with the recurrence's state carried on."""
    if case["name"] == "ones" and dtype == "bfloat16":
        pytest.skip("covered by the other two")
    from ninfer_amd import EngineOptions, load_model
    n = 230
    cfg, w = util.read_folder(case["dirs"][dtype])
    toks = safe_prompt(w, cfg, n, 9)
    ref = plain.forward(cfg, w, toks)[0]
    runner = load_model(case["dirs"][dtype], EngineOptions(
        dtype=dtype, max_context=256, num_sequences=2, page_size=16, num_pages=18, check_pages=True))
    got = util.run_schedule(runner, util.schedule_tail("x", toks, n - 3))["x"]
    sub = {"name": case["name"], "ref": {dtype: {"x": ref}}, "noise": {dtype: {"x": noise_of(cfg, w, toks, ref)}}}
    check_logits(sub, dtype, {"x": got}, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_from_a_captured_graph(case, dtype):
    """Decode-only steps replayed from a HIP graph (the first step of a shape runs eagerly, the
    second is captured, the rest are replays), two requests side by side, every replay against
    the plain implementation: the recurrent state travels in the memory the graph reads and writes."""
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
    """Configurations drawn at random (sizes, head counts, kinds and order of layers, chunks,
    what is absent), in both precisions: whole, in portions and in a mixed batch."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    raw = fopinex_cases.random_config(seed)
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
            margins = []
            logits = plain.forward(cfg, w, toks, margins=margins)[0][-1]
            top = torch.topk(logits, 2).values
            if top[0] - top[1] < 1e-3 or any(float(m[-1]) < 1e-3 for m in margins):
                break   # too close to call: the comparison ends here for this prompt
            toks.append(int(logits.argmax()))
        want.append(toks[len(p):])
    eng = Ninfer(case["dirs"]["float32"], max_context=128, prefill_chunk=16, num_sequences=2,
                 dtype="float32", page_size=8, num_pages=30)
    got = eng.generate(prompts, SamplingParams.greedy(new), stop_ids=[])
    eng.close()
    assert sum(len(x) for x in want) >= new
    assert [g[:len(x)] for g, x in zip(got, want)] == want


def test_trace_replay_program(case, tmp_path):
    """bin/trace_run on a model folder: a mixed schedule as JSON lines, the logits files
    against the plain implementation."""
    if case["name"] != "odd":
        pytest.skip("one configuration is enough for the program")
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
    assert stats["groups"][0]["in_use"] == 0
