"""Tuzapel without a GPU: the configuration reader, the model the builder makes (tensor names
and shapes, caches shared between layers, state), the plain implementation's own properties
(window mask, sink, convolution in pieces, frequency bands, routing by hand), and the engine's
host logic on plain stand-ins for the kernels."""
import copy
import math

import pytest
import torch

import plain_tuzapel as plain
import tuzapel_cases
import util

D = torch.float64
STD = 0.25


def _spec(raw):
    from ninfer_amd import build_spec
    return build_spec(raw)


# ---- reader and builder ----------------------------------------------------------------------

def test_reader_reads_every_key():
    cfg, _ = _spec(tuzapel_cases.config_odd())
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.logit_softcap) == (211, 72, 1e-5, 20.0)
    a = cfg.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.taps, a.window, a.kv_from) == (6, 3, 20, 12, 4, 10, None)
    assert (a.rot.dims, a.rot.scaling.factor, a.rot.scaling.low, a.rot.scaling.high, a.rot.scaling.original) == \
        (10, 3.0, 1.0, 6.0, 48)
    m = cfg.layers[1].mixer
    assert (m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank, m.rot.dims) == (3, 12, 6, 20, 40, 24, 6)
    assert cfg.layers[2].mixer.kv_from == 0 and cfg.layers[2].mlp is None
    f = cfg.layers[0].mlp
    assert (f.kind, f.ff, f.experts, f.top, f.limit) == ("moe", 24, 7, 3, 1.5)
    assert cfg.layers[1].mlp.kind == "dense" and cfg.layers[1].mlp.limit == 0.7
    ones, _ = _spec(tuzapel_cases.config_ones())
    assert ones.logit_softcap == 0.0 and ones.layers[2].mixer.window is None and ones.layers[2].mixer.taps == 0
    assert ones.layers[1].mixer.q_rank is None


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].update(low=9.0), "scaling"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=16), "kv_from"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=8), "top"),
    (lambda c: c["layers"][1]["mlp"].update(limit=0.0), "limit"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "kind"),
    (lambda c: c["layers"][1]["mixer"].update(scale=-1.0), "scale"),
])
def test_reader_names_the_key_it_refuses(change, word):
    from ninfer_amd.config import ConfigError
    raw = copy.deepcopy(tuzapel_cases.config_odd())
    change(raw)
    with pytest.raises(ConfigError, match=word):
        _spec(raw)


@pytest.mark.parametrize("name", list(tuzapel_cases.CASES))
def test_builder_names_every_tensor(name):
    raw = tuzapel_cases.CASES[name][0]()
    cfg, spec = _spec(raw)
    specs = spec.tensor_specs()
    w = raw["width"]
    assert specs["embed"].shape == (raw["vocab"], w) and specs["final.norm"].shape == (w,)
    assert "head" not in specs     # the logits come from the embedding table
    for i, layer in enumerate(raw["layers"]):
        m, p = layer["mixer"], f"l{i}."
        assert specs[p + "norm1"].shape == (w,) and specs[p + "norm1b"].shape == (w,)
        if layer["type"] == "latent_attention":
            q_width = m["heads"] * (m["dim"] + m["rot_dim"])
            if m.get("q_rank"):
                assert specs[p + "mix.dq"].shape == (m["q_rank"], w)
                assert specs[p + "mix.dq.norm"].shape == (m["q_rank"],)
                assert specs[p + "mix.uq"].shape == (q_width, m["q_rank"])
            else:
                assert specs[p + "mix.q"].shape == (q_width, w) and p + "mix.dq" not in specs
            assert specs[p + "mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], w)
            assert specs[p + "mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert specs[p + "mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"])
            assert specs[p + "mix.o"].shape == (w, m["heads"] * m["vdim"])
        else:
            owns = m.get("kv_from") is None
            assert specs[p + "mix.q"].shape == (m["heads"] * m["dim"], w)
            assert specs[p + "mix.q.norm"].shape == (m["dim"],)
            assert specs[p + "mix.o"].shape == (w, m["heads"] * m["vdim"])
            for key in ("k", "v", "k.norm", "k.conv", "v.conv"):
                assert (p + "mix." + key in specs) == (owns and (m.get("conv", 0) > 0 or "conv" not in key))
            if m.get("conv"):
                assert specs[p + "mix.q.conv"].shape == (m["heads"] * m["dim"], m["conv"])
                if owns:
                    assert specs[p + "mix.v.conv"].shape == (m["kv_heads"] * m["vdim"], m["conv"])
        c = layer["mlp"]
        assert (p + "norm2" in specs) == bool(c) and (p + "norm2b" in specs) == bool(c)
        if c and c["kind"] == "dense":
            assert specs[p + "mlp.gate"].shape == (c["ff"], w) and specs[p + "mlp.down"].shape == (w, c["ff"])
        elif c:
            e = c["router"]["experts"]
            assert specs[p + "mlp.router"].shape == (e, w) and specs[p + "mlp.router.b"].shape == (e,)
            assert specs[f"{p}mlp.e{e - 1}.up"].shape == (c["expert"]["ff"], w)
            assert f"{p}mlp.e{e}.up" not in specs


def test_shared_caches_state_and_kept_spans():
    """A layer that reads another's keys and values has no cache of its own; the owner's cache
    keeps what the widest window among its readers sees; the state holds taps - 1 projected rows."""
    cfg, spec = _spec(tuzapel_cases.config_odd())
    assert [c.cache_from for c in spec.plan] == [None, None, 0, None, 0]
    mixers = [b.mixer for b in spec.blocks]
    assert mixers[0].cache_need().window == 27 and mixers[0].window == 10
    assert mixers[2].cache_need() is None and mixers[2].window == 27 and mixers[4].window == 5
    assert mixers[3].cache_need().window == 33
    assert mixers[1].cache_need().window is None
    k, v = mixers[0].cache_need().pools
    assert (k.outer, k.inner, v.inner) == ((3,), (20,), (12,))
    assert mixers[0].state_floats() == 3 * (6 * 20 + 3 * 20 + 3 * 12)
    assert mixers[2].state_floats() == 1 * 6 * 20 and mixers[1].state_floats() == 0
    _, ones = _spec(tuzapel_cases.config_ones())
    assert ones.blocks[0].mixer.state_floats() == 0 and ones.blocks[2].mixer.cache_need().window is None


# ---- the plain implementation's own properties -----------------------------------------------

def test_plain_window_mask_and_sink():
    vis = plain.visible(6, 3)
    assert vis[4].tolist() == [False, False, True, True, True, False]
    assert vis[1].tolist() == [True, True, False, False, False, False]
    assert plain.visible(4, None)[3].all() and plain.visible(5, 1).sum() == 5
    s = torch.tensor([[0.0, 0.0, 5.0]], dtype=D)
    p = plain.softmax_rows(s, torch.tensor([[True, True, False]]), True)
    assert torch.allclose(p, torch.tensor([[1 / 3, 1 / 3, 0.0]], dtype=D))
    p = plain.softmax_rows(s - 50, torch.tensor([[True, True, True]]), True)
    assert p.sum() < 1e-19    # a row may attend to (almost) nothing
    assert torch.allclose(plain.softmax_rows(s, plain.visible(3, None)[2:], False).sum(), torch.ones((), dtype=D))


def test_plain_convolution_in_pieces_and_by_hand():
    g = torch.Generator().manual_seed(1)
    u, w = torch.randn(11, 5, generator=g, dtype=D), torch.randn(5, 4, generator=g, dtype=D)
    whole = plain.short_conv(u, w)
    assert torch.allclose(whole[0], w[:, 3] * u[0]) and torch.allclose(whole[2], w[:, 1] * u[0] + w[:, 2] * u[1] + w[:, 3] * u[2])
    first = plain.short_conv(u[:6], w)
    rest = plain.short_conv(u[6:], w, before=u[3:6])
    assert torch.allclose(torch.cat([first, rest]), whole)


def test_plain_frequency_bands_and_pairings():
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}
    f = plain.frequencies(rot)
    plain_f = [100.0 ** (-2 * i / 8) for i in range(4)]
    waves = [2 * math.pi / x for x in plain_f]          # 6.3, 19.9, 62.8, 198.7 against bounds 10 and 40
    assert waves[0] < 10 < waves[1] < 40 < waves[2]
    assert f[0] == plain_f[0] and abs(f[2] - plain_f[2] / 4) < 1e-15 and abs(f[3] - plain_f[3] / 4) < 1e-15
    s = (40 / waves[1] - 1.0) / 3.0
    assert abs(f[1] - ((1 - s) * plain_f[1] / 4 + s * plain_f[1])) < 1e-15
    x = torch.randn(3, 2, 10, dtype=D, generator=torch.Generator().manual_seed(2))
    pos = torch.tensor([0, 5, 9])
    for pairing in ("half", "interleaved"):
        y = plain.rotate(x, pos, rot, pairing)
        assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
        assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    a = 5 * float(f[1])
    y = plain.rotate(x, pos, rot, "interleaved")[1, 0]
    assert abs(y[2] - (x[1, 0, 2] * math.cos(a) - x[1, 0, 3] * math.sin(a))) < 1e-12
    y = plain.rotate(x, pos, rot, "half")[1, 0]
    assert abs(y[5] - (x[1, 0, 5] * math.cos(a) + x[1, 0, 1] * math.sin(a))) < 1e-12


def test_plain_routing_and_clamps_by_hand():
    w = {"r.router": torch.eye(4, dtype=D), "r.router.b": torch.tensor([0.0, 0.0, 3.0, 0.0], dtype=D)}
    h = torch.tensor([[2.0, 1.0, -1.5, 0.0]], dtype=D)      # logits 2, 1, 1.5, 0
    ids, wts, margin = plain.route(w, "r.", {"router": {"experts": 4, "top": 2}}, h)
    assert ids.tolist() == [[0, 2]] and abs(float(margin) - 0.5) < 1e-12
    assert torch.allclose(wts, torch.softmax(torch.tensor([[2.0, 1.5]], dtype=D), -1))
    e = {"e.gate": torch.tensor([[1.0]], dtype=D), "e.up": torch.tensor([[1.0]], dtype=D),
         "e.down": torch.tensor([[1.0]], dtype=D)}
    big = plain.expert(e, "e.", 2.0, torch.tensor([[10.0]], dtype=D))
    assert abs(float(big) - 2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0) < 1e-12
    low = plain.expert(e, "e.", 2.0, torch.tensor([[-10.0]], dtype=D))
    assert abs(float(low) - (-10.0) / (1 + math.exp(17.02)) * (-2.0 + 1)) < 1e-12


# ---- the engine's host logic on plain stand-ins ----------------------------------------------

@pytest.fixture(scope="module", params=list(tuzapel_cases.CASES))
def host_case(request, tmp_path_factory):
    import ninfer_amd
    make, seed = tuzapel_cases.CASES[request.param]
    raw = make()
    d = str(tmp_path_factory.mktemp(f"tuzapel_host_{request.param}"))
    ninfer_amd.write_random_model(d, raw, seed, dtype="float32", std=STD)
    cfg, w = util.read_folder(d)
    g = torch.Generator().manual_seed(seed)
    reqs = {f"r{i}": torch.randint(0, raw["vocab"], (n,), generator=g).tolist()
            for i, n in enumerate([37, 1, 12, 50, 23])}
    ref, clear = {}, {}
    for k, v in reqs.items():
        z, _, margin = plain.forward(cfg, w, v)
        ref[k], clear[k] = z, margin > 1e-3
    return {"name": request.param, "dir": d, "cfg": raw, "reqs": reqs, "ref": ref, "clear": clear}


def _host_runner(case, **more):
    from ninfer_amd import EngineOptions, load_model
    from plain_ops import PlainOps
    opt = dict(dtype="float32", device="cpu", max_context=64, num_sequences=4, page_size=4, num_pages=40,
               check_pages=True)
    opt.update(more)
    return load_model(case["dir"], EngineOptions(**opt), ops=PlainOps())


def _close(case, got):
    for rid, g in got.items():
        rid = rid.split("#")[0]
        ok = case["clear"][rid]
        # a close call at one row changes what that row leaves in the cache for all later rows
        upto = int((~ok).nonzero()[0]) if (~ok).any() else len(ok)
        torch.testing.assert_close(g.double()[:upto], case["ref"][rid][:upto], atol=2e-4, rtol=2e-4)


def test_host_every_way_of_cutting(host_case):
    runner = _host_runner(host_case)
    for rid, toks in host_case["reqs"].items():
        scheds = [util.schedule_whole(rid, toks), util.schedule_portions(rid, toks, seed=len(toks))]
        if len(toks) > 1:
            scheds.append(util.schedule_tail(rid, toks, 9))
        for sched in scheds:
            _close(host_case, util.run_schedule(runner, sched))
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_host_mixed_batches_reuse_pages_and_slots(host_case):
    """Portions beside single tokens, a pool that forces pages to be used again, two state
    slots for five requests and their repeats: a slot's convolution state starts at zero for
    every request that takes it, and the windows give their pages back as they move on."""
    runner = _host_runner(host_case, num_sequences=2, num_pages=26)
    reqs = dict(host_case["reqs"])
    reqs.update({k + "#2": v for k, v in host_case["reqs"].items()})
    _close(host_case, util.run_schedule(runner, util.schedule_mixed(reqs, seed=2, max_live=2)))
    assert runner.cache.pages_reused() > 0
    if host_case["name"] == "odd":
        assert sum(g.window_freed for g in runner.cache.groups) > 0
    runner.cache.check()


def test_host_generation_through_the_scheduler(host_case):
    """Greedy generation by the scheduler (admission, portions under a token budget, batched
    decoding with fewer slots than requests), token for token the plain choice."""
    from ninfer_amd import Request, Sampler, SamplingParams, Scheduler
    from plain_ops import PlainOps
    cfg, w = util.read_folder(host_case["dir"])
    prompts = [host_case["reqs"]["r2"], host_case["reqs"]["r1"], host_case["reqs"]["r4"][:7],
               host_case["reqs"]["r0"][:15]]
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(6):
            z, _, margin = plain.forward(cfg, w, toks)
            top = torch.topk(z[-1], 2).values
            if top[0] - top[1] < 1e-3 or float(margin.min()) < 1e-3:
                break
            toks.append(int(z[-1].argmax()))
        want.append(toks[len(p):])
    runner = _host_runner(host_case, num_sequences=2, prefill_chunk=8, num_pages=14)
    sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
    reqs = [Request(f"q{i}", list(p), SamplingParams.greedy(6)) for i, p in enumerate(prompts)]
    for r in reqs:
        sched.add(r)
    sched.run()
    assert all(r.status == "finished" for r in reqs), [r.error for r in reqs]
    assert [r.output[:len(x)] for r, x in zip(reqs, want)] == want
