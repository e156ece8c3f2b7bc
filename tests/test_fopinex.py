"""Fopinex without a GPU: the configuration reader, the model the builder makes (tensor names
and shapes, caches shared between layers, state), random-weights folders, the plain
implementation's own properties (the chunked mask, the routing rule, the recurrence against its
written-out sum), and the engine's host logic on plain stand-ins for the kernels."""
import copy
import math

import pytest
import torch

import fopinex_cases
import plain_fopinex as plain
import util

D = torch.float64


def _spec(raw):
    from ninfer_amd import build_spec
    return build_spec(raw)


@pytest.mark.parametrize("name", list(fopinex_cases.CASES))
def test_builder_names_every_tensor(name, tmp_path):
    import ninfer_amd
    make, seed = fopinex_cases.CASES[name]
    raw = make()
    cfg, spec = _spec(raw)
    specs = spec.tensor_specs()
    w = raw["width"]
    assert specs["embed"].shape == (raw["vocab"], w) and specs["head"].shape == (raw["vocab"], w)
    assert specs["final.norm"].shape == (w,)
    for i, layer in enumerate(raw["layers"]):
        m, p = layer["mixer"], f"l{i}."
        assert specs[p + "norm1"].shape == (w,) and specs[p + "rg1"].shape == (w, w)
        assert specs[p + "rg1.b"].shape == (w,)
        if layer["type"] == "attention":
            assert specs[p + "mix.q"].shape == (m["heads"] * m["dim"], w)
            assert specs[p + "mix.o"].shape == (w, m["heads"] * m["vdim"])
            assert specs[p + "mix.talk"].shape == (m["heads"], m["heads"])
            assert specs[p + "mix.pb"].shape == (m["heads"],)
            # a layer that reads another's keys and values has no projections of its own
            owns = m.get("kv_from") is None
            assert (p + "mix.k" in specs) == owns and (p + "mix.v" in specs) == owns
            if owns:
                assert specs[p + "mix.k"].shape == (m["kv_heads"] * m["dim"], w)
                assert specs[p + "mix.v"].shape == (m["kv_heads"] * m["vdim"], w)
        else:
            assert specs[p + "mix.q"].shape == (m["heads"] * m["dim"], w)
            assert specs[p + "mix.v"].shape == (m["heads"] * m["vdim"], w)
            assert specs[p + "mix.a1"].shape == (m["rank"], w)
            assert specs[p + "mix.a2"].shape == (m["heads"] * m["dim"], m["rank"])
            assert specs[p + "mix.a2.b"].shape == (m["heads"] * m["dim"],)
            assert specs[p + "mix.norm"].shape == (m["vdim"],)
        c = layer["mlp"]
        assert (p + "norm2" in specs) == bool(c) and (p + "rg2" in specs) == bool(c)
        if c:
            e, extra = c["router"]["experts"], c["router"].get("identity", 0)
            assert specs[p + "mlp.router"].shape == (e + extra, w)
            assert specs[p + "mlp.correction"].shape == (e + extra,)
            assert specs[p + f"mlp.e{e - 1}.down"].shape == (w, c["expert"]["ff"])
            assert p + f"mlp.e{e}.down" not in specs      # identity experts have no tensors
    # the state of a request: every gla layer's heads x dim x vdim numbers
    want_state = sum(l["mixer"]["heads"] * l["mixer"]["dim"] * l["mixer"]["vdim"]
                     for l in raw["layers"] if l["type"] == "gla")
    assert sum(spec.blocks[c.layer].state_floats() for c in spec.plan) == want_state
    # keys and values are kept once for the layers that share them
    assert [c.cache_from for c in spec.plan] == [l["mixer"].get("kv_from") for l in raw["layers"]]
    # a folder of random weights holds exactly these tensors, and the plain implementation runs on it
    d = str(tmp_path)
    ninfer_amd.write_random_model(d, raw, seed, dtype="float32", std=0.2)
    cfg2, w2 = util.read_folder(d)
    assert set(w2) == set(specs)
    toks = util.random_tokens(30, raw["vocab"], 1)
    logits, streams = plain.forward(cfg2, w2, toks)
    assert logits.shape == (30, raw["vocab"]) and torch.isfinite(logits).all()
    assert streams.shape == (len(raw["layers"]), 30, w)
    # causal: the logits of a prefix are those of the whole
    torch.testing.assert_close(plain.forward(cfg2, w2, toks[:11])[0], logits[:11], atol=1e-12, rtol=0)


def test_config_errors_name_the_key():
    from ninfer_amd.config import ConfigError, FopinexConfig
    good = fopinex_cases.config_odd()
    FopinexConfig.from_dict(good)
    for path, value, word in (
            (("vocab",), None, "vocab"), (("norm", "eps"), 0.0, "norm.eps"),
            (("residual_mult",), None, "residual_mult"),
            (("layers", 0, "type"), "lightning", "type"), (("layers", 0, "mixer", "kv_heads"), 4, "kv_heads"),
            (("layers", 1, "mixer", "tau"), 0.0, "tau"), (("layers", 2, "mixer", "kv_from"), 1, "kv_from"),
            (("layers", 2, "mixer", "kv_from"), 3, "kv_from"), (("layers", 2, "mixer", "dim"), 16, "layer 0"),
            (("layers", 0, "mlp", "kind"), "dense", "kind"), (("layers", 0, "mlp", "router", "top"), 0, "top"),
            (("layers", 0, "mixer", "scale"), None, "scale")):
        raw = copy.deepcopy(good)
        at = raw
        for k in path[:-1]:
            at = at[k]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError) as e:
            FopinexConfig.from_dict(raw)
        assert word in str(e.value), (path, str(e.value))


def test_what_may_be_absent():
    from ninfer_amd.config import FopinexConfig
    cfg = FopinexConfig.from_dict(fopinex_cases.config_ones())
    a = cfg.layers[0]
    assert a.mixer.chunk is None and a.mixer.kv_from is None and a.mlp.identity == 0 and a.mlp.groups == 1
    assert cfg.layers[2].mlp is None and cfg.layers[3].mixer.kv_from == 2
    raw = fopinex_cases.config_odd()
    del raw["layers"][1]["mixer"]["rank"]
    assert FopinexConfig.from_dict(raw).layers[1].mixer.rank is None


def test_the_architecture_key_chooses_the_builder():
    from ninfer_amd.config import FopinexConfig
    cfg, spec = _spec(fopinex_cases.config_even())
    assert isinstance(cfg, FopinexConfig) and len(spec.plan) == 5


# ---- the plain implementation's own properties --------------------------------------------------

def test_plain_chunk_mask():
    m = plain.chunk_mask(7, 3)
    assert m[2].tolist() == [True, True, True, False, False, False, False]
    assert m[3].tolist() == [False, False, False, True, False, False, False]     # a chunk's first row sees itself alone
    assert m[5].tolist() == [False, False, False, True, True, True, False]
    assert plain.chunk_mask(4, None).tolist() == torch.ones(4, 4).tril().bool().tolist()
    assert plain.chunk_mask(3, 1).tolist() == torch.eye(3).bool().tolist()


def _router(scores_logits, correction, **r):
    total = len(correction)
    w = {"p.router": torch.eye(total, dtype=D), "p.correction": torch.tensor(correction, dtype=D)}
    h = torch.log(torch.tensor([scores_logits], dtype=D))      # softmax of log s = s / sum s
    return plain.route(w, "p.", {"router": dict(r)}, h)


def test_plain_routing_rule():
    s = [0.05, 0.30, 0.10, 0.15, 0.25, 0.15]
    # no groups, no correction: the largest scores, which are also the weights
    ids, wts, _ = _router(s, [0.0] * 6, experts=6, top=2)
    assert ids.tolist() == [[1, 4]]
    torch.testing.assert_close(wts, torch.tensor([[0.30, 0.25]], dtype=D))
    # the correction moves the choice and not the weights (a negative choice score still wins
    # over what is not allowed)
    ids, wts, _ = _router(s, [0.5, -0.4, 0.0, 0.0, 0.0, 0.0], experts=6, top=2)
    assert ids.tolist() == [[0, 4]]
    torch.testing.assert_close(wts, torch.tensor([[0.05, 0.25]], dtype=D))
    # three groups of two, one kept: a group's score is its largest choice score
    ids, _, _ = _router(s, [0.0] * 6, experts=4, identity=2, top=2, groups={"count": 3, "keep": 1})
    assert ids.tolist() == [[1, 0]]
    # with every choice score below zero the kept group's experts still come before the others
    ids, _, _ = _router(s, [-1.0] * 6, experts=6, top=2, groups={"count": 3, "keep": 1})
    assert ids.tolist() == [[1, 0]]
    # the last router outputs are identity experts: groups are formed over all of them
    s = [0.05, 0.20, 0.10, 0.15, 0.30, 0.20]
    ids, wts, _ = _router(s, [0.0] * 6, experts=4, identity=2, top=3, groups={"count": 2, "keep": 1})
    assert ids.tolist() == [[4, 5, 3]]
    torch.testing.assert_close(wts.sum(), torch.tensor(0.65, dtype=D))        # not renormalised


def test_plain_identity_experts_return_their_input():
    g = torch.Generator().manual_seed(3)
    width, ff = 6, 4
    w = {"p.router": torch.zeros(3, width, dtype=D), "p.correction": torch.tensor([0.0, 0.0, 1.0], dtype=D)}
    for e in range(2):
        for n, shape in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))):
            w[f"p.e{e}.{n}"] = torch.randn(shape, generator=g, dtype=D)
    h = torch.randn(5, width, generator=g, dtype=D)
    mlp = {"router": {"experts": 2, "identity": 1, "top": 1}, "expert": {"ff": ff, "limit": 1.0}}
    torch.testing.assert_close(plain.moe(w, "p.", mlp, h), h / 3)     # all scores are 1/3
    # the expert: the gate is capped from above alone, the other branch from both sides
    big = {"p.e0.gate": torch.tensor([[5.0], [-5.0]], dtype=D), "p.e0.up": torch.tensor([[9.0], [-9.0]], dtype=D),
           "p.e0.down": torch.eye(2, dtype=D)}
    y = plain.expert(big, "p.e0.", 2.0, torch.ones(1, 1, dtype=D))
    want = [2.0 * torch.sigmoid(torch.tensor(1.702 * 2.0, dtype=D)) * 3.0,
            -5.0 * torch.sigmoid(torch.tensor(1.702 * -5.0, dtype=D)) * -1.0]
    torch.testing.assert_close(y, torch.stack(want)[None])


def test_plain_recurrence_against_its_sum():
    """o_t written out: sum over j <= t of (q_t . (k_j * prod of the decays after j)) v_j."""
    g = torch.Generator().manual_seed(5)
    width, mixer = 10, {"heads": 2, "dim": 3, "vdim": 4, "tau": 2.0}
    w = {"p." + n: torch.randn(shape, generator=g, dtype=D) for n, shape in (
        ("q", (6, width)), ("k", (6, width)), ("v", (8, width)), ("g", (8, width)), ("o", (width, 8)),
        ("a1", (2, width)), ("a2", (6, 2)), ("a2.b", (6,)), ("norm", (4,)))}
    h = torch.randn(9, width, generator=g, dtype=D)
    y, state = plain.gla(w, "p.", mixer, h, 1e-5)
    alpha = plain.gla_decay(w, "p.", mixer, h)
    assert ((alpha > 0) & (alpha < 1)).all()
    z = plain.lin(w, "p.a2", plain.lin(w, "p.a1", h)) + w["p.a2.b"]
    torch.testing.assert_close(alpha.reshape(9, 6), torch.sigmoid(z) ** 0.5)
    q = plain.lin(w, "p.q", h).reshape(9, 2, 3) / math.sqrt(3)
    k = plain.lin(w, "p.k", h).reshape(9, 2, 3)
    v = plain.lin(w, "p.v", h).reshape(9, 2, 4)
    o = torch.zeros(9, 2, 4, dtype=D)
    for t in range(9):
        for j in range(t + 1):
            kd = k[j] * alpha[j + 1:t + 1].prod(0)
            o[t] += (q[t] * kd).sum(-1, keepdim=True) * v[j]
    o = plain.rms(o, 1e-5) * w["p.norm"]
    gate = plain.lin(w, "p.g", h)
    torch.testing.assert_close(y, plain.lin(w, "p.o", o.reshape(9, 8) * gate * torch.sigmoid(gate)))
    # in two pieces, the state handed on
    y1, s1 = plain.gla(w, "p.", mixer, h[:4], 1e-5)
    y2, s2 = plain.gla(w, "p.", mixer, h[4:], 1e-5, state=s1)
    torch.testing.assert_close(torch.cat([y1, y2]), y)
    torch.testing.assert_close(s2, state)


def test_plain_attention_is_not_normalised_and_mixes_heads():
    """One key per row (chunks of 1): the output is sigmoid(score + bias) of every head, mixed
    by the heads' matrix, times the row's own value."""
    g = torch.Generator().manual_seed(9)
    width, mixer = 8, {"heads": 4, "kv_heads": 2, "dim": 3, "vdim": 2, "scale": 0.7, "mask": {"size": 1}}
    w = {"p." + n: torch.randn(shape, generator=g, dtype=D) for n, shape in (
        ("q", (12, width)), ("k", (6, width)), ("v", (4, width)), ("o", (width, 8)), ("pb", (4,)), ("talk", (4, 4)))}
    h = torch.randn(5, width, generator=g, dtype=D)
    kv = plain.keys_values(w, "p.", mixer, h)
    y = plain.sigmoid_attention(w, "p.", mixer, h, kv)
    q = plain.lin(w, "p.q", h).reshape(5, 4, 3)
    k, v = plain.lin(w, "p.k", h).reshape(5, 2, 3), plain.lin(w, "p.v", h).reshape(5, 2, 2)
    wt = torch.stack([torch.sigmoid((q[:, a] * k[:, a // 2]).sum(-1) * 0.7 + w["p.pb"][a]) for a in range(4)], 1)
    mixed = wt @ w["p.talk"].T                                                   # [n, H]
    out = torch.stack([mixed[:, a, None] * v[:, a // 2] for a in range(4)], 1)   # [n, H, vdim]
    torch.testing.assert_close(y, plain.lin(w, "p.o", out.reshape(5, 8)))


# ---- the engine's host logic on the CPU, with plain stand-ins for the kernels ------------------

@pytest.fixture(scope="module", params=["odd", "ones"])
def host_case(request, tmp_path_factory):
    import ninfer_amd
    make, seed = fopinex_cases.CASES[request.param]
    raw = make()
    d = str(tmp_path_factory.mktemp("fopinex_host_" + request.param))
    ninfer_amd.write_random_model(d, raw, seed, dtype="float32", std=0.25)
    cfg, w = util.read_folder(d)
    reqs = {f"r{i}": util.random_tokens(n, raw["vocab"], 20 + i) for i, n in enumerate([33, 1, 12, 47, 20])}
    margins = {k: [] for k in reqs}
    ref = {k: plain.forward(cfg, w, v, margins=margins[k])[0] for k, v in reqs.items()}
    # rows at which a routing decision is a close call are left out of the comparisons
    clear = {k: torch.stack([m > 1e-5 for m in margins[k]]).all(0) if margins[k]
             else torch.ones(len(reqs[k]), dtype=torch.bool) for k in reqs}
    return {"dir": d, "cfg": raw, "reqs": reqs, "ref": ref, "clear": clear}


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
        # a close call at one row changes what that row leaves in cache and state for all later rows
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
    slots for five requests and their repeats: a slot's recurrent state starts at zero for
    every request that takes it."""
    runner = _host_runner(host_case, num_sequences=2, num_pages=26)
    reqs = dict(host_case["reqs"])
    reqs.update({k + "#2": v for k, v in host_case["reqs"].items()})
    _close(host_case, util.run_schedule(runner, util.schedule_mixed(reqs, seed=2, max_live=2)))
    assert runner.cache.pages_reused() > 0
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
            margins = []
            logits = plain.forward(cfg, w, toks, margins=margins)[0][-1]
            top = torch.topk(logits, 2).values
            if top[0] - top[1] < 1e-3 or any(float(m.min()) < 1e-3 for m in margins):
                break
            toks.append(int(logits.argmax()))
        want.append(toks[len(p):])
    runner = _host_runner(host_case, num_sequences=2, prefill_chunk=8, num_pages=14)
    sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
    reqs = [Request(f"q{i}", list(p), SamplingParams.greedy(6)) for i, p in enumerate(prompts)]
    for r in reqs:
        sched.add(r)
    sched.run()
    assert all(r.status == "finished" for r in reqs), [r.error for r in reqs]
    assert [r.output[:len(x)] for r, x in zip(reqs, want)] == want
