"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of Qwen1.5-MoE-A2.7B (24 layers, hidden
2048, 16 heads of 128, 60 experts top-4 of 1408, shared expert 5632, vocabulary
151936) with random bf16 weights generated on the device, a batch of 8
requests and a context of 8192 tokens each (the cache is filled with random
keys and values; token ids are seeded random). A step is one decode step: one
new token for every request of the batch through the engine's step function
(replayed from a captured HIP graph unless --no-graph) and its device sampler. One JSON line is printed: decoded tokens a second as
`value`; the 2,048-token prefill under "prefill"; the decode step's memory
roofline under "roofline" (with the rate of a plain read of HBM measured beside it, and the
step's fraction of that); decode at batch 1 and 64 under "points"; and under
"graph_check" the largest difference between replayed and eager decode steps at
those batches (untimed; 0.0 when the replays are exact).
Peaks: HBM 8 TB/s; dense bf16 MFMA 2.5 PFLOP/s (fp32 157.3 TFLOP/s).

    python bench.py --scenario designs [--sizes small,medium]

is a third measurement, again with a JSON line of its own: Getodra (latent attention and
lightning attention layers with input convolutions and output norms) beside a dense
Qwen2-style model of the same width, depth, heads and feed-forward size, both with random
weights: prompt portions of 512 and 2,048 tokens and decode steps at batch 1, 8 and 64.

    python bench.py --scenario designs --design sosepel [--sizes small,medium] [--only sosepel|sparse]

runs the same measurement for Sosepel (parallel blocks of differential attention and a dense or
sparse feed-forward, a hashed pair embedding, layers that run twice) beside a Qwen2-MoE model of
the same width, heads and experts with as many layers as the other has layer runs.

    python bench.py --scenario designs --design fopinex [--sizes small,medium] [--only fopinex|sparse]

the same for Fopinex (gated parallel blocks of attention without a softmax or gated linear
attention and routed experts beside identity experts) beside a Qwen2-MoE model of the same
width, depth, heads and experts.

    python bench.py --scenario designs --design tuzapel [--sizes small,medium] [--only tuzapel|sparse]

the same for Tuzapel (layer norms before and after every sublayer; latent attention with a
query latent, or windowed attention with a convolution on q, k and v, normed heads, a sink
and layers that read another layer's keys and values; a clamped gated feed-forward, dense or
as routed experts) beside a Qwen2-MoE model of the same width, depth, heads, window and experts.

    python bench.py --scenario long [--model 57b-a14b] [--requests 8] [--prompt 32768] [--new 256]

is another measurement with a JSON line of its own: the scheduler serves
`--requests` concurrent requests with random prompts of `--prompt` tokens,
prefilled in portions of 2,048 tokens interleaved with the decoding of the
others, `--new` tokens each, sampled at temperature 0.7 from fixed seeds.
"""
import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

CONFIG_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 24, "hidden_size": 2048, "num_attention_heads": 16,
    "num_key_value_heads": 16, "head_dim": 128, "intermediate_size": 5632,
    "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632,
    "num_experts": 60, "num_experts_per_tok": 4, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": 151936,
    "rope_theta": 1000000.0, "use_sliding_window": False, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "hidden_act": "silu",
}


CONFIG_D = dict(CONFIG_C, num_hidden_layers=28, hidden_size=3584, num_attention_heads=28,
                num_key_value_heads=4, intermediate_size=18944, moe_intermediate_size=2560,
                shared_expert_intermediate_size=20480, num_experts=64, num_experts_per_tok=8)
MODELS = {"a2.7b": ("Qwen1.5-MoE-A2.7B", CONFIG_C), "57b-a14b": ("Qwen2-57B-A14B", CONFIG_D)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the comparison of replayed with eager decode steps (untimed)")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="length of the timed prefill (the headline figure is at 2,048)")
    ap.add_argument("--graph", dest="graph", action="store_true", default=True,
                    help="decode steps replayed from a captured HIP graph (the default)")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="every decode step launched kernel by kernel")
    ap.add_argument("--model", default="a2.7b", choices=sorted(MODELS),
                    help="layer sizes: a2.7b (the default and the headline) or 57b-a14b")
    ap.add_argument("--profile", action="store_true",
                    help="also time every kind of kernel call of one eager decode step and one "
                         "prefill with device events, with the bytes and flops of each kind, its "
                         "floor and the fraction of it reached (untimed runs of their own; the "
                         "table goes to stderr and under \"profile\")")
    ap.add_argument("--scenario", default="decode", choices=["decode", "long", "designs"])
    ap.add_argument("--sizes", default="small,medium",
                    help="--scenario designs: which of the layer sizes to run (small, medium)")
    ap.add_argument("--design", default="getodra", choices=["getodra", "sosepel", "fopinex", "tuzapel"],
                    help="--scenario designs: the design to run beside the closest model the engine had")
    ap.add_argument("--only", default="", help="--scenario designs: run this one of the two models only")
    ap.add_argument("--requests", type=int, default=8, help="--scenario long: concurrent requests")
    ap.add_argument("--prompt", type=int, default=32768, help="--scenario long: prompt tokens")
    ap.add_argument("--new", type=int, default=256, help="--scenario long: new tokens a request")
    ap.add_argument("--portion", type=int, default=2048,
                    help="--scenario long: the scheduler's token budget of a step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    import ninfer_amd
    from ninfer_amd import Chunk, EngineOptions, random_model
    from ninfer_amd.parts.moe import SparseMoE
    from ninfer_amd.sampling import SampleRow, Sampler, SamplingParams
    from collections import Counter

    model_name, model_cfg = MODELS[args.model]
    raw = dict(model_cfg)
    layers_full = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    L = raw["num_hidden_layers"]
    H, Hq, Hkv, D = raw["hidden_size"], raw["num_attention_heads"], raw["num_key_value_heads"], \
        raw["head_dim"]
    Im, Is, E, k, V = raw["moe_intermediate_size"], raw["shared_expert_intermediate_size"], \
        raw["num_experts"], raw["num_experts_per_tok"], raw["vocab_size"]
    esize = 2 if args.dtype == "bfloat16" else 4
    page = 16
    if args.scenario == "long":
        return long_scenario(args, raw, model_name, layers_full)
    if args.scenario == "designs":
        return designs_scenario(args)
    max_b = args.batch if args.no_points else max(args.batch, 64)
    ctx = args.context
    opt = EngineOptions(dtype=args.dtype, max_context=ctx, prefill_chunk=max(args.prefill_tokens, max_b),
                        num_sequences=max_b, page_size=page, use_graph=args.graph)
    t0 = time.time()
    runner = random_model(raw, 1234, opt)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    for pools in runner.cache.pools.values():   # a cache full of synthetic keys and values
        for pool in pools.values():
            pool.normal_()
    sampler = Sampler(runner.ops, runner.device)
    gen = torch.Generator().manual_seed(7)
    greedy = SamplingParams.greedy()
    moes = [b.feed_forward for b in runner.spec.blocks if isinstance(b.feed_forward, SparseMoE)]

    def decode_run(batch: int, steps: int, warmup: int):
        start = ctx - (steps + warmup) - 1
        slots = [runner.open() for _ in range(batch)]
        for s in slots:                       # positions 0..start-1 count as cached
            runner.cache.reserve(s, start)
            runner.cache.commit(s, start)
        toks = torch.randint(0, V, (batch,), generator=gen).tolist()
        rows = [SampleRow(greedy, Counter(), i, 0, 1) for i in range(batch)]

        def one():
            nonlocal toks
            logits = runner.step([Chunk(s, [t], [0]) for s, t in zip(slots, toks)])
            toks = sampler.sample(logits, rows)

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / steps
        distinct = [int(torch.unique(m.last_ids).numel()) for m in moes if m.last_ids is not None]
        for s in slots:
            runner.close(s)
        n_exp = sum(distinct) / max(len(distinct), 1)
        per_layer = ((Hq + 2 * Hkv) * D * H + H * Hq * D + E * H + n_exp * 3 * Im * H
                     + 3 * Is * H + H) * esize
        kv = batch * 2 * L * Hkv * D * (ctx - steps / 2) * esize
        nbytes = L * per_layer + V * H * esize + kv
        return dt, nbytes, n_exp

    def prefill_run(T: int, reps: int):
        toks = torch.randint(0, V, (T,), generator=gen).tolist()
        times = []
        for _ in range(reps + 2):
            s = runner.open()
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.step([Chunk(s, toks, [T - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.close(s)
        dt = sorted(times[2:])[len(times[2:]) // 2]
        print(f"[bench] prefill of {T} tokens, ms: " + " ".join(f"{x * 1e3:.2f}" for x in times)
              + " (the first two are warm-up; the median of the rest counts)", file=sys.stderr, flush=True)
        flops = T * 2 * L * ((Hq + 2 * Hkv) * D * H + Hq * D * H + E * H + k * 3 * Im * H
                             + 3 * Is * H + H) + L * 2 * Hq * D * T * T + 2 * V * H
        return dt, flops

    def graph_check(batch: int) -> float:
        """Replayed steps against the same steps launched kernel by kernel, at this batch (so
        with the same library products inside the graph): `batch` requests with a real
        64-token prompt each, then four decode steps of fixed tokens, once with replays and
        once with the graphs forgotten before every step (the first step of a shape runs
        eagerly, under the same context bound as its graph), with an eager step of another
        shape between the replays. Largest difference of any logit (0.0: replays are exact)."""
        prompts = [torch.randint(0, V, (64,), generator=gen).tolist() for _ in range(batch)]
        feed = [torch.randint(0, V, (batch,), generator=gen).tolist() for _ in range(4)]
        outs = []
        for replay in (True, False):
            runner._graphs.clear()
            slots = [runner.open() for _ in range(batch)]
            for i in range(0, batch, 16):
                runner.step([Chunk(s, p, []) for s, p in zip(slots[i:i + 16], prompts[i:i + 16])])
            got = []
            for n, toks in enumerate(feed):
                if not replay:
                    runner._graphs.clear()
                logits = runner.step([Chunk(s, [t], [0]) for s, t in zip(slots, toks)])
                got.append(logits.float().clone())
                if n == 1 and batch < max_b:
                    extra = runner.open()
                    runner.step([Chunk(extra, prompts[0][:9], [8])])
                    runner.close(extra)
            outs.append(got)
            for s in slots:
                runner.close(s)
        runner._graphs.clear()
        return max(float((a - b).abs().max()) for a, b in zip(*outs))

    def call_cost(name, a, kw):
        """What one call of the kernel library has to move and to compute, from its own
        arguments: a function, evaluated after the step (it may read device tensors such as
        the experts' offsets), that returns (bytes, flops). Bytes: every operand read once and
        every result written once (weights of experts that got rows only; the cached keys and
        values a request's rows can see, once per request); flops: two per multiply-add."""
        def nbytes(*ts):
            return sum(t.numel() * t.element_size() for t in ts if t is not None)

        def product(x_rows, x, w_rows, w, out_rows, out_cols, out):
            k_ = x.shape[1]
            return (x_rows * k_ * x.element_size() + w_rows * k_ * w.element_size()
                    + out_rows * out_cols * out.element_size(), 2.0 * x_rows * w_rows * k_)

        def grouped(x, w, offsets, n_rows, out):
            def cost():
                counts = (offsets[1:] - offsets[:-1]).cpu()
                used = int((counts > 0).sum())
                per_expert = w.shape[1] * w.shape[2]
                return (used * per_expert * w.element_size() + n_rows * x.shape[1] * x.element_size()
                        + nbytes(out), 2.0 * n_rows * per_expert)
            return cost

        if name == "linear":
            x, w, out = a[0], a[1], a[2]
            return lambda: product(x.shape[0], x, w.shape[0], w, out.shape[0], out.shape[1], out)
        if name == "swiglu_linear":
            x, w, out = a[0], a[1], a[2]
            return lambda: product(x.shape[0], x, w.shape[0], w, out.shape[0], out.shape[1], out)
        if name == "qkv_rope":
            x, w, qkv = a[0], a[1], a[3]
            return lambda: product(x.shape[0], x, w.shape[0], w, qkv.shape[0], qkv.shape[1], qkv)
        if name == "grouped_swiglu":
            return grouped(a[0], a[1], a[2], a[3].shape[0], a[5])
        if name == "grouped_down":
            return grouped(a[0], a[1], a[2], a[3].shape[0], a[4])
        if name == "paged_attention":
            qkv, k_pool, sctx, n_q, n_kv, d, window = a[0], a[1], a[4], a[5], a[6], a[7], a[9]
            out = kw.get("out", a[11] if len(a) > 11 else None)

            def cost():
                pos = sctx.positions.cpu().tolist()
                seq = sctx.row_seq.cpu().tolist()
                seen = [min(p + 1, window) if window else p + 1 for p in pos]
                keys = {}
                for s_, p, n_ in zip(seq, pos, seen):     # keys a request's rows see, all told
                    lo, hi = keys.get(s_, (p - n_ + 1, p))
                    keys[s_] = (min(lo, p - n_ + 1), max(hi, p))
                kv = sum(hi - lo + 1 for lo, hi in keys.values()) * 2 * n_kv * d * k_pool.element_size()
                return (kv + len(pos) * n_q * d * qkv.element_size() + nbytes(out),
                        4.0 * n_q * d * sum(seen))
            return cost
        if name == "rmsnorm":
            x, out = a[0], a[3]
            rs = kw.get("rows_sum")
            extra = nbytes(kw.get("delta")) + (nbytes(rs.y, rs.shared) if rs is not None else 0)
            touched = out.shape[0] * x.shape[1] * 4
            return lambda: (2 * touched + nbytes(out) + extra, 0.0)   # residual read and written
        if name == "_launch_held":
            def cost():
                total_b = total_f = 0.0
                for g, keep in a[0]:
                    x, w, out, offsets = keep[0], keep[1], keep[2], keep[4]
                    w_rows = g.N * (2 if g.epilogue else 1)
                    if offsets is None:
                        b_, f_ = product(g.M, x, w_rows, w, g.M, g.N, out)
                    else:
                        counts = (offsets[1:] - offsets[:-1]).cpu()
                        used = int((counts > 0).sum())
                        b_ = (used * w_rows * g.K * w.element_size() + g.M * g.K * x.element_size()
                              + g.M * g.N * out.element_size())
                        f_ = 2.0 * g.M * w_rows * g.K
                    total_b += b_
                    total_f += f_
                return total_b, total_f
            return cost
        tensors = [t for t in list(a) + list(kw.values()) if isinstance(t, torch.Tensor)]
        if name in ("embed",):      # a gather: the rows read, not the table
            return lambda: (2 * nbytes(a[2]), 0.0)
        if name in ("rope_kv_write",):   # q and k rotated in place, k and v written to pages
            return lambda: (2 * nbytes(a[0]), 0.0)
        return lambda: (nbytes(*[t for t in tensors if t.numel() < (1 << 28)]), 0.0)

    def profile_calls(label: str, chunks) -> dict:
        """One eager step by kind of kernel call: microseconds (every call of the kernel
        library is bracketed by device events; calls inside `together()` are launched when it
        ends and are timed there, as one kind), the bytes and flops the calls have to move
        and compute (`call_cost`), their floor max(bytes / 8 TB/s, flops / peak) and the
        fraction floor / time; the floors add up to the step's. Everything runs on one stream
        here (a long portion's shared expert otherwise runs beside the routed path, and times
        would overlap). The reference prints its table of times per phase
        (src/models/model.hip:1066-1081)."""
        ops = runner.ops
        spans = []
        one_stream, ops.beside_min_rows = ops.beside_min_rows, 1 << 30

        def kind(name, a):
            if name in ("linear", "swiglu_linear"):
                return f"{name} {a[0].shape[0]}x{a[1].shape[1]}->{a[2].shape[1]}"
            if name in ("grouped_swiglu", "grouped_down"):
                return f"{name} {a[0].shape[0]} rows"
            return name

        names = ["embed", "rmsnorm", "qkv_rope", "rope_kv_write", "paged_attention", "linear",
                 "swiglu_linear", "grouped_swiglu", "grouped_down", "moe_route",
                 "moe_combine", "_launch_held"]
        saved = {n: getattr(ops, n) for n in names}

        depth = [0]

        def wrap(n):
            def call(*a, **kw):
                if depth[0]:
                    return saved[n](*a, **kw)       # part of a call that is timed
                # inside `together()` a call is either held back (it is launched, and timed,
                # when the block ends) or runs at once (the vendor library's products do)
                waiting = (len(ops._held), ops._held_route) if ops._held is not None else None
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                cost = call_cost(n, a, kw)
                s.record()
                depth[0] += 1
                try:
                    out = saved[n](*a, **kw)
                finally:
                    depth[0] -= 1
                e.record()
                if waiting is not None and ops._held is not None \
                        and (len(ops._held), ops._held_route) != waiting:
                    return out                      # held back
                spans.append(("products launched together" if n == "_launch_held" else kind(n, a),
                              s, e, cost))
                return out
            return call

        use_graph, runner.options.use_graph = runner.options.use_graph, False
        try:
            for n in names:
                setattr(ops, n, wrap(n))
            runner.step(chunks)
            torch.cuda.synchronize()
        finally:
            for n in names:
                setattr(ops, n, saved[n])
            runner.options.use_graph = use_graph
            ops.beside_min_rows = one_stream
        peak = FLOP_PEAK[args.dtype]
        table = {}
        for k_, s, e, cost in spans:
            b_, f_ = cost()
            row = table.setdefault(k_, [0, 0.0, 0.0, 0.0, 0.0])
            row[0] += 1
            row[1] += s.elapsed_time(e) * 1e3
            row[2] += b_
            row[3] += f_
            row[4] += max(b_ / HBM_PEAK, f_ / peak) * 1e6
        total = sum(r[1] for r in table.values())
        floor = sum(r[4] for r in table.values())
        print(f"[bench] {label}: {total:.0f} us in kernel calls (eager, with event overhead); "
              f"floor {floor:.0f} us = {floor / total:.3f} of it", file=sys.stderr)
        print(f"[bench]   {'us':>9} {'%':>5} {'calls':>5} {'MB':>9} {'GFLOP':>9} {'floor us':>9} "
              f"{'frac':>5}  kind", file=sys.stderr)
        for k_, (calls, us, b_, f_, fl) in sorted(table.items(), key=lambda kv: -kv[1][1]):
            print(f"[bench]   {us:9.1f} {100 * us / total:5.1f} {calls:5d} {b_ / 1e6:9.1f} "
                  f"{f_ / 1e9:9.1f} {fl:9.1f} {fl / us:5.2f}  {k_}", file=sys.stderr)
        out = {k_: {"us": round(us, 1), "mb": round(b_ / 1e6, 1), "gflop": round(f_ / 1e9, 1),
                    "floor_us": round(fl, 1), "frac": round(fl / us, 3)}
               for k_, (_, us, b_, f_, fl) in table.items()}
        out["step"] = {"us": round(total, 1), "floor_us": round(floor, 1),
                       "frac": round(floor / total, 3)}
        return out

    def read_rate() -> float:
        """Bytes a second at which a kernel that only reads streams 4 GiB from HBM (the
        library's read probe: 16-byte non-temporal loads, nothing written): what the memory
        system gives a decode step's weights and cache at best."""
        src = torch.empty(1 << 30, dtype=torch.float32, device=runner.device).normal_()
        for _ in range(2):
            runner.ops.read_probe(src)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(5):
            runner.ops.read_probe(src)
        torch.cuda.synchronize()
        return 5 * src.numel() * 4 / (time.perf_counter() - t)

    dt, nbytes, n_exp = decode_run(args.batch, args.steps, args.warmup)
    result = {
        "metric": f"decode tok/s at batch {args.batch} ({model_name} shapes, context {ctx})",
        "value": round(args.batch / dt, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"{model_name} shapes, random weights", "global_batch": args.batch,
                   "seq_len": ctx, "parallelism": "single GPU", "layers": L,
                   "layers_full": layers_full, "hidden": H, "heads": Hq, "kv_heads": Hkv,
                   "head_dim": D, "moe_intermediate": Im, "shared_intermediate": Is,
                   "intermediate": raw["intermediate_size"], "experts": E, "top_k": k, "vocab": V,
                   "page_size": page, "graph": bool(args.graph)},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / dt / 1e9, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(nbytes / dt / HBM_PEAK, 4),
                     "distinct_experts_per_layer": round(n_exp, 1)},
    }
    plain_read = read_rate()
    result["roofline"]["measured_read"] = round(plain_read / 1e9, 1)
    result["roofline"]["frac_of_read"] = round(nbytes / dt / plain_read, 4)
    if not args.no_prefill:
        pt = min(args.prefill_tokens, ctx)
        pdt, flops = prefill_run(pt, 5)
        result["prefill"] = {"value": round(pt / pdt, 1), "tokens": pt,
                             "ms": round(pdt * 1e3, 3),
                             "frac": round(flops / pdt / FLOP_PEAK[args.dtype], 4)}
    if not args.no_points:
        points, fracs = {}, {}
        for b in (1, 64):
            steps = max(8, args.steps // (4 if b == 64 else 1))
            d, nb, _ = decode_run(b, steps, max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b / d, 2)
            fracs[f"decode_b{b}"] = round(nb / d / HBM_PEAK, 4)
        result["points"] = points
        result["points_hbm_frac"] = fracs   # the same roofline as the default step's, per point
    if args.profile:
        slots = [runner.open() for _ in range(args.batch)]
        for sl in slots:
            runner.cache.reserve(sl, ctx - 2)
            runner.cache.commit(sl, ctx - 2)
        toks = torch.randint(0, V, (args.batch,), generator=gen).tolist()
        step = [Chunk(sl, [t], [0]) for sl, t in zip(slots, toks)]
        profile_calls("warm-up", step)
        result["profile"] = {"decode": profile_calls(f"decode step, batch {args.batch}", step)}
        for sl in slots:
            runner.close(sl)
        pt = min(args.prefill_tokens, ctx)
        ptoks = torch.randint(0, V, (pt,), generator=gen).tolist()
        for label in ("warm-up", f"prefill of {pt} tokens"):
            sl = runner.open()
            table = profile_calls(label, [Chunk(sl, ptoks, [pt - 1])])
            runner.close(sl)
        result["profile"]["prefill"] = table
    if args.graph and not args.no_check:
        batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
        worst = max(graph_check(b) for b in batches)
        result["graph_check"] = {"batches": batches, "max_abs_diff": worst}
        if worst != 0.0:
            print(f"[bench] WARNING: replayed steps differ from eager steps by {worst}",
                  file=sys.stderr, flush=True)
    print(json.dumps(result), flush=True)
    return 0


DESIGN_SIZES = {
    # width, feed-forward, layers, heads, head size (attention: unrotated + rotated = head), latent
    "small": dict(width=1024, ff=2816, layers=8, heads=8, head=128, rot=32, vdim=64, rank=256,
                  vocab=32000, positions=4096),
    "medium": dict(width=2048, ff=5632, layers=8, heads=16, head=128, rot=64, vdim=128, rank=512,
                   vocab=32000, positions=4096),
}


def getodra_config(z: dict) -> dict:
    """Three latent-attention layers to one lightning layer, the first latent layer of each
    four run twice with its own cache (as the design's `weights_of` allows)."""
    latent = {"heads": z["heads"], "dim": z["head"] - z["rot"], "rot_dim": z["rot"],
              "vdim": z["vdim"], "kv_rank": z["rank"], "scale": z["head"] ** -0.5,
              "rot": {"base": 10000.0, "dims": z["rot"],
                      "scaling": {"factor": 8.0, "original": 1024, "fast": 16.0, "slow": 2.0}}}
    lightning = {"heads": z["heads"], "dim": z["head"], "vdim": z["vdim"],
                 "decay": [1.0 - 2.0 ** -(3 + 5 * h / max(z["heads"] - 1, 1)) for h in range(z["heads"])]}
    mlp = {"kind": "dense", "ff": z["ff"]}
    layers = []
    for i in range(z["layers"]):
        if i % 4 == 0:
            layers.append({"type": "lightning", "mixer": lightning, "mlp": mlp})
        elif i % 4 == 2:
            layers.append({"type": "latent_attention", "mixer": latent, "mlp": mlp, "weights_of": i - 1})
        else:
            layers.append({"type": "latent_attention", "mixer": latent, "mlp": mlp})
    return {"architecture": "Getodra", "vocab": z["vocab"], "width": z["width"],
            "max_positions": z["positions"], "norm": {"eps": 1e-5}, "canon": {"taps": 4},
            "layers": layers}


def dense_config(z: dict) -> dict:
    """The closest model the engine had before: pre-norm blocks of rotary attention (as many
    heads of the same size, each with keys and values of its own) and a gated feed-forward."""
    return dict(CONFIG_C, num_hidden_layers=z["layers"], hidden_size=z["width"],
                num_attention_heads=z["heads"], num_key_value_heads=z["heads"], head_dim=z["head"],
                intermediate_size=z["ff"], num_experts=0, num_experts_per_tok=0,
                moe_intermediate_size=0, shared_expert_intermediate_size=0, vocab_size=z["vocab"],
                hidden_act="gelu_pytorch_tanh")


SOSEPEL_SIZES = {
    # width, dense feed-forward, layers (layers 1 .. layers - 2 run twice), query and kv heads,
    # sizes of a map's query and key and of a value, experts
    "small": dict(width=1024, ff=2816, layers=5, heads=8, kv_heads=2, dim=64, vdim=128, experts=16,
                  top=2, groups=(4, 2), expert_ff=704, shared_ff=1408, vocab=32000, positions=4096),
    "medium": dict(width=2048, ff=5632, layers=6, heads=16, kv_heads=4, dim=64, vdim=128, experts=32,
                   top=4, groups=(4, 2), expert_ff=1408, shared_ff=2816, vocab=32000, positions=4096),
}


def sosepel_config(z: dict) -> dict:
    """A dense first layer, then sparse ones; the layers between the first and the last run
    twice, each run with a cache of its own."""
    mixer = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"],
             "diff": 0.5, "scale": z["dim"] ** -0.5, "softcap": 30.0, "q_temp": {"coef": 0.25, "every": 128}}
    moe = {"kind": "moe", "expert": {"ff": z["expert_ff"]}, "shared": {"ff": z["shared_ff"]},
           "router": {"experts": z["experts"], "top": z["top"],
                      "groups": {"count": z["groups"][0], "keep": z["groups"][1]}}}
    layers = [{"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": z["ff"]}}]
    layers += [{"type": "attention", "mixer": mixer, "mlp": moe} for _ in range(z["layers"] - 1)]
    return {"architecture": "Sosepel", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
            "logit_softcap": 20.0, "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 31,
                                                                         "mul_cur": 3}},
            "layers": layers, "loop": {"start": 1, "stop": z["layers"] - 1, "times": 2}}


def sosepel_runs(z: dict) -> int:
    return 2 * z["layers"] - 2


def sparse_config(z: dict) -> dict:
    """The closest model the engine had: Qwen2-MoE blocks (rotary attention with as many query
    and kv heads, heads of 2 x dim; routed experts beside a gated shared expert) of the same
    width, as many layers as the other model has layer runs, the first one dense."""
    return dict(CONFIG_C, num_hidden_layers=sosepel_runs(z), hidden_size=z["width"],
                num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"], head_dim=2 * z["dim"],
                intermediate_size=z["ff"], num_experts=z["experts"], num_experts_per_tok=z["top"],
                moe_intermediate_size=z["expert_ff"], shared_expert_intermediate_size=z["shared_ff"],
                mlp_only_layers=[0], decoder_sparse_step=1, vocab_size=z["vocab"], hidden_act="silu",
                use_sliding_window=False)


FOPINEX_SIZES = {
    # width, layers (of every four: attention, gated linear attention, attention on the first
    # one's keys and values, attention), query and kv heads, sizes of a key and a value, the
    # chunk of positions a row sees, the recurrence's heads and sizes, experts
    "small": dict(width=1024, layers=8, heads=8, kv_heads=2, dim=128, vdim=128, chunk=1024,
                  gla_heads=8, gla_dim=64, gla_vdim=128, rank=32, experts=16, identity=2, top=2,
                  groups=(3, 2), expert_ff=704, vocab=32000, positions=4096),
    "medium": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, vdim=128, chunk=1024,
                   gla_heads=16, gla_dim=64, gla_vdim=128, rank=64, experts=32, identity=4, top=4,
                   groups=(4, 2), expert_ff=1408, vocab=32000, positions=4096),
}


def fopinex_config(z: dict) -> dict:
    attention = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"],
                 "scale": z["dim"] ** -0.5, "mask": {"size": z["chunk"]}}
    gla = {"heads": z["gla_heads"], "dim": z["gla_dim"], "vdim": z["gla_vdim"], "tau": 8.0,
           "rank": z["rank"]}
    moe = {"kind": "moe", "expert": {"ff": z["expert_ff"], "limit": 7.0},
           "router": {"experts": z["experts"], "identity": z["identity"], "top": z["top"],
                      "groups": {"count": z["groups"][0], "keep": z["groups"][1]}}}
    layers = []
    for i in range(z["layers"]):
        if i % 4 == 1:
            layers.append({"type": "gla", "mixer": gla, "mlp": moe})
        elif i % 4 == 2:
            layers.append({"type": "attention", "mixer": dict(attention, kv_from=i - 2), "mlp": moe})
        else:
            layers.append({"type": "attention", "mixer": attention, "mlp": moe})
    return {"architecture": "Fopinex", "vocab": z["vocab"], "width": z["width"],
            "norm": {"eps": 1e-6}, "residual_mult": 0.7, "layers": layers}


def sparse_for_fopinex_config(z: dict) -> dict:
    """The closest model the engine had: Qwen2-MoE blocks (rotary attention with as many query
    and kv heads of the same size, as many routed experts of the same size, no shared expert)
    of the same width and depth."""
    return dict(CONFIG_C, num_hidden_layers=z["layers"], hidden_size=z["width"],
                num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"], head_dim=z["dim"],
                intermediate_size=z["expert_ff"], num_experts=z["experts"],
                num_experts_per_tok=z["top"], moe_intermediate_size=z["expert_ff"],
                shared_expert_intermediate_size=0, mlp_only_layers=[], decoder_sparse_step=1,
                vocab_size=z["vocab"], hidden_act="silu", use_sliding_window=False)


TUZAPEL_SIZES = {
    # width, layers (of every four: latent attention, windowed attention, windowed attention on
    # the layer before's keys and values, windowed attention; feed-forwards in turn routed and
    # dense), query and kv heads, sizes of a key and a value, window, taps, the latent
    # attention's sizes, experts
    "small": dict(width=1024, layers=8, heads=8, kv_heads=2, dim=128, vdim=128, window=1024, taps=4,
                  lat_dim=96, lat_rot=32, lat_vdim=64, rank=256, q_rank=384, ff=2816, experts=16,
                  top=2, expert_ff=704, vocab=32000, positions=4096),
    "medium": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, vdim=128, window=1024, taps=4,
                   lat_dim=64, lat_rot=64, lat_vdim=128, rank=512, q_rank=768, ff=5632, experts=32,
                   top=4, expert_ff=1408, vocab=32000, positions=4096),
}


def tuzapel_config(z: dict) -> dict:
    rot = {"base": 500000.0, "dims": z["dim"] // 2,
           "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 2048}}
    attention = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"],
                 "scale": z["dim"] ** -0.5, "conv": z["taps"], "mask": {"size": z["window"]}, "rot": rot}
    latent = {"heads": z["heads"], "dim": z["lat_dim"], "rot_dim": z["lat_rot"], "vdim": z["lat_vdim"],
              "kv_rank": z["rank"], "q_rank": z["q_rank"], "scale": (z["lat_dim"] + z["lat_rot"]) ** -0.5,
              "rot": {"base": 10000.0, "dims": z["lat_rot"]}}
    moe = {"kind": "moe", "expert": {"ff": z["expert_ff"], "limit": 7.0},
           "router": {"experts": z["experts"], "top": z["top"]}}
    dense = {"kind": "dense", "ff": z["ff"], "limit": 7.0}
    layers = []
    for i in range(z["layers"]):
        mlp = moe if i % 2 else dense
        if i % 4 == 0:
            layers.append({"type": "latent_attention", "mixer": latent, "mlp": mlp})
        elif i % 4 == 2:
            layers.append({"type": "attention", "mixer": dict(attention, kv_from=i - 1), "mlp": mlp})
        else:
            layers.append({"type": "attention", "mixer": attention, "mlp": mlp})
    return {"architecture": "Tuzapel", "vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
            "logit_softcap": 30.0, "layers": layers}


def sparse_for_tuzapel_config(z: dict) -> dict:
    """The closest model the engine had: Qwen2-MoE blocks (rotary attention with as many query
    and kv heads of the same size behind the same window, routed experts of the same size on the
    same layers and a dense feed-forward on the others, no shared expert) of the same width and
    depth."""
    return dict(CONFIG_C, num_hidden_layers=z["layers"], hidden_size=z["width"],
                num_attention_heads=z["heads"], num_key_value_heads=z["kv_heads"], head_dim=z["dim"],
                intermediate_size=z["ff"], num_experts=z["experts"], num_experts_per_tok=z["top"],
                moe_intermediate_size=z["expert_ff"], shared_expert_intermediate_size=0,
                mlp_only_layers=[i for i in range(z["layers"]) if i % 2 == 0], decoder_sparse_step=1,
                vocab_size=z["vocab"], hidden_act="silu", use_sliding_window=True,
                sliding_window=z["window"], max_window_layers=0)


def designs_scenario(args) -> int:
    import torch
    from ninfer_amd import Chunk, EngineOptions, random_model
    sosepel = args.design == "sosepel"
    tuzapel = args.design == "tuzapel"

    gen = torch.Generator().manual_seed(11)
    fopinex = args.design == "fopinex"
    out = {"metric": "prefill and decode throughput, " + ("Sosepel beside a Qwen2-MoE model" if sosepel
                     else "Fopinex beside a Qwen2-MoE model" if fopinex
                     else "Tuzapel beside a Qwen2-MoE model" if tuzapel
                     else "Getodra beside a dense model") + " of equal size",
           "unit": "tok/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic", "sizes": {}}
    for size in args.sizes.split(","):
        z = (SOSEPEL_SIZES if sosepel else FOPINEX_SIZES if fopinex else TUZAPEL_SIZES if tuzapel
             else DESIGN_SIZES)[size]
        ctx = z["positions"]
        row = {"shape": z}
        pairs = (("sosepel", sosepel_config(z)), ("sparse", sparse_config(z))) if sosepel else \
            (("fopinex", fopinex_config(z)), ("sparse", sparse_for_fopinex_config(z))) if fopinex else \
            (("tuzapel", tuzapel_config(z)), ("sparse", sparse_for_tuzapel_config(z))) if tuzapel else \
            (("getodra", getodra_config(z)), ("dense", dense_config(z)))
        for name, raw in pairs:
            if args.only and name != args.only:
                continue
            opt = EngineOptions(dtype=args.dtype, max_context=ctx, prefill_chunk=2048,
                                num_sequences=64, page_size=16, use_graph=args.graph)
            runner = random_model(raw, 99, opt)
            for pools in runner.cache.pools.values():
                for pool in pools.values():
                    pool.normal_()
            res = {}
            for T in (512, 2048):
                toks = torch.randint(0, z["vocab"], (T,), generator=gen).tolist()
                times = []
                for _ in range(5):
                    s = runner.open()
                    torch.cuda.synchronize()
                    t = time.perf_counter()
                    runner.step([Chunk(s, toks, [T - 1])])
                    torch.cuda.synchronize()
                    times.append(time.perf_counter() - t)
                    runner.close(s)
                dt = sorted(times[2:])[1]
                res[f"prefill_{T}"] = {"tok_s": round(T / dt, 1), "ms": round(dt * 1e3, 3)}
            steps, warm = max(8, args.steps // 2), 4
            for batch in (1, 8, 64):
                start = ctx - steps - warm - 1
                slots = [runner.open() for _ in range(batch)]
                for s in slots:
                    runner.cache.reserve(s, start)
                    runner.cache.commit(s, start)
                toks = torch.randint(0, z["vocab"], (batch,), generator=gen).tolist()
                for i in range(steps + warm):
                    if i == warm:
                        torch.cuda.synchronize()
                        t = time.perf_counter()
                    runner.step([Chunk(s, [tk], [0]) for s, tk in zip(slots, toks)])
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t) / steps
                for s in slots:
                    runner.close(s)
                res[f"decode_b{batch}_ctx{ctx}"] = {"tok_s": round(batch / dt, 1),
                                                    "ms_per_step": round(dt * 1e3, 4)}
            res["kv_bytes_per_token"] = runner.cache.kv_bytes_per_token(2 if args.dtype == "bfloat16" else 4)
            res["state_bytes_per_request"] = runner.cache.state_bytes_per_request()
            row[name] = res
            print(f"[bench] {size} {name}: {json.dumps(res)}", file=sys.stderr, flush=True)
            runner.release()
            del runner
            torch.cuda.empty_cache()
        out["sizes"][size] = row
    print(json.dumps(out), flush=True)
    return 0


def long_scenario(args, raw, model_name, layers_full) -> int:
    """Long prompts through the scheduler: portions of prompts beside decode tokens."""
    import torch
    from ninfer_amd import EngineOptions, Request, Scheduler, random_model
    from ninfer_amd.sampling import Sampler, SamplingParams

    n, plen, new = args.requests, args.prompt, args.new
    page, chunk = 16, args.portion
    ctx = -(-(plen + new) // page) * page
    opt = EngineOptions(dtype=args.dtype, max_context=ctx, prefill_chunk=chunk, num_sequences=n,
                        page_size=page, use_graph=args.graph)
    t0 = time.time()
    runner = random_model(raw, 1234, opt)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    sampler = Sampler(runner.ops, runner.device)
    gen = torch.Generator().manual_seed(11)
    V = raw["vocab_size"]

    def serve(n_req, prompt_len, new_tokens):
        sched = Scheduler(runner, sampler, max_batch_tokens=chunk, max_seqs=n_req)
        reqs = [Request(id=f"r{i}", prompt=torch.randint(0, V, (prompt_len,), generator=gen).tolist(),
                        params=SamplingParams(temperature=0.7, seed=100 + i, max_new_tokens=new_tokens))
                for i in range(n_req)]
        for r in reqs:
            sched.add(r)
        torch.cuda.synchronize()
        t = time.perf_counter()
        last = t
        while sched.has_work():
            sched.step()
            if time.perf_counter() - last > 20:
                last = time.perf_counter()
                fed = sum(r.cached for r in reqs if r.status == "running")
                print(f"[bench] step {sched.steps}: {fed} tokens cached by running requests, "
                      f"{len(sched.finished)} finished", file=sys.stderr, flush=True)
        torch.cuda.synchronize()
        return time.perf_counter() - t, sched, reqs

    serve(min(n, 2), 3 * chunk // 2, 4)                     # warm-up: every kind of step once
    dt, sched, reqs = serve(n, plen, new)
    generated = sum(len(r.output) for r in reqs)
    failed = [r.id for r in reqs if r.status != "finished"]
    print(json.dumps({
        "metric": f"long-context serving ({model_name} shapes): {n} x {plen}-token prompts in "
                  f"{chunk}-token portions interleaved with decode, {new} new tokens each",
        "value": round((n * plen + generated) / dt, 1), "unit": "tok/s (prompt + generated)",
        "seconds": round(dt, 3), "steps": sched.steps,
        "prompt_tokens": n * plen, "generated_tokens": generated,
        "preemptions": sum(r.preemptions for r in reqs), "failed": failed,
        "n_gpus": 1, "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic", "config": {"model": f"{model_name} shapes, random weights",
                                        "layers": raw["num_hidden_layers"], "layers_full": layers_full,
                                        "requests": n, "prompt": plen, "new_tokens": new,
                                        "portion": chunk, "page_size": page, "temperature": 0.7,
                                        "graph": bool(args.graph)}}), flush=True)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
