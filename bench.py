#!/usr/bin/env python3
"""Headline benchmark of the MoE-layer path on one MI355X.

Workload (BASELINE.json configs[4]): decode through a 48-layer MoE stack at the stand-in
scale -- hidden 3072, 512 experts, top-10, expert intermediate 1024, affine Q4 group 64,
about 130 GB of expert records resident in HBM -- at decode batch 1.  Every layer's router
has its own seed and Zipf(1.1)-skewed expert offsets.  A step is one token batch through
all 48 layers: ONE launch of the persistent decode kernel.  Inputs are resident in HBM
before the timed region; timing uses HIP events on the stream the kernel runs on.

Prints one JSON line.  `roofline.achieved` = algorithmic bytes of one launch (router +
shared gate + distinct routed records + shared record + activations, summed over the 48
layers) / average launch duration.  `cpu_baseline` = the CPU oracle (a restatement of the
reference arithmetic; the reference has no CPU path of its own) on a bounded sample of the
same workload, on this box's host cores.  `other_configs` holds, timed in the same run: the same stack with the
guessing switched off, at decode batch 8 and 64, and the 2048-token prefill layer -- each with its time per step, tokens/s
and its own fraction of the roofline that bounds it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
# HBM bytes per launch of the default workload (48 layers, batch 1): counters cannot be read from inside this process, so
# the figure comes from two rocprofv3 --pmc runs of this program (FETCH_SIZE, then WRITE_SIZE, each with --calibrate) whose
# CSV output `bench.py --traffic-from <fetch dir> <write dir>` turns into this tracked file.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_stack_kernel_F48_batch1_traffic.json")
INPUTS = 8   # distinct token batches the timed steps cycle through
sys.path.insert(0, ROOT)


def single_layer(ctx, name, tokens, prefill, reps, warmup=3, skew=("zipf", 1.1)):
    """One MoE layer of a single-layer configuration (hidden 2048, 512 experts, top-10, intermediate 512), timed with
    weights and inputs resident.  FLOP count: 2 * tokens * hidden * intermediate * 3 projections * (top-k + shared)
    + the router product."""
    from zerocool_amd import workload
    c = workload.config(name)
    lw = workload.LayerWeights(ctx, c, workload.BASE_SEED + 77, skew)
    x = workload.hidden_rows(ctx, tokens, c.hidden, workload.BASE_SEED + 78 + tokens)
    out = ctx.alloc(tokens * c.hidden * 4)
    ws = ctx.alloc(ctx.moe_prefill_workspace_bytes(c, tokens) if prefill else ctx.moe_workspace_bytes(c, tokens))
    step = ctx.moe_prefill if prefill else ctx.moe_forward
    for _ in range(warmup):
        step(c, lw.layer, x, tokens, out, ws)
    ctx.finish(); ctx.moe_check()
    ctx.timer_start()
    for _ in range(reps):
        step(c, lw.layer, x, tokens, out, ws)
    ms_layer = ctx.timer_stop() / reps
    for b in (x, out, ws, lw.router, lw.shared_gate, lw.shared_record, lw.records):
        ctx.free(b)
    flops = 2.0 * tokens * c.hidden * c.inter * 3 * (c.topk + 1) + 2.0 * tokens * c.hidden * c.experts
    return {"tokens": tokens, "us_per_layer": ms_layer * 1e3, "tokens_per_s": tokens / (ms_layer * 1e-3),
            "TFLOPs": flops / (ms_layer * 1e-3) / 1e12, "router_skew": list(skew) if skew else None,
            "path": "bf16 matrix-core prefill" if prefill else "exact operator path"}


def write_traffic_file(fetch_dir, write_dir):
    """Turns the CSV output of the two counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE --output-format csv, each over
    `bench.py --no-cpu --calibrate`) into the tracked traffic file: per-dispatch averages of the decode kernel in KiB, each
    scaled by what the same counter reads for the 1 GiB device-to-device copy of --calibrate (1,048,576 KiB each way)."""
    import collections, csv, glob
    def averages(folder, counter):
        values = collections.defaultdict(list)
        files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
        for row in csv.DictReader(open(max(files, key=os.path.getmtime))):   # a folder that was used before: the latest run's file
            if row["Counter_Name"] == counter:
                values[row["Kernel_Name"]].append(float(row["Counter_Value"]))
        pick = lambda word: [v for k, v in values.items() if word in k]
        copies, = pick("copyBuffer")          # the runtime's copy kernel also serves small copies: the 1 GiB one is the largest
        kernel, = pick("decode_stack_kernel")
        return sum(kernel) / len(kernel), max(copies), len(kernel)
    fetch, fetch_copy, calls = averages(fetch_dir, "FETCH_SIZE")
    write, write_copy, _ = averages(write_dir, "WRITE_SIZE")
    read_bytes = fetch * (1048576.0 / fetch_copy) * 1024
    written_bytes = write * (1048576.0 / write_copy) * 1024
    record = {"kernel": "zc::decode_stack_kernel<false>", "workload": "48 F-shape layers, batch 1 (the default run of bench.py)",
              "dispatches_averaged": calls, "FETCH_SIZE_KiB": fetch, "FETCH_SIZE_KiB_of_1GiB_copy": fetch_copy,
              "WRITE_SIZE_KiB": write, "WRITE_SIZE_KiB_of_1GiB_copy": write_copy,
              "hbm_bytes_read": int(read_bytes), "hbm_bytes_written": int(written_bytes),
              "hbm_bytes_per_launch": int(read_bytes + written_bytes)}
    json.dump(record, open(TRAFFIC_FILE, "w"), indent=1)
    print(json.dumps(record))


def one_launch_layer(ctx, name, tokens, reps, warmup=5, skew=("zipf", 1.1), speculate=True):
    """The same single-layer configuration through the persistent decode kernels as a stack of one layer: one launch per
    step up to sixty-four tokens (pieces of sixty-four above that); over 8 distinct inputs in rotation."""
    import numpy as np
    import zerocool_amd as z
    from zerocool_amd import workload
    c = workload.config(name)
    lw = workload.LayerWeights(ctx, c, workload.BASE_SEED + 77, skew)
    stack = ctx.stack_create(c, [lw.layer], max(8, tokens))
    ctx.stack_set_speculation(stack, speculate)
    xs = [workload.hidden_rows(ctx, tokens, c.hidden, workload.BASE_SEED + 78 + tokens + 97 * i) for i in range(INPUTS)]
    out = ctx.alloc(tokens * c.hidden * 4)
    ws = ctx.alloc(ctx.moe_workspace_bytes(c, tokens))
    ref = ctx.alloc(tokens * c.hidden * 4)
    ids, wts = ctx.alloc(tokens * c.topk * 4), ctx.alloc(tokens * c.topk * 4)
    unique = []
    for x in xs:   # parity gate: the operator path's bytes (glue of layer 0 is the identity on the input)
        ctx.stack_decode(stack, x, tokens, out, z.StackTrace(ids.ptr, wts.ptr, None, None))
        ctx.moe_forward(c, lw.layer, x, tokens, ref, ws)
        ctx.moe_check()
        if out.numpy(np.float32).tobytes() != ref.numpy(np.float32).tobytes():
            raise SystemExit("bench.py: one-launch layer and operator path disagree; refusing to time")
        unique.append(len(np.unique(ids.numpy(np.int32))))
    nbytes = float(np.mean([workload.layer_bytes(c, u, tokens, ctx) for u in unique]))
    for i in range(warmup):
        ctx.stack_decode(stack, xs[i % INPUTS], tokens, out)
    ctx.finish()
    ctx.timer_start()
    for i in range(reps):
        ctx.stack_decode(stack, xs[i % INPUTS], tokens, out)
    ms = ctx.timer_stop() / reps
    ctx.moe_check()
    persistent = ctx.stack_is_persistent(stack, tokens)
    ctx.stack_destroy(stack)
    for b in xs + [out, ws, ref, ids, wts, lw.router, lw.shared_gate, lw.shared_record, lw.records]:
        ctx.free(b)
    return {"tokens": tokens, "us_per_layer": ms * 1e3, "tokens_per_s": tokens / (ms * 1e-3), "router_skew": list(skew) if skew else None,
            "distinct_experts": float(np.mean(unique)), "slots_per_distinct_expert": tokens * c.topk / float(np.mean(unique)),
            "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 8e12,
            "guessing": bool(speculate), "path": "persistent single-launch kernel" if persistent else "layer by layer"}


def prefill_workload(ctx, args):
    # The configuration names no router skew: the headline is the unskewed layer (every expert is touched, about 40 rows
    # each); the same layer behind Zipf(1.1) router offsets (a third of the experts, most rows on ten of them) stands beside it.
    r = single_layer(ctx, "S", args.prefill_tokens, True, args.steps, args.warmup, skew=None)
    skewed = single_layer(ctx, "S", args.prefill_tokens, True, args.steps, args.warmup)
    print(json.dumps({
        "metric": "moe_prefill_tokens_per_s", "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": r["us_per_layer"] * 1e-3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u4 codes as bf16 x bf16 inputs, fp32 accumulation", "data": "synthetic (seeded generator)",
        "config": {"workload": "BASELINE configs[2]: one MoE layer, 2048-token prefill batch, hidden 2048, 512 experts, top-10, "
                               "intermediate 512, affine Q4 group 64, no router skew", "tokens": args.prefill_tokens,
                   "with_zipf_1.1_router_offsets": {"us_per_layer": skewed["us_per_layer"], "tokens_per_s": skewed["tokens_per_s"], "TFLOPs": skewed["TFLOPs"]}},
        "roofline": {"bound": "mfma", "achieved": r["TFLOPs"], "peak": 2500.0, "unit": "TFLOP/s", "frac": r["TFLOPs"] / 2500.0,
                     "traffic": None, "kernel": "zc::prefill_gemm_kernel (whole-layer rate: router, routing, dispatch, "
                                                "both grouped products, exact recomputation and combine included)"}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--headline-only", action="store_true", help="skip the other_configs block (batch 1 without guessing, batch 8 and 64, the prefill layer)")
    ap.add_argument("--extra", action="store_true", help="also time batch 32, milder router skews, the capped-HBM stack and the single-layer configurations")
    ap.add_argument("--workload", choices=("stack", "prefill"), default="stack",
                    help="stack: the 48-layer decode stack (the headline); prefill: one 2048-token batch through one layer of "
                         "hidden 2048 / 512 experts / top-10 / intermediate 512 on the bf16 matrix cores")
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="--workload prefill: tokens of the batch")
    ap.add_argument("--capped-layers", type=int, default=48, help="--extra: layers of the capped-HBM run")
    ap.add_argument("--capped-homes", type=int, default=12,
                    help="--extra: pinned-host homes of the capped-HBM run's records; layer l shares the home of layer l mod this number "
                         "(48 distinct homes would pin 130 GB of host memory, more than this pool's boxes grant; 24 are 65 GB)")
    ap.add_argument("--capped-only", action="store_true", help="--extra: only the capped-HBM runs")
    ap.add_argument("--calibrate", action="store_true", help="also run one 1 GiB device-to-device copy (a dispatch of known traffic for counter runs)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="no GPU work: rewrite the tracked traffic file from the output folders of the two counter runs")
    args = ap.parse_args()
    if args.traffic_from:
        return write_traffic_file(*args.traffic_from)
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus must be 1 "
              "(the design notes describe how the path would shard by expert)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import zerocool_amd as z
    from zerocool_amd import synth, workload

    ctx = z.Context(0)
    if args.workload == "prefill":
        return prefill_workload(ctx, args)
    cfg = workload.config("F")
    L, T = args.layers, args.batch
    layers = [workload.LayerWeights(ctx, cfg, workload.BASE_SEED + 4 * 1000 + l, ("zipf", 1.1)) for l in range(L)]
    ctx.finish()
    stack = ctx.stack_create(cfg, [l.layer for l in layers], max(T, 64))

    def run(stack, cfg, n_layers, tokens, steps, warmup, speculate=True, inputs=INPUTS, seed=workload.BASE_SEED + 4 * 7):
        """Times `steps` launches that cycle through `inputs` distinct token batches (a decode loop never sees the same
        hidden rows twice; the one-token kernel guesses each layer's experts from the step before, so a replayed input
        would make every guess a hit).  Every input is first checked against the layer-by-layer operator path, byte for
        byte, and its route ids are kept: they give the distinct records (the algorithmic bytes) of each launch and the
        share of a step's experts that the step before had also chosen (what the guessing can hit)."""
        xs = [workload.hidden_rows(ctx, tokens, cfg.hidden, seed + tokens + 97 * i) for i in range(inputs)]
        out = ctx.alloc(tokens * cfg.hidden * 4)
        n = tokens * cfg.topk
        ids, w = ctx.alloc(n_layers * n * 4), ctx.alloc(n_layers * n * 4)
        ctx.stack_set_speculation(stack, speculate)
        chosen, nbytes, unique = [], [], []
        for x in xs:
            ctx.stack_decode(stack, x, tokens, out, z.StackTrace(ids.ptr, w.ptr, None, None))
            ctx.moe_check()
            fused = out.numpy(np.float32).tobytes()
            ctx.stack_decode(stack, x, tokens, out, layered=True)
            ctx.moe_check()
            if out.numpy(np.float32).tobytes() != fused:
                raise SystemExit("bench.py: persistent kernel and layer-by-layer path disagree; refusing to time")
            rows = ids.numpy(np.int32).reshape(n_layers, n).copy()
            chosen.append(rows)
            u = [len(np.unique(r)) for r in rows]
            unique.append(float(np.mean(u)))
            nbytes.append(sum(workload.layer_bytes(cfg, v, tokens, ctx) for v in u))
        repeats = [np.mean([len(np.intersect1d(a[l], b[l])) / len(np.unique(a[l])) for l in range(n_layers)])
                   for a, b in zip(chosen[1:] + chosen[:1], chosen)] if inputs > 1 else [1.0]
        for i in range(warmup):
            ctx.stack_decode(stack, xs[i % inputs], tokens, out)
        ctx.finish()
        ctx.timer_start()
        for i in range(steps):
            ctx.stack_decode(stack, xs[(warmup + i) % inputs], tokens, out)
        ms = ctx.timer_stop() / steps
        ctx.moe_check()
        for b in xs + [out, ids, w]:
            ctx.free(b)
        return {"ms": ms, "bytes": float(np.mean(nbytes)), "unique": float(np.mean(unique)), "repeat_share": float(np.mean(repeats))}

    if args.calibrate:
        gib = 1 << 30
        a, b = ctx.alloc(gib), ctx.alloc(gib)
        ctx.fill(a, 1)
        ctx.copy(b, a, gib)
        ctx.finish()
        ctx.free(a); ctx.free(b)
    r = run(stack, cfg, L, T, args.steps, args.warmup)
    ms, nbytes = r["ms"], r["bytes"]
    persistent = ctx.stack_is_persistent(stack, T)
    achieved = nbytes / (ms * 1e-3) / 1e9
    traffic = None
    if (L, T) == (48, 1) and os.path.exists(TRAFFIC_FILE):
        traffic = json.load(open(TRAFFIC_FILE))["hbm_bytes_per_launch"]
    result = {
        "metric": "moe_decode_tokens_per_s", "value": T / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u4 codes x bf16 inputs, fp32 accumulation",
        "data": "synthetic (counter-based generator, seeded; random-init weights of the named shape)",
        "config": {"workload": "BASELINE configs[4]: 48-layer MoE stack decode, hidden 3072, 512 experts, top-10, "
                               "intermediate 1024, affine Q4 group 64, ~130 GB of expert records resident in HBM, "
                               "Zipf(1.1) router offsets, one seed per layer",
                   "layers": L, "decode_batch": T, "hbm_resident_bytes": int(ctx.allocated),
                   "inputs": f"{INPUTS} distinct token batches in rotation", "distinct_experts_per_layer": r["unique"],
                   "experts_repeated_from_previous_step": r["repeat_share"],
                   "path": "persistent single-launch kernel" if persistent else "layer by layer",
                   "parity_gate": "output bytes equal the layer-by-layer operator path on this input (checked before timing)"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": 8000.0, "unit": "GB/s", "frac": achieved / 8000.0,
                     "traffic": traffic, "traffic_source": os.path.relpath(TRAFFIC_FILE, ROOT) if traffic else None,
                     "kernel": "zc::decode_stack_kernel (one launch = one step)" if T == 1 else "zc::decode_multi_kernel (one launch = one step)",
                     "algorithmic_bytes_per_launch": int(nbytes), "launch_us": ms * 1e3},
    }

    if not args.headline_only and (L, T) == (48, 1):
        # The other configurations on the same clock, each with its own fraction of the roofline that bounds it: the same stack
        # with the guessing switched off (every gate/up tile waits for the routing), at decode batch 8 and 64 (bytes = the
        # DISTINCT records of a step), and BASELINE configs[2], the 2048-token prefill layer on the bf16 matrix cores.
        quick = max(8, args.steps // 2)
        def line(m, tokens, kernel):
            return {"ms_per_step": m["ms"], "tokens_per_s": tokens / (m["ms"] * 1e-3), "GBps": m["bytes"] / (m["ms"] * 1e-3) / 1e9,
                    "frac": m["bytes"] / (m["ms"] * 1e-3) / 8e12, "bound": "hbm", "distinct_experts_per_layer": m["unique"], "kernel": kernel}
        also = {"stack_batch1_without_guessing": line(run(stack, cfg, L, 1, quick, 2, speculate=False), 1, "zc::decode_stack_kernel"),
                "stack_batch8": line(run(stack, cfg, L, 8, quick, 2), 8, "zc::decode_multi_kernel"),
                "stack_batch64": line(run(stack, cfg, L, 64, max(4, quick // 4), 1, inputs=2), 64, "zc::decode_wide_kernel")}
        ctx.stack_set_speculation(stack, True)
        pf = single_layer(ctx, "S", 2048, True, 20, 3, skew=None)
        s_cfg = workload.config("S")
        weight_bytes = s_cfg.experts * ctx.record_bytes(s_cfg) + ctx.record_bytes(s_cfg, shared=True) + 2 * s_cfg.hidden * s_cfg.experts
        also["prefill_layer_2048_tokens"] = {
            "ms_per_step": pf["us_per_layer"] * 1e-3, "tokens_per_s": pf["tokens_per_s"], "TFLOPs": pf["TFLOPs"], "bound": "mfma",
            "frac": pf["TFLOPs"] / 2500.0, "frac_of_hbm_floor": weight_bytes / 8e12 / (pf["us_per_layer"] * 1e-6),
            "workload": "BASELINE configs[2]: hidden 2048, 512 experts, top-10, intermediate 512, affine Q4, no router skew",
            "kernel": "zc::prefill_gemm_kernel and the layer's other kernels (whole-layer rate)"}
        result["other_configs"] = also

    if not args.no_cpu:
        import oracle
        sample_layers = 2
        threads = min(os.cpu_count() or 1, 16)
        ocfg = oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])
        x = workload.hidden_rows(ctx, T, cfg.hidden, workload.BASE_SEED + 4 * 7 + T).numpy(np.float32)
        hosts = [layers[l].host() for l in range(sample_layers)]
        def cpu_pass():
            cur = x.reshape(T, cfg.hidden)
            for h in hosts:
                cur = oracle.moe_layer(ocfg, h["router"], h["shared_gate"], h["shared_record"], h["records"], h["stride"],
                                       cur, T, router_offsets=h["offsets"], threads=threads)
        cpu_pass()
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10 and reps < 200):
            cpu_pass(); reps += 1
        per_layer = (time.perf_counter() - t0) / reps / sample_layers
        result["cpu_baseline"] = {"value": T / (per_layer * L), "unit": "tokens/s", "cores": threads, "kind": "port",
                                  "sample": f"{sample_layers} of {L} layers x {reps} repetitions at batch {T}, per-layer mean "
                                            f"extrapolated to {L} layers (the CPU oracle, OpenMP over output rows)",
                                  "ms_per_layer": per_layer * 1e3}
    if args.extra:
        extra = {}
        quick = max(8, args.steps // 2)
        if not args.capped_only:
            if T == 1:
                off = run(stack, cfg, L, 1, quick, 2, speculate=False)
                extra["stack_batch1_without_guessing"] = {"tokens_per_s": 1 / (off["ms"] * 1e-3), "ms_per_step": off["ms"],
                                                          "GBps": off["bytes"] / (off["ms"] * 1e-3) / 1e9}
            r8 = run(stack, cfg, L, 8, quick, 2)
            extra["stack_batch8"] = {"tokens_per_s": 8 / (r8["ms"] * 1e-3), "ms_per_step": r8["ms"], "GBps": r8["bytes"] / (r8["ms"] * 1e-3) / 1e9,
                                     "frac_of_hbm_peak": r8["bytes"] / (r8["ms"] * 1e-3) / 8e12, "distinct_experts_per_layer": r8["unique"],
                                     "kernel": "zc::decode_multi_kernel"}
            for tokens in (32, 64):   # one launch of the kernel for nine to sixty-four tokens
                rw = run(stack, cfg, L, tokens, max(4, quick // 4), 1, inputs=2)
                extra[f"stack_batch{tokens}"] = {"tokens_per_s": tokens / (rw["ms"] * 1e-3), "ms_per_step": rw["ms"], "GBps": rw["bytes"] / (rw["ms"] * 1e-3) / 1e9,
                                                 "distinct_experts_per_layer": rw["unique"], "kernel": "zc::decode_wide_kernel"}
            # The same records behind routers with a milder popularity skew (Zipf exponent 0.5: the offsets span 3.1 instead
            # of 6.9) and with none at all, so that consecutive tokens share fewer experts and a batch of eight touches
            # several times more records.
            for name, exponent in (("mild_skew_zipf_0.5", 0.5), ("no_skew", None)):
                offsets = [ctx.upload(synth.zipf_offsets(cfg.experts, (workload.BASE_SEED + 4 * 1000 + l) * 16 + 5, exponent))
                           for l in range(L)] if exponent else [None] * L
                other = ctx.stack_create(cfg, [z.Layer(w.router.ptr, o.ptr if o else None, w.shared_gate.ptr, w.shared_record.ptr,
                                                       w.records.ptr, w.stride) for w, o in zip(layers, offsets)], 8)
                extra[name] = {}
                for tokens, spec in ((1, True), (1, False), (8, True)):
                    m = run(other, cfg, L, tokens, quick, 2, speculate=spec)
                    extra[name][f"batch{tokens}" + ("" if spec else "_without_guessing")] = {
                        "tokens_per_s": tokens / (m["ms"] * 1e-3), "ms_per_step": m["ms"], "GBps": m["bytes"] / (m["ms"] * 1e-3) / 1e9,
                        "distinct_experts_per_layer": m["unique"], "experts_repeated_from_previous_step": m["repeat_share"]}
                ctx.stack_destroy(other)
                for o in offsets:
                    if o: ctx.free(o)
        # The capped-HBM run of the same configuration: the records' home is pinned host memory and 2000 of the 24576
        # records fit in HBM slots.  The host cannot pin all 130 GB, so the 48 layers share --capped-homes pinned homes
        # (layer l holds the records of layer l mod that number; routers, shared experts and offsets are every layer's
        # own, and the slot cache keys every (layer, expert) separately, so the slot traffic is that of 48 distinct layers).
        # Each step is one launch of the same persistent kernels, which take every record's address from the store's
        # table: an HBM slot, or the record's home over the host link; after the launch the store admits what was read
        # from home (fills on its side stream).  Timed by the host clock: the step includes the wait for the launch, the
        # readback of the routes and the store's bookkeeping.
        ctx.stack_destroy(stack)
        for l in layers:
            for b in (l.router, l.shared_gate, l.shared_record, l.records):
                ctx.free(b)
        CL = args.capped_layers
        homes = min(CL, args.capped_homes)
        extra["capped_hbm"] = {}
        # 2000 slots (the configuration), and as many slots as one token selects experts per step (48 x top-10 = 480): fewer than
        # the eight rotating inputs touch, so every step misses and the slots turn over
        # ... and the 2000 slots again behind routers without any skew, where consecutive tokens share fewer experts: the
        # steady state keeps missing
        big = max(cfg.topk + 2, 2000 * CL // 48)
        for name, slots, batches, skew in ((f"{big}_slots", big, (1, 8), ("zipf", 1.1)), (f"{CL * cfg.topk}_slots", CL * cfg.topk, (1,), ("zipf", 1.1)),
                                           (f"{big}_slots_no_router_skew", big, (1,), None), (f"{big // 4}_slots_no_router_skew", big // 4, (1,), None)):
            capped = workload.StoreBackedStack(ctx, cfg, [workload.BASE_SEED + 4 * 1000 + l for l in range(CL)], skew, slots, home_layers=homes)
            cstack = capped.decode_stack(8)
            report = {"layers": CL, "hbm_slots": int(slots), "records": CL * cfg.experts, "router_skew": list(skew) if skew else None,
                      "record_homes": homes, "pinned_home_bytes": homes * cfg.experts * int(capped.store.stride)}
            for tokens in batches:
                xs = [workload.hidden_rows(ctx, tokens, cfg.hidden, workload.BASE_SEED + 4 * 7 + tokens + 97 * i) for i in range(INPUTS)]
                out = ctx.alloc(tokens * cfg.hidden * 4)
                t0 = time.perf_counter()
                ctx.stack_decode(cstack, xs[0], tokens, out)      # cold: every record comes over the host link
                ctx.finish()
                cold = time.perf_counter() - t0
                for i in range(2 * INPUTS):
                    ctx.stack_decode(cstack, xs[i % INPUTS], tokens, out)
                ctx.finish(); ctx.moe_check(); ctx.stack_settle(cstack)
                seen0, st0 = capped.store.table_stats(), capped.store.stats()
                reads0, slot0, home0, fill0, evict0, joined0 = seen0.reads, seen0.slot_reads, seen0.home_read_bytes, st0.bytes, st0.evictions, seen0.joined
                n_steps = max(16, args.steps)
                t0 = time.perf_counter()
                for i in range(n_steps):
                    ctx.stack_decode(cstack, xs[i % INPUTS], tokens, out)
                ctx.finish()
                dt = (time.perf_counter() - t0) / n_steps
                ctx.moe_check(); ctx.stack_settle(cstack)
                seen, st = capped.store.table_stats(), capped.store.stats()
                report[f"batch{tokens}"] = {
                    "ms_per_step": dt * 1e3, "us_per_layer": dt / CL * 1e6, "tokens_per_s": tokens / dt * CL / 48 * 48 / CL,
                    "first_step_ms": cold * 1e3, "slot_hit_rate": (seen.slot_reads - slot0) / max(1, seen.reads - reads0),
                    "bytes_read_from_home_per_token": (seen.home_read_bytes - home0) / n_steps / tokens,
                    "bytes_filled_into_slots_per_token": (st.bytes - fill0) / n_steps / tokens,
                    "evictions_per_step": (st.evictions - evict0) / n_steps,
                    "fills_joined_by_a_launch_per_step": (seen.joined - joined0) / n_steps}
                for b in xs + [out]:
                    ctx.free(b)
            extra["capped_hbm"][name] = report
            ctx.stack_destroy(cstack)
            capped.close()
        if not args.capped_only:
            # Single-layer configurations: decode batches through the exact operator path, and batches through the
            # sorted-token grouped product on the bf16 matrix cores.
            # BASELINE configs[1]: continuous-batching decode of the single-layer shape behind N(0, 0.5) router offsets: GEMV
            # bandwidth over the distinct records of a step, and the expert dedup across its tokens (slots per distinct expert)
            extra["single_layer_q4_one_launch_normal_0.5"] = [one_launch_layer(ctx, "S", t, 200 if t <= 8 else 50, skew=("normal", 0.5)) for t in (1, 8, 32, 64)]
            extra["single_layer_q4_one_launch"] = [one_launch_layer(ctx, "S", t, 200 if t <= 8 else 50) for t in (1, 8, 32, 64)]
            # raw random inputs behind an unskewed router share next to no experts from one step to the next: every guess of
            # the one-token kernel misses, which prices the guessing at its worst
            extra["single_layer_q4_one_launch_all_guesses_miss"] = [one_launch_layer(ctx, "S", 1, 200, skew=None, speculate=on) for on in (True, False)]
            extra["single_layer_q4_normal_0.5"] = [single_layer(ctx, "S", t, False, 30, skew=("normal", 0.5)) for t in (1, 8, 32, 64)]
            extra["single_layer_q4"] = [single_layer(ctx, "S", t, False, 50) for t in (1, 8, 32, 64)]
            extra["single_layer_mixed_one_launch"] = [one_launch_layer(ctx, "S-mixed", t, 100) for t in (1, 8, 16)]
            extra["single_layer_mixed"] = [single_layer(ctx, "S-mixed", t, False, 50) for t in (1, 8, 16)]
            extra["prefill_q4"] = [single_layer(ctx, "S", t, True, 20) for t in (32, 64, 256, 2048)]
            extra["prefill_mixed"] = [single_layer(ctx, "S-mixed", t, True, 20, skew=None) for t in (256, 2048)]
        result["extra"] = extra

    print(json.dumps(result))


if __name__ == "__main__":
    main()
