#!/usr/bin/env python3
"""Benchmark of the expert-specialized grouped GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1|c2|c3|c4] [--op gemm|quant] [--force-bm 0|16|...]

One "step" is one call of the operator (through torch.ops.expert_specialization.*) over one batch
of synthetic, already-quantised operands resident in HBM.  Prints ONE JSON line.  The default
workload is c1: the DeepSeek-V3 gate_up projection, one GPU's 32-expert share (K=7168, N=4096,
FP8-blockwise, 4096 tokens routed top-8 over 256 experts with Zipf(1.2) popularity, seed 0).
"""
import argparse
import json
import os
import sys
import time

import torch

# HBM bytes per launch of the dominant kernel, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of
# this script (summaries under profiles/), each scaled by the same counter's reading for a 1 GiB copy kernel.
# Keyed by (config, op); None where not measured.
MEASURED_TRAFFIC_BYTES = {
    ("c1", "gemm"): 1.546e9,     # FETCH 728,218.9 x 2.000 KiB + WRITE 52,804.0 x 1.000 KiB
    ("c2", "gemm"): 4.485e8,     # FETCH 217,195.5 x 2.000 KiB + WRITE 3,643.1 x 1.000 KiB
    ("c4", "gemm"): 1.452e9,     # FETCH 676,216.6 x 2.000 KiB + WRITE 65,709.2 x 1.000 KiB
    ("c4", "quant"): 1.785e8,    # FETCH 57,378.0 x 2.000 KiB + WRITE 59,584.5 x 1.000 KiB
}


def settle(step, ms):
    """Untimed: keeps the GPU on this step's work for `ms` milliseconds before the warm-up steps.  A chip that has
    been idle runs its first tens of milliseconds of work at lower clocks, whatever the number of warm-up steps."""
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(20):
            step()
        torch.cuda.synchronize()


def cpu_model():
    """Model name of the host CPU (first "model name" line of /proc/cpuinfo), or "unknown"."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def time_batches(step, steps, batches):
    """Mean milliseconds per step of `batches` further batches of `steps` steps each (events on the current stream)."""
    out = []
    for _ in range(batches):
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(steps):
            step()
        ev1.record()
        torch.cuda.synchronize()
        out.append(ev0.elapsed_time(ev1) / steps)
    return out


def calibration_copy():
    src = torch.empty((1 << 30,), dtype=torch.uint8, device="cuda:0").fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=300,
                    help="untimed steps before the timed ones; the chip needs some tens of milliseconds of this work before its "
                         "clocks settle (C1: 314 us per step after 5 warm-up steps, 285 after 50, 276 after 500)")
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="untimed: run the step for this many milliseconds before the warm-up steps, so that a small "
                         "--warmup does not time the chip's clock ramp (0 = off)")
    ap.add_argument("--config", default="c1", choices=["c1", "c2", "c3", "c4", "dense", "dense_mx"],
                    help="dense, dense_mx: one expert of 12288 rows, N=4096, K=7168 (fp8-blockwise, mxfp8): the tall tiles alone")
    ap.add_argument("--tokens", type=int, default=8192, help="c3 only")
    ap.add_argument("--routing", default="zipf", choices=["zipf", "uniform"], help="c3 only")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--op", default="gemm", choices=["gemm", "quant", "quant_act", "quant_weight", "route", "swiglu_quant"],
                    help="quant: the MXFP8 grouped quantisation of the workload's activation rows (c4 stage 1); "
                         "quant_act: the FP8 1x128 activation quantisation of the same rows; "
                         "quant_weight: the FP8 128x128 quantisation of the workload's [E, N, K] weights; "
                         "route: top-k ids -> per-expert metadata + row packing of the workload's routing; "
                         "swiglu_quant: fused SwiGLU + 1x128 quantisation of the workload's [rows, N] output")
    ap.add_argument("--force-bm", type=int, default=0, help="single M-tile shape for every expert (0 = device schedule)")
    ap.add_argument("--fuse-swiglu", action="store_true",
                    help="gemm op: the projection with the fused SwiGLU + re-quantisation epilogue (1x128 fp32 scales for the "
                         "fp8-blockwise configs, 1x32 E8M0 scales for c4; the workload's N is read as 2 * inter); the output "
                         "bytes counted are the e4m3 + scale bytes")
    ap.add_argument("--single-tile-sweep", action="store_true",
                    help="gemm op: after the timed region also time the same kernel with every single tile height forced "
                         "(16 .. 192 rows) and report the best one and its ratio to the device schedule's time")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="default c1 run only: skip the `secondary` object (the other workloads of the path, measured "
                         "after the timed region); profiler runs of one kernel want this")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="after the timed region also run three 1 GiB device copies (a kernel of known traffic, for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline sample")
    return ap.parse_args()


def cpu_baseline(prob, ops, budget_s):
    """The reference's torch CPU path (dequantise with torch ops, fp32 torch.mm, cast: oracle/torch_path.py) timed
    on this host on a bounded sample: experts in index order, whole passes, until two thirds of the time budget are
    used.  Nothing but torch ops runs inside the timed sections.  The numpy oracle that the parity tests use
    (oracle/fp8_blockwise.py, oracle/mxfp8.py: numpy dequantisation in front of the same matmul) is timed the same
    way on the rest of the budget and reported beside it."""
    from oracle import fp8_blockwise as ofp8
    from oracle import mxfp8 as omx
    from oracle import torch_path as otp
    import numpy as np

    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()
    rows = prob.rows
    offs = [0]
    for m in rows[:-1]:
        offs.append(offs[-1] + m)
    mx = prob.kind != "fp8_blockwise"
    kc = prob.k // 32
    a_cpu = ops["a"].contiguous().cpu()
    a_codes = a_cpu.view(torch.uint8).numpy()
    order = [e for _ in range(64) for e in range(len(rows)) if rows[e]]   # whole passes over the experts with rows

    def operands_of(e):
        m = rows[e]
        b_e = ops["b_phys"][e].contiguous().cpu()
        if not mx:
            return (a_cpu[offs[e]:offs[e] + m], b_e, ops["scales_a"][offs[e]:offs[e] + m].float().cpu(),
                    ops["scales_b_phys"][e].float().cpu())
        bso = int(ops["blockscale_offsets"][e])
        sfa = ops["sfa"].reshape(-1)[bso * kc:(bso + (m + 127) // 128 * 128) * kc].cpu().numpy()
        sfb = ops["sfb_phys"][e].reshape(-1).cpu().numpy()
        return a_cpu[offs[e]:offs[e] + m], b_e, sfa, sfb

    def run(budget, torch_only):
        flops, used, done = 0.0, 0.0, 0
        for e in order:
            m = rows[e]
            a_e, b_e, s_a, s_b = operands_of(e)
            if torch_only:
                if mx:   # row-major scale codes, prepared outside the timed section
                    s_a = torch.from_numpy(omx.unswizzle_scales(s_a, m, prob.k))
                    s_b = torch.from_numpy(omx.unswizzle_scales(s_b, prob.n, prob.k))
                t0 = time.perf_counter()
                (otp.mx_scaled_mm if mx else otp.scaled_mm)(a_e, b_e, s_a, s_b)
                used += time.perf_counter() - t0
            else:
                ac, bc = a_e.view(torch.uint8).numpy(), b_e.view(torch.uint8).numpy()[None]
                ps = [[m, prob.n, prob.k]]
                t0 = time.perf_counter()
                if mx:
                    omx.grouped_mm(ac, bc, s_a, s_b, ps, [0], [0])
                else:
                    ofp8.grouped_mm(ac, bc, s_a.numpy(), s_b.numpy()[None], ps, [0])
                used += time.perf_counter() - t0
            flops += 2.0 * m * prob.n * prob.k
            done += 1
            if used > budget:
                break
        return flops, used, done

    active = max(1, sum(1 for m in rows if m))
    run(0.0, True)   # one untimed expert: thread pool and allocator warm
    t_flops, t_used, t_done = run(budget_s * 2 / 3, True)
    o_flops, o_used, o_done = run(budget_s / 3, False)
    return {
        "value": t_flops / t_used / 1e12 if t_used else 0.0, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "cpu_model": cpu_model(),
        "sample": f"torch ops only (dequantise, fp32 torch.mm, cast): {t_done} expert problems of the same workload in "
                  f"index order, {t_done / active:.2f} passes ({t_flops / 1e9:.1f} GFLOP, {t_used:.1f} s)",
        "numpy_oracle_value": o_flops / o_used / 1e12 if o_used else 0.0,
        "numpy_oracle_sample": f"the parity tests' numpy oracle: {o_done} expert problems ({o_flops / 1e9:.1f} GFLOP, {o_used:.1f} s)",
    }


def bench_quant(args, prob, es, W):
    """MXFP8 grouped quantisation (bf16 rows -> e4m3 bytes + swizzled E8M0 scales) of the workload's rows, or
    (--op quant_act) their FP8 1x128 quantisation (e4m3 bytes + fp32 scale per 128-wide block)."""
    import numpy as np

    act = args.op == "quant_act"

    dev = "cuda:0"
    rows, k, total = prob.rows, prob.k, prob.total_rows
    gen = torch.Generator().manual_seed(args.seed)
    x = torch.randn((total, k), generator=gen).to(torch.bfloat16)
    xd = x.to(dev)
    ps = torch.tensor([[m, prob.n, k] for m in rows], dtype=torch.int32, device=dev)
    eo = torch.tensor(W.offsets_of(rows), dtype=torch.int32, device=dev)
    bso_np, sf_rows = W.blockscale_offsets_of(rows)
    bso = torch.tensor(bso_np, dtype=torch.int32, device=dev)
    q = torch.empty((total, k), dtype=torch.uint8, device=dev)
    sf = torch.zeros((sf_rows * (k // 32),), dtype=torch.uint8, device=dev)

    sc = torch.empty((total, k // 128), dtype=torch.float32, device=dev)

    def step():
        if act:
            es.es_fp8_quant_act_1x128(xd, q, sc)
        else:
            es.es_sm100_mxfp8_blockscaled_grouped_quant(xd, ps, eo, bso, q, sf)

    settle(step, args.settle_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = start.elapsed_time(stop) / args.steps
    nbytes = float(total) * k * (2 + 1 + 4 / 128.0) if act else W.quant_bytes(rows, k)
    t = ms_per_step * 1e-3
    roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": W.HBM_BYTES_PER_S / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get((prob.name, args.op))
    roof["algorithmic_bytes"] = nbytes
    roof["roofline_us"] = nbytes / W.HBM_BYTES_PER_S * 1e6
    out = {
        "metric": ("FP8 1x128 activation quantisation, algorithmic GB/s (bf16 in, e4m3 + fp32 scales out)" if act else
                   "MXFP8 grouped quantisation, algorithmic GB/s (bf16 in, e4m3 + E8M0 out)"),
        "value": nbytes / t / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 -> fp8_e4m3 + fp32 scales" if act else "bf16 -> fp8_e4m3 + e8m0", "data": "synthetic",
        "config": {"workload": f"{prob.name} {args.op}: E={len(rows)} K={k} rows={total} max_rows={max(rows)} seed={args.seed}"},
        "roofline": roof,
    }
    if args.calibration_copy:
        calibration_copy()
    if not args.no_cpu_baseline:
        from oracle import fp8_blockwise as ofp8
        from oracle import mxfp8 as omx

        xs = x[: min(total, 512)].float().numpy()   # bounded sample: the first rows, repeated until the budget is used
        used, nrows = 0.0, 0
        while used < args.cpu_seconds:
            t0 = time.perf_counter()
            ofp8.quant_act_1x128(xs) if act else omx.quant_rows(xs)
            used += time.perf_counter() - t0
            nrows += xs.shape[0]
        out["cpu_baseline"] = {"value": nbytes / total * nrows / used / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{nrows} rows of the same input through the numpy oracle ({used:.1f} s)"}
    print(json.dumps(out), flush=True)


def bench_swiglu_quant(args, prob, es, W):
    """Fused SwiGLU + quantisation of a [rows, N] gate_up output (N = 2 * inter): FP8 1x128 for the fp8-blockwise
    workloads, MXFP8 (grouped, swizzled E8M0 scales) for the mxfp8 workload."""
    dev = "cuda:0"
    mx = prob.kind == "mxfp8"
    total, inter = prob.total_rows, prob.n // 2
    x = torch.randn((total, 2 * inter), generator=torch.Generator().manual_seed(args.seed)).to(torch.bfloat16)
    xd = x.to(dev)
    q = torch.empty((total, inter), dtype=torch.uint8, device=dev)
    if mx:
        bso_np, sf_rows = W.blockscale_offsets_of(prob.rows)
        ps = torch.tensor([[m, prob.n, inter] for m in prob.rows], dtype=torch.int32, device=dev)
        eo = torch.tensor(W.offsets_of(prob.rows), dtype=torch.int32, device=dev)
        bso = torch.tensor(bso_np, dtype=torch.int32, device=dev)
        sc = torch.empty((sf_rows * (inter // 32),), dtype=torch.uint8, device=dev)
    else:
        sc = torch.empty((total, inter // 128), dtype=torch.float32, device=dev)

    def step():
        if mx:
            es.es_swiglu_mxfp8_grouped_quant(xd, ps, eo, bso, q, sc)
        else:
            es.es_swiglu_quant_1x128(xd, q, sc)

    settle(step, args.settle_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = start.elapsed_time(stop) / args.steps
    nbytes = float(total) * inter * (4 + 1 + (1 / 32.0 if mx else 4 / 128.0))
    t = ms_per_step * 1e-3
    roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": W.HBM_BYTES_PER_S / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None
    roof["algorithmic_bytes"] = nbytes
    roof["roofline_us"] = nbytes / W.HBM_BYTES_PER_S * 1e6
    out = {
        "metric": ("fused SwiGLU + MXFP8 grouped quantisation, algorithmic GB/s (bf16 [rows, 2I] in, e4m3 + E8M0 scales out)" if mx else
                   "fused SwiGLU + FP8 1x128 quantisation, algorithmic GB/s (bf16 [rows, 2I] in, e4m3 + fp32 scales out)"),
        "value": nbytes / t / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 -> fp32 -> bf16 -> fp8_e4m3 + " + ("e8m0 scales" if mx else "fp32 scales"), "data": "synthetic",
        "config": {"workload": f"{prob.name} swiglu_quant: rows={total} inter={inter} seed={args.seed}"},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        import numpy as np
        from oracle import fp8_blockwise as ofp8
        from oracle import mxfp8 as omx

        xs = x[: min(total, 256)].float().numpy()
        used, nrows = 0.0, 0
        while used < args.cpu_seconds:
            t0 = time.perf_counter()
            with np.errstate(over="ignore"):
                if mx:
                    omx.quant_rows(ofp8.swiglu(xs))
                else:
                    ofp8.quant_act_1x128(ofp8.swiglu(xs))
            used += time.perf_counter() - t0
            nrows += xs.shape[0]
        out["cpu_baseline"] = {"value": nbytes / total * nrows / used / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{nrows} rows of the same input through the numpy oracle ({used:.1f} s)"}
    print(json.dumps(out), flush=True)


def bench_route(args, prob, es, W):
    """Routing metadata (counts, offsets, packing order) + row packing for the workload's expert row counts:
    one pair per packed row, in a shuffled order, as a router would emit them."""
    import numpy as np

    dev = "cuda:0"
    e, n, k, total = prob.num_experts, prob.n, prob.k, prob.total_rows
    rng = np.random.default_rng(args.seed)
    ids = np.repeat(np.arange(e, dtype=np.int32), prob.rows)
    rng.shuffle(ids)
    d_ids = torch.from_numpy(ids).to(dev)
    x = torch.randn((total, k), generator=torch.Generator().manual_seed(args.seed)).to(torch.bfloat16).to(dev)
    packed = torch.empty_like(x)

    def step():
        ps, eo, bso, dst = es.es_route_metadata(d_ids, 0, e, n, k)
        es.es_permute_rows(x, dst, 1, packed)

    settle(step, args.settle_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = start.elapsed_time(stop) / args.steps
    nbytes = float(total) * (k * 2 * 2 + 4 * 3)    # rows read and written once, ids read twice, dst_row written
    t = ms_per_step * 1e-3
    roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": W.HBM_BYTES_PER_S / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None
    roof["algorithmic_bytes"] = nbytes
    roof["roofline_us"] = nbytes / W.HBM_BYTES_PER_S * 1e6
    out = {
        "metric": "routing metadata + row packing, algorithmic GB/s (4 kernels)",
        "value": nbytes / t / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32 ids, bf16 rows", "data": "synthetic",
        "config": {"workload": f"{prob.name} route: E={e} K={k} pairs={total} seed={args.seed}"},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        from oracle import routing as oroute

        used, reps = 0.0, 0
        xs = x[: min(total, 2048)].float().cpu().numpy()
        while used < args.cpu_seconds:
            t0 = time.perf_counter()
            r = oroute.route_metadata(ids, 0, e, n, k)
            oroute.permute_rows(xs, r[3][: xs.shape[0]] % xs.shape[0], 1, xs.shape[0])
            used += time.perf_counter() - t0
            reps += 1
        out["cpu_baseline"] = {"value": reps * (total * 12.0 + xs.size * 8.0) / used / 1e9, "unit": "GB/s", "cores": 1,
                               "kind": "port", "sample": f"{reps} passes: all ids, first {xs.shape[0]} rows packed ({used:.1f} s)"}
    print(json.dumps(out), flush=True)


def bench_quant_weight(args, prob, es, W):
    """Quantisation of the workload's bf16 weights [E, N, K] (offline operand preparation): FP8 128x128 blocks
    for the fp8-blockwise workloads, MXFP8 with swizzled E8M0 scales for the mxfp8 workload."""
    dev = "cuda:0"
    mx = prob.kind == "mxfp8"
    e, n, k = prob.num_experts, prob.n, prob.k
    gen = torch.Generator().manual_seed(args.seed)
    w1 = (torch.randn((n, k), generator=gen) * 0.02).to(torch.bfloat16)
    w = w1.to(dev).unsqueeze(0).repeat(e, 1, 1).contiguous()     # same values in every expert: timing does not depend on them
    q = torch.empty((e, n, k), dtype=torch.uint8, device=dev)
    sc = (torch.empty((e, n, k // 32), dtype=torch.uint8, device=dev) if mx else
          torch.empty((e, n // 128, k // 128), dtype=torch.float32, device=dev))

    def step():
        if mx:
            es.es_mxfp8_quant_weight(w, q, sc)
        else:
            es.es_fp8_quant_weight_128x128(w, q, sc)

    settle(step, args.settle_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = start.elapsed_time(stop) / args.steps
    nbytes = float(e) * n * k * 3 + (float(e) * n * (k // 32) if mx else float(e) * (n // 128) * (k // 128) * 4)
    t = ms_per_step * 1e-3
    roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": W.HBM_BYTES_PER_S / 1e9, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get((prob.name, args.op))
    roof["algorithmic_bytes"] = nbytes
    roof["roofline_us"] = nbytes / W.HBM_BYTES_PER_S * 1e6
    out = {
        "metric": ("MXFP8 weight quantisation, algorithmic GB/s (bf16 in, e4m3 + E8M0 scales out)" if mx else
                   "FP8 128x128 weight quantisation, algorithmic GB/s (bf16 in, e4m3 + fp32 scales out)"),
        "value": nbytes / t / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 -> fp8_e4m3 + " + ("e8m0 scales" if mx else "fp32 scales"), "data": "synthetic",
        "config": {"workload": f"{prob.name} quant_weight: E={e} N={n} K={k} seed={args.seed}"},
        "roofline": roof,
    }
    if args.calibration_copy:
        calibration_copy()
    if not args.no_cpu_baseline:
        from oracle import fp8_blockwise as ofp8
        from oracle import mxfp8 as omx

        ws = w1[: min(n, 512)].float().numpy()
        used, nrows = 0.0, 0
        while used < args.cpu_seconds:
            t0 = time.perf_counter()
            if mx:
                omx.quant_rows(ws)
            else:
                ofp8.quant_weight_128x128(ws)
            used += time.perf_counter() - t0
            nrows += ws.shape[0]
        out["cpu_baseline"] = {"value": nrows * k * 3.0 / used / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{nrows} weight rows through the numpy oracle ({used:.1f} s)"}
    print(json.dumps(out), flush=True)


class GemmCase:
    """Operands of one grouped-GEMM workload on the GPU and the ways to call it."""

    def __init__(self, es, native, W, prob, dev, seed):
        self.es, self.native, self.lib, self.W, self.prob, self.dev = es, native, native.lib, W, prob, dev
        self.mx = prob.kind == "mxfp8"
        self.ops = (W.make_mxfp8_operands if self.mx else W.make_fp8_blockwise_operands)(prob, dev, seed=seed)
        self.ws_bytes = self.lib.esmoe_gemm_workspace_bytes(prob.num_experts)
        self.ws = torch.empty((self.ws_bytes,), dtype=torch.uint8, device=dev)

    def op_step(self):
        """The operator as the reference's callers call it (torch.ops.expert_specialization.*)."""
        es, ops = self.es, self.ops
        if self.mx:
            def step():
                es.es_sm100_mxfp8_blockscaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                         ops["problem_sizes"], ops["expert_offsets"],
                                                         ops["blockscale_offsets"])
        else:
            def step():
                es.es_fp8_blockwise_scaled_grouped_mm(ops["output"], ops["a"], ops["b"], ops["scales_a"], ops["scales_b"],
                                                      ops["stride_a"], ops["stride_b"], ops["stride_d"],
                                                      ops["problem_sizes"], ops["expert_offsets"], ops["workspace"])
        return step

    def forced_step(self, force_bm):
        """Single-tile-shape baseline: same kernel, one M-tile height for every expert (C ABI only)."""
        import ctypes

        lib, ops, prob, native = self.lib, self.ops, self.prob, self.native
        e, n, k, total = prob.num_experts, prob.n, prob.k, prob.total_rows
        ws, ws_bytes = self.ws, self.ws_bytes

        def vp(t):
            return ctypes.c_void_p(t.data_ptr())

        def step():
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            if self.mx:
                rc = lib.esmoe_mxfp8_grouped_mm(vp(ops["output"]), 0, vp(ops["a"]), vp(ops["b_phys"]), vp(ops["sfa"]),
                                                vp(ops["sfb_phys"]), vp(ops["problem_sizes"]), vp(ops["expert_offsets"]),
                                                vp(ops["blockscale_offsets"]), e, total, n, k, force_bm, vp(ws),
                                                ws_bytes, stream)
            else:
                rc = lib.esmoe_fp8_blockwise_grouped_mm(vp(ops["output"]), 0, vp(ops["a"]), vp(ops["b_phys"]),
                                                        vp(ops["scales_a"]), vp(ops["scales_b_phys"]),
                                                        vp(ops["problem_sizes"]), vp(ops["expert_offsets"]), e, total, n,
                                                        k, force_bm, vp(ws), ws_bytes, stream)
            assert rc == 0, native.last_error()
        return step

    def fused_step(self):
        es, ops, prob, dev = self.es, self.ops, self.prob, self.dev
        n, total = prob.n, prob.total_rows
        assert n % 256 == 0, "--fuse-swiglu needs N a multiple of 256"
        q_f = torch.empty((total, n // 2), dtype=torch.uint8, device=dev)
        if self.mx:
            sf_f = torch.empty((ops["sfa"].shape[0], n // 64), dtype=torch.uint8, device=dev)

            def step():
                es.es_mxfp8_blockscaled_grouped_mm_swiglu_quant(q_f, sf_f, ops["a"], ops["b"], ops["sfa"], ops["sfb"],
                                                                ops["problem_sizes"], ops["expert_offsets"],
                                                                ops["blockscale_offsets"])
        else:
            sc_f = torch.empty((total, n // 256), dtype=torch.float32, device=dev)

            def step():
                es.es_fp8_blockwise_scaled_grouped_mm_swiglu_quant(q_f, sc_f, ops["a"], ops["b"], ops["scales_a"],
                                                                   ops["scales_b"], ops["problem_sizes"],
                                                                   ops["expert_offsets"], ops["workspace"])
        return step

    def single_tile_sweep(self, schedule_ms, warmup, steps):
        """The best any single tile height does on this workload, on the same kernel and the same operands."""
        sweep = {}
        for bm in (16, 32, 64, 128, 192):
            fn = self.forced_step(bm)
            for _ in range(warmup):
                fn()
            torch.cuda.synchronize()
            sweep[bm] = min(time_batches(fn, steps, 2)) * 1e3
        best = min(sweep, key=sweep.get)
        return {"us_by_tile_rows": sweep, "best_single_tile_rows": best, "best_single_tile_us": sweep[best],
                "device_schedule_us": schedule_ms * 1e3, "ratio": sweep[best] / (schedule_ms * 1e3)}


def secondary(args, es, native, W, dev):
    """The other workloads of the path, measured after the timed region of the default run (never part of `value`):
    each is kept on the GPU for 100 ms untimed, then timed as three batches of 30 steps (mean of all, fastest batch).
    GEMM entries go through the operator like the headline; fractions are of the workload's own roofline."""
    sec = {}

    def timed(step, steps=30):
        settle(step, 100.0)
        b = time_batches(step, steps, 3)
        return sum(b) / len(b), min(b)

    def gemm_entry(name, sweep=False, **kw):
        prob = W.config_problem(name, seed=args.seed, **kw)
        case = GemmCase(es, native, W, prob, dev, args.seed)
        ms, ms_min = timed(case.op_step())
        flops = W.gemm_flops(prob.rows, prob.n, prob.k)
        nbytes = W.gemm_bytes(prob.rows, prob.n, prob.k, prob.kind)
        t_roof = W.gemm_roofline_seconds(prob.rows, prob.n, prob.k, prob.kind)
        ent = {"workload": f"{prob.name}: E={prob.num_experts} K={prob.k} N={prob.n} rows={prob.total_rows} kind={prob.kind}",
               "us": ms * 1e3, "min_us": ms_min * 1e3, "tflops": flops / (ms * 1e-3) / 1e12,
               "bound": "hbm" if nbytes / W.HBM_BYTES_PER_S >= flops / W.FP8_FLOPS_PER_S else "mfma",
               "roofline_us": t_roof * 1e6, "frac": t_roof / (ms * 1e-3)}
        if sweep:
            st = case.single_tile_sweep(ms, 20, 30)
            ent["single_tile_sweep"] = {"us_by_tile_rows": st["us_by_tile_rows"], "best_single_tile_rows": st["best_single_tile_rows"],
                                        "ratio": st["ratio"]}
        sec[prob.name] = ent
        return prob, case

    gemm_entry("c2", sweep=True)
    torch.cuda.empty_cache()
    prob4, case4 = gemm_entry("c4")
    # c4 stage 1: the MXFP8 grouped quantisation of the same rows
    x = case4.ops["a_hp"]
    o = case4.ops
    q = torch.empty((prob4.total_rows, prob4.k), dtype=torch.uint8, device=dev)
    sf = torch.zeros_like(o["sfa"])

    def quant_step():
        es.es_sm100_mxfp8_blockscaled_grouped_quant(x, o["problem_sizes"], o["expert_offsets"], o["blockscale_offsets"], q, sf)

    ms, ms_min = timed(quant_step, steps=100)
    qb = W.quant_bytes(prob4.rows, prob4.k)
    sec["c4_quant"] = {"workload": f"c4 stage 1: {prob4.total_rows} x {prob4.k} bf16 -> e4m3 + E8M0", "us": ms * 1e3, "min_us": ms_min * 1e3,
                       "gb_per_s": qb / (ms * 1e-3) / 1e9, "bound": "hbm", "roofline_us": qb / W.HBM_BYTES_PER_S * 1e6,
                       "frac": qb / W.HBM_BYTES_PER_S / (ms * 1e-3)}
    del case4, x, o, q, sf
    torch.cuda.empty_cache()
    gemm_entry("c3", tokens=16384, routing="uniform")
    torch.cuda.empty_cache()
    gemm_entry("dense")
    torch.cuda.empty_cache()
    gemm_entry("dense_mx")
    torch.cuda.empty_cache()
    return sec


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import expert_specialization_moe_amd as es
    from expert_specialization_moe_amd import _native
    from expert_specialization_moe_amd import workloads as W

    dev = "cuda:0"
    torch.cuda.set_device(0)
    prob = W.config_problem(args.config, seed=args.seed, tokens=args.tokens, routing=args.routing)
    if args.op == "quant_weight":
        bench_quant_weight(args, prob, es, W)
        return
    if args.op == "route":
        bench_route(args, prob, es, W)
        return
    if args.op == "swiglu_quant":
        bench_swiglu_quant(args, prob, es, W)
        return
    if args.op != "gemm":
        bench_quant(args, prob, es, W)
        return
    case = GemmCase(es, _native, W, prob, dev, args.seed)
    mx, ops = case.mx, case.ops
    e, n, k, total = prob.num_experts, prob.n, prob.k, prob.total_rows

    if args.fuse_swiglu:
        step = case.fused_step()
    elif args.force_bm:
        step = case.forced_step(args.force_bm)
    else:
        step = case.op_step()

    settle(step, args.settle_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = start.elapsed_time(stop) / args.steps
    # outside the timed region: the fastest of the timed batch and five more of the same length
    min_ms_per_step = min([ms_per_step] + time_batches(step, args.steps, 5))

    flops = W.gemm_flops(prob.rows, n, k)
    nbytes = W.gemm_bytes(prob.rows, n, k, prob.kind)
    t_roof = W.gemm_roofline_seconds(prob.rows, n, k, prob.kind)
    if args.fuse_swiglu:
        # e4m3 + scales (fp32 per 128 columns, or one byte per 32) written instead of bf16
        nbytes += total * (n / 2 + (n / 64 if mx else 4.0 * n / 256)) - 2.0 * n * total
        t_roof = max(flops / W.FP8_FLOPS_PER_S, nbytes / W.HBM_BYTES_PER_S)
    t = ms_per_step * 1e-3
    hbm_bound = nbytes / W.HBM_BYTES_PER_S >= flops / W.FP8_FLOPS_PER_S
    if hbm_bound:
        roof = {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": W.HBM_BYTES_PER_S / 1e9, "unit": "GB/s"}
    else:
        roof = {"bound": "mfma", "achieved": flops / t / 1e12, "peak": W.FP8_FLOPS_PER_S / 1e12, "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get((prob.name, "gemm")) if not (args.force_bm or args.fuse_swiglu) else None
    roof["algorithmic_bytes"] = nbytes
    roof["roofline_us"] = t_roof * 1e6
    roof["per_expert_roofline_us"] = W.gemm_roofline_per_expert_seconds(prob.rows, n, k, prob.kind) * 1e6
    out = {
        "metric": "useful FP8 TFLOP/s + % of roofline, DSv3-shape grouped GEMM, Zipf routing",
        "value": flops / t / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "ms_per_step": ms_per_step, "min_ms_per_step": min_ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)", "data": "synthetic",
        "config": {"workload": f"{prob.name}: E={e} K={k} N={n} rows={total} max_rows={max(prob.rows)} "
                               f"active={sum(1 for m in prob.rows if m)} kind={prob.kind} seed={args.seed}",
                   "force_bm": args.force_bm, "fuse_swiglu": bool(args.fuse_swiglu), "routing_meta": prob.meta},
        "roofline": roof, "wall_ms_per_step": wall * 1e3 / args.steps,
    }
    if args.single_tile_sweep:
        out["single_tile_sweep"] = case.single_tile_sweep(ms_per_step, args.warmup, args.steps)
    if args.calibration_copy:
        calibration_copy()
    plain_default = args.config == "c1" and not (args.force_bm or args.fuse_swiglu)
    if plain_default and not args.no_secondary:
        cpu_ops = None if args.no_cpu_baseline else {key: (v.cpu() if torch.is_tensor(v) else v) for key, v in ops.items()
                                                       if key in ("a", "b_phys", "scales_a", "scales_b_phys")}
        del step, case, ops
        torch.cuda.empty_cache()
        out["secondary"] = secondary(args, es, _native, W, dev)
        if cpu_ops is not None:
            out["cpu_baseline"] = cpu_baseline(prob, cpu_ops, args.cpu_seconds)
    elif not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(prob, ops, args.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
