#!/usr/bin/env python3
"""Benchmark of the Q4_K x Q8_K hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (BASELINE.json configs[1]): the dense FFN-shaped skinny GEMM -- Q4_K gate/up
4096->14336 (fused with the SiLU gate) and down 14336->4096 -- at the decode widths
n = 1, 2, 4, 8, 16.  One step = one FFN pass at each of the five widths, each pass on the next
weight set of a ring of distinct sets (792 MB, larger than every cache level), so the weights
always come from HBM.  Activations and weights are resident in HBM before the timed region; the
steps are replayed as HIP graphs (what a serving loop does) unless --eager is given.

Prints one JSON line: whole-job GB/s over the algorithmic bytes (weights once, fp32 activations in,
fp32 outputs out), the roofline of the dominant kernel (fused gate/up), and the CPU baseline (the
oracle's threaded SIMD build -- AVX-512 VNNI where the host has it, AVX2 beside it -- on this box's host cores, bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HIDDEN, INTER = 4096, 14336
WIDTHS = (1, 2, 4, 8, 16)
RING = 8
HBM_PEAK_GBPS = 8000.0
INT8_PEAK_TOPS = 5000.0          # dense int8 MFMA, MI355X
# HBM bytes per launch of the dominant kernel, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of
# `bench.py --kernel-only`: 32,585.1 KiB fetched and 210.0 KiB written per dispatch on average, each scaled by what
# the same counter reads for the 256 MiB copy of `bench.py --copy-calibration` (FETCH_SIZE 131,083.8 KiB -> x2.000,
# WRITE_SIZE 262,144.0 KiB -> x1.000): 66,728,000 B read + 215,000 B written.
TRAFFIC_BYTES_PER_LAUNCH = 66943000
Q4K_MATRIX_BYTES = INTER * (HIDDEN // 256) * 144          # 33,030,144: the same for gate, up and down


def ffn_bytes(n: int) -> int:
    """Algorithmic bytes of one FFN pass: three weight matrices once, fp32 x in, fp32 y out."""
    return 3 * Q4K_MATRIX_BYTES + n * (HIDDEN * 4 + HIDDEN * 4)


def gateup_bytes(n: int) -> int:
    """Algorithmic bytes of one fused gate/up launch: two matrices, fp32 x in, fp32 hidden out."""
    return 2 * Q4K_MATRIX_BYTES + n * (HIDDEN * 4 + INTER * 4)


def moe_bytes(n: int, distinct: int) -> int:
    """One MoE layer (hidden 2048, inter 512): distinct routed experts + the shared one, x in, y out."""
    return (distinct + 1) * 3 * 512 * 8 * 144 + n * (2048 * 4 * 2)


def main() -> int:
    global RING
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--eager", action="store_true", help="launch from Python every step instead of replaying HIP graphs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the GEMV / MoE side measurements")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a 256 MiB device-to-device copy kernel 20 times (the known-size reference for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings) and exit")
    ap.add_argument("--kernel-only-n16", action="store_true",
                    help="the same for the n = 16 form of the launch (skinny16_kernel<2,2,...>: the rows as one tile of sixteen)")
    ap.add_argument("--kernel-only", action="store_true",
                    help="only run the back-to-back launches of the dominant kernel (for counter passes) and exit")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only run the 14336x4096 prefill GEMM at M = 2048 ten times (for counter passes) and exit")
    ap.add_argument("--decode-step-only", type=int, default=0, metavar="N",
                    help="only replay the 40-layer decoder step at N tokens ten times, one launch per graph node (for kernel traces), and exit")
    ap.add_argument("--skeleton", action="store_true",
                    help="with --decode-step-only: time the step's graph, then the same graph captured with every kernel body "
                         "compiled out (mq_debug_set_skeleton: empty kernels of the same grid, block and LDS size) -- the "
                         "cost of the dependent launches alone")
    ap.add_argument("--moe-layer-only", type=int, default=0, metavar="N",
                    help="only run the cfg3 MoE layer (256 + 1 experts, 2048 x 512, top-8) at N tokens forty times over a ring "
                         "of 4 layers (for kernel traces), and exit")
    ap.add_argument("--ring", type=int, default=RING, help="distinct weight sets visited round-robin (1 = cache-hot)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU (one MI355X per box); --gpus N with N > 1 is not run "
              "(the design notes say how the path would shard over more GPUs).", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from densecore_amd import ops, synth

    RING = max(1, args.ring)

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": src.numel(), "bytes_written": dst.numel(), "launches": 20}))
        return 0

    if args.prefill_only:
        W = ops.Q4KWeight.synthetic(synth.tensor_seed("cfg4"), 14336, 4096)
        x = torch.randn((2048, 4096), device=dev, generator=torch.Generator(device=dev).manual_seed(2048))
        y = torch.empty((2048, 14336), dtype=torch.float32, device=dev)
        for _ in range(10):
            ops.gemm(W, x, out=y)
        torch.cuda.synchronize()
        print(json.dumps({"prefill_only": "prefill_gemm_kernel", "M": 2048, "launches": 10}))
        return 0

    if args.decode_step_only:
        from densecore_amd import decode_step
        n = args.decode_step_only
        cfg = decode_step.StepConfig(synthetic_logits=True)
        st = decode_step.DecodeStep(cfg, n)
        x = torch.randn((n, cfg.hidden), device=dev, generator=torch.Generator(device=dev).manual_seed(100 + n))
        st.run(x)
        torch.cuda.synchronize()
        st.x.copy_(x)
        st.capture()
        for _ in range(10):
            st.replay()
        torch.cuda.synchronize()
        out = {"decode_step_only": n, "layers": cfg.n_layers, "replays": 10}
        if args.skeleton:
            from densecore_amd import _lib

            def timed(step):
                best = float("inf")
                for _ in range(5):
                    t = time.perf_counter()
                    for _ in range(10):
                        step.replay()
                    torch.cuda.synchronize()
                    best = min(best, (time.perf_counter() - t) / 10)
                return best

            full = timed(st)
            _lib.lib().mq_debug_set_skeleton(1)
            try:
                sk = decode_step.DecodeStep(cfg, n, layers=st.layers)
                sk.x.copy_(x)
                sk.capture()
            finally:
                _lib.lib().mq_debug_set_skeleton(0)
            sk.replay()
            torch.cuda.synchronize()
            floor = timed(sk)
            out.update({"ms_per_step": round(full * 1e3, 3), "skeleton_ms_per_step": round(floor * 1e3, 3),
                        "us_per_layer": round(full * 1e6 / cfg.n_layers, 2),
                        "skeleton_us_per_layer": round(floor * 1e6 / cfg.n_layers, 2),
                        "note": "skeleton = the same graph with empty kernels of the same grid, block and LDS size"})
        print(json.dumps(out))
        return 0

    if args.moe_layer_only:
        n = args.moe_layer_only
        E, H, I, K = 256, 2048, 512, 8
        layers = []
        for r in range(4):
            ws = [ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, t), rows, cols, e)
                  for t, rows, cols, e in (("gate", I, H, E), ("up", I, H, E), ("down", H, I, E), ("sg", I, H, 1), ("su", I, H, 1), ("sd", H, I, 1))]
            gi = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3", r, "gi"), (H,)) * np.float32(0.02)).to(dev)
            layers.append((ws[0], ws[1], ws[2], (ws[3], ws[4], ws[5], gi)))
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))).to(dev)
        lg = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))).to(dev)
        silu = ops.SILU_EXACT if n <= 4 else ops.SILU_FAST
        for _ in range(10):
            for ge, ue, de, sh in layers:
                ops.moe_layer(ge, ue, de, x, lg, K, shared=sh, silu=silu)
        torch.cuda.synchronize()
        print(json.dumps({"moe_layer_only": n, "layers": 4, "passes": 10}))
        return 0

    # ---------------------------------------------------------------- resident data
    sets = []
    for r in range(RING):
        sets.append(tuple(ops.Q4KWeight.synthetic(synth.tensor_seed("cfg2", r, nm), rows, cols)
                          for nm, rows, cols in (("gate", INTER, HIDDEN), ("up", INTER, HIDDEN), ("down", HIDDEN, INTER))))
    xs = {n: torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg2-x", n), (n, HIDDEN))).to(dev) for n in WIDTHS}
    torch.cuda.synchronize()

    side_stream = torch.cuda.Stream()
    # The fused gate/up kernel alone, back to back on the cold ring, from pre-quantized activations:
    # HIP events on the replay stream around a graph of launches, divided by the launch count.
    def kernel_leg(widths, reps):
        acts = {n: ops.Q8KActs(n, HIDDEN).quantize(xs[n]) for n in widths}
        outs = {n: torch.empty((n, INTER), dtype=torch.float32, device=dev) for n in widths}

        def launches():
            k = 0
            for i in range(RING):
                for n in widths:
                    g, u, _ = sets[k % RING]
                    acts[n].swiglu_mul_mat(g, u, ops.SILU_FAST_FMA, out=outs[n])
                    k += 1
            return RING * len(widths)

        count = launches()
        torch.cuda.synchronize()
        gph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gph, stream=side_stream):
            launches()
        torch.cuda.synchronize()
        gph.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            gph.replay()
        e1.record()
        torch.cuda.synchronize()
        for a in acts.values():
            a.free()
        return e0.elapsed_time(e1) * 1e3 / (reps * count)     # us per launch

    if args.kernel_only_n16:
        us = kernel_leg((16,), 5)
        print(json.dumps({"kernel_only": "skinny16_kernel<2,2,...>", "avg_us": round(us, 3), "widths": (16,)}))
        return 0
    if args.kernel_only:
        narrow = tuple(n for n in WIDTHS if n <= 8)
        us = kernel_leg(narrow, 5)
        print(json.dumps({"kernel_only": "dense_lds_kernel<2,1,...>", "avg_us": round(us, 3), "widths": narrow}))
        return 0

    def run_step(i: int):
        for j, n in enumerate(WIDTHS):
            g, u, d = sets[(i * len(WIDTHS) + j) % RING]
            ops.ffn_swiglu(g, u, d, xs[n], ops.SILU_FAST_FMA)

    for i in range(RING):          # sizes the library workspace before anything is captured
        run_step(i)
    torch.cuda.synchronize()

    graphs = None
    if not args.eager:
        graphs = []
        side = torch.cuda.Stream()
        for i in range(RING):       # step i and step i + RING touch the same weight sets
            gph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gph, stream=side):
                run_step(i)
            graphs.append(gph)
        torch.cuda.synchronize()

    def step(i: int):
        if graphs is None:
            run_step(i)
        else:
            graphs[i % RING].replay()

    # ---------------------------------------------------------------- timed region
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    step_bytes = sum(ffn_bytes(n) for n in WIDTHS)
    value = step_bytes * args.steps / elapsed / 1e9

    # spread of single steps (outside the timed region): an event after every step, differences of neighbours
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(min(args.steps, 200) + 1)]
    marks[0].record()
    for i in range(len(marks) - 1):
        step(i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    singles = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(len(marks) - 1))
    pick = lambda q: round(singles[min(len(singles) - 1, int(q * len(singles)))], 4)
    step_spread = {"p10_ms": pick(0.10), "p50_ms": pick(0.50), "p90_ms": pick(0.90), "steps": len(singles),
                   "how": "HIP events between consecutive steps, after the timed region"}

    # ---------------------------------------------------------------- dominant kernel, live
    narrow = tuple(n for n in WIDTHS if n <= 8)      # one activation tile:  dense_lds_kernel<2,1,...>
    wide = tuple(n for n in WIDTHS if n > 8)         # nine to sixteen rows as one tile of sixteen: skinny16_kernel<2,2,...>
    # (1) the kernel's own duration: start/stop HIP events that the library binds to every gate/up dispatch
    #     of the same FFN passes the timed region runs (the begin/end timestamps a profiler reports); (2) the same kernel launched back to back from pre-quantized
    #     activations, events around the whole graph replay, per launch (what a pipelined loop pays).
    blocker = [torch.empty(1 << 30, dtype=torch.float32, device=dev) for _ in range(2)]

    def census_leg(widths, passes):
        ops.census_reset()
        ops.census_enable(True)
        for _ in range(6):      # ~10 ms of queued copies: the launches below are all submitted while the GPU is
            blocker[1].copy_(blocker[0])   # still busy, so no event interval contains host submission time
        for i in range(passes):
            for n in widths:
                g, u, d = sets[i % RING]
                ops.ffn_swiglu(g, u, d, xs[n], ops.SILU_FAST_FMA)
        torch.cuda.synchronize()
        ops.census_enable(False)
        r = ops.census_read(ops.KIND_DENSE_SWIGLU)
        ops.census_reset()
        return r

    c_narrow = census_leg(narrow, 32)
    us_narrow = kernel_leg(narrow, 25)
    b_narrow = sum(gateup_bytes(n) for n in narrow) / len(narrow)
    achieved = b_narrow / (c_narrow["avg_us"] * 1e-6) / 1e9
    roofline = {
        "bound": "hbm", "kernel": "dense_lds_kernel<2,1,Q4_K,...> (fused gate/up + SwiGLU, 2 x 14336x4096 Q4_K, activations staged in LDS, n=1,2,4,8)",
        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": TRAFFIC_BYTES_PER_LAUNCH, "bytes_per_launch": int(b_narrow), "avg_us": round(c_narrow["avg_us"], 3),
        "min_us": round(c_narrow["min_us"], 3), "launches": c_narrow["count"],
        "how": "start/stop HIP events bound to each dispatch of the kernel (hipExtLaunchKernelGGL), cold ring",
        "back_to_back": {"avg_us": round(us_narrow, 3), "achieved": round(b_narrow / (us_narrow * 1e-6) / 1e9, 1),
                         "frac": round(b_narrow / (us_narrow * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                         "how": "events around graph replays of 32 launches from pre-quantized activations, per launch"},
    }
    if wide:
        c_wide = census_leg(wide, 128)
        us_wide = kernel_leg(wide, 25)
        b_wide = sum(gateup_bytes(n) for n in wide) / len(wide)
        roofline["n16_kernel"] = {"kernel": "skinny16_kernel<2,2,...> (fused gate/up + SwiGLU at n=16: the rows as one activation tile of sixteen)", "avg_us": round(c_wide["avg_us"], 3),
                                  "achieved": round(b_wide / (c_wide["avg_us"] * 1e-6) / 1e9, 1),
                                  "frac": round(b_wide / (c_wide["avg_us"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                                  "back_to_back_us": round(us_wide, 3)}

    del blocker
    # ---------------------------------------------------------------- per-width detail
    def width_detail(n, x):
        for i in range(RING):
            ops.ffn_swiglu(*sets[i], x, ops.SILU_FAST_FMA)
        torch.cuda.synchronize()
        reps = 256
        t1 = time.perf_counter()
        if graphs is None:
            for i in range(reps):
                ops.ffn_swiglu(*sets[i % RING], x, ops.SILU_FAST_FMA)
        else:
            gph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gph, stream=side_stream):
                for i in range(RING):
                    ops.ffn_swiglu(*sets[i], x, ops.SILU_FAST_FMA)
            gph.replay()            # one untimed replay: the first one also uploads the graph
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(reps // RING):
                gph.replay()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t1) / reps
        return {"us": round(dt * 1e6, 2), "GBps": round(ffn_bytes(n) / dt / 1e9, 1),
                "pct_hbm_peak": round(ffn_bytes(n) / dt / 1e9 / HBM_PEAK_GBPS * 100, 1), "tokens_per_s": round(n / dt, 1)}

    per_width = {str(n): width_detail(n, xs[n]) for n in WIDTHS}
    # the same FFN pass at widths between the workload's sixteen rows and the GEMM's prefill widths (not part of `value`)
    wider = {}
    for n in (24, 32, 48, 64):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg2-x", n), (n, HIDDEN))).to(dev)
        wider[str(n)] = width_detail(n, x)
    wider["note"] = ("the cfg2 FFN pass beyond its widths, same cold ring: gate/up on the decode arithmetic up to 64 rows (up to four "
                     "activation tiles of sixteen per weight tile), down likewise up to 32 rows and on the matrix-core GEMM from 33")

    extras = {}
    if not args.no_extras:
        extras = side_measurements(ops, synth, torch, np, dev)

    # ---------------------------------------------------------------- CPU baseline (rank 0, N = 1)
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(sets[0], xs, args.cpu_seconds, np)

    out = {
        "metric": "Q4_K GEMV + MoE mul_mat_id GB/s (% HBM peak); MoE decode tok/s, 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 x int4 -> int32, fp32 accumulate", "data": "synthetic",
        # the metric names three quantities; `value` is the first of them on the configuration it is quoted on, the others
        # are measured in the same run and reported under their own keys
        "value_is": "the Q4_K GEMV / skinny-GEMM part of the metric: algorithmic GB/s of the cfg2 dense FFN passes; MoE mul_mat_id "
                    "GB/s is in moe_layer_mul_mat_id, MoE decode tok/s in moe_decode_step_40_layers",
        "config": {"workload": "cfg2: dense FFN skinny GEMM, Q4_K gate/up 4096->14336 + SiLU gate + down 14336->4096, "
                               "widths n=1,2,4,8,16 per step, cold ring of 8 weight sets (792 MB)",
                   "launch": "eager" if graphs is None else "hip-graph replay",
                   "bytes_per_step": step_bytes},
        "pct_hbm_peak": round(value / HBM_PEAK_GBPS * 100, 1),
        "step_spread": step_spread,
        "per_width": per_width,
        "ffn_pass_wider": wider,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    out.update(extras)
    print(json.dumps(out))
    return 0


def side_measurements(ops, synth, torch, np, dev):
    """cfg1 GEMV and the cfg3 MoE layer, each on a cold ring, replayed as HIP graphs."""
    res = {}
    side = torch.cuda.Stream()

    def time_graph(fn, reps):
        fn()
        torch.cuda.synchronize()
        gph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gph, stream=side):
            fn()
        torch.cuda.synchronize()
        gph.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            gph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / reps

    # cfg1: 4096 x 4096 GEMV, ring of 64 matrices (604 MB)
    ring = [ops.Q4KWeight.synthetic(synth.tensor_seed("cfg1", r), 4096, 4096) for r in range(64)]
    x1 = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg1-x"), (1, 4096))).to(dev)
    dt = time_graph(lambda: [ops.mul_mat(w, x1) for w in ring], 20) / len(ring)
    b = 4096 * 16 * 144 + 2 * 4096 * 4
    res["gemv_4096x4096_n1"] = {"us": round(dt * 1e6, 2), "GBps": round(b / dt / 1e9, 1),
                                "pct_hbm_peak": round(b / dt / 1e9 / HBM_PEAK_GBPS * 100, 1)}
    # the same launch on ONE matrix over and over (9.4 MB: it stays in the last-level cache) -- not the roofline claim
    dt = time_graph(lambda: [ops.mul_mat(ring[0], x1) for _ in range(64)], 20) / 64
    res["gemv_4096x4096_n1"]["cache_hot_single_matrix_us"] = round(dt * 1e6, 2)
    res["gemv_4096x4096_n1"]["note"] = ("one launch per 9.4 MB: an empty launch in a graph costs 1.6 us and the first bytes of cold weights "
                                        "arrive 2 us after the workgroups start, so the single-matrix call is bound by its launch, not "
                                        "by the memory pipes; gemv_4096x4096_n1_four_per_launch is the same work with four matrices "
                                        "handed over together (mq_mul_mat_q4k_multi)")
    # four matrices of the ring per launch on the same activation row (a layer's projections handed over together)
    outs = [torch.empty((4096,), dtype=torch.float32, device=dev) for _ in range(4)]
    dt = time_graph(lambda: [ops.mul_mat_multi(ring[i:i + 4], x1, outs) for i in range(0, len(ring), 4)], 20) / (len(ring) // 4)
    b4 = 4 * 4096 * 16 * 144 + (1 + 4) * 4096 * 4
    res["gemv_4096x4096_n1_four_per_launch"] = {"us": round(dt * 1e6, 2), "us_per_matrix": round(dt * 1e6 / 4, 2),
                                                "GBps": round(b4 / dt / 1e9, 1),
                                                "pct_hbm_peak": round(b4 / dt / 1e9 / HBM_PEAK_GBPS * 100, 1)}
    for w in ring:
        w.free()

    # the sibling K-quant types through the same decode kernels: the FFN down projection 14336 -> 4096 at n = 1 and 8,
    # and at 16 and 32 rows (one and two activation tiles of sixteen), on a ring of 12 matrices per type
    # (Q4_K 396 MB, Q5_K 484 MB, Q6_K 578 MB)
    sib = {}
    for name, gtype, bb in (("Q4_K", synth.GGML_TYPE_Q4_K, 144), ("Q5_K", synth.GGML_TYPE_Q5_K, 176),
                            ("Q6_K", synth.GGML_TYPE_Q6_K, 210)):
        ring = [ops.Q4KWeight.synthetic(synth.tensor_seed("sib", name, r), 4096, 14336, 1, gtype) for r in range(12)]
        per = {}
        for n in (1, 8, 16, 32):
            acts = ops.Q8KActs(n, 14336).quantize(torch.from_numpy(synth.normal_f32(synth.tensor_seed("sib-x", n), (n, 14336))).to(dev))
            y = torch.empty((n, 4096), dtype=torch.float32, device=dev)
            dt = time_graph(lambda: [acts.mul_mat(w, out=y) for w in ring], 20) / len(ring)
            b = 4096 * 56 * bb + n * (14336 + 4096) * 4
            per[str(n)] = {"us": round(dt * 1e6, 2), "GBps": round(b / dt / 1e9, 1),
                           "pct_hbm_peak": round(b / dt / 1e9 / HBM_PEAK_GBPS * 100, 1)}
            acts.free()
        sib[name] = per
        for w in ring:
            w.free()
    sib["note"] = "matmul from pre-quantized activations, 4096 x 14336 weights, bytes = ggml bytes of the type + fp32 in/out"
    res["down_projection_by_weight_type"] = sib

    # Q8_0 weights against Q8_0 activations (the reference's vec_dot_type for the type): the same shape, quantizer
    # launch included, ring of 10 matrices (624 MB)
    ring = [ops.Q4KWeight.synthetic(synth.tensor_seed("sib", "Q8_0", r), 4096, 14336, 1, synth.GGML_TYPE_Q8_0) for r in range(10)]
    per = {}
    for n in (1, 8):
        xq = torch.from_numpy(synth.normal_f32(synth.tensor_seed("sib-x", n), (n, 14336))).to(dev)
        y = torch.empty((n, 4096), dtype=torch.float32, device=dev)
        dt = time_graph(lambda: [ops.mul_mat(w, xq, out=y) for w in ring], 20) / len(ring)
        b = 4096 * (14336 // 32) * 34 + n * (14336 + 4096) * 4
        per[str(n)] = {"us": round(dt * 1e6, 2), "GBps": round(b / dt / 1e9, 1),
                       "pct_hbm_peak": round(b / dt / 1e9 / HBM_PEAK_GBPS * 100, 1)}
    per["note"] = "quantize (Q8_0) + matmul, two launches, 4096 x 14336 weights, bytes = ggml bytes + fp32 in/out"
    res["q8_0_projection"] = per
    for w in ring:
        w.free()

    # the same entry point on the largest matrix of a model, the output projection (a 128,256-token vocabulary, hidden
    # 4096; Q6_K in a Q4_K_M file): what the kernels reach on a launch of several hundred MB, quantizer included
    outp = {}
    for name, gtype, bb in (("Q4_K", synth.GGML_TYPE_Q4_K, 144), ("Q6_K", synth.GGML_TYPE_Q6_K, 210)):
        ring = [ops.Q4KWeight.synthetic(synth.tensor_seed("outp", name, r), 128256, 4096, 1, gtype) for r in range(2)]
        per = {}
        for n in (1, 8, 16):
            x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("outp-x", n), (n, 4096))).to(dev)
            y = torch.empty((n, 128256), dtype=torch.float32, device=dev)
            dt = time_graph(lambda: [ops.mul_mat(w, x, out=y) for w in ring], 10) / len(ring)
            b = 128256 * 16 * bb + n * (4096 + 128256) * 4
            per[str(n)] = {"us": round(dt * 1e6, 1), "GBps": round(b / dt / 1e9, 1),
                           "pct_hbm_peak": round(b / dt / 1e9 / HBM_PEAK_GBPS * 100, 1)}
        outp[name] = per
        for w in ring:
            w.free()
    outp["note"] = "mq_mul_mat_q4k (quantizer included), 128256 x 4096 weights, two matrices alternating, bytes = ggml bytes of the type + fp32 in/out"
    res["output_projection_128256x4096"] = outp

    # cfg3: MoE layer, hidden 2048, 256 + 1 experts, inter 512, top-8; ring of 4 layers (1.8 GB)
    E, H, I, K = 256, 2048, 512, 8
    layers = []
    for r in range(4):
        ge = ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "gate"), I, H, E)
        ue = ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "up"), I, H, E)
        de = ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "down"), H, I, E)
        sh = (ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "sg"), I, H),
              ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "su"), I, H),
              ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "sd"), H, I),
              torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3", r, "gi"), (H,)) * np.float32(0.02)).to(dev))
        layers.append((ge, ue, de, sh))
    moe = {}
    for n in (1, 4, 16, 64):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))).to(dev)
        lg = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))).to(dev)
        silu = ops.SILU_EXACT if n <= 4 else ops.SILU_FAST
        _, ids, _ = ops.moe_layer(*layers[0][:3], x, lg, K, shared=layers[0][3], silu=silu)
        distinct = int(torch.unique(ids).numel())
        dt = time_graph(lambda: [ops.moe_layer(ge, ue, de, x, lg, K, shared=sh, silu=silu)
                                 for ge, ue, de, sh in layers], 20) / len(layers)
        b = moe_bytes(n, distinct)
        moe[str(n)] = {"us": round(dt * 1e6, 2), "distinct_experts": distinct, "GBps": round(b / dt / 1e9, 1),
                       "pct_hbm_peak": round(b / dt / 1e9 / HBM_PEAK_GBPS * 100, 1), "tokens_per_s": round(n / dt, 1)}
    res["moe_layer_mul_mat_id"] = moe
    # the same block at prefill widths: its expert products on the int8 matrix cores (expert-grouped GEMM)
    moe_pf = {}
    for n in (512, 2048):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))).to(dev)
        lg = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))).to(dev)
        dt = time_graph(lambda: [ops.moe_layer(ge, ue, de, x, lg, K, shared=sh, silu=ops.SILU_FAST)
                                 for ge, ue, de, sh in layers], 5) / len(layers)
        tops = 2.0 * n * (K + 1) * 3 * H * I / dt / 1e12
        moe_pf[str(n)] = {"us": round(dt * 1e6, 1), "TOPs": round(tops, 1), "pct_int8_mfma_peak": round(tops / INT8_PEAK_TOPS * 100, 2),
                          "tokens_per_s": round(n / dt, 1)}
    moe_pf["note"] = "useful ops 2 * tokens * (top_k + shared) * 3 matrices * 2048 * 512 over the whole block (routing, gather, combine included)"
    res["moe_layer_prefill"] = moe_pf
    # the layer a Q4_K_M file holds: Q4_K gate/up stacks with Q6_K down experts (the shared expert's down Q6_K too)
    down6 = [(ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "down6"), H, I, E, synth.GGML_TYPE_Q6_K),
              ops.Q4KWeight.synthetic(synth.tensor_seed("cfg3", r, "sd6"), H, I, 1, synth.GGML_TYPE_Q6_K)) for r in range(len(layers))]
    moe_pf6 = {}
    for n in (512, 2048):
        x = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-x", n), (n, H))).to(dev)
        lg = torch.from_numpy(synth.normal_f32(synth.tensor_seed("cfg3-l", n), (n, E))).to(dev)
        dt = time_graph(lambda: [ops.moe_layer(ge, ue, d6, x, lg, K, shared=(sh[0], sh[1], sd6, sh[3]), silu=ops.SILU_FAST)
                                 for (ge, ue, de, sh), (d6, sd6) in zip(layers, down6)], 5) / len(layers)
        tops = 2.0 * n * (K + 1) * 3 * H * I / dt / 1e12
        moe_pf6[str(n)] = {"us": round(dt * 1e6, 1), "TOPs": round(tops, 1), "pct_int8_mfma_peak": round(tops / INT8_PEAK_TOPS * 100, 2),
                           "tokens_per_s": round(n / dt, 1)}
    moe_pf6["note"] = "the same block with Q6_K down experts (gate/up Q4_K): all three expert products on the matrix-core GEMM"
    res["moe_layer_prefill_q6k_down"] = moe_pf6
    for d6, sd6 in down6:
        d6.free()
        sd6.free()
    for ge, ue, de, sh in layers:
        for w in (ge, ue, de) + sh[:3]:
            w.free()

    # cfg4: prefill GEMM 4096 -> 14336 on the int8 matrix cores, quantizer included
    W = ops.Q4KWeight.synthetic(synth.tensor_seed("cfg4"), 14336, 4096)
    pre = {}
    for m in (512, 2048):
        x = torch.randn((m, 4096), device=dev, generator=torch.Generator(device=dev).manual_seed(m))
        y = torch.empty((m, 14336), dtype=torch.float32, device=dev)
        dt = time_graph(lambda: [ops.gemm(W, x, out=y) for _ in range(4)], 10) / 4
        tops = 2.0 * m * 4096 * 14336 / dt / 1e12
        pre[str(m)] = {"us": round(dt * 1e6, 1), "TOPs": round(tops, 1),
                       "pct_int8_mfma_peak": round(tops / INT8_PEAK_TOPS * 100, 2),
                       "pct_int8_mfma_peak_issued": round(tops * 2.25 / INT8_PEAK_TOPS * 100, 2),
                       "tokens_per_s": round(m / dt, 1)}
    pre["note"] = ("useful ops 2*M*N*K over quantize + GEMM time; 'issued' counts the 9 MFMAs of equal duration the "
                   "kernel issues per 4 a plain int8 GEMM would (two scale digits x 4 int8, one fp16 for the min term)")
    res["prefill_gemm_4096x14336"] = pre
    W.free()

    # cfg5: 40-layer synthetic MoE decoder step, one HIP graph per width
    from densecore_amd import decode_step
    cfg = decode_step.StepConfig(synthetic_logits=True)   # router logits N(0,1), as the MoE block is specified
    base = decode_step.DecodeStep(cfg, 1)
    steps = {}
    for n in (1, 4, 8):
        st = base if n == 1 else decode_step.DecodeStep(cfg, n, layers=base.layers)
        x = torch.randn((n, cfg.hidden), device=dev, generator=torch.Generator(device=dev).manual_seed(100 + n))
        st.run(x)
        torch.cuda.synchronize()
        distinct = [int(torch.unique(st.ids[i]).numel()) for i in range(cfg.n_layers)]
        st.x.copy_(x)
        st.capture()
        st.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        reps = 10
        for _ in range(reps):
            st.replay()
        torch.cuda.synchronize()
        dt_nodes = (time.perf_counter() - t) / reps
        # the same layers as one persistent launch (mq_decoder_step)
        fz = decode_step.FusedDecodeStep(cfg, n, base.layers, st.fixed_logits)
        fz.x.copy_(x)
        fz.capture()
        fz.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            fz.replay()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / reps
        fz.status()
        same = bool(torch.equal(fz.ids, st.ids))
        fz.free()
        q4 = lambda r, c: r * c // 256 * 144
        per_expert = 2 * q4(cfg.inter, cfg.hidden) + q4(cfg.hidden, cfg.inter)
        fixed = per_expert + q4(cfg.n_q + 2 * cfg.n_kv, cfg.hidden) + q4(cfg.hidden, cfg.n_q) + cfg.n_experts * cfg.hidden * 4
        step_bytes = sum(d * per_expert + fixed + n * cfg.hidden * 8 for d in distinct)
        dt_fused = dt
        dt = min(dt_fused, dt_nodes)
        steps[str(n)] = {"launch": ("one persistent kernel per step (mq_decoder_step)" if dt_fused <= dt_nodes
                                    else "one launch per graph node, HIP-graph replay"),
                         "same_experts_both_ways": same,
                         "persistent_kernel_ms_per_step": round(dt_fused * 1e3, 3),
                         "node_by_node_ms_per_step": round(dt_nodes * 1e3, 3),
                         "ms_per_step": round(dt * 1e3, 3), "tokens_per_s": round(n / dt, 1),
                         "us_per_layer": round(dt * 1e6 / cfg.n_layers, 2),
                         "distinct_experts_per_layer": round(sum(distinct) / len(distinct), 1),
                         "per_layer_GBps": round(step_bytes / cfg.n_layers / (dt / cfg.n_layers) / 1e9, 1),
                         "pct_hbm_peak": round(step_bytes / dt / 1e9 / HBM_PEAK_GBPS * 100, 2)}
    steps["weights_GB"] = round(cfg.layer_weight_bytes() * cfg.n_layers / 1e9, 2)
    res["moe_decode_step_40_layers"] = steps
    base.free()
    return res


def cpu_baseline(weight_set, xs, seconds, np):
    """The oracle's threaded SIMD build on this box's host cores: the same FFN passes (all five widths) on weight set
    0, repeated for about `seconds` of CPU work.  The widest kernel the reference has for the path is timed: its
    AVX-512 VNNI form where the host has the instructions, else the AVX2 form (which is then also the second figure)."""
    from oracle import binding as orc
    g, u, d = (w.to_ggml() for w in weight_set)
    allowed = len(os.sched_getaffinity(0))
    threads = max(1, min(16, allowed))    # a one-GPU box gives a job 16 cores' worth of the host, whatever it shows
    x_host = {n: xs[n].cpu().numpy() for n in WIDTHS}
    best = "vnni" if orc.host_has_vnni() else "avx2"

    def timed(isa, nthreads, budget, widths):
        orc.simd_ffn_swiglu(g, u, d, HIDDEN, INTER, x_host[1], nthreads, isa=isa)   # page everything in
        done, t0 = 0, time.perf_counter()
        while True:
            for n in widths:
                orc.simd_ffn_swiglu(g, u, d, HIDDEN, INTER, x_host[n], nthreads, isa=isa)
            done += 1
            if time.perf_counter() - t0 >= budget:
                break
        dt = time.perf_counter() - t0
        return done, dt, done * sum(ffn_bytes(n) for n in widths) / dt / 1e9

    done, dt, rate = timed(best, threads, seconds * 0.6, WIDTHS)
    _, _, one_core = timed(best, 1, seconds / 6, (1,))
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    out = {"value": round(rate, 2), "unit": "GB/s", "cores": threads, "kind": "port",
           "isa": "AVX-512 VNNI (256-bit)" if best == "vnni" else "AVX2",
           "sample": f"{done} passes over the five FFN widths (n=1,2,4,8,16) on weight set 0, {dt:.1f} s, "
                     f"{'AVX-512 VNNI' if best == 'vnni' else 'AVX2'} + {threads} pthreads, rows split as ith*ceil(N/nth)",
           "one_core_GBps": round(one_core, 2), "cpu": model,
           "host_cores": os.cpu_count(), "cores_allowed": allowed}
    if best != "avx2":
        done2, dt2, rate2 = timed("avx2", threads, seconds * 0.25, WIDTHS)
        out["avx2"] = {"value": round(rate2, 2), "unit": "GB/s", "cores": threads,
                       "sample": f"{done2} passes, {dt2:.1f} s, AVX2 + {threads} pthreads"}
    return out


if __name__ == "__main__":
    sys.exit(main())
