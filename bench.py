#!/usr/bin/env python3
"""Benchmark of the TQ8 quantized-linear forward path on one MI355X.

A "step" is one batch-1 forward of the Qwen2.5-0.5B-shaped lm_head stored as TQ8
(151936 x 2048, shared rotation, block 512, bf16 activations, fp32 logits): the
bandwidth-bound GEMV the headline metric is quoted on.  K steps are captured in one
HIP graph and timed with HIP events on the launching stream, inputs resident in HBM.

Prints ONE JSON line: throughput (tok/s = layer calls per second), the HBM roofline of
the GEMV kernel, the CPU baseline (the C restatement of the reference's
dequantize_weight_cpu + fp32 matmul, timed on this host), and the secondary
configurations of the metric (4096 x 4096 fp32) under "extra".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per GEMV launch on the headline workload from rocprofv3 FETCH_SIZE / WRITE_SIZE
# (profiles/gemv_lm_head_151936x2048_bs1.txt): 2.0 * 152402.0 KiB + 605.9 KiB.
MEASURED_TRAFFIC_BYTES = 312739738
# Average duration of the headline kernel in the rocprofv3 kernel trace of
# `python bench.py --steps 20 --warmup 5 --no-cpu-baseline` (same file), in microseconds, and the
# kernel's name there.
PROFILED_KERNEL_US = 50.54
HEADLINE_KERNEL = "tq_gemv_wide_kernel<shared, R=2, TILES=1, rows from an LDS counter>"
REFERENCE_PUBLISHED_TOK_S = 47.3      # reference README.md:79-82, 151936x2048 batch 1, Apple Silicon


# A captured graph is replayed untimed until this much GPU time has passed (at least three replays:
# the first uploads the graph, and the replays right after it still run a few per cent slower while
# clocks and memory settle under the load), so the timed region starts on a machine in steady state
# whatever --steps is.
UNTIMED_WARM_SECONDS = 0.05
# One event pair then brackets as many back-to-back replays as it takes to time at least this many
# kernel launches; the time per step is the bracket divided by the steps it holds.
MIN_TIMED_LAUNCHES = 200


def algorithmic_bytes(out, inf, batch, x_bytes, y_bytes):
    # packed primary + residual (one byte per weight), norms, two codebooks, x, y
    return out * inf + 4 * out + 128 + batch * inf * x_bytes + batch * out * y_bytes


def make_layer(tq, torch, out, inf, bs, seed, sigma, shared=True, per_layer_codebooks=False, tails=True):
    """Synthetic layer of BASELINE.json's recipe, produced entirely on the GPU: fp32 weights
    ~N(0, sigma^2) with 1% of the entries drawn from sigma * Student-t(3) (torch Philox generator,
    seeded), quantized by this library's GPU quantizer (the reference's quantize_weight pipeline)
    with analytic or per-layer Lloyd-Max codebooks."""
    import ctypes as C
    import numpy as np
    f32p, u32p = C.POINTER(C.c_float), C.POINTER(C.c_uint32)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    w = torch.randn(out, inf, device="cuda", generator=g) * sigma
    if tails:
        g.manual_seed(seed + 1)
        mask = torch.rand(out, inf, device="cuda", generator=g) < 0.01
        z = torch.randn(4, int(mask.sum().item()), device="cuda", generator=g)
        w[mask] = sigma * z[0] / torch.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3.0)
        del mask, z
    L = tq.lib()
    cbp = np.empty(32, np.float32)
    cbr = np.empty(32, np.float32)
    L.tq_generate_codebook(4, cbp.ctypes.data_as(f32p), None)
    L.tq_generate_codebook(4, cbr.ctypes.data_as(f32p), None)
    if per_layer_codebooks:
        glob = cbp.copy()
        if L.tq_fit_layer_codebooks(w.data_ptr(), out, inf, bs, 4, 4, glob.ctypes.data_as(f32p), 16, 100,
                                    cbp.ctypes.data_as(f32p), cbr.ctypes.data_as(f32p)) != 0:
            raise RuntimeError(tq.last_error())
    pp = torch.empty(out, inf // 2, dtype=torch.uint8, device="cuda")
    pr = torch.empty(out, inf // 2, dtype=torch.uint8, device="cuda")
    norms = torch.empty(out, dtype=torch.float32, device="cuda")
    seeds = np.zeros(3, np.uint32)
    if L.tq_quantize_weight(w.data_ptr(), out, inf, cbp.ctypes.data_as(f32p), 16, cbr.ctypes.data_as(f32p), 16,
                            4, 4, bs, int(shared), pp.data_ptr(), pr.data_ptr(), norms.data_ptr(),
                            seeds.ctypes.data_as(u32p)) != 0:
        raise RuntimeError(tq.last_error())
    del w
    tensors = dict(pp=pp, pr=pr, norms=norms, cbp=cbp[:16].copy(), cbr=cbr[:16].copy(), seeds=seeds)
    h = layer_from_tensors(tq, tensors, out, inf, bs)
    torch.cuda.synchronize()
    return h, tensors


def layer_from_tensors(tq, t, out, inf, bs):
    """A layer handle with its own device copy of the quantized tensors `t` (as make_layer returns them)."""
    import ctypes as C
    f32p, u32p = C.POINTER(C.c_float), C.POINTER(C.c_uint32)
    h = tq.lib().tq_linear_create_from_device(inf, out, t["pp"].data_ptr(), inf // 2, t["pr"].data_ptr(), inf // 2,
                                              t["norms"].data_ptr(), t["seeds"].ctypes.data_as(u32p),
                                              t["cbp"].ctypes.data_as(f32p), 16, t["cbr"].ctypes.data_as(f32p), 16, bs)
    if not h:
        raise RuntimeError(tq.last_error())
    return h


def time_graph_fn(torch, enqueue_step, steps, warmup, launches_per_step=1, spread=None):
    """Capture `steps` calls of enqueue_step(stream_handle) in one HIP graph and time it with HIP events
    on the launching stream.  Returns (seconds per step, timed steps).  `warmup` eager steps run first;
    the graph is then replayed untimed for UNTIMED_WARM_SECONDS, and one event pair brackets enough
    back-to-back replays to hold MIN_TIMED_LAUNCHES kernel launches.  With `spread` (a list): 20 more
    single replays are timed one by one and their seconds per step appended."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(max(warmup, 1)):
            enqueue_step(stream.cuda_stream)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for _ in range(steps):
            enqueue_step(stream.cuda_stream)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    replays = max(1, -(-MIN_TIMED_LAUNCHES // (steps * launches_per_step)))
    with torch.cuda.stream(stream):
        t0 = time.perf_counter()
        done = 0
        while done < 3 or time.perf_counter() - t0 < UNTIMED_WARM_SECONDS:
            graph.replay()
            stream.synchronize()
            done += 1
        torch.cuda.synchronize()
        start.record(stream)
        for _ in range(replays):
            graph.replay()
        end.record(stream)
    torch.cuda.synchronize()
    secs = start.elapsed_time(end) * 1e-3 / (steps * replays)
    if spread is not None:
        for _ in range(20):
            with torch.cuda.stream(stream):
                start.record(stream)
                graph.replay()
                end.record(stream)
            torch.cuda.synchronize()
            spread.append(start.elapsed_time(end) * 1e-3 / steps)
    return secs, steps * replays


def time_graph(tq, torch, handles, x, y, xcode, batch, steps, warmup, spread=None):
    """Seconds per forward and timed forwards, cycling over `handles` (see time_graph_fn)."""
    L = tq.lib()
    n = len(handles)
    turn = [0]

    def step(s):
        if L.tq_linear_forward(handles[turn[0] % n], x.data_ptr(), xcode, batch, y.data_ptr(), 0, s) != 0:
            raise RuntimeError(tq.last_error())
        turn[0] += 1
    return time_graph_fn(torch, step, steps, warmup, 1, spread)


TIMELINE_MARKS = ["wave started", "first weight rows requested", "decode table written", "before the barrier",
                  "behind the barrier", "loop entered", "row group 1 stored", "row group 2 (3)", "row group 3 (5)",
                  "row group 4 (7)", "row group 5 (9)", "row group 6 (11)", "row group 7 (13)", "row group 8 (15)",
                  "last row group stored", "memory operations complete"]


def timeline(tq, torch):
    """Where the time of a batch-1 launch goes: the timeline build of the library (same sources, wall-clock
    marks per wave) on three shapes, 300 back-to-back launches, marks of the last one; microseconds from
    the start of the launch's first wave."""
    import ctypes as C
    import numpy as np
    tq.LIB_PATH = os.path.join(os.path.dirname(tq.LIB_PATH), "libturboquant_amd_timeline.so")
    L = tq.lib()
    L.tq_timeline_read.argtypes = [C.c_void_p]
    for out, inf, dt, code, copies in ((151936, 2048, torch.bfloat16, tq.BF16, 2), (4096, 4096, torch.float32, tq.F32, 16),
                                       (27648, 5120, torch.bfloat16, tq.BF16, 4)):
        hs = [make_layer(tq, torch, out, inf, 512, seed=40 + i, sigma=0.02, shared=True)[0] for i in range(copies)]
        x = torch.randn(1, inf, device="cuda").to(dt)
        y = torch.empty(1, out, device="cuda", dtype=torch.float32)
        for i in range(12):
            if L.tq_linear_forward(hs[i % copies], x.data_ptr(), code, 1, y.data_ptr(), 0, None) != 0:
                raise RuntimeError(tq.last_error())
        torch.cuda.synchronize()
        for pass_ in (1, 2):                               # two passes: what persists from launch to launch
            L.tq_timeline_clear()
            for i in range(300):
                L.tq_linear_forward(hs[i % copies], x.data_ptr(), code, 1, y.data_ptr(), 0, None)
            torch.cuda.synchronize()
            buf = np.zeros(256 * 16 * 16, np.uint64)
            if L.tq_timeline_read(buf.ctypes.data) != 0:
                raise RuntimeError("tq_timeline_read failed")
            t = buf.reshape(256, 16, 16).astype(np.int64)
            live = t[:, :, 0] > 0
            t0 = t[:, :, 0][live].min()
            print(f"--- {out} x {inf}, shared rotation, batch 1, pass {pass_}: {int(live.sum())} waves; us from the first wave's start")
            print(f"  {'mark':34s} {'min':>7s} {'mean':>7s} {'p90':>7s} {'max':>7s}")
            for k in range(16):
                col = t[:, :, k][live & (t[:, :, k] >= t[:, :, 0])]     # a mark older than the wave's start is a previous launch's
                if len(col) == 0:
                    continue
                r = (col - t0) / 100.0
                print(f"  {k:2d} {TIMELINE_MARKS[k]:31s} {r.min():7.2f} {r.mean():7.2f} {np.percentile(r, 90):7.2f} {r.max():7.2f}")
            end = np.where(live, (t[:, :, 14] - t0) / 100.0, 0.0).max(axis=1)
            end = end[end > 0]
            print(f"  last row group stored, per CU: min {end.min():.2f} mean {end.mean():.2f} max {end.max():.2f}")
            per_xcd = [float(np.mean([e for b, e in enumerate(np.where(live, (t[:, :, 14] - t0) / 100.0, 0.0).max(axis=1))
                                      if b % 8 == xc and e > 0])) for xc in range(8)]
            print("  the same, mean over the CUs of each XCD (workgroup id % 8):", " ".join(f"{v:.2f}" for v in per_xcd))
        for h in hs:
            L.tq_linear_free(h)
        torch.cuda.empty_cache()


def rows_table(tq, torch):
    """us per tq_linear_forward call against the number of rows; one line per shape and rotation."""
    L = tq.lib()
    rows = (1, 2, 3, 4, 5, 8, 16, 32)
    print("rows                          " + "".join(f"{r:>8d}" for r in rows))
    for shared in (True, False):
        for outp, inp in ((151936, 2048), (27648, 5120), (5120, 27648)):
            copies = -(-600_000_000 // (outp * inp)) + 1
            hs = [make_layer(tq, torch, outp, inp, 512, seed=700 + i, sigma=0.01, shared=shared,
                             per_layer_codebooks=False, tails=False)[0] for i in range(copies)]
            res = []
            for m in rows:
                x = torch.randn(m, inp, device="cuda").to(torch.bfloat16)
                y = torch.empty(m, outp, device="cuda", dtype=torch.float32)

                def run(n):
                    for i in range(n):
                        if L.tq_linear_forward(hs[i % copies], x.data_ptr(), tq.BF16, m, y.data_ptr(), tq.F32, None) != 0:
                            raise RuntimeError(tq.last_error())
                t_end = time.perf_counter() + 0.1          # the clocks settle over tens of milliseconds
                while time.perf_counter() < t_end:
                    run(copies)
                    torch.cuda.synchronize()
                st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                st.record()
                run(8 * copies)
                en.record()
                torch.cuda.synchronize()
                res.append(st.elapsed_time(en) * 1e3 / (8 * copies))
            tag = f"{outp}x{inp} {'shared' if shared else 'dual'} ({copies} copies)"
            print(f"{tag:30s}" + "".join(f"{v:8.1f}" for v in res), flush=True)
            for h in hs:
                L.tq_linear_free(h)
            torch.cuda.empty_cache()


def cpu_baseline(torch, tensors, out, inf, bs, x_f32):
    """Reference CPU path (dequantize_weight_cpu + fp32 matmul, restated in oracle/) on the
    host cores of this box, whole layer, single thread as the reference's serial loops."""
    import numpy as np
    from oracle import oracle as o
    pp = tensors["pp"].cpu().numpy()
    pr = tensors["pr"].cpu().numpy()
    norms = tensors["norms"].cpu().numpy()
    cbp, cbr = o.Codebook(tensors["cbp"], 4), o.Codebook(tensors["cbr"], 4)
    qw = o.QuantizedWeight(pp, pr, norms, tensors["seeds"])
    o.set_threads(1)
    t0 = time.perf_counter()
    W = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    y = o.matmul_xwT(x_f32, W, acc_double=False)
    dt = time.perf_counter() - t0
    threads = min(16, os.cpu_count() or 1)
    o.set_threads(threads)
    t0 = time.perf_counter()
    W = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
    y_mt = o.matmul_xwT(x_f32, W, acc_double=False)
    dt_mt = time.perf_counter() - t0
    o.set_threads(1)
    assert np.array_equal(y, y_mt)
    return dt, dt_mt, threads, y


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--skip-extra", action="store_true", help="measure the headline configuration only")
    ap.add_argument("--decoder-layer-only", action="store_true",
                    help="of the extra measurements, run only the decoder-layer projections (for kernel profiles)")
    ap.add_argument("--timeline", action="store_true",
                    help="instead of the benchmark: per-wave wall-clock marks inside the batch-1 kernel (the "
                         "timeline build of the library), last of 300 back-to-back launches, as a text table")
    ap.add_argument("--prefill-ablations", metavar="MASK", default=None,
                    help="instead of the benchmark: eight 512-token calls of the prefill workload (27648 x 5120) on "
                         "the build of the library with parts of the prefill panel kernel's loop compiled out "
                         "(`make ablations`; MASK as in csrc/tq_prefill_panel.hip, 0 = the product library).  Meant to "
                         "run under rocprofv3 --pmc: the results are wrong by construction, the cycle counters of "
                         "the kernel are what is compared")
    ap.add_argument("--rows-table", action="store_true",
                    help="instead of the benchmark: time of one tq_linear_forward call against the number of activation "
                         "rows (1..32) on the lm_head and the two large decoder projections, shared and dual rotation, "
                         "bf16 in / fp32 out, eager launches timed with HIP events, weight copies cycled so that the "
                         "planes come from HBM (more than 600 MB per shape)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 256 MiB device-to-device copy three times (reference reading for "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; the TQ8 linear path is not sharded here (--gpus must be 1)",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import __graft_entry__ as entry
    tq = entry.load_package()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.timeline:
        timeline(tq, torch)
        return
    if args.rows_table:
        rows_table(tq, torch)
        return
    if args.prefill_ablations is not None:
        mask = int(args.prefill_ablations)
        if mask:
            tq.LIB_PATH = os.path.join(os.path.dirname(tq.LIB_PATH), "ablate", f"libturboquant_amd_ablate{mask}.so")
        hp, _ = make_layer(tq, torch, 27648, 5120, 512, seed=500, sigma=0.01, shared=True)
        xp = torch.randn(512, 5120, device="cuda").to(torch.bfloat16)
        yp = torch.empty(512, 27648, device="cuda", dtype=torch.bfloat16)
        for _ in range(8):
            if tq.lib().tq_linear_forward(hp, xp.data_ptr(), tq.BF16, 512, yp.data_ptr(), tq.BF16, None) != 0:
                raise RuntimeError(tq.last_error())
        torch.cuda.synchronize()
        print(f"prefill ablation mask {mask}: 8 calls of 27648 x 5120 at 512 tokens done ({tq.LIB_PATH})")
        return

    # ---- headline: lm_head 151936 x 2048, bf16 x, fp32 y, batch 1 -------------------
    out, inf, bs = 151936, 2048, 512
    handle, tensors = make_layer(tq, torch, out, inf, bs, seed=0xCAFEBABE + 1, sigma=0.02, shared=True,
                                 per_layer_codebooks=True)
    g = torch.Generator(device="cuda"); g.manual_seed(0xCAFEBABE + 3)
    x = torch.randn(1, inf, device="cuda", generator=g).to(torch.bfloat16)
    y = torch.empty(1, out, device="cuda", dtype=torch.float32)
    # Two copies of the layer (2 x 311 MB) are cycled, so no launch can find its weights in the 256 MB
    # last-level cache left there by the launch before it: `value` is the HBM-resident rate.  The same
    # graph over one copy is reported beside it.
    handle2 = layer_from_tensors(tq, tensors, out, inf, bs)
    spread = []
    secs, timed = time_graph(tq, torch, [handle, handle2], x, y, tq.BF16, 1, args.steps, args.warmup, spread)
    us = secs * 1e6
    secs_one, _ = time_graph(tq, torch, [handle], x, y, tq.BF16, 1, args.steps, args.warmup)
    tq.lib().tq_linear_free(handle2)
    spread_us = np.sort(np.array(spread)) * 1e6
    B = algorithmic_bytes(out, inf, 1, 2, 4)
    achieved = B / (us * 1e-6) / 1e9

    result = {
        "metric": "TQ8 GEMV throughput, 151936x2048 lm_head, batch 1 (layer calls per second)",
        "value": 1e6 / us,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "timed_launches": timed,
        "timing": f"{args.steps} steps per HIP graph; untimed replays for {UNTIMED_WARM_SECONDS * 1e3:.0f} ms, then "
                  f"{timed // args.steps} back-to-back replays inside one HIP event pair ({timed} kernel launches); "
                  "ms_per_step = bracket / steps in it",
        "ms_per_step": us * 1e-3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": (1e6 / us) / REFERENCE_PUBLISHED_TOK_S,
        "dtype": "f32",
        "data": "synthetic: fp32 weights N(0,0.02^2) with 1% Student-t(3) tails, quantized on the GPU by this "
                "library's TQ8 quantizer with per-layer Lloyd-Max codebooks (shared rotation, block 512); "
                "bf16 N(0,1) activations",
        "config": {"workload": "Qwen2.5-0.5B lm_head as TQ8 linear 151936x2048, shared rotation, block 512, "
                               "x bf16 [1,2048], y f32 [1,151936]; two weight copies cycled (HBM-resident)",
                   "baseline_note": "vs_baseline divides by the reference's published 47.3 tok/s (Apple Silicon)"},
        "us_per_layer": us,
        "us_per_layer_one_weight_copy": secs_one * 1e6,
        "us_per_layer_over_20_more_replays": {"median": float(np.median(spread_us)),
                                              "p10": float(np.percentile(spread_us, 10)),
                                              "p90": float(np.percentile(spread_us, 90))},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel": HEADLINE_KERNEL, "algorithmic_bytes": B,
                     "us_per_launch_hip_events": us,
                     "us_per_launch_kernel_trace": PROFILED_KERNEL_US,
                     "kernel_trace_source": "profiles/gemv_lm_head_151936x2048_bs1.txt (rocprofv3 --kernel-trace "
                                            "--stats of this command; average kernel duration, launch gaps excluded)",
                     "frac_one_weight_copy": B / secs_one / 1e9 / HBM_PEAK_GBS},
    }

    # ---- CPU baseline on this host ---------------------------------------------------
    if not args.no_cpu_baseline:
        x_f32 = x.float().cpu().numpy()
        dt, dt_mt, threads, y_cpu = cpu_baseline(torch, tensors, out, inf, bs, x_f32)
        y_gpu = y.cpu().numpy()
        rel = float(np.linalg.norm(y_gpu - y_cpu) / np.linalg.norm(y_cpu))
        result["cpu_baseline"] = {"value": 1.0 / dt, "unit": "tok/s", "cores": 1, "kind": "port",
                                  "sample": "the whole 151936x2048 layer once: dequantize_weight_cpu restatement "
                                            "+ fp32 matmul, single thread",
                                  "seconds": dt,
                                  "all_cores": {"value": 1.0 / dt_mt, "cores": threads, "seconds": dt_mt},
                                  "gpu_vs_cpu_rel_l2": rel}
    tq.lib().tq_linear_free(handle)
    del tensors
    torch.cuda.empty_cache()

    # ---- what this machine sustains: streaming read and MFMA loops (roofline denominators) ----
    extra = {}
    import ctypes as C
    probe_path = os.path.join(os.path.dirname(tq.LIB_PATH), "libtq_probe.so")      # `make probe`: a library of its own
    probes = {}
    if os.path.exists(probe_path):
        Lp = C.CDLL(probe_path)
        Lp.tq_probe_hbm_read.argtypes = [C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        Lp.tq_probe_mfma_bf16.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_double)]
        Lp.tq_probe_mfma_f16.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_double)]
        Lp.tq_probe_empty_launch.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
        val = C.c_double()
        if Lp.tq_probe_hbm_read(1 << 30, 10, C.byref(val)) == 0:
            probes["hbm_stream_read_gbs"] = val.value
        for name, rnd in (("mfma_bf16_tflops_ones", 0), ("mfma_bf16_tflops_random_operands", 1)):
            if Lp.tq_probe_mfma_bf16(rnd, 20000, C.byref(val)) == 0:
                probes[name] = val.value
        # (the prefill kernels multiply in fp16: same nominal rate, more toggling mantissa bits)
        for name, rnd in (("mfma_f16_tflops_ones", 0), ("mfma_f16_tflops_random_operands", 1)):
            if Lp.tq_probe_mfma_f16(rnd, 20000, C.byref(val)) == 0:
                probes[name] = val.value
        # launch to launch of a kernel that does nothing, as nodes of one HIP graph: a single wave, and the grid of
        # the batch-1 kernel (one workgroup of 16 waves per CU)
        for name, wgs, threads in (("empty_kernel_us_per_graph_node_1x64", 1, 64), ("empty_kernel_us_per_graph_node_256x1024", 256, 1024)):
            if Lp.tq_probe_empty_launch(wgs, threads, 200, C.byref(val)) == 0:
                probes[name] = val.value
    extra["machine_probes"] = probes
    if "hbm_stream_read_gbs" in probes:
        result["roofline"]["frac_of_measured_stream_read"] = achieved / probes["hbm_stream_read_gbs"]
    if args.skip_extra:
        finish(args, torch, extra, result)
        return
    if not args.decoder_layer_only:
        out1, in1 = 4096, 4096
        copies = 32                         # 32 x 16.8 MB > 256 MB of last-level cache: HBM-resident timing
        handles = [make_layer(tq, torch, out1, in1, bs, seed=100 + 2 * i, sigma=0.02, shared=True)[0] for i in range(copies)]
        x1 = torch.randn(1, in1, device="cuda", generator=g)
        y1 = torch.empty(1, out1, device="cuda", dtype=torch.float32)
        steps1 = max(args.steps, copies) // copies * copies
        us_hbm = time_graph(tq, torch, handles, x1, y1, tq.F32, 1, steps1, args.warmup)[0] * 1e6
        us_hot = time_graph(tq, torch, handles[:1], x1, y1, tq.F32, 1, steps1, args.warmup)[0] * 1e6
        B1 = algorithmic_bytes(out1, in1, 1, 4, 4)
        extra["gemv_4096x4096_f32_bs1"] = {"us_per_layer_hbm_resident": us_hbm, "us_per_layer_cache_resident": us_hot,
                                           "weight_copies_cycled": copies, "algorithmic_bytes": B1,
                                           "hbm_frac": B1 / (us_hbm * 1e-6) / 1e9 / HBM_PEAK_GBS}
        for h in handles:
            tq.lib().tq_linear_free(h)
        # The reference's own bench recipe (benchmarks/bench_linear.cpp:10-76), the neighbour of its published
        # 1.49 ms: weights N(0, 1/sqrt(in)) without tails, analytic codebooks, shared rotation, all-ones fp32
        # input, 1 warm-up + 10 forwards each followed by a wait for the result, mean wall clock.
        href = make_layer(tq, torch, out1, in1, bs, seed=0xCAFEBABE, sigma=in1 ** -0.5, shared=True, tails=False)[0]
        ones = torch.ones(1, in1, device="cuda")
        s0 = torch.cuda.current_stream()
        wall = []
        for it in range(11):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            if tq.lib().tq_linear_forward(href, ones.data_ptr(), tq.F32, 1, y1.data_ptr(), 0, s0.cuda_stream) != 0:
                raise RuntimeError(tq.last_error())
            s0.synchronize()
            wall.append(time.perf_counter() - t0)
        extra["gemv_4096x4096_reference_bench_recipe"] = {
            "us_per_call_wall_clock_mean_of_10": float(np.mean(wall[1:]) * 1e6),
            "reference_published_us": 1490.0,
            "method": "one forward + stream wait per iteration, host wall clock (launch and wait latency included)"}
        tq.lib().tq_linear_free(href)
        # the library default of the reference is dual rotation (include/turboquant/quantizer.h:15)
        handles = [make_layer(tq, torch, out1, in1, bs, seed=300 + 2 * i, sigma=0.02, shared=False)[0] for i in range(copies)]
        us_dual = time_graph(tq, torch, handles, x1, y1, tq.F32, 1, steps1, args.warmup)[0] * 1e6
        extra["gemv_4096x4096_f32_bs1_dual_rotation"] = {"us_per_layer_hbm_resident": us_dual,
                                                         "hbm_frac": B1 / (us_dual * 1e-6) / 1e9 / HBM_PEAK_GBS}
        for h in handles:
            tq.lib().tq_linear_free(h)
        del handles
        torch.cuda.empty_cache()

        # ---- prefill: Qwen2.5-32B up-projection 27648 x 5120 at M = 512 and 2048, and the down projection
        # 5120 x 27648 at M = 512 (40 output tiles for 256 CUs: K is cut into ranges), bf16 in / bf16 out ----
        for outp, inp, token_counts in ((27648, 5120, (512, 2048)), (5120, 27648, (512,))):
            hp, _ = make_layer(tq, torch, outp, inp, bs, seed=500, sigma=0.01, shared=True, per_layer_codebooks=True)
            for M in token_counts:
                xp = torch.randn(M, inp, device="cuda", generator=g).to(torch.bfloat16)
                yp = torch.empty(M, outp, device="cuda", dtype=torch.bfloat16)
                L = tq.lib()

                def timed(call, reps=20):
                    """Untimed calls until the chip has been under this load for 0.1 s (its clocks settle over tens
                    of milliseconds: the first calls after a pause run up to 15 % slower), then one event bracket."""
                    t_end = time.perf_counter() + 0.1
                    while time.perf_counter() < t_end:
                        for _ in range(5):
                            call()
                        torch.cuda.synchronize()
                    st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    st.record()
                    for _ in range(reps):
                        call()
                    en.record()
                    torch.cuda.synchronize()
                    return st.elapsed_time(en) * 1e3 / reps

                def ours():
                    if L.tq_linear_forward(hp, xp.data_ptr(), tq.BF16, M, yp.data_ptr(), tq.BF16, None) != 0:
                        raise RuntimeError(tq.last_error())
                usp = timed(ours)
                flops = 2.0 * M * outp * inp
                # The vendor library's plain bf16 GEMM of the same shape on already dequantised weights
                # (torch.matmul -> hipBLASLt): what a matrix kernel with no decode work reaches on this machine.
                wv = (torch.randn(outp, inp, device="cuda", generator=g) * 0.01).to(torch.bfloat16)
                usv = timed(lambda: torch.matmul(xp, wv.t(), out=yp))
                del wv
                extra[f"prefill_{outp}x{inp}_M{M}_bf16"] = {"us_per_layer": usp, "tflops": flops / usp / 1e6,
                                                          "vendor_plain_bf16_gemm_same_shape_us": usv,
                                                          "vendor_plain_bf16_gemm_tflops": flops / usv / 1e6,
                                                          "speed_relative_to_vendor_plain_gemm": usv / usp,
                                                          "mfma_frac_of_2500_tflops": flops / usp / 1e6 / 2500.0,
                                                          "frac_of_measured_mfma_loop_random_operands":
                                                              flops / usp / 1e6 / probes.get("mfma_f16_tflops_random_operands",
                                                                                             float("nan")),
                                                          "includes": "activation rotation kernel + dequant/MFMA GEMM kernel (+ the sum of the K ranges where K is cut)"}
            tq.lib().tq_linear_free(hp)
            torch.cuda.empty_cache()

        # ---- decode MLP block, Qwen2.5-7B shape: gate/up 18944 x 3584, down 3584 x 18944, batch 1 ----
        L = tq.lib()
        hid, inter = 3584, 18944
        for shared in (False, True):
            blocks, keep = [], []
            for c in range(2):                       # two blocks of 204 MB cycled: HBM-resident weights
                hs = [make_layer(tq, torch, o_, i_, bs, seed=700 + 10 * c + k, sigma=0.015, shared=shared,
                                 per_layer_codebooks=True)[0]
                      for k, (o_, i_) in enumerate([(inter, hid), (inter, hid), (hid, inter)])]
                m = L.tq_mlp_create(hs[0], hs[1], hs[2], 1)
                if not m:
                    raise RuntimeError(tq.last_error())
                blocks.append(m); keep.append(hs)
            xm = torch.randn(1, hid, device="cuda", generator=g).to(torch.bfloat16)
            ym = torch.empty(1, hid, device="cuda", dtype=torch.float32)
            turn = [0]

            def mlp_step(s):
                if L.tq_mlp_forward(blocks[turn[0] % 2], xm.data_ptr(), tq.BF16, 1, ym.data_ptr(), tq.F32, s) != 0:
                    raise RuntimeError(tq.last_error())
                turn[0] += 1
            steps_m = max(2, args.steps // 2 * 2)
            us_m = time_graph_fn(torch, mlp_step, steps_m, 2, 3)[0] * 1e6
            Bm = 2 * algorithmic_bytes(inter, hid, 1, 2, 4) + algorithmic_bytes(hid, inter, 1, 4, 4)
            extra["mlp_block_7b_bs1_" + ("shared_rotation" if shared else "dual_rotation")] = {
                "us_per_block": us_m, "algorithmic_bytes": Bm, "hbm_frac": Bm / (us_m * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "kernels_per_block": 3,
                "kernels": "gate + up in one launch, rotation of the 18944-wide row silu(gate) * up, down"}
            for m in blocks:
                L.tq_mlp_free(m)
            for hs in keep:
                for h in hs:
                    L.tq_linear_free(h)
            torch.cuda.empty_cache()

    # ---- decoder-layer projections, Qwen2.5-32B shape, batch 1 / 4 / 8 (grouped launches: and 32), bf16 activations ----
    L = tq.lib()
    shapes = [("q", 5120, 5120), ("k", 1024, 5120), ("v", 1024, 5120), ("o", 5120, 5120),
              ("gate", 27648, 5120), ("up", 27648, 5120), ("down", 5120, 27648)]
    # two decoder layers of 488 MB alternate, as the two lm_head copies do: no call finds its weights in the
    # last-level cache
    layer_sets = [[(n_, o_, i_, make_layer(tq, torch, o_, i_, bs, seed=900 + 20 * c + k, sigma=0.01, shared=True,
                                           per_layer_codebooks=True)[0]) for k, (n_, o_, i_) in enumerate(shapes)]
                  for c in range(2)]
    layers = layer_sets[0]
    for batch in (1, 4, 8):
        xs = {i_: torch.randn(batch, i_, device="cuda", generator=g).to(torch.bfloat16) for i_ in (5120, 27648)}
        ys = {o_: torch.empty(batch, o_, device="cuda", dtype=torch.float32) for o_ in (5120, 1024, 27648)}

        turn = [0]

        def layer_step(s):
            for n_, o_, i_, h in layer_sets[turn[0] % 2]:
                if L.tq_linear_forward(h, xs[i_].data_ptr(), tq.BF16, batch, ys[o_].data_ptr(), tq.F32, s) != 0:
                    raise RuntimeError(tq.last_error())
            turn[0] += 1
        us_l = time_graph_fn(torch, layer_step, max(args.steps // 10, 10), 2, 7)[0] * 1e6
        Bl = sum(algorithmic_bytes(o_, i_, batch, 2, 4) for _, o_, i_, _ in layers)
        extra[f"decoder_layer_projections_32b_bs{batch}"] = {
            "us_per_layer_all_7_projections": us_l, "algorithmic_bytes": Bl,
            "hbm_frac": Bl / (us_l * 1e-6) / 1e9 / HBM_PEAK_GBS}
    # The same seven projections at batch 1 with the layers that read the same activation row sharing a
    # launch (tq_linear_forward_group): q, k, v; o; gate, up; down (+ the rotation of its 27648-wide row).
    import ctypes as C
    by = [{n_: h for n_, _, _, h in ls} for ls in layer_sets]
    out_of = {n_: o_ for n_, o_, _, _ in layers}
    L.tq_linear_forward_group.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_int, C.c_int,
                                          C.POINTER(C.c_void_p), C.c_int, C.c_void_p]
    def grouped(sets, tag):
        for batch in (1, 2, 4, 8, 32):
            xg = {i_: torch.randn(batch, i_, device="cuda", generator=g).to(torch.bfloat16) for i_ in (5120, 27648)}
            yg = {n_: torch.empty(batch, out_of[n_], device="cuda", dtype=torch.float32) for n_ in sets[0]}
            turn = [0]

            def group(names, x, s):
                hs = (C.c_void_p * len(names))(*[sets[turn[0] % 2][n_] for n_ in names])
                yp = (C.c_void_p * len(names))(*[yg[n_].data_ptr() for n_ in names])
                if L.tq_linear_forward_group(hs, len(names), x.data_ptr(), tq.BF16, batch, yp, tq.F32, s) != 0:
                    raise RuntimeError(tq.last_error())

            def grouped_step(s):
                group(("q", "k", "v"), xg[5120], s)
                group(("o",), xg[5120], s)
                group(("gate", "up"), xg[5120], s)
                group(("down",), xg[27648], s)
                turn[0] += 1
            us_g = time_graph_fn(torch, grouped_step, max(args.steps // 10, 10), 2, 4)[0] * 1e6
            Bg = sum(algorithmic_bytes(o_, i_, batch, 2, 4) for _, o_, i_, _ in layers)
            extra[f"decoder_layer_projections_32b_bs{batch}{tag}_grouped_launches"] = {
                "us_per_layer_all_7_projections": us_g, "algorithmic_bytes": Bg,
                "hbm_frac": Bg / (us_g * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "calls": "q+k+v, o, gate+up, down through tq_linear_forward_group"}
    grouped(by, "")
    for ls in layer_sets:
        for _, _, _, h in ls:
            L.tq_linear_free(h)
    torch.cuda.empty_cache()
    # the same layers in the converter's default format: dual rotation (include/turboquant/quantizer.h:15)
    dual = [{n_: make_layer(tq, torch, o_, i_, bs, seed=950 + 20 * c + k, sigma=0.01, shared=False,
                            per_layer_codebooks=True)[0] for k, (n_, o_, i_) in enumerate(shapes)} for c in range(2)]
    grouped(dual, "_dual_rotation")
    for d in dual:
        for h in d.values():
            L.tq_linear_free(h)
    finish(args, torch, extra, result)


def finish(args, torch, extra, result):
    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        src.random_(0, 256)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        extra["copy_calibration_bytes"] = src.numel()
    result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
