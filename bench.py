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
REFERENCE_PUBLISHED_TOK_S = 47.3      # reference README.md:79-82, 151936x2048 batch 1, Apple Silicon


def algorithmic_bytes(out, inf, batch, x_bytes, y_bytes):
    # packed primary + residual (one byte per weight), norms, two codebooks, x, y
    return out * inf + 4 * out + 128 + batch * inf * x_bytes + batch * out * y_bytes


def make_layer(tq, torch, out, inf, bs, seed, shared=True):
    """Synthetic TQ8 tensors generated on the GPU: uniformly random 4-bit indices in both
    planes, corrected norms ~U(0.5, 1.5)*0.02*sqrt(in), analytic 4-bit codebooks."""
    import ctypes as C
    import numpy as np
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    pp = torch.randint(0, 256, (out, inf // 2), dtype=torch.uint8, device="cuda", generator=g)
    pr = torch.randint(0, 256, (out, inf // 2), dtype=torch.uint8, device="cuda", generator=g)
    norms = (torch.rand(out, device="cuda", generator=g) + 0.5) * (0.02 * inf ** 0.5)
    cb = np.array([-2.732590, -2.069017, -1.618046, -1.256231, -0.942340, -0.656759, -0.388048, -0.128395,
                   0.128395, 0.388048, 0.656759, 0.942340, 1.256231, 1.618046, 2.069017, 2.732590], np.float32)
    seeds = np.array([0xCAFEBABE, 0 if shared else 0x1234567, bs], np.uint32)
    L = tq.lib()
    h = L.tq_linear_create_from_device(inf, out, pp.data_ptr(), inf // 2, pr.data_ptr(), inf // 2, norms.data_ptr(),
                                       seeds.ctypes.data_as(C.POINTER(C.c_uint32)),
                                       cb.ctypes.data_as(C.POINTER(C.c_float)), 16,
                                       cb.ctypes.data_as(C.POINTER(C.c_float)), 16, bs)
    if not h:
        raise RuntimeError(tq.last_error())
    torch.cuda.synchronize()
    return h, dict(pp=pp, pr=pr, norms=norms, cb=cb, seeds=seeds)


def time_graph(tq, torch, handles, x, y, xcode, batch, steps, warmup):
    """Capture `steps` forwards (cycling over `handles`) in one HIP graph; return seconds."""
    L = tq.lib()
    stream = torch.cuda.Stream()
    n = len(handles)

    def enqueue(count, s):
        for i in range(count):
            rc = L.tq_linear_forward(handles[i % n], x.data_ptr(), xcode, batch, y.data_ptr(), 0, s.cuda_stream)
            if rc != 0:
                raise RuntimeError(tq.last_error())

    with torch.cuda.stream(stream):
        enqueue(max(warmup, 1), stream)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        enqueue(steps, stream)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        graph.replay()                     # untimed replay: graph upload
        stream.synchronize()
        torch.cuda.synchronize()
        start.record(stream)
        graph.replay()
        end.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(end) * 1e-3


def cpu_baseline(torch, tensors, out, inf, bs, x_f32):
    """Reference CPU path (dequantize_weight_cpu + fp32 matmul, restated in oracle/) on the
    host cores of this box, whole layer, single thread as the reference's serial loops."""
    import numpy as np
    from oracle import oracle as o
    pp = tensors["pp"].cpu().numpy()
    pr = tensors["pr"].cpu().numpy()
    norms = tensors["norms"].cpu().numpy()
    cb = o.Codebook(tensors["cb"], 4)
    qw = o.QuantizedWeight(pp, pr, norms, tensors["seeds"])
    o.set_threads(1)
    t0 = time.perf_counter()
    W = o.dequantize_weight_cpu(qw, cb, cb, bs)
    y = o.matmul_xwT(x_f32, W, acc_double=False)
    dt = time.perf_counter() - t0
    threads = min(16, os.cpu_count() or 1)
    o.set_threads(threads)
    t0 = time.perf_counter()
    W = o.dequantize_weight_cpu(qw, cb, cb, bs)
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

    # ---- headline: lm_head 151936 x 2048, bf16 x, fp32 y, batch 1 -------------------
    out, inf, bs = 151936, 2048, 512
    handle, tensors = make_layer(tq, torch, out, inf, bs, seed=0xCAFEBABE + 1)
    g = torch.Generator(device="cuda"); g.manual_seed(0xCAFEBABE + 3)
    x = torch.randn(1, inf, device="cuda", generator=g).to(torch.bfloat16)
    y = torch.empty(1, out, device="cuda", dtype=torch.float32)
    secs = time_graph(tq, torch, [handle], x, y, tq.BF16, 1, args.steps, args.warmup)
    us = secs / args.steps * 1e6
    B = algorithmic_bytes(out, inf, 1, 2, 4)
    achieved = B / (us * 1e-6) / 1e9

    result = {
        "metric": "TQ8 GEMV throughput, 151936x2048 lm_head, batch 1 (layer calls per second)",
        "value": 1e6 / us,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": us * 1e-3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": (1e6 / us) / REFERENCE_PUBLISHED_TOK_S,
        "dtype": "f32",
        "data": "synthetic: uniformly random 4-bit primary/residual indices, random row norms, analytic "
                "16-entry codebooks, bf16 N(0,1) activations; all generated on the GPU",
        "config": {"workload": "Qwen2.5-0.5B lm_head as TQ8 linear 151936x2048, shared rotation, block 512, "
                               "x bf16 [1,2048], y f32 [1,151936]",
                   "baseline_note": "vs_baseline divides by the reference's published 47.3 tok/s (Apple Silicon)"},
        "us_per_layer": us,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "tq_gemv_kernel<shared,1,2,1024>", "algorithmic_bytes": B},
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

    # ---- secondary configuration of the metric: 4096 x 4096 fp32, batch 1 ------------
    extra = {}
    if args.skip_extra:
        finish(args, torch, extra, result)
        return
    out1, in1 = 4096, 4096
    copies = 32                         # 32 x 16.8 MB > 256 MB of last-level cache: HBM-resident timing
    handles = [make_layer(tq, torch, out1, in1, bs, seed=100 + i)[0] for i in range(copies)]
    x1 = torch.randn(1, in1, device="cuda", generator=g)
    y1 = torch.empty(1, out1, device="cuda", dtype=torch.float32)
    steps1 = max(args.steps, copies) // copies * copies
    us_hbm = time_graph(tq, torch, handles, x1, y1, tq.F32, 1, steps1, args.warmup) / steps1 * 1e6
    us_hot = time_graph(tq, torch, handles[:1], x1, y1, tq.F32, 1, steps1, args.warmup) / steps1 * 1e6
    B1 = algorithmic_bytes(out1, in1, 1, 4, 4)
    extra["gemv_4096x4096_f32_bs1"] = {"us_per_layer_hbm_resident": us_hbm, "us_per_layer_cache_resident": us_hot,
                                       "weight_copies_cycled": copies, "algorithmic_bytes": B1,
                                       "hbm_frac": B1 / (us_hbm * 1e-6) / 1e9 / HBM_PEAK_GBS}
    for h in handles:
        tq.lib().tq_linear_free(h)
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
