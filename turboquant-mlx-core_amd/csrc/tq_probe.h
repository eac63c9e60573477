#ifndef TQ_PROBE_H
#define TQ_PROBE_H

/*
 * Machine probes behind the roofline figures of the benchmark: what this GPU sustains on a
 * pure streaming read and on a pure bf16 or fp16 MFMA loop, and what an empty launch costs.  No counterpart in
 * the reference (its benchmarks report wall-clock only, benchmarks/bench_linear.cpp:50-76).  Built into
 * libtq_probe.so (make probe), which only bench.py loads; not part of the product library or its headers.
 */

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Streams `bytes` (>= 1 MiB) of device memory `repeats` times with 128-bit non-temporal loads;
 * writes the achieved rate in GB/s.  Use a size well above the 256 MB last-level cache.
 * Returns 0 on success. */
int tq_probe_hbm_read(size_t bytes, int repeats, double* gb_per_s);

/* One 512-thread workgroup per CU, every wave a loop of independent v_mfma_f32_32x32x16_bf16 with
 * operands fixed in registers; writes the achieved dense bf16 rate in TFLOP/s.  random_operands = 0
 * uses all-ones operands, 1 uses pseudo-random values in (-1, 1): the sustained clock, and with
 * it the rate, depends on how many bits toggle.  Returns 0 on success. */
int tq_probe_mfma_bf16(int random_operands, int iterations, double* tflops);

/* The same loop with v_mfma_f32_32x32x16_f16, the instruction of the prefill kernel: same nominal rate,
 * more mantissa bits that toggle. */
int tq_probe_mfma_f16(int random_operands, int iterations, double* tflops);

/* `launches` launches of a kernel that does nothing (`workgroups` x `threads`), captured in one HIP graph and
 * replayed: writes the time from one launch to the next in microseconds.  What a layer call costs on this
 * machine before its first instruction: the floor under the microseconds of a small layer. */
int tq_probe_empty_launch(int workgroups, int threads, int launches, double* us_per_launch);

#ifdef __cplusplus
}
#endif

#endif /* TQ_PROBE_H */
