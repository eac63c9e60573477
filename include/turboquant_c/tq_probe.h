#ifndef TURBOQUANT_C_TQ_PROBE_H
#define TURBOQUANT_C_TQ_PROBE_H

/*
 * Machine probes behind the roofline figures of the benchmark: what this GPU sustains on a
 * pure streaming read and on a pure bf16 or fp16 MFMA loop.  No counterpart in the reference (its
 * benchmarks report wall-clock only, benchmarks/bench_linear.cpp:50-76); nothing in the
 * layer path calls these.
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

/* One workgroup of 16 waves per CU; every wave does `per_wave` device-scope relaxed fetch-adds on one of
 * `addresses` (1..64) words, chosen by workgroup; writes the achieved rate in fetch-adds per microsecond
 * over the whole chip.  What a device-wide work counter could hand out: on MI355X about 90 per
 * microsecond on one word (11 ns each, whoever asks), which is why the batch-1 kernel hands its row
 * groups out from counters in LDS and not from one in memory (an lm_head launch has 76 000 of them in
 * 45 us).  Returns 0 on success. */
int tq_probe_device_atomics(int addresses, int per_wave, double* per_microsecond);

#ifdef __cplusplus
}
#endif

#endif /* TURBOQUANT_C_TQ_PROBE_H */
