// Machine probes for the roofline denominators and for design decisions: what this GPU sustains on a pure
// streaming read and on a pure bf16 or fp16 MFMA loop, and what a kernel launch costs before it does anything.
// Measurement support only, a library of its own (libtq_probe.so, `make probe`): nothing in the layer path calls
// them and the product library does not contain them.
#include "tq_probe.h"

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace tq {

namespace {
bool hip_ok(hipError_t e, const char* what) {
    if (e == hipSuccess) return true;
    fprintf(stderr, "tq_probe: %s: %s\n", what, hipGetErrorString(e));
    return false;
}
void set_error(const char* msg) { fprintf(stderr, "%s\n", msg); }
}  // namespace

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 probe_f16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));

// Every workgroup reads a contiguous share of the buffer with 128-bit non-temporal loads.
__global__ __launch_bounds__(512) void tq_probe_read_kernel(const probe_u32x4* __restrict__ src, size_t n16,
                                                            uint32_t* __restrict__ sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
    uint32_t acc = 0;
    for (size_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const probe_u32x4 v = __builtin_nontemporal_load(src + i);
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;                    // keeps the loads alive
}

// 8 waves per CU, each a loop of 16 independent v_mfma_f32_32x32x16_bf16 (HALF: _f16, the instruction
// of the prefill kernel's inner step) per iteration, operands fixed in registers.
template <bool HALF>
__global__ __launch_bounds__(512) void tq_probe_mfma_kernel(float* __restrict__ sink, int iters, int random_operands) {
    probe_f32x16 acc[8];
    for (int i = 0; i < 8; ++i)
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    probe_bf16x8 a, b;
    probe_f16x8 ah, bh;
    uint32_t h = (threadIdx.x + 1) * 2654435761u + blockIdx.x * 40503u;
    for (int j = 0; j < 8; ++j) {
        h = h * 1664525u + 1013904223u;
        const float va = random_operands ? ((int)(h >> 8) % 2001 - 1000) * 1e-3f : 1.0f;
        h = h * 1664525u + 1013904223u;
        const float vb = random_operands ? ((int)(h >> 8) % 2001 - 1000) * 1e-3f : 1.0f;
        a[j] = (__bf16)va; b[j] = (__bf16)vb;
        ah[j] = (_Float16)va; bh[j] = (_Float16)vb;
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if constexpr (HALF) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, acc[i], 0, 0, 0);
                else acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
            }
        __syncthreads();
    }
    float s = 0.0f;
    for (int i = 0; i < 8; ++i) s += acc[i][0];
    if (s == 123.456f) sink[0] = s;
}

// A kernel that does nothing: `waves` waves per workgroup start, end, and that is all.
__global__ void tq_probe_empty_kernel(int* never) {
    if (never && threadIdx.x == 0xffffff) never[0] = 1;
}

}  // namespace tq

extern "C" {

int tq_probe_hbm_read(size_t bytes, int repeats, double* gb_per_s) {
    try {
        if (!gb_per_s || bytes < (1u << 20) || repeats <= 0) { tq::set_error("tq_probe_hbm_read: bad argument"); return 1; }
        void* buf = nullptr; uint32_t* sink = nullptr;
        hipEvent_t t0 = nullptr, t1 = nullptr;
        const size_t n16 = bytes / 16;
        bool ok = tq::hip_ok(hipMalloc(&buf, n16 * 16), "hipMalloc(probe)") &&
                  tq::hip_ok(hipMalloc((void**)&sink, 4), "hipMalloc(sink)") &&
                  tq::hip_ok(hipMemset(buf, 0x5a, n16 * 16), "hipMemset(probe)") &&
                  tq::hip_ok(hipEventCreate(&t0), "event") && tq::hip_ok(hipEventCreate(&t1), "event");
        float ms = 0.0f;
        if (ok) {
            hipLaunchKernelGGL(tq::tq_probe_read_kernel, dim3(2048), dim3(512), 0, nullptr,
                               static_cast<const tq::probe_u32x4*>(buf), n16, sink);            // warm-up
            (void)hipEventRecord(t0, nullptr);
            for (int r = 0; r < repeats; ++r)
                hipLaunchKernelGGL(tq::tq_probe_read_kernel, dim3(2048), dim3(512), 0, nullptr,
                                   static_cast<const tq::probe_u32x4*>(buf), n16, sink);
            (void)hipEventRecord(t1, nullptr);
            ok = tq::hip_ok(hipEventSynchronize(t1), "probe sync") && tq::hip_ok(hipEventElapsedTime(&ms, t0, t1), "elapsed");
        }
        if (ok) *gb_per_s = (double)n16 * 16.0 * repeats / (ms * 1e-3) / 1e9;
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        if (buf) (void)hipFree(buf);
        if (sink) (void)hipFree(sink);
        return ok ? 0 : 1;
    } catch (...) { tq::set_error("tq_probe_hbm_read: exception"); return 1; }
}

static int probe_mfma(bool half, int random_operands, int iterations, double* tflops) {
    try {
        if (!tflops || iterations <= 0) { tq::set_error("tq_probe_mfma: bad argument"); return 1; }
        int dev = 0, cus = 0;
        float* sink = nullptr;
        hipEvent_t t0 = nullptr, t1 = nullptr;
        bool ok = tq::hip_ok(hipGetDevice(&dev), "hipGetDevice") &&
                  tq::hip_ok(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev), "CU count") &&
                  tq::hip_ok(hipMalloc((void**)&sink, 4), "hipMalloc(sink)") &&
                  tq::hip_ok(hipEventCreate(&t0), "event") && tq::hip_ok(hipEventCreate(&t1), "event");
        float ms = 0.0f;
        if (ok) {
            if (half) hipLaunchKernelGGL(tq::tq_probe_mfma_kernel<true>, dim3(cus), dim3(512), 0, nullptr, sink, 64, random_operands);
            else hipLaunchKernelGGL(tq::tq_probe_mfma_kernel<false>, dim3(cus), dim3(512), 0, nullptr, sink, 64, random_operands);
            (void)hipEventRecord(t0, nullptr);
            if (half) hipLaunchKernelGGL(tq::tq_probe_mfma_kernel<true>, dim3(cus), dim3(512), 0, nullptr, sink, iterations, random_operands);
            else hipLaunchKernelGGL(tq::tq_probe_mfma_kernel<false>, dim3(cus), dim3(512), 0, nullptr, sink, iterations, random_operands);
            (void)hipEventRecord(t1, nullptr);
            ok = tq::hip_ok(hipEventSynchronize(t1), "probe sync") && tq::hip_ok(hipEventElapsedTime(&ms, t0, t1), "elapsed");
        }
        // 32 x 32 x 16 multiply-adds = 32768 flop per instruction, 16 per iteration and wave, 8 waves per workgroup
        if (ok) *tflops = (double)cus * 8.0 * iterations * 16.0 * 32768.0 / (ms * 1e-3) / 1e12;
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        if (sink) (void)hipFree(sink);
        return ok ? 0 : 1;
    } catch (...) { tq::set_error("tq_probe_mfma: exception"); return 1; }
}

int tq_probe_mfma_bf16(int random_operands, int iterations, double* tflops) {
    return probe_mfma(false, random_operands, iterations, tflops);
}

int tq_probe_mfma_f16(int random_operands, int iterations, double* tflops) {
    return probe_mfma(true, random_operands, iterations, tflops);
}

int tq_probe_empty_launch(int workgroups, int threads, int launches, double* us_per_launch) {
    try {
        if (!us_per_launch || workgroups < 1 || threads < 64 || threads > 1024 || launches < 1) {
            tq::set_error("tq_probe_empty_launch: bad argument"); return 1;
        }
        hipStream_t st = nullptr;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        hipEvent_t t0 = nullptr, t1 = nullptr;
        bool ok = tq::hip_ok(hipStreamCreate(&st), "stream") && tq::hip_ok(hipEventCreate(&t0), "event") &&
                  tq::hip_ok(hipEventCreate(&t1), "event") &&
                  tq::hip_ok(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal), "begin capture");
        if (ok) {
            for (int i = 0; i < launches; ++i)
                hipLaunchKernelGGL(tq::tq_probe_empty_kernel, dim3(workgroups), dim3(threads), 0, st, (int*)nullptr);
            ok = tq::hip_ok(hipStreamEndCapture(st, &graph), "end capture") &&
                 tq::hip_ok(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "instantiate");
        }
        float ms = 0.0f;
        const int reps = 20;
        if (ok) {
            for (int r = 0; r < 3 && ok; ++r) ok = tq::hip_ok(hipGraphLaunch(exec, st), "graph launch");
            ok = ok && tq::hip_ok(hipStreamSynchronize(st), "sync");
            if (ok) (void)hipEventRecord(t0, st);
            for (int r = 0; r < reps && ok; ++r) ok = tq::hip_ok(hipGraphLaunch(exec, st), "graph launch");
            if (ok) (void)hipEventRecord(t1, st);
            ok = ok && tq::hip_ok(hipEventSynchronize(t1), "probe sync") && tq::hip_ok(hipEventElapsedTime(&ms, t0, t1), "elapsed");
        }
        if (ok) *us_per_launch = (double)ms * 1e3 / ((double)reps * launches);
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        if (st) (void)hipStreamDestroy(st);
        return ok ? 0 : 1;
    } catch (...) { tq::set_error("tq_probe_empty_launch: exception"); return 1; }
}

}  // extern "C"
