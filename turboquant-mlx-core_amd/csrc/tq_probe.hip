// Machine probes for the roofline denominators and for design decisions: what this GPU sustains on a pure
// streaming read, on a pure bf16 or fp16 MFMA loop, and on device-scope fetch-adds from every wave of the chip.
// Measurement support only: nothing in the layer path calls them.
#include "turboquant_c/tq_probe.h"

#include "tq_device.h"

namespace tq {

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

// Every wave of a one-workgroup-per-CU launch does `per_wave` device-scope relaxed fetch-adds (lane 0) on
// one of `addresses` words, 256 bytes apart, chosen by workgroup.
__global__ __launch_bounds__(1024) void tq_probe_atomic_kernel(unsigned* ctr, int per_wave, int addresses, unsigned* sink) {
    const int lane = threadIdx.x & 63;
    unsigned* const c = ctr + (blockIdx.x % addresses) * 64;
    unsigned acc = 0;
    for (int i = 0; i < per_wave; ++i) {
        unsigned t = 0;
        if (lane == 0) t = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        acc += __builtin_amdgcn_readfirstlane(t);
    }
    if (acc == 0xdeadbeefu) sink[0] = acc;
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

int tq_probe_device_atomics(int addresses, int per_wave, double* per_microsecond) {
    try {
        if (!per_microsecond || addresses < 1 || addresses > 64 || per_wave < 1) { tq::set_error("tq_probe_device_atomics: bad argument"); return 1; }
        int dev = 0; hipDeviceProp_t prop;
        if (!tq::hip_ok(hipGetDevice(&dev), "hipGetDevice") || !tq::hip_ok(hipGetDeviceProperties(&prop, dev), "properties")) return 1;
        const int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        unsigned* ctr = nullptr; unsigned* sink = nullptr;
        hipEvent_t t0 = nullptr, t1 = nullptr;
        bool ok = tq::hip_ok(hipMalloc((void**)&ctr, 64 * 64 * sizeof(unsigned)), "hipMalloc(counters)") &&
                  tq::hip_ok(hipMalloc((void**)&sink, 4), "hipMalloc(sink)") &&
                  tq::hip_ok(hipMemset(ctr, 0, 64 * 64 * sizeof(unsigned)), "hipMemset(counters)") &&
                  tq::hip_ok(hipEventCreate(&t0), "event") && tq::hip_ok(hipEventCreate(&t1), "event");
        float ms = 0.0f;
        const int reps = 5;
        if (ok) {
            hipLaunchKernelGGL(tq::tq_probe_atomic_kernel, dim3(cus), dim3(1024), 0, nullptr, ctr, per_wave, addresses, sink);
            (void)hipEventRecord(t0, nullptr);
            for (int r = 0; r < reps; ++r)
                hipLaunchKernelGGL(tq::tq_probe_atomic_kernel, dim3(cus), dim3(1024), 0, nullptr, ctr, per_wave, addresses, sink);
            (void)hipEventRecord(t1, nullptr);
            ok = tq::hip_ok(hipEventSynchronize(t1), "probe sync") && tq::hip_ok(hipEventElapsedTime(&ms, t0, t1), "elapsed");
        }
        if (ok) *per_microsecond = (double)cus * 16.0 * per_wave * reps / (ms * 1e3);
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        if (ctr) (void)hipFree(ctr);
        if (sink) (void)hipFree(sink);
        return ok ? 0 : 1;
    } catch (...) { tq::set_error("tq_probe_device_atomics: exception"); return 1; }
}

}  // extern "C"
