// Offline TQ8 quantizer on the GPU: the input generator of every layer.
//
// Replaces quantize_weight (src/quantizer.cpp:41-261), derive_seed (:12-28), the scalar
// quantiser (src/codebook.cpp:284-302), the CPU Lloyd-Max fit (src/codebook.cpp:99-143) and the
// per-layer codebook recipe (src/converter.cpp:291-372).  Every fp32 step is the reference's
// operation in the reference's order (normalise, sign, butterfly, 1/sqrt(bs), sqrt(in), lower-bound
// binning, residual, second rotation for dual mode, reconstruction, corrected norm); sums that the
// reference leaves to its tensor runtime (row sums of squares) are accumulated in double in a
// fixed order and rounded once.
//
// One wave handles one (row, 2048-column slab); a lane owns 32 consecutive columns, so the block
// butterflies are the same in-register / cross-lane code the forward kernels use.
#include "tq_device.h"

namespace tq {

constexpr int kQWaves = 4;

struct QuantArgs {
    const float* w;          // [out, in] fp32
    float* orig_norm;        // [out]
    double* recon_partial;   // [out, slabs] sum of squares of the reconstruction
    float* scaled_out;       // optional [out, in]: rotated * sqrt(in) samples (codebook fitting), or NULL
    uint8_t* packed_primary; // [out, in/2] or [out, in]
    uint8_t* packed_residual;// [out, in/2]
    const float* tables;     // [0..31] primary centroids, [32..62] primary boundaries,
                             // [64..79] residual centroids, [80..94] residual boundaries
    int out, in, chunks, slabs;
    int n_primary, n_residual;       // centroid counts
    int primary_bits, residual_bits;
    int shared_rotation;
    uint32_t bs, seed_p, seed_r;
    float scale_factor, inv_scale, inv_sqrt_bs;
    int quantize;            // 0: only write scaled_out
};

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
    return v;
}

// Row sums of squares -> L2 norms (src/quantizer.cpp:56-58).  One wave per row; every lane adds
// its strided elements in order, then a fixed shuffle tree.
__global__ __launch_bounds__(256) void tq_row_norm_kernel(const float* __restrict__ w, float* __restrict__ norms,
                                                          int out, int in) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= out) return;
    const float* p = w + (size_t)row * in;
    double acc = 0.0;
    for (int j = lane; j < in; j += kWave) { const float sq = p[j] * p[j]; acc += (double)sq; }
    acc = wave_sum_f64(acc);
    if (lane == 0) norms[row] = sqrtf((float)acc);
}

// std::lower_bound over the boundaries: number of boundaries strictly below v (src/codebook.cpp:295-297).
__device__ __forceinline__ uint32_t bin_of(float v, const float* bounds, int nb) {
    uint32_t idx = 0;
    for (int k = 0; k < nb; ++k) idx += (bounds[k] < v) ? 1u : 0u;
    return idx;
}

__device__ __forceinline__ void inverse_rotate(float (&v)[kChunk], uint32_t bs, int lane, uint32_t seed,
                                               uint32_t col0, float inv_sqrt_bs) {
    fwht_lane32(v, bs, lane);
#pragma unroll
    for (int k = 0; k < kChunk; ++k) v[k] *= inv_sqrt_bs * sign_of(seed, (col0 + k) & (bs - 1));
}

__device__ __forceinline__ void forward_rotate(float (&v)[kChunk], uint32_t bs, int lane, uint32_t seed,
                                               uint32_t col0, float inv_sqrt_bs) {
#pragma unroll
    for (int k = 0; k < kChunk; ++k) v[k] *= sign_of(seed, (col0 + k) & (bs - 1));
    fwht_lane32(v, bs, lane);
#pragma unroll
    for (int k = 0; k < kChunk; ++k) v[k] *= inv_sqrt_bs;
}

__global__ __launch_bounds__(kQWaves* kWave) void tq_quantize_kernel(QuantArgs a) {
    __shared__ float tab[96];
    for (int i = threadIdx.x; i < 96; i += blockDim.x) tab[i] = a.tables[i];
    __syncthreads();
    const float* cP = tab;
    const float* bP = tab + 32;
    const float* cR = tab + 64;
    const float* bR = tab + 80;

    const int lane = threadIdx.x & 63;
    const long long wid = (long long)blockIdx.x * kQWaves + (threadIdx.x >> 6);
    const int row = (int)(wid / a.slabs);
    const int slab = (int)(wid % a.slabs);
    if (row >= a.out) return;
    const int chunk = slab * kWave + lane;
    const bool active = chunk < a.chunks;
    const uint32_t bs = a.bs;
    const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);
    const size_t elem0 = (size_t)row * a.in + (size_t)chunk * kChunk;

    // normalise (src/quantizer.cpp:62-66), rotate and scale (:74-79)
    float v[kChunk];
    if (active) {
        load_chunk(a.w, kF32, elem0, v);
        const float nrm = a.orig_norm[row];
        const float safe = nrm > 1e-10f ? nrm : 1e-10f;
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = v[k] / safe;
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    forward_rotate(v, bs, lane, a.seed_p, col0, a.inv_sqrt_bs);
#pragma unroll
    for (int k = 0; k < kChunk; ++k) v[k] *= a.scale_factor;

    if (a.scaled_out && active) {
        float4* dst = reinterpret_cast<float4*>(a.scaled_out + elem0);
#pragma unroll
        for (int i = 0; i < 8; ++i) dst[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    }
    if (!a.quantize) return;

    // primary indices (:82-84), clamp as the reference does (codebook.cpp:297)
    uint32_t ip[kChunk], ir[kChunk];
    const int nbp = a.n_primary - 1, nbr = a.n_residual - 1;
#pragma unroll
    for (int k = 0; k < kChunk; ++k) {
        uint32_t idx = bin_of(v[k], bP, nbp);
        ip[k] = idx >= (uint32_t)a.n_primary ? a.n_primary - 1 : idx;
        ir[k] = 0;
    }

    float rec[kChunk];                  // reconstruction in normalised space
    if (a.residual_bits > 0) {
        float res[kChunk];
#pragma unroll
        for (int k = 0; k < kChunk; ++k) res[k] = v[k] - cP[ip[k]];                  // :114-119
        if (!a.shared_rotation) {                                                     // :131-145
#pragma unroll
            for (int k = 0; k < kChunk; ++k) res[k] *= a.inv_scale;
            inverse_rotate(res, bs, lane, a.seed_p, col0, a.inv_sqrt_bs);
            forward_rotate(res, bs, lane, a.seed_r, col0, a.inv_sqrt_bs);
#pragma unroll
            for (int k = 0; k < kChunk; ++k) res[k] *= a.scale_factor;
        }
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
            uint32_t idx = bin_of(res[k], bR, nbr);
            ir[k] = idx >= (uint32_t)a.n_residual ? a.n_residual - 1 : idx;
        }
    }

    // reconstruction (:166-234)
    if (a.residual_bits > 0 && a.shared_rotation) {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
            const float combined = cP[ip[k]] + cR[ir[k] & 15u];
            rec[k] = active ? combined * a.inv_scale : 0.0f;
        }
        inverse_rotate(rec, bs, lane, a.seed_p, col0, a.inv_sqrt_bs);
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) rec[k] = active ? cP[ip[k]] * a.inv_scale : 0.0f;
        inverse_rotate(rec, bs, lane, a.seed_p, col0, a.inv_sqrt_bs);
        if (a.residual_bits > 0) {
            float r2[kChunk];
#pragma unroll
            for (int k = 0; k < kChunk; ++k) r2[k] = active ? cR[ir[k] & 15u] * a.inv_scale : 0.0f;
            inverse_rotate(r2, bs, lane, a.seed_r, col0, a.inv_sqrt_bs);
#pragma unroll
            for (int k = 0; k < kChunk; ++k) rec[k] = rec[k] + r2[k];
        }
    }
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < kChunk; ++k) { const float sq = rec[k] * rec[k]; acc += (double)sq; }
    acc = wave_sum_f64(acc);
    if (lane == 0) a.recon_partial[(size_t)row * a.slabs + slab] = acc;

    // pack (src/quantizer.cpp:33-39,93-107,151-156)
    if (active) {
        if (a.primary_bits <= 4) {
            uint32_t w4[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                uint32_t w = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    w |= ((ip[8 * d + 2 * j] & 15u) | ((ip[8 * d + 2 * j + 1] & 15u) << 4)) << (8 * j);
                w4[d] = w;
            }
            *reinterpret_cast<uint4*>(a.packed_primary + (size_t)row * (a.in >> 1) + (size_t)chunk * 16) =
                make_uint4(w4[0], w4[1], w4[2], w4[3]);
        } else {
            uint32_t w8[8];
#pragma unroll
            for (int d = 0; d < 8; ++d)
                w8[d] = ip[4 * d] | (ip[4 * d + 1] << 8) | (ip[4 * d + 2] << 16) | (ip[4 * d + 3] << 24);
            uint4* dst = reinterpret_cast<uint4*>(a.packed_primary + (size_t)row * a.in + (size_t)chunk * 32);
            dst[0] = make_uint4(w8[0], w8[1], w8[2], w8[3]);
            dst[1] = make_uint4(w8[4], w8[5], w8[6], w8[7]);
        }
        uint32_t r4[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w |= ((ir[8 * d + 2 * j] & 15u) | ((ir[8 * d + 2 * j + 1] & 15u) << 4)) << (8 * j);
            r4[d] = w;
        }
        *reinterpret_cast<uint4*>(a.packed_residual + (size_t)row * (a.in >> 1) + (size_t)chunk * 16) =
            make_uint4(r4[0], r4[1], r4[2], r4[3]);
    }
}

// ---------------------------------------------------------------------------
// The same pipeline for blocks of 1 to 16 columns, i.e. every width that is not a multiple of 32 (the block rule
// of src/converter.cpp:228-240 then picks 16 columns at most) and blocks of one column: the reference quantises
// whatever width is a multiple of its block (src/quantizer.cpp:41-79).  One thread per unit of max(BS, 2)
// columns (whole bytes of the nibble planes), blocks entirely in registers; the butterfly is the in-register
// part of fwht_lanes, so every fp32 operation and its order are those of the kernel above.  No tuning: these
// shapes are small.
// ---------------------------------------------------------------------------
template <int BS>
__device__ __forceinline__ void small_forward(float* x, uint32_t seed, float inv_sqrt_bs) {
#pragma unroll
    for (int k = 0; k < BS; ++k) x[k] *= sign_of(seed, (uint32_t)k);
#pragma unroll
    for (int h = 1; h < BS; h <<= 1)
#pragma unroll
        for (int i = 0; i < BS; i += 2 * h)
#pragma unroll
            for (int j = i; j < i + h; ++j) { const float p = x[j], q = x[j + h]; x[j] = p + q; x[j + h] = p - q; }
#pragma unroll
    for (int k = 0; k < BS; ++k) x[k] *= inv_sqrt_bs;
}

template <int BS>
__device__ __forceinline__ void small_inverse(float* x, uint32_t seed, float inv_sqrt_bs) {
#pragma unroll
    for (int h = 1; h < BS; h <<= 1)
#pragma unroll
        for (int i = 0; i < BS; i += 2 * h)
#pragma unroll
            for (int j = i; j < i + h; ++j) { const float p = x[j], q = x[j + h]; x[j] = p + q; x[j + h] = p - q; }
#pragma unroll
    for (int k = 0; k < BS; ++k) x[k] *= inv_sqrt_bs * sign_of(seed, (uint32_t)k);
}

template <int BS>
__global__ __launch_bounds__(256) void tq_quantize_small_kernel(QuantArgs a) {
    constexpr int U = BS < 2 ? 2 : BS;              // columns of one thread
    constexpr int NB = U / BS;                      // its blocks
    __shared__ float tab[96];
    for (int i = threadIdx.x; i < 96; i += blockDim.x) tab[i] = a.tables[i];
    __syncthreads();
    const float* cP = tab;
    const float* bP = tab + 32;
    const float* cR = tab + 64;
    const float* bR = tab + 80;
    const int units = a.in / U;                     // a.slabs == units: one partial sum of squares per unit
    const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
    const int row = (int)(id / units);
    const int unit = (int)(id - (long long)row * units);
    if (row >= a.out) return;
    const size_t elem0 = (size_t)row * a.in + (size_t)unit * U;

    float v[U];
    const float nrm = a.orig_norm[row];
    const float safe = nrm > 1e-10f ? nrm : 1e-10f;
#pragma unroll
    for (int k = 0; k < U; ++k) v[k] = a.w[elem0 + k] / safe;
#pragma unroll
    for (int b = 0; b < NB; ++b) small_forward<BS>(v + b * BS, a.seed_p, a.inv_sqrt_bs);
#pragma unroll
    for (int k = 0; k < U; ++k) v[k] *= a.scale_factor;
    if (a.scaled_out) {
#pragma unroll
        for (int k = 0; k < U; ++k) a.scaled_out[elem0 + k] = v[k];
    }
    if (!a.quantize) return;

    uint32_t ip[U], ir[U];
    const int nbp = a.n_primary - 1, nbr = a.n_residual - 1;
#pragma unroll
    for (int k = 0; k < U; ++k) {
        const uint32_t idx = bin_of(v[k], bP, nbp);
        ip[k] = idx >= (uint32_t)a.n_primary ? a.n_primary - 1 : idx;
        ir[k] = 0;
    }
    float rec[U];
    if (a.residual_bits > 0) {
        float res[U];
#pragma unroll
        for (int k = 0; k < U; ++k) res[k] = v[k] - cP[ip[k]];
        if (!a.shared_rotation) {
#pragma unroll
            for (int k = 0; k < U; ++k) res[k] *= a.inv_scale;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                small_inverse<BS>(res + b * BS, a.seed_p, a.inv_sqrt_bs);
                small_forward<BS>(res + b * BS, a.seed_r, a.inv_sqrt_bs);
            }
#pragma unroll
            for (int k = 0; k < U; ++k) res[k] *= a.scale_factor;
        }
#pragma unroll
        for (int k = 0; k < U; ++k) {
            const uint32_t idx = bin_of(res[k], bR, nbr);
            ir[k] = idx >= (uint32_t)a.n_residual ? a.n_residual - 1 : idx;
        }
    }
    if (a.residual_bits > 0 && a.shared_rotation) {
#pragma unroll
        for (int k = 0; k < U; ++k) rec[k] = (cP[ip[k]] + cR[ir[k] & 15u]) * a.inv_scale;
#pragma unroll
        for (int b = 0; b < NB; ++b) small_inverse<BS>(rec + b * BS, a.seed_p, a.inv_sqrt_bs);
    } else {
#pragma unroll
        for (int k = 0; k < U; ++k) rec[k] = cP[ip[k]] * a.inv_scale;
#pragma unroll
        for (int b = 0; b < NB; ++b) small_inverse<BS>(rec + b * BS, a.seed_p, a.inv_sqrt_bs);
        if (a.residual_bits > 0) {
            float r2[U];
#pragma unroll
            for (int k = 0; k < U; ++k) r2[k] = cR[ir[k] & 15u] * a.inv_scale;
#pragma unroll
            for (int b = 0; b < NB; ++b) small_inverse<BS>(r2 + b * BS, a.seed_r, a.inv_sqrt_bs);
#pragma unroll
            for (int k = 0; k < U; ++k) rec[k] = rec[k] + r2[k];
        }
    }
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < U; ++k) { const float sq = rec[k] * rec[k]; acc += (double)sq; }
    a.recon_partial[(size_t)row * units + unit] = acc;

    // pack: lo nibble = even column (src/quantizer.cpp:33-39); 5-bit primaries one index per byte
    if (a.primary_bits <= 4) {
        uint8_t* dst = a.packed_primary + (size_t)row * (a.in >> 1) + (size_t)unit * (U / 2);
#pragma unroll
        for (int k = 0; k < U; k += 2) dst[k >> 1] = (uint8_t)((ip[k] & 15u) | ((ip[k + 1] & 15u) << 4));
    } else {
        uint8_t* dst = a.packed_primary + elem0;
#pragma unroll
        for (int k = 0; k < U; ++k) dst[k] = (uint8_t)ip[k];
    }
    uint8_t* dstr = a.packed_residual + (size_t)row * (a.in >> 1) + (size_t)unit * (U / 2);
#pragma unroll
    for (int k = 0; k < U; k += 2) dstr[k >> 1] = (uint8_t)((ir[k] & 15u) | ((ir[k + 1] & 15u) << 4));
}

// corrected_norm = orig / max(||recon||, 1e-10)  (src/quantizer.cpp:237-248)
__global__ void tq_finish_norms_kernel(const float* __restrict__ orig, const double* __restrict__ partial,
                                       float* __restrict__ norms, int out, int slabs) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= out) return;
    double acc = 0.0;
    for (int s = 0; s < slabs; ++s) acc += partial[(size_t)r * slabs + s];
    const float rn = sqrtf((float)acc);
    const float safe = rn > 1e-10f ? rn : 1e-10f;
    norms[r] = orig[r] / safe;
}

// FNV-1a over sampled bytes of the fp32 weight, salts 0 and 1 (src/quantizer.cpp:12-28).
__global__ __launch_bounds__(1024) void tq_derive_seed_kernel(const uint8_t* __restrict__ bytes, size_t byte_count,
                                                              uint32_t* __restrict__ seeds_out) {
    __shared__ uint8_t sample[8192];
    const size_t stride = (byte_count > 4096) ? (byte_count / 4096) : 1;
    const size_t count = (byte_count + stride - 1) / stride;       // < 8192
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) sample[i] = bytes[i * stride];
    __syncthreads();
    if (threadIdx.x < 2) {
        uint32_t hash = 2166136261u ^ (uint32_t)threadIdx.x;
        for (size_t i = 0; i < count; ++i) { hash ^= sample[i]; hash *= 16777619u; }
        seeds_out[threadIdx.x] = hash;
    }
}

// One Lloyd-Max assignment pass (src/codebook.cpp:111-120): per-bin double sums and counts.
// Every thread owns a private set of bins in LDS and adds its strided samples in order; the
// workgroup then folds the sets in a fixed order and writes one partial per workgroup, which the
// host-side driver folds in workgroup order, so the result does not depend on scheduling.
// With `subtract` set the sample is the residual against `gcent/gbounds` (src/converter.cpp:348-356).
constexpr int kFitThreads = 256;
__global__ __launch_bounds__(kFitThreads) void tq_lloyd_pass_kernel(const float* __restrict__ data, size_t n,
                                                                    const float* __restrict__ bounds, int nc,
                                                                    int subtract, const float* __restrict__ gcent,
                                                                    const float* __restrict__ gbounds, int ngc,
                                                                    double* __restrict__ part_sum,
                                                                    unsigned long long* __restrict__ part_cnt) {
    __shared__ double s_sum[32 * kFitThreads];
    __shared__ unsigned int s_cnt[32 * kFitThreads];
    __shared__ float s_b[32], s_gb[32], s_gc[32];
    const int tid = threadIdx.x;
    if (tid < 32) {
        s_b[tid] = tid < nc - 1 ? bounds[tid] : 0.0f;
        s_gb[tid] = (subtract && tid < ngc - 1) ? gbounds[tid] : 0.0f;
        s_gc[tid] = (subtract && tid < ngc) ? gcent[tid] : 0.0f;
    }
    for (int k = 0; k < nc; ++k) { s_sum[k * kFitThreads + tid] = 0.0; s_cnt[k * kFitThreads + tid] = 0u; }
    __syncthreads();
    const size_t per_wg = (n + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per_wg;
    const size_t hi = lo + per_wg < n ? lo + per_wg : n;
    for (size_t i = lo + tid; i < hi; i += kFitThreads) {
        float v = data[i];
        if (subtract) {
            uint32_t g = bin_of(v, s_gb, ngc - 1);
            if (g >= (uint32_t)ngc) g = ngc - 1;
            v = v - s_gc[g];
        }
        uint32_t idx = bin_of(v, s_b, nc - 1);
        if (idx >= (uint32_t)nc) idx = nc - 1;
        s_sum[idx * kFitThreads + tid] += (double)v;
        s_cnt[idx * kFitThreads + tid] += 1u;
    }
    __syncthreads();
    if (tid < nc) {
        double s = 0.0; unsigned long long c = 0;
        for (int t = 0; t < kFitThreads; ++t) { s += s_sum[tid * kFitThreads + t]; c += s_cnt[tid * kFitThreads + t]; }
        part_sum[(size_t)blockIdx.x * 32 + tid] = s;
        part_cnt[(size_t)blockIdx.x * 32 + tid] = c;
    }
}

// ---------------------------------------------------------------------------
// Scalar codebook maps (reference src/codebook.cpp:284-321): value -> bin index, index -> centroid.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void tq_codebook_quantize_kernel(const float* __restrict__ values, size_t n,
                                                                   const float* __restrict__ bounds, int nc,
                                                                   uint8_t* __restrict__ indices) {
    __shared__ float s_b[32];
    if (threadIdx.x < 32) s_b[threadIdx.x] = (int)threadIdx.x < nc - 1 ? bounds[threadIdx.x] : 0.0f;
    __syncthreads();
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t idx = bin_of(values[i], s_b, nc - 1);
        if (idx >= (uint32_t)nc) idx = nc - 1;
        indices[i] = (uint8_t)idx;
    }
}

__global__ __launch_bounds__(256) void tq_codebook_lookup_kernel(const uint8_t* __restrict__ indices, size_t n,
                                                                 const float* __restrict__ centroids, int nc,
                                                                 float* __restrict__ values) {
    __shared__ float s_c[32];
    if (threadIdx.x < 32) s_c[threadIdx.x] = (int)threadIdx.x < nc ? centroids[threadIdx.x] : 0.0f;
    __syncthreads();
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t idx = indices[i];
        if (idx >= (uint32_t)nc) idx = nc - 1;                  // src/codebook.cpp:316
        values[i] = s_c[idx];
    }
}

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
static unsigned elementwise_grid(size_t n) {
    const size_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

hipError_t launch_codebook_quantize(const float* values, size_t n, const float* bounds_dev, int nc, uint8_t* indices,
                                    hipStream_t stream) {
    hipLaunchKernelGGL(tq_codebook_quantize_kernel, dim3(elementwise_grid(n)), dim3(256), 0, stream, values, n,
                       bounds_dev, nc, indices);
    return hipGetLastError();
}

hipError_t launch_codebook_lookup(const uint8_t* indices, size_t n, const float* centroids_dev, int nc, float* values,
                                  hipStream_t stream) {
    hipLaunchKernelGGL(tq_codebook_lookup_kernel, dim3(elementwise_grid(n)), dim3(256), 0, stream, indices, n,
                       centroids_dev, nc, values);
    return hipGetLastError();
}

hipError_t launch_row_norms(const float* w, float* norms, int out, int in, hipStream_t stream) {
    hipLaunchKernelGGL(tq_row_norm_kernel, dim3((out + 3) / 4), dim3(256), 0, stream, w, norms, out, in);
    return hipGetLastError();
}

hipError_t launch_derive_seeds(const float* w, size_t n_floats, uint32_t* seeds_dev, hipStream_t stream) {
    hipLaunchKernelGGL(tq_derive_seed_kernel, dim3(1), dim3(1024), 0, stream,
                       reinterpret_cast<const uint8_t*>(w), n_floats * sizeof(float), seeds_dev);
    return hipGetLastError();
}

// Partial sums of squares per row that launch_quantize_rows writes (what recon_partial must hold and
// launch_finish_norms is told): 2048-column slabs, or for blocks of at most 16 columns on widths the lane
// kernel does not take, units of max(block, 2) columns.
int quantize_partials_per_row(int in, uint32_t bs) {
    if (lanes_supported(in, bs)) return (in / kChunk + kWave - 1) / kWave;
    return in / (int)(bs < 2 ? 2 : bs);
}

hipError_t launch_quantize_rows(const QuantArgsHost& h, hipStream_t stream) {
    QuantArgs a{};
    a.w = h.w; a.orig_norm = h.orig_norm; a.recon_partial = h.recon_partial; a.scaled_out = h.scaled_out;
    a.packed_primary = h.packed_primary; a.packed_residual = h.packed_residual; a.tables = h.tables;
    a.out = h.out; a.in = h.in; a.chunks = h.in / kChunk; a.slabs = (a.chunks + kWave - 1) / kWave;
    a.n_primary = h.n_primary; a.n_residual = h.n_residual;
    a.primary_bits = h.primary_bits; a.residual_bits = h.residual_bits; a.shared_rotation = h.shared_rotation;
    a.bs = h.bs; a.seed_p = h.seed_p; a.seed_r = h.seed_r;
    a.scale_factor = h.scale_factor; a.inv_scale = h.inv_scale; a.inv_sqrt_bs = h.inv_sqrt_bs;
    a.quantize = h.quantize;
    if (!lanes_supported(h.in, h.bs)) {                 // blocks of 1 to 16 columns, in registers
        if (!layout_valid(h.in, h.bs) || h.bs > 16) return hipErrorInvalidValue;
        a.slabs = quantize_partials_per_row(h.in, h.bs);
        const long long threads = (long long)a.out * a.slabs;
        const long long g = (threads + 255) / 256;
        if (g > 0x7fffffffLL) return hipErrorInvalidValue;
        const dim3 grid((unsigned)g), block(256);
        switch (h.bs) {
            case 1: hipLaunchKernelGGL(tq_quantize_small_kernel<1>, grid, block, 0, stream, a); break;
            case 2: hipLaunchKernelGGL(tq_quantize_small_kernel<2>, grid, block, 0, stream, a); break;
            case 4: hipLaunchKernelGGL(tq_quantize_small_kernel<4>, grid, block, 0, stream, a); break;
            case 8: hipLaunchKernelGGL(tq_quantize_small_kernel<8>, grid, block, 0, stream, a); break;
            default: hipLaunchKernelGGL(tq_quantize_small_kernel<16>, grid, block, 0, stream, a); break;
        }
        return hipGetLastError();
    }
    const long long waves = (long long)a.out * a.slabs;
    const long long grid = (waves + kQWaves - 1) / kQWaves;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tq_quantize_kernel, dim3((unsigned)grid), dim3(kQWaves * kWave), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_finish_norms(const float* orig, const double* partial, float* norms, int out, int slabs,
                               hipStream_t stream) {
    hipLaunchKernelGGL(tq_finish_norms_kernel, dim3((out + 255) / 256), dim3(256), 0, stream, orig, partial, norms,
                       out, slabs);
    return hipGetLastError();
}

hipError_t launch_lloyd_pass(const float* data, size_t n, const float* bounds_dev, int nc, int subtract,
                             const float* gcent_dev, const float* gbounds_dev, int ngc,
                             double* part_sum, unsigned long long* part_cnt, int workgroups, hipStream_t stream) {
    hipLaunchKernelGGL(tq_lloyd_pass_kernel, dim3(workgroups), dim3(kFitThreads), 0, stream, data, n, bounds_dev, nc,
                       subtract, gcent_dev, gbounds_dev, ngc, part_sum, part_cnt);
    return hipGetLastError();
}

}  // namespace tq
