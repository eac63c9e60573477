// Materialising dequantiser and stand-alone block rotation for gfx950.
//
// tq_dequant_kernel rebuilds the fp32 weight [out, in] from the packed indices and
// follows the reference CPU dequantiser operation by operation
// (src/dequantizer.cpp:52-256 with the inverse rotation of src/rotation.cpp:323-350):
// lookup, * 1/sqrt(in), butterfly, * (1/sqrt(bs) * sign), [+ residual plane], * norm.
// Every step is a single fp32 operation in the reference's order (this file is
// compiled with -ffp-contract=off), so the output is bit-identical to the CPU path.
//
// One wave handles one (row, 2048-column slab); a lane owns 32 consecutive columns.
#include "tq_device.h"

namespace tq {

constexpr int kDqWaves = 4;   // waves per workgroup

__device__ __forceinline__ void unpack_nibbles(const uint4& P, uint32_t (&idx)[kChunk]) {
    const uint32_t w[4] = {P.x, P.y, P.z, P.w};
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t byte = (w[d] >> (8 * j)) & 0xffu;
            idx[8 * d + 2 * j]     = byte & 0x0fu;   // lo nibble = even column (src/dequantizer.cpp:46)
            idx[8 * d + 2 * j + 1] = byte >> 4;      // hi nibble = odd column  (src/dequantizer.cpp:47)
        }
}

__global__ __launch_bounds__(kDqWaves* kWave) void tq_dequant_kernel(LayerView L, void* __restrict__ Wout,
                                                                      int w_dtype, int chunks, int slabs) {
    __shared__ float tab[256];
    for (int i = threadIdx.x; i < 256; i += blockDim.x) tab[i] = L.tables[i];
    __syncthreads();

    const int lane = threadIdx.x & (kWave - 1);
    const long long wid = (long long)blockIdx.x * kDqWaves + (threadIdx.x >> 6);
    const int row = (int)(wid / slabs);
    const int slab = (int)(wid % slabs);
    if (row >= L.out_features) return;          // whole wave leaves together
    const int chunk = slab * kWave + lane;
    const bool active = chunk < chunks;
    const int in = L.in_features;
    const uint32_t bs = L.block_size;
    const bool five = (L.mode >= kShared5);
    const bool has_res = (L.mode != kPrimaryOnly && L.mode != kPrimaryOnly5);
    const bool shared = (L.mode == kSharedLut || L.mode == kShared5);

    uint32_t pi[kChunk], ri[kChunk];
    float v[kChunk];
    if (active && L.mode == kSharedLut) {
        // combined plane: one byte per weight, residual nibble high, primary nibble low
        const uint4* p = reinterpret_cast<const uint4*>(L.packed_combined + (size_t)row * in + (size_t)chunk * 32);
        const uint4 a = p[0], b = p[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int d = 0; d < 8; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t c = (w[d] >> (8 * j)) & 0xffu;
                pi[4 * d + j] = c & 0x0fu;
                ri[4 * d + j] = c >> 4;
            }
    } else if (active && five && L.packed_combined) {
        // 5-bit primary with a residual of at most 3 bits: one byte per weight, residual index in
        // the top 3 bits (both already clamped to their codebooks when the plane was built)
        const uint4* p = reinterpret_cast<const uint4*>(L.packed_combined + (size_t)row * in + (size_t)chunk * 32);
        const uint4 a = p[0], b = p[1];
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int d = 0; d < 8; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t c = (w[d] >> (8 * j)) & 0xffu;
                pi[4 * d + j] = c & 0x1fu;
                ri[4 * d + j] = c >> 5;
            }
    } else if (active) {
        if (five) {
            const uint4* p = reinterpret_cast<const uint4*>(L.packed_primary + (size_t)row * in + (size_t)chunk * 32);
            const uint4 a = p[0], b = p[1];
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int d = 0; d < 8; ++d)
#pragma unroll
                for (int j = 0; j < 4; ++j) pi[4 * d + j] = (w[d] >> (8 * j)) & 0xffu;
        } else {
            unpack_nibbles(*reinterpret_cast<const uint4*>(L.packed_primary + (size_t)row * (in >> 1) + (size_t)chunk * 16), pi);
        }
        if (has_res)
            unpack_nibbles(*reinterpret_cast<const uint4*>(L.packed_residual + (size_t)row * (in >> 1) + (size_t)chunk * 16), ri);
    }

    const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);
    const float nrm = L.norms[row];

    if (L.mode == kSharedLut) {
        // path A: 256-entry table of centroid sums (src/dequantizer.cpp:136-184)
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = active ? tab[(ri[k] << 4) | pi[k]] * L.inv_scale : 0.0f;
    } else {
        const int roff = five ? 32 : 16;
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
            float c = 0.0f;
            if (active) {
                c = tab[five ? (pi[k] > 31u ? 31u : pi[k]) : pi[k]];
                if (shared) c = c + tab[roff + ri[k]];       // path B (src/dequantizer.cpp:186-212)
            }
            v[k] = c * L.inv_scale;
        }
    }
    fwht_lane32(v, bs, lane);
#pragma unroll
    for (int k = 0; k < kChunk; ++k) v[k] *= L.inv_sqrt_bs * sign_of(L.seed_primary, (col0 + k) & (bs - 1));

    if (has_res && !shared) {
        // path C second plane (src/dequantizer.cpp:220-245)
        const int roff = five ? 32 : 16;
        float u[kChunk];
#pragma unroll
        for (int k = 0; k < kChunk; ++k) u[k] = active ? tab[roff + ri[k]] * L.inv_scale : 0.0f;
        fwht_lane32(u, bs, lane);
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
            u[k] *= L.inv_sqrt_bs * sign_of(L.seed_residual, (col0 + k) & (bs - 1));
            v[k] = v[k] + u[k];
        }
    }

    if (!active) return;
    const size_t elem = (size_t)row * in + (size_t)chunk * kChunk;
    if (w_dtype == kF32) {
        float4* dst = reinterpret_cast<float4*>(static_cast<float*>(Wout) + elem);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            dst[i] = make_float4(v[4 * i] * nrm, v[4 * i + 1] * nrm, v[4 * i + 2] * nrm, v[4 * i + 3] * nrm);
    } else {
        // The fp32 weight rounded to nearest-even, the cast src/turboquant_c_dequant.cpp:166 applies.
        uint4* dst = reinterpret_cast<uint4*>(static_cast<uint16_t*>(Wout) + elem);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t h[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float f = v[8 * i + j] * nrm;
                h[j] = (w_dtype == kBF16) ? (uint32_t)float_to_bf16_bits(f)
                                          : (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
            }
            dst[i] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
        }
    }
}

hipError_t launch_dequant(const LayerView& L, void* w, int w_dtype, hipStream_t stream) {
    const int chunks = L.in_features / kChunk;
    const int slabs = (chunks + kWave - 1) / kWave;
    const long long waves = (long long)L.out_features * slabs;
    const long long grid = (waves + kDqWaves - 1) / kDqWaves;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tq_dequant_kernel, dim3((unsigned)grid), dim3(kDqWaves * kWave), 0, stream, L, w, w_dtype, chunks,
                       slabs);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Block rotation of an fp32 matrix (reference src/rotation.cpp:291-350).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kDqWaves* kWave) void tq_wht_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                                  int rows, int cols, int chunks, int slabs,
                                                                  uint32_t seed, uint32_t bs, float inv_sqrt_bs,
                                                                  int inverse) {
    const int lane = threadIdx.x & (kWave - 1);
    const long long wid = (long long)blockIdx.x * kDqWaves + (threadIdx.x >> 6);
    const int row = (int)(wid / slabs);
    const int slab = (int)(wid % slabs);
    if (row >= rows) return;
    const int chunk = slab * kWave + lane;
    const bool active = chunk < chunks;
    const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);

    float v[kChunk];
    if (active) {
        load_chunk(in, kF32, (size_t)row * cols + (size_t)chunk * kChunk, v);
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    if (!inverse) {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= sign_of(seed, (col0 + k) & (bs - 1));
    }
    fwht_lane32(v, bs, lane);
    if (!inverse) {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= inv_sqrt_bs;
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= inv_sqrt_bs * sign_of(seed, (col0 + k) & (bs - 1));
    }
    if (active) {
        float4* dst = reinterpret_cast<float4*>(out + (size_t)row * cols + (size_t)chunk * kChunk);
#pragma unroll
        for (int i = 0; i < 8; ++i) dst[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    }
}

hipError_t launch_wht(const float* in, float* out, int rows, int cols, uint32_t seed,
                      uint32_t block_size, float inv_sqrt_bs, int inverse, hipStream_t stream) {
    const int chunks = cols / kChunk;
    const int slabs = (chunks + kWave - 1) / kWave;
    const long long waves = (long long)rows * slabs;
    const long long grid = (waves + kDqWaves - 1) / kDqWaves;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tq_wht_kernel, dim3((unsigned)grid), dim3(kDqWaves * kWave), 0, stream,
                       in, out, rows, cols, chunks, slabs, seed, block_size, inv_sqrt_bs, inverse);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// "Does the residual plane hold any non-zero byte" (src/dequantizer.cpp:118-128)
// for tensors that already live on the GPU.
// ---------------------------------------------------------------------------
__global__ void tq_any_nonzero_kernel(const uint8_t* __restrict__ data, size_t n, int* flag) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
    const size_t n16 = n / 16;
    const uint4* p = reinterpret_cast<const uint4*>(data);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
        const uint4 t = p[i];
        acc |= t.x | t.y | t.z | t.w;
    }
    for (size_t i = n16 * 16 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) acc |= data[i];
    if (acc) atomicOr(flag, 1);
}

// Interleave the two nibble planes into one byte per weight (residual high, primary low),
// the layout the shared-rotation GEMV streams.  One thread per packed byte pair.
__global__ void tq_combine_planes_kernel(const uint8_t* __restrict__ primary, const uint8_t* __restrict__ residual,
                                         uint16_t* __restrict__ combined, size_t plane_bytes) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < plane_bytes; i += stride) {
        const uint32_t pb = primary[i], rb = residual[i];
        const uint32_t even = (pb & 0x0fu) | ((rb & 0x0fu) << 4);   // src/dequantizer.cpp:163
        const uint32_t odd = (pb >> 4) | (rb & 0xf0u);              // src/dequantizer.cpp:168
        combined[i] = (uint16_t)(even | (odd << 8));
    }
}

hipError_t launch_combine_planes(const uint8_t* primary, const uint8_t* residual, uint8_t* combined,
                                 size_t plane_bytes, hipStream_t stream) {
    hipLaunchKernelGGL(tq_combine_planes_kernel, dim3(2048), dim3(256), 0, stream, primary, residual,
                       reinterpret_cast<uint16_t*>(combined), plane_bytes);
    return hipGetLastError();
}

// 5-bit primary (one index per byte) + residual nibbles of at most 3 significant bits -> one byte
// per weight: min(r, n_residual - 1) << 5 | min(p, n_primary - 1)  (clamps of src/dequantizer.cpp:94,103).
__global__ void tq_combine_planes5_kernel(const uint8_t* __restrict__ primary, const uint8_t* __restrict__ residual,
                                          uint16_t* __restrict__ combined, size_t residual_bytes, uint32_t pmax,
                                          uint32_t rmax) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < residual_bytes; i += stride) {
        const uint32_t rb = residual[i];
        const uint32_t p0 = min((uint32_t)primary[2 * i], pmax), p1 = min((uint32_t)primary[2 * i + 1], pmax);
        const uint32_t r0 = min(rb & 0x0fu, rmax), r1 = min(rb >> 4, rmax);
        combined[i] = (uint16_t)((r0 << 5) | p0 | (((r1 << 5) | p1) << 8));
    }
}

hipError_t launch_combine_planes5(const uint8_t* primary, const uint8_t* residual, uint8_t* combined,
                                  size_t residual_bytes, int n_primary, int n_residual, hipStream_t stream) {
    hipLaunchKernelGGL(tq_combine_planes5_kernel, dim3(2048), dim3(256), 0, stream, primary, residual,
                       reinterpret_cast<uint16_t*>(combined), residual_bytes, (uint32_t)(n_primary - 1),
                       (uint32_t)(n_residual - 1));
    return hipGetLastError();
}

__global__ void tq_silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up, void* __restrict__ out,
                                   int out_dtype, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float g = gate[i];
        store_scalar(out, out_dtype, i, g / (1.0f + expf(-g)) * up[i]);
    }
}

hipError_t launch_silu_mul(const float* gate, const float* up, void* out, int out_dtype, size_t n, hipStream_t stream) {
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(tq_silu_mul_kernel, dim3((unsigned)(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks))), dim3(256), 0,
                       stream, gate, up, out, out_dtype, n);
    return hipGetLastError();
}

// out[i] = a[i] + b[i] over n fp32 values, written as out_dtype; out may be a itself.
__global__ void tq_add_kernel(const float* a, const float* __restrict__ b, void* out, int out_dtype, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        store_scalar(out, out_dtype, i, a[i] + b[i]);
}

hipError_t launch_add(const float* a, const float* b, void* out, int out_dtype, size_t n, hipStream_t stream) {
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(tq_add_kernel, dim3((unsigned)(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks))), dim3(256), 0,
                       stream, a, b, out, out_dtype, n);
    return hipGetLastError();
}

hipError_t launch_any_nonzero(const uint8_t* data, size_t n, int* flag_dev, hipStream_t stream) {
    hipLaunchKernelGGL(tq_any_nonzero_kernel, dim3(1024), dim3(256), 0, stream, data, n, flag_dev);
    return hipGetLastError();
}

}  // namespace tq
