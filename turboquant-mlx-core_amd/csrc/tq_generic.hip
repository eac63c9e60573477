// Fused TQ8 forward for every shape and mode the reference accepts and the tuned kernels do not take:
// rows wider than 32768 columns, widths that are a multiple of the block size but not of 32 (blocks of
// 1 to 16 columns), 5-bit primaries with their own residual rotation or a 4-bit residual
// (metal/turboquant_dequant_mm.metal:240-248, 277-292; src/dequantizer.cpp:625-626, 657).  The only
// rule the reference has is in_features % block_size == 0 (src/rotation.cpp:374, 396).
//
// Same identity as the tuned kernels: the activation row is rotated once per seed,
//   y[r] = norm[r] / sqrt(in * bs) * ( sum_i cP[p(r,i)] x~p[i]  +  sum_i cR[q(r,i)] x~r[i] ),
// here by a kernel of its own into an fp32 scratch row, and the product is a plain wave-per-row dot
// product with the centroid tables in LDS.  No per-shape tuning: correctness for the whole domain.
// Also here: the materialising dequantiser and the stand-alone rotation for blocks narrower than 32
// columns (one thread per block; the wave-per-slab kernels of tq_dequant.hip need in % 32 == 0).
#include "tq_device.h"

namespace tq {

namespace {

__device__ __forceinline__ float widen(const void* x, int dtype, size_t i) {
    if (dtype == kF32) return static_cast<const float*>(x)[i];
    const uint16_t h = static_cast<const uint16_t*>(x)[i];
    return dtype == kBF16 ? bf16_bits_to_float(h) : (float)__builtin_bit_cast(_Float16, h);
}

// Unnormalised Walsh-Hadamard butterfly over the first bs of 16 values held by one thread, stage order
// and (a + b, a - b) convention of src/rotation.cpp:14-25.
__device__ __forceinline__ void fwht16(float (&v)[16], uint32_t bs) {
#pragma unroll
    for (int h = 1; h < 16; h <<= 1) {
        if ((uint32_t)h < bs) {
#pragma unroll
            for (int i = 0; i < 16; i += 2 * h)
#pragma unroll
                for (int j = i; j < i + h; ++j) { const float a = v[j], b = v[j + h]; v[j] = a + b; v[j + h] = a - b; }
        }
    }
}

}  // namespace

// x~ = H (s (.) x) of one activation row for one or two seeds, fp32, natural column order,
// out[p * cols + c].  cols % 32 == 0, blocks of 2 to 2048 columns: one wave per 2048-column slab.
__global__ __launch_bounds__(256) void tq_rotate_slab_kernel(const void* __restrict__ x, int x_dtype,
                                                             float* __restrict__ out, int cols, int chunks,
                                                             uint32_t seed0, uint32_t seed1, uint32_t bs) {
    const int lane = threadIdx.x & (kWave - 1);
    const int slab = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6);
    const int chunk = slab * kWave + lane;
    if (slab * kWave >= chunks) return;                      // whole wave leaves together
    const bool active = chunk < chunks;
    const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);
    const uint32_t seed = blockIdx.y ? seed1 : seed0;
    float v[kChunk];
    if (active) {
        load_chunk(x, x_dtype, (size_t)chunk * kChunk, v);
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= sign_of(seed, (col0 + k) & (bs - 1));
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    fwht_lane32(v, bs, lane);
    if (active) {
        float4* dst = reinterpret_cast<float4*>(out + (size_t)blockIdx.y * cols + (size_t)chunk * kChunk);
#pragma unroll
        for (int i = 0; i < 8; ++i) dst[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    }
}

// The same for blocks of 1 to 16 columns and any width that is a multiple of the block: one thread per block.
__global__ __launch_bounds__(256) void tq_rotate_small_kernel(const void* __restrict__ x, int x_dtype,
                                                              float* __restrict__ out, int cols, int blocks,
                                                              uint32_t seed0, uint32_t seed1, uint32_t bs) {
    const int blk = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (blk >= blocks) return;
    const uint32_t seed = blockIdx.y ? seed1 : seed0;
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k)
        v[k] = (uint32_t)k < bs ? widen(x, x_dtype, (size_t)blk * bs + k) * sign_of(seed, (uint32_t)k) : 0.0f;
    fwht16(v, bs);
    float* dst = out + (size_t)blockIdx.y * cols + (size_t)blk * bs;
#pragma unroll
    for (int k = 0; k < 16; ++k)
        if ((uint32_t)k < bs) dst[k] = v[k];
}

struct GenericArgs {
    LayerView L;
    const float* xrot;       // [planes][in] rotated activations of one batch row
    void* y;                 // this batch row's outputs
    int y_dtype;
    float out_scale;         // inv_scale * inv_sqrt_bs
    const float* gate;       // optional fp32 [out] of this batch row
};

// One wave per row, lanes stride over the row two columns (one packed byte) at a time.
// Decode tables as build_tables (tq_linear_c.cpp) lays them out; index clamps of
// src/dequantizer.cpp:94,103,229 are in the tables (4-bit indices cannot exceed them) or applied
// here (a 5-bit plane holds whole bytes).
template <int MODE>
__global__ __launch_bounds__(256) void tq_gemv_generic_kernel(GenericArgs a) {
    __shared__ float tab[256];
    for (int i = threadIdx.x; i < 256; i += blockDim.x) tab[i] = a.L.tables[i];
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const int in = a.L.in_features, out = a.L.out_features;
    const int pairs = in >> 1;                               // in is even: it is a multiple of a block of >= 2
                                                             // columns, or packs two columns per byte
    constexpr bool combined = (MODE == kSharedLut);          // one byte per weight: residual index high, primary low
    constexpr bool five = (MODE >= kShared5);
    constexpr bool has_res = (MODE != kPrimaryOnly && MODE != kPrimaryOnly5);
    constexpr bool dual = (MODE == kDual || MODE == kDual5);
    constexpr int roff = five ? 32 : 16;
    const float* xp = a.xrot;
    const float* xr = a.xrot + in;
    const bool by_eight = (in & 7) == 0;                     // uniform: widths that allow 8-byte loads of a row
    for (int row = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6); row < out; row += (int)gridDim.x * 4) {
        float sp = 0.0f, sr = 0.0f;
        // Eight consecutive columns per lane and step: one 8- or 4-byte load per plane, two 16-byte loads per
        // rotated activation vector (the byte-wise loop below is left for widths that are not a multiple of 8).
        for (int c = 8 * lane; by_eight && c < in; c += 8 * kWave) {
            uint32_t p[8], r[8];
            if constexpr (combined || five) {
                const uint2 w = *reinterpret_cast<const uint2*>((combined ? a.L.packed_combined : a.L.packed_primary) + (size_t)row * in + c);
#pragma unroll
                for (int j = 0; j < 4; ++j) { p[j] = (w.x >> (8 * j)) & 255u; p[4 + j] = (w.y >> (8 * j)) & 255u; }
                if constexpr (five) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) p[j] = p[j] > 31u ? 31u : p[j];
                }
            } else {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(a.L.packed_primary + (size_t)row * pairs + (c >> 1));
#pragma unroll
                for (int j = 0; j < 4; ++j) { p[2 * j] = (w >> (8 * j)) & 15u; p[2 * j + 1] = (w >> (8 * j + 4)) & 15u; }
            }
            if constexpr (has_res && !combined) {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(a.L.packed_residual + (size_t)row * pairs + (c >> 1));
#pragma unroll
                for (int j = 0; j < 4; ++j) { r[2 * j] = (w >> (8 * j)) & 15u; r[2 * j + 1] = (w >> (8 * j + 4)) & 15u; }
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) r[j] = 0;
            }
            const float4 xa = *reinterpret_cast<const float4*>(xp + c), xb = *reinterpret_cast<const float4*>(xp + c + 4);
            const float x[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
            if constexpr (combined || !has_res) {
#pragma unroll
                for (int j = 0; j < 8; ++j) sp = __builtin_fmaf(tab[p[j]], x[j], sp);
            } else if constexpr (dual) {
                const float4 ya = *reinterpret_cast<const float4*>(xr + c), yb = *reinterpret_cast<const float4*>(xr + c + 4);
                const float y[8] = {ya.x, ya.y, ya.z, ya.w, yb.x, yb.y, yb.z, yb.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    sp = __builtin_fmaf(tab[p[j]], x[j], sp);
                    sr = __builtin_fmaf(tab[roff + r[j]], y[j], sr);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) sp = __builtin_fmaf(tab[p[j]] + tab[roff + r[j]], x[j], sp);
            }
        }
        for (int u = lane; !by_eight && u < pairs; u += kWave) {
            const int c = 2 * u;
            uint32_t p0, p1, r0 = 0, r1 = 0;
            if constexpr (combined) {
                p0 = a.L.packed_combined[(size_t)row * in + c];
                p1 = a.L.packed_combined[(size_t)row * in + c + 1];
            } else {
                if constexpr (five) {
                    p0 = a.L.packed_primary[(size_t)row * in + c];
                    p1 = a.L.packed_primary[(size_t)row * in + c + 1];
                    p0 = p0 > 31u ? 31u : p0;
                    p1 = p1 > 31u ? 31u : p1;
                } else {
                    const uint32_t b = a.L.packed_primary[(size_t)row * pairs + u];
                    p0 = b & 15u; p1 = b >> 4;               // lo nibble = even column (src/dequantizer.cpp:46-47)
                }
                if constexpr (has_res) {
                    const uint32_t b = a.L.packed_residual[(size_t)row * pairs + u];
                    r0 = b & 15u; r1 = b >> 4;
                }
            }
            const float x0 = xp[c], x1 = xp[c + 1];
            if constexpr (combined || !has_res) {
                sp = __builtin_fmaf(tab[p0], x0, sp);
                sp = __builtin_fmaf(tab[p1], x1, sp);
            } else if constexpr (dual) {
                sp = __builtin_fmaf(tab[p0], x0, sp);
                sp = __builtin_fmaf(tab[p1], x1, sp);
                sr = __builtin_fmaf(tab[roff + r0], xr[c], sr);
                sr = __builtin_fmaf(tab[roff + r1], xr[c + 1], sr);
            } else {                                         // shared rotation, 5-bit primary: primary + residual centroid
                sp = __builtin_fmaf(tab[p0] + tab[roff + r0], x0, sp);      // (src/dequantizer.cpp:186-212)
                sp = __builtin_fmaf(tab[p1] + tab[roff + r1], x1, sp);
            }
        }
        float t = sp + sr;
        t += lane_xor<1>(t); t += lane_xor<2>(t); t += lane_xor<4>(t);
        t += lane_xor<8>(t); t += lane_xor<16>(t); t += lane_xor<32>(t);
        if (lane == 0) {
            t *= a.out_scale * a.L.norms[row];
            if (a.gate) { const float g = a.gate[row]; t = g / (1.0f + expf(-g)) * t; }
            store_scalar(a.y, a.y_dtype, (size_t)row, t);
        }
    }
}

// Every layer the layout allows: power-of-two blocks of 1 to 2048 columns that divide the width
// (src/rotation.cpp:374, 396), an even width (two columns share a packed byte), and the fp32 scratch
// row for the rotated activations that every layer handle owns.
bool generic_supported(const LayerView& L) {
    const uint32_t bs = L.block_size;
    if (bs < 1 || bs > 2048 || (bs & (bs - 1))) return false;
    if (L.in_features <= 0 || L.in_features % (int)bs != 0 || (L.in_features & 1)) return false;
    return L.xrot_work != nullptr;
}

// x~ of one activation row into L.xrot_work (both rotations where the mode has two).
static hipError_t rotate_row_generic(const LayerView& L, const void* x, int x_dtype, hipStream_t stream) {
    const bool two = (L.mode == kDual || L.mode == kDual5);
    const int in = L.in_features;
    if (in % kChunk == 0 && L.block_size >= 2) {
        const int chunks = in / kChunk;
        const int slabs = (chunks + kWave - 1) / kWave;
        hipLaunchKernelGGL(tq_rotate_slab_kernel, dim3((slabs + 3) / 4, two ? 2 : 1), dim3(256), 0, stream,
                           x, x_dtype, L.xrot_work, in, chunks, L.seed_primary, L.seed_residual, L.block_size);
    } else {
        const int blocks = in / (int)L.block_size;
        hipLaunchKernelGGL(tq_rotate_small_kernel, dim3((blocks + 255) / 256, two ? 2 : 1), dim3(256), 0, stream,
                           x, x_dtype, L.xrot_work, in, blocks, L.seed_primary, L.seed_residual, L.block_size);
    }
    return hipGetLastError();
}

hipError_t launch_gemv_generic(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                               int num_cus, hipStream_t stream, const float* gate) {
    if (!generic_supported(L)) return hipErrorInvalidValue;
    const size_t xe = (x_dtype == kF32) ? 4 : 2, ye = (y_dtype == kF32) ? 4 : 2;
    int grid = (L.out_features + 3) / 4;
    if (grid > num_cus * 8) grid = num_cus * 8;
    for (int b = 0; b < batch; ++b) {
        hipError_t e = rotate_row_generic(L, static_cast<const char*>(x) + (size_t)b * L.in_features * xe, x_dtype, stream);
        if (e != hipSuccess) return e;
        GenericArgs a{};
        a.L = L;
        a.xrot = L.xrot_work;
        a.y = static_cast<char*>(y) + (size_t)b * L.out_features * ye;
        a.y_dtype = y_dtype;
        a.out_scale = L.inv_scale * L.inv_sqrt_bs;
        a.gate = gate ? gate + (size_t)b * L.out_features : nullptr;
        switch (L.mode) {
            case kPrimaryOnly:  hipLaunchKernelGGL(tq_gemv_generic_kernel<kPrimaryOnly>, dim3(grid), dim3(256), 0, stream, a); break;
            case kSharedLut:    hipLaunchKernelGGL(tq_gemv_generic_kernel<kSharedLut>, dim3(grid), dim3(256), 0, stream, a); break;
            case kDual:         hipLaunchKernelGGL(tq_gemv_generic_kernel<kDual>, dim3(grid), dim3(256), 0, stream, a); break;
            case kShared5:      hipLaunchKernelGGL(tq_gemv_generic_kernel<kShared5>, dim3(grid), dim3(256), 0, stream, a); break;
            case kPrimaryOnly5: hipLaunchKernelGGL(tq_gemv_generic_kernel<kPrimaryOnly5>, dim3(grid), dim3(256), 0, stream, a); break;
            case kDual5:        hipLaunchKernelGGL(tq_gemv_generic_kernel<kDual5>, dim3(grid), dim3(256), 0, stream, a); break;
            default: return hipErrorInvalidValue;
        }
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// ---------------------------------------------------------------------------
// Blocks of 1 to 16 columns: materialising dequantiser and stand-alone rotation, one thread per
// (row, block), the operations of src/dequantizer.cpp:52-256 and src/rotation.cpp:291-350 in their
// order (single fp32 operations, no contraction): bit-identical to the CPU path.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void tq_dequant_small_kernel(LayerView L, void* __restrict__ Wout, int w_dtype,
                                                               int blocks_per_row) {
    __shared__ float tab[256];
    for (int i = threadIdx.x; i < 256; i += blockDim.x) tab[i] = L.tables[i];
    __syncthreads();
    const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
    const int row = (int)(id / blocks_per_row);
    const int blk = (int)(id % blocks_per_row);
    if (row >= L.out_features) return;
    const int in = L.in_features;
    const uint32_t bs = L.block_size;
    const bool five = (L.mode >= kShared5);
    const bool has_res = (L.mode != kPrimaryOnly && L.mode != kPrimaryOnly5);
    const bool shared = (L.mode == kSharedLut || L.mode == kShared5);
    const int roff = five ? 32 : 16;
    const float nrm = L.norms[row];
    float v[16], u[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        v[k] = 0.0f; u[k] = 0.0f;
        if ((uint32_t)k < bs) {
            const size_t col = (size_t)blk * bs + k;
            uint32_t p, r = 0;
            if (L.packed_combined) {                        // one byte per weight (4-bit: r << 4 | p, 5-bit: r << 5 | p)
                const uint32_t c = L.packed_combined[(size_t)row * in + col];
                p = five ? (c & 31u) : (c & 15u);
                r = five ? (c >> 5) : (c >> 4);
            } else {
                if (five) { p = L.packed_primary[(size_t)row * in + col]; p = p > 31u ? 31u : p; }
                else { const uint32_t b = L.packed_primary[(size_t)row * (in >> 1) + (col >> 1)]; p = (col & 1) ? (b >> 4) : (b & 15u); }
                if (has_res) { const uint32_t b = L.packed_residual[(size_t)row * (in >> 1) + (col >> 1)]; r = (col & 1) ? (b >> 4) : (b & 15u); }
            }
            if (L.mode == kSharedLut) v[k] = tab[(r << 4) | p] * L.inv_scale;          // path A
            else {
                float c = tab[p];
                if (shared) c = c + tab[roff + r];                                       // path B
                v[k] = c * L.inv_scale;
                if (has_res && !shared) u[k] = tab[roff + r] * L.inv_scale;              // path C, second plane
            }
        }
    }
    fwht16(v, bs);
    if (has_res && !shared) fwht16(u, bs);
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        if ((uint32_t)k < bs) {
            float w = v[k] * (L.inv_sqrt_bs * sign_of(L.seed_primary, (uint32_t)k));
            if (has_res && !shared) {
                const float w2 = u[k] * (L.inv_sqrt_bs * sign_of(L.seed_residual, (uint32_t)k));
                w = w + w2;
            }
            w = w * nrm;
            const size_t e = (size_t)row * in + (size_t)blk * bs + k;
            store_scalar(Wout, w_dtype, e, w);
        }
    }
}

hipError_t launch_dequant_small(const LayerView& L, void* w, int w_dtype, hipStream_t stream) {
    if (L.block_size > 16) return hipErrorInvalidValue;
    const int bpr = L.in_features / (int)L.block_size;
    const long long threads = (long long)L.out_features * bpr;
    const long long grid = (threads + 255) / 256;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tq_dequant_small_kernel, dim3((unsigned)grid), dim3(256), 0, stream, L, w, w_dtype, bpr);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void tq_wht_small_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                           long long blocks, uint32_t seed, uint32_t bs,
                                                           float inv_sqrt_bs, int inverse) {
    const long long blk = (long long)blockIdx.x * 256 + threadIdx.x;
    if (blk >= blocks) return;
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        v[k] = (uint32_t)k < bs ? in[blk * bs + k] : 0.0f;
        if (!inverse && (uint32_t)k < bs) v[k] *= sign_of(seed, (uint32_t)k);
    }
    fwht16(v, bs);
#pragma unroll
    for (int k = 0; k < 16; ++k)
        if ((uint32_t)k < bs) out[blk * bs + k] = inverse ? v[k] * (inv_sqrt_bs * sign_of(seed, (uint32_t)k)) : v[k] * inv_sqrt_bs;
}

hipError_t launch_wht_small(const float* in, float* out, int rows, int cols, uint32_t seed, uint32_t block_size,
                            float inv_sqrt_bs, int inverse, hipStream_t stream) {
    if (block_size > 16) return hipErrorInvalidValue;
    const long long blocks = (long long)rows * (cols / (int)block_size);
    const long long grid = (blocks + 255) / 256;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tq_wht_small_kernel, dim3((unsigned)grid), dim3(256), 0, stream, in, out, blocks, seed, block_size,
                       inv_sqrt_bs, inverse);
    return hipGetLastError();
}

}  // namespace tq
