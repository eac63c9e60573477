// Fused TQ8 dequant + GEMV for gfx950 (batch 1..4 per launch).
//
// Replaces the reference's per-row-FWHT kernel (metal/turboquant_dequant_mm.metal:152-313)
// and its host side (src/dequantizer.cpp:606-721).  Instead of running an inverse
// Walsh-Hadamard transform on every weight block, the activation is rotated once:
//
//   y[r] = norm[r] / sqrt(in*bs) * sum_i L[r,i] * xt[i],   xt_blk = H (s (.) x_blk)
//
// where L is the centroid (sum) selected by the packed nibbles, H the unnormalised
// Hadamard matrix of the block and s the seed-derived sign vector.
//
// Work decomposition: a lane owns 32 consecutive columns (16 packed bytes = one
// 128-bit load from each index plane), a wave owns a 2048-column slab, and the
// rotated activations of the slab stay in registers for the whole kernel.  A
// workgroup is W slabs (covering one row) times S independent row streams; every
// stream walks a contiguous range of row groups.  Centroid tables sit in LDS with
// one private 4-byte column per lane (entry pitch 256 B), so lookups never conflict
// and the LDS byte address is assembled with a single v_perm_b32.
#include "tq_device.h"

namespace tq {

struct GemvArgs {
    LayerView L;
    const void* x;
    void* y;
    int x_dtype, y_dtype;
    int chunks;      // in / 32
    int W, S;        // slabs per row, row streams per workgroup
    int groups;      // ceil(out / R)
    int iters;       // uniform trip count: ceil(groups / (gridDim.x * S))
    float out_scale; // inv_scale * inv_sqrt_bs
};

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over the 64 lanes of a wave; the result is uniform.
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);   // row_half_mirror
    v = dpp_add<0x140>(v);   // row_mirror
    int iv = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    return (r0 + r1) + (r2 + r3);
}

// LDS byte address of table entry `byte j of idx`, private column of this lane:
// (entry << 8) | (lane << 2), built by one byte permute.
template <int J>
__device__ __forceinline__ uint32_t entry_addr(uint32_t idx_bytes, uint32_t laneoff) {
    return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0000u | ((4u + J) << 8));
}

__device__ __forceinline__ float lds_f32(const char* lds, uint32_t byte_addr) {
    return *reinterpret_cast<const float*>(lds + byte_addr);
}

// One row, shared-rotation 4-bit mode: a single 256-entry table indexed by
// (residual_nibble << 4) | primary_nibble  (reference src/dequantizer.cpp:144-169).
template <int NB>
__device__ __forceinline__ void row_lut256(const uint4& P, const uint4& Q, const float (&xt)[NB][kChunk],
                                           float (&acc)[NB], const char* lds, uint32_t laneoff) {
    const uint32_t pw[4] = {P.x, P.y, P.z, P.w};
    const uint32_t rw[4] = {Q.x, Q.y, Q.z, Q.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t ce = ((rw[d] << 4) & 0xF0F0F0F0u) | (pw[d] & 0x0F0F0F0Fu);          // even columns
        const uint32_t co = (rw[d] & 0xF0F0F0F0u) | ((pw[d] >> 4) & 0x0F0F0F0Fu);         // odd columns
        float le[4], lo[4];
        le[0] = lds_f32(lds, entry_addr<0>(ce, laneoff)); lo[0] = lds_f32(lds, entry_addr<0>(co, laneoff));
        le[1] = lds_f32(lds, entry_addr<1>(ce, laneoff)); lo[1] = lds_f32(lds, entry_addr<1>(co, laneoff));
        le[2] = lds_f32(lds, entry_addr<2>(ce, laneoff)); lo[2] = lds_f32(lds, entry_addr<2>(co, laneoff));
        le[3] = lds_f32(lds, entry_addr<3>(ce, laneoff)); lo[3] = lds_f32(lds, entry_addr<3>(co, laneoff));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                acc[b] = __builtin_fmaf(le[j], xt[b][8 * d + 2 * j], acc[b]);
                acc[b] = __builtin_fmaf(lo[j], xt[b][8 * d + 2 * j + 1], acc[b]);
            }
        }
    }
}

// One row, one 16-entry table (primary or residual plane) at LDS offset TABLE_OFF.
template <int NB, int TABLE_OFF>
__device__ __forceinline__ void row_tab16(const uint4& P, const float (&xt)[NB][kChunk],
                                          float (&acc)[NB], const char* lds, uint32_t laneoff) {
    const uint32_t pw[4] = {P.x, P.y, P.z, P.w};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t ce = pw[d] & 0x0F0F0F0Fu;
        const uint32_t co = (pw[d] >> 4) & 0x0F0F0F0Fu;
        float le[4], lo[4];
        le[0] = lds_f32(lds + TABLE_OFF, entry_addr<0>(ce, laneoff)); lo[0] = lds_f32(lds + TABLE_OFF, entry_addr<0>(co, laneoff));
        le[1] = lds_f32(lds + TABLE_OFF, entry_addr<1>(ce, laneoff)); lo[1] = lds_f32(lds + TABLE_OFF, entry_addr<1>(co, laneoff));
        le[2] = lds_f32(lds + TABLE_OFF, entry_addr<2>(ce, laneoff)); lo[2] = lds_f32(lds + TABLE_OFF, entry_addr<2>(co, laneoff));
        le[3] = lds_f32(lds + TABLE_OFF, entry_addr<3>(ce, laneoff)); lo[3] = lds_f32(lds + TABLE_OFF, entry_addr<3>(co, laneoff));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                acc[b] = __builtin_fmaf(le[j], xt[b][8 * d + 2 * j], acc[b]);
                acc[b] = __builtin_fmaf(lo[j], xt[b][8 * d + 2 * j + 1], acc[b]);
            }
        }
    }
}

constexpr int kLut256Bytes = 256 * 256;   // 256 entries x 64 lanes x 4 B
constexpr int kTab16Bytes = 16 * 256;

template <int MODE>
__host__ __device__ constexpr int table_bytes() {
    return MODE == kSharedLut ? kLut256Bytes : (MODE == kDual ? 2 * kTab16Bytes : kTab16Bytes);
}

// Rotated activations of this lane's chunk for one batch row: H (s (.) x).
__device__ __forceinline__ void rotate_chunk(const void* x, int x_dtype, size_t row_off, int chunk,
                                             bool active, uint32_t seed, uint32_t bs, int lane,
                                             float (&v)[kChunk]) {
    if (active) {
        load_chunk(x, x_dtype, row_off + (size_t)chunk * kChunk, v);
        const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= sign_of(seed, (col0 + k) & (bs - 1));
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    fwht_lane32(v, bs, lane);
}

template <int MODE, int NB, int R, int MAXT>
__global__ __launch_bounds__(MAXT) void tq_gemv_kernel(GemvArgs a) {
    extern __shared__ __align__(16) char smem[];
    constexpr int kTable = table_bytes<MODE>();
    float* partial = reinterpret_cast<float*>(smem + kTable);   // [2][S][W][R*NB]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int slab = wave % a.W;
    const int stream = wave / a.W;
    const int chunk = slab * kWave + lane;
    const bool active = chunk < a.chunks;
    const uint32_t laneoff = (uint32_t)lane << 2;
    const int out = a.L.out_features;
    const size_t row_bytes = (size_t)a.L.in_features >> 1;
    const bool use_res = (MODE != kPrimaryOnly);

    const long long gs = (long long)blockIdx.x * a.S + stream;
    const long long ts = (long long)gridDim.x * a.S;
    const int g_begin = (int)(gs * a.groups / ts);
    const int g_end = (int)((gs + 1) * a.groups / ts);

    const uint8_t* pp = a.L.packed_primary + (size_t)chunk * 16;
    const uint8_t* pr = a.L.packed_residual + (size_t)chunk * 16;

    uint4 P[2][R], Q[2][R];
    auto fetch = [&](int buf, int g) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int r = g * R + i;
            if (active && g < g_end && r < out) {
                P[buf][i] = *reinterpret_cast<const uint4*>(pp + (size_t)r * row_bytes);
                if (use_res) Q[buf][i] = *reinterpret_cast<const uint4*>(pr + (size_t)r * row_bytes);
            } else {
                P[buf][i] = make_uint4(0, 0, 0, 0);
                if (use_res) Q[buf][i] = make_uint4(0, 0, 0, 0);
            }
        }
    };

    // First weight fetch goes out before the prologue so its latency overlaps it.
    fetch(0, g_begin);

    // Decode tables -> LDS, one private column per lane.
    {
        const int entries = (MODE == kSharedLut) ? 256 : (MODE == kDual ? 32 : 16);
        float4* dst = reinterpret_cast<float4*>(smem);
        for (int i = tid; i < entries * 16; i += blockDim.x) {
            const float v = a.L.tables[i >> 4];
            dst[i] = make_float4(v, v, v, v);
        }
    }

    // Rotated activations, kept in registers for the whole kernel.
    float xt[NB][kChunk];
    float xr[NB][kChunk];   // second rotation, dual mode only
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                     a.L.seed_primary, a.L.block_size, lane, xt[b]);
        if constexpr (MODE == kDual)
            rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                         a.L.seed_residual, a.L.block_size, lane, xr[b]);
    }
    __syncthreads();

    auto consume = [&](int buf, int g, int it) {
        float acc[R][NB];
#pragma unroll
        for (int i = 0; i < R; ++i) {
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[i][b] = 0.0f;
            if constexpr (MODE == kSharedLut) {
                row_lut256<NB>(P[buf][i], Q[buf][i], xt, acc[i], smem, laneoff);
            } else {
                row_tab16<NB, 0>(P[buf][i], xt, acc[i], smem, laneoff);
                if constexpr (MODE == kDual) row_tab16<NB, kTab16Bytes>(Q[buf][i], xr, acc[i], smem, laneoff);
            }
        }
        float sums[R][NB];
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int b = 0; b < NB; ++b) sums[i][b] = wave_sum(acc[i][b]);

        if (a.W == 1) {
            if (lane == 0 && g < g_end) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int r = g * R + i;
                    if (r < out) {
                        const float s = a.out_scale * a.L.norms[r];
#pragma unroll
                        for (int b = 0; b < NB; ++b)
                            store_scalar(a.y, a.y_dtype, (size_t)b * out + r, sums[i][b] * s);
                    }
                }
            }
        } else {
            float* slot = partial + (size_t)(it & 1) * a.S * a.W * (R * NB) + (size_t)stream * a.W * (R * NB);
            if (lane == 0) {
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int b = 0; b < NB; ++b) slot[slab * (R * NB) + i * NB + b] = sums[i][b];
            }
            __syncthreads();
            if (slab == 0 && lane < R * NB && g < g_end) {
                const int i = lane / NB, b = lane % NB;
                const int r = g * R + i;
                if (r < out) {
                    float t = 0.0f;
                    for (int w = 0; w < a.W; ++w) t += slot[w * (R * NB) + lane];
                    store_scalar(a.y, a.y_dtype, (size_t)b * out + r, t * (a.out_scale * a.L.norms[r]));
                }
            }
        }
    };

    // Double-buffered main loop (unrolled by two so the buffers are static).
    for (int it = 0; it < a.iters; it += 2) {
        const int g0 = g_begin + it;
        fetch(1, g0 + 1);
        consume(0, g0, it);
        if (it + 1 < a.iters) {
            fetch(0, g0 + 2);
            consume(1, g0 + 1, it + 1);
        }
    }
}

template <int MODE, int NB, int R, int MAXT>
static hipError_t launch_one(const GemvArgs& a, int grid, int threads, size_t lds, hipStream_t stream) {
    auto kern = tq_gemv_kernel<MODE, NB, R, MAXT>;
    static thread_local bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 4096);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, stream, a);
    return hipGetLastError();
}

template <int MODE, int NB, int MAXT>
static hipError_t launch_nb(GemvArgs a, int num_cus, hipStream_t stream) {
    const int out = a.L.out_features;
    a.chunks = a.L.in_features / kChunk;
    a.W = (a.chunks + kWave - 1) / kWave;
    if (a.W * kWave > MAXT) return hipErrorInvalidValue;
    a.S = (a.W >= 8) ? 1 : (8 / a.W);
    const int threads = a.W * a.S * kWave;
    const int max_grid = num_cus * 2;

    // Largest row-group size that still gives every resident stream work.
    int R = 4;
    while (R > 1 && (long long)((out + R - 1) / R) < (long long)max_grid * a.S) R >>= 1;
    a.groups = (out + R - 1) / R;
    int grid = (a.groups + a.S - 1) / a.S;
    if (grid > max_grid) grid = max_grid;
    if (grid < 1) grid = 1;
    const long long ts = (long long)grid * a.S;
    a.iters = (int)((a.groups + ts - 1) / ts);
    const size_t lds = (size_t)table_bytes<MODE>() + (size_t)2 * a.S * a.W * R * NB * sizeof(float);

    switch (R) {
        case 4: return launch_one<MODE, NB, 4, MAXT>(a, grid, threads, lds, stream);
        case 2: return launch_one<MODE, NB, 2, MAXT>(a, grid, threads, lds, stream);
        default: return launch_one<MODE, NB, 1, MAXT>(a, grid, threads, lds, stream);
    }
}

// Batch rows are served 4, 2 or 1 per launch: the rotated activations of every
// batch row live in registers, which bounds how many fit next to the weight
// buffers (workgroups of up to 512 threads get 256 VGPRs per lane, larger ones 128).
template <int MODE>
static hipError_t launch_mode(const GemvArgs& base, int batch, int num_cus, hipStream_t stream) {
    const size_t xe = (base.x_dtype == kF32) ? 4 : 2;
    const size_t ye = (base.y_dtype == kF32) ? 4 : 2;
    const int in = base.L.in_features, out = base.L.out_features;
    const int W = (in / kChunk + kWave - 1) / kWave;
    int done = 0;
    while (done < batch) {
        GemvArgs a = base;
        a.x = static_cast<const char*>(base.x) + (size_t)done * in * xe;
        a.y = static_cast<char*>(base.y) + (size_t)done * out * ye;
        const int left = batch - done;
        hipError_t e;
        int step = 1;
        if constexpr (MODE == kDual) {
            e = (W <= 8) ? launch_nb<MODE, 1, 512>(a, num_cus, stream) : launch_nb<MODE, 1, 1024>(a, num_cus, stream);
        } else {
            if (left >= 4 && W <= 8)      { step = 4; e = launch_nb<MODE, 4, 512>(a, num_cus, stream); }
            else if (left >= 2 && W <= 8) { step = 2; e = launch_nb<MODE, 2, 512>(a, num_cus, stream); }
            else                          { step = 1; e = launch_nb<MODE, 1, 1024>(a, num_cus, stream); }
        }
        if (e != hipSuccess) return e;
        done += step;
    }
    return hipSuccess;
}

hipError_t launch_gemv(const LayerView& L, const void* x, int x_dtype, int batch,
                       void* y, int y_dtype, int num_cus, hipStream_t stream) {
    GemvArgs a{};
    a.L = L;
    a.x = x; a.y = y; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
    a.out_scale = L.inv_scale * L.inv_sqrt_bs;
    switch (L.mode) {
        case kSharedLut:   return launch_mode<kSharedLut>(a, batch, num_cus, stream);
        case kDual:        return launch_mode<kDual>(a, batch, num_cus, stream);
        case kPrimaryOnly: return launch_mode<kPrimaryOnly>(a, batch, num_cus, stream);
        default:           return hipErrorInvalidValue;
    }
}

}  // namespace tq
