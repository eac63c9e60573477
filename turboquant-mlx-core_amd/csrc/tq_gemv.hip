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
    int share_x;     // rotate the activations once per workgroup and pass them through LDS
    float out_scale; // inv_scale * inv_sqrt_bs
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 128-bit streaming load (weights are read exactly once).
__device__ __forceinline__ uint4 load_stream16(const uint8_t* p) {
    const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Value held by lane (lane ^ MASK).
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
    if constexpr (MASK == 1) return dpp_mov<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (MASK == 2) return dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (MASK == 8) return dpp_mov<0x128>(v);  // row_ror:8
    else return __shfl_xor(v, MASK, kWave);
}

// Transposed wave reduction of N per-lane partial sums (N a power of two <= 16):
// afterwards lane l holds the sum over all 64 lanes of value (l % N).  Every
// exchange step halves the number of live values, so the cost is about
// N + log2(64) shuffles instead of N * log2(64).
template <int N, int MASK>
__device__ __forceinline__ float reduce_rec(float (&cur)[N], int lane) {
    if constexpr (N == 1) {
        float v = cur[0];
        if constexpr (MASK <= 1) v += lane_xor<1>(v);
        if constexpr (MASK <= 2) v += lane_xor<2>(v);
        if constexpr (MASK <= 4) v += dpp_mov<0x124>(v);     // row_ror:4; with row_ror:8 below: l, l+4, l+8, l+12
        if constexpr (MASK <= 8) v += lane_xor<8>(v);
        if constexpr (MASK <= 16) v += lane_xor<16>(v);
        v += lane_xor<32>(v);
        return v;
    } else {
        float nxt[N / 2];
        const bool up = (lane & MASK) != 0;
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const float keep = up ? cur[2 * i + 1] : cur[2 * i];
            const float give = up ? cur[2 * i] : cur[2 * i + 1];
            nxt[i] = keep + lane_xor<MASK>(give);
        }
        return reduce_rec<N / 2, MASK * 2>(nxt, lane);
    }
}

// LDS byte address of table entry `byte J of idx`, private column of this lane:
// (entry << 8) | (lane << 2), built by one byte permute.
template <int J>
__device__ __forceinline__ uint32_t entry_addr(uint32_t idx_bytes, uint32_t laneoff) {
    return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0000u | ((4u + J) << 8));
}

__device__ __forceinline__ float lds_f32(const char* lds, uint32_t byte_addr) {
    return *reinterpret_cast<const float*>(lds + byte_addr);
}

// Centroid values of the 32 columns a lane owns, from one 16-entry table
// (TABLE_OFF selects it) or from the 256-entry sum table of shared rotation
// (reference src/dequantizer.cpp:144-169: index = residual_nibble << 4 | primary_nibble).
template <bool LUT256, int TABLE_OFF>
__device__ __forceinline__ void lookup32(const uint4& P, const uint4& Q, const char* lds, uint32_t laneoff,
                                         float (&val)[kChunk]) {
    const uint32_t pw[4] = {P.x, P.y, P.z, P.w};
    const uint32_t rw[4] = {Q.x, Q.y, Q.z, Q.w};
    uint32_t ce[4], co[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        if constexpr (LUT256) {
            ce[d] = ((rw[d] << 4) & 0xF0F0F0F0u) | (pw[d] & 0x0F0F0F0Fu);     // even columns
            co[d] = (rw[d] & 0xF0F0F0F0u) | ((pw[d] >> 4) & 0x0F0F0F0Fu);    // odd columns
        } else {
            ce[d] = pw[d] & 0x0F0F0F0Fu;
            co[d] = (pw[d] >> 4) & 0x0F0F0F0Fu;
        }
    }
    const char* tab = lds + TABLE_OFF;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        val[8 * d + 0] = lds_f32(tab, entry_addr<0>(ce[d], laneoff));
        val[8 * d + 1] = lds_f32(tab, entry_addr<0>(co[d], laneoff));
        val[8 * d + 2] = lds_f32(tab, entry_addr<1>(ce[d], laneoff));
        val[8 * d + 3] = lds_f32(tab, entry_addr<1>(co[d], laneoff));
        val[8 * d + 4] = lds_f32(tab, entry_addr<2>(ce[d], laneoff));
        val[8 * d + 5] = lds_f32(tab, entry_addr<2>(co[d], laneoff));
        val[8 * d + 6] = lds_f32(tab, entry_addr<3>(ce[d], laneoff));
        val[8 * d + 7] = lds_f32(tab, entry_addr<3>(co[d], laneoff));
    }
}

constexpr int kLut256Bytes = 256 * 256;          // 256 entries x 64 lanes x 4 B
constexpr int kTab16Bytes = 16 * 256;
constexpr int kPartialBytes = 2 * 16 * 16 * 4;   // [2 buffers][<=16 waves][<=16 values]
constexpr int kShareBytes = 4 * kSlab * 4;       // activation hand-over: up to 4 slab images

template <int MODE>
__host__ __device__ constexpr int table_bytes() {
    return MODE == kSharedLut ? kLut256Bytes : (MODE == kDual ? 2 * kTab16Bytes : kTab16Bytes);
}
template <int MODE>
__host__ __device__ constexpr int table_region_bytes() {
    return table_bytes<MODE>() > kShareBytes ? table_bytes<MODE>() : kShareBytes;
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
    constexpr int kRegion = table_region_bytes<MODE>();
    constexpr int V = R * NB;                       // sums produced per row group
    __shared__ __align__(16) char smem[kRegion + kPartialBytes];
    float* partial = reinterpret_cast<float*>(smem + kRegion);   // [2][waves][V]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slab = wave % a.W;
    const int stream = wave / a.W;
    const int chunk = slab * kWave + lane;
    const bool active = chunk < a.chunks;
    const int chunk_c = active ? chunk : a.chunks - 1;      // idle lanes re-read a valid chunk; their xt is 0
    const uint32_t laneoff = (uint32_t)lane << 2;
    const int out = a.L.out_features;
    const size_t row_bytes = (size_t)a.L.in_features >> 1;
    constexpr bool use_res = (MODE != kPrimaryOnly);

    const long long gs = (long long)blockIdx.x * a.S + stream;
    const long long ts = (long long)gridDim.x * a.S;
    const int g_begin = (int)(gs * a.groups / ts);
    const int g_end = (int)((gs + 1) * a.groups / ts);

    const uint8_t* pp = a.L.packed_primary + (size_t)chunk_c * 16;
    const uint8_t* pr = a.L.packed_residual + (size_t)chunk_c * 16;

    uint4 P[2][R], Q[2][R];
    auto fetch = [&](int buf, int g) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            int r = g * R + i;
            r = r < out ? r : out - 1;                      // rows past the end re-read the last row; never stored
            P[buf][i] = load_stream16(pp + (size_t)r * row_bytes);
            if constexpr (use_res)
                Q[buf][i] = load_stream16(pr + (size_t)r * row_bytes);
            else
                Q[buf][i] = make_uint4(0, 0, 0, 0);
        }
    };

    // First weight fetch goes out before the prologue so its latency overlaps it.
    fetch(0, g_begin);

    // Rotated activations, kept in registers for the whole kernel.
    float xt[NB][kChunk];
    float xr[NB][kChunk];   // second rotation, dual mode only
    if (a.share_x) {
        // One stream rotates, every stream of the workgroup picks the result up from LDS
        // (value k of lane l at float index k*64 + l: conflict-free both ways).
        float* xs = reinterpret_cast<float*>(smem);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (stream == 0) {
                rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                             a.L.seed_primary, a.L.block_size, lane, xt[b]);
#pragma unroll
                for (int k = 0; k < kChunk; ++k) xs[slab * kSlab + k * kWave + lane] = xt[b][k];
            }
            __syncthreads();
            if (stream != 0) {
#pragma unroll
                for (int k = 0; k < kChunk; ++k) xt[b][k] = xs[slab * kSlab + k * kWave + lane];
            }
            __syncthreads();
            if constexpr (MODE == kDual) {
                if (stream == 0) {
                    rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                                 a.L.seed_residual, a.L.block_size, lane, xr[b]);
#pragma unroll
                    for (int k = 0; k < kChunk; ++k) xs[slab * kSlab + k * kWave + lane] = xr[b][k];
                }
                __syncthreads();
                if (stream != 0) {
#pragma unroll
                    for (int k = 0; k < kChunk; ++k) xr[b][k] = xs[slab * kSlab + k * kWave + lane];
                }
                __syncthreads();
            }
        }
    } else {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                         a.L.seed_primary, a.L.block_size, lane, xt[b]);
            if constexpr (MODE == kDual)
                rotate_chunk(a.x, a.x_dtype, (size_t)b * a.L.in_features, chunk, active,
                             a.L.seed_residual, a.L.block_size, lane, xr[b]);
        }
    }

    // Decode tables -> LDS, one private column per lane.
    {
        constexpr int entries = (MODE == kSharedLut) ? 256 : (MODE == kDual ? 32 : 16);
        float4* dst = reinterpret_cast<float4*>(smem);
        for (int i = tid; i < entries * 16; i += blockDim.x) {
            const float v = a.L.tables[i >> 4];
            dst[i] = make_float4(v, v, v, v);
        }
    }
    __syncthreads();

    auto consume = [&](int buf, int g, int it) {
        float acc[V];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            float val[kChunk];
            lookup32<MODE == kSharedLut, 0>(P[buf][i], Q[buf][i], smem, laneoff, val);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
                for (int k = 0; k < kChunk; k += 2) {
                    s0 = __builtin_fmaf(val[k], xt[b][k], s0);
                    s1 = __builtin_fmaf(val[k + 1], xt[b][k + 1], s1);
                }
                acc[i * NB + b] = s0 + s1;
            }
            if constexpr (MODE == kDual) {
                lookup32<false, kTab16Bytes>(Q[buf][i], Q[buf][i], smem, laneoff, val);
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
                    for (int k = 0; k < kChunk; k += 2) {
                        s0 = __builtin_fmaf(val[k], xr[b][k], s0);
                        s1 = __builtin_fmaf(val[k + 1], xr[b][k + 1], s1);
                    }
                    acc[i * NB + b] += s0 + s1;
                }
            }
        }
        // Lane l < V now gets the wave total of value l = i*NB + b.
        const float total = reduce_rec<V, 1>(acc, lane);
        const int i = lane / NB, b = lane % NB;
        const int r = g * R + i;
        const bool owner = lane < V && g < g_end && r < out;

        if (a.W == 1) {
            if (owner) store_scalar(a.y, a.y_dtype, (size_t)b * out + r, total * (a.out_scale * a.L.norms[r]));
        } else {
            float* buf_base = partial + (it & 1) * (16 * 16);
            if (lane < V) buf_base[wave * V + lane] = total;
            __syncthreads();
            if (slab == 0 && owner) {
                float t = 0.0f;
                for (int w = 0; w < a.W; ++w) t += buf_base[(stream * a.W + w) * V + lane];
                store_scalar(a.y, a.y_dtype, (size_t)b * out + r, t * (a.out_scale * a.L.norms[r]));
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
static hipError_t launch_one(const GemvArgs& a, int grid, int threads, hipStream_t stream) {
    hipLaunchKernelGGL((tq_gemv_kernel<MODE, NB, R, MAXT>), dim3(grid), dim3(threads), 0, stream, a);
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
    a.share_x = (a.S > 1 && a.W * kSlab * 4 <= kShareBytes) ? 1 : 0;

    // Largest row-group size that still gives every resident stream work.
    int R = 4;
    while (R > 1 && (long long)((out + R - 1) / R) < (long long)max_grid * a.S) R >>= 1;
    a.groups = (out + R - 1) / R;
    int grid = (a.groups + a.S - 1) / a.S;
    if (grid > max_grid) grid = max_grid;
    if (grid < 1) grid = 1;
    const long long ts = (long long)grid * a.S;
    a.iters = (int)((a.groups + ts - 1) / ts);

    switch (R) {
        case 4: return launch_one<MODE, NB, 4, MAXT>(a, grid, threads, stream);
        case 2: return launch_one<MODE, NB, 2, MAXT>(a, grid, threads, stream);
        default: return launch_one<MODE, NB, 1, MAXT>(a, grid, threads, stream);
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
