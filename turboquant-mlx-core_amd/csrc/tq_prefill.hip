// TQ8 prefill: dequantise-into-LDS + bf16 MFMA GEMM for gfx950 (batch >= 16, 16-bit activations).
//
// The reference has no batched-GEMM path: batch is a grid dimension of its per-row-FWHT kernel
// (src/dequantizer.cpp:545-549), so every weight block is inverse-transformed once per batch row.
// Here the activations are rotated once (X~ = H (s (.) X) per block, fp32 butterfly, rounded to
// bf16) and the layer becomes one dense contraction
//
//   Y[m, n] = norm[n] / sqrt(in * bs) * sum_k X~[m, k] * L[n, k],   L = centroid (sum) of the indices
//
// Workgroup tile 256 (M) x 256 (N) x 64 (K), 8 waves as 2 (M) x 4 (N), each wave 128 x 64 built
// from v_mfma_f32_32x32x16_bf16.  Per K step every thread fetches 64 B of X~ and 32 index bytes
// (32 weights), turns the indices into bf16 through the lane-private LDS table, and parks both in
// registers while the MFMAs of the current step run; the tiles are then written to LDS in the
// k-contiguous layout both MFMA operands want (row pitch 144 B: conflict-free 128-bit reads).
#include "tq_device.h"

namespace tq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kPitch = (kBK + 8) * 2;                 // bytes per LDS tile row (bf16), padded
constexpr int kTileBytes = 256 * kPitch;              // 36864
constexpr int kGemmThreads = 512;
constexpr int kGemmLutBytes = 256 * 256;

struct PrefillArgs {
    const uint16_t* xt;        // rotated activations bf16 [planes][M, K]
    const uint8_t* plane0;     // combined bytes [N, K] (shared) or primary nibbles [N, K/2]
    const uint8_t* plane1;     // residual nibbles [N, K/2] (dual) or NULL
    const float* tables;       // 256 floats (see build_tables in tq_linear_c.cpp)
    const float* norms;
    void* y;
    int y_dtype;
    int M, N, K;
    int mode;
    int m_tiles, n_tiles;
    float out_scale;
};

__device__ __forceinline__ uint32_t gemm_entry_addr(uint32_t idx_bytes, uint32_t laneoff, int j) {
    switch (j) {
        case 0: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0400u);
        case 1: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0500u);
        case 2: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0600u);
        default: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0700u);
    }
}

// Table entries are fp32 bit patterns already rounded to bf16 (low 16 bits zero): two of them
// pack into one bf16x2 register with a single byte permute.
__device__ __forceinline__ uint32_t pack_bf16x2(uint32_t lo_val, uint32_t hi_val) {
    return __builtin_amdgcn_perm(hi_val, lo_val, 0x07060302u);   // {lo.b2, lo.b3, hi.b2, hi.b3}
}

template <int MODE>
__global__ __launch_bounds__(kGemmThreads) void tq_prefill_gemm_kernel(PrefillArgs a) {
    __shared__ __align__(16) char smem[kGemmLutBytes + 2 * kTileBytes];
    char* As = smem + kGemmLutBytes;
    char* Bs = As + kTileBytes;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t laneoff = (uint32_t)lane << 2;

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs (id % 8), so the
    // M tiles that share one N tile of weights are given to the same XCD back to back.
    const int id = blockIdx.x;
    const int xcd = id & 7, slot = id >> 3;
    const int n_tile = (slot / a.m_tiles) * 8 + xcd;
    const int m_tile = slot % a.m_tiles;
    if (n_tile >= a.n_tiles) return;                       // whole workgroup leaves together
    const int m0 = m_tile * kBM, n0 = n_tile * kBN;

    // Loader mapping: thread -> (tile row, 32-column half).
    const int lrow = tid >> 1, lhalf = tid & 1;
    const int a_row = (m0 + lrow < a.M) ? m0 + lrow : a.M - 1;
    const int b_row = (n0 + lrow < a.N) ? n0 + lrow : a.N - 1;

    constexpr bool combined = (MODE == kSharedLut);
    constexpr int kPlanes = (MODE == kDual) ? 2 : 1;
    const int ksteps = a.K / kBK;

    // MFMA mapping: 2 x 4 waves, each 128 x 64.
    const int wm = wave >> 2, wn = wave & 3;
    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    for (int plane = 0; plane < kPlanes; ++plane) {
        // Decode table of this plane -> LDS, one private column per lane, values rounded to bf16.
        __syncthreads();
        {
            const int entries = combined ? 256 : 16;
            const float* src = a.tables + (plane == 0 ? 0 : 16);
            uint4* dst = reinterpret_cast<uint4*>(smem);
            for (int i = tid; i < entries * 16; i += kGemmThreads) {
                const uint32_t v = (uint32_t)float_to_bf16_bits(src[i >> 4]) << 16;
                dst[i] = make_uint4(v, v, v, v);
            }
        }
        __syncthreads();

        const uint16_t* xa = a.xt + (size_t)plane * a.M * a.K + (size_t)a_row * a.K + lhalf * 32;
        const uint8_t* wb = combined ? a.plane0 + (size_t)b_row * a.K + lhalf * 32
                                     : (plane == 0 ? a.plane0 : a.plane1) + (size_t)b_row * (a.K >> 1) + lhalf * 16;

        u32x4v ra[4];         // 32 bf16 of X~
        uint32_t rb[16];      // 32 decoded bf16 weights
        auto fetch_decode = [&](int ks) {
            const u32x4v* pa = reinterpret_cast<const u32x4v*>(xa + (size_t)ks * kBK);
#pragma unroll
            for (int i = 0; i < 4; ++i) ra[i] = pa[i];
            if constexpr (combined) {
                const uint4* pb = reinterpret_cast<const uint4*>(wb + (size_t)ks * kBK);
                const uint4 b0 = pb[0], b1 = pb[1];
                const uint32_t w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                for (int d = 0; d < 8; ++d) {
                    const uint32_t v0 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w[d], laneoff, 0));
                    const uint32_t v1 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w[d], laneoff, 1));
                    const uint32_t v2 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w[d], laneoff, 2));
                    const uint32_t v3 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w[d], laneoff, 3));
                    rb[2 * d] = pack_bf16x2(v0, v1);
                    rb[2 * d + 1] = pack_bf16x2(v2, v3);
                }
            } else {
                const uint4 b0 = *reinterpret_cast<const uint4*>(wb + (size_t)ks * (kBK >> 1));
                const uint32_t w[4] = {b0.x, b0.y, b0.z, b0.w};
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t ce = w[d] & 0x0F0F0F0Fu, co = (w[d] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t ve = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(ce, laneoff, j));
                        const uint32_t vo = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(co, laneoff, j));
                        rb[4 * d + j] = pack_bf16x2(ve, vo);
                    }
                }
            }
        };
        auto park = [&]() {
            u32x4v* da = reinterpret_cast<u32x4v*>(As + lrow * kPitch + lhalf * 64);
            u32x4v* db = reinterpret_cast<u32x4v*>(Bs + lrow * kPitch + lhalf * 64);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                da[i] = ra[i];
                u32x4v t = {rb[4 * i], rb[4 * i + 1], rb[4 * i + 2], rb[4 * i + 3]};
                db[i] = t;
            }
        };

        fetch_decode(0);
        park();
        __syncthreads();

        for (int ks = 0; ks < ksteps; ++ks) {
            if (ks + 1 < ksteps) fetch_decode(ks + 1);       // loads + lookups fly under the MFMAs

#pragma unroll
            for (int s = 0; s < kBK / 16; ++s) {
                bf16x8 fa[4], fb[2];
                const int koff = s * 32 + (lane >> 5) * 16;          // bytes
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    fa[i] = *reinterpret_cast<const bf16x8*>(As + (wm * 128 + i * 32 + (lane & 31)) * kPitch + koff);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    fb[j] = *reinterpret_cast<const bf16x8*>(Bs + (wn * 64 + j * 32 + (lane & 31)) * kPitch + koff);
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
            __syncthreads();                                  // every wave is done reading the tiles
            if (ks + 1 < ksteps) park();
            __syncthreads();
        }
    }

    // Epilogue: * norm[n] / sqrt(in * bs), convert, store.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        const bool col_ok = col < a.N;
        const float s = col_ok ? a.out_scale * a.norms[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * 128 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (col_ok && row < a.M) store_scalar(a.y, a.y_dtype, (size_t)row * a.N + col, acc[i][j][r] * s);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Rotate activations [M, K] (f32 / f16 / bf16) -> bf16 [M, K]: X~ = H (s (.) X) per block.
// One wave per (row, 2048-column slab), 32 consecutive columns per lane, fp32 butterfly.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void tq_rotate_bf16_kernel(const void* __restrict__ x, int x_dtype,
                                                             uint16_t* __restrict__ out, int rows, int cols,
                                                             int chunks, int slabs, uint32_t seed, uint32_t bs) {
    const int lane = threadIdx.x & 63;
    const long long wid = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row = (int)(wid / slabs);
    const int slab = (int)(wid % slabs);
    if (row >= rows) return;
    const int chunk = slab * kWave + lane;
    const bool active = chunk < chunks;
    const uint32_t col0 = ((uint32_t)chunk * kChunk) & (bs - 1);
    float v[kChunk];
    if (active) {
        load_chunk(x, x_dtype, (size_t)row * cols + (size_t)chunk * kChunk, v);
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] *= sign_of(seed, (col0 + k) & (bs - 1));
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    fwht_lane32(v, bs, lane);
    if (active) {
        uint4* dst = reinterpret_cast<uint4*>(out + (size_t)row * cols + (size_t)chunk * kChunk);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = (uint32_t)float_to_bf16_bits(v[8 * i + 2 * j]) | ((uint32_t)float_to_bf16_bits(v[8 * i + 2 * j + 1]) << 16);
            dst[i] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

size_t prefill_workspace_bytes(const LayerView& L, int batch) {
    const size_t planes = (L.mode == kDual) ? 2 : 1;
    return planes * (size_t)batch * L.in_features * sizeof(uint16_t);
}

bool prefill_supported(const LayerView& L, int x_dtype, int batch) {
    if (x_dtype == kF32 || batch < 16) return false;          // fp32 activations keep the exact fp32 GEMV path
    if (L.mode != kSharedLut && L.mode != kDual && L.mode != kPrimaryOnly) return false;
    return L.in_features % kBK == 0;
}

hipError_t launch_prefill(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                          void* workspace, hipStream_t stream) {
    const int K = L.in_features, N = L.out_features, M = batch;
    uint16_t* xt = static_cast<uint16_t*>(workspace);
    const int chunks = K / kChunk;
    const int slabs = (chunks + kWave - 1) / kWave;
    const long long waves = (long long)M * slabs;
    const unsigned rgrid = (unsigned)((waves + 3) / 4);
    hipLaunchKernelGGL(tq_rotate_bf16_kernel, dim3(rgrid), dim3(256), 0, stream, x, x_dtype, xt, M, K, chunks, slabs,
                       L.seed_primary, L.block_size);
    if (L.mode == kDual)
        hipLaunchKernelGGL(tq_rotate_bf16_kernel, dim3(rgrid), dim3(256), 0, stream, x, x_dtype, xt + (size_t)M * K,
                           M, K, chunks, slabs, L.seed_residual, L.block_size);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;

    PrefillArgs a{};
    a.xt = xt;
    a.plane0 = (L.mode == kSharedLut) ? L.packed_combined : L.packed_primary;
    a.plane1 = L.packed_residual;
    a.tables = L.tables;
    a.norms = L.norms;
    a.y = y; a.y_dtype = y_dtype;
    a.M = M; a.N = N; a.K = K; a.mode = L.mode;
    a.m_tiles = (M + kBM - 1) / kBM;
    a.n_tiles = (N + kBN - 1) / kBN;
    a.out_scale = L.inv_scale * L.inv_sqrt_bs;
    const int n_groups = (a.n_tiles + 7) / 8;
    const unsigned grid = (unsigned)(n_groups * 8 * a.m_tiles);
    switch (L.mode) {
        case kSharedLut:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kSharedLut>, dim3(grid), dim3(kGemmThreads), 0, stream, a); break;
        case kDual:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kDual>, dim3(grid), dim3(kGemmThreads), 0, stream, a); break;
        default:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kPrimaryOnly>, dim3(grid), dim3(kGemmThreads), 0, stream, a); break;
    }
    return hipGetLastError();
}

}  // namespace tq
