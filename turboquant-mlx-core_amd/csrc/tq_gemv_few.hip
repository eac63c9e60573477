// Fused TQ8 dequant + matrix-vector products for gfx950, two to twelve activation rows, blocks of at most 512
// columns: shared-rotation layers (one byte per weight) and, further down, nibble planes (dual rotation, primary only).
//
// The batch-1 kernel (tq_gemv_wide.hip) reads the plane in whole rows and runs at the rate of its table reads.  The
// small-batch kernel (tq_skinny.hip) puts the activation rows on v_mfma_f32_16x16x32_f16, whose operand layout
// wants 16 weight rows per load instruction, 64 bytes of each; it cuts K over the workgroups and adds the parts in a
// second kernel.  Four activation rows fit v_mfma_f32_4x4x4_16b_f16 instead (five to twelve: two or three such sets on
// the same decoded weights): 16 independent 4 x 4 x 4 blocks per instruction, block = lane / 4.  The four lanes of a
// block hold the same 16 columns of four consecutive weight rows (A operand: four decoded weights per step) and of
// the four activation rows (B operand), so
//   * a load instruction of a wave fetches 256 contiguous bytes of each of four rows (whole cache lines, streaming
//     hint), a wave covers U such segments of its four rows, and the waves of a row stream cover the whole row: no
//     cut along K, the cross-wave sum stays inside the workgroup and there is no second kernel;
//   * a decoded weight costs one address permute, one table read and half a pack (as in the small-batch kernel)
//     whatever the number of activation rows; the products are four matrix instructions per 16 bytes of a lane;
//   * the kernel keeps the batch-1 kernel's shape: one workgroup of up to 16 waves per CU, lane-private table
//     in LDS, the rotated activations of a lane's columns in registers (fp16 pairs, scaled by 1 / sqrt(bs) before
//     they are rounded, as in the small-batch and prefill kernels), every load slot requested again as soon as it
//     has been decoded.
// The activation rows are rotated once per CU (the waves share out the 512-column tiles of all rows and hand the
// result over through fp16 images in LDS), or, where the images do not fit, there are more than four rows (every
// CU rotating every row costs 0.15 us per tile and row) or the layer has nibble planes, by a small kernel of its
// own into the layer's scratch row or a workspace.
// Sums are fp32.  The reference has no batched path (src/dequantizer.cpp:545-549: batch is a grid dimension of its
// per-row kernel).
#include "tq_device.h"
#include "tq_gemv_common.h"

namespace tq {

namespace {

constexpr int kSegCols = 256;                    // columns of a segment: 16 blocks x 16 columns
constexpr int kFewMaxBatch = 12;                 // byte plane; nibble planes: 8
constexpr int kFewImageBytes = 88 * 1024;        // fp16 images of the activation rows in LDS
constexpr int kFewMaxU = 8;
constexpr int kFewSumStride = 48;                 // floats per wave in the cross-wave buffer: 16 sums x up to 3 sets of rows
constexpr int kFewPartialBytes = 2 * 16 * kFewSumStride * 4;   // [2 buffers][<= 16 waves][kFewSumStride]

// (Two quads of weight rows per trip of the main loop, for twice the loads in flight and half the cross-wave sums,
// measured no faster on the large layers and slower on the small ones, whose streams have one or two quads.)

struct FewArgs {
    LayerView L;
    const void* x;       // activations [batch, in] (x_dtype), or PRE: rotated, scaled fp16 [batch, in]
    void* y;
    int x_dtype, y_dtype;
    int batch;
    int W, S;            // waves per row quad, quad streams per workgroup
    int w_inv;           // (w * w_inv) >> 8 == w / W
    int iters;           // uniform trip count: the longest range of a stream, in quads
    int quads_q, quads_rem;
    int ntiles, nt_inv;  // 512-column tiles of a row; (i * nt_inv) >> 16 == i / ntiles for the job numbers in use
    int planes, segs;    // nibble planes: planes of the layer (1 or 2) and 512-column segments of a plane
};

typedef _Float16 few_h4 __attribute__((ext_vector_type(4)));
typedef float few_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t few_u2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint4 few_load16(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, int row_off) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off, row_off, 2);
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint4 few_pack8(const float (&v)[8], float s) {
    uint4 o;
    o.x = (uint32_t)float_to_f16_bits(v[0] * s) | ((uint32_t)float_to_f16_bits(v[1] * s) << 16);
    o.y = (uint32_t)float_to_f16_bits(v[2] * s) | ((uint32_t)float_to_f16_bits(v[3] * s) << 16);
    o.z = (uint32_t)float_to_f16_bits(v[4] * s) | ((uint32_t)float_to_f16_bits(v[5] * s) << 16);
    o.w = (uint32_t)float_to_f16_bits(v[6] * s) | ((uint32_t)float_to_f16_bits(v[7] * s) << 16);
    return o;
}
// The same for values that carry their scale already: four packed conversions (round to nearest even, saturating
// like the above).
__device__ __forceinline__ uint4 few_pack8(const float (&v)[8]) {
    uint4 o;
    o.x = pack_f16_saturating(v[0], v[1]);
    o.y = pack_f16_saturating(v[2], v[3]);
    o.z = pack_f16_saturating(v[4], v[5]);
    o.w = pack_f16_saturating(v[6], v[7]);
    return o;
}

// One butterfly stage across lanes l and l ^ 16 (or 32) for two values at once: v_permlane16_swap / _permlane32_swap
// exchange rows (halves) between two registers, so a swap, a sum, a difference and a second swap serve both values,
// four instructions where lane_xor + select + fma take six.  Lower lane a + b, upper lane a - b with a the lower
// lane's value: the bits of butterfly_lanes.
template <int MASK>
__device__ __forceinline__ void few_butterfly_pair(float& a, float& b) {
    static_assert(MASK == 16 || MASK == 32, "row and half swaps");
    const unsigned ua = __builtin_bit_cast(unsigned, a), ub = __builtin_bit_cast(unsigned, b);
    float lo, hi;
    if constexpr (MASK == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(ua, ub, false, false);
        lo = __builtin_bit_cast(float, (unsigned)r[0]); hi = __builtin_bit_cast(float, (unsigned)r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(ua, ub, false, false);
        lo = __builtin_bit_cast(float, (unsigned)r[0]); hi = __builtin_bit_cast(float, (unsigned)r[1]);
    }
    const float sum = lo + hi, dif = lo - hi;
    const unsigned us = __builtin_bit_cast(unsigned, sum), ud = __builtin_bit_cast(unsigned, dif);
    if constexpr (MASK == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(us, ud, false, false);
        a = __builtin_bit_cast(float, (unsigned)r[0]); b = __builtin_bit_cast(float, (unsigned)r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(us, ud, false, false);
        a = __builtin_bit_cast(float, (unsigned)r[0]); b = __builtin_bit_cast(float, (unsigned)r[1]);
    }
}

// rotate_tile() with the signs handed in: blocks are at most one tile wide and tiles start at multiples of 512, so
// the sign of a column depends on its position inside the tile alone, and a wave computes its eight once for all
// the tiles it rotates (the hash is a quarter of the instructions of a rotation).  The signs may carry a scale.
__device__ __forceinline__ void few_rotate(const TileRaw& raw, int x_dtype, bool active, const float (&sg)[8],
                                           uint32_t bs, int lane, float (&v)[8]) {
    if (active) {
        if (x_dtype == kF32) {
            const uint32_t w[8] = {raw.a.x, raw.a.y, raw.a.z, raw.a.w, raw.b.x, raw.b.y, raw.b.z, raw.b.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = __builtin_bit_cast(float, w[j]);
        } else {
            const uint32_t w[4] = {raw.a.x, raw.a.y, raw.a.z, raw.a.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (x_dtype == kBF16) {
                    v[2 * j]     = bf16_bits_to_float(w[j] & 0xffffu);
                    v[2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
                } else {
                    v[2 * j]     = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] & 0xffffu));
                    v[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] >> 16));
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] *= sg[j];
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = 0.0f;
    }
    // fwht_lanes<8> with the stages across 16 and 32 lanes done two values at a time.
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
        if ((uint32_t)h < bs) {
#pragma unroll
            for (int i = 0; i < 8; i += 2 * h) {
#pragma unroll
                for (int k = i; k < i + h; ++k) {
                    const float p = v[k], q = v[k + h];
                    v[k] = p + q;
                    v[k + h] = p - q;
                }
            }
        }
    }
    if (8u < bs) butterfly_lanes<1, 8>(v, lane);
    if (16u < bs) butterfly_lanes<2, 8>(v, lane);
    if (32u < bs) butterfly_lanes<4, 8>(v, lane);
    if (64u < bs) butterfly_lanes<8, 8>(v, lane);
    if (128u < bs) {
#pragma unroll
        for (int k = 0; k < 8; k += 2) few_butterfly_pair<16>(v[k], v[k + 1]);
    }
    if (256u < bs) {
#pragma unroll
        for (int k = 0; k < 8; k += 2) few_butterfly_pair<32>(v[k], v[k + 1]);
    }
}

// SETS sets of four activation rows, U segments per wave (wave w of a quad stream owns segments U w .. U w + U - 1 of
// its rows), TL tile jobs of the rotation per wave (PRE: none, the rows come rotated).
template <int SETS, int U, int TL, bool PRE>
__device__ __forceinline__ void few_body(const FewArgs& a, const int block) {
    static_assert(SETS == 1 || PRE, "more than four activation rows come rotated");
    constexpr int kImage = PRE ? 0 : kFewImageBytes;
    __shared__ __align__(16) char smem[kLut256Bytes + kFewPartialBytes + kImage];
    float* const partial = reinterpret_cast<float*>(smem + kLut256Bytes);     // [2][waves][SETS][16]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = blockDim.x >> 6;
    const int stream = (wave * a.w_inv) >> 8;
    const int unit = wave - stream * a.W;
    const uint32_t laneoff = (uint32_t)lane << 2;
    const int out = a.L.out_features, K = a.L.in_features;
    const int blk = lane >> 2, q = lane & 3;      // block of the matrix instruction; weight row of the quad and activation row of a set

    int col[U];
    bool act[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        col[u] = (unit * U + u) * kSegCols + 16 * blk;
        act[u] = col[u] < K;
    }

    // Quads of this stream: a contiguous range, one more for the first quads_rem streams.
    const int gs = block * a.S + stream;
    const int q_begin = gs * a.quads_q + (gs < a.quads_rem ? gs : a.quads_rem);
    const int q_end = q_begin + a.quads_q + (gs < a.quads_rem ? 1 : 0);
    const int r_begin = 4 * q_begin;
    const int r_end = 4 * q_end < out ? 4 * q_end : out;
    const int r_base = r_begin < out ? r_begin : out - 1;

    // The plane through a buffer descriptor based at the stream's first row.  Segments past the row and rows past
    // the range ask for an offset beyond the descriptor and fetch nothing (zeros: entry 0 of the table, times
    // activations that are zero, or sums that are not stored).
    constexpr uint32_t kNoFetch = 0x80000000u;
    uint32_t off[U];
#pragma unroll
    for (int u = 0; u < U; ++u) off[u] = act[u] ? (uint32_t)q * (uint32_t)K + (uint32_t)col[u] : kNoFetch;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(a.L.packed_combined) + (size_t)r_base * (size_t)K, 0, 0x7fffffff, 0x00020000);
    // One load slot per segment, requested again as soon as it is decoded.  Two segments per wave (three sets of
    // rows) would leave 2 KB per wave in flight, so they keep the slots of two trips.  (With three and four
    // segments per wave two trips were slower: 27648 x 5120 28.2 / 29.4 / 31.5 against 27.4 / 28.8 / 30.4 us.)
    constexpr int D = U <= 2 ? 2 : 1;
    using D0 = std::integral_constant<int, 0>;
    using D1 = std::integral_constant<int, D - 1>;
    uint4 P[D][U];
    auto fetch = [&](auto Dc, auto Uc, int r0) {
        constexpr int d = decltype(Dc)::value, u = decltype(Uc)::value;
        P[d][u] = few_load16(rs, r0 + q < r_end ? off[u] : kNoFetch, (r0 - r_base) * K);
    };
    auto norm_of = [&](int r0) {
        const int rn = r0 + ((lane >> 2) & 3);
        return a.L.norms[rn < out ? rn : out - 1];
    };

    // Small requests first (loads complete in order): the activation tiles this wave rotates, or its columns of
    // the rotated rows; then the norms of the first quad and the first weights.
    uint32_t xh[SETS][U][8];                  // fp16 pairs of activation row q + 4 e: columns 2 j, 2 j + 1 of segment u
    TileRaw raw[PRE ? 1 : TL];
    const int jobs = a.batch * a.ntiles;
    if constexpr (PRE) {
        const char* xr = static_cast<const char*>(a.x);
#pragma unroll
        for (int e = 0; e < SETS; ++e)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool on = act[u] && q + 4 * e < a.batch;
                const uint4* p = reinterpret_cast<const uint4*>(xr + ((size_t)(on ? q + 4 * e : 0) * K + (on ? col[u] : 0)) * 2);
                const uint4 lo = p[0], hi = p[1];
                xh[e][u][0] = lo.x; xh[e][u][1] = lo.y; xh[e][u][2] = lo.z; xh[e][u][3] = lo.w;
                xh[e][u][4] = hi.x; xh[e][u][5] = hi.y; xh[e][u][6] = hi.z; xh[e][u][7] = hi.w;
            }
    } else {
#pragma unroll
        for (int k = 0; k < TL; ++k) {            // jobs past the last re-read the start of the first row and are not used
            const int job = wave + k * nwaves;
            const int tok = (job * a.nt_inv) >> 16;
            const int c = (job - tok * a.ntiles) * kTile + lane * 8;
            const bool on = job < jobs && c < K;
            raw[k] = load_tile_raw(a.x, a.x_dtype, (size_t)(on ? tok : 0) * K, on ? c : 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    float nrm = norm_of(r_begin);
    fetch(D0{}, std::integral_constant<int, 0>{}, r_begin);
    if constexpr (U > 1) fetch(D0{}, std::integral_constant<int, 1>{}, r_begin);
    if constexpr (U > 2) fetch(D0{}, std::integral_constant<int, 2>{}, r_begin);
    if constexpr (U > 3) fetch(D0{}, std::integral_constant<int, 3>{}, r_begin);
    if constexpr (D == 2) {
        fetch(D1{}, std::integral_constant<int, 0>{}, r_begin + 4);
        if constexpr (U > 1) fetch(D1{}, std::integral_constant<int, 1>{}, r_begin + 4);
    }

    // Decode table -> LDS, one private column per lane: fp16 value in the upper half of the entry.  Values through
    // scalar loads (a vector memory instruction holds the CU's address unit for 16 cycles, and 16 waves share it).
    {
        typedef const __attribute__((address_space(4))) float cfloat;
        cfloat* const tab = (cfloat*)a.L.tables;
        uint32_t* const dst = reinterpret_cast<uint32_t*>(smem) + lane;
        for (int c = wave; c < 16; c += nwaves) {
#pragma unroll
            for (int e = 0; e < 16; ++e) dst[(c * 16 + e) * kWave] = (uint32_t)float_to_f16_bits(tab[c * 16 + e]) << 16;
        }
    }

    if constexpr (PRE) {
        __syncthreads();                                       // table visible to every wave
#pragma unroll
        for (int e = 0; e < SETS; ++e)
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < 8; ++j) xh[e][u][j] = (act[u] && q + 4 * e < a.batch) ? xh[e][u][j] : 0u;   // idle lanes contribute 0
    } else {
        char* const image = smem + kLut256Bytes + kFewPartialBytes;               // [batch][K] fp16
        float sg[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)        // (with the scale 1 / sqrt(bs): the rotation is linear)
            sg[j] = sign_of(a.L.seed_primary, (uint32_t)(lane * 8 + j) & (a.L.block_size - 1)) * a.L.inv_sqrt_bs;
#pragma unroll
        for (int k = 0; k < TL; ++k) {
            const int job = wave + k * nwaves;
            if (job < jobs) {                                  // wave-uniform
                const int tok = (job * a.nt_inv) >> 16;
                const int c = (job - tok * a.ntiles) * kTile + lane * 8;
                float v[8];
                few_rotate(raw[k], a.x_dtype, c < K, sg, a.L.block_size, lane, v);
                if (c < K) *reinterpret_cast<uint4*>(image + ((size_t)tok * K + c) * 2) = few_pack8(v);
            }
        }
        __syncthreads();                                       // images and table visible to every wave
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool on = act[u] && q < a.batch;
            const uint4* p = reinterpret_cast<const uint4*>(image + ((size_t)(on ? q : 0) * K + (on ? col[u] : 0)) * 2);
            const uint4 lo = p[0], hi = p[1];
            xh[0][u][0] = on ? lo.x : 0u; xh[0][u][1] = on ? lo.y : 0u; xh[0][u][2] = on ? lo.z : 0u; xh[0][u][3] = on ? lo.w : 0u;
            xh[0][u][4] = on ? hi.x : 0u; xh[0][u][5] = on ? hi.y : 0u; xh[0][u][6] = on ? hi.z : 0u; xh[0][u][7] = on ? hi.w : 0u;
        }
    }
    // The other load slots are requested behind the barrier: a wave whose requests queue up in the memory pipeline
    // would otherwise keep the whole workgroup waiting there.
    if constexpr (U > 4) fetch(D0{}, std::integral_constant<int, 4>{}, r_begin);
    if constexpr (U > 5) fetch(D0{}, std::integral_constant<int, 5>{}, r_begin);
    if constexpr (U > 6) fetch(D0{}, std::integral_constant<int, 6>{}, r_begin);
    if constexpr (U > 7) fetch(D0{}, std::integral_constant<int, 7>{}, r_begin);

    // Four weights of this lane's row -> one A operand (entries are fp32 patterns with the fp16 value in the upper half).
    auto operand = [&](uint32_t w) {
        const uint32_t v0 = *reinterpret_cast<const uint32_t*>(smem + entry_addr<0>(w, laneoff));
        const uint32_t v1 = *reinterpret_cast<const uint32_t*>(smem + entry_addr<1>(w, laneoff));
        const uint32_t v2 = *reinterpret_cast<const uint32_t*>(smem + entry_addr<2>(w, laneoff));
        const uint32_t v3 = *reinterpret_cast<const uint32_t*>(smem + entry_addr<3>(w, laneoff));
        const few_u2 r = {__builtin_amdgcn_perm(v1, v0, 0x07060302u), __builtin_amdgcn_perm(v3, v2, 0x07060302u)};
        return __builtin_bit_cast(few_h4, r);
    };

    auto trip = [&](auto Dc, int it) {
        const int r0 = r_begin + 4 * it;
        const float nrm_next = norm_of(r0 + 4);
        few_f4 acc[SETS];                                      // results D[i][q] of the lane's block: weight rows r0 + i
#pragma unroll
        for (int e = 0; e < SETS; ++e) acc[e] = few_f4{0.0f, 0.0f, 0.0f, 0.0f};
        auto segment = [&](auto Uc) {
            constexpr int u = decltype(Uc)::value;
            const uint4 p = P[decltype(Dc)::value][u];
            fetch(Dc, Uc, r0 + 4 * D);
            const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const few_h4 wq = operand(pw[d]);
#pragma unroll
                for (int e = 0; e < SETS; ++e) {
                    const few_u2 xb = {xh[e][u][2 * d], xh[e][u][2 * d + 1]};
                    acc[e] = __builtin_amdgcn_mfma_f32_4x4x4f16(wq, __builtin_bit_cast(few_h4, xb), acc[e], 0, 0, 0);
                }
            }
        };
        segment(std::integral_constant<int, 0>{});
        if constexpr (U > 1) segment(std::integral_constant<int, 1>{});
        if constexpr (U > 2) segment(std::integral_constant<int, 2>{});
        if constexpr (U > 3) segment(std::integral_constant<int, 3>{});
        if constexpr (U > 4) segment(std::integral_constant<int, 4>{});
        if constexpr (U > 5) segment(std::integral_constant<int, 5>{});
        if constexpr (U > 6) segment(std::integral_constant<int, 6>{});
        if constexpr (U > 7) segment(std::integral_constant<int, 7>{});

        // Sum over the 16 blocks (the columns of the wave): afterwards every lane holds the wave total of weight row
        // (lane / 4) % 4 of the quad and activation row lane % 4 of each set.
        float total[SETS];
#pragma unroll
        for (int e = 0; e < SETS; ++e) {
            float v[4] = {acc[e][0], acc[e][1], acc[e][2], acc[e][3]};
            total[e] = reduce_rec<4, 4>(v, lane);
        }
        const int r = r0 + ((lane >> 2) & 3);
        const bool owner = lane < 16 && r < r_end;
        bool store = owner;
        if (a.W > 1) {                                         // cross-wave sum of the row's segments
            float* const buf_base = partial + (it & 1) * (16 * kFewSumStride);
            if (lane < 16) {
#pragma unroll
                for (int e = 0; e < SETS; ++e) buf_base[wave * kFewSumStride + 16 * e + lane] = total[e];
            }
            __syncthreads();
            store = owner && unit == 0;
            if (store) {
#pragma unroll
                for (int e = 0; e < SETS; ++e) {
                    float t = 0.0f;
                    for (int w = 0; w < a.W; ++w) t += buf_base[(stream * a.W + w) * kFewSumStride + 16 * e + lane];
                    total[e] = t;
                }
            }
        }
        if (store) {
#pragma unroll
            for (int e = 0; e < SETS; ++e)
                if (q + 4 * e < a.batch) store_scalar(a.y, a.y_dtype, (size_t)(q + 4 * e) * out + r, total[e] * (a.L.inv_scale * nrm));
        }
        nrm = nrm_next;
    };
    int it = 0;
    for (; it + D <= a.iters; it += D) {
        trip(D0{}, it);
        if constexpr (D == 2) trip(D1{}, it + 1);
    }
    if (it < a.iters) trip(D0{}, it);
}

template <int SETS, int U, int TL, bool PRE>
__global__ __launch_bounds__(1024) void tq_gemv_few_kernel(FewArgs a) {
    few_body<SETS, U, TL, PRE>(a, (int)blockIdx.x);
}

// Nibble planes (dual rotation: two planes, each with its own rotation and 16-entry table; primary only: one).  The
// same scheme on a plane of two weights per byte: a segment is 256 bytes of a row, 512 columns; a lane's 16 bytes are
// 32 columns; the table is indexed by a whole byte and an entry holds the fp16 centroids of both its nibbles (low
// nibble = even column), i.e. half an A operand, so four weights cost two table reads and no pack.  Both planes'
// tables share the 64 KB one took: an entry holds 32 lane columns of the primary plane's value, then 32 of the
// residual plane's, and lanes l and l + 32 share a column (the LDS serves a wave's 32-bit reads in two halves of 32
// lanes, so they never meet).  The units of a row are its primary segments, then its residual segments; wave w of a
// quad stream owns units U w .. U w + U - 1 and multiplies each with the activations of that plane's rotation, and
// the cross-wave sum adds the planes.  The rows always come rotated ([plane][batch][in] fp16): every CU rotating
// every row twice costs more than the rotation kernel.
template <int SETS, int U>
__device__ __forceinline__ void few_nibble_body(const FewArgs& a, const int block) {
    __shared__ __align__(16) char smem[kLut256Bytes + kFewPartialBytes];
    float* const partial = reinterpret_cast<float*>(smem + kLut256Bytes);     // [2][waves][SETS][16]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = blockDim.x >> 6;
    const int stream = (wave * a.w_inv) >> 8;
    const int unit = wave - stream * a.W;
    const int out = a.L.out_features, K = a.L.in_features;
    const int pitch = K >> 1;                     // bytes of a row of a plane
    const int blk = lane >> 2, q = lane & 3;
    const int units = a.planes * a.segs;

    int col[U], plane[U];
    bool act[U];
    uint32_t laneoff[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int g = unit * U + u;
        plane[u] = g >= a.segs ? 1 : 0;           // wave-uniform
        col[u] = (g - plane[u] * a.segs) * 512 + 32 * blk;
        act[u] = g < units && col[u] < K;
        laneoff[u] = ((uint32_t)(lane & 31) << 2) | ((uint32_t)plane[u] << 7);
    }

    const int gs = block * a.S + stream;
    const int q_begin = gs * a.quads_q + (gs < a.quads_rem ? gs : a.quads_rem);
    const int q_end = q_begin + a.quads_q + (gs < a.quads_rem ? 1 : 0);
    const int r_begin = 4 * q_begin;
    const int r_end = 4 * q_end < out ? 4 * q_end : out;
    const int r_base = r_begin < out ? r_begin : out - 1;

    constexpr uint32_t kNoFetch = 0x80000000u;
    uint32_t off[U];
    __amdgpu_buffer_rsrc_t rs[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        off[u] = act[u] ? (uint32_t)q * (uint32_t)pitch + (uint32_t)(col[u] >> 1) : kNoFetch;
        const uint8_t* const base = (plane[u] && a.planes == 2) ? a.L.packed_residual : a.L.packed_primary;
        rs[u] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base) + (size_t)r_base * (size_t)pitch, 0, 0x7fffffff, 0x00020000);
    }
    // Load slots: one per unit, requested again as soon as it has been decoded; two units per wave (two sets of rows)
    // would leave 2 KB per wave in flight, so they keep the slots of two trips.
    constexpr int D = U <= 2 ? 2 : 1;
    uint4 P[D][U];
    auto fetch = [&](auto Dc, auto Uc, int r0) {
        constexpr int d = decltype(Dc)::value, u = decltype(Uc)::value;
        P[d][u] = few_load16(rs[u], r0 + q < r_end ? off[u] : kNoFetch, (r0 - r_base) * pitch);
    };
    auto norm_of = [&](int r0) {
        const int rn = r0 + ((lane >> 2) & 3);
        return a.L.norms[rn < out ? rn : out - 1];
    };

    // The lane's columns of the rotated rows of its units' planes, then the norms and the first weights.
    uint32_t xh[SETS][U][16];                 // fp16 pairs of activation row q + 4 e: columns 2 j, 2 j + 1 of unit u
    {
        const char* xr = static_cast<const char*>(a.x);
#pragma unroll
        for (int e = 0; e < SETS; ++e)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool on = act[u] && q + 4 * e < a.batch;
                const size_t row = on ? (size_t)plane[u] * a.batch + q + 4 * e : 0;
                const uint4* p = reinterpret_cast<const uint4*>(xr + (row * K + (on ? col[u] : 0)) * 2);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint4 t = p[k];
                    xh[e][u][4 * k] = t.x; xh[e][u][4 * k + 1] = t.y; xh[e][u][4 * k + 2] = t.z; xh[e][u][4 * k + 3] = t.w;
                }
            }
    }
    __builtin_amdgcn_sched_barrier(0);
    float nrm = norm_of(r_begin);
    using D0 = std::integral_constant<int, 0>;
    using D1 = std::integral_constant<int, D - 1>;
    fetch(D0{}, std::integral_constant<int, 0>{}, r_begin);
    if constexpr (U > 1) fetch(D0{}, std::integral_constant<int, 1>{}, r_begin);
    if constexpr (U > 2) fetch(D0{}, std::integral_constant<int, 2>{}, r_begin);
    if constexpr (U > 3) fetch(D0{}, std::integral_constant<int, 3>{}, r_begin);
    if constexpr (D == 2) {
        fetch(D1{}, std::integral_constant<int, 0>{}, r_begin + 4);
        if constexpr (U > 1) fetch(D1{}, std::integral_constant<int, 1>{}, r_begin + 4);
    }

    // Byte-pair tables of both planes -> LDS.  (Both planes' entries are made from scalar loads and chosen per lane
    // afterwards: a choice between the two addresses instead becomes a vector load, which queues behind the
    // weight requests above.)
    {
        typedef const __attribute__((address_space(4))) float cfloat;
        cfloat* const tab = (cfloat*)a.L.tables;
        uint32_t* const dst = reinterpret_cast<uint32_t*>(smem) + lane;
        const bool second = lane >= 32;
        auto pair_entry = [&](int base, int c, int e) {
            const uint32_t h = (uint32_t)float_to_f16_bits(tab[base + c]);
            const uint32_t l = (uint32_t)float_to_f16_bits(tab[base + e]);
            return (uint32_t)__builtin_amdgcn_readfirstlane((int)((h << 16) | l));
        };
        for (int c = wave; c < 16; c += nwaves) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t u0 = pair_entry(0, c, e), u1 = pair_entry(16, c, e);
                dst[(c * 16 + e) * kWave] = second ? u1 : u0;
            }
        }
    }
    __syncthreads();                                           // tables visible to every wave
#pragma unroll
    for (int e = 0; e < SETS; ++e)
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < 16; ++j) xh[e][u][j] = (act[u] && q + 4 * e < a.batch) ? xh[e][u][j] : 0u;   // idle lanes contribute 0

    auto trip = [&](auto Dc, int it) {
        const int r0 = r_begin + 4 * it;
        const float nrm_next = norm_of(r0 + 4);
        few_f4 acc[SETS];
#pragma unroll
        for (int e = 0; e < SETS; ++e) acc[e] = few_f4{0.0f, 0.0f, 0.0f, 0.0f};
        auto segment = [&](auto Uc) {
            constexpr int u = decltype(Uc)::value;
            const uint4 p = P[decltype(Dc)::value][u];
            fetch(Dc, Uc, r0 + 4 * D);
            const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {                      // dword d: columns 8 d .. 8 d + 7 of the lane's 32
                const few_u2 w0 = {*reinterpret_cast<const uint32_t*>(smem + entry_addr<0>(pw[d], laneoff[u])),
                                   *reinterpret_cast<const uint32_t*>(smem + entry_addr<1>(pw[d], laneoff[u]))};
                const few_u2 w1 = {*reinterpret_cast<const uint32_t*>(smem + entry_addr<2>(pw[d], laneoff[u])),
                                   *reinterpret_cast<const uint32_t*>(smem + entry_addr<3>(pw[d], laneoff[u]))};
#pragma unroll
                for (int e = 0; e < SETS; ++e) {
                    const few_u2 x0 = {xh[e][u][4 * d], xh[e][u][4 * d + 1]}, x1 = {xh[e][u][4 * d + 2], xh[e][u][4 * d + 3]};
                    acc[e] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(few_h4, w0), __builtin_bit_cast(few_h4, x0), acc[e], 0, 0, 0);
                    acc[e] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(few_h4, w1), __builtin_bit_cast(few_h4, x1), acc[e], 0, 0, 0);
                }
            }
        };
        segment(std::integral_constant<int, 0>{});
        if constexpr (U > 1) segment(std::integral_constant<int, 1>{});
        if constexpr (U > 2) segment(std::integral_constant<int, 2>{});
        if constexpr (U > 3) segment(std::integral_constant<int, 3>{});

        float total[SETS];
#pragma unroll
        for (int e = 0; e < SETS; ++e) {
            float v[4] = {acc[e][0], acc[e][1], acc[e][2], acc[e][3]};
            total[e] = reduce_rec<4, 4>(v, lane);
        }
        const int r = r0 + ((lane >> 2) & 3);
        const bool owner = lane < 16 && r < r_end;
        bool store = owner;
        if (a.W > 1) {
            float* const buf_base = partial + (it & 1) * (16 * kFewSumStride);
            if (lane < 16) {
#pragma unroll
                for (int e = 0; e < SETS; ++e) buf_base[wave * kFewSumStride + 16 * e + lane] = total[e];
            }
            __syncthreads();
            store = owner && unit == 0;
            if (store) {
#pragma unroll
                for (int e = 0; e < SETS; ++e) {
                    float t = 0.0f;
                    for (int w = 0; w < a.W; ++w) t += buf_base[(stream * a.W + w) * kFewSumStride + 16 * e + lane];
                    total[e] = t;
                }
            }
        }
        if (store) {
#pragma unroll
            for (int e = 0; e < SETS; ++e)
                if (q + 4 * e < a.batch) store_scalar(a.y, a.y_dtype, (size_t)(q + 4 * e) * out + r, total[e] * (a.L.inv_scale * nrm));
        }
        nrm = nrm_next;
    };
    int it = 0;
    for (; it + D <= a.iters; it += D) {
        trip(D0{}, it);
        if constexpr (D == 2) trip(D1{}, it + 1);
    }
    if (it < a.iters) trip(D0{}, it);
}

template <int SETS, int U>
__global__ __launch_bounds__(1024) void tq_gemv_few_nibble_kernel(FewArgs a) {
    few_nibble_body<SETS, U>(a, (int)blockIdx.x);
}

// Two or three layers of equal width on the same activation rows (q, k, v or gate, up), one launch: the
// workgroups are shared out over the layers by rows.
struct FewGroup {
    FewArgs a[3];
    int first[4];          // layer j owns workgroups first[j] .. first[j + 1] - 1
};
template <int SETS, int U, int TL, bool PRE>
__global__ __launch_bounds__(1024) void tq_gemv_few_group_kernel(FewGroup g) {
    const int b = (int)blockIdx.x;
    const int j = b >= g.first[2] ? 2 : (b >= g.first[1] ? 1 : 0);
    few_body<SETS, U, TL, PRE>(g.a[j], b - g.first[j]);
}
template <int SETS, int U>
__global__ __launch_bounds__(1024) void tq_gemv_few_nibble_group_kernel(FewGroup g) {
    const int b = (int)blockIdx.x;
    const int j = b >= g.first[2] ? 2 : (b >= g.first[1] ? 1 : 0);
    few_nibble_body<SETS, U>(g.a[j], b - g.first[j]);
}

// Rotated, scaled activation rows as fp16 [batch, in] for the calls whose workgroups do not rotate them themselves:
// one wave per 512-column tile, row and rotation (the layers of a group have rotations of their own, a dual-rotation
// layer two).
struct FewRotate {
    const void* x;
    int x_dtype, K;
    uint32_t seed[6], bs[6];
    float scale[6];
    uint16_t* out[6];
};
__global__ __launch_bounds__(64) void tq_rotate_rows_f16_kernel(FewRotate r) {
    const int lane = threadIdx.x, t = blockIdx.y, j = blockIdx.z;
    const int c = blockIdx.x * kTile + lane * 8;
    const TileRaw raw = load_tile_raw(r.x, r.x_dtype, (size_t)t * r.K, c < r.K ? c : 0);
    float v[8];
    rotate_tile(raw, r.x_dtype, c, c < r.K, r.seed[j], r.bs[j], lane, v);
    if (c < r.K) *reinterpret_cast<uint4*>(r.out[j] + (size_t)t * r.K + c) = few_pack8(v, r.scale[j]);
}

bool few_nibble(const LayerView& L) { return L.mode == kDual || L.mode == kPrimaryOnly; }
int few_planes(const LayerView& L) { return L.mode == kDual ? 2 : 1; }

// The shape of a launch: sets of four activation rows, units per wave, waves per row quad, quad streams, rotation
// jobs per wave, whether the rows come rotated.  A unit is a 256-byte segment of a row of a plane (256 columns of the
// byte plane, 512 of a nibble plane; a dual-rotation row has its primary segments, then its residual ones).  Among
// the splits of the row's units over 1 to 16 waves with no more units each than the registers hold (byte plane: 8,
// with two sets 4; nibble planes, twice the activations per unit: 4 and 2), the one that keeps most lanes busy (units
// that exist, waves that exist) or comes within 0.07 of it with nearer to four units per wave: streams short enough
// for layers of a few thousand rows, long enough between two barriers.  A function of the layer's width and mode and the batch
// alone: the order in which a row's products are added depends on it, and a layer must give the same bits in a launch
// of its own and in one it shares.  W == 0: no such split.
struct FewShape { int sets, U, W, S, threads, tl; bool pre; };
FewShape few_shape(const LayerView& L, int batch) {
    FewShape s{};
    const int K = L.in_features;
    const bool nib = few_nibble(L);
    s.sets = (batch + 3) / 4;
    const int max_u = nib ? (s.sets == 2 ? 2 : 4) : (s.sets >= 3 ? 2 : s.sets == 2 ? 4 : kFewMaxU);
    const int units = nib ? few_planes(L) * ((K + 511) / 512) : (K + kSegCols - 1) / kSegCols;
    auto efficiency = [&](int W, int& U) {
        U = (units + W - 1) / W;
        if (U > max_u) return -1.0;
        if (U < 2) U = 2;
        return (double)units / (W * U) * (W * (16 / W)) / 16.0;
    };
    double best = -1.0;
    for (int W = 1; W <= 16; ++W) { int U; best = std::max(best, efficiency(W, U)); }
    // Among the splits within 0.07 of the best: the one nearest four units per wave, then the busier, then the one
    // with fewer waves per row.  (5120 columns: five waves of four segments, three streams, 15 waves, against four
    // waves of five, four streams: the decoder layer at batch 4 142.5 against 148.2 us per call, 115.0 / 116.2 grouped.)
    double chosen = -1.0;
    for (int W = 1; W <= 16; ++W) {
        int U;
        const double eff = efficiency(W, U);
        if (eff < 0.0 || eff < best - 0.07) continue;
        const int d = (U - 4) * (U - 4), d0 = (s.U - 4) * (s.U - 4);
        if (chosen < 0.0 || d < d0 || (d == d0 && eff > chosen + 1e-9)) { chosen = eff; s.U = U; s.W = W; s.S = 16 / W; }
    }
    if (best < 0.0) return s;
    s.threads = s.W * s.S * kWave;
    const int ntiles = (K + kTile - 1) / kTile, waves = s.W * s.S;
    const int per_wave = (batch * ntiles + waves - 1) / waves;
    s.pre = nib || s.sets >= 2 || (size_t)batch * K * 2 > (size_t)kFewImageBytes || per_wave > 6;
    s.tl = per_wave <= 3 ? 3 : 6;
    return s;
}

void few_ranges(FewArgs& a, const FewShape& s, int grid, int batch) {
    const int quads = (a.L.out_features + 3) / 4, ts = grid * s.S;
    a.batch = batch;
    a.W = s.W; a.S = s.S;
    a.w_inv = (256 + s.W - 1) / s.W;
    a.quads_q = quads / ts;
    a.quads_rem = quads % ts;
    a.iters = a.quads_q + (a.quads_rem ? 1 : 0);
    a.ntiles = (a.L.in_features + kTile - 1) / kTile;
    a.nt_inv = 65536 / a.ntiles + 1;       // exact quotients for job numbers below 16 x 6 (at most 64 tiles per row)
    a.planes = few_planes(a.L);
    a.segs = (a.L.in_features + 511) / 512;
}

// GROUP: FewGroup and the kernels that serve several layers; otherwise FewArgs.  NIB: nibble planes.
template <int U, bool GROUP, bool NIB, typename Args>
hipError_t launch_few_u(const Args& a, const FewShape& s, int grid, hipStream_t stream) {
    const dim3 g(grid), b(s.threads);
    if constexpr (NIB) {
        if constexpr (U > 4) return hipErrorInvalidValue;      // few_shape() rules this out
        else if constexpr (GROUP) {
            if (s.sets == 2) {
                if constexpr (U <= 2) hipLaunchKernelGGL((tq_gemv_few_nibble_group_kernel<2, U>), g, b, 0, stream, a);
                else return hipErrorInvalidValue;
            } else hipLaunchKernelGGL((tq_gemv_few_nibble_group_kernel<1, U>), g, b, 0, stream, a);
        } else {
            if (s.sets == 2) {
                if constexpr (U <= 2) hipLaunchKernelGGL((tq_gemv_few_nibble_kernel<2, U>), g, b, 0, stream, a);
                else return hipErrorInvalidValue;
            } else hipLaunchKernelGGL((tq_gemv_few_nibble_kernel<1, U>), g, b, 0, stream, a);
        }
    } else if constexpr (GROUP) {
        if (s.sets == 3) {
            if constexpr (U <= 2) hipLaunchKernelGGL((tq_gemv_few_group_kernel<3, U, 1, true>), g, b, 0, stream, a);
            else return hipErrorInvalidValue;
        }
        else if (s.sets == 2) {
            if constexpr (U <= 4) hipLaunchKernelGGL((tq_gemv_few_group_kernel<2, U, 1, true>), g, b, 0, stream, a);
            else return hipErrorInvalidValue;
        }
        else if (s.pre) hipLaunchKernelGGL((tq_gemv_few_group_kernel<1, U, 1, true>), g, b, 0, stream, a);
        else if (s.tl == 3) hipLaunchKernelGGL((tq_gemv_few_group_kernel<1, U, 3, false>), g, b, 0, stream, a);
        else hipLaunchKernelGGL((tq_gemv_few_group_kernel<1, U, 6, false>), g, b, 0, stream, a);
    } else {
        if (s.sets == 3) {
            if constexpr (U <= 2) hipLaunchKernelGGL((tq_gemv_few_kernel<3, U, 1, true>), g, b, 0, stream, a);
            else return hipErrorInvalidValue;
        }
        else if (s.sets == 2) {
            if constexpr (U <= 4) hipLaunchKernelGGL((tq_gemv_few_kernel<2, U, 1, true>), g, b, 0, stream, a);
            else return hipErrorInvalidValue;
        }
        else if (s.pre) hipLaunchKernelGGL((tq_gemv_few_kernel<1, U, 1, true>), g, b, 0, stream, a);
        else if (s.tl == 3) hipLaunchKernelGGL((tq_gemv_few_kernel<1, U, 3, false>), g, b, 0, stream, a);
        else hipLaunchKernelGGL((tq_gemv_few_kernel<1, U, 6, false>), g, b, 0, stream, a);
    }
    return hipGetLastError();
}

// What the kernels ask of a layer whatever the launch: shared rotation (the byte plane) or nibble planes, centroids
// that fit fp16, blocks of at most 512 columns (a block never leaves the tile a wave rotates), rows of at most 64
// tiles that some split covers.
bool few_layer_ok(const LayerView& L, int batch) {
    if (batch < 2 || batch > (few_nibble(L) ? 8 : kFewMaxBatch)) return false;
    if (!L.fp16_centroids_ok) return false;
    if (L.mode == kSharedLut) { if (!L.packed_combined) return false; }
    else if (few_nibble(L)) { if (!L.packed_primary || (L.mode == kDual && !L.packed_residual)) return false; }
    else return false;
    if (!lanes_supported(L.in_features, L.block_size) || L.block_size > (uint32_t)kTile) return false;
    return L.in_features <= 16 * kFewMaxU * kSegCols && few_shape(L, batch).W > 0;
}
// A stream's share of the plane stays below the 2 GB of its buffer descriptor (one stream per CU at least).
bool few_share_ok(const LayerView& L, int num_cus) {
    const long long cus = num_cus > 0 ? num_cus : 1;
    const long long max_rows = (L.out_features + cus - 1) / cus + 24;
    return (unsigned long long)max_rows * (unsigned long long)L.in_features < (1ull << 31);
}
// Where the rotated rows of a call go when its workgroups do not rotate them: the layer's scratch row (shared-
// rotation rows wider than 16384 columns have one: 2 x in floats = 4 rows of fp16) or a workspace of the caller.
bool few_uses_scratch_row(const LayerView& L, int batch) { return !few_nibble(L) && batch <= 4 && L.xrot_work != nullptr; }
// Every workgroup rotates all the activation rows for itself: about 0.15 us per 512-column tile and row, whatever
// the size of the plane, where the small-batch kernel pays 4 us for its second kernel and loses about 0.06 us per MB
// of plane to its load pattern (same-box comparisons of the two on eleven shapes, weight copies cycled).  Few rows
// of a wide plane go to the small-batch kernel.  (Up to 40 tiles whatever the plane: the layers of a group, large
// and small, should agree on the kernel, or the group is run layer by layer.)  Rows that come rotated cost a kernel
// of their own (4.6 to 4.8 us), which only a plane of some size repays.
bool few_worth_it(const LayerView& L, const FewShape& s, int batch) {
    const int K = L.in_features;
    const long long plane_bytes = (long long)L.out_features * K * (few_nibble(L) ? few_planes(L) : 2) / 2;
    // (five to eight rows, same-box comparisons with the small-batch kernel: 27648 x 5120 35.1 against 42.2 us,
    // 28672 x 8192 47.7 / 59.7, but 14336 x 4096 23.7 / 20.7, 8192 x 8192 23.8 / 21.8, 5120 x 5120 17.1 / 14.3)
    // (nibble planes, two to four rows: 27648 x 5120 34.6 against 40.2 us, 28672 x 8192 47.9 / 62.0, but 8192 x 8192
    // 23.9 / 21.7; five to eight: 28672 x 8192 59.8 / 68.1, but 27648 x 5120, whose 20 units make two per wave of 10
    // waves, 56.2 / 44.4: two sets want a workgroup of 14 waves and more)
    // (nine to twelve rows, three sets, two segments per wave: 28672 x 8192 53.9 / 55.3 against 59.8 / 63.2 us at 9 / 12
    // rows, 65536 x 4096 60.4 / 62.0 against 70.2 / 74.3, but the lm_head of 2048 columns, four waves per row and four
    // streams, 94.1 / 95.5 against 87.9 / 94.1: rows of eight waves and more.  Four sets, 128 registers and ten spilled,
    // took 104-111 us where the small-batch kernel takes 65-103.)
    if (s.sets >= 2 && s.W * s.S < 14) return false;
    if (s.sets == 3 && s.W < 8) return false;
    if (s.pre) return plane_bytes >= ((s.sets >= 2 || few_nibble(L)) ? (96ll << 20) : (64ll << 20));
    const long long jobs = (long long)batch * ((K + kTile - 1) / kTile);
    return jobs <= 40 || jobs * 5 <= 135 + plane_bytes / 500000;           // jobs <= 27 + 0.4 per MB
}

template <typename F>
hipError_t few_dispatch_u(int U, F&& f) {
    switch (U) {
        case 2: return f(std::integral_constant<int, 2>{});
        case 3: return f(std::integral_constant<int, 3>{});
        case 4: return f(std::integral_constant<int, 4>{});
        case 5: return f(std::integral_constant<int, 5>{});
        case 6: return f(std::integral_constant<int, 6>{});
        case 7: return f(std::integral_constant<int, 7>{});
        case 8: return f(std::integral_constant<int, 8>{});
        default: return hipErrorInvalidValue;
    }
}

size_t few_rotated_bytes(const LayerView& L, int batch) {
    return ((size_t)few_planes(L) * batch * L.in_features * 2 + 255) & ~(size_t)255;
}

// The rotation kernel of a call whose rows come rotated: layer j's rows ([plane][batch][in]) go to its scratch row
// or to the j-th part of the workspace; as[j].x is set to them.
hipError_t few_rotate_rows(FewArgs* as, int n, const void* x, int x_dtype, int batch, void* workspace, hipStream_t stream) {
    FewRotate r{};
    r.x = x; r.x_dtype = x_dtype; r.K = as[0].L.in_features;
    const size_t part = few_rotated_bytes(as[0].L, batch);
    const int planes = few_planes(as[0].L);
    for (int j = 0; j < n; ++j) {
        const LayerView& L = as[j].L;
        uint16_t* const base = few_uses_scratch_row(L, batch) ? reinterpret_cast<uint16_t*>(L.xrot_work)
                             : workspace ? reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + j * part) : nullptr;
        if (!base) return hipErrorInvalidValue;
        for (int p = 0; p < planes; ++p) {
            r.seed[j * planes + p] = p ? L.seed_residual : L.seed_primary;
            r.bs[j * planes + p] = L.block_size; r.scale[j * planes + p] = L.inv_sqrt_bs;
            r.out[j * planes + p] = base + (size_t)p * batch * r.K;
        }
        as[j].x = base;
    }
    hipLaunchKernelGGL(tq_rotate_rows_f16_kernel, dim3((r.K + kTile - 1) / kTile, batch, n * planes), dim3(64), 0, stream, r);
    return hipGetLastError();
}

}  // namespace

// Two to twelve rows (nibble planes: eight) of any activation type.
bool gemv_few_supported(const LayerView& L, int batch, int num_cus) {
    if (!few_layer_ok(L, batch) || !few_share_ok(L, num_cus)) return false;
    return few_worth_it(L, few_shape(L, batch), batch);
}

// Bytes of workspace a call needs for its rotated rows (0: none).
size_t gemv_few_workspace_bytes(const LayerView& L, int batch) {
    if (!few_layer_ok(L, batch) || !few_shape(L, batch).pre || few_uses_scratch_row(L, batch)) return 0;
    return few_rotated_bytes(L, batch);
}

hipError_t launch_gemv_few(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                           void* workspace, int num_cus, hipStream_t stream) {
    const FewShape s = few_shape(L, batch);
    FewArgs a{};
    a.L = L; a.x = x; a.y = y; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
    const int quads = (L.out_features + 3) / 4;
    int grid = (quads + s.S - 1) / s.S;
    if (grid > num_cus) grid = num_cus;
    if (grid < 1) grid = 1;
    few_ranges(a, s, grid, batch);
    if (s.pre) {
        const hipError_t e = few_rotate_rows(&a, 1, x, x_dtype, batch, workspace, stream);
        if (e != hipSuccess) return e;
    }
    if (few_nibble(L))
        return few_dispatch_u(s.U, [&](auto Uc) { return launch_few_u<decltype(Uc)::value, false, true>(a, s, grid, stream); });
    return few_dispatch_u(s.U, [&](auto Uc) { return launch_few_u<decltype(Uc)::value, false, false>(a, s, grid, stream); });
}

// Layers that can share a launch: two or three of equal width and mode, each taken by the kernel in a launch of its own.
bool gemv_few_group_supported(const LayerView* Ls, int n, int batch, int num_cus) {
    if (n < 2 || n > 3 || num_cus < n) return false;
    for (int j = 0; j < n; ++j) {
        if (Ls[j].in_features != Ls[0].in_features || Ls[j].mode != Ls[0].mode) return false;
        if (!gemv_few_supported(Ls[j], batch, 1)) return false;      // (1 CU: the strictest bound on a stream's share)
    }
    return true;
}

// workspace: n x gemv_few_workspace_bytes() of the first layer (every layer has rotations of its own).
hipError_t launch_gemv_few_group(const LayerView* Ls, int n, const void* x, int x_dtype, int batch, void* const* ys,
                                 int y_dtype, void* workspace, int num_cus, hipStream_t stream) {
    long long total = 0;
    for (int j = 0; j < n; ++j) total += Ls[j].out_features;
    const FewShape s = few_shape(Ls[0], batch);
    // Workgroups per layer in proportion to its rows.
    int blocks[3] = {0, 0, 0}, used = 0;
    for (int j = 0; j < n; ++j) {
        blocks[j] = (int)((long long)num_cus * Ls[j].out_features / total);
        if (blocks[j] < 1) blocks[j] = 1;
        used += blocks[j];
    }
    for (int j = 0; used < num_cus; j = (j + 1) % n) { ++blocks[j]; ++used; }
    for (int j = 0; used > num_cus; j = (j + 1) % n) if (blocks[j] > 1) { --blocks[j]; --used; }
    FewGroup g{};
    g.first[0] = 0;
    for (int j = 0; j < 3; ++j) g.first[j + 1] = g.first[j] + (j < n ? blocks[j] : 0);
    for (int j = n; j < 3; ++j) { g.first[j] = 1 << 30; g.first[j + 1] = 1 << 30; }     // no workgroup reaches an unused slot
    for (int j = 0; j < n; ++j) {
        FewArgs& a = g.a[j];
        a.L = Ls[j]; a.x = x; a.y = ys[j]; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
        few_ranges(a, s, blocks[j], batch);
    }
    if (s.pre) {
        const hipError_t e = few_rotate_rows(g.a, n, x, x_dtype, batch, workspace, stream);
        if (e != hipSuccess) return e;
    }
    if (few_nibble(Ls[0]))
        return few_dispatch_u(s.U, [&](auto Uc) { return launch_few_u<decltype(Uc)::value, true, true>(g, s, used, stream); });
    return few_dispatch_u(s.U, [&](auto Uc) { return launch_few_u<decltype(Uc)::value, true, false>(g, s, used, stream); });
}

}  // namespace tq
