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
#include "tq_gemv_common.h"
#include <cstdlib>

namespace tq {


// Load 16 consecutive activations and widen them to fp32.
__device__ __forceinline__ void load_run16(const void* x, int x_dtype, size_t elem, float (&v)[16]) {
    if (x_dtype == kF32) {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(x) + elem);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 t = p[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(x) + elem);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4 t = p[i];
            const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (x_dtype == kBF16) {
                    v[8 * i + 2 * j]     = bf16_bits_to_float(w[j] & 0xffffu);
                    v[8 * i + 2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
                } else {
                    v[8 * i + 2 * j]     = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] & 0xffffu));
                    v[8 * i + 2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] >> 16));
                }
            }
        }
    }
}

// The 32 activations of the columns one lane owns (two runs of 16, or 32 consecutive), as fp32.
template <bool SPLIT>
__device__ __forceinline__ void load_owned(const void* x, int x_dtype, size_t row_off, int col_a, int col_b,
                                           bool act_a, bool act_b, float (&xin)[kChunk]) {
    float va[16], vb[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) { va[k] = 0.0f; vb[k] = 0.0f; }
    if (act_a) load_run16(x, x_dtype, row_off + col_a, va);
    if (act_b) load_run16(x, x_dtype, row_off + col_b, vb);
#pragma unroll
    for (int k = 0; k < 16; ++k) { xin[k] = va[k]; xin[16 + k] = vb[k]; }
}

// Rotated activations H (s (.) x) of the columns one lane owns, computed by the wave on its own
// (no LDS, no barrier): used when a workgroup has few row streams, so nothing would be shared.
// Split ownership: the two 16-column runs are transformed as 16 values per lane; a 2048-column
// block additionally pairs the runs in a last stage.  Block sizes up to 2048.
template <bool SPLIT>
__device__ __forceinline__ void rotate_private(const float (&xin)[kChunk], int col_a, int col_b,
                                               uint32_t seed, uint32_t bs, int lane, float (&xt)[kChunk]) {
    if constexpr (SPLIT) {
        float va[16], vb[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            va[k] = xin[k] * sign_of(seed, ((uint32_t)col_a + k) & (bs - 1));
            vb[k] = xin[16 + k] * sign_of(seed, ((uint32_t)col_b + k) & (bs - 1));
        }
        const uint32_t bsr = bs > 1024u ? 1024u : bs;     // stages inside one 1024-column run
        fwht_lanes<16>(va, bsr, lane);
        fwht_lanes<16>(vb, bsr, lane);
        if (bs > 1024u) {                                  // h = 1024: column c pairs with c + 1024
#pragma unroll
            for (int k = 0; k < 16; ++k) { const float p = va[k], q = vb[k]; va[k] = p + q; vb[k] = p - q; }
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) { xt[k] = va[k]; xt[16 + k] = vb[k]; }
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) xt[k] = xin[k] * sign_of(seed, ((uint32_t)col_a + k) & (bs - 1));
        fwht_lane32(xt, bs, lane);
    }
}

// Shared variant for narrow layers (at most 8 tiles = 2 slabs, block sizes up to 512): wave t
// rotates 512-column tile t (8 values per lane), the slabs are handed over one at a time
// through an 8 KB staging image (value k of lane l at float index k*64 + l), and every wave picks
// up the 32 values of its own columns.  `raw` must hold tile `wave`'s activations.
template <bool SPLIT>
__device__ __forceinline__ void rotate_shared(const TileRaw& raw, int x_dtype, int in_features, int W,
                                              uint32_t seed, uint32_t bs, float* stage, int wave, int lane,
                                              int slab, bool act_a, bool act_b, float (&xt)[kChunk]) {
    const int col = wave * kTile + lane * 8;
    const bool mine = wave * kTile < in_features;           // wave-uniform
    float v[8];
    if (mine) rotate_tile(raw, x_dtype, col, col < in_features, seed, bs, lane, v);
    for (int p = 0; p < W; ++p) {
        if (p > 0) __syncthreads();                          // previous slab image has been read
        if (mine && (wave >> 2) == p) {
            float* dst = stage + stage_index<SPLIT>(col & (kSlab - 1));
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j * kWave] = v[j];      // 8 columns stay inside one 16-run
        }
        __syncthreads();
        if (slab == p) {
            const float* src = stage + lane;
#pragma unroll
            for (int k = 0; k < kChunk; ++k)
                xt[k] = ((k < 16) ? act_a : act_b) ? src[k * kWave] : 0.0f;   // idle runs contribute 0
        }
    }
}

template <int MODE, int NB, int R, int MAXT, int NS>
__global__ __launch_bounds__(MAXT) void tq_gemv_kernel(GemvArgs a) {
    constexpr int V = R * NB;                       // sums produced per row group
    __shared__ __align__(16) char smem[kRegionBytes + kPartialBytes + kStageBytes];
    float* partial = reinterpret_cast<float*>(smem + kRegionBytes);   // [2][waves][V]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = blockDim.x >> 6;
    // (no integer division on the device: the waves of a CU share one scalar unit and a division
    // is a few hundred instructions; the host passes the quotients)
    const int stream = (wave * a.w_inv) >> 8;               // wave / a.W
    const int slab = wave - stream * a.W;
    // Shared-rotation mode streams the combined plane (one byte per weight); the other modes
    // stream 16 B from each nibble plane.  See stage_index for the column ownership.
    constexpr bool combined = (MODE == kSharedLut);
    const int col_a = slab * kSlab + (combined ? 16 * lane : 32 * lane);
    const int col_b = combined ? col_a + 1024 : col_a + 16;
    const bool act_a = col_a < a.L.in_features, act_b = col_b < a.L.in_features;
    const uint32_t laneoff = (uint32_t)lane << 2;
    const int out = a.L.out_features;
    const size_t row_bytes = combined ? (size_t)a.L.in_features : ((size_t)a.L.in_features >> 1);
    constexpr bool use_res = (MODE != kPrimaryOnly);

    // Contiguous row range of this stream: rows_q rows, one more for the first rows_rem streams.
    const int gs = (int)blockIdx.x * a.S + stream;
    const int r_begin = gs * a.rows_q + (gs < a.rows_rem ? gs : a.rows_rem);
    const int r_end = r_begin + a.rows_q + (gs < a.rows_rem ? 1 : 0);

    // Idle runs re-read a valid address; their rotated activations are 0.
    // Row bases are wave-uniform (scalar); the lane adds a fixed 32-bit byte offset.
    const uint8_t* pp = combined ? a.L.packed_combined : a.L.packed_primary;
    const uint8_t* pr = combined ? a.L.packed_combined : a.L.packed_residual;
    const uint32_t off_p = combined ? (uint32_t)(act_a ? col_a : 0) : (uint32_t)(act_a ? (col_a >> 1) : 0);
    const uint32_t off_r = combined ? (uint32_t)(act_b ? col_b : 0) : off_p;

    uint4 P[NS][R], Q[NS][R];                 // NS-stage register ring of row groups in flight
    float nrm[NS];                            // norm of the row this lane will store (lanes < V)
    auto fetch = [&](int buf, int r0) {
        if (r0 + R <= r_end) {                               // wave-uniform: a full group, straight-line
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const size_t rb = (size_t)(r0 + i) * row_bytes;
                P[buf][i] = load_stream16(pp + rb + off_p);
                if constexpr (use_res) Q[buf][i] = load_stream16(pr + rb + off_r);
            }
        } else {
#pragma unroll
            for (int i = 0; i < R; ++i) {
                if (r0 + i < r_end) {
                    const size_t rb = (size_t)(r0 + i) * row_bytes;
                    P[buf][i] = load_stream16(pp + rb + off_p);
                    if constexpr (use_res) Q[buf][i] = load_stream16(pr + rb + off_r);
                }
            }
        }
        // The norm travels with its rows so the store at the end of the group never waits on memory.
        const int rn = r0 + (lane % V) / NB;
        nrm[buf] = a.L.norms[rn < out ? rn : out - 1];
    };

    // Prologue.  Everything that has to come from memory is requested up front, the small things
    // first (table values, activations), then the first NS-1 weight groups: loads complete in
    // order, so the prologue only waits for what it needs while the weights keep streaming in.
    constexpr int kEntries = (MODE == kSharedLut) ? 256 : (MODE == kDual ? 32 : 16);
    // (table values are the same for all lanes: scalar loads, which leave the CU's vector memory
    // address unit to the weights)
    typedef const __attribute__((address_space(4))) float cfloat;
    cfloat* const tab = (cfloat*)a.L.tables;
    constexpr bool kEarlyX = (NB == 1 && MODE != kDual);
    const bool shared_rot = (a.S >= 4 && a.L.block_size <= (uint32_t)kTile);      // W <= 2: at most 8 tiles
    TileRaw raw[NB];
    float xt[NB][kChunk];   // rotated activations, kept in registers for the whole kernel
    float xr[NB][kChunk];   // second rotation, dual mode only
    if (shared_rot) {
        const int col = wave * kTile + lane * 8;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            if (col < a.L.in_features) raw[b] = load_tile_raw(a.x, a.x_dtype, (size_t)b * a.L.in_features, col);
    } else if constexpr (kEarlyX) {
        load_owned<combined>(a.x, a.x_dtype, 0, col_a, col_b, act_a, act_b, xt[0]);
    }

#pragma unroll
    for (int u = 0; u < NS - 1; ++u) fetch(u, r_begin + u * R);

    // Decode tables -> LDS, one private column per lane: wave w writes entries 16 w .. 16 w + 15,
    // then 16 (w + nwaves) .., lane l into bytes 4 l .. of each entry's 256.
    {
        float* const dst = reinterpret_cast<float*>(smem) + lane;
        for (int c = wave; c * 16 < kEntries; c += nwaves) {
#pragma unroll
            for (int e = 0; e < 16; ++e) dst[(c * 16 + e) * kWave] = tab[c * 16 + e];
        }
    }

    if (shared_rot) {
        float* stage = reinterpret_cast<float*>(smem + kRegionBytes + kPartialBytes);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b > 0) __syncthreads();
            rotate_shared<combined>(raw[b], a.x_dtype, a.L.in_features, a.W, a.L.seed_primary, a.L.block_size,
                                    stage, wave, lane, slab, act_a, act_b, xt[b]);
            if constexpr (MODE == kDual) {
                __syncthreads();
                rotate_shared<combined>(raw[b], a.x_dtype, a.L.in_features, a.W, a.L.seed_residual, a.L.block_size,
                                        stage, wave, lane, slab, act_a, act_b, xr[b]);
            }
        }
    } else {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if constexpr (!kEarlyX)  // register budget: load late, one batch row at a time
                load_owned<combined>(a.x, a.x_dtype, (size_t)b * a.L.in_features, col_a, col_b, act_a, act_b, xt[b]);
            if (a.pre_rotated) {     // rotated by tq_rotate_row_kernel (one batch row): nothing to do but pick them up
                if constexpr (MODE == kDual)
                    load_owned<combined>(a.x, a.x_dtype, (size_t)a.L.in_features, col_a, col_b, act_a, act_b, xr[b]);
            } else {
                if constexpr (MODE == kDual)
                    rotate_private<combined>(xt[b], col_a, col_b, a.L.seed_residual, a.L.block_size, lane, xr[b]);
                rotate_private<combined>(xt[b], col_a, col_b, a.L.seed_primary, a.L.block_size, lane, xt[b]);
            }
        }
    }
    __syncthreads();                                          // tables visible to every wave

    auto decode_row = [&](int buf, int i, float (&acc)[V]) {
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
    };

    auto consume = [&](int buf, int r0, int it) {
        float acc[V];
        const float row_scale = a.out_scale * nrm[buf];
        if (r0 + R <= r_end) {                               // wave-uniform: a full group, straight-line
#pragma unroll
            for (int i = 0; i < R; ++i) decode_row(buf, i, acc);
        } else {                                             // ragged end of the range: skip missing rows
#pragma unroll
            for (int i = 0; i < R; ++i) {
#pragma unroll
                for (int b = 0; b < NB; ++b) acc[i * NB + b] = 0.0f;
                if (r0 + i < r_end) decode_row(buf, i, acc);
            }
        }
        // Lane l < V now gets the wave total of value l = i*NB + b.
        const float total = reduce_rec<V, 1>(acc, lane);
        const int i = lane / NB, b = lane % NB;
        const int r = r0 + i;
        const bool owner = lane < V && r < r_end;

        if (a.W == 1) {
            if (owner) store_scalar(a.y, a.y_dtype, (size_t)b * out + r,
                                    apply_gate(a.gate, (size_t)b * out + r, total * row_scale));
        } else {
            float* buf_base = partial + (it & 1) * (16 * 16);
            if (lane < V) buf_base[wave * V + lane] = total;
            __syncthreads();
            if (slab == 0 && owner) {
                float t = 0.0f;
                for (int w = 0; w < a.W; ++w) t += buf_base[(stream * a.W + w) * V + lane];
                store_scalar(a.y, a.y_dtype, (size_t)b * out + r, apply_gate(a.gate, (size_t)b * out + r, t * row_scale));
            }
        }
    };

    // Main loop over the register ring (unrolled NS times so the stages are static): group it+NS-1
    // is requested while group it is decoded, which keeps NS-1 groups of loads in flight per wave.
    // The trip count is uniform over the grid; a stream whose range ends early skips the work of
    // the missing rows.
    for (int it0 = 0; it0 < a.iters; it0 += NS) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const int it = it0 + u;
            if (it < a.iters) {
                fetch((u + NS - 1) % NS, r_begin + (it + NS - 1) * R);
                consume(u, r_begin + it * R, it);
            }
        }
    }
}

// H (s (.) x) of one activation row for one or two seeds, fp32, natural column order: out[p * cols + c].
// One wave per 512-column tile (blocks of at most 512 columns).  Rows wider than 16384 columns run one
// workgroup per CU whose waves would otherwise each rotate a slab of the row on their own, the same
// work on every CU, which took a quarter of the kernel's time.
// x_gate (optional, x fp32): the row is silu(x_gate) * x, the activation of a gated MLP block, formed here
// in fp32 with the expression of apply_gate.
__global__ __launch_bounds__(256) void tq_rotate_row_kernel(const void* __restrict__ x, int x_dtype,
                                                            const float* __restrict__ x_gate,
                                                            float* __restrict__ out, int cols, uint32_t seed0,
                                                            uint32_t seed1, uint32_t bs) {
    const int lane = threadIdx.x & (kWave - 1);
    const int tile0 = ((int)blockIdx.x * 4 + (int)(threadIdx.x >> 6)) * kTile;
    if (tile0 >= cols) return;
    const int col = tile0 + lane * 8;
    const bool active = col < cols;
    TileRaw raw = load_tile_raw(x, x_dtype, 0, active ? col : 0);
    if (x_gate) {                                           // wave-uniform; x is fp32 here
        const float4* gp = reinterpret_cast<const float4*>(x_gate + (active ? col : 0));
        const float4 g0 = gp[0], g1 = gp[1];
        const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        uint32_t* w[8] = {&raw.a.x, &raw.a.y, &raw.a.z, &raw.a.w, &raw.b.x, &raw.b.y, &raw.b.z, &raw.b.w};
#pragma unroll
        for (int j = 0; j < 8; ++j)
            *w[j] = __builtin_bit_cast(uint32_t, gv[j] / (1.0f + expf(-gv[j])) * __builtin_bit_cast(float, *w[j]));
    }
    float v[8];
    rotate_tile(raw, x_dtype, col, active, blockIdx.y ? seed1 : seed0, bs, lane, v);
    if (active) {
        float4* dst = reinterpret_cast<float4*>(out + (size_t)blockIdx.y * cols + col);
        dst[0] = make_float4(v[0], v[1], v[2], v[3]);
        dst[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
}

template <int MODE, int NB, int R, int MAXT, int NS>
static hipError_t launch_one(const GemvArgs& a, int grid, int threads, hipStream_t stream) {
    hipLaunchKernelGGL((tq_gemv_kernel<MODE, NB, R, MAXT, NS>), dim3(grid), dim3(threads), 0, stream, a);
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
    // Two workgroups per CU fit (LDS, registers) up to 8 waves each; wider rows run one per CU so
    // the prologue is not repeated in a second round.
    const int max_grid = (a.W > 8) ? num_cus : num_cus * 2;

    int grid = (out + a.S - 1) / a.S;
    if (grid > max_grid) grid = max_grid;
    if (grid < 1) grid = 1;
    const int ts = grid * a.S;                              // row streams
    a.rows_q = out / ts;
    a.rows_rem = out % ts;
    a.w_inv = (256 + a.W - 1) / a.W;                        // (w * w_inv) >> 8 == w / W for w < 16, W <= 16
    const int max_rows = a.rows_q + (a.rows_rem ? 1 : 0);   // longest row range of any stream
    // Four rows per group only where the register budget allows it without spilling.
    int R = (max_rows >= 4 && MAXT <= 512 && NB < 4) ? 4 : (max_rows >= 2 ? 2 : 1);
    if (MODE == kDual && MAXT > 512) R = 1;
    a.iters = (max_rows + R - 1) / R;

    switch (R) {
        case 4: return launch_one<MODE, NB, 4, MAXT, 2>(a, grid, threads, stream);
        case 2: return launch_one<MODE, NB, 2, MAXT, 2>(a, grid, threads, stream);
        default: return launch_one<MODE, NB, 1, MAXT, 2>(a, grid, threads, stream);
    }
}

// One batch row of a layer wider than 16384 columns: rotate it once for the whole grid (if the layer
// has the scratch for it and blocks of at most 512 columns) and hand the kernel the result.
static void pre_rotate(GemvArgs& a, hipStream_t stream) {
    const LayerView& L = a.L;
    if (!L.xrot_work || L.block_size > (uint32_t)kTile || L.in_features <= 8 * kSlab) return;
    const int tiles = (L.in_features + kTile - 1) / kTile;
    hipLaunchKernelGGL(tq_rotate_row_kernel, dim3((tiles + 3) / 4, L.mode == kDual ? 2 : 1), dim3(256), 0, stream,
                       a.x, a.x_dtype, a.x_gate, L.xrot_work, L.in_features, L.seed_primary, L.seed_residual, L.block_size);
    a.x = L.xrot_work;
    a.x_dtype = kF32;
    a.pre_rotated = 1;
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
        a.gate = base.gate ? base.gate + (size_t)done * out : nullptr;
        const int left = batch - done;
        hipError_t e;
        int step = 1;
        if constexpr (MODE == kDual) {
            if (gemv_wide_supported(a.L, num_cus)) e = launch_gemv_wide(a, num_cus, stream);
            else if (W <= 8) e = launch_nb<MODE, 1, 512>(a, num_cus, stream);
            else {
                pre_rotate(a, stream);
                if (a.pre_rotated && gemv_wide_supported(a.L, num_cus, true)) e = launch_gemv_wide(a, num_cus, stream);
                else e = launch_nb<MODE, 1, 1024>(a, num_cus, stream);
            }
        } else {
            if (left >= 4 && W <= 8)      { step = 4; e = launch_nb<MODE, 4, 512>(a, num_cus, stream); }
            else if (left >= 2 && W <= 8) { step = 2; e = launch_nb<MODE, 2, 512>(a, num_cus, stream); }
            else if (gemv_wide_supported(a.L, num_cus)) { step = 1; e = launch_gemv_wide(a, num_cus, stream); }
            else {
                step = 1;
                if (W > 8) pre_rotate(a, stream);
                if (a.pre_rotated && gemv_wide_supported(a.L, num_cus, true)) e = launch_gemv_wide(a, num_cus, stream);
                else e = launch_nb<MODE, 1, 1024>(a, num_cus, stream);
            }
        }
        if (e != hipSuccess) return e;
        done += step;
    }
    return hipSuccess;
}

// silu(x_gate) * x can be formed on the way where the row goes through tq_rotate_row_kernel.
bool gemv_x_gate_supported(const LayerView& L) {
    return L.xrot_work && shape_supported(L.in_features, L.block_size) && L.block_size <= (uint32_t)kTile &&
           L.in_features > 8 * kSlab &&
           (L.mode == kSharedLut || L.mode == kDual || L.mode == kPrimaryOnly);
}

hipError_t launch_gemv(const LayerView& L, const void* x, int x_dtype, int batch,
                       void* y, int y_dtype, int num_cus, hipStream_t stream, const float* gate, const float* x_gate) {
    if (x_gate && (batch != 1 || x_dtype != kF32 || !gemv_x_gate_supported(L))) return hipErrorInvalidValue;
    GemvArgs a{};
    a.L = L;
    a.gate = gate;
    a.x_gate = x_gate;
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
