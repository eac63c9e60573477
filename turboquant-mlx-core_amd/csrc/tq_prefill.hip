// TQ8 prefill: dequantise-into-LDS + fp16 MFMA GEMM for gfx950 (batch >= 16, or >= 33 where the small-batch kernels take the layer; activations of any type).
//
// The reference has no batched-GEMM path: batch is a grid dimension of its per-row-FWHT kernel
// (src/dequantizer.cpp:545-549), so every weight block is inverse-transformed once per batch row.
// Here the activations are rotated once (X~ = H (s (.) X) per block, fp32 butterfly, rounded to
// fp16 after the 1 / sqrt(bs) normalisation) and the layer becomes one dense contraction
//
//   Y[m, n] = norm[n] / sqrt(in) * sum_k X~[m, k] * L[n, k],   L = centroid (sum) of the indices
//
// Workgroup tile 256 (M) x 256 (N), 8 waves as 2 (M) x 4 (N), each wave 128 x 64 built from
// v_mfma_f32_32x32x16_f16.  K advances in 32-column steps.  Activation tiles are copied from
// global memory straight into LDS (three tiles in rotation, requested two steps ahead; the
// rotate kernel stores X~ as ready-made tile images).  Index bytes travel through registers
// (64-column stages, requested four steps ahead), are turned into fp16 through the lane-private
// LDS table and written to one of two weight tiles.  One barrier per step; the two waves of a
// SIMD run the decode and the multiply half of a step in opposite order, which keeps the matrix
// pipe fed during the decodes.
#include "tq_prefill_common.h"

namespace tq {

constexpr int kBM = 256, kBN = 256;
constexpr int kBK = 32;                               // K extent of one LDS tile (one step)
constexpr int kKLoad = 64;                            // K extent of one register stage of index bytes (two steps)
constexpr int kBPitch = (kBK + 8) * 2;                // weight tile: bytes per row (fp16), padded -> 80
constexpr int kBTile = 256 * kBPitch;                 // 20480
constexpr int kATile = 256 * kBK * 2;                 // activation tile image: 256 rows x 64 B, swizzled -> 16384
constexpr int kGemmThreads = 512;
constexpr int kGemmLutBytes = 256 * 256;
constexpr int kBOff = kGemmLutBytes;                  // two weight tiles
constexpr int kAOff = kBOff + 2 * kBTile;             // three activation tiles
constexpr int kGemmSmem = kAOff + 3 * kATile;         // 155648 of the CU's 163840 bytes

struct PrefillArgs {
    const uint16_t* xt;        // rotated activations, fp16 tile images [planes][m_tiles][K/32][16 KB]
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
    // K cut into ranges (blockIdx.y) when the output tiles alone would leave most CUs idle: a range is
    // steps_per_split 32-column steps (even; the last range may be shorter), and every workgroup writes
    // its fp32 products to partial[range][M][N] instead of y (NULL: one range, y written directly).
    int steps_per_split;
    float* partial;
};

// Position of the 16-byte slot that holds columns [8c, 8c+8) of row r inside a 64-byte tile row.
// The XOR spreads the 16 rows a 128-bit LDS read touches at once over all 16 slot phases
// (row & 3 picks the 64-byte quarter of the 256-byte bank line, (row >> 2) & 3 the slot in it).
__device__ __forceinline__ int a_slot(int row, int c) { return c ^ ((row >> 2) & 3); }

// Index bytes of one thread for a 64-column stage: two pieces, one per 32-column step.
template <bool COMBINED> struct PrefillStage { u32x4v b[2]; };
template <> struct PrefillStage<false> { u32x2v b[2]; };

// The global->LDS copies and the index loads below are issued from inline assembly and waited
// for by hand: the memory counter retires in order, every request in the loop is unconditional,
// and the wait before each barrier (at most 4 younger requests outstanding) is therefore exact.
// Letting the compiler place these waits makes every LDS read after a global->LDS copy wait for
// that copy, which serialises the pipeline.
template <int MODE>
__global__ __launch_bounds__(kGemmThreads) void tq_prefill_gemm_kernel(PrefillArgs a) {
    __shared__ __align__(16) char smem[kGemmSmem];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t laneoff = (uint32_t)lane << 2;

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs (id % 8), so the
    // M tiles that share one N tile of weights are given to the same XCD back to back.
    // With K ranges (few tiles) the tiles are numbered densely instead: an XCD would otherwise be handed
    // whole N tiles times all ranges, more workgroups than it has CUs, while others idle.
    const int id = blockIdx.x;
    const int xcd = id & 7, slot = id >> 3;
    const int n_tile = a.partial ? id / a.m_tiles : (slot / a.m_tiles) * 8 + xcd;
    const int m_tile = a.partial ? id % a.m_tiles : slot % a.m_tiles;
    if (n_tile >= a.n_tiles) return;                       // whole workgroup leaves together
    const int m0 = m_tile * kBM, n0 = n_tile * kBN;

    constexpr bool combined = (MODE == kSharedLut);
    constexpr int kPlanes = (MODE == kDual) ? 2 : 1;
    const int T_all = a.K / kBK;                           // 32-column steps of the whole row (even)
    const int t_begin = (int)blockIdx.y * a.steps_per_split;          // this workgroup's K range
    const int T = T_all - t_begin < a.steps_per_split ? T_all - t_begin : a.steps_per_split;   // its steps (even)
    const int G = T / 2;                                   // 64-column index stages

    // Weight loader mapping: thread -> (tile row, 16-column half of a 32-column tile).
    const int lrow = tid >> 1, lh = tid & 1;
    const int b_row = (n0 + lrow < a.N) ? n0 + lrow : a.N - 1;
    const uint32_t b_voff = combined ? (uint32_t)b_row * (uint32_t)a.K + (uint32_t)t_begin * kBK + lh * 16
                                     : (uint32_t)b_row * (uint32_t)(a.K >> 1) + (uint32_t)t_begin * (kBK / 2) + lh * 8;
    // Activation copy: wave w moves bytes [2048 w, 2048 w + 2048) of every 16 KB tile image.
    const uint32_t dma_voff = (uint32_t)wave * 2048 + (uint32_t)lane * 16;
    const uint32_t lds_base = (uint32_t)(uintptr_t)smem;

    // MFMA mapping: 2 x 4 waves, each 128 x 64; waves w and w+4 share a SIMD.
    const int wm = wave >> 2, wn = wave & 3;
    const int a_frag0 = (wm * 128 + (lane & 31)) * 64 + (a_slot(lane & 31, lane >> 5) << 4);        // s = 0
    const int a_frag1 = (wm * 128 + (lane & 31)) * 64 + (a_slot(lane & 31, 2 + (lane >> 5)) << 4);  // s = 1
    const int b_frag = (wn * 64 + (lane & 31)) * kBPitch + (lane >> 5) * 16;

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    using Stage = PrefillStage<combined>;

    for (int plane = 0; plane < kPlanes; ++plane) {
        // (second plane: nothing of the first is in flight, and its table has been read for the last time)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const char* a_tiles = reinterpret_cast<const char*>(a.xt) +
                              (((size_t)plane * a.m_tiles + m_tile) * (size_t)T_all + t_begin) * kATile;
        const uint8_t* w_plane = combined ? a.plane0 : (plane == 0 ? a.plane0 : a.plane1);

        // Activation tile t -> LDS tile `buf`, straight from global memory.
        auto copy_a = [&](int t, int buf) {
            const char* src = a_tiles + (size_t)(t < T ? t : T - 1) * kATile;
            const uint32_t dst = lds_base + kAOff + buf * kATile + wave * 2048;
            asm volatile("s_mov_b32 m0, %0\n\t"
                         "global_load_lds_dwordx4 %1, %2\n\t"
                         "global_load_lds_dwordx4 %1, %2 offset:1024"
                         :: "s"(dst), "v"(dma_voff), "s"(src));
        };
        // Index bytes of stage g -> registers.
        auto load_b = [&](Stage& st, int g) {
            const uint32_t off = b_voff + (uint32_t)(g < G ? g : G - 1) * (combined ? kKLoad : kKLoad / 2);
            if constexpr (combined)
                asm volatile("global_load_dwordx4 %0, %2, %3\n\t"
                             "global_load_dwordx4 %1, %2, %3 offset:32"
                             : "=&v"(st.b[0]), "=&v"(st.b[1]) : "v"(off), "s"(w_plane));
            else
                asm volatile("global_load_dwordx2 %0, %2, %3\n\t"
                             "global_load_dwordx2 %1, %2, %3 offset:16"
                             : "=&v"(st.b[0]), "=&v"(st.b[1]) : "v"(off), "s"(w_plane));
        };

        // Decode half u of a stage into weight tile `buf`.
        auto fill = [&](const Stage& st, int u, int buf) {
            uint32_t rb[8];
            if constexpr (combined) {
                const uint32_t w4[4] = {st.b[u].x, st.b[u].y, st.b[u].z, st.b[u].w};
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t w = w4[d];
                    const uint32_t v0 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w, laneoff, 0));
                    const uint32_t v1 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w, laneoff, 1));
                    const uint32_t v2 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w, laneoff, 2));
                    const uint32_t v3 = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w, laneoff, 3));
                    rb[2 * d] = pack_half2(v0, v1);
                    rb[2 * d + 1] = pack_half2(v2, v3);
                }
            } else {
                const uint32_t w2[2] = {st.b[u].x, st.b[u].y};
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    const uint32_t w = w2[d];
                    const uint32_t ce = w & 0x0F0F0F0Fu, co = (w >> 4) & 0x0F0F0F0Fu;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t ve = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(ce, laneoff, j));
                        const uint32_t vo = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(co, laneoff, j));
                        rb[4 * d + j] = pack_half2(ve, vo);
                    }
                }
            }
            u32x4v* db = reinterpret_cast<u32x4v*>(smem + kBOff + buf * kBTile + lrow * kBPitch + lh * 32);
            const u32x4v t0 = {rb[0], rb[1], rb[2], rb[3]}, t1 = {rb[4], rb[5], rb[6], rb[7]};
            db[0] = t0;
            db[1] = t1;
        };

        Stage S0, S1, S2;
        // Everything requested so far except the 4 youngest requests has arrived.  The stage
        // registers are tied to the statement so no use of them can be scheduled above it.
        auto wait_all_but_4 = [&]() {
            asm volatile("s_waitcnt vmcnt(4)"
                         : "+v"(S0.b[0]), "+v"(S0.b[1]), "+v"(S1.b[0]), "+v"(S1.b[1]), "+v"(S2.b[0]), "+v"(S2.b[1])
                         :: "memory");
        };
        // Step t = 6q + R: multiply activation tile R % 3 with weight tile R % 2, decode step t+1
        // into the other weight tile, request activation tile t+2 and (odd steps) the index stage
        // three ahead of the one whose second half was just decoded.
        // The 8 table reads of decode half h (0/1) of stage half u, and their packing into 4
        // registers of fp16 pairs.
        auto lookup_half = [&](const Stage& st, int u, int h, uint32_t (&lv)[8]) {
            if constexpr (combined) {
                const uint32_t w2[2] = {h == 0 ? st.b[u].x : st.b[u].z, h == 0 ? st.b[u].y : st.b[u].w};
#pragma unroll
                for (int d = 0; d < 2; ++d)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        lv[4 * d + j] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w2[d], laneoff, j));
            } else {
                const uint32_t w = h == 0 ? st.b[u].x : st.b[u].y;
                const uint32_t ce = w & 0x0F0F0F0Fu, co = (w >> 4) & 0x0F0F0F0Fu;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    lv[2 * j] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(ce, laneoff, j));
                    lv[2 * j + 1] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(co, laneoff, j));
                }
            }
        };
        auto pack_half = [&](const uint32_t (&lv)[8], uint32_t* rb) {
#pragma unroll
            for (int q = 0; q < 4; ++q) rb[q] = pack_half2(lv[2 * q], lv[2 * q + 1]);
        };

        // Step t = 6q + R: multiply activation tile R % 3 with weight tile R % 2, decode step t+1
        // into the other weight tile, request activation tile t+2 and (odd steps) the index stage
        // three ahead of the one whose second half was just decoded.  The order below is a hand
        // made software pipeline: every LDS read and every memory request is issued with matrix
        // instructions of the same wave in flight behind it, and the scheduling fences keep the
        // compiler from regrouping it.
        auto step = [&](int t, int abuf, int bbuf, const Stage& st, int u, Stage* reload) {
            const char* As = smem + kAOff + abuf * kATile;
            const char* Bs = smem + kBOff + bbuf * kBTile + b_frag;
            const bool do_fill = t + 1 < T;
            f16x8 fa0[4], fb0[2], fa1[4], fb1[2];
            uint32_t lv[8], rb[8];
            auto mm = [&](int i, const f16x8 (&fa)[4], const f16x8 (&fb)[2]) {
                acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[0], acc[i][0], 0, 0, 0);
                acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[1], acc[i][1], 0, 0, 0);
            };
#pragma unroll
            for (int j = 0; j < 2; ++j) fb0[j] = *reinterpret_cast<const f16x8*>(Bs + j * 32 * kBPitch);
#pragma unroll
            for (int i = 0; i < 4; ++i) fa0[i] = *reinterpret_cast<const f16x8*>(As + a_frag0 + i * 32 * 64);
            if (do_fill) lookup_half(st, u, 0, lv);
            __builtin_amdgcn_sched_barrier(0);
            mm(0, fa0, fb0);
            copy_a(t + 2, (abuf + 2) % 3);
            mm(1, fa0, fb0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < 2; ++j) fb1[j] = *reinterpret_cast<const f16x8*>(Bs + j * 32 * kBPitch + 32);
#pragma unroll
            for (int i = 0; i < 4; ++i) fa1[i] = *reinterpret_cast<const f16x8*>(As + a_frag1 + i * 32 * 64);
            if (do_fill) {
                pack_half(lv, rb);
                lookup_half(st, u, 1, lv);
            }
            __builtin_amdgcn_sched_barrier(0);
            mm(2, fa0, fb0);
            if (reload) load_b(*reload, (t >> 1) + 3);
            mm(3, fa0, fb0);
            __builtin_amdgcn_sched_barrier(0);
            mm(0, fa1, fb1);
            mm(1, fa1, fb1);
            if (do_fill) {
                pack_half(lv, rb + 4);
                u32x4v* db = reinterpret_cast<u32x4v*>(smem + kBOff + (bbuf ^ 1) * kBTile + lrow * kBPitch + lh * 32);
                const u32x4v t0 = {rb[0], rb[1], rb[2], rb[3]}, t1 = {rb[4], rb[5], rb[6], rb[7]};
                db[0] = t0;
                db[1] = t1;
            }
            __builtin_amdgcn_sched_barrier(0);
            mm(2, fa1, fb1);
            mm(3, fa1, fb1);
            wait_all_but_4();
            __syncthreads();
        };

        copy_a(0, 0);
        copy_a(1, 1);
        load_b(S0, 0);
        load_b(S1, 1);
        load_b(S2, 2);
        // The table is built while those requests travel.  Its values come through scalar loads (the
        // same for all lanes; the compiler's waits for vector loads would not know about the requests
        // above): wave w writes entries 32 w .. 32 w + 31, lane l into bytes 4 l .. of each entry's 256.
        {
            constexpr int entries = combined ? 256 : 16;
            typedef const __attribute__((address_space(4))) float cfloat;
            cfloat* const src = (cfloat*)(a.tables + (plane == 0 ? 0 : 16));
            uint32_t* const dst = reinterpret_cast<uint32_t*>(smem) + lane;
            constexpr int per_wave = (entries + 7) / 8;
#pragma unroll
            for (int e = 0; e < per_wave; ++e) {
                const int entry = wave * per_wave + e;
                if (entry < entries) dst[entry * 64] = (uint32_t)float_to_f16_bits(src[entry]) << 16;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(S0.b[0]), "+v"(S0.b[1]), "+v"(S1.b[0]), "+v"(S1.b[1]), "+v"(S2.b[0]), "+v"(S2.b[1])
                     :: "memory");
        __syncthreads();                                   // table and first activation tiles visible
        fill(S0, 0, 0);
        __syncthreads();
        // Whole groups of six steps in the loop (one exit only, so the accumulators stay in place),
        // then the two or four steps that remain.
        int t = 0;
        for (; t + 6 <= T; t += 6) {
            step(t, 0, 0, S0, 1, nullptr);
            step(t + 1, 1, 1, S1, 0, &S0);
            step(t + 2, 2, 0, S1, 1, nullptr);
            step(t + 3, 0, 1, S2, 0, &S1);
            step(t + 4, 1, 0, S2, 1, nullptr);
            step(t + 5, 2, 1, S0, 0, &S2);
        }
        if (t < T) {
            step(t, 0, 0, S0, 1, nullptr);
            step(t + 1, 1, 1, S1, 0, &S0);
        }
        if (t + 2 < T) {
            step(t + 2, 2, 0, S1, 1, nullptr);
            step(t + 3, 0, 1, S2, 0, &S1);
        }
    }
    // No copy into LDS may outlive the loop: after this barrier LDS is free for the epilogue.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // Epilogue: * norm[n] / sqrt(in * bs), convert, store.  Each wave transposes its 128 x 64 tile
    // through a private LDS region so that every store instruction writes whole 128-byte rows;
    // row counts that break the 16-byte alignment of those stores take the element-wise path.
    // (K ranges: the raw fp32 products go to this range's slice of the partial buffer; the sum kernel scales)
    void* const y_out = a.partial ? static_cast<void*>(a.partial + (size_t)blockIdx.y * a.M * a.N) : a.y;
    const int y_type = a.partial ? (int)kF32 : a.y_dtype;
    float scale[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        scale[j] = col < a.N ? (a.partial ? 1.0f : a.out_scale * a.norms[col]) : 0.0f;
    }
    constexpr int kEpiPitch = 144;                                   // 128 data bytes + 16: conflict-light, 16-byte aligned
    char* const stage = smem + wave * (128 * kEpiPitch);
    const int row_base = m0 + wm * 128, col_base = n0 + wn * 64;
    if (y_type != kF32 && (a.N & 7) == 0) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                    const float v = acc[i][j][r] * scale[j];
                    const uint16_t h = y_type == kBF16 ? float_to_bf16_bits(v)
                                                          : __builtin_bit_cast(uint16_t, (_Float16)v);
                    *reinterpret_cast<uint16_t*>(stage + row * kEpiPitch + (j * 32 + (lane & 31)) * 2) = h;
                }
        uint16_t* y = static_cast<uint16_t*>(y_out);
#pragma unroll
        for (int it = 0; it < 16; ++it) {
            const int row = it * 8 + (lane >> 3), piece = lane & 7;
            const u32x4v v = *reinterpret_cast<const u32x4v*>(stage + row * kEpiPitch + piece * 16);
            const int grow = row_base + row, gcol = col_base + piece * 8;
            if (grow < a.M && gcol < a.N) *reinterpret_cast<u32x4v*>(y + (size_t)grow * a.N + gcol) = v;
        }
    } else if (y_type == kF32 && (a.N & 3) == 0) {
        float* y = static_cast<float*>(y_out);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                    *reinterpret_cast<float*>(stage + row * kEpiPitch + (lane & 31) * 4) = acc[i][j][r] * scale[j];
                }
#pragma unroll
            for (int it = 0; it < 16; ++it) {
                const int row = it * 8 + (lane >> 3), piece = lane & 7;
                const u32x4v v = *reinterpret_cast<const u32x4v*>(stage + row * kEpiPitch + piece * 16);
                const int grow = row_base + row, gcol = col_base + j * 32 + piece * 4;
                if (grow < a.M && gcol < a.N) *reinterpret_cast<u32x4v*>(y + (size_t)grow * a.N + gcol) = v;
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = col_base + j * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = row_base + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                    if (col < a.N && row < a.M)
                        store_scalar(y_out, y_type, (size_t)row * a.N + col, acc[i][j][r] * scale[j]);
                }
        }
    }
}

// ---------------------------------------------------------------------------
// Rotate activations [M, K] (f32 / f16 / bf16) -> fp16 tile images: X~ = H (s (.) X) / sqrt(bs) per block,
// stored as [M/256][K/32] images of 256 rows x 64 bytes in the exact byte order the GEMM keeps
// them in LDS (16-byte slots permuted by a_slot), so a tile is one contiguous 16 KB copy.
// One wave per 64 consecutive 32-column chunks of the row-major input (whole blocks: no half-empty wave at the end
// of a row), 32 consecutive columns per lane, fp32 butterfly.  (Measured and not kept: 32 rows x 512 columns per
// workgroup with 1 KB loads and the images written in 1 KB runs through LDS, 21-27 us against 21-26 us for 2048
// rows of 5120 columns and 10.9 against 8.5 us for 512 rows: the kernel is bound by neither its 64-byte accesses
// nor, since the signs come from a table, its arithmetic.)
// PANEL: fragment images for tq_prefill_panel_kernel instead, [M/512][K/16][4 waves][4 row blocks][64 lanes x 16 B]:
// the 8 columns [16 u + 8 g, +8) of row r sit where lane 32 g + r % 32 of wave (r % 128) / 32 expects the
// A operand of its row block (r % 512) / 128 in sub-step u (the first 128 rows of a panel are the first row block of
// all four waves: a call of few rows keeps every SIMD busy with its first blocks).
// ---------------------------------------------------------------------------
template <bool PANEL>
__global__ __launch_bounds__(256) void tq_rotate_f16_kernel(const void* __restrict__ x, int x_dtype,
                                                             uint16_t* __restrict__ out, int rows, int cols,
                                                             int chunks, uint32_t seed, uint32_t bs, float scale) {
    // The signs of one block as +-1.0f, hashed once per workgroup instead of once per value (the hash is two
    // 32-bit multiplications per index): entry (32 j + k) at float index 36 j + k, so that the 16-byte reads
    // of lanes with neighbouring j fall on different banks.
    __shared__ __align__(16) float signs[64 * 36];
    const int tid = threadIdx.x;
    const uint32_t span = bs < 32 ? 32 : bs;                          // (blocks below 32 columns repeat inside a chunk)
    for (uint32_t i = tid; i < span; i += 256) signs[(i >> 5) * 36 + (i & 31)] = sign_of(seed, i & (bs - 1));
    __syncthreads();

    // The (row, 32-column chunk) pairs of the whole input in row-major order, 64 to a wave: whole blocks (a row
    // holds a whole number of them, and 64 chunks are a multiple of every block size up to 2048 columns).
    const int lane = tid & 63;
    const long long c = ((long long)blockIdx.x * 4 + (tid >> 6)) * kWave + lane;
    const bool active = c < (long long)rows * chunks;
    const int row = active ? (int)(c / chunks) : 0;
    const int chunk = active ? (int)(c - (long long)row * chunks) : 0;
    float v[kChunk];
    if (active) {
        load_chunk(x, x_dtype, (size_t)row * cols + (size_t)chunk * kChunk, v);
        const float4* sg = reinterpret_cast<const float4*>(signs + (chunk & (int)((span >> 5) - 1)) * 36);
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const float4 t = sg[q];
            v[4 * q] *= t.x; v[4 * q + 1] *= t.y; v[4 * q + 2] *= t.z; v[4 * q + 3] *= t.w;
        }
    } else {
#pragma unroll
        for (int k = 0; k < kChunk; ++k) v[k] = 0.0f;
    }
    fwht_lane32(v, bs, lane);
    if (active) {
        const int m_tile = row >> 8, r = row & 255;
        uint4* dst = reinterpret_cast<uint4*>(out + (((size_t)m_tile * chunks + chunk) * 256 + r) * kBK);
        // (PANEL: 16-byte units; sub-step 2 chunk + i / 2 of panel row >> 9, block of (wave, row block), lane)
        uint4* pdst = reinterpret_cast<uint4*>(out) + ((((size_t)(row >> 9) * chunks + chunk) * 2 * 4 + ((row >> 5) & 3)) * 4 + ((row >> 7) & 3)) * 64 + (row & 31);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = pack_f16_saturating(v[8 * i + 2 * j] * scale, v[8 * i + 2 * j + 1] * scale);
            if constexpr (PANEL) pdst[(i >> 1) * 1024 + (i & 1) * 32] = make_uint4(w[0], w[1], w[2], w[3]);
            else dst[a_slot(r, i)] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

// Fragment images for blocks of at most 512 columns, the whole call in one launch: a wave takes R consecutive rows
// of one 512-column segment, 8 columns per lane, so a load instruction reads 1 KB of one row (the kernel above
// reads 64 bytes per lane with the lanes 64 bytes apart: every line passes through the CU's cache four times, and
// 2048 rows of 27648 columns took 132 us against 72-99 us here).  R = 8: the 8 rows of a lane's 8 columns are 128
// consecutive bytes of the image (rows r % 32 = 8 j .. 8 j + 7 of lane group g); they change lanes through a
// wave-private piece of LDS so that a store instruction writes eight whole 128-byte lines.  R = 2, for calls
// with few rows (less than two waves of 8 rows per SIMD): the launch is as long as one wave's chain of loads,
// butterflies and stores, so the waves are kept short and store their 2 x 16 bytes themselves.
// planes = 2: both rotations of the dual layout from one read of the activations (images out and out2).
// (The same kernel writing the 256-row tile images of tq_prefill_gemm_kernel was measured and not kept: there a lane of
// tq_rotate_f16_kernel already stores the 64 contiguous bytes of its chunk; 512 x 27648 took 25.5 us instead of 19.8,
// 1024 x 5120 9.4 instead of 10.0.)
constexpr int kRotPitch = 144;                 // bytes of a lane's 8 x 16 B in LDS, padded: 16-byte accesses spread over the banks
template <int R>
__global__ __launch_bounds__(256) void tq_rotate_panel_kernel(const void* __restrict__ x, int x_dtype,
                                                               uint16_t* __restrict__ out, uint16_t* __restrict__ out2,
                                                               int rows, int cols, int segs, int planes,
                                                               uint32_t seed, uint32_t seed2, uint32_t bs, float scale) {
    __shared__ __align__(16) char stage_all[R == 8 ? 4 * kWave * kRotPitch : 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    char* const stage = stage_all + (R == 8 ? wave * (kWave * kRotPitch) : 0);
    const long long task = (long long)blockIdx.x * 4 + wave;           // (row group, segment), segment fastest
    const int rg = (int)(task / segs), seg = (int)(task - (long long)rg * segs);
    const int row0 = rg * R;
    if (row0 >= rows) return;                                          // wave-uniform; no workgroup barrier below
    const int col = seg * 512 + lane * 8;
    const bool active = col < cols;                                    // (the last segment of a width that is no multiple of 512)

    uint4 raw[R][2];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = row0 + r < rows ? row0 + r : rows - 1;
        const size_t e = (size_t)row * cols + (active ? col : 0);
        if (x_dtype == kF32) {
            const uint4* p = reinterpret_cast<const uint4*>(static_cast<const float*>(x) + e);
            raw[r][0] = p[0]; raw[r][1] = p[1];
        } else {
            raw[r][0] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(x) + e);
        }
    }
    const int U_all = cols >> 4;
    const int g_own = seg * 64 + lane;                                 // this lane's 8-column group of the row
    for (int plane = 0; plane < planes; ++plane) {
        const uint32_t sd = plane ? seed2 : seed;
        uint4* const img = reinterpret_cast<uint4*>(plane ? out2 : out);
        float sg[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) sg[j] = active ? sign_of(sd, (uint32_t)(col + j) & (bs - 1)) : 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float v[8];
            if (x_dtype == kF32) {
                const uint32_t w[8] = {raw[r][0].x, raw[r][0].y, raw[r][0].z, raw[r][0].w, raw[r][1].x, raw[r][1].y, raw[r][1].z, raw[r][1].w};
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = __builtin_bit_cast(float, w[j]);
            } else {
                const uint32_t w[4] = {raw[r][0].x, raw[r][0].y, raw[r][0].z, raw[r][0].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (x_dtype == kBF16) {
                        v[2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
                        v[2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
                    } else {
                        v[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] & 0xffffu));
                        v[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[j] >> 16));
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= sg[j];
            fwht_lanes<8>(v, bs, lane);
            uint4 o;
            o.x = pack_f16_saturating(v[0] * scale, v[1] * scale); o.y = pack_f16_saturating(v[2] * scale, v[3] * scale);
            o.z = pack_f16_saturating(v[4] * scale, v[5] * scale); o.w = pack_f16_saturating(v[6] * scale, v[7] * scale);
            if constexpr (R == 8) {
                *reinterpret_cast<uint4*>(stage + lane * kRotPitch + r * 16) = o;
            } else {
                const int row = row0 + r;
                if (active)
                    img[((size_t)(row >> 9) * U_all + (g_own >> 1)) * 1024 + (size_t)(((row >> 5) & 3) * 4 + ((row >> 7) & 3)) * 64 +
                        (row & 31) + (g_own & 1) * 32] = o;
            }
        }
        if constexpr (R == 8) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            // Store instruction i: lane -> (column group 8 i + lane / 8, row lane % 8): eight lanes write one line.
            const int r = lane & 7, row = row0 + r;
            const size_t row_unit = (size_t)(((row >> 5) & 3) * 4 + ((row >> 7) & 3)) * 64 + (row & 31);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int g_in_seg = 8 * i + (lane >> 3);
                const uint4 o = *reinterpret_cast<const uint4*>(stage + g_in_seg * kRotPitch + r * 16);
                const int g = seg * 64 + g_in_seg;                      // 8-column group of the row
                if (g * 8 < cols)
                    img[((size_t)(row >> 9) * U_all + (g >> 1)) * 1024 + row_unit + (g & 1) * 32] = o;
            }
            __builtin_amdgcn_wave_barrier();                           // (the next plane writes the piece again)
        }
    }
}

// Sum of the K ranges: y[m, n] = out_scale * norm[n] * (partial[0][m, n] + partial[1][m, n] + ...), ranges added
// in their order.  One thread per four neighbouring outputs (QUAD: N is a multiple of 4) or per output.
template <bool QUAD>
__global__ __launch_bounds__(256) void tq_prefill_sum_kernel(const float* __restrict__ partial, int splits,
                                                              const float* __restrict__ norms, float out_scale,
                                                              void* __restrict__ y, int y_dtype, int M, int N) {
    const size_t total = (size_t)M * N;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * (QUAD ? 4 : 1);
    if (i >= total) return;
    const int n = (int)(i % (size_t)N);
    if constexpr (QUAD) {
        float4 s = *reinterpret_cast<const float4*>(partial + i);
        for (int k = 1; k < splits; ++k) {
            const float4 v = *reinterpret_cast<const float4*>(partial + (size_t)k * total + i);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        store_scalar(y, y_dtype, i, s.x * (out_scale * norms[n]));          // (the caller's norms need not be 16-byte aligned)
        store_scalar(y, y_dtype, i + 1, s.y * (out_scale * norms[n + 1]));
        store_scalar(y, y_dtype, i + 2, s.z * (out_scale * norms[n + 2]));
        store_scalar(y, y_dtype, i + 3, s.w * (out_scale * norms[n + 3]));
    } else {
        float s = partial[i];
        for (int k = 1; k < splits; ++k) s += partial[(size_t)k * total + i];
        store_scalar(y, y_dtype, i, s * (out_scale * norms[n]));
    }
}

size_t prefill_workspace_bytes(const LayerView& L, int batch) {
    const size_t planes = (L.mode == kDual) ? 2 : 1;
    const size_t m_tiles = ((size_t)batch + kBM - 1) / kBM;            // whole tile images
    return planes * m_tiles * kBM * L.in_features * sizeof(uint16_t);
}

// How a call is cut.  With fewer output tiles than half the CUs (few output rows: the q, o and down projections;
// few tokens) K is cut into ranges so that about one workgroup per CU runs, no range shorter than 32 steps; the
// ranges' fp32 products follow the tile images in the workspace.  capacity: bytes the caller can give
// (fewer ranges are used where the products would not fit).
PrefillPlan prefill_plan(const LayerView& L, int batch, int num_cus, size_t capacity) {
    PrefillPlan p{};
    const int steps = L.in_features / kBK;
    const long long tiles = (long long)((batch + kBM - 1) / kBM) * ((L.out_features + kBN - 1) / kBN);
    p.xt_bytes = (prefill_workspace_bytes(L, batch) + 255) & ~(size_t)255;
    int splits = 1;
    if (tiles * 2 <= num_cus) {
        splits = (int)(num_cus / tiles);
        if (splits > steps / 32) splits = steps / 32;
        if (splits < 1) splits = 1;
    }
    const size_t one = (size_t)batch * L.out_features * sizeof(float);
    for (;; --splits) {
        int per = (steps + splits - 1) / splits;
        per += per & 1;                                               // even: the kernel steps in pairs
        p.steps_per_split = per;
        p.splits = (steps + per - 1) / per;
        p.total_bytes = p.xt_bytes + (p.splits > 1 ? (size_t)p.splits * one : 0);
        if (p.splits == 1 || p.total_bytes <= capacity) break;
    }
    return p;
}

// Largest workspace any call of 16 .. max_batch rows needs (fewer rows can mean more ranges, and the two kernels
// cut differently: every row count at which the choice of kernel or the number of tiles changes is looked at).
size_t prefill_reserve_bytes(const LayerView& L, int max_batch, int num_cus) {
    size_t need = 0;
    auto look = [&](int rows) {
        if (rows < 16 || rows > max_batch) return;
        const size_t n = prefill_panel_supported(L, rows, num_cus, ~(size_t)0) ? prefill_panel_workspace_bytes(L, rows, num_cus, ~(size_t)0)
                                                                             : prefill_plan(L, rows, num_cus, ~(size_t)0).total_bytes;
        if (n > need) need = n;
    };
    look(16); look(kSkinnyMaxRows); look(kSkinnyMaxRows + 1); look(128); look(129);
    for (int rows = kBM; rows < max_batch + kBM; rows += kBM) { look(rows); look(rows + 1); }
    look(max_batch);
    return need;
}

bool prefill_supported(const LayerView& L, int x_dtype, int batch) {
    if (batch < 16) return false;                             // (fp32 activations too: the fp16 operands keep 1e-3)
    if (L.mode != kSharedLut && L.mode != kDual && L.mode != kPrimaryOnly) return false;
    if (!L.fp16_centroids_ok) return false;                   // decoded weights are kept in fp16
    if (!lanes_supported(L.in_features, L.block_size)) return false;
    // (the kernel addresses the index plane with 32-bit byte offsets)
    if ((unsigned long long)L.out_features * (unsigned long long)L.in_features >= (1ull << 32)) return false;
    return L.in_features % kKLoad == 0;
}

// Rotated activations of `batch` rows as fp16 tile images in `workspace` (both rotations for dual mode).
hipError_t launch_rotate_tiles(const LayerView& L, const void* x, int x_dtype, int batch, void* workspace,
                               hipStream_t stream, bool panel) {
    const int K = L.in_features, M = batch;
    uint16_t* xt = static_cast<uint16_t*>(workspace);
    const int chunks = K / kChunk;
    const dim3 rgrid((unsigned)(((long long)M * chunks + 4 * kWave - 1) / (4 * kWave)));   // 256 chunks per workgroup
    const int tile_m = panel ? kPanelM : kBM;                      // rows of one image
    uint16_t* const xt2 = xt + (size_t)((M + tile_m - 1) / tile_m) * tile_m * K;
    if (panel && L.block_size <= 512) {
        const int segs = (K + 511) / 512;
        const int planes = L.mode == kDual ? 2 : 1;
        const long long tasks8 = (long long)((M + 7) / 8) * segs;
        if (tasks8 >= 2048) {
            hipLaunchKernelGGL(tq_rotate_panel_kernel<8>, dim3((unsigned)((tasks8 + 3) / 4)), dim3(256), 0, stream, x, x_dtype,
                               xt, xt2, M, K, segs, planes, L.seed_primary, L.seed_residual, L.block_size, L.inv_sqrt_bs);
        } else {
            const long long tasks2 = (long long)((M + 1) / 2) * segs;
            hipLaunchKernelGGL(tq_rotate_panel_kernel<2>, dim3((unsigned)((tasks2 + 3) / 4)), dim3(256), 0, stream, x, x_dtype,
                               xt, xt2, M, K, segs, planes, L.seed_primary, L.seed_residual, L.block_size, L.inv_sqrt_bs);
        }
        return hipGetLastError();
    }
    if (panel) {
        hipLaunchKernelGGL(tq_rotate_f16_kernel<true>, rgrid, dim3(256), 0, stream, x, x_dtype, xt, M, K, chunks,
                           L.seed_primary, L.block_size, L.inv_sqrt_bs);
        if (L.mode == kDual)
            hipLaunchKernelGGL(tq_rotate_f16_kernel<true>, rgrid, dim3(256), 0, stream, x, x_dtype, xt2, M, K, chunks,
                               L.seed_residual, L.block_size, L.inv_sqrt_bs);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(tq_rotate_f16_kernel<false>, rgrid, dim3(256), 0, stream, x, x_dtype, xt, M, K, chunks,
                       L.seed_primary, L.block_size, L.inv_sqrt_bs);
    if (L.mode == kDual)
        hipLaunchKernelGGL(tq_rotate_f16_kernel<false>, rgrid, dim3(256), 0, stream, x, x_dtype, xt2, M, K, chunks,
                           L.seed_residual, L.block_size, L.inv_sqrt_bs);
    return hipGetLastError();
}

hipError_t launch_prefill(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                          void* workspace, const PrefillPlan& plan, hipStream_t stream) {
    const int K = L.in_features, N = L.out_features, M = batch;
    uint16_t* xt = static_cast<uint16_t*>(workspace);
    hipError_t e = launch_rotate_tiles(L, x, x_dtype, batch, workspace, stream);
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
    a.out_scale = L.inv_scale;                          // (1 / sqrt(bs) is in the rotated activations)
    a.steps_per_split = plan.steps_per_split;
    a.partial = plan.splits > 1 ? reinterpret_cast<float*>(static_cast<char*>(workspace) + plan.xt_bytes) : nullptr;
    const int n_groups = (a.n_tiles + 7) / 8;
    // (x: tiles, in XCD-aware order or, with K ranges, densely numbered; y: K ranges)
    const dim3 grid((unsigned)(plan.splits > 1 ? a.n_tiles * a.m_tiles : n_groups * 8 * a.m_tiles), (unsigned)plan.splits);
    switch (L.mode) {
        case kSharedLut:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kSharedLut>, grid, dim3(kGemmThreads), 0, stream, a); break;
        case kDual:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kDual>, grid, dim3(kGemmThreads), 0, stream, a); break;
        default:
            hipLaunchKernelGGL(tq_prefill_gemm_kernel<kPrimaryOnly>, grid, dim3(kGemmThreads), 0, stream, a); break;
    }
    e = hipGetLastError();
    if (e != hipSuccess || plan.splits == 1) return e;
    const size_t total = (size_t)M * N;
    if ((N & 3) == 0)
        hipLaunchKernelGGL(tq_prefill_sum_kernel<true>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream,
                           a.partial, plan.splits, L.norms, L.inv_scale, y, y_dtype, M, N);
    else
        hipLaunchKernelGGL(tq_prefill_sum_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                           a.partial, plan.splits, L.norms, L.inv_scale, y, y_dtype, M, N);
    return hipGetLastError();
}

}  // namespace tq
