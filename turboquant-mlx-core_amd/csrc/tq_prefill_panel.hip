// TQ8 prefill, many tokens: 512 x 128 workgroup tiles, one wave per SIMD, for gfx950.
//
// Same contraction as tq_prefill.hip (Y = X~ L^T, fp16 operands of v_mfma_f32_32x32x16_f16, fp32 accumulation), cut
// differently.  A workgroup is four waves, one per SIMD; wave w owns rows [128 w, 128 w + 128) of a 512-row panel
// of activations and all 128 weight rows of the tile: a 128 x 128 accumulator tile (256 registers, the wave's
// AccVGPRs).  What this buys:
//   * the rotated activations never touch LDS.  tq_rotate_f16_kernel<PANEL> stores them as fragment images, i.e.
//     in the exact register order of the MFMA A operand, so a wave fetches its operands with contiguous 1 KB
//     global loads (four per 16-column sub-step) into a ring of eight sub-steps, seven sub-steps ahead;
//   * a tile of weights (128 rows x 64 columns) is decoded once per workgroup and 512 rows of activations, through
//     the lane-private LDS table, into one of two fp16 tiles in LDS, a quarter per sub-step;
//   * per 64-column tile a wave issues 64 matrix instructions against 16 fragment reads, 16-32 table reads and 4
//     tile writes, and the workgroup meets at ONE barrier, placed three quarters into the tile so that the first
//     fragments of the next tile are read while the last 16 matrix instructions of this one run;
//   * a single wave per SIMD has nobody to fill the matrix pipe while it issues other instructions, so the side
//     work goes out two or three instructions at a time behind each matrix instruction (one scheduling fence per
//     matrix instruction), and the memory waits are the compiler's exact counts: every request in the loop is an
//     ordinary load it can see;
//   * the weights are the first MFMA operand, so a lane's 16 results are 4 x 4 consecutive output columns of one
//     token: the epilogue needs no transposition of single values (16-bit outputs are gathered into whole rows
//     through LDS as packed pairs, fp32 outputs go out as 16-byte stores), and all stores go through a buffer
//     descriptor that drops what lies past the output instead of branching;
//   * the tiles left over after the last full round of the chip (at most half a round) are cut into K ranges so
//     that the last round is a half or a quarter of a tile long; a second kernel adds their fp32 products.
// The reference has no batched path at all (src/dequantizer.cpp:545-549: batch is a grid dimension of its
// per-row kernel).
#include "tq_prefill_common.h"

#include <type_traits>

// Measurement builds (make ablations; bench.py --prefill-ablations): -DTQ_PANEL_ABLATE=<mask> compiles parts of the
// main loop out.  Results are then wrong; what is compared is SQ_WAVE_CYCLES of the kernel, not its time (the clock
// of the chip follows the power drawn, which follows the operand values).
//   1 no activation loads in the loop    2 no decode (table reads, packs, tile writes)    4 no barrier
//   8 no index-byte loads in the loop   16 no weight-fragment reads                      32 no epilogue
#ifndef TQ_PANEL_ABLATE
#define TQ_PANEL_ABLATE 0
#endif
#define PANEL_ABL TQ_PANEL_ABLATE
namespace tq {

namespace {

constexpr int kPN = 128;                          // weight rows (output columns) of a workgroup tile
constexpr int kPThreads = 256;
constexpr int kSubK = 16;                         // columns of one sub-step (the K extent of one matrix instruction)
constexpr int kTileK = 64;                        // columns of one weight tile in LDS: four sub-steps
constexpr int kWPitch = kTileK * 2 + 16;          // bytes per weight-tile row: 64 fp16 + one 16-byte slot -> 144
constexpr int kWTile = kPN * kWPitch;             // 18432
constexpr int kPLut = 256 * 256;                  // lane-private decode table: 256 entries x 64 lanes x 4 bytes
constexpr int kPSmem = kPLut + 2 * kWTile;        // 102400
constexpr int kSubImage = kPanelM * kSubK * 2;    // fragment image of one sub-step of a panel: 16384 bytes
constexpr int kUnroll = 16;                       // sub-steps per loop iteration: K must be a multiple of 256

struct PanelArgs {
    const char* xt;            // fragment images [planes][panels][K / 16][16 KB]
    const uint8_t* plane0;     // combined bytes [N, K] (shared rotation) or primary nibbles [N, K / 2]
    const uint8_t* plane1;     // residual nibbles [N, K / 2] (dual rotation) or NULL
    const float* tables;       // 256 floats (build_tables in tq_linear_c.cpp)
    const float* norms;
    void* y;
    int y_dtype;
    int M, N, K;
    int panels, n_tiles, n_per_xcd;
    float out_scale;
    // The last `tail_tiles` tiles (in panel-major order; all tiles where the call has fewer tiles than the chip has
    // CUs) are cut into `parts` parts: K ranges of part_subs sub-steps, with the dual rotation one per (plane, K
    // range), plane = part & 1.  They are run by the workgroups [first_part_wg, first_part_wg + tail_tiles * parts),
    // which write their raw fp32 products to partial[(tile, part)][512][128]; tq_prefill_panel_sum_kernel adds the
    // parts.  tail_tiles == 0: no such tiles.
    int tail_tiles, parts, part_subs, first_part_wg;
    float* partial;
};

// Waits for this wave's LDS traffic, then the workgroup barrier.  Written out because __syncthreads() also
// waits for every global load in flight, and the activation ring lives on loads that stay in flight.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <bool COMBINED> struct TileBytes { u32x4v v[2]; };     // index bytes of one thread for one weight tile
template <> struct TileBytes<false> { u32x4v v[1]; };

}  // namespace

// NBLK: row blocks of 32 tokens per wave.  4: whole panels.  1..3: a call of at most 128 NBLK rows (one panel, of
// which the first NBLK blocks of every wave hold tokens: rows 128 i + 32 w + l are block i of wave w); the matrix
// instructions, activation loads and stores of the other blocks are not compiled, the decode of the weight tile,
// which the four waves share, is the same.
// KG = 2 (one row block per wave, whole tiles of a width that is a multiple of 512 columns): eight waves, two per
// SIMD.  Waves 4..7 are a second group that walks the second half of the sub-steps with tile buffers of its own
// and hands its products to the first group through LDS at the end: with one block of matrix instructions per
// sub-step a lone wave per SIMD spends its time waiting for its own table reads, and a second wave fills the gaps.
// Both groups run the same number of sub-steps, so they meet at every barrier.
template <int MODE, int NBLK, int KG = 1>
__global__ __launch_bounds__(kPThreads * KG) void tq_prefill_panel_kernel(PanelArgs a) {
    static_assert(KG == 1 || (KG == 2 && NBLK == 1), "a second wave group: one row block per wave");
    constexpr int kExchange = 4 * 64 * 272;            // past the epilogue's stage: the second group's products
    __shared__ __align__(16) char smem[KG == 2 ? (kPLut + 4 * kWTile) : kPSmem];
    static_assert(KG == 1 || kExchange + 4 * 64 * 64 * 4 <= kPLut + 4 * kWTile, "exchange area inside the workgroup's LDS");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);          // wave of its group
    const int kg = KG == 2 ? __builtin_amdgcn_readfirstlane(tid >> 8) : 0;    // wave group
    const uint32_t laneoff = (uint32_t)lane << 2;

    // Workgroup ids go round the XCDs (id % 8).  The workgroups an XCD runs side by side share a panel of
    // activations (the big operand: 512 x K fp16 per tile against 128 x K bytes of indices), so its L2
    // fetches the panel once for all of them; each takes another tile of weights.
    constexpr bool combined = (MODE == kSharedLut);
    constexpr int kPlanes = (MODE == kDual) ? 2 : 1;
    const int U_all = a.K / kSubK;                         // sub-steps of a row (a multiple of kUnroll)
    const int id = blockIdx.x;
    int panel, n_tile, part = -1, part_slot = 0;            // part_slot: index of the part's fp32 product
    int u_begin = 0, u_end = U_all, plane_begin = 0, plane_end = kPlanes;
    if (id < a.first_part_wg) {
        const int xcd = id & 7, slot = id >> 3;
        panel = slot / a.n_per_xcd;
        n_tile = (slot - panel * a.n_per_xcd) * 8 + xcd;
        if (n_tile >= a.n_tiles) return;                   // whole workgroup leaves together
        if (panel * a.n_tiles + n_tile >= a.panels * a.n_tiles - a.tail_tiles) return;     // a tail tile: run in parts
    } else {
        // Workgroup ids go round the XCDs: XCD x takes the x-th eighth of the (part, tile) pairs in part-major
        // order, so that the workgroups it runs side by side walk the same K range of the same panel and its L2
        // fetches that range of the activations once.
        const int k0 = id - a.first_part_wg, units = a.tail_tiles * a.parts;
        const int x = k0 & 7, per = units >> 3, extra = units & 7;
        const int k = x * per + (x < extra ? x : extra) + (k0 >> 3);
        part = k / a.tail_tiles;
        const int part_tile = k - part * a.tail_tiles;
        part_slot = part_tile * a.parts + part;
        const int t = a.panels * a.n_tiles - a.tail_tiles + part_tile;
        panel = t / a.n_tiles;
        n_tile = t - panel * a.n_tiles;
        int range = part;
        if constexpr (MODE == kDual) {
            plane_begin = part & 1;
            plane_end = plane_begin + 1;
            range = part >> 1;
        }
        u_begin = range * a.part_subs;
        u_end = u_begin + a.part_subs < U_all ? u_begin + a.part_subs : U_all;
    }
    if constexpr (KG == 2) {                              // (the host sends only whole tiles of 32 k sub-steps here)
        const int half = (u_end - u_begin) >> 1;
        if (kg == 0) u_end = u_begin + half; else u_begin += half;
    }
    const int m0 = panel * kPanelM, n0 = n_tile * kPN;
    const int tiles_end = u_end / 4;                       // 64-column weight tiles end here

    // Decode mapping: thread -> (tile row, 32-column half).  The 16 lanes that write a 128-bit piece together
    // hold 16 consecutive rows, which the 144-byte pitch spreads over all 16 slot phases.
    const int drow = wave * 32 + (lane & 31), dh = lane >> 5;
    const int b_row = (n0 + drow < a.N) ? n0 + drow : a.N - 1;
    char* const wdst = smem + kPLut + kg * (2 * kWTile) + drow * kWPitch + dh * 64;
    // Fragment reads: lane -> (row lane % 32 of a 32-row block, 8 columns (lane / 32) of the sub-step).
    const char* const bfrag = smem + kPLut + kg * (2 * kWTile) + (lane & 31) * kWPitch + (lane >> 5) * 16;

    f32x16 acc[NBLK][4];
#pragma unroll
    for (int i = 0; i < NBLK; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    using Bytes = TileBytes<combined>;

    for (int plane = plane_begin; plane < plane_end; ++plane) {
        if (plane > plane_begin) lds_barrier();            // the first plane's table and tiles are done with
        const char* const ap = a.xt + ((size_t)(plane * a.panels + panel) * U_all) * kSubImage + wave * 4096 + lane * 16;
        const uint8_t* const bp = combined ? a.plane0 + (size_t)b_row * a.K + dh * 32
                                           : (plane == 0 ? a.plane0 : a.plane1) + (size_t)b_row * (a.K >> 1) + dh * 16;

        // One row block per wave and no token among this wave's 32 rows: the wave re-reads the first image it was
        // given (one KB, in L1 after the first read) instead of pulling K x 64 bytes of padding through L2.  Its
        // products are never stored.
        const size_t a_step = (NBLK == 1 && m0 + wave * 32 >= a.M) ? 0 : (size_t)kSubImage;
        f16x8 A[8][NBLK];                                  // ring of eight sub-steps of this wave's 32 NBLK rows
        f16x8 Bf[2][4];                                    // weight fragments of the current and the next sub-step
        Bytes By[4];                                       // ring of four tiles of index bytes

        auto load_a = [&](auto Sc, int u) {
            constexpr int s = decltype(Sc)::value;
            const char* p = ap + (size_t)(u < u_end ? u : u_end - 1) * a_step;
#pragma unroll
            for (int i = 0; i < NBLK; ++i) A[s][i] = *reinterpret_cast<const f16x8*>(p + i * 1024);
        };
        auto load_bytes = [&](auto Sc, int tile) {
            constexpr int s = decltype(Sc)::value;
            const uint8_t* p = bp + (size_t)(tile < tiles_end ? tile : tiles_end - 1) * (combined ? kTileK : kTileK / 2);
            By[s].v[0] = *reinterpret_cast<const u32x4v*>(p);
            if constexpr (combined) By[s].v[1] = *reinterpret_cast<const u32x4v*>(p + 16);
        };
        // Quarter q of a tile for this thread: 8 columns.  lookups() issues the table reads, finish() packs and
        // writes the 16 bytes of fp16.
        auto lookups = [&](auto Sc, auto Qc, uint32_t (&lv)[8]) {
            constexpr int s = decltype(Sc)::value, q = decltype(Qc)::value;
            if constexpr (combined) {
                const u32x4v& src = By[s].v[q >> 1];
                const uint32_t w0 = (q & 1) ? src.z : src.x, w1 = (q & 1) ? src.w : src.y;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    lv[j] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w0, laneoff, j));
                    lv[4 + j] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w1, laneoff, j));
                }
            } else {
                const uint32_t w = By[s].v[0][q];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    lv[j] = *reinterpret_cast<const uint32_t*>(smem + gemm_entry_addr(w, laneoff, j));
            }
        };
        auto finish = [&](auto Qc, int buf, const uint32_t (&lv)[8]) {
            constexpr int q = decltype(Qc)::value;
            u32x4v o;
            if constexpr (combined) {
                o.x = pack_half2(lv[0], lv[1]); o.y = pack_half2(lv[2], lv[3]);
                o.z = pack_half2(lv[4], lv[5]); o.w = pack_half2(lv[6], lv[7]);
            } else {
                o.x = lv[0]; o.y = lv[1]; o.z = lv[2]; o.w = lv[3];     // a byte-pair entry is two fp16 already
            }
            *reinterpret_cast<u32x4v*>(wdst + buf * kWTile + q * 16) = o;
        };
        auto read_frags = [&](auto Sc, int buf, int ks) {
            constexpr int s = decltype(Sc)::value;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                Bf[s][j] = *reinterpret_cast<const f16x8*>(bfrag + buf * kWTile + j * 32 * kWPitch + ks * 32);
        };

        // Requests first: index bytes of the first four tiles, activations of the first seven sub-steps.
        const int t_begin = u_begin >> 2;
        load_bytes(std::integral_constant<int, 0>{}, t_begin);
        load_bytes(std::integral_constant<int, 1>{}, t_begin + 1);
        load_bytes(std::integral_constant<int, 2>{}, t_begin + 2);
        load_bytes(std::integral_constant<int, 3>{}, t_begin + 3);
        load_a(std::integral_constant<int, 0>{}, u_begin);
        load_a(std::integral_constant<int, 1>{}, u_begin + 1);
        load_a(std::integral_constant<int, 2>{}, u_begin + 2);
        load_a(std::integral_constant<int, 3>{}, u_begin + 3);
        load_a(std::integral_constant<int, 4>{}, u_begin + 4);
        load_a(std::integral_constant<int, 5>{}, u_begin + 5);
        load_a(std::integral_constant<int, 6>{}, u_begin + 6);

        // The table, while those travel: wave w writes entries 64 w .. 64 w + 63, lane l into bytes 4 l .. of each
        // entry's 256.  Values come through scalar loads.  Shared rotation: entry b = fp16(lut[b]) in the upper half.
        // Nibble planes: entry b = the fp16 centroids of both nibbles of byte b (low nibble = even column).
        {
            typedef const __attribute__((address_space(4))) float cfloat;
            cfloat* const src = (cfloat*)(a.tables + (plane == 0 ? 0 : 16));
            uint32_t* const dst = reinterpret_cast<uint32_t*>(smem) + lane;
#pragma unroll 8
            for (int e = 0; e < 64 / KG; ++e) {
                const int entry = (kg * 4 + wave) * (64 / KG) + e;
                uint32_t v;
                if constexpr (combined) v = (uint32_t)float_to_f16_bits(src[entry]) << 16;
                else v = (uint32_t)float_to_f16_bits(src[entry & 15]) | ((uint32_t)float_to_f16_bits(src[entry >> 4]) << 16);
                dst[entry * 64] = v;
            }
        }
        lds_barrier();
        // Tile 0 and the first quarter of tile 1, then the first fragments.
        {
            uint32_t lv[8];
            lookups(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, lv);
            finish(std::integral_constant<int, 0>{}, 0, lv);
            lookups(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, lv);
            finish(std::integral_constant<int, 1>{}, 0, lv);
            lookups(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{}, lv);
            finish(std::integral_constant<int, 2>{}, 0, lv);
            lookups(std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{}, lv);
            finish(std::integral_constant<int, 3>{}, 0, lv);
            lookups(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, lv);
            finish(std::integral_constant<int, 0>{}, 1, lv);
        }
        load_bytes(std::integral_constant<int, 0>{}, t_begin + 4);
        lds_barrier();
        read_frags(std::integral_constant<int, 0>{}, 0, 0);

        // Sub-step u = ub + U.  Its operands: A[U % 8] (requested seven sub-steps ago) and Bf[U % 2] (read during
        // the previous sub-step).  Beside its 16 matrix instructions it reads the fragments of sub-step u + 1,
        // decodes quarter (u + 1) % 4 of tile (u + 1) / 4 + 1, requests the activations of sub-step u + 7 into the
        // slot sub-step u - 1 left, and, after the last quarter of a tile, the index bytes of the tile four further.
        // The barrier at the top of sub-steps u % 4 == 3 separates the writes of tile (u + 1) / 4 from its reads
        // and the reads of tile u / 4 from the writes that overwrite it (which begin in this very sub-step).
        auto sub = [&](auto Uc, int ub) {
            constexpr int U = decltype(Uc)::value;
            constexpr int q = (U + 1) % 4;
            constexpr int dtile = (U + 1) / 4 + 1;                 // relative to tile ub / 4 (ub / 4 is a multiple of 4)
            constexpr int fbuf = ((U + 1) / 4) % 2, fks = (U + 1) % 4;
            constexpr int sa = U % 8, san = (U + 7) % 8, sb = U % 2, sbn = (U + 1) % 2, sby = dtile % 4;
            if constexpr (U % 4 == 3 && !(PANEL_ABL & 4)) lds_barrier();
            // This thread's index bytes of the quarter, the table addresses, the table values, the packed result.
            uint32_t w0, w1 = 0, ad[8], lv[8];
            u32x4v o;
            if constexpr (combined) {
                const u32x4v& src = By[sby].v[q >> 1];
                w0 = (q & 1) ? src.z : src.x;
                w1 = (q & 1) ? src.w : src.y;
            } else {
                w0 = By[sby].v[0][q];
            }
            const int un = ub + U + 7;
            const char* const pa = ap + (size_t)(un < u_end ? un : u_end - 1) * a_step;
            // One matrix instruction, then the k-th share of the side work, fenced: a single wave per SIMD has
            // nobody to fill the matrix pipe while it issues a run of other instructions, so they go out two or
            // three at a time in the shadow of the instruction before them.
            auto slot = [&](auto Kc) {
                constexpr int k = decltype(Kc)::value;
                constexpr int i = k >> 2, j = k & 3;
                // (weights as the first operand: a lane's 16 results are then 4 x 4 consecutive output columns of
                // one token, which the epilogue stores without a transposition)
                if constexpr (i < NBLK)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Bf[sb][j], A[sa][i], acc[i][j], 0, 0, 0);
                if constexpr (k < 4 && !(PANEL_ABL & 16))
                    Bf[sbn][k] = *reinterpret_cast<const f16x8*>(bfrag + fbuf * kWTile + k * 32 * kWPitch + fks * 32);
                if constexpr (!(PANEL_ABL & 2)) {
                    if constexpr (combined) {
                        // addresses in even slots 0..6, reads in odd slots 1..7, packs in 9..12, write in 13
                        if constexpr (k < 8 && (k & 1) == 0) {
                            ad[k] = gemm_entry_addr(k < 4 ? w0 : w1, laneoff, k & 3);
                            ad[k + 1] = gemm_entry_addr(k < 4 ? w0 : w1, laneoff, (k & 3) + 1);
                        }
                        if constexpr (k < 8 && (k & 1) == 1) {
                            lv[k - 1] = *reinterpret_cast<const uint32_t*>(smem + ad[k - 1]);
                            lv[k] = *reinterpret_cast<const uint32_t*>(smem + ad[k]);
                        }
                        if constexpr (k == 9) o.x = pack_half2(lv[0], lv[1]);
                        if constexpr (k == 10) o.y = pack_half2(lv[2], lv[3]);
                        if constexpr (k == 11) o.z = pack_half2(lv[4], lv[5]);
                        if constexpr (k == 12) o.w = pack_half2(lv[6], lv[7]);
                        if constexpr (k == 13) *reinterpret_cast<u32x4v*>(wdst + (dtile % 2) * kWTile + q * 16) = o;
                    } else {
                        // a byte-pair entry is two fp16 already
                        if constexpr (k == 4 || k == 6) {
                            ad[k - 4] = gemm_entry_addr(w0, laneoff, k - 4);
                            ad[k - 3] = gemm_entry_addr(w0, laneoff, k - 3);
                        }
                        if constexpr (k == 5 || k == 7) {
                            lv[k - 5] = *reinterpret_cast<const uint32_t*>(smem + ad[k - 5]);
                            lv[k - 4] = *reinterpret_cast<const uint32_t*>(smem + ad[k - 4]);
                        }
                        if constexpr (k == 13) {
                            o.x = lv[0]; o.y = lv[1]; o.z = lv[2]; o.w = lv[3];
                            *reinterpret_cast<u32x4v*>(wdst + (dtile % 2) * kWTile + q * 16) = o;
                        }
                    }
                }
                if constexpr (k >= 8 && k < 8 + NBLK && !(PANEL_ABL & 1))
                    A[san][k - 8] = *reinterpret_cast<const f16x8*>(pa + (k - 8) * 1024);
                if constexpr (k == 14 && q == 3 && !(PANEL_ABL & 8)) {
                    const int tile = (ub >> 2) + dtile + 4;
                    const uint8_t* p = bp + (size_t)(tile < tiles_end ? tile : tiles_end - 1) * (combined ? kTileK : kTileK / 2);
                    By[sby].v[0] = *reinterpret_cast<const u32x4v*>(p);
                    if constexpr (combined) By[sby].v[1] = *reinterpret_cast<const u32x4v*>(p + 16);
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            slot(std::integral_constant<int, 0>{});
            slot(std::integral_constant<int, 1>{});
            slot(std::integral_constant<int, 2>{});
            slot(std::integral_constant<int, 3>{});
            slot(std::integral_constant<int, 4>{});
            slot(std::integral_constant<int, 5>{});
            slot(std::integral_constant<int, 6>{});
            slot(std::integral_constant<int, 7>{});
            slot(std::integral_constant<int, 8>{});
            slot(std::integral_constant<int, 9>{});
            slot(std::integral_constant<int, 10>{});
            slot(std::integral_constant<int, 11>{});
            slot(std::integral_constant<int, 12>{});
            slot(std::integral_constant<int, 13>{});
            slot(std::integral_constant<int, 14>{});
            slot(std::integral_constant<int, 15>{});
        };

        for (int ub = u_begin; ub < u_end; ub += kUnroll) {
            sub(std::integral_constant<int, 0>{}, ub);
            sub(std::integral_constant<int, 1>{}, ub);
            sub(std::integral_constant<int, 2>{}, ub);
            sub(std::integral_constant<int, 3>{}, ub);
            sub(std::integral_constant<int, 4>{}, ub);
            sub(std::integral_constant<int, 5>{}, ub);
            sub(std::integral_constant<int, 6>{}, ub);
            sub(std::integral_constant<int, 7>{}, ub);
            sub(std::integral_constant<int, 8>{}, ub);
            sub(std::integral_constant<int, 9>{}, ub);
            sub(std::integral_constant<int, 10>{}, ub);
            sub(std::integral_constant<int, 11>{}, ub);
            sub(std::integral_constant<int, 12>{}, ub);
            sub(std::integral_constant<int, 13>{}, ub);
            sub(std::integral_constant<int, 14>{}, ub);
            sub(std::integral_constant<int, 15>{}, ub);
        }
    }
    lds_barrier();                                         // LDS is free for the epilogue
    if constexpr (KG == 2) {
        // The second group's products go to the first: [wave][register][lane] floats, past the stage the epilogue
        // uses, so that no further barrier is needed.
        float* const ex = reinterpret_cast<float*>(smem + kExchange) + wave * (64 * 64) + lane;
        if (kg == 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) ex[(j * 16 + r) * 64] = acc[0][j][r];
        }
        lds_barrier();
        if (kg == 1) return;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][j][r] += ex[(j * 16 + r) * 64];
    }

    // Epilogue: * norm[n] / sqrt(in) (1 / sqrt(bs) is in the rotated activations), convert, store.  Block (i, j) of
    // a lane holds token m0 + 128 i + 32 wave + lane % 32 and, in registers 4 g .. 4 g + 3, the four consecutive
    // output columns n0 + 32 j + 8 g + 4 (lane / 32) + (0..3): one 8-byte (16-bit outputs) or 16-byte (fp32) store
    // each, straight from the accumulators.  The whole workgroup does nothing else meanwhile (one wave per SIMD,
    // one workgroup per CU), so the epilogue is kept to a read, a multiply, a packed conversion and a store.
    // Column counts that are not a multiple of four take the element-wise path.  A part of a tail tile stores
    // its raw fp32 products as a 512 x 128 block of the partial buffer instead.
    if constexpr (PANEL_ABL & 32) {       // no epilogue: one value per lane keeps the accumulators alive
        float t = 0.0f;
#pragma unroll
        for (int i = 0; i < NBLK; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) t += acc[i][j][r];
        if (t == 1.2345f) static_cast<float*>(a.y)[tid] = t;
        return;
    }
    const bool is_part = part >= 0;
    void* const y_out = is_part ? static_cast<void*>(a.partial + (size_t)part_slot * (kPanelM * kPN)) : a.y;
    const int y_type = is_part ? (int)kF32 : a.y_dtype;
    const int yN = is_part ? kPN : a.N, yM = is_part ? kPanelM : a.M;          // row pitch / row limit of y_out
    const int col0 = (is_part ? 0 : n0) + (lane >> 5) * 4;
    const int row0 = (is_part ? 0 : m0) + wave * 32 + (lane & 31);
    // Stores go through a buffer descriptor that ends with the output: rows and columns past the end are given an
    // offset beyond it and dropped by the hardware, so the loop nest carries no branches.
    // (all scales first: a load issued between stores would wait for every store before it, the memory counter
    // retires in order)
    const bool vec = (yN & 3) == 0;
    const uint32_t es = y_type == kF32 ? 4u : 2u;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(y_out, 0, (int)((uint32_t)yM * (uint32_t)yN * es), 0x00020000);
    constexpr uint32_t kDropped = 0xfffffff0u;
    float4 scs[4][4];
    uint32_t coff[4][4], roff[NBLK];
#pragma unroll
    for (int i = 0; i < NBLK; ++i) roff[i] = (uint32_t)(row0 + 128 * i) * (uint32_t)yN * es;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = col0 + 32 * j + 8 * g;
            coff[j][g] = (uint32_t)col * es;
            float4 nr = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
            if (!is_part) {
                if (vec) {
                    if (col < yN) nr = *reinterpret_cast<const float4*>(a.norms + col);
                } else {
                    nr.x = col < yN ? a.norms[col] : 0.0f;
                    nr.y = col + 1 < yN ? a.norms[col + 1] : 0.0f;
                    nr.z = col + 2 < yN ? a.norms[col + 2] : 0.0f;
                    nr.w = col + 3 < yN ? a.norms[col + 3] : 0.0f;
                }
                nr = make_float4(nr.x * a.out_scale, nr.y * a.out_scale, nr.z * a.out_scale, nr.w * a.out_scale);
            }
            scs[j][g] = nr;
        }
    auto store_all = [&](auto Tc, auto Vc) {
        constexpr int T = decltype(Tc)::value;             // output type: one instance of the loop nest per type
        constexpr bool kVec = decltype(Vc)::value;         // and per store width
        typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));
        typedef float f32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = col0 + 32 * j + 8 * g;
                const float4 sc = scs[j][g];
#pragma unroll
                for (int i = 0; i < NBLK; ++i) {
                    const float v0 = acc[i][j][4 * g] * sc.x, v1 = acc[i][j][4 * g + 1] * sc.y;
                    const float v2 = acc[i][j][4 * g + 2] * sc.z, v3 = acc[i][j][4 * g + 3] * sc.w;
                    const bool row_ok = row0 + 128 * i < yM;
                    const uint32_t at = (row_ok && col < yN) ? roff[i] + coff[j][g] : kDropped;
                    if constexpr (kVec) {
                        if constexpr (T == kF32) {
                            const u32x4v o = {__builtin_bit_cast(uint32_t, v0), __builtin_bit_cast(uint32_t, v1),
                                              __builtin_bit_cast(uint32_t, v2), __builtin_bit_cast(uint32_t, v3)};
                            __builtin_amdgcn_raw_buffer_store_b128(o, rs, (int)at, 0, 0);
                        } else {
                            const f32x2 lo = {v0, v1}, hi = {v2, v3};
                            u32x2v o;
                            if constexpr (T == kBF16) {
                                o.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, b16x2));
                                o.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, b16x2));
                            } else {
                                o.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, h16x2));
                                o.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, h16x2));
                            }
                            __builtin_amdgcn_raw_buffer_store_b64(o, rs, (int)at, 0, 0);
                        }
                    } else {                               // column counts that are not a multiple of four
                        const float vs[4] = {v0, v1, v2, v3};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t ae = (row_ok && col + e < yN) ? roff[i] + coff[j][g] + e * es : kDropped;
                            if constexpr (T == kF32)
                                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, vs[e]), rs, (int)ae, 0, 0);
                            else if constexpr (T == kBF16)
                                __builtin_amdgcn_raw_buffer_store_b16(float_to_bf16_bits(vs[e]), rs, (int)ae, 0, 0);
                            else
                                __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, (_Float16)vs[e]), rs, (int)ae, 0, 0);
                        }
                    }
                }
            }
    };
    // 16-bit outputs in whole rows of the tile: the packed pairs go through a wave-private LDS region, 64 tokens at
    // a time (row pitch 272 bytes: conflict-free 64-bit writes and 128-bit reads), and leave as 16-byte pieces of
    // which 16 neighbouring lanes cover the 256 bytes a token has in this tile: whole 128-byte lines instead of
    // 16-byte pieces of 32 different lines per store instruction.
    auto store_rows16 = [&](auto Tc) {
        constexpr int T = decltype(Tc)::value;
        typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        constexpr int kPitch = 272;
        char* const stage = smem + wave * (64 * kPitch);
        char* const wr = stage + (lane & 31) * kPitch + (lane >> 5) * 8;
        const char* const rd = stage + (lane >> 4) * kPitch + (lane & 15) * 16;
        const uint32_t cbyte = (uint32_t)(n0 + (lane & 15) * 8) * 2u;
        const bool col_ok = n0 + (lane & 15) * 8 < yN;
#pragma unroll
        for (int half = 0; half < (NBLK + 1) / 2; ++half) {
#pragma unroll
            for (int ii = 0; ii < (2 * half + 1 < NBLK ? 2 : 1); ++ii)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int i = 2 * half + ii;
                        const float4 sc = scs[j][g];
                        const f32x2 lo = {acc[i][j][4 * g] * sc.x, acc[i][j][4 * g + 1] * sc.y};
                        const f32x2 hi = {acc[i][j][4 * g + 2] * sc.z, acc[i][j][4 * g + 3] * sc.w};
                        u32x2v o;
                        if constexpr (T == kBF16) {
                            o.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, b16x2));
                            o.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, b16x2));
                        } else {
                            o.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, h16x2));
                            o.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, h16x2));
                        }
                        *reinterpret_cast<u32x2v*>(wr + ii * 32 * kPitch + (32 * j + 8 * g) * 2) = o;
                    }
#pragma unroll
            for (int it = 0; it < (2 * half + 1 < NBLK ? 16 : 8); ++it) {
                const u32x4v v = *reinterpret_cast<const u32x4v*>(rd + it * 4 * kPitch);
                // (row it * 4 + lane / 16 of the stage: row block 2 half + it / 8, row (it % 8) * 4 + lane / 16 of it)
                const int row = m0 + wave * 32 + (lane >> 4) + (2 * half + (it >> 3)) * 128 + (it & 7) * 4;
                const uint32_t at = (row < yM && col_ok) ? (uint32_t)row * (uint32_t)yN * 2u + cbyte : kDropped;
                __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)at, 0, 0);
            }
        }
    };
    if (!is_part && y_type != kF32 && (yN & 7) == 0) {
        if (y_type == kBF16) store_rows16(std::integral_constant<int, kBF16>{});
        else store_rows16(std::integral_constant<int, kF16>{});
    } else if (vec) {
        if (y_type == kF32) store_all(std::integral_constant<int, kF32>{}, std::true_type{});
        else if (y_type == kBF16) store_all(std::integral_constant<int, kBF16>{}, std::true_type{});
        else store_all(std::integral_constant<int, kF16>{}, std::true_type{});
    } else {
        if (y_type == kF32) store_all(std::integral_constant<int, kF32>{}, std::false_type{});
        else if (y_type == kBF16) store_all(std::integral_constant<int, kBF16>{}, std::false_type{});
        else store_all(std::integral_constant<int, kF16>{}, std::false_type{});
    }
}

// Sum of the parts of the tail tiles: y[m, n] = out_scale * norm[n] * (part 0 + part 1 + ...), parts added in
// their order.  One workgroup per (tail tile, 32 rows), one thread per four neighbouring columns.
__global__ __launch_bounds__(256) void tq_prefill_panel_sum_kernel(PanelArgs a) {
    const int tile_k = blockIdx.x >> 4, rows0 = (blockIdx.x & 15) * 32;
    const int t = a.panels * a.n_tiles - a.tail_tiles + tile_k;
    const int panel = t / a.n_tiles, n_tile = t - panel * a.n_tiles;
    const int c4 = (threadIdx.x & 31) * 4, r = rows0 + (threadIdx.x >> 5);
    const int col = n_tile * kPN + c4;
#pragma unroll
    for (int rr = 0; rr < 32; rr += 8) {
        const int row = panel * kPanelM + r + rr;
        if (row >= a.M || col >= a.N) continue;
        const float* src = a.partial + ((size_t)tile_k * a.parts) * (kPanelM * kPN) + (size_t)(r + rr) * kPN + c4;
        float4 s = *reinterpret_cast<const float4*>(src);
#pragma unroll 4
        for (int k = 1; k < a.parts; ++k) {
            const float4 v = *reinterpret_cast<const float4*>(src + (size_t)k * (kPanelM * kPN));
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        const float vals[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < a.N) store_scalar(a.y, a.y_dtype, (size_t)row * a.N + col + e, vals[e] * (a.out_scale * a.norms[col + e]));
    }
}

namespace {

// How a call is cut: all tiles whole (tail_tiles == 0), or the tiles that are left after the last full round of
// the chip (every tile, where the call has fewer tiles than the chip has CUs) in `parts` parts each; the fp32
// parts follow the fragment images in the workspace.  The cut is the cheapest by a count in sub-steps of one
// workgroup: rounds of whole tiles and of parts on the CUs, a fixed cost per workgroup (table, first requests,
// epilogue), and the hand-over of the parts through memory.
struct PanelPlan { int tail_tiles, parts, part_subs; size_t xt_bytes, total_bytes; };

constexpr double kWorkgroupCost = 20.0;        // prologue + epilogue of a workgroup, in sub-steps (0.4 us each)
constexpr double kSumFixedCost = 5.0;          // the launch of the sum kernel
constexpr double kSumCostPerPart = 0.19;       // 256 KB written and read again, at the rate the sum kernel reaches
constexpr size_t kMaxPartBytes = (size_t)512 << 20;


PanelPlan panel_plan(const LayerView& L, int batch, int num_cus, size_t capacity) {
    PanelPlan p{};
    const int planes = (L.mode == kDual) ? 2 : 1;
    const size_t panels = ((size_t)batch + kPanelM - 1) / kPanelM;     // whole fragment images
    p.xt_bytes = ((size_t)planes * panels * kPanelM * L.in_features * sizeof(uint16_t) + 255) & ~(size_t)255;
    p.total_bytes = p.xt_bytes;
    const long long tiles = (long long)panels * ((L.out_features + kPN - 1) / kPN);
    const int subs = L.in_features / kSubK;
    const long long cut = tiles < num_cus ? tiles : tiles % num_cus;   // tiles that would be cut
    if (cut == 0) return p;
    const double whole = (double)subs * planes + kWorkgroupCost;
    double best = 0.97 * (double)((tiles + num_cus - 1) / num_cus) * whole;        // (of no cut at all)
    for (int ranges = 1; ranges <= 8; ++ranges) {
        const int per = ((subs + ranges - 1) / ranges + kUnroll - 1) / kUnroll * kUnroll;
        const int parts = (subs + per - 1) / per * planes;
        if (parts < 2 || (ranges > 1 && (subs + per - 1) / per != ranges)) continue;
        const long long units = cut * parts;
        const size_t bytes = (size_t)units * kPanelM * kPN * sizeof(float);
        if (bytes > kMaxPartBytes || p.xt_bytes + bytes > capacity) continue;
        const double cost = (double)((tiles - cut) / num_cus) * whole +
                            (double)((units + num_cus - 1) / num_cus) * (per + kWorkgroupCost) +
                            kSumFixedCost + kSumCostPerPart * (double)units;
        if (cost < best) {
            best = cost;
            p.tail_tiles = (int)cut; p.parts = parts; p.part_subs = per; p.total_bytes = p.xt_bytes + bytes;
        }
    }
    return p;
}

}  // namespace

size_t prefill_panel_workspace_bytes(const LayerView& L, int batch, int num_cus, size_t capacity) {
    return panel_plan(L, batch, num_cus, capacity).total_bytes;
}

// More than 32 rows (up to there: the small-batch kernels), a width that fills the unrolled loop, and 512 x 128
// tiles for more than half the CUs.  With fewer tiles the other kernel, which cuts K with 256 x 256 tiles, is as
// fast or faster even when every tile here is cut along K so that the parts fill the chip (512 and 1024 rows of
// 3584 x 18944, 4096 x 14336 and 8192 x 8192 took 4-12 % longer that way) - except up to 128 rows of long rows,
// where the instance with one row block per wave and every tile cut wins (33 / 64 / 128 rows: 5120 x 27648 62 / 64 /
// 71 us against 70 / 74 / 82, 8192 x 8192 41 / 42 / 44 against 42 / 45 / 50).  capacity: the workspace bytes the
// caller can give (the cut needs room for its parts).
bool prefill_panel_supported(const LayerView& L, int batch, int num_cus, size_t capacity) {
    if (batch <= kSkinnyMaxRows) return false;                 // (up to 32 rows: the small-batch kernels)
    if (L.mode != kSharedLut && L.mode != kDual && L.mode != kPrimaryOnly) return false;
    if (!L.fp16_centroids_ok) return false;
    if (!lanes_supported(L.in_features, L.block_size)) return false;
    if (L.in_features % (kSubK * kUnroll) != 0) return false;
    if ((unsigned long long)L.out_features * (unsigned long long)L.in_features >= (1ull << 32)) return false;
    // (the epilogue addresses the output with 32-bit byte offsets through a buffer descriptor)
    if ((unsigned long long)batch * (unsigned long long)L.out_features * 4ull >= (1ull << 31)) return false;
    const long long tiles = (long long)((batch + kPanelM - 1) / kPanelM) * ((L.out_features + kPN - 1) / kPN);
    if (tiles * 2 > num_cus) return true;
    return batch <= 128 && L.in_features >= 8192 && panel_plan(L, batch, num_cus, capacity).tail_tiles > 0;
}

hipError_t launch_prefill_panel(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                                void* workspace, size_t workspace_bytes, int num_cus, hipStream_t stream) {
    const PanelPlan plan = panel_plan(L, batch, num_cus, workspace_bytes);
    hipError_t e = launch_rotate_tiles(L, x, x_dtype, batch, workspace, stream, true);
    if (e != hipSuccess) return e;
    PanelArgs a{};
    a.xt = static_cast<const char*>(workspace);
    a.plane0 = (L.mode == kSharedLut) ? L.packed_combined : L.packed_primary;
    a.plane1 = L.packed_residual;
    a.tables = L.tables;
    a.norms = L.norms;
    a.y = y; a.y_dtype = y_dtype;
    a.M = batch; a.N = L.out_features; a.K = L.in_features;
    a.panels = (batch + kPanelM - 1) / kPanelM;
    a.n_tiles = (a.N + kPN - 1) / kPN;
    a.n_per_xcd = (a.n_tiles + 7) / 8;
    a.out_scale = L.inv_scale;
    a.tail_tiles = plan.tail_tiles; a.parts = plan.parts; a.part_subs = plan.part_subs;
    // (all tiles cut: no workgroups for whole tiles)
    a.first_part_wg = plan.tail_tiles == a.panels * a.n_tiles ? 0 : 8 * a.n_per_xcd * a.panels;
    a.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + plan.xt_bytes);
    const dim3 grid((unsigned)(a.first_part_wg + a.tail_tiles * a.parts));
    // Row blocks per wave: a single panel of at most 384 rows is run by the kernel that multiplies only the blocks
    // that hold tokens.
    const int nblk = batch > 3 * 128 ? 4 : (batch + 127) / 128;
    auto launch = [&](auto Mode) {
        constexpr int M = decltype(Mode)::value;
        switch (nblk) {
            case 1:
                // (whole tiles whose sub-steps halve into multiples of the unrolled loop: two wave groups)
                if (a.tail_tiles == 0 && a.K % (2 * kSubK * kUnroll) == 0)
                    hipLaunchKernelGGL((tq_prefill_panel_kernel<M, 1, 2>), grid, dim3(2 * kPThreads), 0, stream, a);
                else
                    hipLaunchKernelGGL((tq_prefill_panel_kernel<M, 1>), grid, dim3(kPThreads), 0, stream, a);
                break;
            case 2: hipLaunchKernelGGL((tq_prefill_panel_kernel<M, 2>), grid, dim3(kPThreads), 0, stream, a); break;
            case 3: hipLaunchKernelGGL((tq_prefill_panel_kernel<M, 3>), grid, dim3(kPThreads), 0, stream, a); break;
            default: hipLaunchKernelGGL((tq_prefill_panel_kernel<M, 4>), grid, dim3(kPThreads), 0, stream, a); break;
        }
    };
    switch (L.mode) {
        case kSharedLut: launch(std::integral_constant<int, kSharedLut>{}); break;
        case kDual: launch(std::integral_constant<int, kDual>{}); break;
        default: launch(std::integral_constant<int, kPrimaryOnly>{}); break;
    }
    e = hipGetLastError();
    if (e != hipSuccess || a.tail_tiles == 0) return e;
    hipLaunchKernelGGL(tq_prefill_panel_sum_kernel, dim3((unsigned)(a.tail_tiles * 16)), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace tq
