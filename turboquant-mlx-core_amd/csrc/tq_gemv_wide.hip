// Fused TQ8 dequant + GEMV for gfx950, one batch row, rows of up to 8 slabs (16384 columns), blocks
// of at most 512 columns, shared-rotation and primary-only layers: the batch-1 decode kernel.
//
// Same mathematics and same per-lane work as tq_gemv.hip (a lane owns 32 columns of a 2048-column
// slab, lane-private centroid table in LDS, rotated activations in registers).  What differs is the
// shape of the workgroup.  The other kernel runs two workgroups of up to 8 waves per CU; from three
// slabs on that leaves room for only one or two row streams per workgroup, and every stream
// rotated the activation row for itself, which cost as much as decoding a dozen rows.  Here ONE
// workgroup of up to 16 waves runs per CU:
//   * the decode table is built once per CU;
//   * the activation row is rotated once per CU: the waves split its 512-column tiles among
//     themselves and hand the result over through an image of the whole row in LDS (up to 64 KB);
//   * 16 / W row streams share the CU, each with W waves (one per slab) and, for W > 1, a
//     cross-wave sum per row group.
// Rows whose width is an odd number of 1024-column halves (5120 = 5 x 1024) would leave half of the
// last slab's wave idle.  For those (PAIR) a wave owns one 1024-column half instead, 16 columns per
// lane, and its two 16-byte loads fetch the same columns of two consecutive rows.
// Dual rotation (two nibble planes, each with its own rotation and 16-entry table): the waves of a
// row are split by plane, even units decode the primary plane against the primary rotation, odd
// units the residual plane against the residual rotation, and the cross-wave sum adds the two.
// A wave then needs one rotated activation vector and one table, as for a primary-only layer, and
// the kernel keeps its 16 waves per CU (the other kernel, holding both rotations in registers,
// fits 8).
// Every trip of the main loop issues the same loads whatever is left of a stream's row range
// (past it they re-read its last row), and everything loaded is marked as consumed on every path,
// so the compiler knows exactly how many loads are in flight and waits for no more than the row
// it is about to decode; the prefetched group stays in flight.
// The start of the kernel is kept short, because with 16 waves per CU everything a wave does there
// is done 16 times on shared units: no integer division on the device (the waves of a CU share one
// scalar unit; the host passes quotients), table values through scalar loads (every vector memory
// instruction holds the CU's address unit for 16 cycles), one barrier, and the second stage of the
// register ring requested behind that barrier.  Rows of one slab are handed to the waves of a CU
// group by group from a counter in LDS.
#include "tq_device.h"
#include "tq_gemv_common.h"
#include <atomic>

namespace tq {

// Timeline build (make timeline: libturboquant_amd_timeline.so, used by bench.py --timeline): lane 0 of
// every wave of the first 256 workgroups notes the 100 MHz wall clock at fixed points of the kernel.
//   0 wave started            1 first weight rows requested      2 decode table written
//   3 before the barrier      4 behind the barrier               5 rotated activations in registers (loop entered)
//   6 .. 13 after the 1st, 2nd, .. 8th row group (rows from the LDS counter: every other group)
//   14 last row group stored  15 all memory operations of the wave complete
// In the regular build the marks are nothing.
#ifdef TQ_TIMELINE
__device__ unsigned long long g_timeline[256 * 16 * 16];
#define TQ_MARK(k) do { if (lane == 0 && blockIdx.x < 256) g_timeline[(blockIdx.x * 16 + wave) * 16 + (k)] = wall_clock64(); } while (0)
#else
#define TQ_MARK(k) do { } while (0)
#endif

namespace {

constexpr int kMaxImageCols = 16384;             // widest rotated-activation image in LDS (64 KB)
constexpr int kPairDualSlabs = 8;                // dual rotation with byte-pair tables: rows of up to 8 slabs
constexpr int kTwoImageSlabs = 5;                // ... of which up to 5 keep an image per rotation side by side (80 KB)

// Marks a loaded value as consumed here.  A load whose result is only read on some paths stays
// "possibly in flight" for the compiler on the others, and it then waits for it (and, as loads
// complete in order, for every load issued before it, i.e. the prefetched weights) wherever that
// register is reused, on every trip of the main loop.
__device__ __forceinline__ void consumed(float v) { asm volatile("" :: "v"(v)); }
__device__ __forceinline__ void consumed(const uint4& v) { asm volatile("" :: "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w)); }

// 128-bit streaming load (weights are read exactly once): descriptor + per-lane byte offset +
// wave-uniform byte offset, non-temporal.  No 64-bit address per lane.
__device__ __forceinline__ uint4 load_stream16(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, int row_off) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off, row_off, 2);
    return make_uint4(t.x, t.y, t.z, t.w);
}

// One 512-column tile of the activation row as loaded: always two 16-byte loads, whatever the type
// (a 16-bit tile is 16 bytes: its second load reads the same bytes again), so the number of loads
// in flight does not depend on a branch.
__device__ __forceinline__ TileRaw load_tile_fixed(const void* x, int x_dtype, int col) {
    TileRaw r;
    const int esz = (x_dtype == kF32) ? 4 : 2;
    const char* p = static_cast<const char*>(x) + (size_t)col * esz;
    r.a = *reinterpret_cast<const uint4*>(p);
    r.b = *reinterpret_cast<const uint4*>(p + (esz == 4 ? 16 : 0));
    return r;
}

// Wave w rotates tiles w, w + nwaves, ... (8 values per lane and tile) and writes them into the
// image of the whole row (the host checks that it fits): value k of lane l of a slab sits at float
// index k*64 + l of the slab's 8 KB.  raw[t] holds the activations of tile wave + t * nwaves (any
// valid address for tiles past the row).
template <bool SPLIT, int TILES>
__device__ __forceinline__ void rotate_to_image(const TileRaw (&raw)[TILES], int x_dtype, int in_features,
                                                uint32_t seed, uint32_t bs, float* image, int wave, int nwaves,
                                                int lane) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int tile0 = (wave + t * nwaves) * kTile;
        if (tile0 < in_features) {                                // wave-uniform
            float v[8];
            rotate_tile(raw[t], x_dtype, tile0 + lane * 8, tile0 + lane * 8 < in_features, seed, bs, lane, v);
            const int col = tile0 + lane * 8;
            float* dst = image + (col & ~(kSlab - 1)) + stage_index<SPLIT>(col & (kSlab - 1));
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j * kWave] = v[j];      // 8 columns stay inside one 16-run
        }
    }
}

// After the barrier that follows: a wave picks up the 32 values of the columns it owns.
// unit: the slab of the wave, or with PAIR its 1024-column half (xt then holds 16 values).
template <bool PAIR, int NX>
__device__ __forceinline__ void take_from_image(const float* image, int lane, int unit, bool act_a, bool act_b,
                                                float (&xt)[NX]) {
    if constexpr (PAIR) {
        const int first = unit * (kSlab / 2);                     // first column of the half
        const float* src = image + (first & ~(kSlab - 1)) + ((unit & 1) << 4) * kWave + lane;
#pragma unroll
        for (int k = 0; k < NX; ++k) xt[k] = src[k * kWave];
    } else {
        const float* src = image + unit * kSlab + lane;
#pragma unroll
        for (int k = 0; k < NX; ++k)
            xt[k] = ((k < 16) ? act_a : act_b) ? src[k * kWave] : 0.0f;   // idle runs contribute 0
    }
}

// MODE: kSharedLut (combined byte plane), kPrimaryOnly, or kDual (a.W counts slab-plane pairs: unit
// 2 s is slab s of the primary plane, unit 2 s + 1 slab s of the residual plane).  R rows per group, TILES activation tiles
// per wave (the host checks that TILES * waves covers the row and that blocks are at most 512 wide).
// PAIR (combined plane only): a.W counts 1024-column halves; a group is R row pairs.
// DYN (rows of one slab, a.W == 1): the waves of a workgroup do not own fixed row ranges.  The
// workgroup owns a contiguous range, cut into row groups, and every wave takes its next group from a
// counter in LDS.  Waves of one CU progress at different rates (the spread between the first and the
// last wave of a CU to finish equal shares was a fifth of the run time); with the counter they all
// finish within one row group of each other.
// PRE (rows of 9 to 16 slabs): a.x holds the rotated activations as fp32 (tq_rotate_row_kernel); the
// waves pick their columns up from there, and no image is kept in LDS.
// PT (nibble planes): the table is indexed by a whole byte of the plane and an entry holds the
// centroids of both its nibbles, rounded to fp16: one table read and two mixed-precision FMAs
// (v_fma_mix_f32) per byte instead of two reads, two permutes and two FMAs.  64 KB per plane.
// block: index of the workgroup among those of this layer (a launch may serve several layers).
// BOTH (dual rotation, rows of one slab): a wave decodes both planes of its rows (two rotated
// activation vectors in registers, one row per group), so the waves need no cross-wave sum and take
// their rows from the LDS counter like the other one-slab layers.
template <int MODE, int R, int TILES, bool PAIR, bool DYN, bool PRE = false, bool PT = false, bool BOTH = false>
__device__ __forceinline__ void wide_body(const GemvArgs& a, const int block) {
    static_assert(!BOTH || (MODE == kDual && PT && !(DYN && PRE) && !PAIR && R <= 2), "both planes per wave: dual rotation, pair tables");
    static_assert(!PT || MODE != kSharedLut, "pair tables serve the nibble planes");
    constexpr int kRegion = kRegionBytes;           // decode tables
    constexpr bool kTwoPlaneTable = PT && MODE == kDual;    // both planes' byte-pair tables in one region (below)
    static_assert(!PRE || (!PAIR && !DYN && (MODE != kDual || BOTH) && TILES == 1), "pre-rotated rows: plain slab streams");
    static_assert(!PAIR || MODE == kSharedLut, "row pairs need the one-byte-per-weight plane");
    static_assert(!DYN || (!PAIR && (MODE != kDual || BOTH)), "the group counter serves one-wave row streams");
    constexpr int NS = 2;                           // register ring: one group decoded, one in flight
    constexpr int V = PAIR ? 2 * R : R;             // rows, and sums, per row group
    constexpr int NX = PAIR ? 16 : kChunk;          // rotated activations per lane
    // tables | cross-wave partial sums | activation image.  A static array: its address is a constant
    // the compiler folds into the LDS instructions (with a dynamic one every table read carried an
    // address addition of its own, a third of the vector instructions of the decode).
    constexpr int kImageBytes = PRE ? 0 : (kTwoPlaneTable ? 2 * kTwoImageSlabs * kSlab : kMaxImageCols) * (int)sizeof(float);
    __shared__ __align__(16) char smem[kRegion + kPartialBytes + kImageBytes];
    float* partial = reinterpret_cast<float*>(smem + kRegion);   // [2][waves][V]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TQ_MARK(0);
    const int nwaves = blockDim.x >> 6;
    // (divisions cost a few hundred scalar instructions per wave, and all waves of a CU share one
    // scalar unit: the host supplies the quotients)
    const int stream = (wave * a.w_inv) >> 8;               // wave / a.W
    const int unit = wave - stream * a.W;
    const int slab = (MODE == kDual && !BOTH) ? unit >> 1 : unit;
    const int plane = (MODE == kDual && !BOTH) ? unit & 1 : 0;       // 0: primary plane / rotation / table
    constexpr bool combined = (MODE == kSharedLut);
    const int col_a = PAIR ? slab * (kSlab / 2) + 16 * lane : slab * kSlab + (combined ? 16 * lane : 32 * lane);
    const int col_b = PAIR ? col_a : (combined ? col_a + 1024 : col_a + 16);
    const bool act_a = col_a < a.L.in_features, act_b = col_b < a.L.in_features;
    // Table entries are 256 bytes apart and a lane reads its own 4-byte column of an entry.  One table: 64 columns.
    // Byte-pair tables of both planes: an entry holds 32 columns of the primary plane's value, then 32 of the
    // residual plane's; lanes l and l + 32 share a column (the LDS serves a wave's 32-bit reads in two halves of
    // 32 lanes, so they never meet), and both tables take the 64 KB that one took.
    const uint32_t laneoff = kTwoPlaneTable ? (uint32_t)(lane & 31) << 2 : (uint32_t)lane << 2;
    [[maybe_unused]] const uint32_t laneoff_plane = kTwoPlaneTable ? laneoff | ((uint32_t)plane << 7) : laneoff;
    [[maybe_unused]] const uint32_t table_bits = plane ? 0x10101010u : 0u;               // 16-entry tables: kTab16Bytes = 16 entries
    [[maybe_unused]] const uint32_t laneoff_res = laneoff | 128u;                        // BOTH: the residual plane's columns
    const int out = a.L.out_features;
    const size_t row_bytes = combined ? (size_t)a.L.in_features : ((size_t)a.L.in_features >> 1);
    constexpr bool use_res = (MODE == kSharedLut) || BOTH;  // second 16-byte load per row

    // Contiguous row range of this stream (DYN: of the workgroup): rows_q rows, one more for the
    // first rows_rem ranges.
    const int gs = DYN ? block : block * a.S + stream;
    const int r_begin = gs * a.rows_q + (gs < a.rows_rem ? gs : a.rows_rem);
    const int r_end = r_begin + a.rows_q + (gs < a.rows_rem ? 1 : 0);
    const int r_base = r_begin < out ? r_begin : out - 1;
    const int r_last = r_end > r_begin ? r_end - 1 : r_base;

    // The weight plane is read through a buffer descriptor based at the first row of the stream
    // (offsets inside a stream's rows stay far below 2 GB; the host checks).  Idle runs (columns past the row in
    // its last slab) ask for an offset beyond the descriptor's 2 GB: the hardware returns zeros without touching
    // memory (with a valid address instead, half a wave re-read the first bytes of its row on every load: 3584-
    // column rows fetched 9 % more than they hold); their rotated activations are 0.
    constexpr uint32_t kNoFetch = 0x80000000u;
    const uint8_t* pp = combined ? a.L.packed_combined : (plane ? a.L.packed_residual : a.L.packed_primary);
    const uint32_t off_p = act_a ? (combined ? (uint32_t)col_a : (uint32_t)(col_a >> 1)) : kNoFetch;
    const uint32_t off_q = act_b ? (uint32_t)col_b : kNoFetch;      // combined plane only (PAIR: same columns, next row)
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(pp) + (size_t)r_base * row_bytes, 0, 0x7fffffff, 0x00020000);
    const int row_stride = (int)row_bytes;
    // (BOTH: the residual plane through a descriptor of its own; same offsets as the primary plane)
    const __amdgpu_buffer_rsrc_t rs2 = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(BOTH ? a.L.packed_residual : pp) + (size_t)r_base * row_bytes, 0, 0x7fffffff, 0x00020000);

    uint4 P[NS][R], Q[NS][R];                 // register ring of row groups
    float nrm[NS];                            // norm of the row this lane will store (lanes < V)
    float gte[NS];                            // gate value of that output (the norm again when there is no gate)
    const float* gsrc = a.gate ? a.gate : a.L.norms;
    auto fetch = [&](int buf, int r0) {
        // The norm (and gate value) travel ahead of their rows: loads complete in order, so they
        // have arrived once the first weights of the group have.
        const int rn = r0 + lane % V;
        const int rc = rn < out ? rn : out - 1;
        nrm[buf] = a.L.norms[rc];
        gte[buf] = gsrc[rc];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            // Rows past the stream's range are requested like the others (the number of loads in flight must not
            // depend on a branch) but beyond the descriptor: nothing is fetched for them.  (They used to re-read
            // the range's last row: with 18.5 rows per stream and groups of two, 8 % more bytes than the plane holds.)
            const int ra = PAIR ? r0 + 2 * i : r0 + i;
            const int r = ra < r_last ? ra : r_last;
            const int soff = (r - r_base) * row_stride;
            const uint32_t vp = ra > r_last ? kNoFetch : off_p;           // wave-uniform condition
            P[buf][i] = load_stream16(rs, vp, soff);
            if constexpr (PAIR) {
                const int rq = ra + 1 < r_last ? ra + 1 : r_last;
                Q[buf][i] = load_stream16(rs, ra + 1 > r_last ? kNoFetch : off_q, (rq - r_base) * row_stride);
            } else if constexpr (BOTH) {
                Q[buf][i] = load_stream16(rs2, vp, soff);
            } else if constexpr (use_res) {
                Q[buf][i] = load_stream16(rs, ra > r_last ? kNoFetch : off_q, soff);
            }
        }
    };

    // Prologue.  Everything that has to come from memory is requested up front: the activation
    // tiles, then the weights.  (Every vector memory instruction of a wave occupies the CU's
    // address unit for 16 cycles, and 16 waves share it: the table values, which are the same for
    // all lanes, come through scalar loads instead.)
    constexpr int kEntries = PT ? 256 : (MODE == kSharedLut) ? 256 : (MODE == kDual ? 32 : 16);
    // Wave w writes table entries 16 w .. 16 w + 15 (then 16 (w + nwaves) ..); the first 16 values
    // are requested here.
    typedef const __attribute__((address_space(4))) float cfloat;     // uniform address: scalar load
    cfloat* const tab = (cfloat*)a.L.tables;
    const int e0 = wave * 16 < kEntries ? wave * 16 : 0;
    float tv[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) tv[e] = PT ? 0.0f : tab[e0 + e];
    TileRaw raw[TILES];
    float xt[NX];       // rotated activations, kept in registers for the whole kernel
    float xr[BOTH ? NX : 1];   // BOTH: those of the residual rotation
    if constexpr (PRE) {
        const float4* pa = reinterpret_cast<const float4*>(static_cast<const float*>(a.x) + (act_a ? col_a : 0));
        const float4* pb = reinterpret_cast<const float4*>(static_cast<const float*>(a.x) + (act_b ? col_b : 0));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 u = pa[i], w = pb[i];
            xt[4 * i] = u.x; xt[4 * i + 1] = u.y; xt[4 * i + 2] = u.z; xt[4 * i + 3] = u.w;
            xt[16 + 4 * i] = w.x; xt[17 + 4 * i] = w.y; xt[18 + 4 * i] = w.z; xt[19 + 4 * i] = w.w;
        }
        if constexpr (BOTH) {          // the residual rotation follows in_features floats further on
            const float4* qa = pa + (a.L.in_features >> 2);
            const float4* qb = pb + (a.L.in_features >> 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 u = qa[i], w = qb[i];
                xr[4 * i] = u.x; xr[4 * i + 1] = u.y; xr[4 * i + 2] = u.z; xr[4 * i + 3] = u.w;
                xr[16 + 4 * i] = w.x; xr[17 + 4 * i] = w.y; xr[18 + 4 * i] = w.z; xr[19 + 4 * i] = w.w;
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < TILES; ++t) {     // tiles past the row re-read its start and are not used
            const int col = (wave + t * nwaves) * kTile + lane * 8;
            raw[t] = load_tile_fixed(a.x, a.x_dtype, col < a.L.in_features ? col : 0);
        }
    }
    // The weight requests stay behind the small ones: loads complete in order, and the rotation
    // must not wait for weights.
    __builtin_amdgcn_sched_barrier(0);
    fetch(0, DYN ? r_begin + wave * V : r_begin);

    TQ_MARK(1);
    // Decode tables -> LDS, one private column per lane.
    int* const next_group = reinterpret_cast<int*>(partial);    // DYN: first group nobody has taken yet
    if (DYN && tid == 0) *next_group = 2 * nwaves;              // (groups w and w + nwaves are wave w's first two)
    if constexpr (PT) {
        // Entry e of a plane's table: fp16 centroid of nibble e & 15 in the low half, of nibble e >> 4
        // in the high half.  Chunk c = 16 entries with the same high nibble.  Both planes: lanes 0..31 write
        // the primary plane's columns, lanes 32..63 the residual plane's (16 table values further on).
        uint32_t* const dst = reinterpret_cast<uint32_t*>(smem) + lane;
        const bool second = kTwoPlaneTable && lane >= 32;
        // (both planes' entries are made from scalar loads and chosen per lane afterwards: a choice between the
        // two addresses instead becomes a vector load, which queues behind the weight requests above)
        auto pair_entry = [&](int base, int c, int e) {
            const uint32_t h = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)tab[base + c]);
            const uint32_t l = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)tab[base + e]);
            return (uint32_t)__builtin_amdgcn_readfirstlane((int)((h << 16) | l));
        };
        for (int c = wave; c * 16 < kEntries; c += nwaves) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t u0 = pair_entry(0, c, e);
                if constexpr (kTwoPlaneTable) {
                    const uint32_t u1 = pair_entry(16, c, e);
                    dst[(c * 16 + e) * kWave] = second ? u1 : u0;
                } else {
                    dst[(c * 16 + e) * kWave] = u0;
                }
            }
        }
    } else {
        // Lane l stores each entry's value into its own column, 4 l bytes into the entry's 256.
        float* const dst = reinterpret_cast<float*>(smem) + lane;
        if (wave * 16 < kEntries) {
#pragma unroll
            for (int e = 0; e < 16; ++e) dst[(e0 + e) * kWave] = tv[e];
        }
        for (int c = wave + nwaves; c * 16 < kEntries; c += nwaves) {
#pragma unroll
            for (int e = 0; e < 16; ++e) dst[(c * 16 + e) * kWave] = tab[c * 16 + e];
        }
    }

    TQ_MARK(2);
    if constexpr (PRE) {
        __syncthreads();              // tables visible to every wave
        fetch(1, r_begin + V);
#pragma unroll
        for (int k = 0; k < NX; ++k) xt[k] = ((k < 16) ? act_a : act_b) ? xt[k] : 0.0f;   // idle runs contribute 0
        if constexpr (BOTH) {
#pragma unroll
            for (int k = 0; k < NX; ++k) xr[k] = ((k < 16) ? act_a : act_b) ? xr[k] : 0.0f;
        }
    } else {
    float* const image = reinterpret_cast<float*>(smem + kRegion + kPartialBytes);
    rotate_to_image<combined, TILES>(raw, a.x_dtype, a.L.in_features, a.L.seed_primary, a.L.block_size, image, wave,
                                     nwaves, lane);
    // (byte-pair tables of both planes leave room for a second image of rows up to 5 slabs wide: both rotations
    // before the one barrier)
    [[maybe_unused]] float* const image2 = image + a.img_cols;
    const bool two_images = kTwoPlaneTable && a.img_cols <= kTwoImageSlabs * kSlab;      // uniform over the launch
    if (two_images)
        rotate_to_image<combined, TILES>(raw, a.x_dtype, a.L.in_features, a.L.seed_residual, a.L.block_size, image2,
                                         wave, nwaves, lane);
    TQ_MARK(3);
    __syncthreads();                  // image and tables (and the group counter) visible to every wave
    TQ_MARK(4);
    // The second stage of the ring is requested behind the barrier: a wave whose requests queue up
    // in the memory pipeline would otherwise keep the whole workgroup waiting there.
    fetch(1, DYN ? r_begin + (wave + nwaves) * V : r_begin + V);
    if (two_images) {
        if constexpr (BOTH) {
            take_from_image<PAIR, NX>(image, lane, slab, act_a, act_b, xt);
            take_from_image<PAIR, NX>(image2, lane, slab, act_a, act_b, xr);
        } else {
            take_from_image<PAIR, NX>(plane ? image2 : image, lane, slab, act_a, act_b, xt);
        }
    } else {
    if (plane == 0) take_from_image<PAIR, NX>(image, lane, slab, act_a, act_b, xt);
    if constexpr (MODE == kDual) {
        __syncthreads();                                      // everyone has read the first rotation
        rotate_to_image<combined, TILES>(raw, a.x_dtype, a.L.in_features, a.L.seed_residual, a.L.block_size, image,
                                         wave, nwaves, lane);
        __syncthreads();
        if constexpr (BOTH) take_from_image<PAIR, NX>(image, lane, slab, act_a, act_b, xr);
        else if (plane == 1) take_from_image<PAIR, NX>(image, lane, slab, act_a, act_b, xt);
    }
    }
#pragma unroll
    for (int t = 0; t < TILES; ++t) { consumed(raw[t].a); consumed(raw[t].b); }
    }
    TQ_MARK(5);

    // One row (or with PAIR the same columns of two rows: p -> sum, q -> sum2).
    auto decode_row = [&](const uint4& p, const uint4& q, float& sum, float& sum2) {
        if constexpr (BOTH) {
            const uint32_t pw[4] = {p.x, p.y, p.z, p.w}, qw[4] = {q.x, q.y, q.z, q.w};
            float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                uint32_t pv[4], qv[4];
                pv[0] = *reinterpret_cast<const uint32_t*>(smem + entry_addr<0>(pw[d], laneoff));
                pv[1] = *reinterpret_cast<const uint32_t*>(smem + entry_addr<1>(pw[d], laneoff));
                pv[2] = *reinterpret_cast<const uint32_t*>(smem + entry_addr<2>(pw[d], laneoff));
                pv[3] = *reinterpret_cast<const uint32_t*>(smem + entry_addr<3>(pw[d], laneoff));
                qv[0] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<0>(qw[d], laneoff_res));
                qv[1] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<1>(qw[d], laneoff_res));
                qv[2] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<2>(qw[d], laneoff_res));
                qv[3] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<3>(qw[d], laneoff_res));
#pragma unroll
                for (int j = 0; j < 4; ++j) {        // byte 4 d + j: columns 8 d + 2 j and 8 d + 2 j + 1
                    const int c = 8 * d + 2 * j;
                    s0 = __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(pv[j] & 0xffffu)), xt[c], s0);
                    s1 = __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(pv[j] >> 16)), xt[c + 1], s1);
                    s2 = __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(qv[j] & 0xffffu)), xr[c], s2);
                    s3 = __builtin_fmaf((float)__builtin_bit_cast(_Float16, (uint16_t)(qv[j] >> 16)), xr[c + 1], s3);
                }
            }
            sum = (s0 + s1) + (s2 + s3);
            return;
        }
        if constexpr (PT) {
            // (the table of the wave's plane: 64 KB per plane, the plane number travels in the address permute)
            const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
            uint32_t pv[16];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                pv[4 * d + 0] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<0>(pw[d], laneoff_plane));
                pv[4 * d + 1] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<1>(pw[d], laneoff_plane));
                pv[4 * d + 2] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<2>(pw[d], laneoff_plane));
                pv[4 * d + 3] = *reinterpret_cast<const uint32_t*>(smem + entry_addr_hi<3>(pw[d], laneoff_plane));
            }
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {       // byte i: columns 2 i (low nibble) and 2 i + 1
                const _Float16 lo = __builtin_bit_cast(_Float16, (uint16_t)(pv[i] & 0xffffu));
                const _Float16 hi = __builtin_bit_cast(_Float16, (uint16_t)(pv[i] >> 16));
                s0 = __builtin_fmaf((float)lo, xt[2 * i], s0);
                s1 = __builtin_fmaf((float)hi, xt[2 * i + 1], s1);
            }
            sum = s0 + s1;
            return;
        }
        float val[kChunk];
        // (dual rotation: the residual table follows the primary one, 16 entries of 256 bytes each)
        lookup32<MODE == kSharedLut, 0>(p, q, smem, laneoff, val, table_bits);
        if constexpr (PAIR) {
            float s0 = 0.0f, s1 = 0.0f, t0 = 0.0f, t1 = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; k += 2) {
                s0 = __builtin_fmaf(val[k], xt[k], s0);
                s1 = __builtin_fmaf(val[k + 1], xt[k + 1], s1);
                t0 = __builtin_fmaf(val[16 + k], xt[k], t0);
                t1 = __builtin_fmaf(val[17 + k], xt[k + 1], t1);
            }
            sum = s0 + s1;
            sum2 = t0 + t1;
        } else {
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int k = 0; k < kChunk; k += 2) {
                s0 = __builtin_fmaf(val[k], xt[k], s0);
                s1 = __builtin_fmaf(val[k + 1], xt[k + 1], s1);
            }
            sum = s0 + s1;
        }
    };

    auto consume = [&](int buf, int r0, int it) {
        float acc[V];
        float unused = 0.0f;
        if (r0 + V <= r_end) {                               // wave-uniform: a full group, straight-line
#pragma unroll
            for (int i = 0; i < R; ++i) {
                if constexpr (PAIR) decode_row(P[buf][i], Q[buf][i], acc[2 * i], acc[2 * i + 1]);
                else decode_row(P[buf][i], Q[buf][i], acc[i], unused);
            }
        } else {                                             // ragged end of the range: skip the rows past it
#pragma unroll
            for (int i = 0; i < R; ++i) {
                if constexpr (PAIR) {
                    acc[2 * i] = 0.0f; acc[2 * i + 1] = 0.0f;
                    // the second row of a pair past the range is decoded with the first and not stored
                    if (r0 + 2 * i < r_end) decode_row(P[buf][i], Q[buf][i], acc[2 * i], acc[2 * i + 1]);
                } else {
                    acc[i] = 0.0f;
                    if (r0 + i < r_end) decode_row(P[buf][i], Q[buf][i], acc[i], unused);
                }
            }
        }
        consumed(nrm[buf]); consumed(gte[buf]);
        const float row_scale = a.out_scale * nrm[buf];
        // Lane l < V now gets the wave total of row l of the group.
        const float total = reduce_rec<V, 1>(acc, lane);
        const int r = r0 + lane;
        const bool owner = lane < V && r < r_end;

        float t = total;
        bool store = owner;
        if (!DYN && a.W > 1) {                               // cross-wave sum of the row's slabs
            float* buf_base = partial + (it & 1) * (16 * 16);
            if (lane < V) buf_base[wave * V + lane] = total;
            __syncthreads();
            store = owner && unit == 0;
            if (store) {
                t = 0.0f;
                for (int w = 0; w < a.W; ++w) t += buf_base[(stream * a.W + w) * V + lane];
            }
        }
        if (store) {
            t *= row_scale;
            if (a.gate) { const float g = gte[buf]; t = g / (1.0f + expf(-g)) * t; }   // silu(gate) * y
            store_scalar(a.y, a.y_dtype, (size_t)r, t);
        }
    };

    // Main loop over the register ring, unrolled twice so the stages are static: a stage is
    // requested again as soon as it has been decoded, so two groups are in flight or being decoded
    // at any time.  The trip count is uniform over the grid.  Whole rounds of two stages run
    // without a condition inside; an odd last group is a tail.
    if constexpr (DYN) {
        const int groups = (r_end - r_begin + V - 1) / V;
        int g0 = wave, g1 = wave + nwaves;                  // groups held by the two ring stages
        // Takes the group for the stage being emptied.  Every lane adds to a slot of its own, lane
        // 0's is the counter (no branch around the LDS operation); the answer is picked up after the
        // decode, when it has long arrived.  Groups are handed out in increasing order.
        int* const slot = next_group + lane;
        auto take = [&]() { return __hip_atomic_fetch_add(slot, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); };
        auto taken = [&](int t) { asm volatile("" : "+v"(t)); return __builtin_amdgcn_readfirstlane(t); };
        int t = take();
        [[maybe_unused]] int rounds = 0;
        while (g0 < groups) {
            consume(0, r_begin + g0 * V, 0);
            if (rounds < 8) TQ_MARK(6 + rounds);
            ++rounds;
            g0 = taken(t);
            t = take();
            fetch(0, r_begin + g0 * V);
            if (g1 >= groups) break;
            consume(1, r_begin + g1 * V, 0);
            g1 = taken(t);
            t = take();
            fetch(1, r_begin + g1 * V);
        }
        TQ_MARK(14);
#ifdef TQ_TIMELINE
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
        TQ_MARK(15);
        return;
    }
    int it0 = 0;
    for (; it0 + NS <= a.iters; it0 += NS) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            consume(u, r_begin + (it0 + u) * V, it0 + u);
            if (it0 + u < 8) TQ_MARK(6 + it0 + u);
            fetch(u, r_begin + (it0 + u + NS) * V);
        }
    }
    if (it0 < a.iters) consume(0, r_begin + it0 * V, it0);
    TQ_MARK(14);
#ifdef TQ_TIMELINE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
    TQ_MARK(15);
}

template <int MODE, int R, int TILES, bool PAIR, bool DYN, bool PRE = false, bool PT = false, bool BOTH = false>
__global__ __launch_bounds__(1024) void tq_gemv_wide_kernel(GemvArgs a) {
    wide_body<MODE, R, TILES, PAIR, DYN, PRE, PT, BOTH>(a, (int)blockIdx.x);
}

// Two or three layers that read the same activation row (q, k, v or gate, up of a decoder layer),
// one launch: the workgroups are shared out over the layers by rows, each workgroup serves one
// layer with that layer's seeds, tables and row ranges.  One start of the kernel instead of three.
struct GemvGroup {
    GemvArgs a[3];
    int first[4];          // layer j owns workgroups first[j] .. first[j + 1] - 1
};
template <int MODE, int R, bool PAIR, bool PT, bool BOTH = false>
__global__ __launch_bounds__(1024) void tq_gemv_wide_group_kernel(GemvGroup g) {
    const int b = (int)blockIdx.x;
    const int j = b >= g.first[2] ? 2 : (b >= g.first[1] ? 1 : 0);
    wide_body<MODE, R, 1, PAIR, false, false, PT, BOTH>(g.a[j], b - g.first[j]);
}

template <int MODE, int R, int TILES, bool PAIR, bool DYN = false, bool PRE = false, bool PT = false, bool BOTH = false>
hipError_t launch_wide_one(const GemvArgs& a, int grid, int threads, hipStream_t stream) {
    hipLaunchKernelGGL((tq_gemv_wide_kernel<MODE, R, TILES, PAIR, DYN, PRE, PT, BOTH>), dim3(grid), dim3(threads), 0, stream, a);
    return hipGetLastError();
}

// Dual rotation on pair tables, rows of 3 to 5 slabs: one wave per slab that decodes both planes (two images of
// the row, one per rotation) instead of a wave per (slab, plane).  Measured, eager launches on one box, both
// planes per wave against one: 10240 x 10240 27.0 against 29.5 us, 27648 x 5120 32.8 / 33.9; rows of two slabs:
// 18944 x 3584 18.8 / 19.0-20.0, 8192 x 8192 equal, 4096 x 4096 8.8 / 8.5: they stay with a wave per plane.  (A
// property of the layer's width alone: a grouped launch must take the kernel a launch of its own would.)
// (Also measured and not kept: a wave per 1024-column half at 5120 columns, 8 bytes per lane, plane and row, so
// that no wave carries the half-empty third slab: 27648 x 5120 33.1 us, 5120 x 5120 12.4, no better than the above.)
bool wants_both_planes(int slabs, bool fp16_ok) {
    return fp16_ok && slabs >= 3 && slabs <= kTwoImageSlabs;
}

// Row pairs are used where the width is an odd number of 1024-column halves.
bool wants_pairs(const LayerView& L) {
    return L.mode == kSharedLut && L.in_features % kSlab == kSlab / 2 && L.in_features / (kSlab / 2) >= 3 &&
           L.in_features <= kMaxImageCols;
}

template <int MODE, bool PAIR, bool PT>
hipError_t launch_wide_shape(const GemvArgs& a, int grid, int threads, int R, bool two, int out, hipStream_t stream) {
    if constexpr (!PAIR && MODE != kDual) {
        if (a.pre_rotated) return R == 2 ? launch_wide_one<MODE, 2, 1, false, false, true, PT>(a, grid, threads, stream)
                                         : launch_wide_one<MODE, 1, 1, false, false, true, PT>(a, grid, threads, stream);
        if (a.W == 1) {                                     // one slab: 16 one-wave streams fed from a group counter
            const int rows_wg = (out + grid - 1) / grid;
            if (rows_wg >= 4 * a.S) return launch_wide_one<MODE, 2, 1, false, true, false, PT>(a, grid, threads, stream);
            return launch_wide_one<MODE, 1, 1, false, true, false, PT>(a, grid, threads, stream);
        }
    }
    if constexpr (MODE != kSharedLut) {
        if (R == 4) return two ? launch_wide_one<MODE, 4, 2, PAIR, false, false, PT>(a, grid, threads, stream)
                               : launch_wide_one<MODE, 4, 1, PAIR, false, false, PT>(a, grid, threads, stream);
    }
    if (R == 2) return two ? launch_wide_one<MODE, 2, 2, PAIR, false, false, PT>(a, grid, threads, stream)
                           : launch_wide_one<MODE, 2, 1, PAIR, false, false, PT>(a, grid, threads, stream);
    return two ? launch_wide_one<MODE, 1, 2, PAIR, false, false, PT>(a, grid, threads, stream)
               : launch_wide_one<MODE, 1, 1, PAIR, false, false, PT>(a, grid, threads, stream);
}

template <int MODE, bool PAIR>
hipError_t launch_wide_mode(GemvArgs a, int num_cus, hipStream_t stream) {
    const int out = a.L.out_features;
    const int slabs = a.W;
    if (PAIR) a.W = a.L.in_features / (kSlab / 2);           // halves per row
    // Dual rotation: (slab, plane) pairs per row; rows of one slab whose centroids fit fp16 keep both
    // planes in one wave instead.
    const bool both = MODE == kDual && a.L.fp16_centroids_ok &&
                      (slabs == 1 || a.pre_rotated || wants_both_planes(slabs, true));
    if (MODE == kDual && !both) a.W = 2 * slabs;
    a.S = 16 / a.W;                                          // row streams sharing the CU
    const int threads = a.W * a.S * kWave;
    const int padded = slabs * kSlab;
    if (padded > kMaxImageCols && !a.pre_rotated) return hipErrorInvalidValue;   // gemv_wide_supported() rules this out
    a.img_cols = padded;

    int grid = (out + a.S - 1) / a.S;
    if (grid > num_cus) grid = num_cus;
    if (grid < 1) grid = 1;
    const bool shared_range = !PAIR && (MODE != kDual || both) && a.W == 1;   // one range per workgroup (group counter)
    const int ts = shared_range ? grid : grid * a.S;        // row ranges
    a.rows_q = out / ts;
    a.rows_rem = out % ts;
    a.w_inv = (256 + a.W - 1) / a.W;                        // (w * w_inv) >> 8 == w / W for w < 16, W <= 16
    const int max_rows = (int)(((long long)out + grid * a.S - 1) / (grid * a.S));   // longest share of a stream
    const int per_r = PAIR ? 2 : 1;                         // rows per unit of R
    // (nibble planes: a row is 16 bytes per lane, so four rows make the group of loads of two byte-plane rows)
    const int R = (MODE != kSharedLut && !a.pre_rotated && !both && max_rows >= 4) ? 4 : max_rows >= 2 * per_r ? 2 : 1;
    a.iters = (max_rows + R * per_r - 1) / (R * per_r);

    if constexpr (MODE == kDual) {
        if (a.pre_rotated) {          // 9 to 16 slabs, one wave per slab, both planes per wave
            if (!a.L.fp16_centroids_ok) return hipErrorInvalidValue;     // gemv_wide_supported() rules this out
            return R == 2 ? launch_wide_one<kDual, 2, 1, false, false, true, true, true>(a, grid, threads, stream)
                          : launch_wide_one<kDual, 1, 1, false, false, true, true, true>(a, grid, threads, stream);
        }
        if (both && slabs > 1) {      // 2 to 5 slabs: one wave per slab, both planes per wave, an image per rotation
            const int ntiles = (a.L.in_features + kTile - 1) / kTile;
            const bool two = ntiles > threads / kWave;
            const int Rb = max_rows >= 2 ? 2 : 1;
            a.iters = (max_rows + Rb - 1) / Rb;
            if (Rb == 2) return two ? launch_wide_one<kDual, 2, 2, false, false, false, true, true>(a, grid, threads, stream)
                                    : launch_wide_one<kDual, 2, 1, false, false, false, true, true>(a, grid, threads, stream);
            return two ? launch_wide_one<kDual, 1, 2, false, false, false, true, true>(a, grid, threads, stream)
                       : launch_wide_one<kDual, 1, 1, false, false, false, true, true>(a, grid, threads, stream);
        }
        if (both) {
            const int rows_wg = (out + grid - 1) / grid;
            if (rows_wg >= 4 * a.S) return launch_wide_one<kDual, 2, 1, false, true, false, true, true>(a, grid, threads, stream);
            return launch_wide_one<kDual, 1, 1, false, true, false, true, true>(a, grid, threads, stream);
        }
    }
    const int ntiles = (a.L.in_features + kTile - 1) / kTile;
    const bool two = ntiles > threads / kWave;              // at most two tiles per wave: checked by the caller
    if constexpr (MODE == kSharedLut) return launch_wide_shape<MODE, PAIR, false>(a, grid, threads, R, two, out, stream);
    else if constexpr (MODE == kPrimaryOnly)
        return a.L.fp16_centroids_ok ? launch_wide_shape<MODE, PAIR, true>(a, grid, threads, R, two, out, stream)
                                     : launch_wide_shape<MODE, PAIR, false>(a, grid, threads, R, two, out, stream);
    else return (slabs <= kPairDualSlabs && a.L.fp16_centroids_ok)
                    ? launch_wide_shape<MODE, PAIR, true>(a, grid, threads, R, two, out, stream)
                    : launch_wide_shape<MODE, PAIR, false>(a, grid, threads, R, two, out, stream);
}

template <int MODE, int R, bool PAIR, bool PT, bool BOTH = false>
hipError_t launch_group_one(const GemvGroup& g, int grid, int threads, hipStream_t stream) {
    hipLaunchKernelGGL((tq_gemv_wide_group_kernel<MODE, R, PAIR, PT, BOTH>), dim3(grid), dim3(threads), 0, stream, g);
    return hipGetLastError();
}

// BOTH (dual rotation on pair tables, rows of up to 5 slabs): one wave per slab decodes both planes.
template <int MODE, bool PAIR, bool PT, bool BOTH = false>
hipError_t launch_group_mode(GemvGroup& g, int n, int num_cus, hipStream_t stream) {
    const int in = g.a[0].L.in_features;
    const int slabs = (in / kChunk + kWave - 1) / kWave;
    const int W = PAIR ? in / (kSlab / 2) : ((MODE == kDual && !BOTH) ? 2 * slabs : slabs);
    const int S = 16 / W;
    const int threads = W * S * kWave;
    long long total = 0;
    for (int j = 0; j < n; ++j) total += g.a[j].L.out_features;
    // Workgroups per layer in proportion to its rows (the layers have rows of equal width).
    int blocks[3] = {0, 0, 0}, used = 0;
    for (int j = 0; j < n; ++j) {
        blocks[j] = (int)((long long)num_cus * g.a[j].L.out_features / total);
        if (blocks[j] < 1) blocks[j] = 1;
        used += blocks[j];
    }
    for (int j = 0; used < num_cus; j = (j + 1) % n) { ++blocks[j]; ++used; }
    for (int j = 0; used > num_cus; j = (j + 1) % n) if (blocks[j] > 1) { --blocks[j]; --used; }
    const int per_r = PAIR ? 2 : 1;
    int min_rows = 1 << 30;
    for (int j = 0; j < n; ++j) {
        GemvArgs& a = g.a[j];
        a.chunks = in / kChunk;
        a.W = W; a.S = S;
        a.img_cols = slabs * kSlab;
        a.pre_rotated = 0;
        const int ts = blocks[j] * S;
        a.rows_q = a.L.out_features / ts;
        a.rows_rem = a.L.out_features % ts;
        a.w_inv = (256 + W - 1) / W;
        const int max_rows = a.rows_q + (a.rows_rem ? 1 : 0);
        if (max_rows < min_rows) min_rows = max_rows;
    }
    const int R = (MODE != kSharedLut && !BOTH && min_rows >= 4) ? 4 : min_rows >= 2 * per_r ? 2 : 1;
    g.first[0] = 0;
    for (int j = 0; j < 3; ++j) g.first[j + 1] = g.first[j] + (j < n ? blocks[j] : 0);
    for (int j = n; j < 3; ++j) g.first[j + 1] = 1 << 30;        // no workgroup reaches an unused slot
    for (int j = n; j < 3; ++j) g.first[j] = 1 << 30;
    for (int j = 0; j < n; ++j) {
        const int max_rows = g.a[j].rows_q + (g.a[j].rows_rem ? 1 : 0);
        g.a[j].iters = (max_rows + R * per_r - 1) / (R * per_r);
    }
    if constexpr (MODE != kSharedLut && !BOTH) {
        if (R == 4) return launch_group_one<MODE, 4, PAIR, PT>(g, used, threads, stream);
    }
    if (R == 2) return launch_group_one<MODE, 2, PAIR, PT, BOTH>(g, used, threads, stream);
    return launch_group_one<MODE, 1, PAIR, PT, BOTH>(g, used, threads, stream);
}

}  // namespace

// Layers that can share a launch: two or three, same mode (shared or dual rotation), same width,
// each fit for the kernel on its own, rows of more than one wave (no group counter) and one
// activation tile per wave.
bool gemv_wide_group_supported(const LayerView* Ls, int n, int num_cus) {
    if (n < 2 || n > 3 || num_cus < n) return false;
    const LayerView& L0 = Ls[0];
    if (L0.mode != kSharedLut && L0.mode != kDual) return false;
    const int slabs = (L0.in_features / kChunk + kWave - 1) / kWave;
    bool fp16_all = true;
    for (int j = 0; j < n; ++j) fp16_all = fp16_all && Ls[j].fp16_centroids_ok;
    const bool both = L0.mode == kDual && wants_both_planes(slabs, fp16_all);     // as launch_gemv_wide_group decides
    const int W = wants_pairs(L0) ? L0.in_features / (kSlab / 2) : ((L0.mode == kDual && !both) ? 2 * slabs : slabs);
    if (W < 2 || W > 16) return false;
    if (L0.mode == kDual && slabs == 1) return false;       // one-slab dual rows: one wave per row (both planes), no sharing
    const int threads = W * (16 / W) * kWave;
    if ((L0.in_features + kTile - 1) / kTile > threads / kWave) return false;
    for (int j = 0; j < n; ++j) {
        if (Ls[j].mode != L0.mode || Ls[j].in_features != L0.in_features) return false;
        if (!gemv_wide_supported(Ls[j], 1, false)) return false;      // (1 CU: the strictest bound on a stream's share)
    }
    return true;
}

// as[j]: x, y, types, gate and out_scale of layer j set by the caller (same x for all).
hipError_t launch_gemv_wide_group(const GemvArgs* as, int n, int num_cus, hipStream_t stream) {
    GemvGroup g{};
    for (int j = 0; j < n; ++j) g.a[j] = as[j];
    const LayerView& L = g.a[0].L;
    const int slabs = (L.in_features / kChunk + kWave - 1) / kWave;
    if (L.mode == kSharedLut)
        return wants_pairs(L) ? launch_group_mode<kSharedLut, true, false>(g, n, num_cus, stream)
                              : launch_group_mode<kSharedLut, false, false>(g, n, num_cus, stream);
    bool fp16_ok = true;
    for (int j = 0; j < n; ++j) fp16_ok = fp16_ok && g.a[j].L.fp16_centroids_ok;
    if (wants_both_planes(slabs, fp16_ok)) return launch_group_mode<kDual, false, true, true>(g, n, num_cus, stream);
    return (slabs <= kPairDualSlabs && fp16_ok) ? launch_group_mode<kDual, false, true>(g, n, num_cus, stream)
                                                : launch_group_mode<kDual, false, false>(g, n, num_cus, stream);
}

// One batch row, blocks of at most 512 columns, per-stream share of the plane below 2 GB.
// Shared rotation and primary only: rows of 1 to 8 slabs, or (shared rotation) of an odd number,
// 3 to 15, of 1024-column halves.  Dual rotation: rows of 1 to 8 slabs.
bool gemv_wide_supported(const LayerView& L, int num_cus, bool pre_rotated) {
    if (L.mode != kSharedLut && L.mode != kPrimaryOnly && L.mode != kDual) return false;
    if (!shape_supported(L.in_features, L.block_size)) return false;
    if (L.block_size > (uint32_t)kTile) return false;
    const int slabs = (L.in_features / kChunk + kWave - 1) / kWave;
    int W = slabs;
    if (pre_rotated) { if ((L.mode == kDual && !L.fp16_centroids_ok) || slabs < 9 || slabs > 16) return false; }
    else if (wants_pairs(L)) W = L.in_features / (kSlab / 2);
    else if (L.mode == kDual) { if (slabs > 8) return false; W = 2 * slabs; }   // two waves per slab
    else if (slabs < 1 || slabs > 8) return false;
    const int S = 16 / W;
    const int ntiles = (L.in_features + kTile - 1) / kTile;
    if (!pre_rotated && ntiles > 2 * W * S) return false;
    const size_t row_bytes = L.mode == kSharedLut ? (size_t)L.in_features : (size_t)L.in_features / 2;
    const bool shared_range = W == 1 && L.mode != kDual;    // one row range per workgroup, shared by its waves
    const long long streams = (long long)(num_cus > 0 ? num_cus : 1) * (shared_range ? 1 : S);
    const long long max_rows = (L.out_features + streams - 1) / streams + 4;
    return (unsigned long long)max_rows * row_bytes < (1ull << 31);
}

hipError_t launch_gemv_wide(const GemvArgs& base, int num_cus, hipStream_t stream) {
    GemvArgs a = base;
    a.chunks = a.L.in_features / kChunk;
    a.W = (a.chunks + kWave - 1) / kWave;
    if (a.L.mode == kSharedLut)
        return (!a.pre_rotated && wants_pairs(a.L)) ? launch_wide_mode<kSharedLut, true>(a, num_cus, stream)
                                : launch_wide_mode<kSharedLut, false>(a, num_cus, stream);
    if (a.L.mode == kDual) return launch_wide_mode<kDual, false>(a, num_cus, stream);
    return launch_wide_mode<kPrimaryOnly, false>(a, num_cus, stream);
}

}  // namespace tq

#ifdef TQ_TIMELINE
// Timeline build only: copies the marks of the last launches to the host / clears them.
extern "C" int tq_timeline_read(unsigned long long* host) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(tq::g_timeline), sizeof(tq::g_timeline));
}
extern "C" int tq_timeline_clear(void) {
    static unsigned long long zeros[256 * 16 * 16];
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(tq::g_timeline), zeros, sizeof(zeros));
}
#endif
