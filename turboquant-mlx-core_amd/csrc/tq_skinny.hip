// TQ8 small-batch forward for gfx950: 2..32 activation rows (any activation type), shared-rotation
// layers (one byte per weight).
//
// The batch-1 kernel multiplies every decoded weight with the activation of each batch row on the
// vector ALU, so its time grows with the batch.  Here the batch rows are the M side of
// v_mfma_f32_16x16x32_f16: a decoded weight costs one table read and half a byte permute however
// many rows there are, and the kernel stays bound by the same table-read rate as batch 1.
//
//   Y[m, n] = norm[n] / sqrt(in) * sum_k X~[m, k] * L[n, k],   X~ = H (s (.) X) / sqrt(bs)
//
// K is cut into 512-column chunks.  A wave keeps the rotated activations of its chunk for all 16
// (padded) batch rows in registers as MFMA A operands (64 VGPRs; two such sets for 17..32 rows, which
// multiply the same decoded weights), walks 16-row groups of the weight
// plane, decodes 16 x 512 weights per group through the lane-private LDS table (entries rounded to
// fp16, as in the prefill kernel) and writes the 16 x 16 fp32 partial product of the chunk.  A
// second small kernel adds the chunks, applies the row norm and converts.
// The rotated activations come from tq_rotate_f16_kernel (tile images, see tq_prefill.hip).
#include "tq_device.h"
#include "tq_gemv_common.h"

namespace tq {

typedef _Float16 sk_f16x8 __attribute__((ext_vector_type(8)));
typedef float sk_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kSkChunk = 512;            // columns per K chunk
constexpr int kSkThreads = 512;          // 8 waves per workgroup, one workgroup per CU
constexpr int kSkLutBytes = 256 * 256;
constexpr int kSkStageBytes = 16 * kSkChunk * 2;   // 16 rows x 512 fp16 rotated activations
constexpr int kSkMaxRows = kSkinnyMaxRows;   // two sets of 16 batch rows per decoded weight

struct SkinnyArgs {
    const void* x;             // FUSED: activations [batch, K], f32, f16 or bf16
    int x_dtype;
    uint32_t seed, block_size; // FUSED: rotation of the layer (blocks of at most 512 columns)
    float x_scale;             // FUSED: 1 / sqrt(block_size), applied to the rotated activations before they are rounded
    const uint16_t* xt;        // otherwise: rotated activations, fp16 tile images [K/32][256 rows x 64 B] (rows >= batch unset)
    const uint8_t* plane;      // combined bytes [N, K]
    const float* tables;       // 256-entry sum table
    float* partial;            // [chunks][batch][N] fp32
    int batch, N, K;
    int chunks;                // K / 512
    int groups;                // ceil(N / 16)
    int wgs_per_chunk;
    int groups_q, groups_rem;  // groups / workers and groups % workers (workers = waves sharing a chunk)
};

__device__ __forceinline__ uint32_t sk_entry_addr(uint32_t idx_bytes, uint32_t laneoff, int j) {
    switch (j) {
        case 0: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0400u);
        case 1: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0500u);
        case 2: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0600u);
        default: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0700u);
    }
}

// FUSED: the workgroup rotates the 16 x 512 activations of its chunk itself (blocks of at most 512
// columns: a block never leaves the chunk), instead of reading tile images a separate kernel wrote.
// chunk, wg_in_chunk: the 512-column chunk of this workgroup and its index among the workgroups that
// share the chunk for this layer (a launch may serve several layers).
// SETS: 1 (up to 16 batch rows) or 2 (17..32 rows: a second set of A operands multiplies the same decoded
// weights, so the weights are still read and decoded once).
// RAGGED: the row does not fill its last 512-column chunk (a kernel of its own, so that the loads of whole
// chunks keep their constant offsets and the compiler its exact wait counts).
template <bool FUSED, int SETS, bool RAGGED>
__device__ __forceinline__ void skinny_body(const SkinnyArgs& a, const int chunk, const int wg_in_chunk) {
    static_assert(FUSED || !RAGGED, "blocks wider than a chunk divide the row into whole chunks");
    // table | 16 SETS x 512 fp16 rotated activations (FUSED).  One workgroup of 8 waves per CU: 16 waves
    // gained nothing, and 8 have the registers for two row groups in flight.
    __shared__ __align__(16) char smem[kSkLutBytes + SETS * kSkStageBytes];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t laneoff = (uint32_t)lane << 2;

    // (no integer division in the kernel: the waves of a CU share one scalar unit and a division is a
    // few hundred instructions)
    const int m = lane & 15, g = lane >> 4;               // A operand: batch row, k group; B operand: weight row, k group

    // Row groups of this wave: the groups are dealt out evenly over all waves that share the chunk.
    const int me = wg_in_chunk * (kSkThreads / 64) + wave;
    const int g_begin = me * a.groups_q + (me < a.groups_rem ? me : a.groups_rem);
    const int g_end = g_begin + a.groups_q + (me < a.groups_rem ? 1 : 0);
    const size_t col0 = (size_t)chunk * kSkChunk + 16 * g;
    auto row_ptr = [&](int grp) {
        int row = grp * 16 + m;
        if (row >= a.N) row = a.N - 1;                     // rows past N re-read row N-1: never stored
        return a.plane + (size_t)row * a.K + col0;
    };
    // A last chunk that the row does not fill (K a multiple of 64, not of 512; blocks of at most 256 columns):
    // its 64-column pieces past the row are read from piece 0 again (valid memory, any byte decodes to a
    // finite centroid) and multiply rotated activations that are zero.  Wave-uniform.
    const int pieces = (!RAGGED || a.K - chunk * kSkChunk >= kSkChunk) ? 8 : (a.K - chunk * kSkChunk) >> 6;
    int piece_off[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) piece_off[q] = (!RAGGED || q < pieces) ? 64 * q : 0;

    // Everything that has to come from memory is requested up front, the small things first (loads
    // complete in order): table values, the activations this wave rotates, then the first row group,
    // which travels while the activations are rotated and the table is built.
    constexpr int kSlots = 256 * 16 / kSkThreads;
    float tv[kSlots];
#pragma unroll
    for (int k = 0; k < kSlots; ++k) tv[k] = a.tables[(tid + k * kSkThreads) >> 4];
    TileRaw xin[2 * SETS];
    if constexpr (FUSED) {
#pragma unroll
        for (int t = 0; t < 2 * SETS; ++t) {               // batch rows w, w + 8, .. (row 0 again past the batch: not used)
            const int b = wave + 8 * t;
            const int col = chunk * kSkChunk + lane * 8;     // (columns past the row: read column 0, rotated as zeros)
            xin[t] = load_tile_raw(a.x, a.x_dtype, (size_t)(b < a.batch ? b : 0) * a.K, (!RAGGED || col < a.K) ? col : 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // Plain loads, not streaming ones: a load instruction touches 64 bytes of each of 16 rows, half
    // a cache line, and the other half is asked for by a later instruction; with the streaming
    // hint that half was fetched from memory again (13 % more time).
    sk_u32x4 rawA[8], rawB[8];                             // two row groups: one decoded, one in flight
    auto request = [&](sk_u32x4 (&raw)[8], int grp) {
        const uint8_t* p = row_ptr(grp);
#pragma unroll
        for (int q = 0; q < 8; ++q) raw[q] = (*reinterpret_cast<const sk_u32x4*>(p + piece_off[q]));
    };
    if (g_begin < g_end) request(rawA, g_begin);

    // Decode table -> LDS, one private column per lane, values rounded to fp16 (upper half of the dword).
    {
        uint4* dst = reinterpret_cast<uint4*>(smem);
#pragma unroll
        for (int k = 0; k < kSlots; ++k) {
            const uint32_t v = (uint32_t)float_to_f16_bits(tv[k]) << 16;
            dst[tid + k * kSkThreads] = make_uint4(v, v, v, v);
        }
    }

    sk_f16x8 afrag[SETS][16];
    char* const stage = smem + kSkLutBytes;
    if constexpr (FUSED) {
        // Wave w rotates batch rows w, w + 8, .. of the chunk (one 512-column tile each, 8 values per
        // lane; blocks of at most 512 columns: a block never leaves the chunk) and writes them, scaled by 1 / sqrt(bs), as fp16,
        // [16 SETS rows][512]; rows past the batch are zero.
        constexpr int kPitch = kSkChunk * 2;
#pragma unroll
        for (int t = 0; t < 2 * SETS; ++t) {
            const int b = wave + 8 * t;
            const int col = chunk * kSkChunk + lane * 8;
            uint4 packed = make_uint4(0, 0, 0, 0);
            if (b < a.batch) {                              // wave-uniform
                float v[8];
                rotate_tile(xin[t], a.x_dtype, col, !RAGGED || col < a.K, a.seed, a.block_size, lane, v);
                packed.x = (uint32_t)float_to_f16_bits(v[0] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[1] * a.x_scale) << 16);
                packed.y = (uint32_t)float_to_f16_bits(v[2] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[3] * a.x_scale) << 16);
                packed.z = (uint32_t)float_to_f16_bits(v[4] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[5] * a.x_scale) << 16);
                packed.w = (uint32_t)float_to_f16_bits(v[6] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[7] * a.x_scale) << 16);
            }
            *reinterpret_cast<uint4*>(stage + b * kPitch + lane * 16) = packed;
        }
        __syncthreads();                                    // table and activations visible
        // k-step s covers columns 64 (s/2) + 16 g + 8 (s%2) + [0, 8) of the chunk, the same columns
        // the B operand of that step decodes (any column order is fine as long as both agree).
#pragma unroll
        for (int e = 0; e < SETS; ++e)
#pragma unroll
            for (int s = 0; s < 16; ++s)
                afrag[e][s] = *reinterpret_cast<const sk_f16x8*>(stage + (m + 16 * e) * kPitch + (64 * (s >> 1) + 16 * g + 8 * (s & 1)) * 2);
    } else {
        // Tile images written by tq_rotate_f16_kernel: [K/32][256][32] fp16 with 16-byte slots
        // XOR-permuted per row; same column order as above.
#pragma unroll
        for (int e = 0; e < SETS; ++e)
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                const int off = 16 * g + 8 * (s & 1);              // column inside the 64-column piece
                const int kt = chunk * 16 + 2 * (s >> 1) + (off >> 5);
                const int slot = ((off & 31) >> 3) ^ ((m >> 2) & 3);      // (rows m and m + 16: the same permutation)
                afrag[e][s] = *reinterpret_cast<const sk_f16x8*>(reinterpret_cast<const char*>(a.xt) +
                                                                  ((size_t)kt * 256 + m + 16 * e) * 64 + slot * 16);
            }
        __syncthreads();                                    // table visible
    }

    auto lookup2 = [&](uint32_t w) {                       // 4 weights -> 2 registers of fp16 pairs
        const uint32_t v0 = *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 0));
        const uint32_t v1 = *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 1));
        const uint32_t v2 = *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 2));
        const uint32_t v3 = *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 3));
        // entries are fp32 patterns with the value in the upper half: {v0.hi, v1.hi}, {v2.hi, v3.hi}
        return make_uint2(__builtin_amdgcn_perm(v1, v0, 0x07060302u), __builtin_amdgcn_perm(v3, v2, 0x07060302u));
    };
    // One row group: 16 x 512 weights of the chunk -> 16 x 16 partial product.
    auto multiply = [&](const sk_u32x4 (&raw)[8], int grp) {
        sk_f32x4 acc[SETS];
#pragma unroll
        for (int e = 0; e < SETS; ++e) acc[e] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const sk_u32x4 w = raw[q];
            const uint2 p0 = lookup2(w.x), p1 = lookup2(w.y), p2 = lookup2(w.z), p3 = lookup2(w.w);
            const sk_u32x4 b0 = {p0.x, p0.y, p1.x, p1.y}, b1 = {p2.x, p2.y, p3.x, p3.y};
#pragma unroll
            for (int e = 0; e < SETS; ++e) {
                acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[e][2 * q], __builtin_bit_cast(sk_f16x8, b0), acc[e], 0, 0, 0);
                acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[e][2 * q + 1], __builtin_bit_cast(sk_f16x8, b1), acc[e], 0, 0, 0);
            }
        }
        // D layout: lane holds weight row n = lane % 16 and batch rows 16 e + 4 (lane / 16) + r.
        const int n = grp * 16 + m;
        if (n < a.N) {
#pragma unroll
            for (int e = 0; e < SETS; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int b = 16 * e + 4 * g + r;
                    if (b < a.batch) a.partial[((size_t)chunk * a.batch + b) * a.N + n] = acc[e][r];
                }
        }
    };

    // The next group is requested before the current one is decoded (unrolled twice: static buffers).
    for (int grp = g_begin; grp < g_end; grp += 2) {
        if (grp + 1 < g_end) request(rawB, grp + 1);
        multiply(rawA, grp);
        if (grp + 1 >= g_end) break;
        if (grp + 2 < g_end) request(rawA, grp + 2);
        multiply(rawB, grp + 1);
    }
}

// grid = chunks x workgroups per chunk
template <bool FUSED, int SETS, bool RAGGED>
__global__ __launch_bounds__(kSkThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void tq_skinny_kernel(SkinnyArgs a) {
    skinny_body<FUSED, SETS, RAGGED>(a, (int)blockIdx.x, (int)blockIdx.y);
}

// Two or three layers of equal width on the same activation rows (q, k, v or gate, up), one launch:
// the workgroups of a chunk are shared out over the layers by rows (layer j owns blockIdx.y in
// first[j] .. first[j + 1] - 1).
struct SkinnyGroup {
    SkinnyArgs a[3];
    int first[4];
};
template <int SETS, bool RAGGED>
__global__ __launch_bounds__(kSkThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void tq_skinny_group_kernel(SkinnyGroup g) {
    const int b = (int)blockIdx.y;
    const int j = b >= g.first[2] ? 2 : (b >= g.first[1] ? 1 : 0);
    skinny_body<true, SETS, RAGGED>(g.a[j], (int)blockIdx.x, b - g.first[j]);
}

// Nibble planes (dual rotation, primary only): the same scheme on a plane of two weights per
// byte with a 16-entry table.  A work unit is (512-column chunk, plane): units of the primary plane
// use the primary rotation and table, units of the residual plane the residual ones, and the
// reduction kernel adds all units, which is the sum of the two passes.  Blocks of at most 512
// columns only (the workgroup rotates its chunk itself).
struct SkinnyNibbleArgs {
    const void* x;             // activations [batch, K], f32, f16 or bf16
    int x_dtype;
    uint32_t seed[2], block_size;
    float x_scale;             // 1 / sqrt(block_size), applied to the rotated activations before they are rounded
    const uint8_t* plane[2];   // [N, K/2] each; plane[1] unused for primary-only layers
    const float* tables;       // 16 primary centroids, then 16 residual ones
    float* partial;            // [units][batch][N] fp32
    int batch, N, K;
    int units;                 // (K / 512) * planes
    int planes;                // 1 or 2
    int groups;                // ceil(N / 16)
    int wgs_per_unit;
    int groups_q, groups_rem;  // groups / workers and groups % workers (workers = waves sharing a unit)
};

// unit, wg_in_unit: the (chunk, plane) unit of this workgroup and its index among the workgroups that
// share the unit for this layer (a launch may serve several layers).
template <int SETS, bool RAGGED>
__device__ __forceinline__ void skinny_nibble_body(const SkinnyNibbleArgs& a, const int unit, const int wg_in_unit) {
    // The table is indexed by a whole byte of the plane: an entry holds the fp16 centroids of both
    // its nibbles, i.e. one register of the B operand, so two weights cost one table read.
    constexpr int kTabBytes = kSkLutBytes;                 // 256 entries, one private column per lane
    __shared__ __align__(16) char smem[kTabBytes + SETS * kSkStageBytes];   // table | 16 SETS x 512 fp16 rotated activations
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t laneoff = (uint32_t)lane << 2;

    // (unit = chunk * planes + plane; one workgroup per CU)
    const int chunk = a.planes == 2 ? unit >> 1 : unit, pl = a.planes == 2 ? unit & 1 : 0;
    const int m = lane & 15, g = lane >> 4;

    const int me = wg_in_unit * (kSkThreads / 64) + wave;
    const int g_begin = me * a.groups_q + (me < a.groups_rem ? me : a.groups_rem);
    const int g_end = g_begin + a.groups_q + (me < a.groups_rem ? 1 : 0);
    const uint8_t* plane = a.plane[pl];
    const size_t row_bytes = (size_t)a.K >> 1;
    const size_t byte0 = (size_t)chunk * (kSkChunk / 2) + 16 * g;
    auto row_ptr = [&](int grp) {
        int row = grp * 16 + m;
        if (row >= a.N) row = a.N - 1;                     // rows past N re-read row N-1: never stored
        return plane + (size_t)row * row_bytes + byte0;
    };
    // A last chunk that the row does not fill (K a multiple of 128, not of 512): its 128-column pieces past
    // the row are read from piece 0 again and multiply rotated activations that are zero.  Wave-uniform.
    const int pieces = (!RAGGED || a.K - chunk * kSkChunk >= kSkChunk) ? 4 : (a.K - chunk * kSkChunk) >> 7;
    int piece_off[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) piece_off[q] = (!RAGGED || q < pieces) ? 64 * q : 0;

    // Small loads first (they complete in order), then the first row group, which travels while the
    // activations are rotated.
    // Table slots of this thread: slot i = tid + 512 k is entry i >> 4, whose low nibble is the same
    // for all k and whose high nibble is (tid >> 8) + 2 k.
    const float tlo = a.tables[16 * pl + ((tid >> 4) & 15)];
    float thi[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) thi[k] = a.tables[16 * pl + (tid >> 8) + 2 * k];
    TileRaw xin[2 * SETS];
#pragma unroll
    for (int t = 0; t < 2 * SETS; ++t) {                   // batch rows w, w + 8, .. (row 0 again past the batch: not used)
        const int b = wave + 8 * t;
        const int col = chunk * kSkChunk + lane * 8;         // (columns past the row: read column 0, rotated as zeros)
        xin[t] = load_tile_raw(a.x, a.x_dtype, (size_t)(b < a.batch ? b : 0) * a.K, (!RAGGED || col < a.K) ? col : 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    sk_u32x4 rawA[4], rawB[4];                             // two row groups: one decoded, one in flight
    auto request = [&](sk_u32x4 (&raw)[4], int grp) {
        const uint8_t* p = row_ptr(grp);
#pragma unroll
        for (int q = 0; q < 4; ++q) raw[q] = (*reinterpret_cast<const sk_u32x4*>(p + piece_off[q]));
    };
    if (g_begin < g_end) request(rawA, g_begin);

    {                                                       // 256 entries x 16 slots of 16 bytes, values rounded to fp16
        const uint32_t lo = (uint32_t)float_to_f16_bits(tlo);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint32_t v = lo | ((uint32_t)float_to_f16_bits(thi[k]) << 16);
            reinterpret_cast<uint4*>(smem)[tid + k * kSkThreads] = make_uint4(v, v, v, v);
        }
    }
    // Rotate batch rows w, w + 8, .. of the chunk with this plane's seed -> fp16 [16 SETS][512] in LDS.
    constexpr int kPitch = kSkChunk * 2;
    char* const stage = smem + kTabBytes;
#pragma unroll
    for (int t = 0; t < 2 * SETS; ++t) {
        const int b = wave + 8 * t;
        const int col = chunk * kSkChunk + lane * 8;
        uint4 packed = make_uint4(0, 0, 0, 0);
        if (b < a.batch) {                                  // wave-uniform
            float v[8];
            rotate_tile(xin[t], a.x_dtype, col, !RAGGED || col < a.K, a.seed[pl], a.block_size, lane, v);
            packed.x = (uint32_t)float_to_f16_bits(v[0] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[1] * a.x_scale) << 16);
            packed.y = (uint32_t)float_to_f16_bits(v[2] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[3] * a.x_scale) << 16);
            packed.z = (uint32_t)float_to_f16_bits(v[4] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[5] * a.x_scale) << 16);
            packed.w = (uint32_t)float_to_f16_bits(v[6] * a.x_scale) | ((uint32_t)float_to_f16_bits(v[7] * a.x_scale) << 16);
        }
        *reinterpret_cast<uint4*>(stage + b * kPitch + lane * 16) = packed;
    }
    __syncthreads();                                        // table and activations visible
    // A operands.  Matrix step s = 4 q + d multiplies columns 128 q + 32 g + 8 d + [0, 8) of the chunk:
    // the 8 nibbles of dword d of the lane's 16-byte piece q (piece q of lane group g starts at byte
    // 64 q + 16 g of the row's 256 bytes).
    sk_f16x8 afrag[SETS][16];
#pragma unroll
    for (int e = 0; e < SETS; ++e)
#pragma unroll
        for (int s = 0; s < 16; ++s)
            afrag[e][s] = *reinterpret_cast<const sk_f16x8*>(stage + (m + 16 * e) * kPitch + (128 * (s >> 2) + 32 * g + 8 * (s & 3)) * 2);

    // One dword = 8 weights of 8 consecutive columns (low nibble first) -> one B operand: byte j of
    // the dword selects the register that holds columns 2 j and 2 j + 1.
    auto operand = [&](uint32_t w) {
        const sk_u32x4 r = {*reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 0)),
                            *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 1)),
                            *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 2)),
                            *reinterpret_cast<const uint32_t*>(smem + sk_entry_addr(w, laneoff, 3))};
        return __builtin_bit_cast(sk_f16x8, r);
    };
    auto multiply = [&](const sk_u32x4 (&raw)[4], int grp) {
        sk_f32x4 acc[SETS];
#pragma unroll
        for (int e = 0; e < SETS; ++e) acc[e] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const sk_u32x4 w = raw[q];
            const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {                   // one operand, then the matrix instructions that use it
                const sk_f16x8 b = operand(wd[d]);
#pragma unroll
                for (int e = 0; e < SETS; ++e)
                    acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[e][4 * q + d], b, acc[e], 0, 0, 0);
            }
        }
        const int n = grp * 16 + m;
        if (n < a.N) {
#pragma unroll
            for (int e = 0; e < SETS; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int b = 16 * e + 4 * g + r;
                    if (b < a.batch) a.partial[((size_t)unit * a.batch + b) * a.N + n] = acc[e][r];
                }
        }
    };
    // The next group is requested before the current one is decoded (unrolled twice: static buffers).
    for (int grp = g_begin; grp < g_end; grp += 2) {
        if (grp + 1 < g_end) request(rawB, grp + 1);
        multiply(rawA, grp);
        if (grp + 1 >= g_end) break;
        if (grp + 2 < g_end) request(rawA, grp + 2);
        multiply(rawB, grp + 1);
    }
}

// grid = units x workgroups per unit
template <int SETS, bool RAGGED>
__global__ __launch_bounds__(kSkThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void tq_skinny_nibble_kernel(SkinnyNibbleArgs a) {
    skinny_nibble_body<SETS, RAGGED>(a, (int)blockIdx.x, (int)blockIdx.y);
}

// Layers of equal width and mode on the same activation rows, one launch (see SkinnyGroup).
struct SkinnyNibbleGroup {
    SkinnyNibbleArgs a[3];
    int first[4];
};
template <int SETS, bool RAGGED>
__global__ __launch_bounds__(kSkThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void tq_skinny_nibble_group_kernel(SkinnyNibbleGroup g) {
    const int b = (int)blockIdx.y;
    const int j = b >= g.first[2] ? 2 : (b >= g.first[1] ? 1 : 0);
    skinny_nibble_body<SETS, RAGGED>(g.a[j], (int)blockIdx.x, b - g.first[j]);
}

// y[b, n] = norm[n] * out_scale * sum over chunks of partial[c][b][n]
// grid = blocks of 64 columns x batch rows.  The four waves of a block share the chunks of those 64
// columns (wave w takes chunks w, w + 4, ..., eight loads in flight at a time) and add up through
// LDS: a single thread per output walking all chunks four at a time spent one memory latency per
// four chunks, 4.5 us for a kernel that moves a few hundred KB.
__device__ __forceinline__ void skinny_reduce_body(const float* __restrict__ partial, const float* __restrict__ norms,
                                                   void* __restrict__ y, int y_dtype, int N, int chunks,
                                                   float out_scale, const int block) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.y;
    const int n = block * 64 + lane;
    const bool live = n < N;
    const float nrm = live ? norms[n] : 0.0f;
    const float* p = partial + (size_t)b * N + (live ? n : 0);
    const size_t step = (size_t)gridDim.y * N;          // one chunk: [batch][N]
    float s[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    int c = wave;
    for (; c + 28 < chunks; c += 32) {
#pragma unroll
        for (int k = 0; k < 8; ++k) s[k] += p[(size_t)(c + 4 * k) * step];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
        if (c + 4 * k < chunks) s[k] += p[(size_t)(c + 4 * k) * step];
    part[wave][lane] = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    __syncthreads();
    if (wave == 0 && live) {
        const float t = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
        store_scalar(y, y_dtype, (size_t)b * N + n, t * (out_scale * nrm));
    }
}

__global__ __launch_bounds__(256) void tq_skinny_reduce_kernel(const float* __restrict__ partial,
                                                               const float* __restrict__ norms, void* __restrict__ y,
                                                               int y_dtype, int batch, int N, int chunks, float out_scale) {
    skinny_reduce_body(partial, norms, y, y_dtype, N, chunks, out_scale, (int)blockIdx.x);
}

struct SkinnyReduceGroup {
    const float* partial[3];
    const float* norms[3];
    void* y[3];
    int N[3];
    float out_scale[3];
    int first[4];              // layer j owns blockIdx.x in first[j] .. first[j + 1] - 1
    int y_dtype, chunks;
};
__global__ __launch_bounds__(256) void tq_skinny_reduce_group_kernel(SkinnyReduceGroup r) {
    const int b = (int)blockIdx.x;
    const int j = b >= r.first[2] ? 2 : (b >= r.first[1] ? 1 : 0);
    skinny_reduce_body(r.partial[j], r.norms[j], r.y[j], r.y_dtype, r.N[j], r.chunks, r.out_scale[j], b - r.first[j]);
}

static bool skinny_nibble(const LayerView& L) {
    return (L.mode == kDual || L.mode == kPrimaryOnly) && L.block_size <= (uint32_t)kSkChunk;
}

bool skinny_supported(const LayerView& L, int x_dtype, int batch) {
    if (batch < 2 || batch > kSkMaxRows) return false;                                   // (any activation type)
    // whole 64-column pieces (nibble planes: 128-column pieces); a row that does not fill its last 512-column
    // chunk has blocks of at most 256 columns, which the workgroup rotates itself
    if (L.in_features % ((L.mode == kSharedLut) ? 64 : 128) != 0) return false;
    if (!lanes_supported(L.in_features, L.block_size)) return false;
    if (!L.fp16_centroids_ok) return false;                   // decoded weights are kept in fp16
    return (L.mode == kSharedLut && L.packed_combined) || skinny_nibble(L);
}

size_t skinny_partial_bytes(const LayerView& L, int batch) {
    const size_t units = (size_t)((L.in_features + kSkChunk - 1) / kSkChunk) * (L.mode == kDual ? 2 : 1);
    return units * (size_t)batch * L.out_features * sizeof(float);
}

// Rotated-activation workspace of launch_skinny: only layers with blocks wider than a chunk go
// through the separate rotation kernel; everything else rotates inside the kernel.
size_t skinny_workspace_bytes(const LayerView& L, int batch) {
    if (skinny_nibble(L) || L.block_size <= (uint32_t)kSkChunk) return 0;
    return prefill_workspace_bytes(L, batch);
}

// xt_workspace: skinny_workspace_bytes (may be NULL when that is 0); partial: skinny_partial_bytes.
hipError_t launch_skinny(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                         void* xt_workspace, float* partial, int num_cus, hipStream_t stream) {
    if (skinny_nibble(L)) {
        SkinnyNibbleArgs n{};
        n.x = x; n.x_dtype = x_dtype; n.seed[0] = L.seed_primary; n.seed[1] = L.seed_residual; n.block_size = L.block_size;
        n.x_scale = L.inv_sqrt_bs;
        n.plane[0] = L.packed_primary; n.plane[1] = L.packed_residual;
        n.tables = L.tables;
        n.partial = partial;
        n.batch = batch; n.N = L.out_features; n.K = L.in_features;
        n.planes = L.mode == kDual ? 2 : 1;
        n.units = (L.in_features + kSkChunk - 1) / kSkChunk * n.planes;
        n.groups = (L.out_features + 15) / 16;
        n.wgs_per_unit = num_cus / n.units > 0 ? num_cus / n.units : 1;   // one workgroup per CU
        const int workers_n = n.wgs_per_unit * (kSkThreads / 64);
        n.groups_q = n.groups / workers_n;
        n.groups_rem = n.groups % workers_n;
        const dim3 grid_n(n.units, n.wgs_per_unit);
        const bool two = batch > 16, ragged = L.in_features % kSkChunk != 0;
        if (two && ragged) hipLaunchKernelGGL((tq_skinny_nibble_kernel<2, true>), grid_n, dim3(kSkThreads), 0, stream, n);
        else if (two) hipLaunchKernelGGL((tq_skinny_nibble_kernel<2, false>), grid_n, dim3(kSkThreads), 0, stream, n);
        else if (ragged) hipLaunchKernelGGL((tq_skinny_nibble_kernel<1, true>), grid_n, dim3(kSkThreads), 0, stream, n);
        else hipLaunchKernelGGL((tq_skinny_nibble_kernel<1, false>), grid_n, dim3(kSkThreads), 0, stream, n);
        hipError_t en = hipGetLastError();
        if (en != hipSuccess) return en;
        const unsigned blocks_n = (unsigned)((L.out_features + 63) / 64);
        hipLaunchKernelGGL(tq_skinny_reduce_kernel, dim3(blocks_n, batch), dim3(256), 0, stream,
                           partial, L.norms, y, y_dtype, batch, L.out_features, n.units, L.inv_scale);
        return hipGetLastError();
    }
    const bool fused = L.block_size <= (uint32_t)kSkChunk;
    hipError_t e = hipSuccess;
    if (!fused) {
        e = launch_rotate_tiles(L, x, x_dtype, batch, xt_workspace, stream);
        if (e != hipSuccess) return e;
    }
    SkinnyArgs a{};
    a.x = x; a.x_dtype = x_dtype; a.seed = L.seed_primary; a.block_size = L.block_size; a.x_scale = L.inv_sqrt_bs;
    a.xt = static_cast<const uint16_t*>(xt_workspace);
    a.plane = L.packed_combined;
    a.tables = L.tables;
    a.partial = partial;
    a.batch = batch; a.N = L.out_features; a.K = L.in_features;
    a.chunks = (L.in_features + kSkChunk - 1) / kSkChunk;
    a.groups = (L.out_features + 15) / 16;
    a.wgs_per_chunk = num_cus / a.chunks > 0 ? num_cus / a.chunks : 1;   // one workgroup per CU
    const int workers = a.wgs_per_chunk * (kSkThreads / 64);
    a.groups_q = a.groups / workers;
    a.groups_rem = a.groups % workers;
    const dim3 grid(a.chunks, a.wgs_per_chunk);
    const bool two = batch > 16, ragged = L.in_features % kSkChunk != 0;     // (ragged rows have blocks <= 256: fused)
    if (fused && ragged && two) hipLaunchKernelGGL((tq_skinny_kernel<true, 2, true>), grid, dim3(kSkThreads), 0, stream, a);
    else if (fused && ragged) hipLaunchKernelGGL((tq_skinny_kernel<true, 1, true>), grid, dim3(kSkThreads), 0, stream, a);
    else if (fused && two) hipLaunchKernelGGL((tq_skinny_kernel<true, 2, false>), grid, dim3(kSkThreads), 0, stream, a);
    else if (fused) hipLaunchKernelGGL((tq_skinny_kernel<true, 1, false>), grid, dim3(kSkThreads), 0, stream, a);
    else if (two) hipLaunchKernelGGL((tq_skinny_kernel<false, 2, false>), grid, dim3(kSkThreads), 0, stream, a);
    else hipLaunchKernelGGL((tq_skinny_kernel<false, 1, false>), grid, dim3(kSkThreads), 0, stream, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    const unsigned blocks = (unsigned)((L.out_features + 63) / 64);
    hipLaunchKernelGGL(tq_skinny_reduce_kernel, dim3(blocks, batch), dim3(256), 0, stream,
                       partial, L.norms, y, y_dtype, batch, L.out_features, a.chunks, L.inv_scale);
    return hipGetLastError();
}

// Layers that can share the two launches: two or three layers of equal width and mode with blocks
// of at most 512 columns (the workgroup rotates its chunk itself), 2..32 rows,
// and at least one workgroup per work unit and layer.
bool skinny_group_supported(const LayerView* Ls, int n, int x_dtype, int batch, int num_cus) {
    if (n < 2 || n > 3) return false;
    const bool nibble = Ls[0].mode == kDual || Ls[0].mode == kPrimaryOnly;
    for (int j = 0; j < n; ++j) {
        if (Ls[j].mode != Ls[0].mode || Ls[j].block_size > (uint32_t)kSkChunk) return false;
        if (!nibble && (Ls[j].mode != kSharedLut || !Ls[j].packed_combined)) return false;
        if (Ls[j].in_features != Ls[0].in_features || !skinny_supported(Ls[j], x_dtype, batch)) return false;
    }
    const int units = (Ls[0].in_features + kSkChunk - 1) / kSkChunk * (Ls[0].mode == kDual ? 2 : 1);
    return num_cus / units >= n;
}

hipError_t launch_skinny_group(const LayerView* Ls, int n, const void* x, int x_dtype, int batch, void* const* ys,
                               int y_dtype, float* const* partials, int num_cus, hipStream_t stream) {
    const bool nibble = Ls[0].mode == kDual || Ls[0].mode == kPrimaryOnly;
    const int planes = Ls[0].mode == kDual ? 2 : 1;
    const int K = Ls[0].in_features, chunks = (K + kSkChunk - 1) / kSkChunk * planes;   // work units: (chunk, plane)
    const int total_wgs = num_cus / chunks;                       // workgroups per unit, all layers together
    long long rows = 0;
    for (int j = 0; j < n; ++j) rows += Ls[j].out_features;
    int wgs[3] = {0, 0, 0}, used = 0;
    for (int j = 0; j < n; ++j) {
        wgs[j] = (int)((long long)total_wgs * Ls[j].out_features / rows);
        if (wgs[j] < 1) wgs[j] = 1;
        used += wgs[j];
    }
    for (int j = 0; used < total_wgs; j = (j + 1) % n) { ++wgs[j]; ++used; }
    for (int j = 0; used > total_wgs; j = (j + 1) % n) if (wgs[j] > 1) { --wgs[j]; --used; }
    SkinnyGroup g{};
    SkinnyNibbleGroup gn{};
    SkinnyReduceGroup r{};
    g.first[0] = 0; gn.first[0] = 0; r.first[0] = 0;
    for (int j = 0; j < 3; ++j) {
        if (j < n) {
            const LayerView& L = Ls[j];
            SkinnyNibbleArgs& q = gn.a[j];
            q.x = x; q.x_dtype = x_dtype; q.seed[0] = L.seed_primary; q.seed[1] = L.seed_residual; q.block_size = L.block_size;
            q.x_scale = L.inv_sqrt_bs;
            q.plane[0] = L.packed_primary; q.plane[1] = L.packed_residual;
            q.tables = L.tables;
            q.partial = partials[j];
            q.batch = batch; q.N = L.out_features; q.K = K;
            q.planes = planes;
            q.units = chunks;
            q.groups = (L.out_features + 15) / 16;
            q.wgs_per_unit = wgs[j];
            q.groups_q = q.groups / (wgs[j] * (kSkThreads / 64));
            q.groups_rem = q.groups % (wgs[j] * (kSkThreads / 64));
            gn.first[j + 1] = gn.first[j] + wgs[j];
            SkinnyArgs& a = g.a[j];
            a.x = x; a.x_dtype = x_dtype; a.seed = L.seed_primary; a.block_size = L.block_size; a.x_scale = L.inv_sqrt_bs;
            a.xt = nullptr;
            a.plane = L.packed_combined;
            a.tables = L.tables;
            a.partial = partials[j];
            a.batch = batch; a.N = L.out_features; a.K = K;
            a.chunks = chunks;
            a.groups = (L.out_features + 15) / 16;
            a.wgs_per_chunk = wgs[j];
            const int workers = wgs[j] * (kSkThreads / 64);
            a.groups_q = a.groups / workers;
            a.groups_rem = a.groups % workers;
            r.partial[j] = partials[j]; r.norms[j] = L.norms; r.y[j] = ys[j]; r.N[j] = L.out_features;
            r.out_scale[j] = L.inv_scale;
            g.first[j + 1] = g.first[j] + wgs[j];
            r.first[j + 1] = r.first[j] + (L.out_features + 63) / 64;
        } else {
            g.first[j] = 1 << 30; g.first[j + 1] = 1 << 30;       // no workgroup reaches an unused slot
            gn.first[j] = 1 << 30; gn.first[j + 1] = 1 << 30;
            r.first[j] = 1 << 30; r.first[j + 1] = 1 << 30;
        }
    }
    int reduce_blocks = 0;
    for (int j = 0; j < n; ++j) reduce_blocks += (Ls[j].out_features + 63) / 64;
    r.y_dtype = y_dtype; r.chunks = chunks;
    const dim3 grid(chunks, used);
    const bool two = batch > 16, ragged = K % kSkChunk != 0;
    if (nibble) {
        if (two && ragged) hipLaunchKernelGGL((tq_skinny_nibble_group_kernel<2, true>), grid, dim3(kSkThreads), 0, stream, gn);
        else if (two) hipLaunchKernelGGL((tq_skinny_nibble_group_kernel<2, false>), grid, dim3(kSkThreads), 0, stream, gn);
        else if (ragged) hipLaunchKernelGGL((tq_skinny_nibble_group_kernel<1, true>), grid, dim3(kSkThreads), 0, stream, gn);
        else hipLaunchKernelGGL((tq_skinny_nibble_group_kernel<1, false>), grid, dim3(kSkThreads), 0, stream, gn);
    } else {
        if (two && ragged) hipLaunchKernelGGL((tq_skinny_group_kernel<2, true>), grid, dim3(kSkThreads), 0, stream, g);
        else if (two) hipLaunchKernelGGL((tq_skinny_group_kernel<2, false>), grid, dim3(kSkThreads), 0, stream, g);
        else if (ragged) hipLaunchKernelGGL((tq_skinny_group_kernel<1, true>), grid, dim3(kSkThreads), 0, stream, g);
        else hipLaunchKernelGGL((tq_skinny_group_kernel<1, false>), grid, dim3(kSkThreads), 0, stream, g);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(tq_skinny_reduce_group_kernel, dim3(reduce_blocks, batch), dim3(256), 0, stream, r);
    return hipGetLastError();
}

}  // namespace tq
