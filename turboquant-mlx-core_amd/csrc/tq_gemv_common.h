// Pieces shared by the batch-1..4 kernels of the fused TQ8 forward (tq_gemv.hip, tq_gemv_wide.hip):
// launch arguments, the transposed wave reduction, the lane-private table lookup, the rotation
// of one 512-column activation tile and the layout of the rotated-activation image in LDS.
#pragma once
#include "tq_device.h"

namespace tq {

struct GemvArgs {
    LayerView L;
    const void* x;
    void* y;
    int x_dtype, y_dtype;
    int chunks;      // in / 32
    int W, S;        // slabs per row, row streams per workgroup
    int iters;       // uniform trip count: ceil(longest row range / R)
    float out_scale; // inv_scale * inv_sqrt_bs
    const float* gate;   // optional [batch, out] fp32: the stored value becomes silu(gate) * y (gated MLP)
    int img_cols;    // wide kernel only: columns of the rotated-activation image in LDS (a multiple of 2048)
    int rows_q, rows_rem;   // rows per row range, and how many ranges hold one more
    int w_inv;       // (w * w_inv) >> 8 == w / W
    int pre_rotated; // narrow kernel: x holds fp32 rotated activations (second rotation in_features further on)
    const float* x_gate;  // optional fp32 [in]: the row to multiply is silu(x_gate) * x (x fp32; rows wider than 16384 columns)
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// y, or silu(g) * y = g / (1 + exp(-g)) * y when a gate vector is given (fp32, as between the
// linears of a gated MLP block).
__device__ __forceinline__ float apply_gate(const float* gate, size_t idx, float y) {
    if (!gate) return y;
    const float g = gate[idx];
    return g / (1.0f + expf(-g)) * y;
}

// 128-bit streaming load (weights are read exactly once).
__device__ __forceinline__ uint4 load_stream16(const uint8_t* p) {
    const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
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

// The same with bits 16..23 of laneoff kept: (table << 16) | (entry << 8) | (lane << 2), for 64 KB
// tables that follow each other in LDS.
template <int J>
__device__ __forceinline__ uint32_t entry_addr_hi(uint32_t idx_bytes, uint32_t laneoff) {
    return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c020000u | ((4u + J) << 8));
}

__device__ __forceinline__ float lds_f32(const char* lds, uint32_t byte_addr) {
    return *reinterpret_cast<const float*>(lds + byte_addr);
}

// Centroid values of the 32 columns a lane owns.
//   LUT256: P, Q are the lane's 32 combined bytes (residual_nibble << 4 | primary_nibble, one per
//           column); each byte indexes the 256-entry sum table of shared rotation
//           (reference src/dequantizer.cpp:144-169).
//   else  : P holds 32 nibbles of one plane (lo nibble = even column); 16-entry table at TABLE_OFF.
//           table_bits: 0, or 0x10101010 for the 16-entry table that follows the first one (entry
//           numbers 16..31; selecting the table in the index costs one OR per eight lookups, a table
//           base that is not a constant one addition per lookup).
template <bool LUT256, int TABLE_OFF>
__device__ __forceinline__ void lookup32(const uint4& P, const uint4& Q, const char* lds, uint32_t laneoff,
                                         float (&val)[kChunk], uint32_t table_bits = 0) {
    const char* tab = lds + TABLE_OFF;
    if constexpr (LUT256) {
        const uint32_t w[8] = {P.x, P.y, P.z, P.w, Q.x, Q.y, Q.z, Q.w};
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            val[4 * d + 0] = lds_f32(tab, entry_addr<0>(w[d], laneoff));
            val[4 * d + 1] = lds_f32(tab, entry_addr<1>(w[d], laneoff));
            val[4 * d + 2] = lds_f32(tab, entry_addr<2>(w[d], laneoff));
            val[4 * d + 3] = lds_f32(tab, entry_addr<3>(w[d], laneoff));
        }
    } else {
        const uint32_t pw[4] = {P.x, P.y, P.z, P.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t ce = (pw[d] & 0x0F0F0F0Fu) | table_bits;
            const uint32_t co = ((pw[d] >> 4) & 0x0F0F0F0Fu) | table_bits;
            val[8 * d + 0] = lds_f32(tab, entry_addr<0>(ce, laneoff));
            val[8 * d + 1] = lds_f32(tab, entry_addr<0>(co, laneoff));
            val[8 * d + 2] = lds_f32(tab, entry_addr<1>(ce, laneoff));
            val[8 * d + 3] = lds_f32(tab, entry_addr<1>(co, laneoff));
            val[8 * d + 4] = lds_f32(tab, entry_addr<2>(ce, laneoff));
            val[8 * d + 5] = lds_f32(tab, entry_addr<2>(co, laneoff));
            val[8 * d + 6] = lds_f32(tab, entry_addr<3>(ce, laneoff));
            val[8 * d + 7] = lds_f32(tab, entry_addr<3>(co, laneoff));
        }
    }
}

constexpr int kLut256Bytes = 256 * 256;          // 256 entries x 64 lanes x 4 B
constexpr int kTab16Bytes = 16 * 256;
constexpr int kRegionBytes = kLut256Bytes;       // decode tables
constexpr int kRegionFloats = kRegionBytes / 4;
constexpr int kPartialBytes = 2 * 16 * 16 * 4;   // [2 buffers][<=16 waves][<=16 values]
constexpr int kStageBytes = kSlab * 4;           // one slab image of rotated activations
constexpr int kTile = 512;                       // columns rotated by one wave in the prologue (8 per lane)

// Rotate one 512-column tile of an activation row: lane owns 8 consecutive columns.
// Valid for block sizes up to 512 (a block never straddles a tile).  The raw load is split
// from the arithmetic so that a wave can have the loads of all its tiles in flight at once.
struct TileRaw { uint4 a, b; };

__device__ __forceinline__ TileRaw load_tile_raw(const void* x, int x_dtype, size_t row_off, int col) {
    TileRaw r;
    if (x_dtype == kF32) {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const float*>(x) + row_off + col);
        r.a = p[0]; r.b = p[1];
    } else {
        r.a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(x) + row_off + col);
        r.b = make_uint4(0, 0, 0, 0);
    }
    return r;
}

__device__ __forceinline__ void rotate_tile(const TileRaw& raw, int x_dtype, int col, bool active,
                                            uint32_t seed, uint32_t bs, int lane, float (&v)[8]) {
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
        for (int j = 0; j < 8; ++j) v[j] *= sign_of(seed, ((uint32_t)col + j) & (bs - 1));
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = 0.0f;
    }
    fwht_lanes<8>(v, bs, lane);
}

// Column ownership.  A lane owns two runs of 16 columns inside its wave's 2048-column slab:
//   SPLIT (combined byte plane): columns 16*lane.. and 1024 + 16*lane..  so that each of the
//          lane's two 16-byte loads is contiguous across the wave (1 KB per load instruction);
//   else  (nibble planes): columns 32*lane.. and 32*lane + 16..  (one 16-byte load per plane).
// Value k (0..31) of lane l sits at float index k*64 + l of the slab's staging image.
template <bool SPLIT>
__device__ __forceinline__ int stage_index(int col_in_slab) {
    if constexpr (SPLIT) {
        const int h = col_in_slab >> 10, rem = col_in_slab & 1023;
        return ((h << 4) + (rem & 15)) * kWave + (rem >> 4);
    } else {
        return (col_in_slab & 31) * kWave + (col_in_slab >> 5);
    }
}

// One batch row, rows of up to 8 slabs (tq_gemv_wide.hip): one workgroup per CU, tables and rotated
// activations built once per CU.  `a` as for the narrow kernel (x, y, gate already at the batch row).
bool gemv_wide_supported(const LayerView& L, int num_cus, bool pre_rotated = false);
hipError_t launch_gemv_wide(const GemvArgs& a, int num_cus, hipStream_t stream);
// Two or three layers of equal width and mode reading the same activation row, one launch.
bool gemv_wide_group_supported(const LayerView* Ls, int n, int num_cus);
hipError_t launch_gemv_wide_group(const GemvArgs* as, int n, int num_cus, hipStream_t stream);

}  // namespace tq
