// Internal declarations shared by the gfx950 kernels and the C-ABI layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

namespace tq {

// Activation / output element types (same numbering as TQ_DTYPE_* in tq_linear.h).
enum : int { kF32 = 0, kF16 = 1, kBF16 = 2 };

// Decode modes (same numbering as TQ_MODE_* in tq_linear.h).
enum : int {
    kPrimaryOnly = 0, kSharedLut = 1, kDual = 2,
    kShared5 = 3, kPrimaryOnly5 = 4, kDual5 = 5
};

constexpr int kWave = 64;          // gfx950 wavefront width
constexpr int kChunk = 32;         // columns owned by one lane (16 packed bytes)
constexpr int kSlab = kWave * kChunk;   // columns covered by one wave

// Device-side description of one TQ8 layer.
struct LayerView {
    const uint8_t* packed_primary;   // [out, in/2] nibble pairs (or [out, in] bytes for 5-bit)
    const uint8_t* packed_residual;  // [out, in/2]
    const uint8_t* packed_combined;  // shared-rotation 4-bit mode only: [out, in], one byte per weight =
                                     // residual_nibble << 4 | primary_nibble (the LUT index of reference
                                     // src/dequantizer.cpp:163-169); the two planes above are then NULL
    const float*   norms;            // [out]
    const float*   tables;           // decode tables, layout depends on mode (see build_tables)
    int out_features;
    int in_features;
    uint32_t block_size;
    uint32_t seed_primary;
    uint32_t seed_residual;
    int mode;
    float inv_scale;                 // 1/sqrt(in), computed on the host as the reference does
    float inv_sqrt_bs;               // 1/sqrt(block_size), host computed
    int fp16_centroids_ok;           // every centroid fits fp16 with room to spare (the byte-pair tables of the
                                     // batch-1 kernel hold fp16 values); otherwise fp32 tables are used
    float* xrot_work;                // scratch of 2 * in_features floats (rows wider than 16384 columns: the
                                     // batch-1 path rotates the activations once, in a kernel of its own), or NULL
};

// Launchers (tq_gemv.hip, tq_dequant.hip).  All return hipError_t of the launch.
// gate (optional, fp32 [batch, out]): store silu(gate) * y instead of y.
// x_gate (optional, fp32 [in], batch 1, x fp32): the layer is applied to silu(x_gate) * x; only where
// gemv_x_gate_supported() says so (the product is formed by the kernel that rotates the row).
hipError_t launch_gemv(const LayerView& L, const void* x, int x_dtype, int batch,
                       void* y, int y_dtype, int num_cus, hipStream_t stream, const float* gate = nullptr,
                       const float* x_gate = nullptr);
bool gemv_x_gate_supported(const LayerView& L);
// out[i] = silu(gate[i]) * up[i] over n fp32 values, written as out_dtype (gated MLP, batched path).
hipError_t launch_silu_mul(const float* gate, const float* up, void* out, int out_dtype, size_t n, hipStream_t stream);
// out[i] = a[i] + b[i] over n fp32 values, written as out_dtype (out may be a).
hipError_t launch_add(const float* a, const float* b, void* out, int out_dtype, size_t n, hipStream_t stream);
hipError_t launch_combine_planes5(const uint8_t* primary, const uint8_t* residual, uint8_t* combined,
                                  size_t residual_bytes, int n_primary, int n_residual, hipStream_t stream);
hipError_t launch_dequant(const LayerView& L, void* w, int w_dtype, hipStream_t stream);
// Prefill (tq_prefill.hip): rotate the activations to fp16 in `workspace`, then dequant + MFMA GEMM.
bool prefill_supported(const LayerView& L, int x_dtype, int batch);
size_t prefill_workspace_bytes(const LayerView& L, int batch);        // the rotated activations (tile images) alone
// K ranges of a call (splits > 1: few output tiles), their length in 32-column steps, and the workspace: tile
// images (xt_bytes, rounded up to 256) followed by splits x [batch, out] fp32 products.
struct PrefillPlan { int splits; int steps_per_split; size_t xt_bytes; size_t total_bytes; };
PrefillPlan prefill_plan(const LayerView& L, int batch, int num_cus, size_t capacity);
size_t prefill_reserve_bytes(const LayerView& L, int max_batch, int num_cus);
hipError_t launch_prefill(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                          void* workspace, const PrefillPlan& plan, hipStream_t stream);
// panel: fragment images of 512 rows for tq_prefill_panel_kernel instead of 256-row tile images.
hipError_t launch_rotate_tiles(const LayerView& L, const void* x, int x_dtype, int batch, void* workspace,
                               hipStream_t stream, bool panel = false);
// Small batches (tq_skinny.hip): 2..32 rows (any activation type) on shared-rotation layers, batch rows as
// the M side of 16x16x32 MFMAs.  xt_workspace as for launch_prefill; partial: skinny_partial_bytes() for this batch.
constexpr int kSkinnyMaxRows = 32;
bool skinny_supported(const LayerView& L, int x_dtype, int batch);
size_t skinny_partial_bytes(const LayerView& L, int batch);
size_t skinny_workspace_bytes(const LayerView& L, int batch);
hipError_t launch_skinny(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                         void* xt_workspace, float* partial, int num_cus, hipStream_t stream);
// Two or three shared-rotation layers of equal width on the same activation rows: both launches shared.
bool skinny_group_supported(const LayerView* Ls, int n, int x_dtype, int batch, int num_cus);
hipError_t launch_skinny_group(const LayerView* Ls, int n, const void* x, int x_dtype, int batch, void* const* ys,
                               int y_dtype, float* const* partials, int num_cus, hipStream_t stream);
// Two to twelve rows (tq_gemv_few.hip): the batch-1 kernel's shape (whole weight rows per
// stream, no cut along K, no second kernel), four weight rows by four activation rows per 4x4x4 matrix block.
// workspace: gemv_few_workspace_bytes() (0 for most calls of up to four rows: the workgroups rotate the rows
// themselves); a group needs that of its first layer once per layer.
bool gemv_few_supported(const LayerView& L, int batch, int num_cus);
size_t gemv_few_workspace_bytes(const LayerView& L, int batch);
hipError_t launch_gemv_few(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                           void* workspace, int num_cus, hipStream_t stream);
bool gemv_few_group_supported(const LayerView* Ls, int n, int batch, int num_cus);
hipError_t launch_gemv_few_group(const LayerView* Ls, int n, const void* x, int x_dtype, int batch, void* const* ys,
                                 int y_dtype, void* workspace, int num_cus, hipStream_t stream);
hipError_t launch_wht(const float* in, float* out, int rows, int cols, uint32_t seed,
                      uint32_t block_size, float inv_sqrt_bs, int inverse, hipStream_t stream);
hipError_t launch_any_nonzero(const uint8_t* data, size_t n, int* flag_dev, hipStream_t stream);
hipError_t launch_combine_planes(const uint8_t* primary, const uint8_t* residual, uint8_t* combined,
                                 size_t plane_bytes, hipStream_t stream);

// Host-side error reporting shared by the C-ABI translation units (thread-local message).
void set_error(const std::string& msg);
bool hip_ok(hipError_t e, const char* what);

// Offline quantizer (tq_quantize.hip).
struct QuantArgsHost {
    const float* w; float* orig_norm; double* recon_partial; float* scaled_out;
    uint8_t* packed_primary; uint8_t* packed_residual;
    const float* tables;     // device: [0..31] cP, [32..62] bP, [64..79] cR, [80..94] bR
    int out, in, n_primary, n_residual, primary_bits, residual_bits, shared_rotation;
    uint32_t bs, seed_p, seed_r;
    float scale_factor, inv_scale, inv_sqrt_bs;
    int quantize;            // 0: only emit the rotated * sqrt(in) samples
};
hipError_t launch_row_norms(const float* w, float* norms, int out, int in, hipStream_t stream);
hipError_t launch_derive_seeds(const float* w, size_t n_floats, uint32_t* seeds_dev, hipStream_t stream);
hipError_t launch_quantize_rows(const QuantArgsHost& h, hipStream_t stream);
int quantize_partials_per_row(int in, uint32_t bs);      // doubles per row of recon_partial / launch_finish_norms' `slabs`
hipError_t launch_finish_norms(const float* orig, const double* partial, float* norms, int out, int slabs,
                               hipStream_t stream);
hipError_t launch_lloyd_pass(const float* data, size_t n, const float* bounds_dev, int nc, int subtract,
                             const float* gcent_dev, const float* gbounds_dev, int ngc,
                             double* part_sum, unsigned long long* part_cnt, int workgroups, hipStream_t stream);

hipError_t launch_codebook_quantize(const float* values, size_t n, const float* bounds_dev, int nc, uint8_t* indices,
                                    hipStream_t stream);
hipError_t launch_codebook_lookup(const uint8_t* indices, size_t n, const float* centroids_dev, int nc, float* values,
                                  hipStream_t stream);

// Generic kernels (tq_generic.hip): any even width that is a multiple of a power-of-two block of 1 to 2048
// columns, all six modes.  Forward through the layer's fp32 scratch row (xrot_work); dequantiser and
// rotation for blocks of at most 16 columns (widths that are not a multiple of 32).
bool generic_supported(const LayerView& L);
hipError_t launch_gemv_generic(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                               int num_cus, hipStream_t stream, const float* gate);
hipError_t launch_dequant_small(const LayerView& L, void* w, int w_dtype, hipStream_t stream);
hipError_t launch_wht_small(const float* in, float* out, int rows, int cols, uint32_t seed, uint32_t block_size,
                            float inv_sqrt_bs, int inverse, hipStream_t stream);

// What the layout itself requires (the reference's only rule is in % block_size == 0,
// src/rotation.cpp:374,396; its butterfly needs a power of two): blocks of 1 to 2048 columns, an even width.
inline bool layout_valid(int in_features, uint32_t block_size) {
    if (in_features <= 0 || (in_features & 1)) return false;
    if (block_size < 1 || block_size > 2048 || (block_size & (block_size - 1))) return false;
    return in_features % (int)block_size == 0;
}

// True when the wave-per-slab kernels (a lane owns 32 consecutive columns) can handle this shape:
// dequantiser, rotation, quantizer, prefill and small-batch kernels.
inline bool lanes_supported(int in_features, uint32_t block_size) {
    return layout_valid(in_features, block_size) && block_size >= 2 && in_features % kChunk == 0;
}

// True when the batch-1..4 kernels can: additionally at most 16 slabs of 2048 columns per row.
inline bool shape_supported(int in_features, uint32_t block_size) {
    return lanes_supported(in_features, block_size) && in_features <= 16 * kSlab;
}

// ---------------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------------

// +-1 from a u32 hash of (seed, index inside the block); reference
// src/rotation.cpp:32-42 and metal/turboquant_dequant_mm.metal:57-61.
__device__ __forceinline__ float sign_of(uint32_t seed, uint32_t index) {
    uint32_t h = seed * 2654435761u + index * 2246822519u;
    h ^= h >> 16;
    h *= 0x45d9f3bu;
    h ^= h >> 16;
    return (h & 1u) ? 1.0f : -1.0f;
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Value held by lane (lane ^ MASK), without touching LDS:
//   1, 2 : DPP quad_perm;  4 : row_shr:4 / row_shl:4 written under complementary bank masks;
//   8    : DPP row_ror:8;  16, 32 : v_permlane16_swap / v_permlane32_swap (gfx950) plus a select.
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
    if constexpr (MASK == 1) return dpp_mov<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (MASK == 2) return dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (MASK == 4) {
        const int iv = __builtin_bit_cast(int, v);
        int a = __builtin_amdgcn_update_dpp(iv, iv, 0x114, 0xf, 0xa, false);   // row_shr:4 -> lanes with bit 2 set
        a = __builtin_amdgcn_update_dpp(a, iv, 0x104, 0xf, 0x5, false);        // row_shl:4 -> lanes with bit 2 clear
        return __builtin_bit_cast(float, a);
    }
    else if constexpr (MASK == 8) return dpp_mov<0x128>(v);  // row_ror:8
    else if constexpr (MASK == 16) {
        const unsigned u = __builtin_bit_cast(unsigned, v);
        const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        return __builtin_bit_cast(float, (__lane_id() & 16) ? r[0] : r[1]);
    } else {
        static_assert(MASK == 32, "lane_xor: unsupported mask");
        const unsigned u = __builtin_bit_cast(unsigned, v);
        const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        return __builtin_bit_cast(float, (__lane_id() & 32) ? r[0] : r[1]);
    }
}

// One cross-lane butterfly stage over N values per lane: the lower lane of a pair
// gets a+b, the upper lane a-b.  fma(v, +-1, partner) is exact, so the result is
// bit-identical to the add/sub of the CPU butterfly.
template <int MASK, int N>
__device__ __forceinline__ void butterfly_lanes(float (&v)[N], int lane) {
    const float sgn = (lane & MASK) ? -1.0f : 1.0f;
#pragma unroll
    for (int k = 0; k < N; ++k) v[k] = __builtin_fmaf(v[k], sgn, lane_xor<MASK>(v[k]));
}

// Unnormalised natural-order Walsh-Hadamard butterfly over a block that is
// spread as N consecutive values per lane over bs/N neighbouring lanes (or lives
// entirely inside the lane when bs <= N).  Stage order and the (a+b, a-b)
// convention are those of reference src/rotation.cpp:14-25, so the result is
// bit-identical to the CPU butterfly.
template <int N>
__device__ __forceinline__ void fwht_lanes(float (&v)[N], uint32_t bs, int lane) {
#pragma unroll
    for (int h = 1; h < N; h <<= 1) {
        if ((uint32_t)h < bs) {
#pragma unroll
            for (int i = 0; i < N; i += 2 * h) {
#pragma unroll
                for (int j = i; j < i + h; ++j) {
                    float a = v[j], b = v[j + h];
                    v[j] = a + b;
                    v[j + h] = a - b;
                }
            }
        }
    }
    if ((uint32_t)N * 1 < bs) butterfly_lanes<1, N>(v, lane);
    if ((uint32_t)N * 2 < bs) butterfly_lanes<2, N>(v, lane);
    if ((uint32_t)N * 4 < bs) butterfly_lanes<4, N>(v, lane);
    if ((uint32_t)N * 8 < bs) butterfly_lanes<8, N>(v, lane);
    if ((uint32_t)N * 16 < bs) butterfly_lanes<16, N>(v, lane);
    if ((uint32_t)N * 32 < bs) butterfly_lanes<32, N>(v, lane);
}

__device__ __forceinline__ void fwht_lane32(float (&v)[kChunk], uint32_t bs, int lane) {
    fwht_lanes<kChunk>(v, bs, lane);
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) {
    return __builtin_bit_cast(float, b << 16);
}

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// fp32 -> fp16 bit pattern, round to nearest even; values beyond the largest finite fp16 saturate (a
// rotated activation that large has left the range the reference's own f16 cast of the input covers,
// src/dequantizer.cpp:691).  The matrix-core paths keep decoded weights and rotated activations in fp16.
__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
    const float c = (f != f) ? f : __builtin_fminf(__builtin_fmaxf(f, -65504.0f), 65504.0f);
    return __builtin_bit_cast(uint16_t, (_Float16)c);
}

// Two fp32 values -> two fp16 in one register (first value in the low half), round to nearest even, saturating
// like float_to_f16_bits: the packed conversion turns what lies beyond the largest finite fp16 into an infinity,
// which becomes the largest finite value again (0x7c00 -> 0x7bff, sign kept); NaN stays NaN.
__device__ __forceinline__ uint32_t pack_f16_saturating(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t p = {lo, hi};
    const uint32_t h = __builtin_bit_cast(uint32_t, __builtin_convertvector(p, f16x2_t));
    typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
    const u16x2_t hv = __builtin_bit_cast(u16x2_t, h);
    const u16x2_t m = __builtin_bit_cast(u16x2_t, (h & 0x7fff7fffu) ^ 0x7c007c00u);   // a half is 0 exactly where it holds an infinity
    const u16x2_t one = {1, 1}, fifteen = {15, 15};
    const u16x2_t is_inf = (u16x2_t)(m - one) >> fifteen;             // m <= 0x7fff: only m == 0 wraps to 0xffff (packed 16-bit ops)
    return __builtin_bit_cast(uint32_t, (u16x2_t)(hv - is_inf));
}

// Load the 32 consecutive activations a lane owns and widen them to fp32.
__device__ __forceinline__ void load_chunk(const void* base, int dtype, size_t elem_offset,
                                           float (&v)[kChunk]) {
    if (dtype == kF32) {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(base) + elem_offset);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float4 t = p[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + elem_offset);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 t = p[i];
            uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (dtype == kBF16) {
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

__device__ __forceinline__ void store_scalar(void* base, int dtype, size_t idx, float v) {
    if (dtype == kF32) static_cast<float*>(base)[idx] = v;
    else if (dtype == kBF16) static_cast<uint16_t*>(base)[idx] = float_to_bf16_bits(v);
    else static_cast<_Float16*>(base)[idx] = (_Float16)v;
}

}  // namespace tq
