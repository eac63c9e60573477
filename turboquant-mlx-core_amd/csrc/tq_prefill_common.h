// Pieces shared by the two prefill GEMM kernels (tq_prefill.hip, tq_prefill_panel.hip).
#pragma once

#include "tq_device.h"

namespace tq {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));

// LDS byte address of table entry `byte j of idx_bytes` in the lane-private table: entry pitch 256 bytes,
// the lane's own 4-byte column inside it (laneoff = lane * 4).
__device__ __forceinline__ uint32_t gemm_entry_addr(uint32_t idx_bytes, uint32_t laneoff, int j) {
    switch (j) {
        case 0: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0400u);
        case 1: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0500u);
        case 2: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0600u);
        default: return __builtin_amdgcn_perm(idx_bytes, laneoff, 0x0c0c0700u);
    }
}

// Table entries hold the fp16 value in the upper half of the dword (low 16 bits zero): two of them
// pack into one register of two halves with a single byte permute.
__device__ __forceinline__ uint32_t pack_half2(uint32_t lo_val, uint32_t hi_val) {
    return __builtin_amdgcn_perm(hi_val, lo_val, 0x07060302u);   // {lo.b2, lo.b3, hi.b2, hi.b3}
}

// The panel kernel (tq_prefill_panel.hip): 512-row activation panels, activations read from global memory in
// MFMA operand order.  Its rotated activations are "fragment images" (rotate_panel_kernel writes them).
constexpr int kPanelM = 512;
bool prefill_panel_supported(const LayerView& L, int batch, int num_cus, size_t capacity);
// Workspace of a call: fragment images, then the fp32 parts of the tiles that are cut along K (none if that would
// exceed `capacity`).  launch_prefill_panel derives the same cut from the bytes it is given.
size_t prefill_panel_workspace_bytes(const LayerView& L, int batch, int num_cus, size_t capacity);
hipError_t launch_prefill_panel(const LayerView& L, const void* x, int x_dtype, int batch, void* y, int y_dtype,
                                void* workspace, size_t workspace_bytes, int num_cus, hipStream_t stream);

}  // namespace tq
