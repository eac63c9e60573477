#pragma once
// Dequantisation and the fused dequant-matmul.  Same functions as the reference's
// include/turboquant/dequantizer.h:1-41, with turboquant::Array in place of mlx::core::array.

#include "array.h"
#include "codebook.h"
#include "quantizer.h"

namespace turboquant {

/// Full-precision fp32 [out, in] weight from the packed representation
/// (reference src/dequantizer.cpp:347-451).  One HIP kernel; the result is bit-identical to the
/// reference's CPU arithmetic (src/dequantizer.cpp:52-256).
Array dequantize_weight_gpu(const QuantizedWeight& qw, const Codebook& primary_codebook,
                            const Codebook& residual_codebook, uint32_t block_size);

/// Source-compatibility name (reference dequantizer.h:11-15).  This library has no CPU
/// dequantizer: the call runs the same kernel as dequantize_weight_gpu and needs a GPU.
Array dequantize_weight_cpu(const QuantizedWeight& qw, const Codebook& primary_codebook,
                            const Codebook& residual_codebook, uint32_t block_size);

/// y = x * W^T without materialising W (reference src/dequantizer.cpp:475-721).
/// input [batch, in] fp32 / fp16 / bf16; output [batch, out] in the input's element type
/// (the reference casts everything to fp16; fp16 in gives fp16 out here as well).
Array fused_dequant_matmul(const QuantizedWeight& qw, const Codebook& primary_codebook,
                           const Codebook& residual_codebook, uint32_t block_size, const Array& input);

}  // namespace turboquant
