#pragma once
// Offline weight quantizer.  Same types and functions as the reference's
// include/turboquant/quantizer.h:1-62, with turboquant::Array in place of mlx::core::array.

#include "array.h"
#include "codebook.h"
#include <cstdint>
#include <string>

namespace turboquant {

struct QuantizerConfig {
    uint8_t primary_bits = 4;       ///< primary pass bit width
    uint8_t residual_bits = 4;      ///< residual pass bit width (0 = no residual)
    uint32_t block_size = 512;      ///< WHT block size
    bool shared_rotation = false;   ///< one rotation for both passes (seeds[1] stored as 0)
    bool norm_correction = true;    ///< corrected row norms (always applied, as in the reference)
    int sensitive_layers_start = 0; ///< converter setting, unused by quantize_weight
    int sensitive_layers_end = 0;   ///< converter setting, unused by quantize_weight
};

struct QuantizedWeight {
    Array packed_primary;    ///< uint8 [out, in/2] (4-bit) or [out, in] (5-bit primary)
    Array packed_residual;   ///< uint8 [out, in/2]
    Array norms;             ///< float32 [out], corrected row norms
    Array seeds;             ///< uint32 [3] = {seed_primary, seed_residual or 0, block_size}
};

/// Block randomised Walsh-Hadamard rotation of the rows of an fp32 [rows, cols] matrix
/// (reference src/rotation.cpp:291-319).  Throws if cols is not a multiple of block_size.
Array apply_wht_rotation(const Array& matrix, uint32_t seed, uint32_t block_size);

/// Its inverse (reference src/rotation.cpp:323-350).
Array apply_inverse_wht_rotation(const Array& matrix, uint32_t seed, uint32_t block_size);

/// Kept for source compatibility with reference quantizer.h:44-53: the flag is stored per
/// thread and reported back, but every element-level operation of this library runs on the
/// GPU regardless (there is no CPU path to force).
void set_force_cpu(bool force_cpu);
bool get_force_cpu();

/// normalise -> rotate -> quantise -> residual pass -> norm correction
/// (reference src/quantizer.cpp:41-261), on the GPU.
QuantizedWeight quantize_weight(const Array& weight, const Codebook& primary_codebook,
                                const Codebook& residual_codebook, const QuantizerConfig& config);

}  // namespace turboquant
