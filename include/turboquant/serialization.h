#pragma once
// TQ8 safetensors files.  read_tq_metadata / write_tq_safetensors are the functions of the
// reference's src/serialization.cpp:13-91 (declared there without a header); load_safetensors /
// save_safetensors stand in for the mlx::core functions of the same names that the reference
// calls (src/serialization.cpp:14,89, src/turboquant_c_dequant.cpp:75,184).

#include "array.h"
#include "codebook.h"
#include "quantizer.h"
#include <string>
#include <unordered_map>
#include <utility>

namespace turboquant {

using TensorMap = std::unordered_map<std::string, Array>;
using MetadataMap = std::unordered_map<std::string, std::string>;

/// Parse a safetensors file: 8-byte little-endian header length, JSON header
/// ({name: {dtype, shape, data_offsets}, "__metadata__": {...}}), raw little-endian data.
/// Throws std::runtime_error on a malformed file.
std::pair<TensorMap, MetadataMap> load_safetensors(const std::string& path);

/// Write a safetensors file (tensors in name order, header padded to 8 bytes).
void save_safetensors(const std::string& path, const TensorMap& tensors, const MetadataMap& metadata = {});

/// The "__metadata__" map of a file; empty if it has none.
MetadataMap read_tq_metadata(const std::string& path);

/// Per weight: {name}.packed_primary / .packed_residual / .norms / .seeds; model-level
/// tq_codebook_primary / tq_codebook_residual; optional {name}.codebook_primary / _residual;
/// metadata quantization_method=turboquant, tq_version=1, tq_primary_bits, tq_residual_bits,
/// tq_total_bits, tq_per_layer_codebooks=true when per-layer codebooks are present.
bool write_tq_safetensors(
    const std::string& path,
    const std::unordered_map<std::string, QuantizedWeight>& weights,
    const Codebook& primary_codebook,
    const Codebook& residual_codebook,
    const std::unordered_map<std::string, std::pair<Codebook, Codebook>>& per_layer_codebooks);

/// One quantized layer of a TQ8 file with the codebooks that decode it (per-layer ones when the
/// file carries them, the model-level ones otherwise), as src/turboquant_c_dequant.cpp:107-149
/// assembles them.
struct TQLayer {
    QuantizedWeight weights;
    Codebook primary_codebook;
    Codebook residual_codebook;
    uint32_t block_size = 512;
};

/// All layers of an already-loaded TQ8 file, keyed by layer name (the tensor name without
/// ".packed_primary").  Throws std::runtime_error if a required tensor is missing.
std::unordered_map<std::string, TQLayer> read_tq_layers(const TensorMap& tensors, const MetadataMap& metadata);

}  // namespace turboquant
