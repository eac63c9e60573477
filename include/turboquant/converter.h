#pragma once
// Model conversion: HuggingFace safetensors directory -> TQ8 directory
// (reference include/turboquant/converter.h:1-31, src/converter.cpp:28-456).

#include "quantizer.h"
#include <functional>
#include <string>

namespace turboquant {

/// Progress callback: (current_weight, total_weights, tensor_name).
using ConversionProgressFn = std::function<void(int, int, const std::string&)>;

struct ConversionConfig {
    QuantizerConfig quantizer;               ///< per-weight settings; block_size is the upper bound per layer
    std::string input_path;                  ///< source model directory
    std::string output_path;                 ///< directory to write
    ConversionProgressFn progress_callback;  ///< optional
    bool per_layer_codebooks = false;        ///< fit Lloyd-Max codebooks to every layer
};

/// Every 2-D tensor whose name ends in ".weight" is quantized (block size: the largest power of
/// two <= quantizer.block_size that divides its width), except in the first
/// sensitive_layers_start and last sensitive_layers_end numbered layers; everything else is
/// copied to "<shard>_passthrough.safetensors".  Other files of the directory are copied and
/// config.json gains a "quantization_config" block.  Returns false if the input directory does
/// not exist.  A weight with an odd number of columns (two columns share a byte of the 4-bit planes) is
/// passed through unchanged, with a line on stderr.
bool convert_model(const ConversionConfig& config);

/// True if some safetensors file in the directory carries quantization_method=turboquant.
bool validate_converted_model(const std::string& model_path);

}  // namespace turboquant
