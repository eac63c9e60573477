// convert_model / validate_converted_model on top of this library's safetensors reader/writer,
// GPU quantizer and per-layer codebook fit (reference src/converter.cpp:28-456).  The reference
// quantizes with worker threads that force its CPU path; here every weight goes through the GPU
// quantizer, one after the other.
#include "turboquant/converter.h"
#include "turboquant/codebook.h"
#include "turboquant/serialization.h"
#include "turboquant_c/tq_quantizer.h"

#include <cstdio>
#include <filesystem>
#include <fstream>
#include <regex>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace fs = std::filesystem;

namespace turboquant {

namespace {

// 2-D tensors named "*.weight" (reference src/converter.cpp:36-46).
bool is_quantizable_weight(const std::string& name, const Array& tensor) {
    static const std::string suffix = ".weight";
    if (tensor.ndim() != 2 || name.size() < suffix.size()) return false;
    return name.compare(name.size() - suffix.size(), suffix.size(), suffix) == 0;
}

// "….layers.N.…" -> N, otherwise -1 (reference src/converter.cpp:52-59).
int extract_layer_index(const std::string& name) {
    static const std::regex layer_pattern(R"(\.layers\.(\d+)\.)");
    std::smatch match;
    if (std::regex_search(name, match, layer_pattern)) return std::stoi(match[1].str());
    return -1;
}

// reference src/converter.cpp:81-94
bool is_sensitive_layer(int layer_index, int max_layer_index, int sensitive_start, int sensitive_end) {
    if (layer_index < 0) return false;
    return layer_index < sensitive_start || layer_index > max_layer_index - sensitive_end;
}

Codebook codebook_of(const float* centroids, int n, uint8_t bits) {
    Codebook cb;
    cb.centroids.assign(centroids, centroids + n);
    cb.boundaries.resize(n > 0 ? n - 1 : 0);
    for (int i = 0; i + 1 < n; ++i) cb.boundaries[i] = 0.5f * (centroids[i] + centroids[i + 1]);
    cb.bits = bits;
    cb.origin = CodebookOrigin::Empirical;
    return cb;
}

// What the layout can hold: an even width (two columns share a byte of the nibble planes) and a power-of-two
// block of at most 2048 columns (the block rule of src/converter.cpp:228-240 never picks more than 512).  An
// odd width is left unquantized and reported.
bool quantizer_takes(int in_features, uint32_t block_size) {
    return in_features % 2 == 0 && block_size >= 1 && block_size <= 2048 && in_features % (int)block_size == 0;
}

}  // namespace

bool convert_model(const ConversionConfig& config) {
    if (!fs::exists(config.input_path) || !fs::is_directory(config.input_path)) return false;

    // Model-level codebooks, shared by every weight that has no per-layer ones.
    const QuantizerConfig& qc = config.quantizer;
    const Codebook primary_codebook = generate_codebook(qc.primary_bits);
    const Codebook residual_codebook = generate_codebook(qc.residual_bits > 0 ? qc.residual_bits : 1);

    std::vector<fs::path> shards;
    for (const auto& entry : fs::directory_iterator(config.input_path))
        if (entry.is_regular_file() && entry.path().extension() == ".safetensors") shards.push_back(entry.path());

    const bool has_sensitive = qc.sensitive_layers_start > 0 || qc.sensitive_layers_end > 0;
    int max_layer_index = -1, total_weights = 0;
    for (const auto& shard : shards) {
        const auto loaded = load_safetensors(shard.string());
        for (const auto& [name, tensor] : loaded.first) {
            if (has_sensitive) max_layer_index = std::max(max_layer_index, extract_layer_index(name));
            if (is_quantizable_weight(name, tensor)) ++total_weights;
        }
    }

    fs::create_directories(config.output_path);
    for (const auto& entry : fs::directory_iterator(config.input_path))
        if (entry.is_regular_file() && entry.path().extension() != ".safetensors")
            fs::copy_file(entry.path(), fs::path(config.output_path) / entry.path().filename(),
                          fs::copy_options::overwrite_existing);

    // config.json: "quantization_config" appended before the last brace, the keys of the
    // reference (src/converter.cpp:141-166).
    {
        const fs::path config_path = fs::path(config.output_path) / "config.json";
        if (fs::exists(config_path)) {
            std::ifstream in(config_path);
            std::string json((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
            in.close();
            const auto last_brace = json.rfind('}');
            if (last_brace != std::string::npos) {
                const std::string block =
                    ",\n  \"quantization_config\": {\n"
                    "    \"quantization_method\": \"turboquant\",\n"
                    "    \"tq_version\": \"1\",\n"
                    "    \"bits\": " + std::to_string(qc.primary_bits) + ",\n"
                    "    \"residual_bits\": " + std::to_string(qc.residual_bits) + ",\n"
                    "    \"block_size\": " + std::to_string(qc.block_size) + ",\n"
                    "    \"shared_rotation\": " + (qc.shared_rotation ? "true" : "false") + ",\n"
                    "    \"sensitive_layers_start\": " + std::to_string(qc.sensitive_layers_start) + ",\n"
                    "    \"sensitive_layers_end\": " + std::to_string(qc.sensitive_layers_end) + "\n"
                    "  }\n";
                json.replace(last_brace, 1, block + "}");
                std::ofstream(config_path, std::ios::trunc) << json;
            }
        }
    }

    int processed = 0, kept = 0, quantized = 0;
    for (const auto& shard : shards) {
        auto loaded = load_safetensors(shard.string());
        std::unordered_map<std::string, QuantizedWeight> weights;
        std::unordered_map<std::string, std::pair<Codebook, Codebook>> layer_codebooks;
        TensorMap passthrough;

        for (auto& [name, tensor] : loaded.first) {
            if (!is_quantizable_weight(name, tensor)) { passthrough.emplace(name, tensor); continue; }
            if (has_sensitive && is_sensitive_layer(extract_layer_index(name), max_layer_index,
                                                    qc.sensitive_layers_start, qc.sensitive_layers_end)) {
                passthrough.emplace(name, tensor);
                ++kept;
                continue;
            }
            const int out_features = tensor.shape()[0], in_features = tensor.shape()[1];
            QuantizerConfig layer_config = qc;
            layer_config.block_size = tq_best_block_size(in_features, qc.block_size);
            if (!quantizer_takes(in_features, layer_config.block_size)) {
                std::fprintf(stderr, "convert_model: %s [%d, %d] left unquantized (width or block size not supported)\n",
                             name.c_str(), out_features, in_features);
                passthrough.emplace(name, tensor);
                continue;
            }
            const std::string layer_name = name.substr(0, name.size() - 7);      // without ".weight"
            const Array fp32 = astype(tensor, Dtype::F32);

            Codebook cb_p = primary_codebook, cb_r = residual_codebook;
            if (config.per_layer_codebooks) {
                // Lloyd-Max on the rotated, scaled layer (and on its primary residual), 100 rounds,
                // as the reference's workers do (src/converter.cpp:291-372).
                float cp[32], cr[32];
                if (tq_fit_layer_codebooks_host(fp32.data<float>(), out_features, in_features, layer_config.block_size,
                                                qc.primary_bits, qc.residual_bits, primary_codebook.centroids.data(),
                                                (int)primary_codebook.centroids.size(), 100, cp, cr) != 0)
                    throw std::runtime_error("convert_model: codebook fit failed for " + name);
                cb_p = codebook_of(cp, 1 << qc.primary_bits, qc.primary_bits);
                if (qc.residual_bits > 0) cb_r = codebook_of(cr, 1 << qc.residual_bits, qc.residual_bits);
                layer_codebooks.emplace(layer_name, std::make_pair(cb_p, cb_r));
            }
            weights.emplace(layer_name, quantize_weight(fp32, cb_p, cb_r, layer_config));
            ++quantized;
            ++processed;
            if (config.progress_callback) config.progress_callback(processed, total_weights, name);
        }

        write_tq_safetensors((fs::path(config.output_path) / shard.filename()).string(), weights, primary_codebook,
                             residual_codebook, layer_codebooks);
        if (!passthrough.empty())
            save_safetensors((fs::path(config.output_path) / (shard.stem().string() + "_passthrough.safetensors")).string(),
                             passthrough);
    }
    if (has_sensitive) std::printf("Sensitive layers: %d weights kept at fp16, %d weights quantized\n", kept, quantized);
    return true;
}

bool validate_converted_model(const std::string& model_path) {
    if (!fs::exists(model_path) || !fs::is_directory(model_path)) return false;
    for (const auto& entry : fs::directory_iterator(model_path)) {
        if (!entry.is_regular_file() || entry.path().extension() != ".safetensors") continue;
        const auto metadata = read_tq_metadata(entry.path().string());
        const auto it = metadata.find("quantization_method");
        if (it != metadata.end() && it->second == "turboquant") return true;
    }
    return false;
}

}  // namespace turboquant
