// The 25 C entry points of include/turboquant_c/turboquant_c.h.
#include "turboquant_c/turboquant_c.h"

#include <cmath>
#include <filesystem>
#include <fstream>
#include <map>
#include <string>
#include <vector>

#include "turboquant/turboquant.h"
#include "turboquant_c/tq_linear.h"

namespace fs = std::filesystem;
using namespace turboquant;

struct tq_model_s {
    std::string model_path;
};

struct tq_kv_cache_s {
    int unused;
};

struct tq_coordinator_s {
    int rank = 0;
    int world_size = 1;
};

struct tq_cluster_s {
    int num_layers = 0, num_heads = 0, head_dim = 0;
    std::vector<double> memory_gb;          // one entry per registered node, rank = position
    std::vector<std::pair<int, int>> plan;  // [layer_start, layer_end) per rank
    bool planned = false;
};

namespace {

// Remove the "quantization_config": {...} member (and the comma before it) from a JSON text,
// the edit src/turboquant_c_dequant.cpp:36-65 makes to the copied config.json.
std::string strip_quantization_config(std::string text) {
    const size_t key = text.find("\"quantization_config\"");
    if (key == std::string::npos) return text;
    const size_t open = text.find('{', key);
    if (open == std::string::npos) return text;
    size_t pos = open + 1;
    for (int depth = 1; pos < text.size() && depth > 0; ++pos) {
        if (text[pos] == '{') ++depth;
        else if (text[pos] == '}') --depth;
    }
    const size_t comma = text.rfind(',', key);
    if (comma != std::string::npos && comma < key) text.erase(comma, pos - comma);
    return text;
}

int c_dtype_of(Dtype d) {
    return d == Dtype::F32 ? TQ_DTYPE_F32 : (d == Dtype::F16 ? TQ_DTYPE_F16 : TQ_DTYPE_BF16);
}

// One TQ8 shard -> one standard shard (src/turboquant_c_dequant.cpp:69-185).
void dequant_shard(const fs::path& shard, const fs::path& model_dir, const fs::path& out_dir) {
    const std::string fname = shard.filename().string();
    auto loaded = load_safetensors(shard.string());
    TensorMap& tensors = loaded.first;
    MetadataMap& metadata = loaded.second;
    auto qm = metadata.find("quantization_method");
    if (qm == metadata.end() || qm->second != "turboquant") {
        fs::copy_file(shard, out_dir / fname, fs::copy_options::overwrite_existing);
        return;
    }

    // Source element type: that of the passthrough tensors when the shard has a companion file.
    TensorMap passthrough;
    const fs::path pt_path = model_dir / (shard.stem().string() + "_passthrough.safetensors");
    Dtype target = Dtype::BF16;
    if (fs::exists(pt_path)) {
        passthrough = load_safetensors(pt_path.string()).first;
        const std::map<std::string, const Array*> by_name = [&] {
            std::map<std::string, const Array*> m;
            for (const auto& kv : passthrough) m[kv.first] = &kv.second;
            return m;
        }();
        if (!by_name.empty()) {
            const Dtype d = by_name.begin()->second->dtype();
            if (d == Dtype::F32 || d == Dtype::F16 || d == Dtype::BF16) target = d;
        }
    }

    TensorMap output;
    for (auto& kv : read_tq_layers(tensors, metadata)) {
        const TQLayer& L = kv.second;
        const int out = L.weights.packed_primary.shape(0);
        const int in = L.weights.packed_residual.shape(1) * 2;
        TurboQuantLinear layer(in, out, L.weights, L.primary_codebook, L.residual_codebook, L.block_size);
        Array w({out, in}, target);
        if (tq_linear_dequantize_as_host(layer.handle(), w.data<void>(), c_dtype_of(target)) != 0)
            throw std::runtime_error(tq_last_error());
        output.emplace(kv.first + ".weight", std::move(w));
    }
    for (auto& kv : passthrough) output.emplace(kv.first, kv.second);
    save_safetensors((out_dir / fname).string(), output);
}

}  // namespace

extern "C" {

// ---- model ------------------------------------------------------------------
tq_model_t tq_model_load(const char* model_path) {
    try {
        if (!model_path || !fs::is_directory(model_path)) return nullptr;
        auto* m = new tq_model_s();
        m->model_path = model_path;
        return m;
    } catch (...) { return nullptr; }
}

void* tq_model_forward(tq_model_t, const void*) { return nullptr; }

void tq_model_free(tq_model_t model) { delete model; }

// ---- KV cache: not built -----------------------------------------------------
tq_kv_cache_t tq_kv_cache_create(int, int, int, int, int, int) { return nullptr; }
void tq_kv_cache_append(tq_kv_cache_t, int, const void*, const void*) {}
void* tq_kv_cache_get_keys_fp16(tq_kv_cache_t, int, int, int) { return nullptr; }
void* tq_kv_cache_get_values_fp16(tq_kv_cache_t, int, int, int) { return nullptr; }
void* tq_kv_cache_attention(tq_kv_cache_t, int, const void*, int, int) { return nullptr; }
int tq_kv_cache_seq_length(tq_kv_cache_t) { return 0; }
void tq_kv_cache_free(tq_kv_cache_t cache) { delete cache; }

// ---- distributed --------------------------------------------------------------
tq_coordinator_t tq_distributed_init(const char*, const char*) { return nullptr; }

tq_coordinator_t tq_distributed_init_local(void) {
    try { return new tq_coordinator_s(); } catch (...) { return nullptr; }
}

int tq_distributed_rank(tq_coordinator_t coord) { return coord ? coord->rank : 0; }
int tq_distributed_world_size(tq_coordinator_t coord) { return coord ? coord->world_size : 1; }
void tq_distributed_free(tq_coordinator_t coord) { delete coord; }

// ---- cluster planning ----------------------------------------------------------
tq_cluster_t tq_cluster_create(int num_layers, int num_heads, int head_dim) {
    try {
        if (num_layers <= 0 || num_heads <= 0 || head_dim <= 0) return nullptr;
        auto* c = new tq_cluster_s();
        c->num_layers = num_layers; c->num_heads = num_heads; c->head_dim = head_dim;
        return c;
    } catch (...) { return nullptr; }
}

int tq_cluster_add_node(tq_cluster_t cluster, const char* hostname, double memory_gb) {
    if (!cluster || !hostname || !(memory_gb > 0.0) || cluster->planned) return -1;
    try { cluster->memory_gb.push_back(memory_gb); return 0; } catch (...) { return -1; }
}

// Layers proportional to usable memory, at least one per node while layers remain, the last
// node takes the remainder (reference src/distributed.cpp:213-252).
int tq_cluster_plan(tq_cluster_t cluster) {
    if (!cluster || cluster->planned || cluster->memory_gb.empty()) return -1;
    try {
        const size_t n = cluster->memory_gb.size();
        double total = 0.0;
        for (double m : cluster->memory_gb) total += m;
        if (total <= 0.0) total = 1.0;
        int next = 0;
        for (size_t i = 0; i < n; ++i) {
            int take = cluster->num_layers - next;
            if (i + 1 < n) {
                int share = (int)std::round((double)cluster->num_layers * cluster->memory_gb[i] / total);
                if (share < 1) share = 1;
                if (share < take) take = share;
            }
            cluster->plan.emplace_back(next, next + take);
            next += take;
        }
        cluster->planned = true;
        return 0;
    } catch (...) { return -1; }
}

int tq_cluster_node_count(tq_cluster_t cluster) { return cluster ? (int)cluster->memory_gb.size() : 0; }

int tq_cluster_get_layer_start(tq_cluster_t cluster, int rank) {
    if (!cluster || !cluster->planned || rank < 0 || rank >= (int)cluster->plan.size()) return -1;
    return cluster->plan[(size_t)rank].first;
}

int tq_cluster_get_layer_end(tq_cluster_t cluster, int rank) {
    if (!cluster || !cluster->planned || rank < 0 || rank >= (int)cluster->plan.size()) return -1;
    return cluster->plan[(size_t)rank].second;
}

void tq_cluster_free(tq_cluster_t cluster) { delete cluster; }

// ---- model dequantisation --------------------------------------------------------
int tq_model_dequant(const char* tq_model_path, const char* output_path) {
    try {
        if (!tq_model_path || !output_path) return 1;
        const fs::path src(tq_model_path), dst(output_path);
        if (!fs::is_directory(src)) return 1;
        fs::create_directories(dst);

        for (const auto& entry : fs::directory_iterator(src))
            if (entry.is_regular_file() && entry.path().extension() != ".safetensors")
                fs::copy_file(entry.path(), dst / entry.path().filename(), fs::copy_options::overwrite_existing);

        const fs::path config = dst / "config.json";
        if (fs::exists(config)) {
            std::ifstream in(config);
            const std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
            in.close();
            const std::string stripped = strip_quantization_config(text);
            if (stripped != text) std::ofstream(config, std::ios::trunc) << stripped;
        }

        for (const auto& entry : fs::directory_iterator(src)) {
            if (entry.path().extension() != ".safetensors") continue;
            if (entry.path().filename().string().find("_passthrough") != std::string::npos) continue;
            dequant_shard(entry.path(), src, dst);
        }
        return 0;
    } catch (...) { return 1; }
}

// ---- utility ----------------------------------------------------------------------
void tq_array_free(void* array) { delete static_cast<Array*>(array); }

const char* tq_version(void) { return turboquant::version(); }

}  // extern "C"
