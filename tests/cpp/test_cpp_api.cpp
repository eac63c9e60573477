// Drives the C++ API (include/turboquant/*.h) on the GPU the way the reference's
// tests/integration/test_linear.cpp, tests/unit/test_serialization.cpp and
// tests/unit/test_quantizer.cpp drive theirs, and writes every result to a safetensors file
// so the Python side can compare them with the CPU oracle.
//   test_cpp_api <inputs.safetensors> <output_dir>
// inputs: "w" f32 [out,in], "x" f32 [batch,in]; metadata "block_size".
#include "turboquant/turboquant.h"

#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

using namespace turboquant;

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { std::printf("  FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } } while (0)

template <typename E, typename F>
static bool throws(F&& f) {
    try { f(); } catch (const E&) { return true; } catch (...) { return false; }
    return false;
}

static bool same_bytes(const Array& a, const Array& b) {
    return a.dtype() == b.dtype() && a.shape() == b.shape() && std::memcmp(a.data<char>(), b.data<char>(), a.nbytes()) == 0;
}

int main(int argc, char** argv) {
    if (argc != 3) { std::fprintf(stderr, "usage: test_cpp_api <inputs.safetensors> <output_dir>\n"); return 2; }
    try {
        auto inputs = load_safetensors(argv[1]);
        const Array& w = inputs.first.at("w");
        const Array& x = inputs.first.at("x");
        const uint32_t bs = (uint32_t)std::atoi(inputs.second.at("block_size").c_str());
        const int out = w.shape(0), in = w.shape(1);
        const std::string out_dir = argv[2];

        CHECK(std::string(version()) == "0.1.0");
        const Codebook cb = generate_codebook(4);
        CHECK(validate_codebook(cb));
        CHECK(cb.centroids.size() == 16 && cb.boundaries.size() == 15 && cb.bits == 4);
        for (int bits = 1; bits <= 5; ++bits) CHECK(validate_codebook(generate_codebook((uint8_t)bits)));
        CHECK(throws<std::invalid_argument>([] { generate_codebook(0); }));
        CHECK(throws<std::invalid_argument>([] { generate_codebook(6); }));
        {
            Codebook broken = cb;
            broken.centroids[3] = broken.centroids[2];
            CHECK(!validate_codebook(broken));
            Codebook skew = cb;
            skew.centroids[15] += 0.25f;
            skew.boundaries[14] = (skew.centroids[14] + skew.centroids[15]) * 0.5f;
            CHECK(!validate_codebook(skew));                   // analytical codebooks must be symmetric
            skew.origin = CodebookOrigin::Empirical;
            CHECK(validate_codebook(skew));
        }

        TensorMap results;
        std::unordered_map<std::string, QuantizedWeight> file_weights;
        for (int shared = 0; shared < 2; ++shared) {
            const std::string tag = shared ? "shared." : "dual.";
            QuantizerConfig cfg;
            cfg.block_size = bs;
            cfg.shared_rotation = shared != 0;
            const QuantizedWeight qw = quantize_weight(w, cb, cb, cfg);
            CHECK(qw.packed_primary.shape(0) == out && qw.packed_primary.shape(1) == in / 2);
            CHECK(qw.seeds.data<uint32_t>()[2] == bs);
            CHECK((qw.seeds.data<uint32_t>()[1] == 0) == (shared != 0));

            TurboQuantLinear layer(in, out, qw, cb, cb, bs);
            CHECK(layer.in_features() == in && layer.out_features() == out);
            const Array y = layer.forward(x);
            CHECK(y.dtype() == Dtype::F32 && y.shape(0) == x.shape(0) && y.shape(1) == out);
            const Array y_bf16_in = layer.forward(astype(x, bfloat16), float32);
            const Array y_f16 = layer.forward(astype(x, float16));
            CHECK(y_f16.dtype() == Dtype::F16);
            const Array wd = dequantize_weight_gpu(qw, cb, cb, bs);
            CHECK(same_bytes(wd, dequantize_weight_cpu(qw, cb, cb, bs)));
            CHECK(same_bytes(wd, layer.dequantize()));
            CHECK(same_bytes(y, fused_dequant_matmul(qw, cb, cb, bs, x)));

            TurboQuantLinear copy = layer;                       // value semantics: shares the handle
            CHECK(same_bytes(y, copy.forward(x)));

            results.emplace(tag + "packed_primary", qw.packed_primary);
            results.emplace(tag + "packed_residual", qw.packed_residual);
            results.emplace(tag + "norms", qw.norms);
            results.emplace(tag + "seeds", qw.seeds);
            results.emplace(tag + "y", y);
            results.emplace(tag + "y_bf16_in", y_bf16_in);
            results.emplace(tag + "y_f16", y_f16);
            results.emplace(tag + "w", wd);
            file_weights.emplace(std::string(shared ? "model.shared_proj" : "model.dual_proj"), qw);
        }

        // Error behaviour (reference src/dequantizer.cpp:494, rotation.cpp:374).
        {
            const QuantizedWeight& qw = file_weights.at("model.dual_proj");
            CHECK(throws<std::runtime_error>([&] { TurboQuantLinear bad(in, out, qw, cb, cb, 3 * bs + 1); }));
            TurboQuantLinear layer(in, out, qw, cb, cb, bs);
            std::vector<float> wrong((size_t)in + 1, 0.0f);
            CHECK(throws<std::runtime_error>([&] { layer.forward(Array(wrong.data(), {1, in + 1})); }));
            CHECK(throws<std::invalid_argument>([&] { apply_wht_rotation(w, 7u, 3 * bs + 1); }));
        }

        // Rotation: forward then inverse (reference tests/unit/test_rotation.cpp).
        const Array rot = apply_wht_rotation(w, 0x1234u, bs);
        results.emplace("rotated", rot);
        results.emplace("unrotated", apply_inverse_wht_rotation(rot, 0x1234u, bs));

        // Scalar codebook maps and the data-adaptive fit.
        const Array flat = x.reshape({(int)x.size()});
        const Array idx = quantize(flat, cb);
        results.emplace("x_indices", idx);
        results.emplace("x_centroids", dequantize(idx, cb));
        {
            std::vector<float> samples(rot.data<float>(), rot.data<float>() + rot.size());
            const float scale = 1.0f / w.data<float>()[0];      // any fixed rescale; the Python side repeats it
            for (float& v : samples) v *= scale;
            const Codebook fit = generate_codebook_from_data(samples, 4);
            CHECK(fit.origin == CodebookOrigin::Empirical && validate_codebook(fit));
            results.emplace("fit_centroids", Array(fit.centroids.data(), {16}));
            CHECK(same_bytes(Array(generate_codebook_from_data({}, 3).centroids.data(), {8}),
                             Array(generate_codebook(3).centroids.data(), {8})));
        }

        // TQ8 file: write, read the metadata back, reload the layers and run them again.
        const std::string tq_path = out_dir + "/model.safetensors";
        std::unordered_map<std::string, std::pair<Codebook, Codebook>> per_layer;
        per_layer.emplace("model.dual_proj", std::make_pair(cb, cb));
        CHECK(write_tq_safetensors(tq_path, file_weights, cb, cb, per_layer));
        const MetadataMap md = read_tq_metadata(tq_path);
        CHECK(md.at("quantization_method") == "turboquant" && md.at("tq_version") == "1");
        CHECK(md.at("tq_primary_bits") == "4" && md.at("tq_residual_bits") == "4" && md.at("tq_total_bits") == "8");
        CHECK(md.at("tq_per_layer_codebooks") == "true");
        CHECK(read_tq_metadata(out_dir + "/does_not_exist.safetensors").empty());
        {
            auto reloaded = load_safetensors(tq_path);
            auto layers = read_tq_layers(reloaded.first, reloaded.second);
            CHECK(layers.size() == 2);
            for (auto& kv : layers) {
                const TQLayer& L = kv.second;
                CHECK(L.block_size == bs);
                TurboQuantLinear layer(in, out, L.weights, L.primary_codebook, L.residual_codebook, L.block_size);
                const char* tag = kv.first == "model.shared_proj" ? "shared.y" : "dual.y";
                CHECK(same_bytes(layer.forward(x), results.at(tag)));
            }
        }

        save_safetensors(out_dir + "/results.safetensors", results);
    } catch (const std::exception& e) {
        std::printf("  FAIL: unexpected exception: %s\n", e.what());
        return 1;
    }
    if (failures) { std::printf("%d check(s) failed\n", failures); return 1; }
    std::printf("cpp api ok\n");
    return 0;
}
