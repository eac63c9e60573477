// C-ABI of the offline TQ8 quantizer (declared in include/turboquant_c/tq_quantizer.h).
// Host-side driver only: argument checks, the Lloyd-Max update step between GPU assignment
// passes (src/codebook.cpp:122-132), buffer ownership.  All per-element work runs on the GPU.
#include "turboquant_c/tq_quantizer.h"

#include <cmath>
#include <cstring>
#include <vector>

#include "tq_device.h"

namespace {

using tq::hip_ok;
using tq::set_error;

// Lloyd-Max optimal centroids for N(0,1) (Zandieh et al.), the values of the reference's tables
// (src/codebook.cpp:16-45).
const float kC1[] = {-0.7978845608f, 0.7978845608f};
const float kC2[] = {-1.510232f, -0.4527800f, 0.4527800f, 1.510232f};
const float kC3[] = {-2.152176f, -1.344318f, -0.756130f, -0.245379f, 0.245379f, 0.756130f, 1.344318f, 2.152176f};
const float kC4[] = {-2.732590f, -2.069017f, -1.618046f, -1.256231f, -0.942340f, -0.656759f, -0.388048f, -0.128395f,
                     0.128395f,  0.388048f,  0.656759f,  0.942340f,  1.256231f,  1.618046f,  2.069017f,  2.732590f};
const float kC5[] = {-3.255544f, -2.685239f, -2.311434f, -2.022174f, -1.780580f, -1.569614f, -1.379896f, -1.205655f,
                     -1.043046f, -0.889350f, -0.742542f, -0.601049f, -0.463598f, -0.329119f, -0.196679f, -0.065429f,
                     0.065429f,  0.196679f,  0.329119f,  0.463598f,  0.601049f,  0.742542f,  0.889350f,  1.043046f,
                     1.205655f,  1.379896f,  1.569614f,  1.780580f,  2.022174f,  2.311434f,  2.685239f,  3.255544f};

void midpoints(const float* c, int n, float* b) {
    for (int i = 0; i + 1 < n; ++i) b[i] = (c[i] + c[i + 1]) * 0.5f;      // src/codebook.cpp:54
}

struct DevBuf {
    void* p = nullptr;
    ~DevBuf() { if (p) (void)hipFree(p); }
    bool alloc(size_t bytes, const char* what) { return hip_ok(hipMalloc(&p, bytes ? bytes : 1), what); }
    template <typename T> T* as() { return static_cast<T*>(p); }
};

bool check_shape(int out, int in, uint32_t bs, const char* who) {
    if (out <= 0 || in <= 0) { set_error(std::string(who) + ": bad dimensions"); return false; }
    if (bs == 0 || in % (int)bs != 0) {
        set_error(std::string(who) + ": in_features must be divisible by block_size"); return false;
    }
    // (what the layout itself needs; widths that are not a multiple of 32 and blocks of one column run on the
    // small-block kernel)
    if (!tq::layout_valid(in, bs) || (!tq::lanes_supported(in, bs) && bs > 16)) {
        set_error(std::string(who) + ": unsupported shape (need an even in_features and a power-of-two block_size "
                  "in [1, 2048])");
        return false;
    }
    return true;
}

// tables: [0..31] cP, [32..62] bP, [64..79] cR, [80..94] bR
void fill_tables(const float* cbp, int np, const float* cbr, int nr, float* t) {
    std::memset(t, 0, 96 * sizeof(float));
    std::memcpy(t, cbp, np * sizeof(float));
    midpoints(cbp, np, t + 32);
    std::memcpy(t + 64, cbr, nr * sizeof(float));
    midpoints(cbr, nr, t + 80);
}

// generate_codebook_from_data_cpu (src/codebook.cpp:99-143) with the assignment pass on the GPU.
bool lloyd_max(const float* samples_dev, size_t n, int bits, int iterations, bool subtract,
               const float* gcent_dev, const float* gbounds_dev, int ngc, float* centroids_out) {
    float cent[32], bounds[32];
    const int nc = tq_generate_codebook(bits, cent, bounds);
    if (nc < 0) { set_error("tq_fit_layer_codebooks: unsupported bit width"); return false; }
    const int wgs = 1024;
    DevBuf d_bounds, d_sum, d_cnt;
    if (!d_bounds.alloc(32 * sizeof(float), "hipMalloc(bounds)") ||
        !d_sum.alloc((size_t)wgs * 32 * sizeof(double), "hipMalloc(bin sums)") ||
        !d_cnt.alloc((size_t)wgs * 32 * sizeof(unsigned long long), "hipMalloc(bin counts)")) return false;
    std::vector<double> h_sum((size_t)wgs * 32);
    std::vector<unsigned long long> h_cnt((size_t)wgs * 32);
    for (int iter = 0; iter < iterations; ++iter) {
        midpoints(cent, nc, bounds);
        if (!hip_ok(hipMemcpy(d_bounds.p, bounds, 32 * sizeof(float), hipMemcpyHostToDevice), "copy bounds") ||
            !hip_ok(tq::launch_lloyd_pass(samples_dev, n, d_bounds.as<float>(), nc, subtract ? 1 : 0, gcent_dev,
                                          gbounds_dev, ngc, d_sum.as<double>(), d_cnt.as<unsigned long long>(),
                                          wgs, nullptr), "lloyd pass") ||
            !hip_ok(hipMemcpy(h_sum.data(), d_sum.p, h_sum.size() * sizeof(double), hipMemcpyDeviceToHost), "copy sums") ||
            !hip_ok(hipMemcpy(h_cnt.data(), d_cnt.p, h_cnt.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost),
                    "copy counts"))
            return false;
        float max_shift = 0.0f;
        for (int k = 0; k < nc; ++k) {
            double s = 0.0; unsigned long long c = 0;
            for (int w = 0; w < wgs; ++w) { s += h_sum[(size_t)w * 32 + k]; c += h_cnt[(size_t)w * 32 + k]; }
            if (c > 0) {                                                         // src/codebook.cpp:124-129
                const float nv = static_cast<float>(s / static_cast<double>(c));
                const float shift = std::fabs(nv - cent[k]);
                if (shift > max_shift) max_shift = shift;
                cent[k] = nv;
            }
        }
        if (max_shift < 1e-6f) break;                                            // src/codebook.cpp:132
    }
    std::memcpy(centroids_out, cent, nc * sizeof(float));
    return true;
}

}  // namespace

extern "C" {

int tq_generate_codebook(int bits, float* centroids, float* boundaries) {
    const float* src;
    switch (bits) {
        case 1: src = kC1; break;
        case 2: src = kC2; break;
        case 3: src = kC3; break;
        case 4: src = kC4; break;
        case 5: src = kC5; break;
        default: set_error("Unsupported bit width; must be 1-5"); return -1;
    }
    if (!centroids) { set_error("tq_generate_codebook: NULL argument"); return -1; }
    const int n = 1 << bits;
    std::memcpy(centroids, src, n * sizeof(float));
    if (boundaries) midpoints(centroids, n, boundaries);
    return n;
}

uint32_t tq_best_block_size(int in_features, uint32_t max_block_size) {
    uint32_t best = 1;
    for (int p = 1; p < 20; ++p) {
        const uint32_t c = 1u << p;
        if (c > max_block_size) break;
        if (in_features % static_cast<int>(c) == 0) best = c;
    }
    return best;
}

int tq_quantize_weight(const float* weight_dev, int out, int in,
                       const float* cbp, int np, const float* cbr, int nr,
                       int primary_bits, int residual_bits, uint32_t block_size, int shared_rotation,
                       uint8_t* pp_dev, uint8_t* pr_dev, float* norms_dev, uint32_t* seeds_host) {
    try {
        if (!weight_dev || !cbp || !cbr || !pp_dev || !pr_dev || !norms_dev || !seeds_host) {
            set_error("tq_quantize_weight: NULL argument"); return 1;
        }
        if (!check_shape(out, in, block_size, "tq_quantize_weight")) return 1;
        if (np < 2 || np > 32 || nr < 2 || nr > 16 || primary_bits < 1 || primary_bits > 5 ||
            residual_bits < 0 || residual_bits > 4) {
            set_error("tq_quantize_weight: bad codebook sizes or bit widths"); return 1;
        }
        const int slabs = tq::quantize_partials_per_row(in, block_size);
        DevBuf d_orig, d_partial, d_tables, d_seeds;
        float tables[96];
        fill_tables(cbp, np, cbr, nr, tables);
        uint32_t seeds[2] = {0, 0};
        if (!d_orig.alloc((size_t)out * sizeof(float), "hipMalloc(norms)") ||
            !d_partial.alloc((size_t)out * slabs * sizeof(double), "hipMalloc(partials)") ||
            !d_tables.alloc(sizeof(tables), "hipMalloc(tables)") ||
            !d_seeds.alloc(2 * sizeof(uint32_t), "hipMalloc(seeds)") ||
            !hip_ok(hipMemcpy(d_tables.p, tables, sizeof(tables), hipMemcpyHostToDevice), "copy tables") ||
            !hip_ok(tq::launch_derive_seeds(weight_dev, (size_t)out * in, d_seeds.as<uint32_t>(), nullptr), "derive_seed") ||
            !hip_ok(hipMemcpy(seeds, d_seeds.p, sizeof(seeds), hipMemcpyDeviceToHost), "copy seeds") ||
            !hip_ok(tq::launch_row_norms(weight_dev, d_orig.as<float>(), out, in, nullptr), "row norms"))
            return 1;
        if (residual_bits == 0 &&
            !hip_ok(hipMemset(pr_dev, 0, (size_t)out * (in / 2)), "zero residual plane")) return 1;

        tq::QuantArgsHost a{};
        a.w = weight_dev; a.orig_norm = d_orig.as<float>(); a.recon_partial = d_partial.as<double>();
        a.scaled_out = nullptr; a.packed_primary = pp_dev; a.packed_residual = pr_dev;
        a.tables = d_tables.as<float>();
        a.out = out; a.in = in; a.n_primary = np; a.n_residual = nr;
        a.primary_bits = primary_bits; a.residual_bits = residual_bits; a.shared_rotation = shared_rotation ? 1 : 0;
        a.bs = block_size; a.seed_p = seeds[0]; a.seed_r = seeds[1];
        a.scale_factor = std::sqrt(static_cast<float>(in));                     // src/quantizer.cpp:51
        a.inv_scale = 1.0f / a.scale_factor;                                    // :52
        a.inv_sqrt_bs = 1.0f / std::sqrt(static_cast<float>(block_size));       // src/rotation.cpp:301
        a.quantize = 1;
        if (!hip_ok(tq::launch_quantize_rows(a, nullptr), "quantize rows") ||
            !hip_ok(tq::launch_finish_norms(d_orig.as<float>(), d_partial.as<double>(), norms_dev, out, slabs, nullptr),
                    "finish norms") ||
            !hip_ok(hipDeviceSynchronize(), "quantize sync"))
            return 1;
        seeds_host[0] = seeds[0];
        seeds_host[1] = (shared_rotation && residual_bits > 0) ? 0u : seeds[1];  // src/quantizer.cpp:255-256
        seeds_host[2] = block_size;
        return 0;
    } catch (...) { set_error("tq_quantize_weight: exception"); return 1; }
}

int tq_fit_layer_codebooks(const float* weight_dev, int out, int in, uint32_t block_size,
                           int primary_bits, int residual_bits,
                           const float* gcp, int ngc, int iterations,
                           float* cbp_out, float* cbr_out) {
    try {
        if (!weight_dev || !gcp || !cbp_out || (residual_bits > 0 && !cbr_out)) {
            set_error("tq_fit_layer_codebooks: NULL argument"); return 1;
        }
        if (!check_shape(out, in, block_size, "tq_fit_layer_codebooks")) return 1;
        if (ngc < 2 || ngc > 32) { set_error("tq_fit_layer_codebooks: bad global codebook"); return 1; }
        const size_t n = (size_t)out * in;
        DevBuf d_orig, d_scaled, d_tables, d_seeds, d_g;
        float tables[96];
        fill_tables(gcp, ngc, gcp, ngc > 16 ? 16 : ngc, tables);
        float gtab[64];
        std::memset(gtab, 0, sizeof(gtab));
        std::memcpy(gtab, gcp, ngc * sizeof(float));
        midpoints(gcp, ngc, gtab + 32);
        uint32_t seeds[2];
        if (!d_orig.alloc((size_t)out * sizeof(float), "hipMalloc(norms)") ||
            !d_scaled.alloc(n * sizeof(float), "hipMalloc(samples)") ||
            !d_tables.alloc(sizeof(tables), "hipMalloc(tables)") ||
            !d_g.alloc(sizeof(gtab), "hipMalloc(global codebook)") ||
            !d_seeds.alloc(2 * sizeof(uint32_t), "hipMalloc(seeds)") ||
            !hip_ok(hipMemcpy(d_tables.p, tables, sizeof(tables), hipMemcpyHostToDevice), "copy tables") ||
            !hip_ok(hipMemcpy(d_g.p, gtab, sizeof(gtab), hipMemcpyHostToDevice), "copy global codebook") ||
            !hip_ok(tq::launch_derive_seeds(weight_dev, n, d_seeds.as<uint32_t>(), nullptr), "derive_seed") ||
            !hip_ok(hipMemcpy(seeds, d_seeds.p, sizeof(seeds), hipMemcpyDeviceToHost), "copy seeds") ||
            !hip_ok(tq::launch_row_norms(weight_dev, d_orig.as<float>(), out, in, nullptr), "row norms"))
            return 1;
        tq::QuantArgsHost a{};
        a.w = weight_dev; a.orig_norm = d_orig.as<float>(); a.scaled_out = d_scaled.as<float>();
        a.tables = d_tables.as<float>();
        a.out = out; a.in = in; a.n_primary = ngc; a.n_residual = 2;
        a.primary_bits = primary_bits; a.bs = block_size; a.seed_p = seeds[0]; a.seed_r = seeds[1];
        a.scale_factor = std::sqrt(static_cast<float>(in));
        a.inv_scale = 1.0f / a.scale_factor;
        a.inv_sqrt_bs = 1.0f / std::sqrt(static_cast<float>(block_size));
        a.quantize = 0;
        if (!hip_ok(tq::launch_quantize_rows(a, nullptr), "rotate samples")) return 1;
        if (!lloyd_max(d_scaled.as<float>(), n, primary_bits, iterations, false, nullptr, nullptr, 0, cbp_out)) return 1;
        if (residual_bits > 0 &&
            !lloyd_max(d_scaled.as<float>(), n, residual_bits, iterations, true, d_g.as<float>(), d_g.as<float>() + 32,
                       ngc, cbr_out))
            return 1;
        return 0;
    } catch (...) { set_error("tq_fit_layer_codebooks: exception"); return 1; }
}

int tq_quantize_weight_host(const float* weight_host, int out, int in,
                            const float* cbp, int np, const float* cbr, int nr,
                            int primary_bits, int residual_bits, uint32_t block_size, int shared_rotation,
                            uint8_t* pp_host, uint8_t* pr_host, float* norms_host, uint32_t* seeds_host) {
    try {
        if (!weight_host || !pp_host || !pr_host || !norms_host) { set_error("tq_quantize_weight_host: NULL argument"); return 1; }
        if (out <= 0 || in <= 0) { set_error("tq_quantize_weight_host: bad dimensions"); return 1; }
        const size_t n = (size_t)out * in;
        const size_t pbytes = primary_bits <= 4 ? n / 2 : n;
        DevBuf w, pp, pr, norms;
        if (!w.alloc(n * sizeof(float), "hipMalloc(weight)") || !pp.alloc(pbytes, "hipMalloc(primary)") ||
            !pr.alloc(n / 2, "hipMalloc(residual)") || !norms.alloc((size_t)out * sizeof(float), "hipMalloc(norms)") ||
            !hip_ok(hipMemcpy(w.p, weight_host, n * sizeof(float), hipMemcpyHostToDevice), "copy weight"))
            return 1;
        if (tq_quantize_weight(w.as<float>(), out, in, cbp, np, cbr, nr, primary_bits, residual_bits, block_size,
                               shared_rotation, pp.as<uint8_t>(), pr.as<uint8_t>(), norms.as<float>(), seeds_host) != 0)
            return 1;
        if (!hip_ok(hipMemcpy(pp_host, pp.p, pbytes, hipMemcpyDeviceToHost), "copy primary") ||
            !hip_ok(hipMemcpy(pr_host, pr.p, n / 2, hipMemcpyDeviceToHost), "copy residual") ||
            !hip_ok(hipMemcpy(norms_host, norms.p, (size_t)out * sizeof(float), hipMemcpyDeviceToHost), "copy norms"))
            return 1;
        return 0;
    } catch (...) { set_error("tq_quantize_weight_host: exception"); return 1; }
}

int tq_fit_layer_codebooks_host(const float* weight_host, int out, int in, uint32_t block_size,
                                int primary_bits, int residual_bits,
                                const float* gcp, int ngc, int iterations, float* cbp_out, float* cbr_out) {
    try {
        if (!weight_host || out <= 0 || in <= 0) { set_error("tq_fit_layer_codebooks_host: bad argument"); return 1; }
        const size_t n = (size_t)out * in;
        DevBuf w;
        if (!w.alloc(n * sizeof(float), "hipMalloc(weight)") ||
            !hip_ok(hipMemcpy(w.p, weight_host, n * sizeof(float), hipMemcpyHostToDevice), "copy weight"))
            return 1;
        return tq_fit_layer_codebooks(w.as<float>(), out, in, block_size, primary_bits, residual_bits, gcp, ngc,
                                      iterations, cbp_out, cbr_out);
    } catch (...) { set_error("tq_fit_layer_codebooks_host: exception"); return 1; }
}

int tq_generate_codebook_from_data_host(const float* data_host, size_t n, int bits, int iterations,
                                        float* centroids_out, float* boundaries_out) {
    try {
        if (!centroids_out || (n > 0 && !data_host)) { set_error("tq_generate_codebook_from_data: NULL argument"); return -1; }
        if (n == 0) return tq_generate_codebook(bits, centroids_out, boundaries_out);   // src/codebook.cpp:101-103
        if (bits < 1 || bits > 5) { set_error("Unsupported bit width; must be 1-5"); return -1; }
        DevBuf d;
        if (!d.alloc(n * sizeof(float), "hipMalloc(samples)") ||
            !hip_ok(hipMemcpy(d.p, data_host, n * sizeof(float), hipMemcpyHostToDevice), "copy samples") ||
            !lloyd_max(d.as<float>(), n, bits, iterations, false, nullptr, nullptr, 0, centroids_out))
            return -1;
        if (boundaries_out) midpoints(centroids_out, 1 << bits, boundaries_out);
        return 1 << bits;
    } catch (...) { set_error("tq_generate_codebook_from_data: exception"); return -1; }
}

int tq_codebook_quantize_host(const float* values_host, size_t n, const float* boundaries_host, int n_centroids,
                              uint8_t* indices_host) {
    try {
        if (n == 0) return 0;
        if (!values_host || !boundaries_host || !indices_host || n_centroids < 2 || n_centroids > 32) {
            set_error("tq_codebook_quantize: bad argument"); return 1;
        }
        DevBuf v, b, o;
        float bounds[32] = {0};
        std::memcpy(bounds, boundaries_host, (n_centroids - 1) * sizeof(float));
        if (!v.alloc(n * sizeof(float), "hipMalloc(values)") || !b.alloc(sizeof(bounds), "hipMalloc(bounds)") ||
            !o.alloc(n, "hipMalloc(indices)") ||
            !hip_ok(hipMemcpy(v.p, values_host, n * sizeof(float), hipMemcpyHostToDevice), "copy values") ||
            !hip_ok(hipMemcpy(b.p, bounds, sizeof(bounds), hipMemcpyHostToDevice), "copy bounds") ||
            !hip_ok(tq::launch_codebook_quantize(v.as<float>(), n, b.as<float>(), n_centroids, o.as<uint8_t>(), nullptr),
                    "codebook quantize") ||
            !hip_ok(hipMemcpy(indices_host, o.p, n, hipMemcpyDeviceToHost), "copy indices"))
            return 1;
        return 0;
    } catch (...) { set_error("tq_codebook_quantize: exception"); return 1; }
}

int tq_codebook_dequantize_host(const uint8_t* indices_host, size_t n, const float* centroids_host, int n_centroids,
                                float* values_host) {
    try {
        if (n == 0) return 0;
        if (!indices_host || !centroids_host || !values_host || n_centroids < 1 || n_centroids > 32) {
            set_error("tq_codebook_dequantize: bad argument"); return 1;
        }
        DevBuf i, c, o;
        float cent[32] = {0};
        std::memcpy(cent, centroids_host, n_centroids * sizeof(float));
        if (!i.alloc(n, "hipMalloc(indices)") || !c.alloc(sizeof(cent), "hipMalloc(centroids)") ||
            !o.alloc(n * sizeof(float), "hipMalloc(values)") ||
            !hip_ok(hipMemcpy(i.p, indices_host, n, hipMemcpyHostToDevice), "copy indices") ||
            !hip_ok(hipMemcpy(c.p, cent, sizeof(cent), hipMemcpyHostToDevice), "copy centroids") ||
            !hip_ok(tq::launch_codebook_lookup(i.as<uint8_t>(), n, c.as<float>(), n_centroids, o.as<float>(), nullptr),
                    "codebook lookup") ||
            !hip_ok(hipMemcpy(values_host, o.p, n * sizeof(float), hipMemcpyDeviceToHost), "copy values"))
            return 1;
        return 0;
    } catch (...) { set_error("tq_codebook_dequantize: exception"); return 1; }
}

}  // extern "C"
