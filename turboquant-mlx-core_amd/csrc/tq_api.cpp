// C++ API of the quantized-linear path (include/turboquant/*.h) on top of the C-ABI.
// Host plumbing only: argument checks, exceptions, buffer ownership.  Every element-level
// operation is a HIP kernel behind the tq_* entry points.
#include "turboquant/turboquant.h"

#include <cmath>
#include <stdexcept>
#include <string>

#include "turboquant_c/tq_linear.h"
#include "turboquant_c/tq_quantizer.h"

namespace turboquant {

namespace {

[[noreturn]] void fail(const char* who) {
    const char* msg = tq_last_error();
    throw std::runtime_error(std::string(who) + ": " + (msg && *msg ? msg : "failed"));
}

int c_dtype(Dtype d, const char* who) {
    switch (d) {
        case Dtype::F32: return TQ_DTYPE_F32;
        case Dtype::F16: return TQ_DTYPE_F16;
        case Dtype::BF16: return TQ_DTYPE_BF16;
        default: throw std::invalid_argument(std::string(who) + ": element type must be fp32, fp16 or bf16");
    }
}

void require(bool ok, const char* msg) {
    if (!ok) throw std::invalid_argument(msg);
}

void check_weights(const QuantizedWeight& qw, const char* who) {
    require(qw.packed_primary.ndim() == 2 && qw.packed_primary.dtype() == Dtype::U8,
            (std::string(who) + ": packed_primary must be uint8 [out, cols]").c_str());
    require(qw.packed_residual.ndim() == 2 && qw.packed_residual.dtype() == Dtype::U8,
            (std::string(who) + ": packed_residual must be uint8 [out, cols]").c_str());
    require(qw.norms.dtype() == Dtype::F32 && (int)qw.norms.size() == qw.packed_primary.shape(0),
            (std::string(who) + ": norms must be float32 [out]").c_str());
    require(qw.seeds.dtype() == Dtype::U32 && qw.seeds.size() >= 3,
            (std::string(who) + ": seeds must be uint32 [3]").c_str());
    require(qw.packed_residual.shape(0) == qw.packed_primary.shape(0),
            (std::string(who) + ": plane row counts differ").c_str());
}

// in_features from the plane shapes (reference src/dequantizer.cpp:59-75): the residual plane is
// always nibble packed, so in = 2 * residual columns.
tq_linear_s* make_handle(int in_features, int out_features, const QuantizedWeight& qw, const Codebook& cbp,
                         const Codebook& cbr, uint32_t block_size, const char* who) {
    check_weights(qw, who);
    tq_linear_s* h = tq_linear_create(in_features, out_features,
                                      qw.packed_primary.data<uint8_t>(), qw.packed_primary.shape(1),
                                      qw.packed_residual.data<uint8_t>(), qw.packed_residual.shape(1),
                                      qw.norms.data<float>(), qw.seeds.data<uint32_t>(),
                                      cbp.centroids.data(), (int)cbp.centroids.size(),
                                      cbr.centroids.data(), (int)cbr.centroids.size(), block_size);
    if (!h) fail(who);
    return h;
}

Codebook codebook_from(const float* c, const float* b, int n, uint8_t bits, CodebookOrigin origin) {
    Codebook cb;
    cb.centroids.assign(c, c + n);
    cb.boundaries.assign(b, b + (n - 1));
    cb.bits = bits;
    cb.origin = origin;
    return cb;
}

uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float bf16_to_f32(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

thread_local bool g_force_cpu = false;

}  // namespace

const char* version() { return "0.1.0"; }

// ---------------------------------------------------------------------------
// Array helpers
// ---------------------------------------------------------------------------
Array astype(const Array& a, Dtype dtype) {
    if (a.dtype() == dtype) return a;
    const bool src_ok = a.dtype() == Dtype::F32 || a.dtype() == Dtype::F16 || a.dtype() == Dtype::BF16;
    const bool dst_ok = dtype == Dtype::F32 || dtype == Dtype::F16 || dtype == Dtype::BF16;
    if (!src_ok || !dst_ok) throw std::invalid_argument("astype: only fp32 / fp16 / bf16 conversions");
    const size_t n = a.size();
    std::vector<float> wide(n);
    if (a.dtype() == Dtype::F32) std::memcpy(wide.data(), a.data<float>(), n * 4);
    else if (a.dtype() == Dtype::BF16) for (size_t i = 0; i < n; ++i) wide[i] = bf16_to_f32(a.data<uint16_t>()[i]);
    else for (size_t i = 0; i < n; ++i) wide[i] = (float)a.data<_Float16>()[i];
    Array out(a.shape(), dtype);
    if (dtype == Dtype::F32) std::memcpy(out.data<float>(), wide.data(), n * 4);
    else if (dtype == Dtype::BF16) for (size_t i = 0; i < n; ++i) out.data<uint16_t>()[i] = f32_to_bf16(wide[i]);
    else for (size_t i = 0; i < n; ++i) out.data<_Float16>()[i] = (_Float16)wide[i];
    return out;
}

// ---------------------------------------------------------------------------
// Codebooks
// ---------------------------------------------------------------------------
Codebook generate_codebook(uint8_t bits) {
    float c[32], b[32];
    const int n = tq_generate_codebook(bits, c, b);
    if (n < 0) throw std::invalid_argument("Unsupported bit width; must be 1-5");
    return codebook_from(c, b, n, bits, CodebookOrigin::Analytical);
}

Codebook generate_codebook_from_data(const std::vector<float>& data, uint8_t bits, int iterations) {
    if (data.empty()) return generate_codebook(bits);
    float c[32], b[32];
    const int n = tq_generate_codebook_from_data_host(data.data(), data.size(), bits, iterations, c, b);
    if (n < 0) {
        if (bits < 1 || bits > 5) throw std::invalid_argument("Unsupported bit width; must be 1-5");
        fail("generate_codebook_from_data");
    }
    return codebook_from(c, b, n, bits, CodebookOrigin::Empirical);
}

Array quantize(const Array& values, const Codebook& codebook) {
    require(values.dtype() == Dtype::F32, "quantize: values must be float32");
    Array out({(int)values.size()}, Dtype::U8);
    if (tq_codebook_quantize_host(values.data<float>(), values.size(), codebook.boundaries.data(),
                                  (int)codebook.centroids.size(), out.data<uint8_t>()) != 0)
        fail("quantize");
    return out;
}

Array dequantize(const Array& indices, const Codebook& codebook) {
    require(indices.dtype() == Dtype::U8, "dequantize: indices must be uint8");
    Array out({(int)indices.size()}, Dtype::F32);
    if (tq_codebook_dequantize_host(indices.data<uint8_t>(), indices.size(), codebook.centroids.data(),
                                    (int)codebook.centroids.size(), out.data<float>()) != 0)
        fail("dequantize");
    return out;
}

bool validate_codebook(const Codebook& codebook) {
    const auto& c = codebook.centroids;
    const auto& b = codebook.boundaries;
    if (codebook.bits > 31 || c.size() != (size_t(1) << codebook.bits)) return false;
    for (size_t i = 1; i < c.size(); ++i)
        if (!(c[i] > c[i - 1])) return false;
    if (b.size() + 1 != c.size()) return false;
    for (size_t i = 0; i < b.size(); ++i)
        if (std::fabs(b[i] - (c[i] + c[i + 1]) * 0.5f) > 1e-5f) return false;
    if (codebook.origin == CodebookOrigin::Analytical)
        for (size_t lo = 0, hi = c.size() - 1; lo < hi; ++lo, --hi)
            if (c[lo] + c[hi] != 0.0f) return false;
    return true;
}

// ---------------------------------------------------------------------------
// Rotation and the quantizer
// ---------------------------------------------------------------------------
static Array rotate(const Array& m, uint32_t seed, uint32_t block_size, int inverse, const char* who) {
    require(m.dtype() == Dtype::F32 && m.ndim() == 2, "WHT rotation: matrix must be float32 [rows, cols]");
    if (block_size == 0 || m.shape(1) % (int)block_size != 0)
        throw std::invalid_argument(std::string(who) + ": columns must be divisible by block_size");
    Array out(m.shape(), Dtype::F32);
    if (m.size() == 0) return out;
    if (tq_wht_rotate_host(m.data<float>(), out.data<float>(), m.shape(0), m.shape(1), seed, block_size, inverse) != 0)
        fail(who);
    return out;
}

Array apply_wht_rotation(const Array& matrix, uint32_t seed, uint32_t block_size) {
    return rotate(matrix, seed, block_size, 0, "apply_wht_rotation");
}

Array apply_inverse_wht_rotation(const Array& matrix, uint32_t seed, uint32_t block_size) {
    return rotate(matrix, seed, block_size, 1, "apply_inverse_wht_rotation");
}

void set_force_cpu(bool force_cpu) { g_force_cpu = force_cpu; }
bool get_force_cpu() { return g_force_cpu; }

QuantizedWeight quantize_weight(const Array& weight, const Codebook& primary_codebook,
                                const Codebook& residual_codebook, const QuantizerConfig& config) {
    require(weight.dtype() == Dtype::F32 && weight.ndim() == 2, "quantize_weight: weight must be float32 [out, in]");
    const int out = weight.shape(0), in = weight.shape(1);
    QuantizedWeight qw;
    qw.packed_primary = Array({out, config.primary_bits <= 4 ? in / 2 : in}, Dtype::U8);
    qw.packed_residual = Array({out, in / 2}, Dtype::U8);
    qw.norms = Array({out}, Dtype::F32);
    qw.seeds = Array({3}, Dtype::U32);
    if (tq_quantize_weight_host(weight.data<float>(), out, in,
                                primary_codebook.centroids.data(), (int)primary_codebook.centroids.size(),
                                residual_codebook.centroids.data(), (int)residual_codebook.centroids.size(),
                                config.primary_bits, config.residual_bits, config.block_size,
                                config.shared_rotation ? 1 : 0,
                                qw.packed_primary.data<uint8_t>(), qw.packed_residual.data<uint8_t>(),
                                qw.norms.data<float>(), qw.seeds.data<uint32_t>()) != 0)
        fail("quantize_weight");
    return qw;
}

// ---------------------------------------------------------------------------
// Dequantizer and the fused forward
// ---------------------------------------------------------------------------
Array dequantize_weight_gpu(const QuantizedWeight& qw, const Codebook& primary_codebook,
                            const Codebook& residual_codebook, uint32_t block_size) {
    check_weights(qw, "dequantize_weight");
    const int out = qw.packed_primary.shape(0);
    const int in = qw.packed_residual.shape(1) * 2;
    std::shared_ptr<tq_linear_s> h(make_handle(in, out, qw, primary_codebook, residual_codebook, block_size,
                                               "dequantize_weight"), tq_linear_free);
    Array w({out, in}, Dtype::F32);
    if (tq_linear_dequantize_host(h.get(), w.data<float>()) != 0) fail("dequantize_weight");
    return w;
}

Array dequantize_weight_cpu(const QuantizedWeight& qw, const Codebook& primary_codebook,
                            const Codebook& residual_codebook, uint32_t block_size) {
    return dequantize_weight_gpu(qw, primary_codebook, residual_codebook, block_size);
}

Array fused_dequant_matmul(const QuantizedWeight& qw, const Codebook& primary_codebook,
                           const Codebook& residual_codebook, uint32_t block_size, const Array& input) {
    check_weights(qw, "fused_dequant_matmul");
    const int out = qw.packed_primary.shape(0);
    const int in = qw.packed_residual.shape(1) * 2;
    TurboQuantLinear layer(in, out, qw, primary_codebook, residual_codebook, block_size);
    return layer.forward(input);
}

// ---------------------------------------------------------------------------
// TurboQuantLinear
// ---------------------------------------------------------------------------
TurboQuantLinear::TurboQuantLinear(int in_features, int out_features, const QuantizedWeight& weights,
                                   const Codebook& primary_codebook, const Codebook& residual_codebook,
                                   uint32_t block_size)
    : in_features_(in_features), out_features_(out_features),
      handle_(make_handle(in_features, out_features, weights, primary_codebook, residual_codebook, block_size,
                          "TurboQuantLinear"), tq_linear_free) {}

Array TurboQuantLinear::forward(const Array& input) { return forward(input, input.dtype()); }

Array TurboQuantLinear::forward(const Array& input, Dtype output_dtype) {
    if (input.ndim() < 1 || input.shape(-1) != in_features_)
        throw std::runtime_error("TurboQuantLinear::forward: input must be [batch, in_features]");
    const int batch = (int)(input.size() / (size_t)in_features_);
    std::vector<int> shape = input.shape();
    shape.back() = out_features_;
    Array y(shape, output_dtype);
    if (batch == 0) return y;
    if (tq_linear_forward_host(handle_.get(), input.data<uint8_t>(), c_dtype(input.dtype(), "forward"), batch,
                               y.data<uint8_t>(), c_dtype(output_dtype, "forward")) != 0)
        fail("TurboQuantLinear::forward");
    return y;
}

void TurboQuantLinear::forward_device(const void* x_dev, Dtype x_dtype, int batch, void* y_dev, Dtype y_dtype,
                                      void* stream) {
    if (tq_linear_forward(handle_.get(), x_dev, c_dtype(x_dtype, "forward_device"), batch, y_dev,
                          c_dtype(y_dtype, "forward_device"), stream) != 0)
        fail("TurboQuantLinear::forward_device");
}

Array TurboQuantLinear::dequantize() const {
    Array w({out_features_, in_features_}, Dtype::F32);
    if (tq_linear_dequantize_host(handle_.get(), w.data<float>()) != 0) fail("TurboQuantLinear::dequantize");
    return w;
}

int TurboQuantLinear::in_features() const { return in_features_; }
int TurboQuantLinear::out_features() const { return out_features_; }

}  // namespace turboquant
