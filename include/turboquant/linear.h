#pragma once
// TQ8 linear layer.  Same class as the reference's include/turboquant/linear.h:11-35, with
// turboquant::Array in place of mlx::core::array, plus device-pointer entry points for
// callers that keep activations in GPU memory.

#include "array.h"
#include "codebook.h"
#include "quantizer.h"
#include <memory>

struct tq_linear_s;

namespace turboquant {

class TurboQuantLinear {
public:
    /// Uploads the packed planes, norms and decode tables to the GPU once.
    /// Throws std::runtime_error on shape errors (reference src/dequantizer.cpp:494).
    TurboQuantLinear(int in_features, int out_features, const QuantizedWeight& weights,
                     const Codebook& primary_codebook, const Codebook& residual_codebook,
                     uint32_t block_size);

    /// input [batch, in_features] fp32 / fp16 / bf16 -> [batch, out_features] in the same
    /// element type (reference linear.h:21-23).
    Array forward(const Array& input);

    /// Same with an explicit output element type (fp32 logits from bf16 activations, say).
    Array forward(const Array& input, Dtype output_dtype);

    /// Activations and outputs already in GPU memory; `stream` is a hipStream_t (NULL = default
    /// stream).  Asynchronous: returns once the kernels are queued.
    void forward_device(const void* x_dev, Dtype x_dtype, int batch, void* y_dev, Dtype y_dtype,
                        void* stream = nullptr);

    /// fp32 [out, in] dequantised weight (same kernel as dequantize_weight_gpu).
    Array dequantize() const;

    int in_features() const;
    int out_features() const;

    /// The C handle behind this layer (owned by the layer).
    tq_linear_s* handle() const { return handle_.get(); }

private:
    int in_features_;
    int out_features_;
    std::shared_ptr<tq_linear_s> handle_;
};

}  // namespace turboquant
