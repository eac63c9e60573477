#pragma once
// Host tensor used at the C++ API boundary in place of the reference's mlx::core::array
// (include/turboquant/quantizer.h:22-27 and every signature in include/turboquant/*.h).
// Value semantics with a shared, immutable-by-convention buffer: copying an Array copies a
// pointer, as copying an mlx array does.  Device memory never appears here; the layer classes
// upload what they need once and keep it resident.

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <vector>

namespace turboquant {

/// Element types, named as the safetensors format names them.
enum class Dtype : uint8_t { F32, F16, BF16, U8, U32, F64, I8, I16, I32, I64, U16, U64, BOOL };

constexpr Dtype float32 = Dtype::F32;
constexpr Dtype float16 = Dtype::F16;
constexpr Dtype bfloat16 = Dtype::BF16;
constexpr Dtype uint8 = Dtype::U8;
constexpr Dtype uint32 = Dtype::U32;

inline size_t dtype_size(Dtype d) {
    switch (d) {
        case Dtype::F64: case Dtype::I64: case Dtype::U64: return 8;
        case Dtype::F32: case Dtype::U32: case Dtype::I32: return 4;
        case Dtype::F16: case Dtype::BF16: case Dtype::I16: case Dtype::U16: return 2;
        default: return 1;
    }
}

class Array {
public:
    Array() : dtype_(Dtype::F32), size_(0) {}

    /// Uninitialised array of the given shape.
    Array(std::vector<int> shape, Dtype dtype) : shape_(std::move(shape)), dtype_(dtype) {
        size_ = 1;
        for (int d : shape_) {
            if (d < 0) throw std::invalid_argument("Array: negative dimension");
            size_ *= static_cast<size_t>(d);
        }
        buf_ = std::shared_ptr<uint8_t>(new uint8_t[nbytes() ? nbytes() : 1], std::default_delete<uint8_t[]>());
    }

    /// Copy `shape` elements of `dtype` from `data`.
    Array(const void* data, std::vector<int> shape, Dtype dtype) : Array(std::move(shape), dtype) {
        if (nbytes()) std::memcpy(buf_.get(), data, nbytes());
    }

    /// fp32 convenience constructor, the form the reference's tests use.
    Array(const float* data, std::vector<int> shape) : Array(data, std::move(shape), Dtype::F32) {}

    const std::vector<int>& shape() const { return shape_; }
    int shape(int axis) const {
        if (axis < 0) axis += static_cast<int>(shape_.size());
        return shape_.at(static_cast<size_t>(axis));
    }
    int ndim() const { return static_cast<int>(shape_.size()); }
    size_t size() const { return size_; }
    size_t nbytes() const { return size_ * dtype_size(dtype_); }
    Dtype dtype() const { return dtype_; }
    bool empty() const { return !buf_; }

    template <typename T> const T* data() const { return reinterpret_cast<const T*>(buf_.get()); }
    template <typename T> T* data() { return reinterpret_cast<T*>(buf_.get()); }

    /// Same buffer, new shape (element count must match).
    Array reshape(std::vector<int> shape) const {
        size_t n = 1;
        for (int d : shape) n *= static_cast<size_t>(d);
        if (n != size_) throw std::invalid_argument("Array::reshape: element count mismatch");
        Array r = *this;
        r.shape_ = std::move(shape);
        return r;
    }

private:
    std::vector<int> shape_;
    Dtype dtype_;
    size_t size_;
    std::shared_ptr<uint8_t> buf_;
};

/// Element-type conversion between fp32, fp16 and bf16 (round to nearest even), on the host.
/// Meant for building inputs and reading outputs; the layer kernels convert on the fly.
Array astype(const Array& a, Dtype dtype);

}  // namespace turboquant
