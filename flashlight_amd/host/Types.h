// Interface types of the AutogradExtension boundary, restated for the HIP
// backend.  Flashlight itself cannot be built offline, so the host layer carries
// its own copies of these small types with the reference's names and meaning.
#pragma once

#include <initializer_list>
#include <stdexcept>
#include <string>
#include <vector>

namespace fl {

using Dim = long long;

// fl::dtype (flashlight/fl/tensor/Types.h:17-30) plus a private bf16 tag: the
// reference has no bf16; here it means bf16 storage with fp32 accumulation.
enum class dtype { f16 = 0, f32 = 1, f64 = 2, b8 = 3, s16 = 4, s32 = 5, s64 = 6, u8 = 7, u16 = 8,
                   u32 = 9, u64 = 10, bf16 = 100 };

inline size_t getTypeSize(dtype t) {
  switch (t) {
    case dtype::f16: case dtype::bf16: case dtype::s16: case dtype::u16: return 2;
    case dtype::f32: case dtype::s32: case dtype::u32: return 4;
    case dtype::f64: case dtype::s64: case dtype::u64: return 8;
    default: return 1;
  }
}

// fl::Shape (flashlight/fl/tensor/Shape.h:20-47): column-major dimensions; {} is a
// scalar (1 element), {0} is empty.
class Shape {
 public:
  Shape() = default;
  Shape(std::initializer_list<Dim> d) : dims_(d) {}
  explicit Shape(std::vector<Dim> d) : dims_(std::move(d)) {}
  int ndim() const { return (int)dims_.size(); }
  Dim dim(int i) const {
    if (i < 0 || i >= ndim()) throw std::invalid_argument("Shape::dim - index out of range");
    return dims_[i];
  }
  Dim operator[](int i) const { return dim(i); }
  Dim elements() const {
    Dim n = 1;
    for (Dim d : dims_) n *= d;
    return n;
  }
  const std::vector<Dim>& get() const { return dims_; }
  bool operator==(const Shape& o) const { return dims_ == o.dims_; }
  bool operator!=(const Shape& o) const { return !(*this == o); }
  std::string toString() const {
    std::string s = "(";
    for (size_t i = 0; i < dims_.size(); ++i) s += (i ? ", " : "") + std::to_string(dims_[i]);
    return s + ")";
  }

 private:
  std::vector<Dim> dims_;
};

// flashlight/fl/common/Defines.h:53-79
enum class PoolingMode { MAX = 0, AVG_INCLUDE_PADDING = 1, AVG_EXCLUDE_PADDING = 2 };
enum class RnnMode { RELU = 0, TANH = 1, LSTM = 2, GRU = 3 };
enum class PaddingMode { SAME = -1 };

// Backends a tensor can live on (flashlight/fl/tensor/TensorBase.h:32 is a closed
// enum; registering this backend inside Flashlight adds the Hip value).
enum class TensorBackendType { Stub, Tensor, ArrayFire, OneDnn, Jit, Hip };
enum class TensorExtensionType { Generic, Autograd, Vision, JitOptimizer };

class DynamicBenchmark;  // DynamicBenchmark.h

}  // namespace fl
