// Minimal device-resident tensor for the HIP backend: a reference-counted HIP
// buffer, a Shape and a dtype, in Flashlight's column-major [W,H,C,N] layout
// (byte-identical to row-major N,C,H,W).  It stands where fl::Tensor with a HIP
// TensorAdapter would stand (flashlight/fl/tensor/TensorAdapter.h:41-263); only
// what the autograd extension and its caller need is provided.
#pragma once

#include <memory>
#include <vector>

#include "Types.h"

namespace fl {

class Tensor {
 public:
  Tensor() = default;                       // empty tensor: shape {0}
  Tensor(const Shape& shape, dtype type);   // uninitialised device memory

  static Tensor fromHost(const Shape& shape, dtype type, const void* data);
  static Tensor fromVector(const Shape& shape, const std::vector<float>& v) {
    return fromHost(shape, dtype::f32, v.data());
  }
  // fl::full (used for default running statistics, onednn/BatchNorm.cpp:116-122)
  static Tensor full(const Shape& shape, double value, dtype type);

  void toHost(void* dst) const;             // blocking copy of the whole buffer
  std::vector<float> toHostVector() const;  // converts f32 / bf16 / f16 to float

  const Shape& shape() const { return shape_; }
  dtype type() const { return type_; }
  int ndim() const { return shape_.ndim(); }
  Dim dim(int i) const { return shape_.dim(i); }
  Dim elements() const { return buf_ ? shape_.elements() : 0; }
  bool isEmpty() const { return elements() == 0; }
  size_t bytes() const { return (size_t)elements() * getTypeSize(type_); }
  TensorBackendType backendType() const { return TensorBackendType::Hip; }
  bool isContiguous() const { return true; }

  // Tensor::astype among f32, bf16 and f16; other conversions are not part of this path.
  Tensor astype(dtype t) const;
  // the same conversion of several tensors of one type in one launch per 64 of them
  // (flhip_convert_many); tensors that already have type t come back as they are
  static std::vector<Tensor> astypeMany(const std::vector<Tensor>& in, dtype t);
  // same buffer, different shape (fl::reshape / moddims)
  Tensor reshaped(const Shape& s) const;
  // a + b elementwise (Variable::addGrad, flashlight/fl/autograd/Variable.cpp:185-218)
  Tensor copy() const;

  // Raw device pointer; nullptr for an empty tensor.  Use through DevicePtr.
  void* device() const { return buf_ ? buf_->ptr : nullptr; }

 private:
  struct Buffer {
    void* ptr = nullptr;
    size_t bytes = 0;
    ~Buffer();
  };
  std::shared_ptr<Buffer> buf_;
  Shape shape_{0};
  dtype type_ = dtype::f32;
};

// fl::DevicePtr (flashlight/fl/common/DevicePtr.cpp:16-33): RAII access to the raw
// buffer; keeps the tensor alive while a kernel may use the pointer; nullptr for an
// empty tensor.
class DevicePtr {
 public:
  explicit DevicePtr(const Tensor& t) : keep_(t) {}
  void* get() const { return keep_.device(); }

 private:
  Tensor keep_;
};

// The stream every kernel of this backend is enqueued on (hipStream_t as void*;
// nullptr = the null stream), and fl::sync() for it.
// Device buffers of destroyed tensors are cached for reuse; these return them to the
// driver / report how many bytes are parked.
void emptyDeviceCache();
size_t deviceCacheBytes();
void* hipBackendStream();
void setHipBackendStream(void* stream);
void sync();

}  // namespace fl
