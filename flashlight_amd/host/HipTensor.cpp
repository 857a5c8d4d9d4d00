#include "HipTensor.h"

#include <hip/hip_runtime.h>

#include <cstring>

#include "flhip.h"

namespace fl {

namespace {
void hipCheck(hipError_t e, const char* what) {
  if (e != hipSuccess)
    throw std::runtime_error(std::string("HIP backend: ") + what + ": " + hipGetErrorString(e));
}
void* g_stream = nullptr;

int tag(dtype t) {
  if (t == dtype::f32) return FLHIP_F32;
  if (t == dtype::bf16) return FLHIP_BF16;
  throw std::runtime_error("HIP backend: conversion supports f32 and bf16 only");
}
}  // namespace

void* hipBackendStream() { return g_stream; }
void setHipBackendStream(void* stream) { g_stream = stream; }
void sync() { hipCheck(hipStreamSynchronize((hipStream_t)g_stream), "sync"); }

Tensor::Buffer::~Buffer() {
  if (ptr) (void)hipFree(ptr);
}

Tensor::Tensor(const Shape& shape, dtype type) : shape_(shape), type_(type) {
  const size_t n = (size_t)shape.elements() * getTypeSize(type);
  if (shape.elements() < 0) throw std::invalid_argument("Tensor: negative dimension");
  if (n == 0) return;
  buf_ = std::make_shared<Buffer>();
  hipCheck(hipMalloc(&buf_->ptr, n), "hipMalloc");
  buf_->bytes = n;
}

Tensor Tensor::fromHost(const Shape& shape, dtype type, const void* data) {
  Tensor t(shape, type);
  if (!t.isEmpty()) {
    // a blocking copy on the backend stream keeps it ordered with earlier kernels
    hipCheck(hipMemcpyAsync(t.device(), data, t.bytes(), hipMemcpyHostToDevice, (hipStream_t)g_stream),
             "copy to device");
    sync();
  }
  return t;
}

Tensor Tensor::full(const Shape& shape, double value, dtype type) {
  if (type != dtype::f32) throw std::runtime_error("Tensor::full: f32 only");
  std::vector<float> v((size_t)shape.elements(), (float)value);
  return fromHost(shape, type, v.data());
}

void Tensor::toHost(void* dst) const {
  if (isEmpty()) return;
  hipCheck(hipMemcpyAsync(dst, device(), bytes(), hipMemcpyDeviceToHost, (hipStream_t)g_stream),
           "copy to host");
  sync();
}

std::vector<float> Tensor::toHostVector() const {
  std::vector<float> out((size_t)elements());
  if (isEmpty()) return out;
  if (type_ == dtype::f32) {
    toHost(out.data());
  } else if (type_ == dtype::bf16) {
    astype(dtype::f32).toHost(out.data());
  } else {
    throw std::runtime_error("toHostVector: f32 and bf16 only");
  }
  return out;
}

Tensor Tensor::astype(dtype t) const {
  if (t == type_ || isEmpty()) {
    Tensor r = *this;
    r.type_ = isEmpty() ? t : type_;
    return r;
  }
  Tensor out(shape_, t);
  const int rc = flhip_convert(device(), tag(type_), out.device(), tag(t), (size_t)elements(), g_stream);
  if (rc != FLHIP_OK) throw std::runtime_error(flhip_last_error());
  return out;
}

Tensor Tensor::reshaped(const Shape& s) const {
  if (s.elements() != shape_.elements()) throw std::invalid_argument("reshape: element count differs");
  Tensor r = *this;
  r.shape_ = s;
  return r;
}

Tensor Tensor::copy() const {
  Tensor out(shape_, type_);
  if (!isEmpty())
    hipCheck(hipMemcpyAsync(out.device(), device(), bytes(), hipMemcpyDeviceToDevice, (hipStream_t)g_stream),
             "copy");
  return out;
}

}  // namespace fl
