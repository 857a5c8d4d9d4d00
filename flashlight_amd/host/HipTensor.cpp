#include "HipTensor.h"
#include "DynamicBenchmark.h"
#include "OpObserver.h"

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstring>
#include <map>
#include <mutex>

#include "flhip.h"

namespace fl {

namespace {
void hipCheck(hipError_t e, const char* what) {
  if (e != hipSuccess)
    throw std::runtime_error(std::string("HIP backend: ") + what + ": " + hipGetErrorString(e));
}
void* g_stream = nullptr;

// Freed buffers are kept and handed out again by size class instead of going back to the
// driver: hipFree waits for the device, and a training step frees hundreds of
// intermediate tensors.  Reuse needs no event because every kernel of this backend is
// enqueued on the one backend stream, in program order.  Flashlight has a caching memory
// manager in the same place (flashlight/fl/memory/managers/CachingMemoryManager.cpp).
class DevicePool {
 public:
  static DevicePool& get() {
    static DevicePool* pool = new DevicePool;   // never destroyed: the HIP runtime may be gone by then
    return *pool;
  }
  static size_t sizeClass(size_t n) {
    const size_t q = n < (1u << 20) ? 512 : (1u << 20);
    return (n + q - 1) / q * q;
  }
  void* take(size_t n, size_t* granted) {
    const size_t cls = sizeClass(n);
    *granted = cls;
    {
      std::lock_guard<std::mutex> lock(mu_);
      auto it = free_.find(cls);
      if (it != free_.end() && !it->second.empty()) {
        void* p = it->second.back();
        it->second.pop_back();
        cached_ -= cls;
        return p;
      }
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
      // out of memory with buffers parked here: give them back and try once more
      (void)hipGetLastError();
      release();
      e = hipMalloc(&p, cls);
    }
    hipCheck(e, "hipMalloc");
    return p;
  }
  void give(void* p, size_t cls) {
    std::lock_guard<std::mutex> lock(mu_);
    free_[cls].push_back(p);
    cached_ += cls;
  }
  void release() {
    std::map<size_t, std::vector<void*>> all;
    {
      std::lock_guard<std::mutex> lock(mu_);
      all.swap(free_);
      cached_ = 0;
    }
    for (auto& kv : all)
      for (void* p : kv.second) (void)hipFree(p);
  }
  size_t cachedBytes() {
    std::lock_guard<std::mutex> lock(mu_);
    return cached_;
  }

 private:
  std::mutex mu_;
  std::map<size_t, std::vector<void*>> free_;
  size_t cached_ = 0;
};

int tag(dtype t) {
  if (t == dtype::f32) return FLHIP_F32;
  if (t == dtype::bf16) return FLHIP_BF16;
  if (t == dtype::f16) return FLHIP_F16;
  throw std::runtime_error("HIP backend: conversion supports f32, bf16 and f16 only");
}
}  // namespace

namespace detail {
namespace {
OpObserver* g_observer = nullptr;
}
OpObserver* opObserver() { return g_observer; }
void setOpObserver(OpObserver* observer) { g_observer = observer; }
}  // namespace detail

// ---- StepProfiler -------------------------------------------------------------------
// ---- DynamicBenchmark --------------------------------------------------------------------
namespace {
bool g_benchmarkMode = false;   // flashlight/fl/common/DynamicBenchmark.cpp:13: off by default
}
void DynamicBenchmark::setBenchmarkMode(bool mode) { g_benchmarkMode = mode; }
bool DynamicBenchmark::getBenchmarkMode() { return g_benchmarkMode; }

// flashlight/fl/common/DynamicBenchmark.cpp:15-42: wait for the device, time the function on the host clock until
// the device has finished what it enqueued
void DynamicBenchmark::audit(const std::function<void()>& function, bool incrementCount) {
  if (!g_benchmarkMode || options_->timingsComplete()) {
    function();
    return;
  }
  sync();
  const auto t0 = std::chrono::steady_clock::now();
  function();
  sync();
  const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  // (the function may have marked its option unusable: then there is nothing left to add to)
  if (!options_->timingsComplete()) options_->accumulateTimeToCurrentOption(seconds, incrementCount);
}

struct StepProfiler::Impl {
  struct Span {
    std::string op;
    hipEvent_t start, stop;
  };
  std::vector<Span> spans;
  std::vector<hipEvent_t> spare;
  int depth = 0;
  hipEvent_t event() {
    if (!spare.empty()) {
      hipEvent_t e = spare.back();
      spare.pop_back();
      return e;
    }
    hipEvent_t e;
    hipCheck(hipEventCreate(&e), "hipEventCreate");
    return e;
  }
};

StepProfiler::StepProfiler() : impl_(new Impl) {}
StepProfiler::~StepProfiler() {
  if (detail::opObserver() == this) detail::setOpObserver(nullptr);
  for (auto& s : impl_->spans) {
    (void)hipEventDestroy(s.start);
    (void)hipEventDestroy(s.stop);
  }
  for (hipEvent_t e : impl_->spare) (void)hipEventDestroy(e);
  delete impl_;
}

void StepProfiler::begin(const char* op) {
  if (impl_->depth++ > 0) return;
  Impl::Span s{op, impl_->event(), impl_->event()};
  hipCheck(hipEventRecord(s.start, (hipStream_t)g_stream), "hipEventRecord");
  impl_->spans.push_back(s);
}

void StepProfiler::end(const detail::OpEvent&) {
  if (--impl_->depth > 0) return;
  hipCheck(hipEventRecord(impl_->spans.back().stop, (hipStream_t)g_stream), "hipEventRecord");
}

// An operation that left early still closes its span (what it enqueued before leaving counts
// towards it), so that depth returns to zero and every span has both events recorded.
void StepProfiler::abort(const char*) {
  if (impl_->depth <= 0 || --impl_->depth > 0) return;
  (void)hipEventRecord(impl_->spans.back().stop, (hipStream_t)g_stream);
}

std::map<std::string, StepProfiler::Entry> StepProfiler::collect() {
  sync();
  impl_->depth = 0;
  std::map<std::string, Entry> out;
  double busy = 0;
  for (auto& s : impl_->spans) {
    float ms = 0;
    hipCheck(hipEventElapsedTime(&ms, s.start, s.stop), "hipEventElapsedTime");
    out[s.op].ms += ms;
    out[s.op].calls += 1;
    busy += ms;
  }
  if (!impl_->spans.empty()) {
    float span = 0;
    hipCheck(hipEventElapsedTime(&span, impl_->spans.front().start, impl_->spans.back().stop), "hipEventElapsedTime");
    out["(span)"].ms = span;
    out["(span)"].calls = 1;
    out["(gaps)"].ms = span - busy;
    out["(gaps)"].calls = 1;
  }
  for (auto& s : impl_->spans) {
    impl_->spare.push_back(s.start);
    impl_->spare.push_back(s.stop);
  }
  impl_->spans.clear();
  return out;
}

void* hipBackendStream() { return g_stream; }
void setHipBackendStream(void* stream) {
  // cached buffers are reused in program order of one stream: drain the old one first
  if (stream != g_stream) sync();
  g_stream = stream;
}
void sync() { hipCheck(hipStreamSynchronize((hipStream_t)g_stream), "sync"); }

void emptyDeviceCache() { DevicePool::get().release(); }
size_t deviceCacheBytes() { return DevicePool::get().cachedBytes(); }

Tensor::Buffer::~Buffer() {
  if (ptr) DevicePool::get().give(ptr, bytes);
}

Tensor::Tensor(const Shape& shape, dtype type) : shape_(shape), type_(type) {
  const size_t n = (size_t)shape.elements() * getTypeSize(type);
  if (shape.elements() < 0) throw std::invalid_argument("Tensor: negative dimension");
  if (n == 0) return;
  buf_ = std::make_shared<Buffer>();
  buf_->ptr = DevicePool::get().take(n, &buf_->bytes);   // bytes = the size class granted
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
  // a fill kernel on the backend stream: no host buffer, no synchronisation
  Tensor t(shape, type);
  if (flhip_fill(t.device(), value, (size_t)t.elements(), tag(type), g_stream) != FLHIP_OK)
    throw std::runtime_error(flhip_last_error());
  return t;
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
  } else if (type_ == dtype::bf16 || type_ == dtype::f16) {
    astype(dtype::f32).toHost(out.data());
  } else {
    throw std::runtime_error("toHostVector: f32, bf16 and f16 only");
  }
  return out;
}

Tensor Tensor::astype(dtype t) const {
  if (t == type_ || isEmpty()) {
    Tensor r = *this;
    r.type_ = isEmpty() ? t : type_;
    return r;
  }
  detail::OpScope scope("astype");
  Tensor out(shape_, t);
  const int rc = flhip_convert(device(), tag(type_), out.device(), tag(t), (size_t)elements(), g_stream);
  if (rc != FLHIP_OK) throw std::runtime_error(flhip_last_error());
  if (scope.on()) scope.done({*this}, {out});
  return out;
}

std::vector<Tensor> Tensor::astypeMany(const std::vector<Tensor>& in, dtype t) {
  std::vector<Tensor> out(in.size());
  std::vector<const void*> src;
  std::vector<void*> dst;
  std::vector<size_t> n;
  std::vector<Tensor> evIn, evOut;
  int from = -1;
  for (size_t i = 0; i < in.size(); ++i) {
    if (in[i].isEmpty() || in[i].type() == t) {
      out[i] = in[i].astype(t);
      continue;
    }
    if (from >= 0 && tag(in[i].type()) != from) throw std::invalid_argument("astypeMany: the tensors must share a type");
    from = tag(in[i].type());
    out[i] = Tensor(in[i].shape(), t);
    src.push_back(in[i].device());
    dst.push_back(out[i].device());
    n.push_back((size_t)in[i].elements());
    evIn.push_back(in[i]);
    evOut.push_back(out[i]);
  }
  if (src.empty()) return out;
  detail::OpScope scope("astype");
  const int rc = flhip_convert_many(src.data(), dst.data(), n.data(), (int)src.size(), from, tag(t), g_stream);
  if (rc != FLHIP_OK) throw std::runtime_error(flhip_last_error());
  if (scope.on()) scope.done(evIn, evOut);   // pairs: inputs[i] -> outputs[i]
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
