// Error state, version and the calibration copy kernel of the C ABI.
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include <cmath>

#include "common.h"

namespace flhip {

// ---- process-wide switches ----
static Options g_options;
static std::once_flag g_options_once;

// One switch from its text; value == nullptr restores the default.  false: unknown name or value.
static bool apply_option(Options& o, const char* name, const char* v) {
  const Options def;
  auto flag = [&](bool* f) {
    *f = v != nullptr && strcmp(v, "0") != 0;
    return true;
  };
  if (!strcmp(name, "CONV_ALGO")) {
    if (!v || !*v) o.conv_algo = def.conv_algo;
    else if (!strcmp(v, "direct")) o.conv_algo = Options::ALGO_DIRECT;
    else if (!strcmp(v, "gather")) o.conv_algo = Options::ALGO_GATHER;
    else if (!strcmp(v, "tapped")) o.conv_algo = Options::ALGO_TAPPED;
    else if (!strcmp(v, "convert")) o.conv_algo = Options::ALGO_CONVERT;
    else if (!strcmp(v, "auto")) o.conv_algo = Options::ALGO_AUTO;
    else return false;
    return true;
  }
  if (!strcmp(name, "CONV_SKIP")) {
    unsigned m = 0;
    if (v) {
      if (strstr(v, "bf16")) m |= Options::SKIP_BF16;
      if (strstr(v, "gemm1x1")) m |= Options::SKIP_GEMM1X1;
      if (strstr(v, "slab")) m |= Options::SKIP_SLAB;
      if (strstr(v, "tapped")) m |= Options::SKIP_TAPPED;
      if (strstr(v, "strip")) m |= Options::SKIP_STRIP;
      if (strstr(v, "first")) m |= Options::SKIP_FIRST;
      if (strstr(v, "wgrad128")) m |= Options::SKIP_WGRAD128;
      if (strstr(v, "pwdma")) m |= Options::SKIP_PWDMA;
      if (strstr(v, "wd32")) m |= Options::SKIP_WD32;
      if (strstr(v, "tap1d")) m |= Options::SKIP_TAP1D;
      if (strstr(v, "cells")) m |= Options::SKIP_CELLS;
      if (strstr(v, "tap2d")) m |= Options::SKIP_TAP2D;
    }
    o.conv_skip = m;
    return true;
  }
  if (!strcmp(name, "PW_PT")) {
    const int n = v ? atoi(v) : def.pw_pt;
    if (n != 2 && n != 4 && n != 8) return false;
    o.pw_pt = n;
    return true;
  }
  if (!strcmp(name, "PW16_PF")) {
    const int n = v ? atoi(v) : 0;
    if (n != 0 && n != 1 && n != 2 && n != 4 && n != 8) return false;
    o.pw16_pf = n;
    return true;
  }
  if (!strcmp(name, "BN_ALGO")) {
    if (!v || !*v || !strcmp(v, "auto")) o.bn_algo = 0;
    else if (!strcmp(v, "split")) o.bn_algo = 1;
    else if (!strcmp(v, "resident")) o.bn_algo = 2;
    else return false;
    return true;
  }
  if (!strcmp(name, "CONV_STACK")) {
    const int n = v ? atoi(v) : 0;
    if (n != 0 && n != 1 && n != 2 && n != 4 && n != 8) return false;
    o.conv_stack = n;
    return true;
  }
  if (!strcmp(name, "SLAB_WAVES")) {
    const int n = v ? atoi(v) : 0;
    if (n != 0 && n != 4 && n != 8) return false;
    o.slab_waves = n;
    return true;
  }
  if (!strcmp(name, "PW16_NO_TAPS")) return flag(&o.pw16_no_taps);
  if (!strcmp(name, "TAPPED_NO_REORDER")) return flag(&o.tapped_no_reorder);
  if (!strcmp(name, "MATMUL_VALU")) return flag(&o.matmul_valu);
  if (!strcmp(name, "MATMUL_FP32_CORES")) return flag(&o.matmul_fp32_cores);
  if (!strcmp(name, "MATMUL_PLANES")) { o.matmul_planes = v ? atoi(v) : def.matmul_planes; return true; }
  if (!strcmp(name, "RNN_UNFUSED")) return flag(&o.rnn_unfused);
  if (!strcmp(name, "TAP2D_ALL")) return flag(&o.tap2d_all);
  return false;
}

static void options_from_environment() {
  static const char* const names[] = {"CONV_ALGO", "CONV_SKIP", "PW_PT", "PW16_PF", "CONV_STACK", "SLAB_WAVES", "BN_ALGO", "PW16_NO_TAPS",
                                      "TAPPED_NO_REORDER", "MATMUL_VALU", "MATMUL_FP32_CORES", "MATMUL_PLANES", "RNN_UNFUSED", "TAP2D_ALL"};
  for (const char* n : names) {
    const std::string var = std::string("FLHIP_") + n;
    if (const char* v = getenv(var.c_str())) apply_option(g_options, n, v);   // unknown values keep the default
  }
}

const Options& options() {
  std::call_once(g_options_once, options_from_environment);
  return g_options;
}

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }
int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}

__global__ void __launch_bounds__(256) copy16_kernel(const uint4* __restrict__ src,
                                                      uint4* __restrict__ dst,
                                                      size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}

template <typename S, typename D>
__global__ void __launch_bounds__(256) convert_kernel(const S* __restrict__ src,
                                                       D* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
    st(dst, i, ld(src, i));
}

// Several conversions in one launch: up to CM_MAX (source, destination, length) triples travel in
// the kernel arguments; workgroup b works on the triple whose range of 2048-element pieces
// contains b.
constexpr int CM_MAX = 64;
struct ConvertMany {
  const void* src[CM_MAX];
  void* dst[CM_MAX];
  unsigned first[CM_MAX + 1];   // first piece of entry i; first[count] = pieces in all
  unsigned long long n[CM_MAX];
  int count;
};
template <typename S, typename D>
__global__ void __launch_bounds__(256) convert_many_kernel(ConvertMany a) {
  int lo = 0, hi = a.count;          // the entry with first[e] <= blockIdx.x < first[e + 1]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.first[mid] <= blockIdx.x) lo = mid; else hi = mid;
  }
  const S* src = static_cast<const S*>(a.src[lo]);
  D* dst = static_cast<D*>(a.dst[lo]);
  const size_t base = (size_t)(blockIdx.x - a.first[lo]) * 2048;
  const size_t n = a.n[lo];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const size_t i = base + (size_t)k * 256 + threadIdx.x;
    if (i < n) st(dst, i, ld(src, i));
  }
}

// fl::SGDOptimizer::step (flashlight/fl/optim/SGDOptimizer.cpp:38-68) over several parameter tensors in one launch, in
// place: g = grad + wd w; with momentum v = mu v + g and g = nesterov ? g + mu v : v; w = w - lr g.  The same packing of
// (tensor, piece) into the grid as convert_many_kernel.
constexpr int SGD_MAX = 48;
struct SgdMany {
  void* w[SGD_MAX];
  const void* g[SGD_MAX];
  void* v[SGD_MAX];
  unsigned first[SGD_MAX + 1];
  unsigned long long n[SGD_MAX];
  int count;
  float lr, mu, wd;
  int nesterov;
};
template <typename T>
__global__ void __launch_bounds__(256) sgd_many_kernel(SgdMany a) {
  int lo = 0, hi = a.count;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.first[mid] <= blockIdx.x) lo = mid; else hi = mid;
  }
  T* w = static_cast<T*>(a.w[lo]);
  const T* g = static_cast<const T*>(a.g[lo]);
  T* v = static_cast<T*>(a.v[lo]);
  const size_t base = (size_t)(blockIdx.x - a.first[lo]) * 2048;
  const size_t n = a.n[lo];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const size_t i = base + (size_t)k * 256 + threadIdx.x;
    if (i < n) {
      const float wi = ld(w, i);
      float gi = ld(g, i);
      if (a.wd != 0.f) gi = gi + a.wd * wi;
      if (a.mu != 0.f) {
        const float vi = a.mu * ld(v, i) + gi;
        st(v, i, vi);
        // the velocity as it is stored (rounded for 16-bit parameters), like the reference's evaluated tensor
        const float vs = ld(v, i);
        gi = a.nesterov ? gi + vs * a.mu : vs;
      }
      st(w, i, wi - a.lr * gi);
    }
  }
}

// fl::AdamOptimizer::step (flashlight/fl/optim/AdamOptimizer.cpp:45-79) the same way: w = w - wd lr w (decoupled decay),
// m = b1 m + (1 - b1) g, v = b2 v + (1 - b2) g g (both stored), w = w - clr m / (sqrt(v) + eps) with the
// bias-corrected rate clr = lr sqrt(1 - b2^t) / (1 - b1^t) computed on the host.
constexpr int ADAM_MAX = 32;
struct AdamMany {
  void* w[ADAM_MAX];
  const void* g[ADAM_MAX];
  void* m[ADAM_MAX];
  void* v[ADAM_MAX];
  unsigned first[ADAM_MAX + 1];
  unsigned long long n[ADAM_MAX];
  int count;
  float b1, b2, eps, decay, clr;      // decay = wd * lr
};
template <typename T>
__global__ void __launch_bounds__(256) adam_many_kernel(AdamMany a) {
  int lo = 0, hi = a.count;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.first[mid] <= blockIdx.x) lo = mid; else hi = mid;
  }
  T* w = static_cast<T*>(a.w[lo]);
  const T* g = static_cast<const T*>(a.g[lo]);
  T* m = static_cast<T*>(a.m[lo]);
  T* v = static_cast<T*>(a.v[lo]);
  const size_t base = (size_t)(blockIdx.x - a.first[lo]) * 2048;
  const size_t n = a.n[lo];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const size_t i = base + (size_t)k * 256 + threadIdx.x;
    if (i < n) {
      float wi = ld(w, i);
      const float gi = ld(g, i);
      if (a.decay != 0.f) wi = wi - a.decay * wi;
      st(m, i, a.b1 * ld(m, i) + (1.f - a.b1) * gi);
      st(v, i, a.b2 * ld(v, i) + (1.f - a.b2) * gi * gi);
      st(w, i, wi - (a.clr * ld(m, i)) / (sqrtf(ld(v, i)) + a.eps));
    }
  }
}

template <typename D>
__global__ void __launch_bounds__(256) fill_kernel(D* __restrict__ dst, float value, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) st(dst, i, value);
}

struct OpAdd {
  __device__ float operator()(float a, float b) const { return a + b; }
};

}  // namespace flhip

using namespace flhip;

// most pieces (workgroups) of one convert_many launch: the grid limit
static uint64_t convert_many_max_pieces() { return 0x7fffffffull; }

extern "C" const char* flhip_last_error(void) { return g_last_error.c_str(); }
extern "C" int flhip_version(void) { return FLHIP_VERSION; }
extern "C" const char* flhip_arch(void) { return "gfx950"; }

extern "C" int flhip_set_option(const char* name, const char* value) {
  FLHIP_REQUIRE(name, "set_option: null name");
  options();   // the environment is read first, so a later first use cannot undo this call
  if (!strncmp(name, "FLHIP_", 6)) name += 6;
  if (!apply_option(g_options, name, value))
    return fail(FLHIP_INVALID_ARGUMENT, std::string("set_option: unknown switch or value: ") + name + "=" +
                                            (value ? value : "(null)"));
  return FLHIP_OK;
}

extern "C" int flhip_conv2d_out_dims(const flhip_conv_desc* d, int32_t* OH, int32_t* OW) {
  FLHIP_REQUIRE(d && OH && OW, "conv2d_out_dims: null argument");
  FLHIP_REQUIRE(d->N > 0 && d->C > 0 && d->H > 0 && d->W > 0 && d->K > 0 &&
                    d->KH > 0 && d->KW > 0,
                "conv2d: sizes must be positive");
  FLHIP_REQUIRE(d->sy > 0 && d->sx > 0 && d->dil_y > 0 && d->dil_x > 0,
                "conv2d: stride and dilation must be positive");
  FLHIP_REQUIRE(d->py >= 0 && d->px >= 0, "conv2d: padding must be non-negative");
  FLHIP_REQUIRE(d->groups > 0 && d->C % d->groups == 0 && d->K % d->groups == 0,
                "conv2d: groups must divide input and output channels");
  FLHIP_REQUIRE(dtype_ok(d->dtype), "conv2d: unknown dtype");
  const int eh = 1 + (d->KH - 1) * d->dil_y, ew = 1 + (d->KW - 1) * d->dil_x;
  FLHIP_REQUIRE(d->H + 2 * d->py >= eh && d->W + 2 * d->px >= ew,
                "conv2d: kernel larger than padded input");
  *OH = 1 + (d->H + 2 * d->py - eh) / d->sy;
  *OW = 1 + (d->W + 2 * d->px - ew) / d->sx;
  return FLHIP_OK;
}

extern "C" int flhip_pool2d_out_dims(const flhip_pool_desc* d, int32_t* OH, int32_t* OW) {
  FLHIP_REQUIRE(d && OH && OW, "pool2d_out_dims: null argument");
  FLHIP_REQUIRE(d->N > 0 && d->C > 0 && d->H > 0 && d->W > 0 && d->wy > 0 && d->wx > 0,
                "pool2d: sizes must be positive");
  FLHIP_REQUIRE(d->sy > 0 && d->sx > 0, "pool2d: stride must be positive");
  FLHIP_REQUIRE(d->py >= 0 && d->px >= 0 && d->py < d->wy && d->px < d->wx,
                "pool2d: padding must be non-negative and smaller than the window");
  FLHIP_REQUIRE(d->mode >= FLHIP_POOL_MAX && d->mode <= FLHIP_POOL_AVG_EXCLUDE_PADDING,
                "pool2d: unknown pooling mode");
  FLHIP_REQUIRE(dtype_ok(d->dtype), "pool2d: unknown dtype");
  FLHIP_REQUIRE(d->H + 2 * d->py >= d->wy && d->W + 2 * d->px >= d->wx,
                "pool2d: window larger than padded input");
  *OH = 1 + (d->H + 2 * d->py - d->wy) / d->sy;
  *OW = 1 + (d->W + 2 * d->px - d->wx) / d->sx;
  return FLHIP_OK;
}

extern "C" int flhip_copy_bytes(const void* src, void* dst, size_t bytes, void* stream) {
  FLHIP_REQUIRE(src && dst, "copy_bytes: null pointer");
  FLHIP_REQUIRE(bytes % 16 == 0, "copy_bytes: size must be a multiple of 16");
  if (bytes == 0) return FLHIP_OK;
  const size_t n16 = bytes / 16;
  size_t blocks = (n16 + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                     reinterpret_cast<const uint4*>(src), reinterpret_cast<uint4*>(dst), n16);
  return check_launch("copy_bytes");
}

extern "C" int flhip_convert(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n,
                             void* stream) {
  FLHIP_REQUIRE(dtype_ok(src_dtype) && dtype_ok(dst_dtype), "convert: unknown dtype");
  if (n == 0) return FLHIP_OK;
  FLHIP_REQUIRE(src && dst, "convert: null pointer");
  size_t blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  const dim3 grid((unsigned)blocks), block(256);
  hipStream_t s = as_stream(stream);
  by_dtype(src_dtype, [&](auto* sp) {
    by_dtype(dst_dtype, [&](auto* dp) {
      using S = FLHIP_T_OF(sp);
      using D = FLHIP_T_OF(dp);
      hipLaunchKernelGGL((convert_kernel<S, D>), grid, block, 0, s, static_cast<const S*>(src), static_cast<D*>(dst), n);
    });
  });
  return check_launch("convert");
}

extern "C" int flhip_convert_many(const void* const* src, void* const* dst, const size_t* n, int count,
                                  int src_dtype, int dst_dtype, void* stream) {
  FLHIP_REQUIRE(dtype_ok(src_dtype) && dtype_ok(dst_dtype), "convert_many: unknown dtype");
  FLHIP_REQUIRE(count >= 0 && (count == 0 || (src && dst && n)), "convert_many: null argument");
  hipStream_t s = as_stream(stream);
  // A launch holds up to CM_MAX tensors and at most 2^31 - 1 pieces of 2048 elements (the grid limit; one
  // tensor is at most 2^29 pieces): a tensor that would pass either limit starts the next launch.
  ConvertMany a{};
  uint64_t pieces = 0;
  auto flush = [&]() {
    if (a.count == 0) return;
    a.first[a.count] = (unsigned)pieces;
    const dim3 grid((unsigned)pieces), block(256);
    by_dtype(src_dtype, [&](auto* sp) {
      by_dtype(dst_dtype, [&](auto* dp) {
        hipLaunchKernelGGL((convert_many_kernel<FLHIP_T_OF(sp), FLHIP_T_OF(dp)>), grid, block, 0, s, a);
      });
    });
    a = ConvertMany{};
    pieces = 0;
  };
  for (int i = 0; i < count; ++i) {
    if (n[i] == 0) continue;
    FLHIP_REQUIRE(src[i] && dst[i], "convert_many: null pointer");
    FLHIP_REQUIRE(n[i] < (1ull << 40), "convert_many: tensor too large");
    const uint64_t mine = (n[i] + 2047) / 2048;
    if (a.count == CM_MAX || pieces + mine > convert_many_max_pieces()) flush();
    a.src[a.count] = src[i];
    a.dst[a.count] = dst[i];
    a.n[a.count] = n[i];
    a.first[a.count] = (unsigned)pieces;
    pieces += mine;
    ++a.count;
  }
  flush();
  return check_launch("convert_many");
}

extern "C" int flhip_sgd_many(void* const* params, const void* const* grads, void* const* velocities, const size_t* n,
                              int count, double lr, double momentum, double weight_decay, int nesterov, int dtype,
                              void* stream) {
  FLHIP_REQUIRE(dtype_ok(dtype), "sgd_many: unknown dtype");
  FLHIP_REQUIRE(count >= 0 && (count == 0 || (params && grads && n)), "sgd_many: null argument");
  FLHIP_REQUIRE(momentum == 0.0 || velocities, "sgd_many: momentum needs velocity buffers");
  hipStream_t s = as_stream(stream);
  SgdMany a{};
  uint64_t pieces = 0;
  auto flush = [&]() {
    if (a.count == 0) return;
    a.first[a.count] = (unsigned)pieces;
    a.lr = (float)lr; a.mu = (float)momentum; a.wd = (float)weight_decay; a.nesterov = nesterov != 0;
    const dim3 grid((unsigned)pieces), block(256);
    by_dtype(dtype, [&](auto* t_) { hipLaunchKernelGGL((sgd_many_kernel<FLHIP_T_OF(t_)>), grid, block, 0, s, a); });
    a = SgdMany{};
    pieces = 0;
  };
  for (int i = 0; i < count; ++i) {
    if (n[i] == 0) continue;
    FLHIP_REQUIRE(params[i] && grads[i] && (momentum == 0.0 || velocities[i]), "sgd_many: null pointer");
    FLHIP_REQUIRE(n[i] < (1ull << 40), "sgd_many: tensor too large");
    const uint64_t mine = (n[i] + 2047) / 2048;
    if (a.count == SGD_MAX || pieces + mine > convert_many_max_pieces()) flush();
    a.w[a.count] = params[i];
    a.g[a.count] = grads[i];
    a.v[a.count] = momentum != 0.0 ? velocities[i] : nullptr;
    a.n[a.count] = n[i];
    a.first[a.count] = (unsigned)pieces;
    pieces += mine;
    ++a.count;
  }
  flush();
  return check_launch("sgd_many");
}

extern "C" int flhip_adam_many(void* const* params, const void* const* grads, void* const* first, void* const* second,
                               const size_t* n, int count, double lr, double beta1, double beta2, double epsilon,
                               double weight_decay, int64_t step, int dtype, void* stream) {
  FLHIP_REQUIRE(dtype_ok(dtype), "adam_many: unknown dtype");
  FLHIP_REQUIRE(count >= 0 && (count == 0 || (params && grads && first && second && n)), "adam_many: null argument");
  FLHIP_REQUIRE(step >= 1, "adam_many: steps count from 1");
  hipStream_t s = as_stream(stream);
  // AdamOptimizer.cpp:47-49, in float like the reference
  const float cb1 = 1.f - std::pow((float)beta1, (float)step), cb2 = 1.f - std::pow((float)beta2, (float)step);
  const float clr = (float)lr * std::sqrt(cb2) / cb1;
  AdamMany a{};
  uint64_t pieces = 0;
  auto flush = [&]() {
    if (a.count == 0) return;
    a.first[a.count] = (unsigned)pieces;
    a.b1 = (float)beta1; a.b2 = (float)beta2; a.eps = (float)epsilon; a.decay = (float)(weight_decay * lr); a.clr = clr;
    const dim3 grid((unsigned)pieces), block(256);
    by_dtype(dtype, [&](auto* t_) { hipLaunchKernelGGL((adam_many_kernel<FLHIP_T_OF(t_)>), grid, block, 0, s, a); });
    a = AdamMany{};
    pieces = 0;
  };
  for (int i = 0; i < count; ++i) {
    if (n[i] == 0) continue;
    FLHIP_REQUIRE(params[i] && grads[i] && first[i] && second[i], "adam_many: null pointer");
    FLHIP_REQUIRE(n[i] < (1ull << 40), "adam_many: tensor too large");
    const uint64_t mine = (n[i] + 2047) / 2048;
    if (a.count == ADAM_MAX || pieces + mine > convert_many_max_pieces()) flush();
    a.w[a.count] = params[i];
    a.g[a.count] = grads[i];
    a.m[a.count] = first[i];
    a.v[a.count] = second[i];
    a.n[a.count] = n[i];
    a.first[a.count] = (unsigned)pieces;
    pieces += mine;
    ++a.count;
  }
  flush();
  return check_launch("adam_many");
}

extern "C" int flhip_convert_many_launches(const size_t* n, int count, int* launch_of) {
  if (count < 0 || (count > 0 && !n)) return -1;
  int launches = 0, held = 0;
  uint64_t pieces = 0;
  for (int i = 0; i < count; ++i) {
    if (launch_of) launch_of[i] = -1;
    if (n[i] == 0) continue;
    if (n[i] >= (1ull << 40)) return -1;
    const uint64_t mine = (n[i] + 2047) / 2048;
    if (held == CM_MAX || pieces + mine > convert_many_max_pieces()) {
      launches += held > 0;
      held = 0;
      pieces = 0;
    }
    if (launch_of) launch_of[i] = launches;
    pieces += mine;
    ++held;
  }
  return launches + (held > 0);
}

extern "C" int flhip_fill(void* dst, double value, size_t n, int dtype, void* stream) {
  FLHIP_REQUIRE(dtype_ok(dtype), "fill: unknown dtype");
  if (n == 0) return FLHIP_OK;
  FLHIP_REQUIRE(dst, "fill: null pointer");
  size_t blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  by_dtype(dtype, [&](auto* t) {
    using T = FLHIP_T_OF(t);
    hipLaunchKernelGGL((fill_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), static_cast<T*>(dst),
                       (float)value, n);
  });
  return check_launch("fill");
}

extern "C" int flhip_add(const void* a, const void* b, void* out, size_t n, int dtype,
                         void* stream) {
  FLHIP_REQUIRE(dtype_ok(dtype), "add: unknown dtype");
  if (n == 0) return FLHIP_OK;
  FLHIP_REQUIRE(a && b && out, "add: null pointer");
  by_dtype(dtype, [&](auto* t) {
    using T = FLHIP_T_OF(t);
    launch_elementwise(static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(out), n, OpAdd{}, as_stream(stream));
  });
  return check_launch("add");
}
