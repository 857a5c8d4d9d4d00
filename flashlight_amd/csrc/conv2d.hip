// conv2d / conv2dBackwardData / conv2dBackwardFilterBias entry points, and the
// direct (one thread per result) kernels that cover every geometry.  The MFMA
// implicit-GEMM kernels in conv2d_mfma.hip are used whenever they accept the
// shape; the switch CONV_ALGO=direct forces the kernels here.
#include <mutex>

#include "conv2d.h"

// Scratch of flhip_conv2d_bwd_filter_static: lives in the code object, one copy per
// device the library is loaded on, never freed.  The name is only a host-side handle;
// the per-device address comes from hipGetSymbolAddress (static_scratch()).
static __device__ __align__(256) unsigned char scratch[FLHIP_STATIC_SCRATCH_BYTES];

namespace flhip {

template <typename T>
__global__ void __launch_bounds__(256)
conv_fwd_direct(ConvGeom g, const T* __restrict__ x, const T* __restrict__ w,
                const float* __restrict__ bias, T* __restrict__ y, size_t total) {
  const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= total) return;
  const int ow = (int)(o % g.OW);
  size_t t = o / g.OW;
  const int oh = (int)(t % g.OH);
  t /= g.OH;
  const int k = (int)(t % g.K);
  const int n = (int)(t / g.K);
  const int grp = k / g.Kg;
  float acc = bias ? bias[k] : 0.f;
  for (int c = 0; c < g.Cg; ++c) {
    const T* xp = x + ((size_t)n * g.C + grp * g.Cg + c) * g.H * g.W;
    const T* wp = w + ((size_t)k * g.Cg + c) * g.KH * g.KW;
    for (int kh = 0; kh < g.KH; ++kh) {
      const int ih = oh * g.sy - g.py + kh * g.dly;
      if (ih < 0 || ih >= g.H) continue;
      for (int kw = 0; kw < g.KW; ++kw) {
        const int iw = ow * g.sx - g.px + kw * g.dlx;
        if (iw < 0 || iw >= g.W) continue;
        acc += ld(xp, (size_t)ih * g.W + iw) * ld(wp, kh * g.KW + kw);
      }
    }
  }
  st(y, o, acc);
}

template <typename T>
__global__ void __launch_bounds__(256)
conv_bwd_data_direct(ConvGeom g, const T* __restrict__ dy, const T* __restrict__ w,
                     T* __restrict__ dx, size_t total) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int iw = (int)(e % g.W);
  size_t t = e / g.W;
  const int ih = (int)(t % g.H);
  t /= g.H;
  const int ci = (int)(t % g.C);
  const int n = (int)(t / g.C);
  const int grp = ci / g.Cg, c = ci % g.Cg;
  float acc = 0.f;
  for (int kk = 0; kk < g.Kg; ++kk) {
    const int k = grp * g.Kg + kk;
    const T* dyp = dy + ((size_t)n * g.K + k) * g.OH * g.OW;
    const T* wp = w + ((size_t)k * g.Cg + c) * g.KH * g.KW;
    for (int kh = 0; kh < g.KH; ++kh) {
      const int th = ih + g.py - kh * g.dly;
      if (th < 0 || th % g.sy != 0) continue;
      const int oh = th / g.sy;
      if (oh >= g.OH) continue;
      for (int kw = 0; kw < g.KW; ++kw) {
        const int tw = iw + g.px - kw * g.dlx;
        if (tw < 0 || tw % g.sx != 0) continue;
        const int ow = tw / g.sx;
        if (ow >= g.OW) continue;
        acc += ld(dyp, (size_t)oh * g.OW + ow) * ld(wp, kh * g.KW + kw);
      }
    }
  }
  st(dx, e, acc);
}

// one block per filter element
template <typename T>
__global__ void __launch_bounds__(256)
conv_bwd_filter_direct(ConvGeom g, const T* __restrict__ x, const T* __restrict__ dy,
                       float* __restrict__ dw) {
  __shared__ float red[8];
  const int e = blockIdx.x;
  const int kw = e % g.KW;
  int t = e / g.KW;
  const int kh = t % g.KH;
  t /= g.KH;
  const int c = t % g.Cg;
  const int k = t / g.Cg;
  const int grp = k / g.Kg;
  const int P = g.OH * g.OW;
  float acc = 0.f;
  for (int n = 0; n < g.N; ++n) {
    const T* xp = x + ((size_t)n * g.C + grp * g.Cg + c) * g.H * g.W;
    const T* dyp = dy + ((size_t)n * g.K + k) * P;
    for (int p = threadIdx.x; p < P; p += 256) {
      const int oh = p / g.OW, ow = p % g.OW;
      const int ih = oh * g.sy - g.py + kh * g.dly, iw = ow * g.sx - g.px + kw * g.dlx;
      if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
        acc += ld(dyp, p) * ld(xp, (size_t)ih * g.W + iw);
    }
  }
  acc = block_sum(acc, red);
  if (threadIdx.x == 0) dw[e] = acc;
}

// db[k] = sum over n and pixels of dy; one block per output channel
template <typename T>
__global__ void __launch_bounds__(256)
conv_bwd_bias_kernel(ConvGeom g, const T* __restrict__ dy, float* __restrict__ db) {
  __shared__ float red[8];
  const int k = blockIdx.x;
  const int P = g.OH * g.OW;
  float acc = 0.f;
  for (int n = 0; n < g.N; ++n) {
    const T* dyp = dy + ((size_t)n * g.K + k) * P;
    for (int p = threadIdx.x; p < P; p += 256) acc += ld(dyp, p);
  }
  acc = block_sum(acc, red);
  if (threadIdx.x == 0) db[k] = acc;
}

// Switch CONV_ALGO: direct = one-thread-per-result kernels, gather = skip the LDS-slab
// kernels, convert = skip the bf16 matrix-core kernels (bf16 storage is then converted on
// load and multiplied in fp32), tapped = prefer the tapped GEMM; otherwise the fastest
// applicable.  CONV_SKIP leaves kernel families out of the dispatch.
static bool algo_is(int a) { return options().conv_algo == a; }
static bool force_direct() { return algo_is(Options::ALGO_DIRECT); }
static bool skip(unsigned family) {
  return algo_is(Options::ALGO_GATHER) || (options().conv_skip & family) != 0;
}
static const unsigned SK_BF16 = Options::SKIP_BF16, SK_GEMM = Options::SKIP_GEMM1X1, SK_SLAB = Options::SKIP_SLAB,
                      SK_TAPPED = Options::SKIP_TAPPED;

// Stride-1 windows over long rows (the 21x1 speech layers: rows of 1500): the gather
// kernel's one-position-per-thread loads are whole contiguous runs there and it
// measures faster than the tapped GEMM, except for backward-data into few channels.
// With its weights reordered (workspace present) the tapped GEMM wins from 128 contraction
// channels on.
// the one-row-window kernels take this storage type (bf16: unless the bf16 families are switched off or converted)
static bool tap1d_on(int dtype) {
  if (force_direct() || skip(Options::SKIP_TAP1D)) return false;
  return dtype == FLHIP_F32 || ((dtype == FLHIP_BF16 || dtype == FLHIP_F16) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT));
}

// 3x3 windows over stacked planes: bf16, planes of at most 64 positions (the 7 x 7 layers) and a sequence of at least
// 2048 positions.  Measured (batch 64 / 32, forward): 7 x 7 x 512 41.9 / 40.3 us against 62.3 / 54.8 on the slab
// kernel; 14 x 14 x 256 42.2 / 33.0 against 34.6 / 31.0 and 28 x 28 x 128 41.3 / 32.5 against 25.5 / 19.7, so larger planes
// stay where they were; fp32 loses at every size (14 x 14 x 256: 221 against 140 us).  TAP2D_ALL lifts the rule.
static bool tap2d_on(const ConvGeom& g, int dtype) {
  if (!tap1d_on(dtype) || skip(Options::SKIP_TAP2D)) return false;
  if (options().tap2d_all) return true;
  return (dtype == FLHIP_BF16 || dtype == FLHIP_F16) && g.H * g.W <= 64 && (long long)g.N * (g.H + 1) * (g.W + 1) >= 2048;
}

static bool long_rows(const ConvGeom& g, int dtype, bool bwd, size_t ws_bytes) {
  if (algo_is(Options::ALGO_TAPPED)) return false;
  const size_t need = mfma_tapped_ws(g, dtype, bwd);
  if (need && ws_bytes >= need && (bwd ? g.K : g.C) >= 128) return false;
  return g.sy == 1 && g.sx == 1 && g.OW >= 64 && (!bwd || g.C >= 128);
}

static int make_geom(const flhip_conv_desc* d, ConvGeom* g) {
  int32_t OH, OW;
  const int rc = flhip_conv2d_out_dims(d, &OH, &OW);
  if (rc != FLHIP_OK) return rc;
  *g = ConvGeom{d->N, d->C, d->H, d->W, d->K, d->KH, d->KW, OH, OW,
                d->sy, d->sx, d->py, d->px, d->dil_y, d->dil_x, d->groups,
                d->C / d->groups, d->K / d->groups};
  FLHIP_REQUIRE((size_t)d->N * d->C * d->H * d->W < (1ull << 31) &&
                    (size_t)d->N * d->K * OH * OW < (1ull << 31),
                "conv2d: tensors of 2^31 elements or more are not supported");
  return FLHIP_OK;
}

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** out) {
  enum { MAX_DEVICES = 64 };
  static std::mutex mu;
  static void* addr[MAX_DEVICES] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(FLHIP_RUNTIME_ERROR, std::string("hipGetDevice: ") + hipGetErrorString(e));
  if (dev < 0 || dev >= MAX_DEVICES) return fail(FLHIP_RUNTIME_ERROR, "static scratch: device index out of range");
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(FLHIP_RUNTIME_ERROR, std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
    addr[dev] = p;
  }
  *out = addr[dev];
  return FLHIP_OK;
}

}  // namespace flhip

using namespace flhip;

extern "C" size_t flhip_conv2d_workspace_bytes(const flhip_conv_desc* d, int pass) {
  ConvGeom g;
  if (make_geom(d, &g) != FLHIP_OK) return 0;
  if (pass == FLHIP_CONV_BWD_FILTER) {
    // the larger of the two filter-gradient plans, so either kernel can run
    size_t a = mfma_conv_bwd_filter_ws(g, d->dtype);
    const size_t b = mfma_slab_wgrad_ws(g, d->dtype);
    size_t c = is_lo16(d->dtype) ? mfma_wgrad16_ws(g) : 0;
    const size_t c2 = is_lo16(d->dtype) ? mfma_wgrad_dma16_ws(g) : 0;
    if (c2 > c) c = c2;
    const size_t e = mfma_pointwise_wgrad_ws(g);
    const size_t f = is_lo16(d->dtype) ? mfma_pointwise16_wgrad_ws(g) : 0;
    const size_t h = is_lo16(d->dtype) ? mfma_first16_wgrad_ws(g) : 0;
    const size_t t1 = mfma_tap1d_wgrad_ws(g, d->dtype);
    if (h > a) a = h;
    if (t1 > a) a = t1;
    if (b > a) a = b;
    if (e > a) a = e;
    if (f > a) a = f;
    return c > a ? c : a;
  }
  // forward / backward-data: the kernels for windows with several taps read reordered
  // weights when the caller brings room for them (they run without it, slower)
  // (bf16: strided 1x1 windows gather the input's lattice points / spread a compact gradient)
  if (pass == FLHIP_CONV_FWD || pass == FLHIP_CONV_BWD_DATA) {
    const size_t a = mfma_tapped_ws(g, d->dtype, pass == FLHIP_CONV_BWD_DATA);
    const size_t b = is_lo16(d->dtype) ? mfma_pointwise16_lattice_ws(g, pass == FLHIP_CONV_BWD_DATA)
                                            : pass == FLHIP_CONV_BWD_DATA ? mfma_pointwise_split_ws(g, d->dtype, true) : 0;
    const size_t c = mfma_tap1d_conv_ws(g, d->dtype, pass == FLHIP_CONV_BWD_DATA);
    // (the stacked-plane kernels: where their rule takes the geometry, and for every plane of at most 32 x 32 positions so
    // that a caller can try them by plan number; beyond that their copy of the input is tens of megabytes nobody asked for)
    const size_t c2 = (tap2d_on(g, d->dtype) || g.H * g.W <= 1024) ? mfma_tap2d_conv_ws(g, d->dtype, pass == FLHIP_CONV_BWD_DATA) : 0;
    return std::max(std::max(a, c2), std::max(b, c));
  }
  return 0;
}

extern "C" int flhip_conv2d_fwd(const flhip_conv_desc* d, const void* x, const void* w,
                                const float* bias, void* y, void* ws, size_t ws_bytes,
                                void* stream) {
  FLHIP_REQUIRE(d && x && w && y, "conv2d_fwd: null argument");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (!force_direct()) {
    int r = -1;
    if (tap1d_on(d->dtype)) r = mfma_tap1d_conv_fwd(g, d->dtype, x, w, bias, y, s, ws, ws_bytes);
    if (r < 0 && tap2d_on(g, d->dtype)) r = mfma_tap2d_conv_fwd(g, d->dtype, x, w, bias, y, s, ws, ws_bytes);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_PWDMA) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_pwd16_conv_fwd(g, x, w, bias, y, s, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_pointwise16_conv_fwd(g, x, w, bias, y, s, ws, ws_bytes, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_FIRST) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_first16_conv_fwd(g, x, w, bias, y, s, d->dtype);
    if (r < 0 && !skip(Options::SKIP_CELLS)) r = mfma_cells_conv_fwd(g, d->dtype, x, w, bias, y, s);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_STRIP) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_strip16_conv_fwd(g, x, w, bias, y, s, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_slab16_conv_fwd(g, x, w, bias, y, s, d->dtype);
    if (r < 0 && !skip(SK_GEMM)) r = mfma_pointwise_conv_fwd(g, d->dtype, x, w, bias, y, s);
    if (r < 0 && algo_is(Options::ALGO_TAPPED)) r = mfma_tapped_conv_fwd(g, d->dtype, x, w, bias, y, s, ws, ws_bytes);
    if (r < 0 && !skip(SK_SLAB)) r = mfma_slab_conv_fwd(g, d->dtype, x, w, bias, y, s);
    if (r < 0 && !skip(SK_TAPPED) && !long_rows(g, d->dtype, false, ws ? ws_bytes : 0))
      r = mfma_tapped_conv_fwd(g, d->dtype, x, w, bias, y, s, ws, ws_bytes);
    if (r < 0) r = mfma_conv_fwd(g, d->dtype, x, w, bias, y, s);
    if (r >= 0) return r;
  }
  const size_t total = (size_t)g.N * g.K * g.OH * g.OW;
  const dim3 grid((unsigned)((total + 255) / 256));
  by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((conv_fwd_direct<T>), grid, dim3(256), 0, s, g,
                       static_cast<const T*>(x), static_cast<const T*>(w), bias,
                       static_cast<T*>(y), total);
  });
  return check_launch("conv2d_fwd");
}

// The kernel families of the two backward passes, in the order of the default rule (the first that takes a geometry
// runs it; each declines what it does not handle or, by measured rules, handles badly).  A plan number forces one
// family: the caller times them instead of trusting the rules.
static const char* const kBwdDataPlans[] = {"bf16 1x1, tiles loaded straight to LDS", "bf16 1x1 / gathered taps", "bf16 3x3 strip",
                                            "bf16 slab", "1x1 GEMM, split contraction", "1x1 GEMM", "slab", "tapped GEMM",
                                            "gather", "direct", "one-row windows", "stride-2 window over few channels, 2 x 2 cells",
                                            "3x3 windows over stacked planes"};
static const char* const kBwdFilterPlans[] = {"bf16 3x3 rows straight to LDS, 32 x 32 tiles", "bf16 3x3 rows straight to LDS, 64 x 64 tiles",
                                              "bf16 1x1 / gathered taps", "bf16 first layer", "bf16 3x3 rows", "1x1 GEMM", "row slab",
                                              "tapped GEMM", "gather", "direct", "one-row windows"};
constexpr int kNumDataPlans = 13, kNumFilterPlans = 11;

static int bwd_data_direct(const flhip_conv_desc* d, const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s) {
  const size_t total = (size_t)g.N * g.C * g.H * g.W;
  const dim3 grid((unsigned)((total + 255) / 256));
  by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((conv_bwd_data_direct<T>), grid, dim3(256), 0, s, g,
                       static_cast<const T*>(dy), static_cast<const T*>(w),
                       static_cast<T*>(dx), total);
  });
  return check_launch("conv2d_bwd_data");
}

// plan < 0: the default rule; otherwise that family alone (FLHIP_DECLINED when it does not take the geometry)
static int bwd_data_impl(const flhip_conv_desc* d, const void* dy, const void* w, void* dx, void* ws, size_t ws_bytes,
                         int plan, void* stream) {
  FLHIP_REQUIRE(d && dy && w && dx, "conv2d_bwd_data: null argument");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (plan >= 0) {
    FLHIP_REQUIRE(plan < kNumDataPlans, "conv2d_bwd_data: unknown plan");
    const bool lo = is_lo16(d->dtype);
    int r = -1;
    switch (plan) {
      case 0: if (lo) r = mfma_pwd16_conv_bwd_data(g, dy, w, nullptr, dx, s, d->dtype); break;
      case 1: if (lo) r = mfma_pointwise16_conv_bwd_data(g, dy, w, dx, s, ws, ws_bytes, d->dtype); break;
      case 2: if (lo) r = mfma_strip16_conv_bwd_data(g, dy, w, dx, s, d->dtype); break;
      case 3: if (lo) r = mfma_slab16_conv_bwd_data(g, dy, w, dx, s, d->dtype); break;
      case 4: r = mfma_pointwise_conv_split(g, d->dtype, true, dy, w, nullptr, dx, ws, ws_bytes, s); break;
      case 5: r = mfma_pointwise_conv_bwd_data(g, d->dtype, dy, w, dx, s); break;
      case 6: r = mfma_slab_conv_bwd_data(g, d->dtype, dy, w, dx, s); break;
      case 7: r = mfma_tapped_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes); break;
      case 8: r = mfma_conv_bwd_data(g, d->dtype, dy, w, dx, s); break;
      case 9: r = bwd_data_direct(d, g, dy, w, dx, s); break;
      case 10: r = mfma_tap1d_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes); break;
      case 11: r = mfma_cells_conv_bwd_data(g, d->dtype, dy, w, dx, s); break;
      default: r = mfma_tap2d_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes);
    }
    return r < 0 ? FLHIP_DECLINED : r;
  }
  if (!force_direct()) {
    int r = -1;
    if (tap1d_on(d->dtype)) r = mfma_tap1d_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes);
    if (r < 0 && tap2d_on(g, d->dtype)) r = mfma_tap2d_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes);
    if (r < 0 && !skip(Options::SKIP_CELLS)) r = mfma_cells_conv_bwd_data(g, d->dtype, dy, w, dx, s);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_PWDMA) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_pwd16_conv_bwd_data(g, dy, w, nullptr, dx, s, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_pointwise16_conv_bwd_data(g, dy, w, dx, s, ws, ws_bytes, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_STRIP) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_strip16_conv_bwd_data(g, dy, w, dx, s, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_slab16_conv_bwd_data(g, dy, w, dx, s, d->dtype);
    if (r < 0 && !skip(SK_GEMM)) r = mfma_pointwise_conv_split(g, d->dtype, true, dy, w, nullptr, dx, ws, ws_bytes, s);
    if (r < 0 && !skip(SK_GEMM)) r = mfma_pointwise_conv_bwd_data(g, d->dtype, dy, w, dx, s);
    if (r < 0 && algo_is(Options::ALGO_TAPPED)) r = mfma_tapped_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes);
    if (r < 0 && !skip(SK_SLAB)) r = mfma_slab_conv_bwd_data(g, d->dtype, dy, w, dx, s);
    if (r < 0 && !skip(SK_TAPPED) && !long_rows(g, d->dtype, true, ws ? ws_bytes : 0))
      r = mfma_tapped_conv_bwd_data(g, d->dtype, dy, w, dx, s, ws, ws_bytes);
    if (r < 0) r = mfma_conv_bwd_data(g, d->dtype, dy, w, dx, s);
    if (r >= 0) return r;
  }
  return bwd_data_direct(d, g, dy, w, dx, s);
}

extern "C" int flhip_conv2d_bwd_data(const flhip_conv_desc* d, const void* dy, const void* w,
                                     void* dx, void* ws, size_t ws_bytes, void* stream) {
  return bwd_data_impl(d, dy, w, dx, ws, ws_bytes, -1, stream);
}

extern "C" int flhip_conv2d_bwd_data_plan(const flhip_conv_desc* d, const void* dy, const void* w, void* dx, void* ws,
                                          size_t ws_bytes, int plan, void* stream) {
  return bwd_data_impl(d, dy, w, dx, ws, ws_bytes, plan, stream);
}

extern "C" int flhip_conv2d_plan_count(int pass) {
  return pass == FLHIP_CONV_BWD_DATA ? kNumDataPlans : pass == FLHIP_CONV_BWD_FILTER ? kNumFilterPlans : 0;
}

extern "C" const char* flhip_conv2d_plan_name(int pass, int plan) {
  if (plan < 0) return nullptr;
  if (pass == FLHIP_CONV_BWD_DATA) return plan < kNumDataPlans ? kBwdDataPlans[plan] : nullptr;
  if (pass == FLHIP_CONV_BWD_FILTER) return plan < kNumFilterPlans ? kBwdFilterPlans[plan] : nullptr;
  return nullptr;
}

extern "C" int flhip_conv2d_bwd_data_add(const flhip_conv_desc* d, const void* dy, const void* w,
                                         const void* addend, void* dx, void* ws, size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(d && dy && w && dx && addend, "conv2d_bwd_data_add: null argument");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  hipStream_t s = as_stream(stream);
  // no kernel may see dx and addend as one buffer: the fused ones read a plane's last 16-byte cell of addend again
  // after another workgroup may have written it (planes that are not a multiple of 8 positions), the others
  // write dx before they read addend
  FLHIP_REQUIRE(dx != addend, "conv2d_bwd_data_add: dx aliases addend");
  if (!force_direct() && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT)) {
    int r = skip(Options::SKIP_PWDMA) ? -1 : mfma_pwd16_conv_bwd_data(g, dy, w, addend, dx, s, d->dtype);
    if (r < 0) r = mfma_pointwise16_conv_bwd_data_add(g, dy, w, addend, dx, s, d->dtype);
    if (r >= 0) return r;
  }
  // every other kernel: the plain pass, then the element-wise sum
  const int r = flhip_conv2d_bwd_data(d, dy, w, dx, ws, ws_bytes, stream);
  if (r != FLHIP_OK) return r;
  return flhip_add(dx, addend, dx, (size_t)g.N * g.C * g.H * g.W, d->dtype, stream);
}

static int bwd_filter_direct(const flhip_conv_desc* d, const ConvGeom& g, const void* x, const void* dy, float* dw, float* db,
                             hipStream_t s) {
  if (dw) {
    const dim3 grid((unsigned)(g.K * g.Cg * g.KH * g.KW));
    by_dtype(d->dtype, [&](auto* t_) {
      using T = FLHIP_T_OF(t_);
      hipLaunchKernelGGL((conv_bwd_filter_direct<T>), grid, dim3(256), 0, s, g,
                         static_cast<const T*>(x), static_cast<const T*>(dy), dw);
    });
  }
  if (db) {
    by_dtype(d->dtype, [&](auto* t_) {
      using T = FLHIP_T_OF(t_);
      hipLaunchKernelGGL((conv_bwd_bias_kernel<T>), dim3(g.K), dim3(256), 0, s, g,
                         static_cast<const T*>(dy), db);
    });
  }
  return check_launch("conv2d_bwd_filter");
}

static int bwd_filter_impl(const flhip_conv_desc* d, const void* x, const void* dy, float* dw, float* db, void* ws,
                           size_t ws_bytes, int plan, void* stream) {
  FLHIP_REQUIRE(d && dy, "conv2d_bwd_filter: null argument");
  FLHIP_REQUIRE(dw || db, "conv2d_bwd_filter: nothing to compute");
  FLHIP_REQUIRE(!dw || x, "conv2d_bwd_filter: filter gradient needs the input");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (plan >= 0) {
    FLHIP_REQUIRE(plan < kNumFilterPlans, "conv2d_bwd_filter: unknown plan");
    if (plan == 9) return bwd_filter_direct(d, g, x, dy, dw, db, s);
    const size_t need = flhip_conv2d_workspace_bytes(d, FLHIP_CONV_BWD_FILTER);
    FLHIP_REQUIRE(ws_bytes >= need && (ws || need == 0), "conv2d_bwd_filter: workspace too small");
    const bool lo = is_lo16(d->dtype);
    int r = -1;
    switch (plan) {
      case 0: if (lo) r = mfma_wgrad_dma16(g, x, dy, dw, db, ws, ws_bytes, s, 32, d->dtype); break;
      case 1: if (lo) r = mfma_wgrad_dma16(g, x, dy, dw, db, ws, ws_bytes, s, 64, d->dtype); break;
      case 2: if (lo) r = mfma_pointwise16_wgrad(g, x, dy, dw, db, ws, ws_bytes, s, nullptr, d->dtype); break;
      case 3: if (lo) r = mfma_first16_wgrad(g, x, dy, dw, db, ws, ws_bytes, s, d->dtype); break;
      case 4: if (lo) r = mfma_wgrad16(g, x, dy, dw, db, ws, ws_bytes, s, d->dtype); break;
      case 5: r = mfma_pointwise_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, false, s); break;
      case 6: r = mfma_slab_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s); break;
      case 7: r = mfma_pointwise_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, true, s); break;
      case 8: r = mfma_conv_bwd_filter(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s); break;
      default: if (dw) r = mfma_tap1d_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s);
    }
    return r < 0 ? FLHIP_DECLINED : r;
  }
  if (!force_direct()) {
    const size_t need = flhip_conv2d_workspace_bytes(d, FLHIP_CONV_BWD_FILTER);
    FLHIP_REQUIRE(ws_bytes >= need && (ws || need == 0), "conv2d_bwd_filter: workspace too small");
    int r = -1;
    // (3x3 stride 1 with rows copied straight to LDS first: it also takes the 7x7 planes that would otherwise go
    // through gathered taps below)
    if (dw && tap1d_on(d->dtype)) r = mfma_tap1d_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_PWDMA) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_wgrad_dma16(g, x, dy, dw, db, ws, ws_bytes, s, 0, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_pointwise16_wgrad(g, x, dy, dw, db, ws, ws_bytes, s, nullptr, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !skip(Options::SKIP_FIRST) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_first16_wgrad(g, x, dy, dw, db, ws, ws_bytes, s, d->dtype);
    if (r < 0 && is_lo16(d->dtype) && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT))
      r = mfma_wgrad16(g, x, dy, dw, db, ws, ws_bytes, s, d->dtype);
    if (r < 0 && !skip(SK_GEMM))
      r = mfma_pointwise_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, algo_is(Options::ALGO_TAPPED), s);
    if (r < 0 && !skip(SK_SLAB)) r = mfma_slab_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s);
    if (r < 0 && !skip(SK_TAPPED)) r = mfma_pointwise_wgrad(g, d->dtype, x, dy, dw, db, ws, ws_bytes, true, s);
    if (r < 0) r = mfma_conv_bwd_filter(g, d->dtype, x, dy, dw, db, ws, ws_bytes, s);
    if (r >= 0) return r;
  }
  return bwd_filter_direct(d, g, x, dy, dw, db, s);
}

extern "C" int flhip_conv2d_bwd_filter(const flhip_conv_desc* d, const void* x, const void* dy,
                                       float* dw, float* db, void* ws, size_t ws_bytes,
                                       void* stream) {
  return bwd_filter_impl(d, x, dy, dw, db, ws, ws_bytes, -1, stream);
}

extern "C" int flhip_conv2d_bwd_filter_plan(const flhip_conv_desc* d, const void* x, const void* dy, float* dw, float* db,
                                            void* ws, size_t ws_bytes, int plan, void* stream) {
  return bwd_filter_impl(d, x, dy, dw, db, ws, ws_bytes, plan, stream);
}

// The forward pass of a strided layer in bf16 storage gathers the input points its windows touch into the start of
// its workspace; the filter gradient needs the same copy.  A caller that keeps those bytes passes them here and
// saves the second gather.
static bool gathered_path(const flhip_conv_desc* d) {
  return is_lo16(d->dtype) && !force_direct() && !skip(SK_BF16) && !algo_is(Options::ALGO_CONVERT);
}

extern "C" size_t flhip_conv2d_gathered_bytes(const flhip_conv_desc* d) {
  ConvGeom g;
  if (!d || make_geom(d, &g) != FLHIP_OK) return 0;
  // one-row windows (bf16 and fp32): the forward pass's channels-last rows (that family runs first where it applies)
  if (tap1d_on(d->dtype) && mfma_tap1d_conv_ws(g, d->dtype, false) > 0) return mfma_tap1d_rows_bytes(g, d->dtype);
  return gathered_path(d) ? mfma_pointwise16_gathered_bytes(g) : 0;
}

extern "C" int flhip_conv2d_bwd_filter_gathered(const flhip_conv_desc* d, const void* gathered, const void* dy,
                                                float* dw, float* db, void* ws, size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(d && gathered && dy && dw, "conv2d_bwd_filter_gathered: null argument");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(flhip_conv2d_gathered_bytes(d) > 0,
                "conv2d_bwd_filter_gathered: this geometry's forward pass leaves no gathered input");
  const size_t need = flhip_conv2d_workspace_bytes(d, FLHIP_CONV_BWD_FILTER);
  FLHIP_REQUIRE(ws_bytes >= need && (ws || need == 0), "conv2d_bwd_filter_gathered: workspace too small");
  const bool one_row = tap1d_on(d->dtype) && mfma_tap1d_conv_ws(g, d->dtype, false) > 0;
  const int r = one_row ? mfma_tap1d_wgrad(g, d->dtype, nullptr, dy, dw, db, ws, ws_bytes, as_stream(stream), gathered)
                        : mfma_pointwise16_wgrad(g, nullptr, dy, dw, db, ws, ws_bytes, as_stream(stream), gathered, d->dtype);
  if (r < 0) return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter_gathered: no kernel takes the gathered input of this geometry");
  return r;
}

extern "C" int flhip_conv2d_bwd_filter_static(const flhip_conv_desc* d, const void* x, const void* dy,
                                              float* dw, float* db, void* stream) {
  FLHIP_REQUIRE(d, "conv2d_bwd_filter_static: null argument");
  ConvGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  const size_t need = flhip_conv2d_workspace_bytes(d, FLHIP_CONV_BWD_FILTER);
  if (need > (size_t)FLHIP_STATIC_SCRATCH_BYTES)
    return fail(FLHIP_INVALID_ARGUMENT,
                "conv2d_bwd_filter_static: this geometry needs " + std::to_string(need) +
                    " bytes of scratch, the static buffer holds " +
                    std::to_string((size_t)FLHIP_STATIC_SCRATCH_BYTES) +
                    "; use flhip_conv2d_bwd_filter with a caller workspace");
  void* ptr = nullptr;
  const int rs = static_scratch(&ptr);
  if (rs != FLHIP_OK) return rs;
  // same plan as the workspace entry point given exactly `need` bytes: every partial
  // the reduction reads is written by this call first, so nothing has to be cleared
  return flhip_conv2d_bwd_filter(d, x, dy, dw, db, ptr, need, stream);
}
