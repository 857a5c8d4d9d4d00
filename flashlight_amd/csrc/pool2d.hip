// pool2d / pool2dBackward: max (with first-maximum argmax bytes) and the two
// average modes.  Bandwidth-bound; no atomics: the backward pass is a gather
// over the windows covering each input position, summed in ascending (oh, ow)
// order, which reproduces the reference's scatter order bit for bit.
#include <float.h>

#include "common.h"

namespace flhip {

struct PoolGeom {
  int N, C, H, W, OH, OW;
  int wy, wx, sy, sx, py, px;
};

// ---------------------------------------------------------------------------
// Generic forward: one thread per output element.
// ---------------------------------------------------------------------------
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_fwd_direct(PoolGeom g, const T* __restrict__ x, T* __restrict__ y,
                uint8_t* __restrict__ argmax, size_t total) {
  const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= total) return;
  const int ow = (int)(o % g.OW);
  const size_t t = o / g.OW;
  const int oh = (int)(t % g.OH);
  const size_t plane = t / g.OH;
  const T* xp = x + plane * (size_t)g.H * g.W;
  const int h0 = oh * g.sy - g.py, w0 = ow * g.sx - g.px;
  float best = -FLT_MAX, sum = 0.f;
  int idx = 0, cnt = 0;
  for (int kh = 0; kh < g.wy; ++kh) {
    const int ih = h0 + kh;
    if (ih < 0 || ih >= g.H) continue;
    for (int kw = 0; kw < g.wx; ++kw) {
      const int iw = w0 + kw;
      if (iw < 0 || iw >= g.W) continue;
      const float v = ld(xp, (size_t)ih * g.W + iw);
      if (MODE == FLHIP_POOL_MAX) {
        if (v > best) {
          best = v;
          idx = kh * g.wx + kw;
        }
      } else {
        sum += v;
        ++cnt;
      }
    }
  }
  if (MODE == FLHIP_POOL_MAX) {
    st(y, o, best);
    if (argmax) argmax[o] = (uint8_t)idx;
  } else if (MODE == FLHIP_POOL_AVG_INCLUDE_PADDING) {
    st(y, o, sum / (float)(g.wy * g.wx));
  } else {
    st(y, o, sum / (float)cnt);
  }
}

// ---------------------------------------------------------------------------
// Generic backward: one thread per input element, gathering from the windows
// that cover it.
// ---------------------------------------------------------------------------
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_bwd_direct(PoolGeom g, const T* __restrict__ dy,
                const uint8_t* __restrict__ argmax, T* __restrict__ dx,
                size_t total) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int w = (int)(e % g.W);
  const size_t t = e / g.W;
  const int h = (int)(t % g.H);
  const size_t plane = t / g.H;
  const size_t obase = plane * (size_t)g.OH * g.OW;
  const int th = h + g.py - g.wy + 1, tw = w + g.px - g.wx + 1;
  const int oh_lo = th <= 0 ? 0 : (th + g.sy - 1) / g.sy;
  const int ow_lo = tw <= 0 ? 0 : (tw + g.sx - 1) / g.sx;
  const int oh_hi = min(g.OH - 1, (h + g.py) / g.sy);
  const int ow_hi = min(g.OW - 1, (w + g.px) / g.sx);
  float acc = 0.f;
  for (int oh = oh_lo; oh <= oh_hi; ++oh) {
    const int kh = h + g.py - oh * g.sy;
    for (int ow = ow_lo; ow <= ow_hi; ++ow) {
      const size_t o = obase + (size_t)oh * g.OW + ow;
      if (MODE == FLHIP_POOL_MAX) {
        const int kw = w + g.px - ow * g.sx;
        if ((int)argmax[o] == kh * g.wx + kw) acc += ld(dy, o);
      } else {
        int cnt = g.wy * g.wx;
        if (MODE == FLHIP_POOL_AVG_EXCLUDE_PADDING) {
          const int a0 = max(oh * g.sy - g.py, 0), a1 = min(oh * g.sy - g.py + g.wy, g.H);
          const int b0 = max(ow * g.sx - g.px, 0), b1 = min(ow * g.sx - g.px + g.wx, g.W);
          cnt = (a1 - a0) * (b1 - b0);
        }
        acc += ld(dy, o) / (float)cnt;
      }
    }
  }
  st(dx, e, acc);
}

template <typename T>
static int launch_fwd(const PoolGeom& g, int mode, const void* x, void* y,
                      uint8_t* argmax, hipStream_t s) {
  const size_t total = (size_t)g.N * g.C * g.OH * g.OW;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  switch (mode) {
    case FLHIP_POOL_MAX:
      hipLaunchKernelGGL((pool_fwd_direct<T, FLHIP_POOL_MAX>), grid, block, 0, s, g, xp, yp, argmax, total);
      break;
    case FLHIP_POOL_AVG_INCLUDE_PADDING:
      hipLaunchKernelGGL((pool_fwd_direct<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), grid, block, 0, s, g, xp, yp, argmax, total);
      break;
    default:
      hipLaunchKernelGGL((pool_fwd_direct<T, FLHIP_POOL_AVG_EXCLUDE_PADDING>), grid, block, 0, s, g, xp, yp, argmax, total);
  }
  return check_launch("pool2d_fwd");
}

template <typename T>
static int launch_bwd(const PoolGeom& g, int mode, const void* dy,
                      const uint8_t* argmax, void* dx, hipStream_t s) {
  const size_t total = (size_t)g.N * g.C * g.H * g.W;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  const T* dyp = static_cast<const T*>(dy);
  T* dxp = static_cast<T*>(dx);
  switch (mode) {
    case FLHIP_POOL_MAX:
      hipLaunchKernelGGL((pool_bwd_direct<T, FLHIP_POOL_MAX>), grid, block, 0, s, g, dyp, argmax, dxp, total);
      break;
    case FLHIP_POOL_AVG_INCLUDE_PADDING:
      hipLaunchKernelGGL((pool_bwd_direct<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), grid, block, 0, s, g, dyp, argmax, dxp, total);
      break;
    default:
      hipLaunchKernelGGL((pool_bwd_direct<T, FLHIP_POOL_AVG_EXCLUDE_PADDING>), grid, block, 0, s, g, dyp, argmax, dxp, total);
  }
  return check_launch("pool2d_bwd");
}

static int make_geom(const flhip_pool_desc* d, PoolGeom* g) {
  int32_t OH, OW;
  const int rc = flhip_pool2d_out_dims(d, &OH, &OW);
  if (rc != FLHIP_OK) return rc;
  *g = PoolGeom{d->N, d->C, d->H, d->W, OH, OW, d->wy, d->wx, d->sy, d->sx, d->py, d->px};
  return FLHIP_OK;
}

}  // namespace flhip

using namespace flhip;

extern "C" int flhip_pool2d_fwd(const flhip_pool_desc* d, const void* x, void* y,
                                uint8_t* argmax, void* stream) {
  FLHIP_REQUIRE(d && x && y, "pool2d_fwd: null argument");
  PoolGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  if (d->mode == FLHIP_POOL_MAX && argmax)
    FLHIP_REQUIRE(d->wy * d->wx <= 256, "pool2d_fwd: argmax needs a window of at most 256 elements");
  return d->dtype == FLHIP_F32 ? launch_fwd<float>(g, d->mode, x, y, argmax, as_stream(stream))
                               : launch_fwd<bf16_t>(g, d->mode, x, y, argmax, as_stream(stream));
}

extern "C" int flhip_pool2d_bwd(const flhip_pool_desc* d, const void* dy,
                                const uint8_t* argmax, void* dx, void* stream) {
  FLHIP_REQUIRE(d && dy && dx, "pool2d_bwd: null argument");
  PoolGeom g;
  const int rc = make_geom(d, &g);
  if (rc != FLHIP_OK) return rc;
  if (d->mode == FLHIP_POOL_MAX) {
    // the reference throws std::invalid_argument without the forward payload
    // (onednn/Pool2D.cpp:190-193)
    FLHIP_REQUIRE(argmax != nullptr, "pool2d_bwd: max pooling needs the argmax of the forward pass");
    FLHIP_REQUIRE(d->wy * d->wx <= 256, "pool2d_bwd: window of at most 256 elements");
  }
  return d->dtype == FLHIP_F32 ? launch_bwd<float>(g, d->mode, dy, argmax, dx, as_stream(stream))
                               : launch_bwd<bf16_t>(g, d->mode, dy, argmax, dx, as_stream(stream));
}
