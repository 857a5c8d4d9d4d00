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

// ---------------------------------------------------------------------------
// Fast path: 3x3 window, stride 2, padding 1, W % 4 == 0 (the ResNet stem pool).
// A thread owns four input columns [4*tq, 4*tq+3] = two output columns of a
// strip of POOL_OHB output rows and walks down the strip, so that every input
// row is fetched once as one 16-byte load per lane; the column left of the
// quad comes from the neighbouring lane.  Rows are visited in window order,
// which keeps the first-maximum tie rule and the fp32 summation order of the
// generic kernels.
// ---------------------------------------------------------------------------
constexpr int POOL_OHB = 2;

struct PoolRow {
  float l;      // column 4*tq - 1 (meaningful when tq > 0)
  float4 v;     // columns 4*tq .. 4*tq + 3
  bool ok;      // row inside the image
};

template <int MODE>
__device__ __forceinline__ void pool_scan3(const PoolRow& r, int kh, bool has_left, float a,
                                           float b, float c, float& best, int& idx, float& sum,
                                           int& cnt, bool first_col) {
  // one window row: candidates (kw = 0, 1, 2) = (a, b, c); for the first output
  // column of the thread, a is the neighbour's value and may be padding.  Rows and
  // columns outside the image are skipped by turning their candidates into values
  // that change nothing (no branches: the strip is straight-line code).
  const bool use_a = r.ok && (!first_col || has_left);
  if (MODE == FLHIP_POOL_MAX) {
    const float ca = use_a ? a : -FLT_MAX, cb = r.ok ? b : -FLT_MAX, cc = r.ok ? c : -FLT_MAX;
    if (ca > best) { best = ca; idx = kh * 3; }
    if (cb > best) { best = cb; idx = kh * 3 + 1; }
    if (cc > best) { best = cc; idx = kh * 3 + 2; }
  } else {
    // same additions in the same order as the generic kernel; skipped terms add
    // nothing because they are not added at all (a select keeps the old sum)
    sum = use_a ? sum + a : sum;
    cnt += use_a ? 1 : 0;
    sum = r.ok ? sum + b : sum;
    sum = r.ok ? sum + c : sum;
    cnt += r.ok ? 2 : 0;
  }
}

__device__ __forceinline__ void st2(float* p, size_t i, float a, float b) {
  *reinterpret_cast<float2*>(p + i) = make_float2(a, b);
}
__device__ __forceinline__ void st2(bf16_t* p, size_t i, float a, float b) {
  *reinterpret_cast<uint32_t*>(p + i) = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}
__device__ __forceinline__ void st2(f16_t* p, size_t i, float a, float b) {
  *reinterpret_cast<uint32_t*>(p + i) = pack_f16(a, b);
}
__device__ __forceinline__ float2 ld2(const f16_t* p, size_t i) {
  const uint32_t r = *reinterpret_cast<const uint32_t*>(p + i);
  return make_float2(f16lo(r), f16hi(r));
}
__device__ __forceinline__ float2 ld2(const float* p, size_t i) {
  return *reinterpret_cast<const float2*>(p + i);
}
__device__ __forceinline__ float2 ld2(const bf16_t* p, size_t i) {
  const uint32_t r = *reinterpret_cast<const uint32_t*>(p + i);
  return make_float2(__uint_as_float(r << 16), __uint_as_float(r & 0xffff0000u));
}

template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_w3s2_fwd(PoolGeom g, const T* __restrict__ x, T* __restrict__ y,
              uint8_t* __restrict__ argmax, int TQ, int nstrips, size_t items) {
  const size_t item0 = (size_t)blockIdx.x * 256 + threadIdx.x;
  const bool active = item0 < items;
  const size_t item = active ? item0 : items - 1;
  const int lane = threadIdx.x & 63;
  const int tq = (int)(item % TQ);
  const size_t t = item / TQ;
  const int oh0 = (int)(t % nstrips) * POOL_OHB;
  const size_t plane = t / nstrips;
  const T* xq = x + plane * (size_t)g.H * g.W + 4 * tq;
  const size_t obase = plane * (size_t)g.OH * g.OW + 2 * tq;
  const bool has_left = tq > 0;

  // All 2*POOL_OHB+1 input rows of the strip are requested before any is used: the
  // 16-byte loads first, then (lane 0 of a wave only) the column left of the quad,
  // which the other lanes get from their neighbour.
  constexpr int NR = 2 * POOL_OHB + 1;
  float4 rv[NR];
  float rl[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    // row index clamped into the image (plane sizes are below 2^31 elements)
    rv[j] = ld4(xq, (size_t)(min(max(2 * oh0 - 1 + j, 0), g.H - 1) * g.W));
    rl[j] = 0.f;
  }
  if (lane == 0 && tq > 0) {
#pragma unroll
    for (int j = 0; j < NR; ++j)
      rl[j] = ld(xq, (size_t)(min(max(2 * oh0 - 1 + j, 0), g.H - 1) * g.W - 1));
  }
  // row j of the strip with its left neighbour; `ok` says whether it lies in the image
  auto row = [&](int j, bool ok) {
    PoolRow r;
    r.ok = ok;
    r.v = rv[j];
    const float up = __shfl_up(rv[j].w, 1, 64);
    r.l = lane == 0 ? rl[j] : up;
    return r;
  };
  PoolRow r0 = row(0, oh0 > 0);
#pragma unroll
  for (int k = 0; k < POOL_OHB; ++k) {
    const int oh = oh0 + k;
    const bool ok = oh < g.OH;
    const PoolRow r1 = row(2 * k + 1, ok && 2 * oh < g.H);
    const PoolRow r2 = row(2 * k + 2, ok && 2 * oh + 1 < g.H);
    float b0 = -FLT_MAX, b1 = -FLT_MAX, s0 = 0.f, s1 = 0.f;
    int i0 = 0, i1 = 0, c0 = 0, c1 = 0;
    pool_scan3<MODE>(r0, 0, has_left, r0.l, r0.v.x, r0.v.y, b0, i0, s0, c0, true);
    pool_scan3<MODE>(r1, 1, has_left, r1.l, r1.v.x, r1.v.y, b0, i0, s0, c0, true);
    pool_scan3<MODE>(r2, 2, has_left, r2.l, r2.v.x, r2.v.y, b0, i0, s0, c0, true);
    pool_scan3<MODE>(r0, 0, true, r0.v.y, r0.v.z, r0.v.w, b1, i1, s1, c1, false);
    pool_scan3<MODE>(r1, 1, true, r1.v.y, r1.v.z, r1.v.w, b1, i1, s1, c1, false);
    pool_scan3<MODE>(r2, 2, true, r2.v.y, r2.v.z, r2.v.w, b1, i1, s1, c1, false);
    if (active && ok) {
      const size_t o = obase + (size_t)oh * g.OW;
      if (MODE == FLHIP_POOL_MAX) {
        st2(y, o, b0, b1);
        if (argmax) *reinterpret_cast<uint16_t*>(argmax + o) = (uint16_t)(i0 | (i1 << 8));
      } else if (MODE == FLHIP_POOL_AVG_INCLUDE_PADDING) {
        st2(y, o, s0 / 9.f, s1 / 9.f);
      } else {
        st2(y, o, s0 / (float)c0, s1 / (float)c1);
      }
    }
    r0 = r2;
  }
}

// Backward for the same geometry.  A thread owns the same four input columns
// and strip; it reads dy / argmax of its two output columns (plus the next one
// from the neighbouring lane) row by row and accumulates the three input rows
// each output row touches, carrying the shared odd row to the next output row so
// that the additions happen in ascending (oh, ow) order.
struct PoolGrad {
  float g0, g1, g2;   // dy (already divided for the average modes) at ow = 2tq, 2tq+1, 2tq+2
  int a0, a1, a2;     // argmax bytes (max mode)
  bool ok;            // output row exists
};

template <typename T, int MODE>
__device__ __forceinline__ PoolGrad pool_load_grad(const PoolGeom& g, const T* dyq,
                                                   const uint8_t* amq, int oh, bool ok, int tq,
                                                   int TQ, int lane) {
  PoolGrad r;
  r.ok = ok;
  float2 d = make_float2(0.f, 0.f);
  int a0 = 255, a1 = 255;
  if (ok) {
    d = ld2(dyq, (size_t)oh * g.OW);
    if (MODE == FLHIP_POOL_MAX) {
      const uint16_t a = *reinterpret_cast<const uint16_t*>(amq + (size_t)oh * g.OW);
      a0 = a & 0xff;
      a1 = a >> 8;
    } else if (MODE == FLHIP_POOL_AVG_INCLUDE_PADDING) {
      d.x = d.x / 9.f;
      d.y = d.y / 9.f;
    } else {
      // in-bounds count of window (oh, ow): rows 2oh-1..2oh+1, cols 2ow-1..2ow+1
      const int rows = min(2 * oh + 2, g.H) - max(2 * oh - 1, 0);
      const int cw0 = min(4 * tq + 2, g.W) - max(4 * tq - 1, 0);
      const int cw1 = min(4 * tq + 4, g.W) - (4 * tq + 1);
      d.x = d.x / (float)(rows * cw0);
      d.y = d.y / (float)(rows * cw1);
    }
  }
  r.g0 = d.x; r.g1 = d.y; r.a0 = a0; r.a1 = a1;
  // the next output column belongs to the next lane
  float g2 = __shfl_down(d.x, 1, 64);
  int a2 = __shfl_down(a0, 1, 64);
  const bool has_right = tq + 1 < TQ;
  if (lane == 63 && has_right && ok) {
    if (MODE == FLHIP_POOL_MAX) {
      g2 = ld(dyq, (size_t)oh * g.OW + 2);
      a2 = amq[(size_t)oh * g.OW + 2];
    } else {
      float v = ld(dyq, (size_t)oh * g.OW + 2);
      if (MODE == FLHIP_POOL_AVG_INCLUDE_PADDING) {
        v = v / 9.f;
      } else {
        const int rows = min(2 * oh + 2, g.H) - max(2 * oh - 1, 0);
        const int cw2 = min(4 * tq + 6, g.W) - (4 * tq + 3);
        v = v / (float)(rows * cw2);
      }
      g2 = v;
    }
  }
  r.g2 = (has_right && ok) ? g2 : 0.f;
  r.a2 = has_right ? a2 : 255;
  return r;
}

// adds the contributions of output row `q` through window row kh to the four columns
template <int MODE>
__device__ __forceinline__ void pool_bwd_row(const PoolGrad& q, int kh, float4& acc) {
  if (!q.ok) return;
  if (MODE == FLHIP_POOL_MAX) {
    acc.x += (q.a0 == kh * 3 + 1) ? q.g0 : 0.f;
    acc.y += (q.a0 == kh * 3 + 2) ? q.g0 : 0.f;
    acc.y += (q.a1 == kh * 3 + 0) ? q.g1 : 0.f;
    acc.z += (q.a1 == kh * 3 + 1) ? q.g1 : 0.f;
    acc.w += (q.a1 == kh * 3 + 2) ? q.g1 : 0.f;
    acc.w += (q.a2 == kh * 3 + 0) ? q.g2 : 0.f;
  } else {
    acc.x += q.g0;
    acc.y += q.g0;
    acc.y += q.g1;
    acc.z += q.g1;
    acc.w += q.g1;
    acc.w += q.g2;
  }
}

template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_w3s2_bwd(PoolGeom g, const T* __restrict__ dy, const uint8_t* __restrict__ argmax,
              T* __restrict__ dx, int TQ, int nstrips, size_t items) {
  const size_t item0 = (size_t)blockIdx.x * 256 + threadIdx.x;
  const bool active = item0 < items;
  const size_t item = active ? item0 : items - 1;
  const int lane = threadIdx.x & 63;
  const int tq = (int)(item % TQ);
  const size_t t = item / TQ;
  const int strip = (int)(t % nstrips);
  const int oh0 = strip * POOL_OHB;
  const size_t plane = t / nstrips;
  const T* dyq = dy + plane * (size_t)g.OH * g.OW + 2 * tq;
  const uint8_t* amq = MODE == FLHIP_POOL_MAX ? argmax + plane * (size_t)g.OH * g.OW + 2 * tq : nullptr;
  T* dxq = dx + plane * (size_t)g.H * g.W + 4 * tq;

  // the strip owns input rows 2*oh0-1 .. 2*oh_end-2 (and 2*oh_end-1 when it is the
  // last strip); row 2*oh0-1 also receives from output row oh0-1
  float4 odd = make_float4(0.f, 0.f, 0.f, 0.f);   // accumulates row 2*oh-1
  {
    const PoolGrad q = pool_load_grad<T, MODE>(g, dyq, amq, oh0 - 1, oh0 > 0, tq, TQ, lane);
    pool_bwd_row<MODE>(q, 2, odd);
  }
#pragma unroll 2
  for (int k = 0; k < POOL_OHB; ++k) {
    const int oh = oh0 + k;
    const bool ok = oh < g.OH;
    const PoolGrad q = pool_load_grad<T, MODE>(g, dyq, amq, oh, ok, tq, TQ, lane);
    pool_bwd_row<MODE>(q, 0, odd);
    float4 even = make_float4(0.f, 0.f, 0.f, 0.f);
    pool_bwd_row<MODE>(q, 1, even);
    if (active && ok) {
      if (2 * oh - 1 >= 0) st4_stream(dxq, (size_t)(2 * oh - 1) * g.W, odd);
      if (2 * oh < g.H) st4_stream(dxq, (size_t)(2 * oh) * g.W, even);
    }
    odd = make_float4(0.f, 0.f, 0.f, 0.f);
    pool_bwd_row<MODE>(q, 2, odd);
    // last output row of the image: nothing below adds to row 2*oh+1
    if (active && ok && oh == g.OH - 1) {
      for (int r = 2 * oh + 1; r < g.H; ++r) {
        st4_stream(dxq, (size_t)r * g.W, odd);
        odd = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Fast path: 2x2 window, stride 2, no padding, H % 2 == 0, W % 4 == 0 (the pooling of
// the README convnet and of VGG-style networks).  Windows do not overlap: a thread owns
// four input columns x two rows = two windows, reads / writes them as 16-byte vectors,
// and every input element belongs to exactly one window, so the backward pass is a
// plain streaming write.  Candidate order (kh, kw) and the strict comparison keep the
// first-maximum rule and the summation order of the generic kernels.
// ---------------------------------------------------------------------------
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_w2s2_fwd(PoolGeom g, const T* __restrict__ x, T* __restrict__ y, uint8_t* __restrict__ argmax,
              size_t items) {
  const size_t it = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (it >= items) return;
  const int TQ = g.W >> 2;
  const int tq = (int)(it % TQ);
  const size_t t = it / TQ;
  const int oh = (int)(t % g.OH);
  const size_t plane = t / g.OH;
  const size_t xo = (plane * g.H + 2 * oh) * (size_t)g.W + 4 * tq;
  const float4 r0 = ld4(x, xo), r1 = ld4(x, xo + g.W);
  const float c[2][4] = {{r0.x, r0.y, r1.x, r1.y}, {r0.z, r0.w, r1.z, r1.w}};
  float out[2];
  int idx[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (MODE == FLHIP_POOL_MAX) {
      float best = -FLT_MAX;
      int bi = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (c[j][k] > best) {
          best = c[j][k];
          bi = k;
        }
      out[j] = best;
      idx[j] = bi;
    } else {
      out[j] = (((c[j][0] + c[j][1]) + c[j][2]) + c[j][3]) / 4.f;
      idx[j] = 0;
    }
  }
  const size_t yo = (plane * g.OH + oh) * (size_t)g.OW + 2 * tq;
  st2(y, yo, out[0], out[1]);
  if (MODE == FLHIP_POOL_MAX && argmax)
    *reinterpret_cast<uint16_t*>(argmax + yo) = (uint16_t)(idx[0] | (idx[1] << 8));
}

template <typename T, int MODE>
__global__ void __launch_bounds__(256)
pool_w2s2_bwd(PoolGeom g, const T* __restrict__ dy, const uint8_t* __restrict__ argmax,
              T* __restrict__ dx, size_t items) {
  const size_t it = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (it >= items) return;
  const int TQ = g.W >> 2;
  const int tq = (int)(it % TQ);
  const size_t t = it / TQ;
  const int oh = (int)(t % g.OH);
  const size_t plane = t / g.OH;
  const size_t yo = (plane * g.OH + oh) * (size_t)g.OW + 2 * tq;
  const float2 d = ld2(dy, yo);
  float v[2][4];
  if (MODE == FLHIP_POOL_MAX) {
    const uint16_t am = *reinterpret_cast<const uint16_t*>(argmax + yo);
    const int i0 = am & 0xff, i1 = am >> 8;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[0][k] = i0 == k ? d.x : 0.f;
      v[1][k] = i1 == k ? d.y : 0.f;
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[0][k] = d.x / 4.f;
      v[1][k] = d.y / 4.f;
    }
  }
  const size_t xo = (plane * g.H + 2 * oh) * (size_t)g.W + 4 * tq;
  st4(dx, xo, make_float4(v[0][0], v[0][1], v[1][0], v[1][1]));
  st4(dx, xo + g.W, make_float4(v[0][2], v[0][3], v[1][2], v[1][3]));
}

static bool w2s2_applies(const PoolGeom& g, const void* a, const void* b, const void* am) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
  return g.wy == 2 && g.wx == 2 && g.sy == 2 && g.sx == 2 && g.py == 0 && g.px == 0 &&
         g.W % 4 == 0 && g.H % 2 == 0 && bits % 16 == 0 && reinterpret_cast<uintptr_t>(am) % 2 == 0;
}

static bool w3s2_applies(const PoolGeom& g, const void* a, const void* b, const void* am) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
  return g.wy == 3 && g.wx == 3 && g.sy == 2 && g.sx == 2 && g.py == 1 && g.px == 1 &&
         g.W % 4 == 0 && g.H >= 2 && bits % 16 == 0 && reinterpret_cast<uintptr_t>(am) % 2 == 0;
}

template <typename T>
static int launch_fwd(const PoolGeom& g, int mode, const void* x, void* y,
                      uint8_t* argmax, hipStream_t s) {
  const size_t total = (size_t)g.N * g.C * g.OH * g.OW;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  if (w2s2_applies(g, x, y, argmax)) {
    const size_t items = (size_t)g.N * g.C * g.OH * (g.W / 4);
    const dim3 fgrid((unsigned)((items + 255) / 256));
    if (mode == FLHIP_POOL_MAX)
      hipLaunchKernelGGL((pool_w2s2_fwd<T, FLHIP_POOL_MAX>), fgrid, block, 0, s, g, xp, yp, argmax, items);
    else   // no padding: both average modes divide by 4
      hipLaunchKernelGGL((pool_w2s2_fwd<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), fgrid, block, 0, s, g, xp, yp, argmax, items);
    return check_launch("pool2d_fwd");
  }
  if (w3s2_applies(g, x, y, argmax)) {
    const int TQ = g.W / 4, nstrips = (g.OH + POOL_OHB - 1) / POOL_OHB;
    const size_t items = (size_t)g.N * g.C * nstrips * TQ;
    const dim3 fgrid((unsigned)((items + 255) / 256));
    switch (mode) {
      case FLHIP_POOL_MAX:
        hipLaunchKernelGGL((pool_w3s2_fwd<T, FLHIP_POOL_MAX>), fgrid, block, 0, s, g, xp, yp, argmax, TQ, nstrips, items);
        break;
      case FLHIP_POOL_AVG_INCLUDE_PADDING:
        hipLaunchKernelGGL((pool_w3s2_fwd<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), fgrid, block, 0, s, g, xp, yp, argmax, TQ, nstrips, items);
        break;
      default:
        hipLaunchKernelGGL((pool_w3s2_fwd<T, FLHIP_POOL_AVG_EXCLUDE_PADDING>), fgrid, block, 0, s, g, xp, yp, argmax, TQ, nstrips, items);
    }
    return check_launch("pool2d_fwd");
  }
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
  if (w2s2_applies(g, dy, dx, argmax)) {
    const size_t items = (size_t)g.N * g.C * g.OH * (g.W / 4);
    const dim3 fgrid((unsigned)((items + 255) / 256));
    if (mode == FLHIP_POOL_MAX)
      hipLaunchKernelGGL((pool_w2s2_bwd<T, FLHIP_POOL_MAX>), fgrid, block, 0, s, g, dyp, argmax, dxp, items);
    else
      hipLaunchKernelGGL((pool_w2s2_bwd<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), fgrid, block, 0, s, g, dyp, argmax, dxp, items);
    return check_launch("pool2d_bwd");
  }
  if (w3s2_applies(g, dy, dx, argmax)) {
    const int TQ = g.W / 4, nstrips = (g.OH + POOL_OHB - 1) / POOL_OHB;
    const size_t items = (size_t)g.N * g.C * nstrips * TQ;
    const dim3 fgrid((unsigned)((items + 255) / 256));
    switch (mode) {
      case FLHIP_POOL_MAX:
        hipLaunchKernelGGL((pool_w3s2_bwd<T, FLHIP_POOL_MAX>), fgrid, block, 0, s, g, dyp, argmax, dxp, TQ, nstrips, items);
        break;
      case FLHIP_POOL_AVG_INCLUDE_PADDING:
        hipLaunchKernelGGL((pool_w3s2_bwd<T, FLHIP_POOL_AVG_INCLUDE_PADDING>), fgrid, block, 0, s, g, dyp, argmax, dxp, TQ, nstrips, items);
        break;
      default:
        hipLaunchKernelGGL((pool_w3s2_bwd<T, FLHIP_POOL_AVG_EXCLUDE_PADDING>), fgrid, block, 0, s, g, dyp, argmax, dxp, TQ, nstrips, items);
    }
    return check_launch("pool2d_bwd");
  }
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
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch_fwd<T>(g, d->mode, x, y, argmax, as_stream(stream));
  });
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
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch_bwd<T>(g, d->mode, dy, argmax, dx, as_stream(stream));
  });
}
