// batchnorm (train / inference) and batchnormBackward.
//
// View: element (o, c, i) at (o*C + c)*inner + i.  Two kernels per pass:
//   1. partial per-feature sums over S slices of the (o, i) domain, written to
//      the workspace as ws[(c*S + s)*2 + {0,1}];
//   2. an elementwise kernel whose prologue folds the S partials of its feature
//      (in double) and then streams the tensor once more.
// inner > 1 ("segment" kernels): every feature owns `outer` contiguous runs of
// `inner` elements; threads stream them with 4-wide loads when inner % 4 == 0.
// inner == 1 ("column" kernels, per-activation mode): features are contiguous, a
// wave covers 64 features and rows are strided by C.
#include <stdlib.h>
#include <string.h>

#include "common.h"

namespace flhip {

int mfma_num_cus();   // compute units of the current device (defined with the convolution kernels)

struct BnGeom {
  long long outer, C, inner;
  int S;            // slices per feature
  long long units;  // seg: outer * inner / VEC   col: outer
  long long ups;    // units per slice
  int step_o, step_i;  // seg: 256 = step_o * (inner/VEC) + step_i
};

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Folds the S (<= 64) partial pairs of feature c; valid in wave 0.
__device__ __forceinline__ void fold_partials(const float* __restrict__ ws, long long c, int S,
                                              double* a, double* b) {
  const int lane = threadIdx.x & 63;
  double p0 = 0.0, p1 = 0.0;
  if (lane < S) {
    p0 = (double)ws[(c * S + lane) * 2 + 0];
    p1 = (double)ws[(c * S + lane) * 2 + 1];
  }
  *a = wave_sum_f64(p0);
  *b = wave_sum_f64(p1);
}

// the two sums of a kernel together where its registers allow (the kernels that hold 25 vectors per thread
// have none to spare for the second sum's lanes in flight)
template <bool TOGETHER, int NW = 0>
__device__ __forceinline__ void block_sums(float& a, float& b, float* red) {
  if (TOGETHER) {
    block_sum2<NW>(a, b, red);
  } else {
    a = block_sum<NW>(a, red);
    b = block_sum<NW>(b, red);
  }
}

template <typename T, int VEC>
struct Vec;
template <typename T>
struct Vec<T, 1> {
  float v[1];
  __device__ __forceinline__ void load(const T* p, size_t i) { v[0] = ld(p, i); }
  __device__ __forceinline__ void store(T* p, size_t i) const { st(p, i, v[0]); }
};
template <typename T>
struct Vec<T, 4> {
  float v[4];
  __device__ __forceinline__ void load(const T* p, size_t i) {
    const float4 f = ld4(p, i);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
  }
  __device__ __forceinline__ void store(T* p, size_t i) const {
    st4_stream(p, i, make_float4(v[0], v[1], v[2], v[3]));
  }
};

// Visits the units [u0, u1) of slice blockIdx.y of feature blockIdx.x, BN_UN at a
// time per thread: f(off, n) gets BN_UN element offsets of which the first n are
// in range (the others repeat a valid offset so loads need no branch).  Issuing
// BN_UN independent 16-byte loads per thread is what keeps enough bytes in flight
// to cover HBM latency.  The feature index is the fast grid dimension:
// workgroups that run together then read neighbouring segments of the same
// outer slice, i.e. one contiguous region of memory, which is what HBM likes.
constexpr int BN_UN = 4;

template <int VEC, bool REVERSE, typename F>
__device__ __forceinline__ void bn_seg_visit(const BnGeom& g, F&& f) {
  // REVERSE: slices are taken from the end of the tensor first.  The second
  // kernel of a pass uses it so that it starts with what the first kernel read
  // last and is most likely still cached.
  const long long c = blockIdx.x;
  const long long innerV = g.inner / VEC;
  const long long slice = REVERSE ? (long long)(gridDim.y - 1 - blockIdx.y) : (long long)blockIdx.y;
  const long long u0 = slice * g.ups;
  const long long u1 = min(u0 + g.ups, g.units);
  long long u = u0 + threadIdx.x;
  long long o = u / innerV;
  long long i = u - o * innerV;
  while (u < u1) {
    size_t off[BN_UN];
    int n = 0;
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
      const size_t here = (size_t)((o * g.C + c) * g.inner + i * VEC);
      const bool in = u < u1;
      off[k] = in ? here : off[0];
      n += in ? 1 : 0;
      u += 256;
      o += g.step_o;
      i += g.step_i;
      if (i >= innerV) {
        i -= innerV;
        ++o;
      }
    }
    f(off, n);
  }
}

// ---- forward, segment mode -------------------------------------------------
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
bn_stats_seg(BnGeom g, const T* __restrict__ x, float* __restrict__ ws) {
  __shared__ float red[8];
  float s1 = 0.f, s2 = 0.f;
  const long long c = blockIdx.x;
  const float shift = ld(x, (size_t)(c * g.inner));
  bn_seg_visit<VEC, false>(g, [&](const size_t (&off)[BN_UN], int n) {
    Vec<T, VEC> a[BN_UN];
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) a[k].load(x, off[k]);
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
      float p1 = 0.f, p2 = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float t = a[k].v[e] - shift;
        p1 += t;
        p2 += t * t;
      }
      if (k < n) {
        s1 += p1;
        s2 += p2;
      }
    }
  });
  block_sum2<4>(s1, s2, red);
  if (threadIdx.x == 0) {
    ws[(c * g.S + blockIdx.y) * 2 + 0] = s1;
    ws[(c * g.S + blockIdx.y) * 2 + 1] = s2;
  }
}

struct BnTrainArgs {
  const float* gamma;
  const float* beta;
  float* save_mean;
  float* save_invstd;
  float* run_mean;
  float* run_var;
  double momentum, eps;
};

// Mean / inverse std of feature c from the folded shifted sums; lane 0 of wave 0
// of slice 0 also publishes the statistics.
// Per-feature scalars of the forward kernels, loaded when the kernel starts: a load issued only where its value
// is used (after the reduction, after the barrier) adds a trip to memory to the chain reduction -> statistics ->
// output, which is most of the time of a layer with small planes.
struct BnTrainPre {
  float gamma, beta, run_mean, run_var;
};
__device__ __forceinline__ BnTrainPre bn_preload(const BnTrainArgs& a, long long c, bool publish = true) {
  BnTrainPre p;
  p.gamma = a.gamma ? a.gamma[c] : 1.f;
  p.beta = a.beta ? a.beta[c] : 0.f;
  const bool run = publish && a.run_mean && a.run_var && a.momentum != 0.0;
  p.run_mean = run ? a.run_mean[c] : 0.f;
  p.run_var = run ? a.run_var[c] : 0.f;
  return p;
}

__device__ __forceinline__ void finish_stats(const BnGeom& g, const BnTrainArgs& a, long long c,
                                             float shift, double p0, double p1, bool publish,
                                             float* sh /* [2] */, const BnTrainPre* pre /* null: loaded here */) {
  if (threadIdx.x == 0) {
    const double M = (double)g.outer * (double)g.inner;
    const double m1 = p0 / M;
    double var = p1 / M - m1 * m1;
    if (var < 0.0) var = 0.0;
    const double mean = (double)shift + m1;
    const double invstd = 1.0 / sqrt(var + a.eps);
    sh[0] = (float)mean;
    sh[1] = (float)invstd;
    if (publish) {
      if (a.save_mean) a.save_mean[c] = (float)mean;
      if (a.save_invstd) a.save_invstd[c] = (float)invstd;
      if (a.run_mean && a.run_var) {
        if (a.momentum == 0.0) {
          a.run_mean[c] = (float)mean;
          a.run_var[c] = (float)var;
        } else {
          const double unb = M > 1.0 ? var * M / (M - 1.0) : var;
          const double rm = pre ? pre->run_mean : a.run_mean[c], rv = pre ? pre->run_var : a.run_var[c];
          a.run_mean[c] = (float)((1.0 - a.momentum) * rm + a.momentum * mean);
          a.run_var[c] = (float)((1.0 - a.momentum) * rv + a.momentum * unb);
        }
      }
    }
  }
}

// Fused epilogue of the forward kernels (FUSE instantiations): y = relu(bn(x) + residual),
// residual optional, ReLU optional.
template <typename T>
struct BnFuseFwd {
  const T* res;   // may be null
  int relu;
  uint8_t* mask;  // may be null: one byte per 4 consecutive elements, bit e = (y[4 i + e] > 0)
};
// Fused prologue of the backward kernels: the incoming gradient passes the ReLU mask of the
// forward result y first (dz = dy where y > 0), and dz itself can be written out for the
// residual branch.
template <typename T>
struct BnFuseBwd {
  const T* y;     // forward result (after the ReLU)
  T* dres;        // may be null
  const uint8_t* mask;   // may be null; when given it stands for y > 0 and y is not read (an eighth of
                         // the bytes of a bf16 y, a sixteenth of an fp32 one)
};

// value as it reads back from storage of type T
__device__ __forceinline__ float rounded(float v, const float*) { return v; }
__device__ __forceinline__ float rounded(float v, const bf16_t*) { return bf16_to_f32(f32_to_bf16(v)); }
__device__ __forceinline__ float rounded(float v, const f16_t*) { return f16_to_f32(f32_to_f16(v)); }
// the ReLU mask of the vector at element offset `off` as values that compare like y: from the mask bytes
// when the caller has them (4-element vectors only), else from y itself
template <int VEC, bool MASK, typename T>
__device__ __forceinline__ void seg_mask_load(Vec<T, VEC>& m, const BnFuseBwd<T>& fu, size_t off) {
  if (VEC == 4 && MASK) {
    const unsigned bits = fu.mask[off >> 2];
#pragma unroll
    for (int e = 0; e < VEC; ++e) m.v[e] = (bits >> e) & 1u ? 1.f : 0.f;
  } else {
    m.load(fu.y, off);
  }
}

template <typename T, int VEC, int FUSE = 0>
__global__ void __launch_bounds__(256)
bn_train_apply_seg(BnGeom g, const T* __restrict__ x, T* __restrict__ y,
                   const float* __restrict__ ws, BnTrainArgs a, BnFuseFwd<T> fu = BnFuseFwd<T>{nullptr, 0, nullptr}) {
  __shared__ float sh[2];
  const BnTrainPre pre = bn_preload(a, blockIdx.x, blockIdx.y == 0);
  if (threadIdx.x < 64) {
    double p0, p1;
    fold_partials(ws, blockIdx.x, g.S, &p0, &p1);
    finish_stats(g, a, blockIdx.x, ld(x, (size_t)(blockIdx.x * g.inner)), p0, p1,
                 blockIdx.y == 0, sh, &pre);
  }
  __syncthreads();
  const float mean = sh[0];
  const float scale = pre.gamma * sh[1];
  const float bt = pre.beta;
  bn_seg_visit<VEC, true>(g, [&](const size_t (&off)[BN_UN], int n) {
    Vec<T, VEC> v[BN_UN], r[BN_UN];
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) v[k].load(x, off[k]);
    if (FUSE && fu.res) {
#pragma unroll
      for (int k = 0; k < BN_UN; ++k) r[k].load(fu.res, off[k]);
    }
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float t = (v[k].v[e] - mean) * scale + bt;
        if (FUSE) {
          if (fu.res) t += r[k].v[e];
          if (fu.relu) t = t > 0.f ? t : 0.f;
        }
        v[k].v[e] = t;
      }
      if (k < n) {
        v[k].store(y, off[k]);
        if (FUSE == 2 && VEC == 4) {
          unsigned bits = 0;
#pragma unroll
          for (int e = 0; e < VEC; ++e) bits |= (rounded(v[k].v[e], y) > 0.f ? 1u : 0u) << e;
          fu.mask[off[k] >> 2] = (uint8_t)bits;
        }
      }
    }
  });
}

// ---- backward, segment mode ------------------------------------------------
template <typename T, int VEC, int FUSE = 0>
__global__ void __launch_bounds__(256)
bn_bwd_stats_seg(BnGeom g, const T* __restrict__ x, const T* __restrict__ dy,
                 const float* __restrict__ save_mean, float* __restrict__ ws,
                 BnFuseBwd<T> fu = BnFuseBwd<T>{nullptr, nullptr, nullptr}) {
  __shared__ float red[8];
  float s1 = 0.f, s2 = 0.f;
  const long long c = blockIdx.x;
  const float mean = save_mean[c];
  constexpr bool MASK = FUSE == 2 && VEC == 4;   // the ReLU mask comes as bytes, not from y
  bn_seg_visit<VEC, false>(g, [&](const size_t (&off)[BN_UN], int n) {
    Vec<T, VEC> a[BN_UN], b[BN_UN], m[BN_UN];
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
      a[k].load(x, off[k]);
      b[k].load(dy, off[k]);
      if (FUSE) seg_mask_load<VEC, MASK>(m[k], fu, off[k]);
    }
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
      float p1 = 0.f, p2 = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (FUSE) b[k].v[e] = m[k].v[e] > 0.f ? b[k].v[e] : 0.f;
        p1 += b[k].v[e];
        p2 += b[k].v[e] * (a[k].v[e] - mean);
      }
      if (k < n) {
        s1 += p1;
        s2 += p2;
      }
    }
  });
  block_sum2<4>(s1, s2, red);
  if (threadIdx.x == 0) {
    ws[(c * g.S + blockIdx.y) * 2 + 0] = s1;
    ws[(c * g.S + blockIdx.y) * 2 + 1] = s2;
  }
}

struct BnBwdArgs {
  const float* gamma;
  const float* save_mean;
  const float* save_invstd;
  float* dgamma;
  float* dbeta;
};

// dx = k_dy*dy + k_x*(x-mean) + k_0 for feature c; publishes dgamma/dbeta.
// (pre: the feature's scalars, loaded when the kernel starts - see BnTrainPre)
struct BnBwdPre {
  float mean, invstd, gamma;
};
__device__ __forceinline__ BnBwdPre bn_preload(const BnBwdArgs& a, long long c) {
  BnBwdPre p;
  p.mean = a.save_mean[c];
  p.invstd = a.save_invstd[c];
  p.gamma = a.gamma ? a.gamma[c] : 1.f;
  return p;
}
__device__ __forceinline__ void finish_bwd(const BnGeom& g, const BnBwdArgs& a, long long c,
                                           double p0, double p1, bool publish, float* sh /*[4]*/, const BnBwdPre& pre) {
  if (threadIdx.x == 0) {
    const double M = (double)g.outer * (double)g.inner;
    const double is = (double)pre.invstd;
    const double gm = (double)pre.gamma;
    sh[0] = pre.mean;
    sh[1] = (float)(gm * is);                    // k_dy
    sh[2] = (float)(-gm * is * is * is * p1 / M);  // k_x
    sh[3] = (float)(-gm * is * p0 / M);          // k_0
    if (publish) {
      if (a.dgamma) a.dgamma[c] = (float)(p1 * is);
      if (a.dbeta) a.dbeta[c] = (float)p0;
    }
  }
}

template <typename T, int VEC, int FUSE = 0>
__global__ void __launch_bounds__(256)
bn_bwd_apply_seg(BnGeom g, const T* __restrict__ x, const T* __restrict__ dy,
                 T* __restrict__ dx, const float* __restrict__ ws, BnBwdArgs a,
                 BnFuseBwd<T> fu = BnFuseBwd<T>{nullptr, nullptr, nullptr}) {
  __shared__ float sh[4];
  const BnBwdPre pre = bn_preload(a, blockIdx.x);
  if (threadIdx.x < 64) {
    double p0, p1;
    fold_partials(ws, blockIdx.x, g.S, &p0, &p1);
    finish_bwd(g, a, blockIdx.x, p0, p1, blockIdx.y == 0, sh, pre);
  }
  __syncthreads();
  const float mean = sh[0], kdy = sh[1], kx = sh[2], k0 = sh[3];
  constexpr bool MASK = FUSE == 2 && VEC == 4;   // the ReLU mask comes as bytes, not from y
  bn_seg_visit<VEC, true>(g, [&](const size_t (&off)[BN_UN], int n) {
    Vec<T, VEC> v[BN_UN], w[BN_UN], m[BN_UN];
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
      v[k].load(x, off[k]);
      w[k].load(dy, off[k]);
      if (FUSE) seg_mask_load<VEC, MASK>(m[k], fu, off[k]);
    }
#pragma unroll
    for (int k = 0; k < BN_UN; ++k) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (FUSE) w[k].v[e] = m[k].v[e] > 0.f ? w[k].v[e] : 0.f;
        v[k].v[e] = kdy * w[k].v[e] + (kx * (v[k].v[e] - mean) + k0);
      }
      if (k < n) {
        v[k].store(dx, off[k]);
        if (FUSE && fu.dres) w[k].store(fu.dres, off[k]);
      }
    }
  });
}

// ---- resident kernels (segment mode, 4-wide) ------------------------------------
// One workgroup (1024 threads, 256 for small features) owns a whole feature and keeps its x values in
// registers between the reduction and the elementwise pass (K 16-byte vectors per
// thread), so x is read from memory once.  The backward kernel also parks the
// first KL vectors of dy per thread in LDS and re-reads only the rest.  Used when
// a feature fits (outer*inner <= 4096*K) and there are enough features to fill
// the machine; no workspace, no second launch.
constexpr int RES_KMAX = 25;
constexpr int RES_KL = 9;             // dy vectors per thread parked in LDS (9 x 16 KiB)
constexpr int RES_MIN_C_FWD = 64;     // fewer features leave too many CUs idle
constexpr int RES_MIN_C_BWD = 128;

// Feature of this workgroup in the resident kernels (one workgroup per feature).  Workgroups go to
// the 8 XCDs in turn; numbering features so that XCD x gets the contiguous range
// [x * C / 8, (x + 1) * C / 8) keeps the cache lines that neighbouring features share - rows of 98
// or 392 bytes on 7x7 / 14x14 planes start and end inside a line - in ONE XCD's L2 instead of
// fetching them into two.
__device__ __forceinline__ int res_feature(const BnGeom& g) {
  const int b = blockIdx.x, C = (int)g.C;
  return (C & 7) ? b : (b & 7) * (C >> 3) + (b >> 3);
}

// The mask bytes of the fused kernels (one byte per 4 consecutive elements) through a buffer descriptor: the byte
// of the vector at byte offset `off` of a tensor of `esz`-byte elements is off / (4 esz); the out-of-range offset
// of the walks below (0x80000000) lands past the mask as well.  No mask: an empty range (stores dropped).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t mask_rsrc(const uint8_t* mask, const void* any, unsigned bytes, int esz) {
  return make_rsrc(mask ? (const void*)mask : any, mask ? bytes >> (esz == 2 ? 3 : 4) : 0u);
}
__device__ __forceinline__ int mask_off(int off, int esz) { return (int)((unsigned)off >> (esz == 2 ? 3 : 4)); }

// Walks this thread's vectors q = tid + 1024*k: f(k, byte offset, in range).  The
// offset is relative to the tensor base and goes through a buffer descriptor; slots
// past the feature get an offset past the descriptor's range, so their loads return
// zero and their stores are dropped without a branch.
// (q0, feature: a workgroup that owns the vectors from q0 on of a feature other than res_feature's)
template <int RES_THREADS, int K, int ESZ, int FENCE, bool REV = false, int VEC = 4, typename F>
__device__ __forceinline__ void res_visit(const BnGeom& g, F&& f, int q0 = 0, int feature = -1) {
  constexpr int OOB = (int)0x80000000;
  const int innerV = (int)(g.inner / VEC);
  const int units = (int)(g.units * 4 / VEC);      // g.units counts 4-element vectors
  const int c = feature >= 0 ? feature : res_feature(g);
  // REV walks k = K-1 .. 0: what the previous walk loaded last is asked for first,
  // while the caches still hold it
  int q = threadIdx.x + q0 + (REV ? (K - 1) * RES_THREADS : 0);
  int o = q / innerV, i = q - o * innerV;
  const int so = RES_THREADS / innerV, si = RES_THREADS - so * innerV;
  const int row = (int)(g.C * g.inner) * ESZ;                 // bytes between outer slices
  int off = ((o * (int)g.C + c) * (int)g.inner + i * VEC) * ESZ;
  const int step = so * row + si * VEC * ESZ;
  const int wrap = row - (int)g.inner * ESZ;
  // Each walk recomputes its offsets (two or three adds per vector): keeping the K
  // offsets of the first walk alive for the next one would cost K registers.
  asm volatile("" : "+v"(off), "+v"(i), "+v"(q));
#pragma unroll
  for (int kk = 0; kk < K; ++kk) {
    const int k = REV ? K - 1 - kk : kk;
    const bool in = q < units;
    f(k, in ? off : OOB, in);
    // FENCE > 0: finish each group of FENCE vectors before starting the next, or the
    // scheduler overlaps the temporaries of all K vectors and runs out of registers
    if (FENCE > 0 && kk % (FENCE > 0 ? FENCE : 1) == (FENCE > 0 ? FENCE : 1) - 1)
      __builtin_amdgcn_sched_barrier(0);
    if (REV) {
      q -= RES_THREADS;
      off -= step;
      i -= si;
      if (i < 0) {
        i += innerV;
        off -= wrap;
      }
    } else {
      q += RES_THREADS;
      off += step;
      i += si;
      if (i >= innerV) {
        i -= innerV;
        off += wrap;
      }
    }
  }
}

// 16-byte (float) / 8-byte (bf16) buffer loads marked non-temporal: data that is read
// once should not displace what a later pass re-reads from the caches
__device__ __forceinline__ float4 buf_ld4_stream(__amdgpu_buffer_rsrc_t r, int byte_off, const float*) {
  const uintx4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 2);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z),
                     __uint_as_float(v.w));
}
__device__ __forceinline__ float4 buf_ld4_stream(__amdgpu_buffer_rsrc_t r, int byte_off, const bf16_t*) {
  const uintx2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 2);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                     __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ float4 buf_ld4_stream(__amdgpu_buffer_rsrc_t r, int byte_off, const f16_t*) {
  const uintx2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 2);
  return make_float4(f16lo(v.x), f16hi(v.x), f16lo(v.y), f16hi(v.y));
}

// the same loads with the widening left for later: a vector that waits in registers stays at its storage size
template <typename T>
struct Raw4;
template <>
struct Raw4<float> {
  uintx4_t v;
};
template <>
struct Raw4<bf16_t> {
  uintx2_t v;
};
template <>
struct Raw4<f16_t> {
  uintx2_t v;
};
__device__ __forceinline__ Raw4<float> buf_ld4_raw(__amdgpu_buffer_rsrc_t r, int byte_off, const float*) {
  return Raw4<float>{__builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 2)};
}
__device__ __forceinline__ Raw4<bf16_t> buf_ld4_raw(__amdgpu_buffer_rsrc_t r, int byte_off, const bf16_t*) {
  return Raw4<bf16_t>{__builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 2)};
}
__device__ __forceinline__ Raw4<f16_t> buf_ld4_raw(__amdgpu_buffer_rsrc_t r, int byte_off, const f16_t*) {
  return Raw4<f16_t>{__builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 2)};
}
__device__ __forceinline__ float4 widen(const Raw4<float>& w) {
  return make_float4(__uint_as_float(w.v.x), __uint_as_float(w.v.y), __uint_as_float(w.v.z), __uint_as_float(w.v.w));
}
__device__ __forceinline__ float4 widen(const Raw4<bf16_t>& w) {
  return make_float4(__uint_as_float(w.v.x << 16), __uint_as_float(w.v.x & 0xffff0000u),
                     __uint_as_float(w.v.y << 16), __uint_as_float(w.v.y & 0xffff0000u));
}
__device__ __forceinline__ float4 widen(const Raw4<f16_t>& w) {
  return make_float4(f16lo(w.v.x), f16hi(w.v.x), f16lo(w.v.y), f16hi(w.v.y));
}

// 16-byte (float) / 8-byte (bf16) buffer store of four values, streaming
__device__ __forceinline__ void buf_st4(__amdgpu_buffer_rsrc_t r, int byte_off, float4 v, float*) {
  const uintx4_t t = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z),
                      __float_as_uint(v.w)};
  __builtin_amdgcn_raw_buffer_store_b128(t, r, byte_off, 0, 2);
}
__device__ __forceinline__ void buf_st4(__amdgpu_buffer_rsrc_t r, int byte_off, float4 v, bf16_t*) {
  const uintx2_t t = {(uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16),
                      (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16)};
  __builtin_amdgcn_raw_buffer_store_b64(t, r, byte_off, 0, 2);
}
__device__ __forceinline__ void buf_st4(__amdgpu_buffer_rsrc_t r, int byte_off, float4 v, f16_t*) {
  const uintx2_t t = {pack_f16(v.x, v.y), pack_f16(v.z, v.w)};
  __builtin_amdgcn_raw_buffer_store_b64(t, r, byte_off, 0, 2);
}

template <typename T, int RES_THREADS, int K, int FUSE = 0, bool RES_EARLY = false>
__global__ void __launch_bounds__(RES_THREADS)
bn_train_resident(BnGeom g, unsigned bytes, const T* __restrict__ x, T* __restrict__ y,
                  BnTrainArgs a, BnFuseFwd<T> fu = BnFuseFwd<T>{nullptr, 0, nullptr}) {
  __shared__ float red[2 * (RES_THREADS / 64)];
  __shared__ float sh[2];
  constexpr int ESZ = (int)sizeof(T);
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), yr_ = make_rsrc(y, bytes);
  const long long c = res_feature(g);
  const float shift = ld(x, (size_t)(c * g.inner));
  // (the kernels that hold 25 vectors per thread have no registers to keep the scalars through the statistics)
  constexpr bool EARLY = K <= 16;
  BnTrainPre pre = EARLY ? bn_preload(a, c) : BnTrainPre{};
  float4 xr[K];
  float s1 = 0.f, s2 = 0.f;
  res_visit<RES_THREADS, K, ESZ, 0>(g, [&](int k, int off, bool in) { xr[k] = buf_ld4_stream(xr_, off, x); });
  // RES_EARLY (workgroups of 4 waves, at most two of them on a CU): the residual is fetched together with x.
  // Fetched where it is used, four vectors at a time (what the large kernels can afford), every group waits for a
  // trip to memory, and with so few waves on a CU nothing else runs meanwhile.  It costs a thread up to 32
  // registers, which layers with more workgroups per CU rather spend on one more of those.
  constexpr bool PRE = FUSE && RES_EARLY;
  const __amdgpu_buffer_rsrc_t rr_ = make_rsrc((FUSE && fu.res) ? fu.res : x, (FUSE && fu.res) ? bytes : 0u);   // no residual: loads give 0
  Raw4<T> rz[PRE ? K : 1];
  if (PRE) res_visit<RES_THREADS, K, ESZ, 0>(g, [&](int k, int off, bool) { rz[k] = buf_ld4_raw(rr_, off, x); });
  res_visit<RES_THREADS, K, ESZ, 1>(g, [&](int k, int, bool in) {
    const float t0 = xr[k].x - shift, t1 = xr[k].y - shift, t2 = xr[k].z - shift,
                t3 = xr[k].w - shift;
    const float p1 = (t0 + t1) + (t2 + t3);
    const float p2 = (t0 * t0 + t1 * t1) + (t2 * t2 + t3 * t3);
    s1 += in ? p1 : 0.f;
    s2 += in ? p2 : 0.f;
    // both sums are finished per vector: otherwise the second one is sunk below the
    // first block reduction and drags every vector's temporaries along
    asm("" : "+v"(s1), "+v"(s2));
  });
  block_sums<(K <= 16), (K <= 16 ? RES_THREADS / 64 : 0)>(s1, s2, red);
  finish_stats(g, a, c, shift, (double)s1, (double)s2, true, sh, EARLY ? &pre : nullptr);
  __syncthreads();
  if (!EARLY) pre = bn_preload(a, c, false);
  const float mean = sh[0];
  const float scale = pre.gamma * sh[1];
  const float bt = pre.beta;
  if (FUSE) {
    const __amdgpu_buffer_rsrc_t mr_ = mask_rsrc(FUSE == 2 ? fu.mask : nullptr, x, bytes, ESZ);   // one byte per vector
    const float lo = fu.relu ? 0.f : -__builtin_huge_valf();
    res_visit<RES_THREADS, K, ESZ, 4>(g, [&](int k, int off, bool) {
      const float4 r = PRE ? widen(rz[PRE ? k : 0]) : buf_ld4_stream(rr_, off, x);
      const float4 v = make_float4(fmaxf((xr[k].x - mean) * scale + bt + r.x, lo), fmaxf((xr[k].y - mean) * scale + bt + r.y, lo),
                                   fmaxf((xr[k].z - mean) * scale + bt + r.z, lo), fmaxf((xr[k].w - mean) * scale + bt + r.w, lo));
      buf_st4(yr_, off, v, y);
      if (FUSE == 2) {
        const unsigned bits = (rounded(v.x, y) > 0.f ? 1u : 0u) | (rounded(v.y, y) > 0.f ? 2u : 0u) |
                              (rounded(v.z, y) > 0.f ? 4u : 0u) | (rounded(v.w, y) > 0.f ? 8u : 0u);
        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)bits, mr_, mask_off(off, ESZ), 0, 0);
      }
    });
    return;
  }
  res_visit<RES_THREADS, K, ESZ, 1>(g, [&](int k, int off, bool) {
    const float4 v = make_float4((xr[k].x - mean) * scale + bt, (xr[k].y - mean) * scale + bt,
                                 (xr[k].z - mean) * scale + bt, (xr[k].w - mean) * scale + bt);
    buf_st4(yr_, off, v, y);
  });
}

__device__ __forceinline__ float4 relu_mask(float4 d, float4 y) {
  return make_float4(y.x > 0.f ? d.x : 0.f, y.y > 0.f ? d.y : 0.f, y.z > 0.f ? d.z : 0.f, y.w > 0.f ? d.w : 0.f);
}
__device__ __forceinline__ float4 relu_bits(float4 d, unsigned bits) {
  return make_float4(bits & 1u ? d.x : 0.f, bits & 2u ? d.y : 0.f, bits & 4u ? d.z : 0.f, bits & 8u ? d.w : 0.f);
}

template <typename T, int RES_THREADS, int K, int FUSE = 0>
__global__ void __launch_bounds__(RES_THREADS)
bn_bwd_resident(BnGeom g, unsigned bytes, int klim, const T* __restrict__ x, const T* __restrict__ dy,
                T* __restrict__ dx, BnBwdArgs a, BnFuseBwd<T> fu = BnFuseBwd<T>{nullptr, nullptr, nullptr}) {
  extern __shared__ float4 dyl[];           // [klim][threads], klim <= min(K, RES_KL)
  __shared__ float red[2 * (RES_THREADS / 64)];
  __shared__ float sh[4];
  constexpr int ESZ = (int)sizeof(T);
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), dyr_ = make_rsrc(dy, bytes),
                               dxr_ = make_rsrc(dx, bytes);
  const long long c = res_feature(g);
  const BnBwdPre pre = bn_preload(a, c);
  const float mean = pre.mean;
  float4 xr[K];
  float s1 = 0.f, s2 = 0.f;
  constexpr bool MASK = FUSE == 2;   // the ReLU mask comes as bytes, not from y
  // Small features (workgroups of 4 waves, or 8 vectors per thread) keep dy in registers as well, at its storage
  // size, and fetch it together with x: in the walk below every vector's loads wait behind the sums of the
  // vector before (the statement that pins the sums orders memory operations too), which the large kernels hide
  // behind their 16 waves and a CU with 4 waves does not - 13 trips to memory one after the other, 10 of the
  // 16 us of a 14x14 layer of 256 features.  Nothing is parked in LDS then, and nothing is read twice.
  constexpr bool REGS = RES_THREADS == 256 || K <= 8;
  constexpr int FB = 4;     // groups of four vectors, or the temporaries of all of them overlap and the registers run out
  Raw4<T> dr[REGS ? K : 1], yw[REGS && FUSE == 1 ? K : 1];
  unsigned mb[REGS && FUSE ? K : 1];
  res_visit<RES_THREADS, K, ESZ, 0>(g, [&](int k, int off, bool) {
    xr[k] = buf_ld4_stream(xr_, off, x);
    if (REGS) {
      dr[REGS ? k : 0] = buf_ld4_raw(dyr_, off, dy);
      if (MASK) mb[REGS && FUSE ? k : 0] = __builtin_amdgcn_raw_buffer_load_b8(mask_rsrc(fu.mask, x, bytes, ESZ), mask_off(off, ESZ), 0, 0);
      else if (FUSE) yw[REGS && FUSE == 1 ? k : 0] = buf_ld4_raw(make_rsrc(fu.y, bytes), off, dy);
    }
  });
  // the gradient of vector k after the mask, from the registers
  auto masked = [&](int k) {
    const float4 d = widen(dr[REGS ? k : 0]);
    return FUSE ? relu_bits(d, mb[REGS && FUSE ? k : 0]) : d;
  };
  res_visit<RES_THREADS, K, ESZ, FB>(g, [&](int k, int off, bool in) {
    float4 d;
    if (REGS) {
      if (FUSE == 1) {
        const float4 yv = widen(yw[REGS && FUSE == 1 ? k : 0]);
        mb[REGS && FUSE ? k : 0] = (yv.x > 0.f ? 1u : 0u) | (yv.y > 0.f ? 2u : 0u) | (yv.z > 0.f ? 4u : 0u) | (yv.w > 0.f ? 8u : 0u);
      }
      d = masked(k);
    } else {
      // dy vectors that stay in LDS are read once; the others come back in the second walk
      d = k < klim ? buf_ld4_stream(dyr_, off, dy) : buf_ld4(dyr_, off, dy);
      if (FUSE) {
        if (MASK) d = relu_bits(d, __builtin_amdgcn_raw_buffer_load_b8(mask_rsrc(fu.mask, x, bytes, ESZ), mask_off(off, ESZ), 0, 0));
        else d = relu_mask(d, k < klim ? buf_ld4_stream(make_rsrc(fu.y, bytes), off, dy) : buf_ld4(make_rsrc(fu.y, bytes), off, dy));
      }
      if (k < klim) dyl[k * RES_THREADS + threadIdx.x] = d;
    }
    const float p1 = (d.x + d.y) + (d.z + d.w);
    const float p2 = (d.x * (xr[k].x - mean) + d.y * (xr[k].y - mean)) +
                     (d.z * (xr[k].z - mean) + d.w * (xr[k].w - mean));
    s1 += in ? p1 : 0.f;
    s2 += in ? p2 : 0.f;
    // both sums are finished per vector: otherwise the second one is sunk below the
    // first block reduction and drags every vector's temporaries along
    asm("" : "+v"(s1), "+v"(s2));
  });
  block_sums<(K <= 16), (K <= 16 ? RES_THREADS / 64 : 0)>(s1, s2, red);
  finish_bwd(g, a, c, (double)s1, (double)s2, true, sh, pre);
  __syncthreads();
  const float kdy = sh[1], kx = sh[2], k0 = sh[3];
  res_visit<RES_THREADS, K, ESZ, FB, true>(g, [&](int k, int off, bool) {
    float4 d = REGS ? masked(k) : k < klim ? dyl[k * RES_THREADS + threadIdx.x] : buf_ld4(dyr_, off, dy);
    // the part of dy that did not fit in LDS passes the mask again (y re-read with it)
    if (!REGS && FUSE && k >= klim) {
      if (MASK) d = relu_bits(d, __builtin_amdgcn_raw_buffer_load_b8(mask_rsrc(fu.mask, x, bytes, ESZ), mask_off(off, ESZ), 0, 0));
      else d = relu_mask(d, buf_ld4(make_rsrc(fu.y, bytes), off, dy));
    }
    const float4 v = make_float4(kdy * d.x + (kx * (xr[k].x - mean) + k0),
                                 kdy * d.y + (kx * (xr[k].y - mean) + k0),
                                 kdy * d.z + (kx * (xr[k].z - mean) + k0),
                                 kdy * d.w + (kx * (xr[k].w - mean) + k0));
    buf_st4(dxr_, off, v, dx);
    if (FUSE && fu.dres) buf_st4(make_rsrc(fu.dres, bytes), off, d, dx);
  });
}

// ---- resident kernels for bf16 storage, eight elements (16 bytes) per slot ----------------
// The same two kernels with the x values kept packed: a register holds two bf16 values, so a
// feature of up to 8 * 25 * 1024 elements stays on chip (56x56 planes at batch 64, which the
// 4-wide kernels above hand to the two-pass path), and every load and store moves 16 bytes
// per lane.  Values are unpacked (a shift / a mask) each time they are used.
__device__ __forceinline__ uint4 buf_ld8(__amdgpu_buffer_rsrc_t r, int byte_off, bool stream) {
  const uintx4_t v = stream ? __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 2)
                            : __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void buf_st8(__amdgpu_buffer_rsrc_t r, int byte_off, uint4 v) {
  const uintx4_t t = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(t, r, byte_off, 0, 2);
}
// (HALF: the two 16-bit values are IEEE halves, else bf16; the kernels below hold either as raw words)
template <bool HALF> __device__ __forceinline__ float bf_lo(uint32_t u) { return HALF ? f16lo(u) : __uint_as_float(u << 16); }
template <bool HALF> __device__ __forceinline__ float bf_hi(uint32_t u) { return HALF ? f16hi(u) : __uint_as_float(u & 0xffff0000u); }
template <bool HALF> __device__ __forceinline__ uint32_t bf_pack(float lo, float hi) {
  if (HALF) return pack_f16(lo, hi);
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}
// keeps the halves of d whose counterpart in y is a positive bf16 value
__device__ __forceinline__ uint32_t relu_mask2(uint32_t d, uint32_t y) {
  const uint32_t lo = (int)(y << 16) > 0 ? 0x0000ffffu : 0u;
  const uint32_t hi = (int)(y & 0xffff0000u) > 0 ? 0xffff0000u : 0u;
  return d & (lo | hi);
}
// Makes the packed values opaque to the optimiser: without it the unpacked floats of one
// walk over the resident vectors are kept alive for the next walk (8 registers per vector)
// instead of being recomputed from the 4 packed ones.
// (not volatile: a volatile statement would also order the loads around it, one vector behind the other)
__device__ __forceinline__ void opaque(uint4& v) { asm("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }
__device__ __forceinline__ uint4 relu_mask8(uint4 d, uint4 y) {
  return make_uint4(relu_mask2(d.x, y.x), relu_mask2(d.y, y.y), relu_mask2(d.z, y.z), relu_mask2(d.w, y.w));
}
// the same from the two mask bytes of the vector: bit e of byte j stands for element 4 j + e
// (bit `at` of b for the low half of the word, bit at + 1 for the high half; the two bits are spread to
// all-ones / zero words with shifts, not with selects: eight selects per vector each want a lane mask in
// scalar registers, and a few vectors' worth of those do not fit)
__device__ __forceinline__ uint32_t relu_bits2(uint32_t d, unsigned b, int at) {
  const uint32_t ml = (uint32_t)((int)(b << (31 - at)) >> 31), mh = (uint32_t)((int)(b << (30 - at)) >> 31);
  return d & ((ml & 0x0000ffffu) | (mh & 0xffff0000u));
}
__device__ __forceinline__ uint4 relu_bits8(uint4 d, unsigned b) {
  return make_uint4(relu_bits2(d.x, b, 0), relu_bits2(d.y, b, 2), relu_bits2(d.z, b, 8), relu_bits2(d.w, b, 10));
}

// A value every lane holds alike, moved to a scalar register (the vector registers of the
// resident kernels are all taken by the held elements).
__device__ __forceinline__ float uniform(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

template <bool HALF, int RES_THREADS, int K, int FUSE = 0, bool RES_EARLY = false>
__global__ void __launch_bounds__(RES_THREADS)
bn_train_resident8(BnGeom g, unsigned bytes, const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                   BnTrainArgs a, BnFuseFwd<bf16_t> fu = BnFuseFwd<bf16_t>{nullptr, 0, nullptr}) {
  __shared__ float red[2 * (RES_THREADS / 64)];
  __shared__ float sh[2];
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), yr_ = make_rsrc(y, bytes);
  const long long c = res_feature(g);
  const float shift = HALF ? f16_to_f32(f16_t{x[(size_t)(c * g.inner)]}) : ld(x, (size_t)(c * g.inner));
  // (the kernels that hold 25 vectors per thread have no registers to keep the scalars through the statistics)
  constexpr bool EARLY = K <= 16;
  BnTrainPre pre = EARLY ? bn_preload(a, c) : BnTrainPre{};
  uint4 xr[K];
  float s1 = 0.f, s2 = 0.f;
  res_visit<RES_THREADS, K, 2, 0, false, 8>(g, [&](int k, int off, bool) { xr[k] = buf_ld8(xr_, off, true); });
  // (RES_EARLY: see bn_train_resident)
  constexpr bool PRE = FUSE && RES_EARLY;
  const __amdgpu_buffer_rsrc_t rr_ = make_rsrc((FUSE && fu.res) ? fu.res : x, (FUSE && fu.res) ? bytes : 0u);
  uint4 rz[PRE ? K : 1];
  if (PRE) res_visit<RES_THREADS, K, 2, 0, false, 8>(g, [&](int k, int off, bool) { rz[k] = buf_ld8(rr_, off, true); });
  res_visit<RES_THREADS, K, 2, 1, false, 8>(g, [&](int k, int, bool in) {
    opaque(xr[k]);
    const uint32_t w[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
    float p1 = 0.f, p2 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float t0 = bf_lo<HALF>(w[j]) - shift, t1 = bf_hi<HALF>(w[j]) - shift;
      p1 += t0 + t1;
      p2 += t0 * t0 + t1 * t1;
    }
    s1 += in ? p1 : 0.f;
    s2 += in ? p2 : 0.f;
    asm("" : "+v"(s1), "+v"(s2));
  });
  block_sums<(K <= 16), (K <= 16 ? RES_THREADS / 64 : 0)>(s1, s2, red);
  finish_stats(g, a, c, shift, (double)s1, (double)s2, true, sh, EARLY ? &pre : nullptr);
  __syncthreads();
  if (!EARLY) pre = bn_preload(a, c, false);
  const float mean = uniform(sh[0]);
  const float scale = uniform(pre.gamma * sh[1]);
  const float bt = uniform(pre.beta);
  const __amdgpu_buffer_rsrc_t mr_ = mask_rsrc(FUSE == 2 ? fu.mask : nullptr, x, bytes, 2);
  const float lo = (FUSE && fu.relu) ? 0.f : -__builtin_huge_valf();
  res_visit<RES_THREADS, K, 2, 1, false, 8>(g, [&](int k, int off, bool) {
    // one 32-bit word (two values) at a time, results written over the packed input: the
    // vector is not needed again
    uint4 v = xr[k];
    opaque(v);
    if (FUSE) {
      const uint4 rv = PRE ? rz[PRE ? k : 0] : buf_ld8(rr_, off, true);      // no residual: the empty range reads zeros
      // (relu leaves no NaN, so the sign tests on the packed words equal y > 0)
      auto pos = [](uint32_t w, unsigned blo, unsigned bhi) {
        return ((int)(w << 16) > 0 ? blo : 0u) | ((int)(w & 0xffff0000u) > 0 ? bhi : 0u);
      };
      v.x = bf_pack<HALF>(fmaxf((bf_lo<HALF>(v.x) - mean) * scale + bt + bf_lo<HALF>(rv.x), lo), fmaxf((bf_hi<HALF>(v.x) - mean) * scale + bt + bf_hi<HALF>(rv.x), lo));
      unsigned bits = pos(v.x, 1u, 2u);
      __builtin_amdgcn_sched_barrier(0);   // one word at a time: the packing temporaries of all four do not fit
      v.y = bf_pack<HALF>(fmaxf((bf_lo<HALF>(v.y) - mean) * scale + bt + bf_lo<HALF>(rv.y), lo), fmaxf((bf_hi<HALF>(v.y) - mean) * scale + bt + bf_hi<HALF>(rv.y), lo));
      bits |= pos(v.y, 4u, 8u);
      __builtin_amdgcn_sched_barrier(0);
      v.z = bf_pack<HALF>(fmaxf((bf_lo<HALF>(v.z) - mean) * scale + bt + bf_lo<HALF>(rv.z), lo), fmaxf((bf_hi<HALF>(v.z) - mean) * scale + bt + bf_hi<HALF>(rv.z), lo));
      bits |= pos(v.z, 0x100u, 0x200u);
      __builtin_amdgcn_sched_barrier(0);
      v.w = bf_pack<HALF>(fmaxf((bf_lo<HALF>(v.w) - mean) * scale + bt + bf_lo<HALF>(rv.w), lo), fmaxf((bf_hi<HALF>(v.w) - mean) * scale + bt + bf_hi<HALF>(rv.w), lo));
      bits |= pos(v.w, 0x400u, 0x800u);
      // two mask bytes per vector (8 elements)
      if (FUSE == 2) __builtin_amdgcn_raw_buffer_store_b16((uint16_t)bits, mr_, mask_off(off, 2), 0, 0);
    } else {
      v.x = bf_pack<HALF>((bf_lo<HALF>(v.x) - mean) * scale + bt, (bf_hi<HALF>(v.x) - mean) * scale + bt);
      v.y = bf_pack<HALF>((bf_lo<HALF>(v.y) - mean) * scale + bt, (bf_hi<HALF>(v.y) - mean) * scale + bt);
      v.z = bf_pack<HALF>((bf_lo<HALF>(v.z) - mean) * scale + bt, (bf_hi<HALF>(v.z) - mean) * scale + bt);
      v.w = bf_pack<HALF>((bf_lo<HALF>(v.w) - mean) * scale + bt, (bf_hi<HALF>(v.w) - mean) * scale + bt);
    }
    buf_st8(yr_, off, v);
  });
}

template <bool HALF, int RES_THREADS, int K, int FUSE = 0>
__global__ void __launch_bounds__(RES_THREADS)
bn_bwd_resident8(BnGeom g, unsigned bytes, int klim, const bf16_t* __restrict__ x, const bf16_t* __restrict__ dy,
                 bf16_t* __restrict__ dx, BnBwdArgs a, BnFuseBwd<bf16_t> fu = BnFuseBwd<bf16_t>{nullptr, nullptr, nullptr}) {
  extern __shared__ uint4 dyl8[];           // [klim][threads] packed gradients (after the mask)
  __shared__ float red[2 * (RES_THREADS / 64)];
  __shared__ float sh[4];
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), dyr_ = make_rsrc(dy, bytes),
                               dxr_ = make_rsrc(dx, bytes);
  const __amdgpu_buffer_rsrc_t yr_ = make_rsrc((FUSE && fu.y) ? fu.y : x, (FUSE && fu.y) ? bytes : 0u);
  const __amdgpu_buffer_rsrc_t mr_ = mask_rsrc(FUSE == 2 ? fu.mask : nullptr, x, bytes, 2);
  const __amdgpu_buffer_rsrc_t drr_ = make_rsrc((FUSE && fu.dres) ? fu.dres : dx, (FUSE && fu.dres) ? bytes : 0u);
  const long long c = res_feature(g);
  const BnBwdPre pre = bn_preload(a, c);
  const float mean = pre.mean;
  uint4 xr[K];
  float s1 = 0.f, s2 = 0.f;
  constexpr bool MASK = FUSE == 2;   // the ReLU mask comes as bytes, not from y
  // (REGS: small features keep dy in registers and fetch it together with x - see bn_bwd_resident)
  constexpr bool REGS = RES_THREADS == 256 || K <= 8;
  constexpr int FB = 4;
  uint4 dr[REGS ? K : 1], yw[REGS && FUSE == 1 ? K : 1];
  unsigned mb[REGS && MASK ? K : 1];
  res_visit<RES_THREADS, K, 2, 0, false, 8>(g, [&](int k, int off, bool) {
    xr[k] = buf_ld8(xr_, off, true);
    if (REGS) {
      dr[REGS ? k : 0] = buf_ld8(dyr_, off, true);
      if (MASK) mb[REGS && MASK ? k : 0] = __builtin_amdgcn_raw_buffer_load_b16(mr_, mask_off(off, 2), 0, 0);
      else if (FUSE) yw[REGS && FUSE == 1 ? k : 0] = buf_ld8(yr_, off, true);
    }
  });
  res_visit<RES_THREADS, K, 2, FB, false, 8>(g, [&](int k, int off, bool in) {
    uint4 d;
    if (REGS) {
      opaque(dr[REGS ? k : 0]);      // (or the widening of all vectors is hoisted to where they arrive)
      d = dr[REGS ? k : 0];
      if (MASK) d = relu_bits8(d, mb[REGS && MASK ? k : 0]);
      else if (FUSE) d = relu_mask8(d, yw[REGS && FUSE == 1 ? k : 0]);
      dr[REGS ? k : 0] = d;          // kept with the mask applied
    } else {
      d = buf_ld8(dyr_, off, k < klim);
      if (FUSE) {
        if (MASK) d = relu_bits8(d, __builtin_amdgcn_raw_buffer_load_b16(mr_, mask_off(off, 2), 0, 0));
        else d = relu_mask8(d, buf_ld8(yr_, off, k < klim));
      }
      if (k < klim) dyl8[k * RES_THREADS + threadIdx.x] = d;
    }
    opaque(xr[k]);
    const uint32_t dw[4] = {d.x, d.y, d.z, d.w}, xw[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
    float p1 = 0.f, p2 = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float d0 = bf_lo<HALF>(dw[j]), d1 = bf_hi<HALF>(dw[j]);
      p1 += d0 + d1;
      p2 += d0 * (bf_lo<HALF>(xw[j]) - mean) + d1 * (bf_hi<HALF>(xw[j]) - mean);
    }
    s1 += in ? p1 : 0.f;
    s2 += in ? p2 : 0.f;
    asm("" : "+v"(s1), "+v"(s2));
  });
  block_sums<(K <= 16), (K <= 16 ? RES_THREADS / 64 : 0)>(s1, s2, red);
  finish_bwd(g, a, c, (double)s1, (double)s2, true, sh, pre);
  __syncthreads();
  const float kdy = sh[1], kx = sh[2], k0 = sh[3];
  res_visit<RES_THREADS, K, 2, FB, true, 8>(g, [&](int k, int off, bool) {
    if (REGS) opaque(dr[REGS ? k : 0]);
    uint4 d = REGS ? dr[REGS ? k : 0] : k < klim ? dyl8[k * RES_THREADS + threadIdx.x] : buf_ld8(dyr_, off, false);
    if (!REGS && FUSE && k >= klim) {
      if (MASK) d = relu_bits8(d, __builtin_amdgcn_raw_buffer_load_b16(mr_, mask_off(off, 2), 0, 0));
      else d = relu_mask8(d, buf_ld8(yr_, off, false));
    }
    opaque(xr[k]);
    const uint32_t dw[4] = {d.x, d.y, d.z, d.w}, xw[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = bf_pack<HALF>(kdy * bf_lo<HALF>(dw[j]) + (kx * (bf_lo<HALF>(xw[j]) - mean) + k0),
                     kdy * bf_hi<HALF>(dw[j]) + (kx * (bf_hi<HALF>(xw[j]) - mean) + k0));
    buf_st8(dxr_, off, make_uint4(o[0], o[1], o[2], o[3]));
    if (FUSE) buf_st8(drr_, off, d);               // no residual branch: the empty range drops the store
  });
}

// ---- resident kernels for rows that are not 16-byte friendly (inner % 4 != 0) -----------
// Same idea with one element per slot: a workgroup owns a feature, a thread holds K
// elements of x (and, backward, of dy) in registers, lanes walk consecutive elements so
// a wave's load is a contiguous run.  Forward moves 2T bytes, backward exactly 3T.
__device__ __forceinline__ void buf_st(__amdgpu_buffer_rsrc_t r, int byte_off, float v, float*) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st(__amdgpu_buffer_rsrc_t r, int byte_off, float v, bf16_t*) {
  __builtin_amdgcn_raw_buffer_store_b16(f32_to_bf16(v), r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st(__amdgpu_buffer_rsrc_t r, int byte_off, float v, f16_t*) {
  __builtin_amdgcn_raw_buffer_store_b16(f32_to_f16(v).bits, r, byte_off, 0, 0);
}

// byte offsets of this thread's elements e = tid + THREADS*k of feature blockIdx.x;
// out-of-range slots get an offset past the descriptor (loads give 0, stores are dropped)
template <int THREADS, int K, int ESZ>
__device__ __forceinline__ void res1_offsets(const BnGeom& g, int (&off)[K]) {
  constexpr int OOB = (int)0x80000000;
  const int inner = (int)g.inner, c = res_feature(g);
  int q = threadIdx.x;
  int o = q / inner, i = q - o * inner;
  const int so = THREADS / inner, si = THREADS - so * inner;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    off[k] = q < (int)g.units ? ((o * (int)g.C + c) * inner + i) * ESZ : OOB;
    q += THREADS;
    o += so;
    i += si;
    if (i >= inner) {
      i -= inner;
      ++o;
    }
  }
}

template <typename T, int THREADS, int K, int FUSE = 0>
__global__ void __launch_bounds__(THREADS)
bn_train_resident1(BnGeom g, unsigned bytes, const T* __restrict__ x, T* __restrict__ y,
                   BnTrainArgs a, BnFuseFwd<T> fu = BnFuseFwd<T>{nullptr, 0, nullptr}) {
  __shared__ float red[2 * (THREADS / 64)];
  __shared__ float sh[2];
  constexpr int OOB = (int)0x80000000;
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), yr_ = make_rsrc(y, bytes);
  const long long c = res_feature(g);
  const float shift = ld(x, (size_t)(c * g.inner));
  // (the kernels that hold 25 vectors per thread have no registers to keep the scalars through the statistics)
  constexpr bool EARLY = K <= 16;
  BnTrainPre pre = EARLY ? bn_preload(a, c) : BnTrainPre{};
  int off[K];
  res1_offsets<THREADS, K, (int)sizeof(T)>(g, off);
  float xv[K];
#pragma unroll
  for (int k = 0; k < K; ++k) xv[k] = buf_ld(xr_, off[k], x);
  // the residual comes with x: fetched after the statistics it would add a trip to memory
  const __amdgpu_buffer_rsrc_t rr_ = make_rsrc((FUSE && fu.res) ? fu.res : x, (FUSE && fu.res) ? bytes : 0u);   // no residual: loads give 0
  float rv[FUSE ? K : 1];
  if (FUSE && EARLY) {
#pragma unroll
    for (int k = 0; k < K; ++k) rv[k] = buf_ld(rr_, off[k], x);
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const float t = off[k] != OOB ? xv[k] - shift : 0.f;
    s1 += t;
    s2 += t * t;
  }
  block_sums<(K <= 16), (K <= 16 ? THREADS / 64 : 0)>(s1, s2, red);
  finish_stats(g, a, c, shift, (double)s1, (double)s2, true, sh, EARLY ? &pre : nullptr);
  __syncthreads();
  if (!EARLY) pre = bn_preload(a, c, false);
  const float mean = sh[0];
  const float scale = pre.gamma * sh[1];
  const float bt = pre.beta;
  if (FUSE) {
    const float lo = fu.relu ? 0.f : -__builtin_huge_valf();
    if (!EARLY) {
#pragma unroll
      for (int k = 0; k < K; ++k) rv[k] = buf_ld(rr_, off[k], x);
    }
#pragma unroll
    for (int k = 0; k < K; ++k) buf_st(yr_, off[k], fmaxf((xv[k] - mean) * scale + bt + rv[k], lo), y);
    return;
  }
#pragma unroll
  for (int k = 0; k < K; ++k) buf_st(yr_, off[k], (xv[k] - mean) * scale + bt, y);
}

template <typename T, int THREADS, int K, int FUSE = 0>
__global__ void __launch_bounds__(THREADS)
bn_bwd_resident1(BnGeom g, unsigned bytes, const T* __restrict__ x, const T* __restrict__ dy,
                 T* __restrict__ dx, BnBwdArgs a, BnFuseBwd<T> fu = BnFuseBwd<T>{nullptr, nullptr, nullptr}) {
  __shared__ float red[2 * (THREADS / 64)];
  __shared__ float sh[4];
  const __amdgpu_buffer_rsrc_t xr_ = make_rsrc(x, bytes), dyr_ = make_rsrc(dy, bytes),
                               dxr_ = make_rsrc(dx, bytes);
  const long long c = res_feature(g);
  const BnBwdPre pre = bn_preload(a, c);
  const float mean = pre.mean;
  int off[K];
  res1_offsets<THREADS, K, (int)sizeof(T)>(g, off);
  float xv[K], dv[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    xv[k] = buf_ld(xr_, off[k], x);
    dv[k] = buf_ld(dyr_, off[k], dy);
  }
  if (FUSE) {
    const __amdgpu_buffer_rsrc_t yr_ = make_rsrc(fu.y, bytes);
#pragma unroll
    for (int k = 0; k < K; ++k) dv[k] = buf_ld(yr_, off[k], dy) > 0.f ? dv[k] : 0.f;
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    // out-of-range slots loaded zeros for dy, so they add nothing
    s1 += dv[k];
    s2 += dv[k] * (xv[k] - mean);
  }
  block_sums<(K <= 16), (K <= 16 ? THREADS / 64 : 0)>(s1, s2, red);
  finish_bwd(g, a, c, (double)s1, (double)s2, true, sh, pre);
  __syncthreads();
  const float kdy = sh[1], kx = sh[2], k0 = sh[3];
#pragma unroll
  for (int k = 0; k < K; ++k) buf_st(dxr_, off[k], kdy * dv[k] + (kx * (xv[k] - mean) + k0), dx);
  if (FUSE && fu.dres) {
    const __amdgpu_buffer_rsrc_t rr_ = make_rsrc(fu.dres, bytes);
#pragma unroll
    for (int k = 0; k < K; ++k) buf_st(rr_, off[k], dv[k], dx);
  }
}

// ---- column mode (inner == 1) ----------------------------------------------
// block = 64 features x 4 row lanes; grid = (ceil(C/64), S); slice s owns rows
// [s*ups, (s+1)*ups).
template <typename T, bool BWD>
__global__ void __launch_bounds__(256)
bn_stats_col(BnGeom g, const T* __restrict__ x, const T* __restrict__ dy,
             const float* __restrict__ save_mean, float* __restrict__ ws) {
  __shared__ float red[2][4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const long long c = (long long)blockIdx.x * 64 + tx;
  const long long r0 = (long long)blockIdx.y * g.ups, r1 = min(r0 + g.ups, g.outer);
  float s1 = 0.f, s2 = 0.f;
  if (c < g.C) {
    const float ref = BWD ? save_mean[c] : ld(x, (size_t)c);
    for (long long r = r0 + ty; r < r1; r += 4) {
      const size_t off = (size_t)(r * g.C + c);
      if (BWD) {
        const float d = ld(dy, off);
        s1 += d;
        s2 += d * (ld(x, off) - ref);
      } else {
        const float t = ld(x, off) - ref;
        s1 += t;
        s2 += t * t;
      }
    }
  }
  red[0][ty][tx] = s1;
  red[1][ty][tx] = s2;
  __syncthreads();
  if (ty == 0 && c < g.C) {
    ws[(c * g.S + blockIdx.y) * 2 + 0] = (red[0][0][tx] + red[0][1][tx]) + (red[0][2][tx] + red[0][3][tx]);
    ws[(c * g.S + blockIdx.y) * 2 + 1] = (red[1][0][tx] + red[1][1][tx]) + (red[1][2][tx] + red[1][3][tx]);
  }
}

// Per-feature coefficients for the column apply kernels: out = k1*in1 + k2*(x-mean) + k0.
// One thread per feature folds the partials serially (S is small).
template <typename T>
__global__ void __launch_bounds__(256)
bn_train_apply_col(BnGeom g, const T* __restrict__ x, T* __restrict__ y,
                   const float* __restrict__ ws, BnTrainArgs a) {
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const long long c = (long long)blockIdx.x * 64 + tx;
  if (c >= g.C) return;
  double p0 = 0.0, p1 = 0.0;
  for (int s = 0; s < g.S; ++s) {
    p0 += (double)ws[(c * g.S + s) * 2 + 0];
    p1 += (double)ws[(c * g.S + s) * 2 + 1];
  }
  const double M = (double)g.outer;
  const double m1 = p0 / M;
  double var = p1 / M - m1 * m1;
  if (var < 0.0) var = 0.0;
  const double mean = (double)ld(x, (size_t)c) + m1;
  const double invstd = 1.0 / sqrt(var + a.eps);
  if (blockIdx.y == 0 && ty == 0) {
    if (a.save_mean) a.save_mean[c] = (float)mean;
    if (a.save_invstd) a.save_invstd[c] = (float)invstd;
    if (a.run_mean && a.run_var) {
      if (a.momentum == 0.0) {
        a.run_mean[c] = (float)mean;
        a.run_var[c] = (float)var;
      } else {
        const double unb = M > 1.0 ? var * M / (M - 1.0) : var;
        a.run_mean[c] = (float)((1.0 - a.momentum) * (double)a.run_mean[c] + a.momentum * mean);
        a.run_var[c] = (float)((1.0 - a.momentum) * (double)a.run_var[c] + a.momentum * unb);
      }
    }
  }
  const float fm = (float)mean;
  const float scale = (a.gamma ? a.gamma[c] : 1.f) * (float)invstd;
  const float bt = a.beta ? a.beta[c] : 0.f;
  const long long r0 = (long long)blockIdx.y * g.ups, r1 = min(r0 + g.ups, g.outer);
  for (long long r = r0 + ty; r < r1; r += 4) {
    const size_t off = (size_t)(r * g.C + c);
    st(y, off, (ld(x, off) - fm) * scale + bt);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
bn_bwd_apply_col(BnGeom g, const T* __restrict__ x, const T* __restrict__ dy,
                 T* __restrict__ dx, const float* __restrict__ ws, BnBwdArgs a) {
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const long long c = (long long)blockIdx.x * 64 + tx;
  if (c >= g.C) return;
  double p0 = 0.0, p1 = 0.0;
  for (int s = 0; s < g.S; ++s) {
    p0 += (double)ws[(c * g.S + s) * 2 + 0];
    p1 += (double)ws[(c * g.S + s) * 2 + 1];
  }
  const double M = (double)g.outer;
  const double is = (double)a.save_invstd[c];
  const double gm = a.gamma ? (double)a.gamma[c] : 1.0;
  const float mean = a.save_mean[c];
  const float kdy = (float)(gm * is), kx = (float)(-gm * is * is * is * p1 / M),
              k0 = (float)(-gm * is * p0 / M);
  if (blockIdx.y == 0 && ty == 0) {
    if (a.dgamma) a.dgamma[c] = (float)(p1 * is);
    if (a.dbeta) a.dbeta[c] = (float)p0;
  }
  const long long r0 = (long long)blockIdx.y * g.ups, r1 = min(r0 + g.ups, g.outer);
  for (long long r = r0 + ty; r < r1; r += 4) {
    const size_t off = (size_t)(r * g.C + c);
    st(dx, off, kdy * ld(dy, off) + (kx * (ld(x, off) - mean) + k0));
  }
}

// ---- inference ---------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
bn_infer_kernel(BnGeom g, const T* __restrict__ x, T* __restrict__ y,
                const float* __restrict__ gamma, const float* __restrict__ beta,
                const float* __restrict__ mean, const float* __restrict__ var, float eps,
                size_t total) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const long long c = (long long)((e / (size_t)g.inner) % (size_t)g.C);
    const float is = 1.0f / sqrtf(var[c] + eps);
    const float gm = gamma ? gamma[c] : 1.f, bt = beta ? beta[c] : 0.f;
    st(y, e, (ld(x, e) - mean[c]) * (gm * is) + bt);
  }
}

// ---- host side ---------------------------------------------------------------
static int make_geom(const flhip_bn_desc* d, BnGeom* g, int* vec) {
  FLHIP_REQUIRE(d, "batchnorm: null descriptor");
  FLHIP_REQUIRE(d->outer > 0 && d->C > 0 && d->inner > 0, "batchnorm: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(d->dtype), "batchnorm: unknown dtype");
  g->outer = d->outer;
  g->C = d->C;
  g->inner = d->inner;
  if (d->inner == 1) {
    *vec = 0;
    const long long cb = (d->C + 63) / 64;
    FLHIP_REQUIRE(cb <= 0x7fffffffLL, "batchnorm: too many features");
    long long S = 4096 / cb;
    const long long maxS = (d->outer + 3) / 4;
    if (S > maxS) S = maxS;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    g->S = (int)S;
    g->units = d->outer;
    g->ups = (g->units + S - 1) / S;
    g->step_o = g->step_i = 0;
  } else {
    FLHIP_REQUIRE(d->C <= 0x7fffffffLL, "batchnorm: too many features");
    *vec = (d->inner % 4 == 0) ? 4 : 1;
    const long long innerV = d->inner / *vec;
    g->units = d->outer * innerV;
    long long S = 8192 / d->C;
    const long long maxS = (g->units + 511) / 512;
    if (S > maxS) S = maxS;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    g->S = (int)S;
    g->ups = (g->units + S - 1) / S;
    g->step_o = (int)(256 / innerV);
    g->step_i = (int)(256 % innerV);
  }
  return FLHIP_OK;
}

// Shape of the resident kernels for this geometry: threads per workgroup and
// vectors per thread; threads = 0 when they do not apply.  FLHIP_BN_ALGO=split
// forces the two-kernel path, =resident lifts the feature-count threshold
// (measurement aids).
struct ResPlan {
  int threads, k, need;
};
#ifndef BN_SMALL_K
#define BN_SMALL_K 16
#endif
static ResPlan resident_plan(const BnGeom& g, int vec, int min_c) {
  const int mode = options().bn_algo;
  ResPlan r{0, 0, 0};
  if (mode == 1 || vec == 0) return r;
  if (vec == 1) {
    // element-wise variant: up to 32 elements per thread
    if (g.units > 32 * 1024 || g.inner > 0x7fffffff) return r;
    if (g.outer * g.C * g.inner * 4 >= (1ll << 31)) return r;
    if (mode != 2 && g.C < min_c) return r;
    // short rows: workgroups of 4 waves (more of them per CU, cheaper barriers, more loads in
    // flight per thread) as long as a thread holds at most 16 elements
    r.threads = g.units <= BN_SMALL_K * 256 ? 256 : 1024;
    const int need = (int)((g.units + r.threads - 1) / r.threads);
    r.k = need <= 8 ? 8 : need <= 16 ? 16 : 32;
    r.need = need;
    return r;
  }
  if (g.units > (long long)RES_KMAX * 1024) return r;
  if (g.outer * g.C * g.inner * 4 >= (1ll << 31)) return r;   // 32-bit buffer offsets
  if (mode != 2 && g.C < min_c) return r;
  if (g.units <= BN_SMALL_K * 256) {
    r.threads = 256;
    r.k = g.units <= 8 * 256 ? 8 : 16;
  } else {
    r.threads = 1024;
    const int need = (int)((g.units + 1023) / 1024);
    r.k = need <= 8 ? 8 : need <= 16 ? 16 : RES_KMAX;
  }
  r.need = (int)((g.units + r.threads - 1) / r.threads);
  return r;
}

// bf16 storage, rows of a multiple of 8 elements: shape of the 8-wide resident kernels
// (threads = 0: they do not apply)
static ResPlan resident8_plan(const BnGeom& g, int vec, int dtype, int min_c) {
  ResPlan r{0, 0, 0};
  const int mode = options().bn_algo;
  if (mode == 1 || vec != 4 || !is_lo16(dtype) || g.inner % 8 != 0) return r;
  const long long units8 = g.units / 2;
  if (units8 > (long long)RES_KMAX * 1024) return r;
  if (g.outer * g.C * g.inner * 2 >= (1ll << 31)) return r;   // 32-bit buffer offsets
  if (mode != 2 && g.C < min_c) return r;
  // fewer than 128 features of more than 16 vectors per thread (64 features of 56x56 planes at batch
  // 64): the 64 workgroups of a quarter-full chip lose to the two-pass kernels (28.7 against 21.6 us)
  if (mode != 2 && g.C < 128 && units8 > 16 * 1024) return r;
  if (units8 <= BN_SMALL_K * 256) {
    r.threads = 256;
    r.k = units8 <= 8 * 256 ? 8 : 16;
  } else {
    r.threads = 1024;
    const int need = (int)((units8 + 1023) / 1024);
    r.k = need <= 8 ? 8 : need <= 16 ? 16 : RES_KMAX;
  }
  r.need = (int)((units8 + r.threads - 1) / r.threads);
  return r;
}

template <bool HALF, int THREADS, int K, int FUSE>
static int launch_train_resident8(const BnGeom& g, const bf16_t* x, bf16_t* y, const BnTrainArgs& a,
                                  const BnFuseFwd<bf16_t>& fu, hipStream_t s) {
  const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * 2);
  if (FUSE && THREADS == 256 && g.C <= 2 * mfma_num_cus())
    hipLaunchKernelGGL((bn_train_resident8<HALF, THREADS, K, FUSE, (FUSE && THREADS == 256)>), dim3((unsigned)g.C), dim3(THREADS), 0, s, g,
                       bytes, x, y, a, fu);
  else
    hipLaunchKernelGGL((bn_train_resident8<HALF, THREADS, K, FUSE>), dim3((unsigned)g.C), dim3(THREADS), 0, s, g, bytes, x, y,
                       a, fu);
  return check_launch("bn_fwd_train (resident, 8-wide)");
}

template <bool HALF, int THREADS, int K, int FUSE>
static int launch_bwd_resident8(const BnGeom& g, int need, const bf16_t* x, const bf16_t* dy, bf16_t* dx,
                                const BnBwdArgs& a, const BnFuseBwd<bf16_t>& fu, hipStream_t s) {
  constexpr int KL = K < RES_KL ? K : RES_KL;
  constexpr size_t max_shmem = (size_t)KL * THREADS * sizeof(uint4);
  auto kernel = bn_bwd_resident8<HALF, THREADS, K, FUSE>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)max_shmem);
  if (attr != hipSuccess)
    return fail(FLHIP_RUNTIME_ERROR, std::string("bn_bwd: LDS limit: ") + hipGetErrorString(attr));
  const int klim = need < KL ? need : KL;
  const size_t shmem = (THREADS == 256 || K <= 8) ? 0 : (size_t)klim * THREADS * sizeof(uint4);   // (small features: dy in registers)
  const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * 2);
  hipLaunchKernelGGL(kernel, dim3((unsigned)g.C), dim3(THREADS), shmem, s, g, bytes, klim, x, dy, dx, a, fu);
  return check_launch("bn_bwd (resident, 8-wide)");
}

template <bool HALF, int FUSE>
static int run_train8(const BnGeom& g, const ResPlan& r, const bf16_t* x, bf16_t* y, const BnTrainArgs& a,
                      const BnFuseFwd<bf16_t>& fu, hipStream_t s) {
  if (r.threads == 256 && r.k == 8) return launch_train_resident8<HALF, 256, 8, FUSE>(g, x, y, a, fu, s);
  if (r.threads == 256) return launch_train_resident8<HALF, 256, 16, FUSE>(g, x, y, a, fu, s);
  if (r.k == 8) return launch_train_resident8<HALF, 1024, 8, FUSE>(g, x, y, a, fu, s);
  if (r.k == 16) return launch_train_resident8<HALF, 1024, 16, FUSE>(g, x, y, a, fu, s);
  return launch_train_resident8<HALF, 1024, RES_KMAX, FUSE>(g, x, y, a, fu, s);
}
template <bool HALF, int FUSE>
static int run_bwd8(const BnGeom& g, const ResPlan& r, const bf16_t* x, const bf16_t* dy, bf16_t* dx,
                    const BnBwdArgs& a, const BnFuseBwd<bf16_t>& fu, hipStream_t s) {
  if (r.threads == 256 && r.k == 8) return launch_bwd_resident8<HALF, 256, 8, FUSE>(g, r.need, x, dy, dx, a, fu, s);
  if (r.threads == 256) return launch_bwd_resident8<HALF, 256, 16, FUSE>(g, r.need, x, dy, dx, a, fu, s);
  if (r.k == 8) return launch_bwd_resident8<HALF, 1024, 8, FUSE>(g, r.need, x, dy, dx, a, fu, s);
  if (r.k == 16) return launch_bwd_resident8<HALF, 1024, 16, FUSE>(g, r.need, x, dy, dx, a, fu, s);
  return launch_bwd_resident8<HALF, 1024, RES_KMAX, FUSE>(g, r.need, x, dy, dx, a, fu, s);
}

template <typename T, int THREADS, int K, int FUSE>
static int launch_train_resident(const BnGeom& g, const T* x, T* y, const BnTrainArgs& a,
                                 const BnFuseFwd<T>& fu, hipStream_t s) {
  const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * (long long)sizeof(T));
  if (FUSE && THREADS == 256 && g.C <= 2 * mfma_num_cus())
    hipLaunchKernelGGL((bn_train_resident<T, THREADS, K, FUSE, (FUSE && THREADS == 256)>), dim3((unsigned)g.C), dim3(THREADS), 0,
                       s, g, bytes, x, y, a, fu);
  else
    hipLaunchKernelGGL((bn_train_resident<T, THREADS, K, FUSE>), dim3((unsigned)g.C), dim3(THREADS), 0, s,
                       g, bytes, x, y, a, fu);
  return check_launch("bn_fwd_train (resident)");
}

template <typename T, int THREADS, int K, int FUSE>
static int launch_bwd_resident(const BnGeom& g, int need, const T* x, const T* dy, T* dx,
                               const BnBwdArgs& a, const BnFuseBwd<T>& fu, hipStream_t s) {
  constexpr int KL = K < RES_KL ? K : RES_KL;
  constexpr size_t max_shmem = (size_t)KL * THREADS * sizeof(float4);
  auto kernel = bn_bwd_resident<T, THREADS, K, FUSE>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
      (int)max_shmem);
  if (attr != hipSuccess)
    return fail(FLHIP_RUNTIME_ERROR, std::string("bn_bwd: LDS limit: ") + hipGetErrorString(attr));
  // dy vectors per thread parked in LDS: all of them when the feature is small
  const int klim = need < KL ? need : KL;
  const size_t shmem = (THREADS == 256 || K <= 8) ? 0 : (size_t)klim * THREADS * sizeof(float4);   // (small features: dy in registers)
  const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * (long long)sizeof(T));
  hipLaunchKernelGGL(kernel, dim3((unsigned)g.C), dim3(THREADS), shmem, s, g, bytes, klim, x, dy,
                     dx, a, fu);
  return check_launch("bn_bwd (resident)");
}

// FUSE: with the epilogue y = relu(bn(x) + residual) (segment modes only); 2: the ReLU's mask is also
// written as bytes
template <typename T, int FUSE>
static int run_train(const BnGeom& g, int vec, const void* x, void* y, float* ws,
                     const BnTrainArgs& a, const BnFuseFwd<T>& fu, hipStream_t s) {
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  constexpr int F1 = FUSE == 2 ? 1 : FUSE;   // element-wise kernels: no mask-byte form (never asked for: vec == 4 only)
  if (sizeof(T) == 2) {          // (bf16 and f16: the same kernels on raw 16-bit words, the arithmetic by type)
    const ResPlan r8 = resident8_plan(g, vec, FLHIP_BF16, RES_MIN_C_FWD);
    if (r8.threads)
      return run_train8<std::is_same<T, f16_t>::value, FUSE>(g, r8, reinterpret_cast<const bf16_t*>(xp), reinterpret_cast<bf16_t*>(yp), a,
                              reinterpret_cast<const BnFuseFwd<bf16_t>&>(fu), s);
  }
  {
    const ResPlan r = resident_plan(g, vec, RES_MIN_C_FWD);
    if (vec == 1 && r.threads) {
      const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * (long long)sizeof(T));
      const dim3 grid((unsigned)g.C);
      if (r.threads == 256 && r.k == 8)
        hipLaunchKernelGGL((bn_train_resident1<T, 256, 8, F1>), grid, dim3(256), 0, s, g, bytes, xp, yp, a, fu);
      else if (r.threads == 256)
        hipLaunchKernelGGL((bn_train_resident1<T, 256, 16, F1>), grid, dim3(256), 0, s, g, bytes, xp, yp, a, fu);
      else if (r.k == 8)
        hipLaunchKernelGGL((bn_train_resident1<T, 1024, 8, F1>), grid, dim3(1024), 0, s, g, bytes, xp, yp, a, fu);
      else if (r.k == 16)
        hipLaunchKernelGGL((bn_train_resident1<T, 1024, 16, F1>), grid, dim3(1024), 0, s, g, bytes, xp, yp, a, fu);
      else
        hipLaunchKernelGGL((bn_train_resident1<T, 1024, 32, F1>), grid, dim3(1024), 0, s, g, bytes, xp, yp, a, fu);
      return check_launch("bn_fwd_train (resident, element-wise)");
    }
    if (r.threads == 256 && r.k == 8) return launch_train_resident<T, 256, 8, FUSE>(g, xp, yp, a, fu, s);
    if (r.threads == 256) return launch_train_resident<T, 256, 16, FUSE>(g, xp, yp, a, fu, s);
    if (r.threads == 1024) {
      if (r.k == 8) return launch_train_resident<T, 1024, 8, FUSE>(g, xp, yp, a, fu, s);
      if (r.k == 16) return launch_train_resident<T, 1024, 16, FUSE>(g, xp, yp, a, fu, s);
      return launch_train_resident<T, 1024, RES_KMAX, FUSE>(g, xp, yp, a, fu, s);
    }
  }
  if (vec == 0) {
    if (FUSE) return fail(FLHIP_INVALID_ARGUMENT, "bn_act: per-activation mode (inner == 1) has no fused kernels");
    const dim3 grid((unsigned)((g.C + 63) / 64), g.S);
    hipLaunchKernelGGL((bn_stats_col<T, false>), grid, dim3(256), 0, s, g, xp, (const T*)nullptr,
                       (const float*)nullptr, ws);
    hipLaunchKernelGGL((bn_train_apply_col<T>), grid, dim3(256), 0, s, g, xp, yp, ws, a);
  } else {
    const dim3 grid((unsigned)g.C, g.S);
    if (vec == 4) {
      hipLaunchKernelGGL((bn_stats_seg<T, 4>), grid, dim3(256), 0, s, g, xp, ws);
      hipLaunchKernelGGL((bn_train_apply_seg<T, 4, FUSE>), grid, dim3(256), 0, s, g, xp, yp, ws, a, fu);
    } else {
      hipLaunchKernelGGL((bn_stats_seg<T, 1>), grid, dim3(256), 0, s, g, xp, ws);
      hipLaunchKernelGGL((bn_train_apply_seg<T, 1, F1>), grid, dim3(256), 0, s, g, xp, yp, ws, a, fu);
    }
  }
  return check_launch("bn_fwd_train");
}

// FUSE: the gradient first passes the ReLU mask of the forward result, read from y (1) or from the mask bytes (2)
template <typename T, int FUSE>
static int run_bwd(const BnGeom& g, int vec, const void* x, const void* dy, void* dx, float* ws,
                   const BnBwdArgs& a, const BnFuseBwd<T>& fu, hipStream_t s) {
  const T* xp = static_cast<const T*>(x);
  const T* dyp = static_cast<const T*>(dy);
  T* dxp = static_cast<T*>(dx);
  constexpr int F1 = FUSE == 2 ? 1 : FUSE;   // element-wise kernels: no mask-byte form (never asked for: vec == 4 only)
  if (sizeof(T) == 2) {
    const ResPlan r8 = resident8_plan(g, vec, FLHIP_BF16, RES_MIN_C_BWD);
    if (r8.threads)
      return run_bwd8<std::is_same<T, f16_t>::value, FUSE>(g, r8, reinterpret_cast<const bf16_t*>(xp), reinterpret_cast<const bf16_t*>(dyp),
                            reinterpret_cast<bf16_t*>(dxp), a, reinterpret_cast<const BnFuseBwd<bf16_t>&>(fu), s);
  }
  {
    const ResPlan r = resident_plan(g, vec, RES_MIN_C_BWD);
    if (vec == 1 && r.threads) {
      const unsigned bytes = (unsigned)(g.outer * g.C * g.inner * (long long)sizeof(T));
      const dim3 grid((unsigned)g.C);
      if (r.threads == 256 && r.k == 8)
        hipLaunchKernelGGL((bn_bwd_resident1<T, 256, 8, F1>), grid, dim3(256), 0, s, g, bytes, xp, dyp, dxp, a, fu);
      else if (r.threads == 256)
        hipLaunchKernelGGL((bn_bwd_resident1<T, 256, 16, F1>), grid, dim3(256), 0, s, g, bytes, xp, dyp, dxp, a, fu);
      else if (r.k == 8)
        hipLaunchKernelGGL((bn_bwd_resident1<T, 1024, 8, F1>), grid, dim3(1024), 0, s, g, bytes, xp, dyp, dxp, a, fu);
      else if (r.k == 16)
        hipLaunchKernelGGL((bn_bwd_resident1<T, 1024, 16, F1>), grid, dim3(1024), 0, s, g, bytes, xp, dyp, dxp, a, fu);
      else
        hipLaunchKernelGGL((bn_bwd_resident1<T, 1024, 32, F1>), grid, dim3(1024), 0, s, g, bytes, xp, dyp, dxp, a, fu);
      return check_launch("bn_bwd (resident, element-wise)");
    }
    if (r.threads == 256 && r.k == 8) return launch_bwd_resident<T, 256, 8, FUSE>(g, r.need, xp, dyp, dxp, a, fu, s);
    if (r.threads == 256) return launch_bwd_resident<T, 256, 16, FUSE>(g, r.need, xp, dyp, dxp, a, fu, s);
    if (r.threads == 1024) {
      if (r.k == 8) return launch_bwd_resident<T, 1024, 8, FUSE>(g, r.need, xp, dyp, dxp, a, fu, s);
      if (r.k == 16) return launch_bwd_resident<T, 1024, 16, FUSE>(g, r.need, xp, dyp, dxp, a, fu, s);
      return launch_bwd_resident<T, 1024, RES_KMAX, FUSE>(g, r.need, xp, dyp, dxp, a, fu, s);
    }
  }
  if (vec == 0) {
    if (FUSE) return fail(FLHIP_INVALID_ARGUMENT, "bn_act: per-activation mode (inner == 1) has no fused kernels");
    const dim3 grid((unsigned)((g.C + 63) / 64), g.S);
    hipLaunchKernelGGL((bn_stats_col<T, true>), grid, dim3(256), 0, s, g, xp, dyp, a.save_mean, ws);
    hipLaunchKernelGGL((bn_bwd_apply_col<T>), grid, dim3(256), 0, s, g, xp, dyp, dxp, ws, a);
  } else {
    const dim3 grid((unsigned)g.C, g.S);
    if (vec == 4) {
      hipLaunchKernelGGL((bn_bwd_stats_seg<T, 4, FUSE>), grid, dim3(256), 0, s, g, xp, dyp, a.save_mean, ws, fu);
      hipLaunchKernelGGL((bn_bwd_apply_seg<T, 4, FUSE>), grid, dim3(256), 0, s, g, xp, dyp, dxp, ws, a, fu);
    } else {
      hipLaunchKernelGGL((bn_bwd_stats_seg<T, 1, F1>), grid, dim3(256), 0, s, g, xp, dyp, a.save_mean, ws, fu);
      hipLaunchKernelGGL((bn_bwd_apply_seg<T, 1, F1>), grid, dim3(256), 0, s, g, xp, dyp, dxp, ws, a, fu);
    }
  }
  return check_launch("bn_bwd");
}

}  // namespace flhip

using namespace flhip;

extern "C" size_t flhip_bn_workspace_bytes(const flhip_bn_desc* d) {
  BnGeom g;
  int vec;
  if (make_geom(d, &g, &vec) != FLHIP_OK) return 0;
  // the partial sums of the two-pass kernels, and never less than 32 bytes per feature
  const size_t two_pass = (size_t)g.C * g.S * 2 * sizeof(float), least = (size_t)g.C * 32;
  return two_pass > least ? two_pass : least;
}

extern "C" int flhip_bn_fwd_train(const flhip_bn_desc* d, const void* x, const float* gamma,
                                  const float* beta, void* y, float* save_mean,
                                  float* save_invstd, float* run_mean, float* run_var,
                                  double momentum, double eps, void* ws, size_t ws_bytes,
                                  void* stream) {
  BnGeom g;
  int vec;
  const int rc = make_geom(d, &g, &vec);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(x && y, "bn_fwd_train: null tensor");
  FLHIP_REQUIRE((run_mean == nullptr) == (run_var == nullptr),
                "bn_fwd_train: running mean and variance must be given together");
  FLHIP_REQUIRE(momentum >= 0.0 && momentum <= 1.0, "bn_fwd_train: momentum must lie in [0, 1]");
  FLHIP_REQUIRE(eps >= 0.0, "bn_fwd_train: epsilon must be non-negative");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_bn_workspace_bytes(d), "bn_fwd_train: workspace too small");
  const BnTrainArgs a{gamma, beta, save_mean, save_invstd, run_mean, run_var, momentum, eps};
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return run_train<T, 0>(g, vec, x, y, static_cast<float*>(ws), a, BnFuseFwd<T>{nullptr, 0, nullptr}, as_stream(stream));
  });
}

static int bn_act_fwd_train_impl(const flhip_bn_desc* d, const void* x, const float* gamma,
                                 const float* beta, const void* residual, int relu, void* y,
                                 void* mask, bool want_mask, float* save_mean, float* save_invstd,
                                 float* run_mean, float* run_var, double momentum, double eps,
                                 void* ws, size_t ws_bytes, void* stream) {
  BnGeom g;
  int vec;
  const int rc = make_geom(d, &g, &vec);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(x && y, "bn_act_fwd_train: null tensor");
  FLHIP_REQUIRE(!want_mask || (mask && vec == 4),
                "bn_act_fwd_train_mask: needs a mask buffer and rows of a multiple of 4 elements "
                "(flhip_bn_act_mask_bytes tells)");
  FLHIP_REQUIRE((run_mean == nullptr) == (run_var == nullptr),
                "bn_act_fwd_train: running mean and variance must be given together");
  FLHIP_REQUIRE(momentum >= 0.0 && momentum <= 1.0, "bn_act_fwd_train: momentum must lie in [0, 1]");
  FLHIP_REQUIRE(eps >= 0.0, "bn_act_fwd_train: epsilon must be non-negative");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_bn_workspace_bytes(d), "bn_act_fwd_train: workspace too small");
  const BnTrainArgs a{gamma, beta, save_mean, save_invstd, run_mean, run_var, momentum, eps};
  uint8_t* mk = want_mask ? static_cast<uint8_t*>(mask) : nullptr;
  float* wsf = static_cast<float*>(ws);
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    const BnFuseFwd<T> fu{static_cast<const T*>(residual), relu, mk};
    return mk ? run_train<T, 2>(g, vec, x, y, wsf, a, fu, as_stream(stream))
              : run_train<T, 1>(g, vec, x, y, wsf, a, fu, as_stream(stream));
  });
}

extern "C" int flhip_bn_act_fwd_train(const flhip_bn_desc* d, const void* x, const float* gamma,
                                      const float* beta, const void* residual, int relu, void* y,
                                      float* save_mean, float* save_invstd, float* run_mean,
                                      float* run_var, double momentum, double eps, void* ws,
                                      size_t ws_bytes, void* stream) {
  return bn_act_fwd_train_impl(d, x, gamma, beta, residual, relu, y, nullptr, false, save_mean, save_invstd,
                               run_mean, run_var, momentum, eps, ws, ws_bytes, stream);
}

extern "C" size_t flhip_bn_act_mask_bytes(const flhip_bn_desc* d) {
  if (!d || d->outer <= 0 || d->C <= 0 || d->inner <= 1 || d->inner % 4 != 0) return 0;
  return (size_t)d->outer * (size_t)d->C * (size_t)d->inner / 4;
}

extern "C" int flhip_bn_act_fwd_train_mask(const flhip_bn_desc* d, const void* x, const float* gamma,
                                           const float* beta, const void* residual, int relu, void* y,
                                           void* mask, float* save_mean, float* save_invstd,
                                           float* run_mean, float* run_var, double momentum, double eps,
                                           void* ws, size_t ws_bytes, void* stream) {
  return bn_act_fwd_train_impl(d, x, gamma, beta, residual, relu, y, mask, true, save_mean, save_invstd,
                               run_mean, run_var, momentum, eps, ws, ws_bytes, stream);
}

extern "C" int flhip_bn_fwd_infer(const flhip_bn_desc* d, const void* x, const float* gamma,
                                  const float* beta, const float* run_mean, const float* run_var,
                                  double eps, void* y, void* stream) {
  BnGeom g;
  int vec;
  const int rc = make_geom(d, &g, &vec);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(x && y && run_mean && run_var, "bn_fwd_infer: null tensor");
  const size_t total = (size_t)g.outer * g.C * g.inner;
  size_t blocks = (total + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((bn_infer_kernel<T>), dim3((unsigned)blocks), dim3(256), 0,
                       as_stream(stream), g, static_cast<const T*>(x),
                       static_cast<T*>(y), gamma, beta, run_mean, run_var, (float)eps, total);
  });
  return check_launch("bn_fwd_infer");
}

extern "C" int flhip_bn_bwd(const flhip_bn_desc* d, const void* x, const void* dy,
                            const float* gamma, const float* save_mean, const float* save_invstd,
                            void* dx, float* dgamma, float* dbeta, void* ws, size_t ws_bytes,
                            void* stream) {
  BnGeom g;
  int vec;
  const int rc = make_geom(d, &g, &vec);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(x && dy && dx, "bn_bwd: null tensor");
  // the reference throws std::invalid_argument without the forward payload
  // (onednn/BatchNorm.cpp:212-215)
  FLHIP_REQUIRE(save_mean && save_invstd, "bn_bwd: needs the saved statistics of the forward pass");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_bn_workspace_bytes(d), "bn_bwd: workspace too small");
  const BnBwdArgs a{gamma, save_mean, save_invstd, dgamma, dbeta};
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return run_bwd<T, 0>(g, vec, x, dy, dx, static_cast<float*>(ws), a, BnFuseBwd<T>{nullptr, nullptr, nullptr}, as_stream(stream));
  });
}

static int bn_act_bwd_impl(const flhip_bn_desc* d, const void* x, const void* dy, const void* y,
                           const void* mask, const float* gamma, const float* save_mean,
                           const float* save_invstd, void* dx, void* dresidual, float* dgamma,
                           float* dbeta, void* ws, size_t ws_bytes, void* stream) {
  BnGeom g;
  int vec;
  const int rc = make_geom(d, &g, &vec);
  if (rc != FLHIP_OK) return rc;
  FLHIP_REQUIRE(x && dy && dx && (y || mask), "bn_act_bwd: null tensor");
  FLHIP_REQUIRE(!mask || vec == 4, "bn_act_bwd_mask: rows must hold a multiple of 4 elements");
  FLHIP_REQUIRE(save_mean && save_invstd, "bn_act_bwd: needs the saved statistics of the forward pass");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_bn_workspace_bytes(d), "bn_act_bwd: workspace too small");
  const BnBwdArgs a{gamma, save_mean, save_invstd, dgamma, dbeta};
  const uint8_t* mk = static_cast<const uint8_t*>(mask);
  float* wsf = static_cast<float*>(ws);
  // FUSE = 1: the mask is read from y, 2: from the mask bytes
  return by_dtype(d->dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    const BnFuseBwd<T> fu{static_cast<const T*>(y), static_cast<T*>(dresidual), mk};
    return mk ? run_bwd<T, 2>(g, vec, x, dy, dx, wsf, a, fu, as_stream(stream))
              : run_bwd<T, 1>(g, vec, x, dy, dx, wsf, a, fu, as_stream(stream));
  });
}

extern "C" int flhip_bn_act_bwd(const flhip_bn_desc* d, const void* x, const void* dy, const void* y,
                                const float* gamma, const float* save_mean, const float* save_invstd,
                                void* dx, void* dresidual, float* dgamma, float* dbeta, void* ws,
                                size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(y, "bn_act_bwd: null tensor");
  return bn_act_bwd_impl(d, x, dy, y, nullptr, gamma, save_mean, save_invstd, dx, dresidual, dgamma, dbeta, ws,
                         ws_bytes, stream);
}

extern "C" int flhip_bn_act_bwd_mask(const flhip_bn_desc* d, const void* x, const void* dy, const void* mask,
                                     const float* gamma, const float* save_mean, const float* save_invstd,
                                     void* dx, void* dresidual, float* dgamma, float* dbeta, void* ws,
                                     size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(mask, "bn_act_bwd_mask: null mask");
  return bn_act_bwd_impl(d, x, dy, nullptr, mask, gamma, save_mean, save_invstd, dx, dresidual, dgamma, dbeta, ws,
                         ws_bytes, stream);
}

