// Operations of the caller closures around the extension (flashlight/fl/autograd/
// Functions.cpp) that a network built from conv / pool / batch-norm layers needs to
// run end to end on device memory: ReLU, the matrix products of Linear, the bias
// reduction, logSoftmax and categorical cross-entropy.  They are not the measured
// path; the kernels are plain and bandwidth-shaped.
//
// Matrices are column-major like Flashlight tensors: element (r, c) of an R x C
// matrix is at r + c*R.
#include "common.h"
#include "conv2d.h"

namespace flhip {
namespace {

// ---- ReLU = max(x, 0) and its mask backward (Functions.cpp:329-338, 1787-1789) ----
struct OpRelu {      // fl::maximum(x, 0): NaN compares false -> 0
  __device__ float operator()(float x, float) const { return x > 0.f ? x : 0.f; }
};
struct OpReluBwd {   // (dy, x) -> dy where x > 0
  __device__ float operator()(float dy, float x) const { return x > 0.f ? dy : 0.f; }
};

// ---- the other element-wise activations of fl::nn (flashlight/fl/nn/modules/Activations.cpp) ----
// forward y = f(x); backward dx = dy * f'(x) from dy and the forward input.  16-bit storage: fp32 arithmetic,
// one rounding of the result.
__device__ __forceinline__ float act_sigmoid(float v) { return 1.f / (1.f + expf(-v)); }
template <int OP>
struct OpAct {
  float a, b;
  __device__ float operator()(float x, float) const {
    if (OP == FLHIP_ACT_ELU) return x >= 0.f ? x : a * (expf(x) - 1.f);               // Activations.cpp:136-139
    if (OP == FLHIP_ACT_CLAMP) return fminf(fmaxf(x, a), b);                          // fl::clip, Functions.cpp:465-466
    if (OP == FLHIP_ACT_TANH) return tanhf(x);                                        // :454-455
    if (OP == FLHIP_ACT_LOG) return logf(x);                                          // :403-404
    if (OP == FLHIP_ACT_SWISH) return x * act_sigmoid(a * x);                         // :498-500
    if (OP == FLHIP_ACT_SCALE) return a * x;
    if (OP == FLHIP_ACT_LEAKY) return fmaxf(x, a * x);                                // Activations.cpp:102-104
    if (OP == FLHIP_ACT_THRESHOLD) return x >= a ? x : 0.f;                           // :151-154
    return act_sigmoid(x);                                                            // :488-489
  }
};
template <int OP>
struct OpActBwd {
  float a, b;
  __device__ float operator()(float dy, float x) const {
    if (OP == FLHIP_ACT_ELU) return x >= 0.f ? dy : dy * a * expf(x);
    if (OP == FLHIP_ACT_CLAMP) return (x > a && x < b) ? dy : 0.f;                    // (result > lo) && (result < hi), :471
    if (OP == FLHIP_ACT_TANH) {
      const float t = tanhf(x);
      return (1.f - t * t) * dy;                                                      // :458-459
    }
    if (OP == FLHIP_ACT_LOG) return dy / x;                                           // :408
    if (OP == FLHIP_ACT_SWISH) {
      const float sg = act_sigmoid(a * x);
      return dy * (sg + x * a * sg * (1.f - sg));
    }
    if (OP == FLHIP_ACT_SCALE) return a * dy;
    if (OP == FLHIP_ACT_LEAKY) return x > a * x ? dy : a * dy;                        // fl::max's mask, Functions.cpp:320-324
    if (OP == FLHIP_ACT_THRESHOLD) return x >= a ? dy : 0.f;
    const float sg = act_sigmoid(x);
    return dy * sg * (1.f - sg);                                                      // :492
  }
};

// ---- fl::gatedlinearunit (Functions.cpp:1567-1610): the halved dimension's two halves are contiguous blocks of m
// elements per outer index: y[o][k] = x[o][0][k] * sigmoid(x[o][1][k]) ----
template <typename T>
__global__ void __launch_bounds__(256) glu_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, size_t n, size_t m) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const size_t o = i / m, k = i - o * m;
    const float a = ld(x, (2 * o) * m + k), g = ld(x, (2 * o + 1) * m + k);
    st(y, i, a * act_sigmoid(g));
  }
}
// dx first half = sigmoid(b) dy, second half = a sigmoid(b) (1 - sigmoid(b)) dy (:1594-1604)
template <typename T>
__global__ void __launch_bounds__(256) glu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x, T* __restrict__ dx,
                                                      size_t n, size_t m) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const size_t o = i / m, k = i - o * m;
    const float a = ld(x, (2 * o) * m + k), sg = act_sigmoid(ld(x, (2 * o + 1) * m + k)), g = ld(dy, i);
    st(dx, (2 * o) * m + k, sg * g);
    st(dx, (2 * o + 1) * m + k, a * sg * (1.f - sg) * g);
  }
}

// ---- fl::dropout (Functions.cpp:1777-1785): y = x * keep / (1 - p).  keep(i) is a counter-based function of
// (seed, i) - two rounds of a 32-bit finaliser, the top 24 bits as a uniform number in [0, 1), kept when >= p - so the
// backward pass regenerates the mask from the seed instead of storing it (the same function the RNN uses between
// layers, with the upper half of the element index in the place of the layer) ----
template <typename T>
__global__ void __launch_bounds__(256) dropout_kernel(const T* __restrict__ x, T* __restrict__ y, size_t n, uint32_t seed_lo,
                                                      uint32_t seed_hi, float p, float scale) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    uint32_t h = (uint32_t)i * 0x9E3779B1u ^ seed_lo;
    h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
    h += seed_hi + (uint32_t)(i >> 32) * 0x632BE5ABu;
    h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
    const bool keep = (float)(h >> 8) * (1.0f / 16777216.0f) >= p;
    st(y, i, keep ? ld(x, i) * scale : 0.f);
  }
}

// ---- WeightNorm (flashlight/fl/nn/modules/WeightNorm.cpp:45-72): w = v * g[r] / ||v_r|| with one g per index r of the
// kept dimension; the tensor is a rows x cols matrix whose rows are either contiguous (the kept dimension is the
// slowest: Conv2D weights, dim 3) or interleaved (it is the fastest: Linear weights, dim 0: element (r, j) at r + j * rows).
// MODE 0: n[r] = ||v_r|| (the initial g).  MODE 1: w.  MODE 2: dv = (g / n) (dw - c v / n^2), dg[r] = c / n with
// c = sum_j dw v (the chain of the reference's norm, division, tileAs and product). ----
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
wn_rows_kernel(const T* __restrict__ v, const T* __restrict__ g, const T* __restrict__ dw, T* __restrict__ out,
               T* __restrict__ dg, long long cols) {
  __shared__ float red[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t base = (size_t)blockIdx.x * (size_t)cols;
  float s2 = 0.f, c = 0.f;
  for (long long j = tid; j < cols; j += 256) {
    const float x = ld(v, base + j);
    s2 += x * x;
    if (MODE == 2) c += ld(dw, base + j) * x;
  }
  s2 = wave_sum(s2);
  if (MODE == 2) c = wave_sum(c);
  if (lane == 0) {
    red[0][wave] = s2;
    red[1][wave] = c;
  }
  __syncthreads();
  s2 = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
  c = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
  const float n = sqrtf(s2);
  if (MODE == 0) {
    if (tid == 0) st(out, blockIdx.x, n);
    return;
  }
  const float scale = ld(g, blockIdx.x) / n;
  if (MODE == 1) {
    for (long long j = tid; j < cols; j += 256) st(out, base + j, ld(v, base + j) * scale);
  } else {
    const float k = c / s2;
    for (long long j = tid; j < cols; j += 256) st(out, base + j, scale * (ld(dw, base + j) - k * ld(v, base + j)));
    if (tid == 0) st(dg, blockIdx.x, c / n);
  }
}
// interleaved rows: lane = row (64 consecutive rows are contiguous), the four waves split the columns
template <typename T, int MODE>
__global__ void __launch_bounds__(256)
wn_cols_kernel(const T* __restrict__ v, const T* __restrict__ g, const T* __restrict__ dw, T* __restrict__ out,
               T* __restrict__ dg, long long rows, long long cols) {
  __shared__ float red[2][4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long long r = (long long)blockIdx.x * 64 + lane;
  const bool rv = r < rows;
  float s2 = 0.f, c = 0.f;
  if (rv)
    for (long long j = wave; j < cols; j += 4) {
      const size_t e = (size_t)r + (size_t)j * (size_t)rows;
      const float x = ld(v, e);
      s2 += x * x;
      if (MODE == 2) c += ld(dw, e) * x;
    }
  red[0][wave][lane] = s2;
  red[1][wave][lane] = c;
  __syncthreads();
  s2 = (red[0][0][lane] + red[0][1][lane]) + (red[0][2][lane] + red[0][3][lane]);
  c = (red[1][0][lane] + red[1][1][lane]) + (red[1][2][lane] + red[1][3][lane]);
  if (!rv) return;
  const float n = sqrtf(s2);
  if (MODE == 0) {
    if (wave == 0) st(out, (size_t)r, n);
    return;
  }
  const float scale = ld(g, (size_t)r) / n, k = c / s2;
  for (long long j = wave; j < cols; j += 4) {
    const size_t e = (size_t)r + (size_t)j * (size_t)rows;
    st(out, e, MODE == 1 ? ld(v, e) * scale : scale * (ld(dw, e) - k * ld(v, e)));
  }
  if (MODE == 2 && wave == 0) st(dg, (size_t)r, c / n);
}

// ---- fl::padding (Functions.cpp:1751-1775): the input inside a tensor of `value`; one thread per result element,
// up to four column-major dimensions; the backward pass copies the inner box back ----
struct PadGeom {
  long long od[4], id[4], lo[4];
};
template <typename T, bool BWD>
__global__ void __launch_bounds__(256) pad_kernel(const T* __restrict__ src, T* __restrict__ dst, size_t n, PadGeom g, float value) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    // forward: i walks the padded result; backward: i walks the input-shaped gradient
    size_t rem = i;
    long long c[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const long long ext = BWD ? g.id[k] : g.od[k];
      c[k] = (long long)(rem % (size_t)ext);
      rem /= (size_t)ext;
    }
    if (BWD) {
      const size_t o = (size_t)(c[0] + g.lo[0]) + (size_t)g.od[0] * ((size_t)(c[1] + g.lo[1]) + (size_t)g.od[1] * ((size_t)(c[2] + g.lo[2]) + (size_t)g.od[2] * (size_t)(c[3] + g.lo[3])));
      st(dst, i, ld(src, o));
    } else {
      bool in = true;
      size_t e = 0, mul = 1;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const long long q = c[k] - g.lo[k];
        in = in && q >= 0 && q < g.id[k];
        e += (size_t)(in ? q : 0) * mul;
        mul *= (size_t)g.id[k];
      }
      st(dst, i, in ? ld(src, e) : value);
    }
  }
}

// ---- C = op(A) op(B) (+ bias per row), 64 x 64 tiles, 256 threads, 4 x 4 per thread ----
constexpr int GT = 64, GK = 16;

template <typename T>
__global__ void __launch_bounds__(256)
matmul_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N,
              int K, int ta, int tb, const float* __restrict__ bias) {
  __shared__ float As[GK][GT + 4];      // As[k][m]
  __shared__ float Bs[GK][GT + 4];      // Bs[k][n]
  const int tid = threadIdx.x;
  const int m0 = blockIdx.x * GT, n0 = blockIdx.y * GT;
  const int tm = (tid & 15) * 4, tn = (tid >> 4) * 4;
  // op(A)(m, k) = ta ? A[k + m*K] : A[m + k*M];  op(B)(k, n) = tb ? B[n + k*N] : B[k + n*K]
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
    for (int e = tid; e < GT * GK; e += 256) {
      // consecutive threads walk the contiguous dimension of each operand
      const int am = ta ? e / GK : e % GT, ak = ta ? e % GK : e / GT;
      const int gm = m0 + am, gk = k0 + ak;
      As[ak][am] = (gm < M && gk < K) ? ld(A, ta ? (size_t)gk + (size_t)gm * K : (size_t)gm + (size_t)gk * M) : 0.f;
      const int bn = tb ? e % GT : e / GK, bk = tb ? e / GT : e % GK;
      const int gn = n0 + bn, gkb = k0 + bk;
      Bs[bk][bn] = (gn < N && gkb < K) ? ld(B, tb ? (size_t)gn + (size_t)gkb * N : (size_t)gkb + (size_t)gn * K) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      const float4 a = *reinterpret_cast<const float4*>(&As[k][tm]);
      const float4 b = *reinterpret_cast<const float4*>(&Bs[k][tn]);
      const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + tm + i, n = n0 + tn + j;
      if (m < M && n < N) st(C, (size_t)m + (size_t)n * M, acc[i][j] + (bias ? bias[m] : 0.f));
    }
}

// ---- out[r] = sum over columns of x[r, c]  (sumAs(gradOutput, bias), Functions.cpp:1287) ----
// 16 rows (one 64-byte run per column) and 64 column groups per workgroup, so that a
// few thousand rows by many columns still fill the machine; fixed summation order
template <typename T>
__global__ void __launch_bounds__(1024)
sum_cols_kernel(const T* __restrict__ x, float* __restrict__ out, int R, int Cn) {
  __shared__ float red[64][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int r = blockIdx.x * 16 + tx;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (r < R) {
    int c = ty;
    for (; c + 192 < Cn; c += 256) {
      s0 += ld(x, (size_t)r + (size_t)c * R);
      s1 += ld(x, (size_t)r + (size_t)(c + 64) * R);
      s2 += ld(x, (size_t)r + (size_t)(c + 128) * R);
      s3 += ld(x, (size_t)r + (size_t)(c + 192) * R);
    }
    for (; c < Cn; c += 64) s0 += ld(x, (size_t)r + (size_t)c * R);
  }
  red[ty][tx] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (ty == 0 && r < R) {
    float s = 0.f;
#pragma unroll 8
    for (int k = 0; k < 64; ++k) s += red[k][tx];
    out[r] = s;
  }
}

// ---- C [M x N] = A [M x K] * B^T with B [N x K], column-major: both operands are
// contiguous along the dimension that survives, which is how the 16x16x4 matrix-core
// instruction wants its operands (a lane per row / column, lane groups along the
// contraction).  64 x 64 tile per workgroup, four waves of 2 x 2 instruction tiles,
// contraction in chunks of 32 double-buffered through LDS as quads {k..k+3} per row so
// that one 16-byte LDS read feeds four instructions.  blockIdx.y cuts the contraction
// into slices, each writing its own partial product (f32) at C + slice * M * N.
template <typename T>
__global__ void __launch_bounds__(256)
gemm_nt_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K,
               int mtiles, int cps) {
  __shared__ __align__(16) float As[2][8][64][4];
  __shared__ __align__(16) float Bs[2][8][64][4];
  const int tid = threadIdx.x, lm = tid & 63, lq = tid >> 6;
  const int wave = tid >> 6, lane = tid & 63, fr = lane & 15, fg = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = (blockIdx.x % mtiles) * 64, n0 = (blockIdx.x / mtiles) * 64;
  const int nchunks = (K + 31) / 32;
  const int cbeg = blockIdx.y * cps, cend = min(nchunks, cbeg + cps);
  const bool am = m0 + lm < M, bn = n0 + lm < N;
  const T* ap = A + m0 + lm;
  const T* bp = B + n0 + lm;
  float sa[2][4], sb[2][4];
  auto gload = [&](int c) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = c * 32 + 4 * (lq + 4 * h) + j;
        sa[h][j] = (am && k < K) ? ld(ap, (size_t)k * M) : 0.f;
        sb[h][j] = (bn && k < K) ? ld(bp, (size_t)k * N) : 0.f;
      }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *reinterpret_cast<float4*>(As[buf][lq + 4 * h][lm]) = make_float4(sa[h][0], sa[h][1], sa[h][2], sa[h][3]);
      *reinterpret_cast<float4*>(Bs[buf][lq + 4 * h][lm]) = make_float4(sb[h][0], sb[h][1], sb[h][2], sb[h][3]);
    }
  };
  floatx4_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  if (cbeg < cend) {
    gload(cbeg);
    sstore(0);
  }
  __syncthreads();
  for (int c = cbeg; c < cend; ++c) {
    const int buf = (c - cbeg) & 1;
    if (c + 1 < cend) gload(c + 1);
#pragma unroll
    for (int g16 = 0; g16 < 2; ++g16) {
      const int q = g16 * 4 + fg;
      float4 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = *reinterpret_cast<const float4*>(As[buf][q][(2 * wm + i) * 16 + fr]);
        b[i] = *reinterpret_cast<const float4*>(Bs[buf][q][(2 * wn + i) * 16 + fr]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].x, b[j].x, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].y, b[j].y, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].z, b[j].z, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].w, b[j].w, acc[i][j], 0, 0, 0);
        }
    }
    if (c + 1 < cend) sstore(buf ^ 1);
    __syncthreads();
  }
  T* cp = C + (size_t)blockIdx.y * M * N;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = m0 + (2 * wm + i) * 16 + 4 * fg, n = n0 + (2 * wn + j) * 16 + fr;
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (m + r < M) st(cp, (size_t)(m + r) + (size_t)n * M, acc[i][j][r]);
    }
}

template <typename T>
int gemm_nt_launch(const T* A, const T* B, T* C, int M, int N, int K, int slices, hipStream_t s) {
  const int mtiles = (M + 63) / 64, ntiles = (N + 63) / 64, nchunks = (K + 31) / 32;
  if ((long long)mtiles * ntiles > 0x7fffffffll) return -1;
  const int cps = (nchunks + slices - 1) / slices;
  hipLaunchKernelGGL((gemm_nt_kernel<T>), dim3((unsigned)(mtiles * ntiles), (unsigned)slices), dim3(256), 0, s, A,
                     B, C, M, N, K, mtiles, cps);
  return check_launch("matmul (A * B^T)");
}

// ---- products with few columns (N <= 128: fl::linear on a batch of feature vectors) ----
// The matrix-core kernels tile columns per image and have one position per column here; these two
// kernels spread a thin product over the whole chip on the vector ALUs instead (a 1000 x 2048 x 64
// product is 0.26 GFLOP).
//
// C (M x N) = A (M x K, column-major) * B (K x N) + bias.  A workgroup owns 64 rows x SK_NT columns;
// its 16 waves split the contraction.  B's block is staged in LDS as fp32 [k][SK_NT] and read by
// all lanes at once (same address: a broadcast); lane = row, so A is read in whole rows of 64.
constexpr int SK_NT = 8, SK_KC = 2048;
template <typename T>
__global__ void __launch_bounds__(1024)
matmul_nn_skinny(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K,
                 const float* __restrict__ bias) {
  __shared__ __align__(16) float sm[SK_KC * SK_NT];      // 64 KiB: B's block, then the waves' partial sums
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = blockIdx.x * 64 + lane, n0 = blockIdx.y * SK_NT;
  const bool mv = m < M;
  float acc[SK_NT];
#pragma unroll
  for (int j = 0; j < SK_NT; ++j) acc[j] = 0.f;
  for (int kc = 0; kc < K; kc += SK_KC) {
    const int kn = min(SK_KC, K - kc);
    if (kc) __syncthreads();
    for (int e = tid; e < kn * SK_NT; e += 1024) {
      const int j = e / kn, k = e - j * kn;               // consecutive threads walk k, contiguous in B
      sm[k * SK_NT + j] = (n0 + j < N) ? ld(B, (size_t)(n0 + j) * K + kc + k) : 0.f;
    }
    __syncthreads();
    const int per = (kn + 15) / 16, k0 = wave * per, k1 = min(kn, k0 + per);
    // 16 rows of A requested before the first is used: a lane's loads are 2 or 4 bytes each, and only the
    // number in flight hides the way to memory (steps past the wave's share repeat its last row and add 0)
    for (int k = k0; k < k1; k += 16) {
      float a[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const float v = ld(A, (size_t)(kc + min(k + u, k1 - 1)) * M + (mv ? m : 0));
        a[u] = (mv && k + u < k1) ? v : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int kk = min(k + u, k1 - 1);
        const float4 b0 = *reinterpret_cast<const float4*>(&sm[kk * SK_NT]);
        const float4 b1 = *reinterpret_cast<const float4*>(&sm[kk * SK_NT + 4]);
        acc[0] += a[u] * b0.x; acc[1] += a[u] * b0.y; acc[2] += a[u] * b0.z; acc[3] += a[u] * b0.w;
        acc[4] += a[u] * b1.x; acc[5] += a[u] * b1.y; acc[6] += a[u] * b1.z; acc[7] += a[u] * b1.w;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < SK_NT; ++j) sm[(wave * SK_NT + j) * 64 + lane] = acc[j];
  __syncthreads();
  if (tid < SK_NT * 64) {
    const int j = tid >> 6;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) s += sm[(w * SK_NT + j) * 64 + lane];
    if (mv && n0 + j < N) st(C, (size_t)(n0 + j) * M + m, s + (bias ? bias[m] : 0.f));
  }
}

// C (M x N) = A^T * B with A stored K x M: both operands are contiguous along the contraction.  A wave
// owns 8 x 8 results; its lanes stride over k and the 64 sums are reduced across the wave at the end.
template <typename T>
__global__ void __launch_bounds__(256)
matmul_tn_skinny(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K,
                 int mtiles, int tiles) {
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= tiles) return;
  const int m0 = (w % mtiles) * 8, n0 = (w / mtiles) * 8;
  float acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
  // rows / columns past the matrix read the last valid one; their sums are not stored
  size_t ao[8], bo[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    ao[i] = (size_t)min(m0 + i, M - 1) * K;
    bo[i] = (size_t)min(n0 + i, N - 1) * K;
  }
  for (int k = lane; k < K; k += 64) {
    float a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a[i] = ld(A, ao[i] + k);
      b[i] = ld(B, bo[i] + k);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] += a[i] * b[j];
  }
  float mine = 0.f;      // lane l keeps the sum of result (l % 8, l / 8)
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float s = wave_sum(acc[i][j]);
      if (lane == j * 8 + i) mine = s;
    }
  const int mi = m0 + (lane & 7), nj = n0 + (lane >> 3);
  if (mi < M && nj < N) st(C, (size_t)nj * M + mi, mine);
}

// ---- logSoftmax over dimension 0 of a C x X matrix (Functions.cpp:1044-1070) ----
// one wave per column
template <typename T>
__global__ void __launch_bounds__(256)
logsoftmax_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, int Cn, int X) {
  const int col = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (col >= X) return;
  const T* xc = x + (size_t)col * Cn;
  float mx = -INFINITY;
  for (int c = lane; c < Cn; c += 64) mx = fmaxf(mx, ld(xc, c));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  float s = 0.f;
  for (int c = lane; c < Cn; c += 64) s += expf(ld(xc, c) - mx);
  s = wave_sum(s);
  const float lse = logf(s) + mx;
  for (int c = lane; c < Cn; c += 64) st(y + (size_t)col * Cn, c, ld(xc, c) - lse);
}

// dx = dy - exp(y) * sum_c dy
template <typename T>
__global__ void __launch_bounds__(256)
logsoftmax_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ y, T* __restrict__ dx,
                      int Cn, int X) {
  const int col = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (col >= X) return;
  const size_t o = (size_t)col * Cn;
  float s = 0.f;
  for (int c = lane; c < Cn; c += 64) s += ld(dy + o, c);
  s = wave_sum(s);
  for (int c = lane; c < Cn; c += 64) st(dx + o, c, ld(dy + o, c) - expf(ld(y + o, c)) * s);
}

// ---- categorical cross-entropy on log-probabilities (Functions.cpp:1078-1154) ----
// stats[0] = sum over counted columns of -x[target, col], stats[1] = counted columns,
// stats[2] = columns whose target is neither in [0, C) nor the ignore index,
// stats[3] = stats[0] / stats[1] (the MEAN reduction).  One block; columns are added
// in a fixed order.
template <typename T>
__global__ void __launch_bounds__(256)
cce_fwd_kernel(const T* __restrict__ x, const int32_t* __restrict__ target, float* __restrict__ stats,
               float* __restrict__ per_col, int Cn, int X, int ignore) {
  __shared__ float red[4];
  float s = 0.f, cnt = 0.f, bad = 0.f;
  for (int i = threadIdx.x; i < X; i += 256) {
    const int t = target[i];
    float v = 0.f;
    if (t == ignore) {
    } else if (t < 0 || t >= Cn) {
      bad += 1.f;
    } else {
      v = -ld(x, (size_t)i * Cn + t);
      cnt += 1.f;
    }
    if (per_col) per_col[i] = v;
    s += v;
  }
  s = block_sum(s, red);
  cnt = block_sum(cnt, red);
  bad = block_sum(bad, red);
  if (threadIdx.x == 0) {
    stats[0] = s;
    stats[1] = cnt;
    stats[2] = bad;
    stats[3] = s / cnt;
  }
}

// dx[c, col] = -(g_col) where c == target[col] and the column counts, else 0;
// g_col = grad[0] / count (mean), grad[0] (sum) or grad[col] (none)
template <typename T>
__global__ void __launch_bounds__(256)
cce_bwd_kernel(const float* __restrict__ grad, const int32_t* __restrict__ target,
               const float* __restrict__ stats, T* __restrict__ dx, int Cn, int X, int reduction,
               int ignore) {
  const size_t total = (size_t)Cn * X;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int col = (int)(e / Cn), c = (int)(e - (size_t)col * Cn);
    const int t = target[col];
    float v = 0.f;
    if (t != ignore && c == t) {
      const float g = reduction == 0 ? grad[col] : reduction == 1 ? grad[0] / stats[1] : grad[0];
      v = -g;
    }
    st(dx, e, v);
  }
}

unsigned blocks_for(size_t n) {
  size_t b = (n + 255) / 256;
  if (b > 16384) b = 16384;
  if (b < 1) b = 1;
  return (unsigned)b;
}

// ---- broadcast scale and shift, y = w * x + b (the affine part of LayerNorm,
// flashlight/fl/nn/modules/LayerNorm.cpp:110-128: tileAs(weight) * output + tileAs(bias)) ----
// The tensor is viewed as [outer][mid][inner]; the parameters have one element per
// mid index (pstride 1) or a single element (pstride 0).
template <typename T>
__global__ void __launch_bounds__(256)
affine_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ b,
                  T* __restrict__ y, size_t n, long long mid, long long inner, int pstride) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
    const size_t m = (size_t)pstride * ((e / (size_t)inner) % (size_t)mid);
    st(y, e, ld(w, m) * ld(x, e) + ld(b, m));
  }
}

// fl::PReLU (flashlight/fl/nn/modules/Activations.cpp:121-124): y = x where x >= 0, w[m] x elsewhere; the
// parameter is tiled along the tensor's first dimension (m = e % d0), or is a single element (pstride 0)
template <typename T>
__global__ void __launch_bounds__(256)
prelu_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, size_t n, long long d0, int pstride) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
    const float v = ld(x, e);
    st(y, e, v >= 0.f ? v : v * ld(w, (size_t)pstride * (e % (size_t)d0)));
  }
}

// dst[i0, i1, i2, i3] = src[...] with dst dimension k taken from src dimension perm[k]
// (column-major, dimension 0 fastest); one thread per dst element, writes coalesced
struct ReorderGeom {
  long long d[4];    // dst extents
  long long ss[4];   // src stride of the dimension that dst dimension k walks
};
template <typename T>
__global__ void __launch_bounds__(256)
reorder_kernel(const T* __restrict__ src, T* __restrict__ dst, size_t n, ReorderGeom g) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
    size_t t = e;
    const size_t i0 = t % (size_t)g.d[0]; t /= (size_t)g.d[0];
    const size_t i1 = t % (size_t)g.d[1]; t /= (size_t)g.d[1];
    const size_t i2 = t % (size_t)g.d[2]; t /= (size_t)g.d[2];
    dst[e] = src[i0 * g.ss[0] + i1 * g.ss[1] + i2 * g.ss[2] + t * g.ss[3]];
  }
}

// Backward: dx = w * dy, and per parameter element the partial sums of dy * x and dy
// over slice blockIdx.y of its elements: part[(m * S + s) * 2 + {0, 1}].
// PRELU: the same walk for fl::PReLU's backward pass: dx = dy where x >= 0 and w[m] dy elsewhere, and the
// parameter's gradient is the sum of dy x over the elements with x < 0 (the second sum is not used).
template <typename T, bool PRELU = false>
__global__ void __launch_bounds__(256)
affine_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ w,
                  T* __restrict__ dx, float* __restrict__ part, long long per, long long chunk,
                  long long mid, long long inner, int S) {
  __shared__ float red[4];
  const long long m = blockIdx.x, s = blockIdx.y;
  const long long j0 = s * chunk, j1 = min(j0 + chunk, per);
  const float wm = w ? ld(w, (size_t)m) : 0.f;
  float s1 = 0.f, s2 = 0.f;
  for (long long j = j0 + threadIdx.x; j < j1; j += 256) {
    const long long o = j / inner, i = j - o * inner;
    const size_t e = (size_t)((o * mid + m) * inner + i);
    const float d = ld(dy, e);
    if (PRELU) {
      const float v = ld(x, e);
      if (part && v < 0.f) s1 += d * v;
      if (dx) st(dx, e, v >= 0.f ? d : wm * d);
      continue;
    }
    if (part) {
      s1 += d * ld(x, e);
      s2 += d;
    }
    if (dx) st(dx, e, wm * d);
  }
  if (!part) return;
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  if (threadIdx.x == 0) {
    part[(m * S + s) * 2 + 0] = s1;
    part[(m * S + s) * 2 + 1] = s2;
  }
}

__global__ void __launch_bounds__(256)
affine_fold_kernel(const float* __restrict__ part, float* __restrict__ dw, float* __restrict__ db,
                   long long nparam, int S) {
  const long long m = (long long)blockIdx.x * 256 + threadIdx.x;
  if (m >= nparam) return;
  double a = 0.0, b = 0.0;
  for (int s = 0; s < S; ++s) {
    a += (double)part[(m * S + s) * 2 + 0];
    b += (double)part[(m * S + s) * 2 + 1];
  }
  if (dw) dw[m] = (float)a;
  if (db) db[m] = (float)b;
}

// slices per parameter element: enough blocks to fill the machine, at least 2048
// elements each
struct AffinePlan {
  long long nparam, per, mid, inner, chunk;
  int S;
};
AffinePlan affine_plan(long long outer, long long mid, long long inner, int scalar) {
  AffinePlan p;
  if (scalar) {                        // one parameter element sees the whole tensor
    p.nparam = 1; p.mid = 1; p.inner = outer * mid * inner; p.per = p.inner;
  } else {
    p.nparam = mid; p.mid = mid; p.inner = inner; p.per = outer * inner;
  }
  long long S = 4096 / p.nparam;
  const long long maxS = (p.per + 2047) / 2048;
  if (S > maxS) S = maxS;
  if (S > 1024) S = 1024;
  if (S < 1) S = 1;
  p.S = (int)S;
  p.chunk = (p.per + S - 1) / S;
  return p;
}

}  // namespace

// C = A * B^T on the matrix cores (see gemm_nt_kernel); with slices > 1 (f32 only) C
// receives that many partial products, M * N floats apart, in slice order.  The number
// of slices actually written is ceil(chunks / ceil(chunks / slices)), chunks = ceil(K / 32).
int gemm_nt(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int slices, hipStream_t s) {
  if (slices < 1 || (slices > 1 && dtype != FLHIP_F32)) return -1;
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return gemm_nt_launch(static_cast<const T*>(A), static_cast<const T*>(B), static_cast<T*>(C), M, N, K, slices, s);
  });
}

}  // namespace flhip

using namespace flhip;

extern "C" int flhip_relu_fwd(const void* x, void* y, size_t n, int dtype, void* stream) {
  FLHIP_REQUIRE((x && y) || n == 0, "relu: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "relu: unknown dtype");
  if (n == 0) return FLHIP_OK;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    launch_elementwise((const T*)x, (const T*)nullptr, (T*)y, n, OpRelu{}, as_stream(stream));
  });
  return check_launch("relu");
}

extern "C" int flhip_relu_bwd(const void* dy, const void* x, void* dx, size_t n, int dtype,
                              void* stream) {
  FLHIP_REQUIRE((dy && x && dx) || n == 0, "relu_bwd: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "relu_bwd: unknown dtype");
  if (n == 0) return FLHIP_OK;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    launch_elementwise((const T*)dy, (const T*)x, (T*)dx, n, OpReluBwd{}, as_stream(stream));
  });
  return check_launch("relu_bwd");
}

extern "C" int flhip_act_fwd(int op, const void* x, void* y, size_t n, double a, double b, int dtype, void* stream) {
  FLHIP_REQUIRE((x && y) || n == 0, "act_fwd: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "act_fwd: unknown dtype");
  FLHIP_REQUIRE(op >= FLHIP_ACT_ELU && op <= FLHIP_ACT_THRESHOLD, "act_fwd: unknown activation");
  FLHIP_REQUIRE(op != FLHIP_ACT_CLAMP || a <= b, "act_fwd: clamp needs lo <= hi");
  if (n == 0) return FLHIP_OK;
  const float fa = (float)a, fb = (float)b;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    auto go = [&](auto f) { launch_elementwise((const T*)x, (const T*)nullptr, (T*)y, n, f, as_stream(stream)); };
    switch (op) {
      case FLHIP_ACT_ELU: go(OpAct<FLHIP_ACT_ELU>{fa, fb}); break;
      case FLHIP_ACT_CLAMP: go(OpAct<FLHIP_ACT_CLAMP>{fa, fb}); break;
      case FLHIP_ACT_TANH: go(OpAct<FLHIP_ACT_TANH>{fa, fb}); break;
      case FLHIP_ACT_LOG: go(OpAct<FLHIP_ACT_LOG>{fa, fb}); break;
      case FLHIP_ACT_SWISH: go(OpAct<FLHIP_ACT_SWISH>{fa, fb}); break;
      case FLHIP_ACT_SCALE: go(OpAct<FLHIP_ACT_SCALE>{fa, fb}); break;
      case FLHIP_ACT_LEAKY: go(OpAct<FLHIP_ACT_LEAKY>{fa, fb}); break;
      case FLHIP_ACT_THRESHOLD: go(OpAct<FLHIP_ACT_THRESHOLD>{fa, fb}); break;
      default: go(OpAct<FLHIP_ACT_SIGMOID>{fa, fb}); break;
    }
  });
  return check_launch("act_fwd");
}

extern "C" int flhip_act_bwd(int op, const void* dy, const void* x, void* dx, size_t n, double a, double b, int dtype,
                             void* stream) {
  FLHIP_REQUIRE((dy && x && dx) || n == 0, "act_bwd: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "act_bwd: unknown dtype");
  FLHIP_REQUIRE(op >= FLHIP_ACT_ELU && op <= FLHIP_ACT_THRESHOLD, "act_bwd: unknown activation");
  if (n == 0) return FLHIP_OK;
  const float fa = (float)a, fb = (float)b;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    auto go = [&](auto f) { launch_elementwise((const T*)dy, (const T*)x, (T*)dx, n, f, as_stream(stream)); };
    switch (op) {
      case FLHIP_ACT_ELU: go(OpActBwd<FLHIP_ACT_ELU>{fa, fb}); break;
      case FLHIP_ACT_CLAMP: go(OpActBwd<FLHIP_ACT_CLAMP>{fa, fb}); break;
      case FLHIP_ACT_TANH: go(OpActBwd<FLHIP_ACT_TANH>{fa, fb}); break;
      case FLHIP_ACT_LOG: go(OpActBwd<FLHIP_ACT_LOG>{fa, fb}); break;
      case FLHIP_ACT_SWISH: go(OpActBwd<FLHIP_ACT_SWISH>{fa, fb}); break;
      case FLHIP_ACT_SCALE: go(OpActBwd<FLHIP_ACT_SCALE>{fa, fb}); break;
      case FLHIP_ACT_LEAKY: go(OpActBwd<FLHIP_ACT_LEAKY>{fa, fb}); break;
      case FLHIP_ACT_THRESHOLD: go(OpActBwd<FLHIP_ACT_THRESHOLD>{fa, fb}); break;
      default: go(OpActBwd<FLHIP_ACT_SIGMOID>{fa, fb}); break;
    }
  });
  return check_launch("act_bwd");
}

extern "C" int flhip_glu_fwd(const void* x, void* y, int64_t outer, int64_t m, int dtype, void* stream) {
  FLHIP_REQUIRE(x && y, "glu_fwd: null argument");
  FLHIP_REQUIRE(outer > 0 && m > 0, "glu_fwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "glu_fwd: unknown dtype");
  const size_t n = (size_t)outer * (size_t)m;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((glu_fwd_kernel<T>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)x, (T*)y, n,
                       (size_t)m);
  });
  return check_launch("glu_fwd");
}

extern "C" int flhip_glu_bwd(const void* dy, const void* x, void* dx, int64_t outer, int64_t m, int dtype, void* stream) {
  FLHIP_REQUIRE(dy && x && dx, "glu_bwd: null argument");
  FLHIP_REQUIRE(outer > 0 && m > 0, "glu_bwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "glu_bwd: unknown dtype");
  const size_t n = (size_t)outer * (size_t)m;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((glu_bwd_kernel<T>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)dy, (const T*)x,
                       (T*)dx, n, (size_t)m);
  });
  return check_launch("glu_bwd");
}

extern "C" int flhip_dropout(const void* x, void* y, size_t n, double p, uint32_t seed_lo, uint32_t seed_hi, int dtype,
                             void* stream) {
  FLHIP_REQUIRE((x && y) || n == 0, "dropout: null argument");
  FLHIP_REQUIRE(p >= 0.0 && p < 1.0, "dropout: the probability must be in [0, 1)");
  FLHIP_REQUIRE(dtype_ok(dtype), "dropout: unknown dtype");
  if (n == 0) return FLHIP_OK;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((dropout_kernel<T>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)x, (T*)y, n,
                       seed_lo, seed_hi, (float)p, (float)(1.0 / (1.0 - p)));
  });
  return check_launch("dropout");
}

template <int MODE>
static int weightnorm_launch(const char* what, const void* v, const void* g, const void* dw, void* out, void* dg,
                             int64_t rows, int64_t cols, int rows_fast, int dtype, void* stream) {
  FLHIP_REQUIRE(v && out && (MODE == 0 || g) && (MODE != 2 || (dw && dg)), "weightnorm: null argument");
  FLHIP_REQUIRE(rows > 0 && cols > 0, "weightnorm: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "weightnorm: unknown dtype");
  FLHIP_REQUIRE(rows <= 0x7fffffffll, "weightnorm: too many rows");
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    if (rows_fast)
      hipLaunchKernelGGL((wn_cols_kernel<T, MODE>), dim3((unsigned)((rows + 63) / 64)), dim3(256), 0, as_stream(stream),
                         (const T*)v, (const T*)g, (const T*)dw, (T*)out, (T*)dg, (long long)rows, (long long)cols);
    else
      hipLaunchKernelGGL((wn_rows_kernel<T, MODE>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const T*)v,
                         (const T*)g, (const T*)dw, (T*)out, (T*)dg, (long long)cols);
  });
  return check_launch(what);
}

extern "C" int flhip_rownorm(const void* v, void* n, int64_t rows, int64_t cols, int rows_fast, int dtype, void* stream) {
  return weightnorm_launch<0>("rownorm", v, nullptr, nullptr, n, nullptr, rows, cols, rows_fast, dtype, stream);
}
extern "C" int flhip_weightnorm_fwd(const void* v, const void* g, void* w, int64_t rows, int64_t cols, int rows_fast,
                                    int dtype, void* stream) {
  return weightnorm_launch<1>("weightnorm_fwd", v, g, nullptr, w, nullptr, rows, cols, rows_fast, dtype, stream);
}
extern "C" int flhip_weightnorm_bwd(const void* dw, const void* v, const void* g, void* dv, void* dg, int64_t rows,
                                    int64_t cols, int rows_fast, int dtype, void* stream) {
  return weightnorm_launch<2>("weightnorm_bwd", v, g, dw, dv, dg, rows, cols, rows_fast, dtype, stream);
}

static int pad_launch(bool bwd, const void* src, void* dst, const int64_t* dims, const int32_t* before, const int32_t* after,
                      double value, int dtype, void* stream) {
  FLHIP_REQUIRE(src && dst && dims && before && after, "padding: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "padding: unknown dtype");
  PadGeom g;
  size_t nin = 1, nout = 1;
  for (int k = 0; k < 4; ++k) {
    FLHIP_REQUIRE(dims[k] > 0, "padding: sizes must be positive");
    FLHIP_REQUIRE(before[k] >= 0 && after[k] >= 0, "padding: widths must not be negative");
    g.id[k] = dims[k];
    g.lo[k] = before[k];
    g.od[k] = dims[k] + before[k] + after[k];
    nin *= (size_t)g.id[k];
    nout *= (size_t)g.od[k];
  }
  const size_t n = bwd ? nin : nout;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    if (bwd)
      hipLaunchKernelGGL((pad_kernel<T, true>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)src, (T*)dst, n,
                         g, 0.f);
    else
      hipLaunchKernelGGL((pad_kernel<T, false>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)src, (T*)dst,
                         n, g, (float)value);
  });
  return check_launch(bwd ? "padding_bwd" : "padding_fwd");
}
extern "C" int flhip_pad_fwd(const void* x, void* y, const int64_t* dims, const int32_t* before, const int32_t* after,
                             double value, int dtype, void* stream) {
  return pad_launch(false, x, y, dims, before, after, value, dtype, stream);
}
extern "C" int flhip_pad_bwd(const void* dy, void* dx, const int64_t* dims, const int32_t* before, const int32_t* after,
                             int dtype, void* stream) {
  return pad_launch(true, dy, dx, dims, before, after, 0.0, dtype, stream);
}

namespace {

// slices of the contraction for A * B^T in fp32 (gemm_nt_kernel: 64 x 64 tiles): enough tiles times slices to
// give every CU a few workgroups, at least eight chunks of 32 per slice
int nt_slices(int M, int N, int K) {
  const long long tiles = (long long)((M + 63) / 64) * ((N + 63) / 64), chunks = (K + 31) / 32;
  long long ns = 1024 / tiles;
  if (ns > chunks / 8) ns = chunks / 8;
  if (ns > 16) ns = 16;
  if (ns < 1) ns = 1;
  const long long cps = (chunks + ns - 1) / ns;
  return (int)((chunks + cps - 1) / cps);
}

__global__ void __launch_bounds__(256) sum_slices_kernel(const float* __restrict__ part, float* __restrict__ out, size_t n,
                                                         int slices) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    float v = part[i];
#pragma unroll 8
    for (int k = 1; k < slices; ++k) v += part[(size_t)k * n + i];      // loads in flight together, sums in slice order
    out[i] = v;
  }
}

}  // namespace

extern "C" size_t flhip_matmul_workspace_bytes(int32_t M, int32_t N, int32_t K, int trans_a, int trans_b, int dtype) {
  if (M <= 0 || N <= 0 || K <= 0 || !dtype_ok(dtype) || trans_a || !trans_b) return 0;
  if (options().matmul_valu) return 0;
  if (is_lo16(dtype)) return options().matmul_fp32_cores ? 0 : mfma_gemm16_ws_bytes(dtype, 2, M, N, K);
  if (dtype != FLHIP_F32) return 0;
  const int ns = nt_slices(M, N, K);
  return ns > 1 ? (size_t)ns * M * N * sizeof(float) : 0;
}

extern "C" int flhip_matmul_ws(const void* A, const void* B, void* C, int32_t M, int32_t N, int32_t K,
                               int trans_a, int trans_b, const float* bias_rows, int dtype, void* ws,
                               size_t ws_bytes, void* stream);

extern "C" int flhip_matmul(const void* A, const void* B, void* C, int32_t M, int32_t N, int32_t K,
                            int trans_a, int trans_b, const float* bias_rows, int dtype,
                            void* stream) {
  return flhip_matmul_ws(A, B, C, M, N, K, trans_a, trans_b, bias_rows, dtype, nullptr, 0, stream);
}

extern "C" int flhip_matmul_ws(const void* A, const void* B, void* C, int32_t M, int32_t N, int32_t K,
                               int trans_a, int trans_b, const float* bias_rows, int dtype, void* ws,
                               size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(A && B && C, "matmul: null argument");
  FLHIP_REQUIRE(M > 0 && N > 0 && K > 0, "matmul: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "matmul: unknown dtype");
  // thin products (a batch of feature vectors through fl::linear): the kernels made for them
  if (N <= 128 && !trans_b && !options().matmul_valu) {
    hipStream_t s = as_stream(stream);
    if (!trans_a) {
      const dim3 grid((unsigned)((M + 63) / 64), (unsigned)((N + SK_NT - 1) / SK_NT));
      by_dtype(dtype, [&](auto* t_) {
        using T = FLHIP_T_OF(t_);
        hipLaunchKernelGGL((matmul_nn_skinny<T>), grid, dim3(1024), 0, s, (const T*)A, (const T*)B,
                           (T*)C, M, N, K, bias_rows);
      });
      return check_launch("matmul (thin, A * B)");
    }
    if (!bias_rows) {
      const int mtiles = (M + 7) / 8, tiles = mtiles * ((N + 7) / 8);
      const dim3 grid((unsigned)((tiles + 3) / 4));
      by_dtype(dtype, [&](auto* t_) {
        using T = FLHIP_T_OF(t_);
        hipLaunchKernelGGL((matmul_tn_skinny<T>), grid, dim3(256), 0, s, (const T*)A, (const T*)B,
                           (T*)C, M, N, K, mtiles, tiles);
      });
      return check_launch("matmul (thin, A^T * B)");
    }
  }
  // the matrix-core kernels of the 1x1 convolutions take the three products fl::linear
  // needs; the tiled vector-ALU kernel below covers the rest.  16-bit storage: on the 16-bit
  // matrix instructions where the shape allows (MATMUL_FP32_CORES keeps them on the fp32 ones).
  if (is_lo16(dtype) && !(trans_a && trans_b) && !options().matmul_valu && !options().matmul_fp32_cores) {
    const int rc = mfma_gemm16(dtype, trans_a ? 1 : trans_b ? 2 : 0, A, B, C, M, N, K, bias_rows, as_stream(stream),
                               ws, ws_bytes);
    if (rc >= 0) return rc;
  }
  if (dtype == FLHIP_F32 && !(trans_a && trans_b) && !options().matmul_valu) {
    // A matrix as ONE image whose plane is its contiguous dimension (mfma_gemm_planes) against one position per
    // image (mfma_gemm, below) or the A * B^T kernel, measured on the products of layers of 80 to 2048 features
    // over 256 to 12000 frames: 1.3 to 2.5 times faster (2000 x 4000 x 2000: 556 -> 308, 529 -> 279, 422 -> 306 us)
    // except with planes of few rows (80: 159 -> 215 us) and, for A * B^T, with few tiles of C over a long
    // contraction (that kernel cuts it into slices).
    const int mode = trans_a ? 1 : trans_b ? 2 : 0, forced = options().matmul_planes;
    const long long tiles = (long long)((M + 63) / 64) * ((N + 63) / 64);
    const bool by_shape = mode == 1 || (M >= 256 && (mode == 0 || tiles >= 512));
    if (forced < 0 ? by_shape : ((forced >> mode) & 1) != 0) {
      const int rc = mfma_gemm_planes(mode, A, B, C, M, N, K, bias_rows, as_stream(stream));
      if (rc >= 0) return rc;
    }
  }
  if (!trans_a && trans_b && !bias_rows && !options().matmul_valu) {
    // fp32 with a workspace: the contraction in slices (the weight gradient of a layer over many frames is few
    // tiles over a long contraction), added in slice order
    const int ns = dtype == FLHIP_F32 && ws ? nt_slices(M, N, K) : 1;
    if (ns > 1 && ws_bytes >= (size_t)ns * M * N * sizeof(float)) {
      const int rc = gemm_nt(dtype, A, B, ws, M, N, K, ns, as_stream(stream));
      if (rc >= 0) {
        if (rc != 0) return rc;
        const size_t n = (size_t)M * N;
        hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 4096)), dim3(256), 0,
                           as_stream(stream), static_cast<const float*>(ws), static_cast<float*>(C), n, ns);
        return check_launch("matmul (A * B^T, slices added)");
      }
    }
    const int rc = gemm_nt(dtype, A, B, C, M, N, K, 1, as_stream(stream));
    if (rc >= 0) return rc;
  }
  if (!(trans_a && trans_b) && !options().matmul_valu) {
    const int rc = mfma_gemm(dtype, trans_a ? 1 : trans_b ? 2 : 0, A, B, C, M, N, K, bias_rows,
                             as_stream(stream));
    if (rc >= 0) return rc;
  }
  const dim3 grid((unsigned)((M + GT - 1) / GT), (unsigned)((N + GT - 1) / GT));
  FLHIP_REQUIRE(grid.y <= 65535, "matmul: too many columns");
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((matmul_kernel<T>), grid, dim3(256), 0, as_stream(stream),
                       (const T*)A, (const T*)B, (T*)C, M, N, K, trans_a, trans_b,
                       bias_rows);
  });
  return check_launch("matmul");
}

namespace {

// the value of a 16-bit element given as bits (the pointer selects the type)
__device__ __forceinline__ float bits_value(const bf16_t*, uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float bits_value(const f16_t*, uint16_t b) { return f16_to_f32(f16_t{b}); }
__device__ __forceinline__ float bits_value(const float*, uint16_t) { return 0.f; }      // fp32 rows are read one per lane

// Column sums in two passes: pass 1, workgroup (row block, column slice): a wave's lanes are consecutive rows (two each
// for 16-bit elements when the row count is even: 256 bytes per load instruction), its four waves take alternate
// columns of the slice, eight loads in flight per lane; the waves' sums meet in LDS and leave as part[slice][row].
// Pass 2 adds the slices in order.
template <typename T, int RPL>
__global__ void __launch_bounds__(256) sum_cols_sliced_kernel(const T* __restrict__ x, float* __restrict__ part, int R,
                                                              int Cn, int cps) {
  __shared__ float red[4][64 * RPL];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = (blockIdx.x * 64 + lane) * RPL;
  const int cbeg = blockIdx.y * cps, cend = min(Cn, cbeg + cps);
  float s[RPL] = {};
  if (r < R) {
    auto add = [&](int c) {
      if (RPL == 2) {
        const uint32_t v = *reinterpret_cast<const uint32_t*>(x + (size_t)c * R + r);
        s[0] += bits_value(x, (uint16_t)(v & 0xffffu));
        s[RPL - 1] += bits_value(x, (uint16_t)(v >> 16));
      } else {
        s[0] += ld(x, (size_t)c * R + r);
      }
    };
    int c = cbeg + wave;
    for (; c + 28 < cend; c += 32) {
#pragma unroll
      for (int u = 0; u < 8; ++u) add(c + 4 * u);
    }
    for (; c < cend; c += 4) add(c);
  }
#pragma unroll
  for (int e = 0; e < RPL; ++e) red[wave][lane * RPL + e] = s[e];
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * RPL; i += 256) {
    const int row = blockIdx.x * 64 * RPL + i;
    if (row < R) part[(size_t)blockIdx.y * R + row] = (red[0][i] + red[1][i]) + (red[2][i] + red[3][i]);
  }
}

// column slices for rows x cols: enough workgroups for four per CU, at least 64 columns per slice
int sum_cols_slices(int rows, int cols, int rpl) {
  if ((long long)rows * cols < (1ll << 21)) return 1;      // a second launch costs more than it saves
  const long long rb = (rows + 64 * rpl - 1) / (64 * rpl);
  long long ns = 1024 / rb;
  if (ns > cols / 64) ns = cols / 64;
  if (ns > 32) ns = 32;      // the second pass reads them one after the other, one thread per row
  if (ns < 1) ns = 1;
  const long long cps = (cols + ns - 1) / ns;
  return (int)((cols + cps - 1) / cps);
}

int sum_cols_rpl(int rows, int dtype) { return (is_lo16(dtype) && rows % 2 == 0) ? 2 : 1; }

}  // namespace

extern "C" size_t flhip_sum_columns_workspace_bytes(int32_t rows, int32_t cols, int dtype) {
  if (rows <= 0 || cols <= 0 || !dtype_ok(dtype)) return 0;
  const int ns = sum_cols_slices(rows, cols, sum_cols_rpl(rows, dtype));
  return ns > 1 ? (size_t)ns * rows * sizeof(float) : 0;
}

extern "C" int flhip_sum_columns_ws(const void* x, float* out, int32_t rows, int32_t cols, int dtype, void* ws,
                                    size_t ws_bytes, void* stream) {
  FLHIP_REQUIRE(x && out, "sum_columns: null argument");
  FLHIP_REQUIRE(rows > 0 && cols > 0, "sum_columns: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "sum_columns: unknown dtype");
  const int rpl = sum_cols_rpl(rows, dtype), ns = sum_cols_slices(rows, cols, rpl);
  if (ns <= 1 || !ws || ws_bytes < (size_t)ns * rows * sizeof(float) || ns > 65535)
    return flhip_sum_columns(x, out, rows, cols, dtype, stream);
  const int cps = (cols + ns - 1) / ns;
  const dim3 grid((unsigned)((rows + 64 * rpl - 1) / (64 * rpl)), (unsigned)ns);
  float* part = static_cast<float*>(ws);
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    if (rpl == 2) hipLaunchKernelGGL((sum_cols_sliced_kernel<T, 2>), grid, dim3(256), 0, as_stream(stream), (const T*)x, part, rows, cols, cps);
    else hipLaunchKernelGGL((sum_cols_sliced_kernel<T, 1>), grid, dim3(256), 0, as_stream(stream), (const T*)x, part, rows, cols, cps);
  });
  hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, as_stream(stream), part, out,
                     (size_t)rows, ns);
  return check_launch("sum_columns (sliced)");
}

extern "C" int flhip_sum_columns(const void* x, float* out, int32_t rows, int32_t cols, int dtype,
                                 void* stream) {
  FLHIP_REQUIRE(x && out, "sum_columns: null argument");
  FLHIP_REQUIRE(rows > 0 && cols > 0, "sum_columns: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "sum_columns: unknown dtype");
  const dim3 grid((unsigned)((rows + 15) / 16));
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((sum_cols_kernel<T>), grid, dim3(1024), 0, as_stream(stream),
                       (const T*)x, out, rows, cols);
  });
  return check_launch("sum_columns");
}

extern "C" int flhip_logsoftmax_fwd(const void* x, void* y, int32_t classes, int32_t cols, int dtype,
                                    void* stream) {
  FLHIP_REQUIRE(x && y, "logsoftmax: null argument");
  FLHIP_REQUIRE(classes > 0 && cols > 0, "logsoftmax: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "logsoftmax: unknown dtype");
  const dim3 grid((unsigned)((cols + 3) / 4));
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((logsoftmax_fwd_kernel<T>), grid, dim3(256), 0, as_stream(stream),
                       (const T*)x, (T*)y, classes, cols);
  });
  return check_launch("logsoftmax");
}

extern "C" int flhip_logsoftmax_bwd(const void* dy, const void* y, void* dx, int32_t classes,
                                    int32_t cols, int dtype, void* stream) {
  FLHIP_REQUIRE(dy && y && dx, "logsoftmax_bwd: null argument");
  FLHIP_REQUIRE(classes > 0 && cols > 0, "logsoftmax_bwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "logsoftmax_bwd: unknown dtype");
  const dim3 grid((unsigned)((cols + 3) / 4));
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((logsoftmax_bwd_kernel<T>), grid, dim3(256), 0, as_stream(stream),
                       (const T*)dy, (const T*)y, (T*)dx, classes, cols);
  });
  return check_launch("logsoftmax_bwd");
}

extern "C" int flhip_cce_fwd(const void* logp, const int32_t* target, float* stats, float* per_column,
                             int32_t classes, int32_t cols, int32_t ignore_index, int dtype,
                             void* stream) {
  FLHIP_REQUIRE(logp && target && stats, "cce: null argument");
  FLHIP_REQUIRE(classes > 0 && cols > 0, "cce: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "cce: unknown dtype");
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((cce_fwd_kernel<T>), dim3(1), dim3(256), 0, as_stream(stream),
                       (const T*)logp, target, stats, per_column, classes, cols, ignore_index);
  });
  return check_launch("cce");
}

extern "C" int flhip_cce_bwd(const float* grad, const int32_t* target, const float* stats, void* dx,
                             int32_t classes, int32_t cols, int reduction, int32_t ignore_index,
                             int dtype, void* stream) {
  FLHIP_REQUIRE(grad && target && stats && dx, "cce_bwd: null argument");
  FLHIP_REQUIRE(classes > 0 && cols > 0, "cce_bwd: sizes must be positive");
  FLHIP_REQUIRE(reduction >= 0 && reduction <= 2, "cce_bwd: unknown reduction");
  FLHIP_REQUIRE(dtype_ok(dtype), "cce_bwd: unknown dtype");
  const size_t total = (size_t)classes * cols;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((cce_bwd_kernel<T>), dim3(blocks_for(total)), dim3(256), 0,
                       as_stream(stream), grad, target, stats, (T*)dx, classes, cols, reduction,
                       ignore_index);
  });
  return check_launch("cce_bwd");
}

extern "C" int flhip_reorder(const void* src, void* dst, const int64_t* dims, const int32_t* perm,
                             int dtype, void* stream) {
  FLHIP_REQUIRE(src && dst && dims && perm, "reorder: null argument");
  FLHIP_REQUIRE(dtype_ok(dtype), "reorder: unknown dtype");
  long long sstride[4], st = 1;
  unsigned seen = 0;
  for (int k = 0; k < 4; ++k) {
    FLHIP_REQUIRE(dims[k] > 0, "reorder: sizes must be positive");
    FLHIP_REQUIRE(perm[k] >= 0 && perm[k] < 4, "reorder: permutation entry out of range");
    seen |= 1u << perm[k];
    sstride[k] = st;
    st *= dims[k];
  }
  FLHIP_REQUIRE(seen == 0xf, "reorder: not a permutation of the four dimensions");
  ReorderGeom g;
  for (int k = 0; k < 4; ++k) {
    g.d[k] = dims[perm[k]];
    g.ss[k] = sstride[perm[k]];
  }
  const size_t n = (size_t)st;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((reorder_kernel<T>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream),
                       (const T*)src, (T*)dst, n, g);
  });
  return check_launch("reorder");
}

extern "C" int flhip_affine_fwd(const void* x, const void* w, const void* b, void* y, int64_t outer,
                                int64_t mid, int64_t inner, int scalar_params, int dtype,
                                void* stream) {
  FLHIP_REQUIRE(x && w && b && y, "affine: null argument");
  FLHIP_REQUIRE(outer > 0 && mid > 0 && inner > 0, "affine: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "affine: unknown dtype");
  const size_t n = (size_t)outer * (size_t)mid * (size_t)inner;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((affine_fwd_kernel<T>), dim3(blocks_for(n)), dim3(256), 0,
                       as_stream(stream), (const T*)x, (const T*)w, (const T*)b,
                       (T*)y, n, (long long)mid, (long long)inner, scalar_params ? 0 : 1);
  });
  return check_launch("affine");
}

extern "C" size_t flhip_affine_bwd_workspace_bytes(int64_t outer, int64_t mid, int64_t inner,
                                                   int scalar_params) {
  if (outer <= 0 || mid <= 0 || inner <= 0) return 0;
  const AffinePlan p = affine_plan(outer, mid, inner, scalar_params);
  return (size_t)p.nparam * (size_t)p.S * 2 * sizeof(float);
}

extern "C" int flhip_affine_bwd(const void* dy, const void* x, const void* w, void* dx, float* dw,
                                float* db, int64_t outer, int64_t mid, int64_t inner,
                                int scalar_params, int dtype, void* workspace,
                                size_t workspace_bytes, void* stream) {
  FLHIP_REQUIRE(dy, "affine_bwd: null argument");
  FLHIP_REQUIRE(outer > 0 && mid > 0 && inner > 0, "affine_bwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "affine_bwd: unknown dtype");
  FLHIP_REQUIRE(!dx || w, "affine_bwd: dx needs the weight");
  const bool sums = dw || db;
  FLHIP_REQUIRE(!sums || x, "affine_bwd: the parameter gradients need x");
  if (!dx && !sums) return FLHIP_OK;
  const AffinePlan p = affine_plan(outer, mid, inner, scalar_params);
  FLHIP_REQUIRE(p.nparam <= 0x7fffffffLL, "affine_bwd: too many parameter elements");
  if (sums)
    FLHIP_REQUIRE(workspace && workspace_bytes >= (size_t)p.nparam * (size_t)p.S * 2 * sizeof(float),
                  "affine_bwd: workspace too small");
  float* part = sums ? static_cast<float*>(workspace) : nullptr;
  const dim3 grid((unsigned)p.nparam, (unsigned)p.S);
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((affine_bwd_kernel<T>), grid, dim3(256), 0, as_stream(stream),
                       (const T*)dy, (const T*)x, (const T*)w, (T*)dx, part,
                       p.per, p.chunk, p.mid, p.inner, p.S);
  });
  if (const int rc = check_launch("affine_bwd")) return rc;
  if (sums) {
    hipLaunchKernelGGL(affine_fold_kernel, dim3((unsigned)((p.nparam + 255) / 256)), dim3(256), 0,
                       as_stream(stream), part, dw, db, p.nparam, p.S);
    return check_launch("affine_bwd (fold)");
  }
  return FLHIP_OK;
}

namespace {

// y[:, i] = w[:, idx[i]]: a workgroup per group of columns, threads along the embedding dimension
template <typename T>
__global__ void __launch_bounds__(256) embedding_fwd_kernel(const int32_t* __restrict__ idx, const T* __restrict__ w,
                                                            T* __restrict__ y, long long n, int dim, int tokens) {
  for (long long i = blockIdx.x; i < n; i += gridDim.x) {
    const int t = idx[i];
    const bool ok = t >= 0 && t < tokens;
    for (int d = threadIdx.x; d < dim; d += 256) y[i * dim + d] = ok ? w[(size_t)t * dim + d] : T{};
  }
}

// dw[:, t] = the sum, in the order of i, of dy[:, i] over the positions i with idx[i] == t.  A workgroup per token:
// its first wave scans the indices 64 at a time (one ballot) and queues the matching positions in LDS, in order;
// then all threads add those columns, each thread its own rows of the embedding dimension, so the order of the
// additions is that of the positions whatever the timing.
template <typename T>
__global__ void __launch_bounds__(256) embedding_bwd_kernel(const int32_t* __restrict__ idx, const T* __restrict__ dy,
                                                            T* __restrict__ dw, long long n, int dim) {
  __shared__ int queue[64];
  __shared__ int qn;
  const int t = blockIdx.x, tid = threadIdx.x;
  constexpr int DPT = 8;                      // rows of the embedding dimension per thread and pass
  for (int d0 = 0; d0 < dim; d0 += 256 * DPT) {
    float acc[DPT];
#pragma unroll
    for (int e = 0; e < DPT; ++e) acc[e] = 0.f;
    for (long long i0 = 0; i0 < n; i0 += 64) {
      if (tid < 64) {      // the first wave
        const long long i = i0 + tid;
        const bool hit = i < n && idx[i] == t;
        const unsigned long long m = __ballot(hit);
        if (hit) queue[__popcll(m & ((1ull << tid) - 1ull))] = tid;
        if (tid == 0) qn = __popcll(m);
      }
      __syncthreads();
      const int q = qn;
      for (int k = 0; k < q; ++k) {
        const long long col = i0 + queue[k];
#pragma unroll
        for (int e = 0; e < DPT; ++e) {
          const int d = d0 + e * 256 + tid;
          if (d < dim) acc[e] += ld(dy, (size_t)col * dim + d);
        }
      }
      __syncthreads();      // every wave is done with the queue and with qn before the first wave writes them again
    }
#pragma unroll
    for (int e = 0; e < DPT; ++e) {
      const int d = d0 + e * 256 + tid;
      if (d < dim) st(dw, (size_t)t * dim + d, acc[e]);
    }
    __syncthreads();
  }
}

}  // namespace

extern "C" int flhip_embedding_fwd(const int32_t* idx, const void* w, void* y, int64_t n, int32_t dim, int32_t tokens,
                                   int dtype, void* stream) {
  FLHIP_REQUIRE(idx && w && y, "embedding: null argument");
  FLHIP_REQUIRE(n > 0 && dim > 0 && tokens > 0, "embedding: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "embedding: unknown dtype");
  const unsigned grid = (unsigned)std::min<int64_t>(n, 65535 * 16);
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((embedding_fwd_kernel<T>), dim3(grid), dim3(256), 0, as_stream(stream), idx, (const T*)w, (T*)y,
                       (long long)n, dim, tokens);
  });
  return check_launch("embedding");
}

extern "C" int flhip_embedding_bwd(const int32_t* idx, const void* dy, void* dw, int64_t n, int32_t dim, int32_t tokens,
                                   int dtype, void* stream) {
  FLHIP_REQUIRE(idx && dy && dw, "embedding_bwd: null argument");
  FLHIP_REQUIRE(n > 0 && dim > 0 && tokens > 0, "embedding_bwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "embedding_bwd: unknown dtype");
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((embedding_bwd_kernel<T>), dim3((unsigned)tokens), dim3(256), 0, as_stream(stream), idx,
                       (const T*)dy, (T*)dw, (long long)n, dim);
  });
  return check_launch("embedding_bwd");
}

extern "C" int flhip_prelu_fwd(const void* x, const void* w, void* y, int64_t outer, int64_t d0, int scalar_param,
                               int dtype, void* stream) {
  FLHIP_REQUIRE(x && w && y, "prelu_fwd: null argument");
  FLHIP_REQUIRE(outer > 0 && d0 > 0, "prelu_fwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "prelu_fwd: unknown dtype");
  const size_t n = (size_t)outer * (size_t)d0;
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((prelu_fwd_kernel<T>), dim3(blocks_for(n)), dim3(256), 0, as_stream(stream), (const T*)x,
                       (const T*)w, (T*)y, n, (long long)d0, scalar_param ? 0 : 1);
  });
  return check_launch("prelu_fwd");
}

extern "C" size_t flhip_prelu_bwd_workspace_bytes(int64_t outer, int64_t d0, int scalar_param) {
  return flhip_affine_bwd_workspace_bytes(outer, d0, 1, scalar_param);
}

extern "C" int flhip_prelu_bwd(const void* dy, const void* x, const void* w, void* dx, float* dw, int64_t outer,
                               int64_t d0, int scalar_param, int dtype, void* workspace, size_t workspace_bytes,
                               void* stream) {
  FLHIP_REQUIRE(dy && x, "prelu_bwd: null argument");
  FLHIP_REQUIRE(outer > 0 && d0 > 0, "prelu_bwd: sizes must be positive");
  FLHIP_REQUIRE(dtype_ok(dtype), "prelu_bwd: unknown dtype");
  FLHIP_REQUIRE(!dx || w, "prelu_bwd: dx needs the parameter");
  if (!dx && !dw) return FLHIP_OK;
  const AffinePlan p = affine_plan(outer, d0, 1, scalar_param);
  FLHIP_REQUIRE(p.nparam <= 0x7fffffffLL, "prelu_bwd: too many parameter elements");
  if (dw)
    FLHIP_REQUIRE(workspace && workspace_bytes >= (size_t)p.nparam * (size_t)p.S * 2 * sizeof(float),
                  "prelu_bwd: workspace too small");
  float* part = dw ? static_cast<float*>(workspace) : nullptr;
  const dim3 grid((unsigned)p.nparam, (unsigned)p.S);
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((affine_bwd_kernel<T, true>), grid, dim3(256), 0, as_stream(stream), (const T*)dy, (const T*)x,
                       (const T*)w, (T*)dx, part, p.per, p.chunk, p.mid, p.inner, p.S);
  });
  if (const int rc = check_launch("prelu_bwd")) return rc;
  if (dw) {
    hipLaunchKernelGGL(affine_fold_kernel, dim3((unsigned)((p.nparam + 255) / 256)), dim3(256), 0, as_stream(stream), part,
                       dw, (float*)nullptr, p.nparam, p.S);
    return check_launch("prelu_bwd (fold)");
  }
  return FLHIP_OK;
}
