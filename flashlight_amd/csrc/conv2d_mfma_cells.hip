// Backward-data of a stride-2 convolution over few input channels (the 7x7 stride-2 stem of ResNet, whose
// input has 3 channels) on the fp32 matrix cores (v_mfma_f32_16x16x4_f32), for fp32 / bf16 / f16 storage.
//
// A window of stride 2 reaches an input position (ih, iw) only through the taps whose row has the parity of
// ih + py and whose column the parity of iw + px.  The input gradient is therefore cut into 2 x 2 cells
// (i, j) -> (2i + e, 2j + f): all four positions of a cell read the same window of the output gradient -
// rows oh = i + base_y + a, columns ow = j + base_x + b, a, b = 0..3 - with weights that depend on (e, f):
//     dx[n][c][2i + e][2j + f] = sum over k, a, b of  dy[n][k][i + base_y + a][j + base_x + b] * W'[k][a][b][c, e, f]
// where W'[k][a][b][c, e, f] = w[k][c][r(e, a)][s(f, b)], or 0 where parity e has no tap at window row a.
// That is a stride-1 window of 4 x 4 taps from K channels onto 4 * C <= 16 columns: one 16-wide operand of the
// matrix instruction (the (c, e, f) columns are its M side, 16 cells of one row its N side, 4 channels its
// contraction).  Lane l of the result holds rows 4 * (l >> 4) .. + 3 = the four positions of the cell
// (l & 15) in channel l >> 4, so a cell row leaves as 8-byte (two-column) stores that are contiguous over lanes.
//
// A workgroup owns 8 rows of cells x CT * 16 columns of one image, a wave one of the rows.  W' (16 taps x K x 12
// floats) is built once per workgroup in LDS from the weights as they lie in memory; the output gradient comes in
// chunks of 4 channels (rows + 3 halo rows, columns + 3 halo columns; positions outside the tensor are buffer loads
// that return zero), fetched into registers while the previous chunk multiplies.  Within a chunk the fragments of
// tap t + 1 are read from LDS between the matrix instructions of tap t.  16-bit storage converts on the way into
// LDS; the arithmetic is fp32 for every storage type.  Of the instruction's work 12 / 16 columns and 49 / 64 taps
// are the stem's: 7.55 GFLOP of convolution at batch 32 are 13.2 GFLOP issued.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

// a workgroup has WV waves and owns WV rows of cells (+ 3 halo rows in its slab)
constexpr int CL_WCOLS = 12;             // columns of W' kept (c < 3 .. the fourth channel needs 16)

struct CellsParams {
  int N, C, H, W, K, KH, KW, OH, OW;
  int plane;                 // OH * OW
  int row_tiles, col_tiles;  // per image
  int base_y, base_x;
  unsigned rpack, spack;     // 4 bits per (e, a) / (f, b): window row / column + 1, 0 = none
  unsigned dy_bytes;
  int wcols;                 // 12 (C <= 3) or 16
  int vec2;                  // results leave two columns at a time
};

template <typename T>
__device__ __forceinline__ float cells_load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
  } else if constexpr (std::is_same<T, bf16_t>::value) {
    return bf16_to_f32((bf16_t)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0));
  } else {
    return f16_to_f32(f16_t{(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0)});
  }
}

__device__ __forceinline__ void cells_store2(float* p, float a, float b) { *reinterpret_cast<float2*>(p) = make_float2(a, b); }
__device__ __forceinline__ void cells_store2(bf16_t* p, float a, float b) { *reinterpret_cast<uint32_t*>(p) = pack_bf16(a, b); }
__device__ __forceinline__ void cells_store2(f16_t* p, float a, float b) { *reinterpret_cast<uint32_t*>(p) = pack_f16(a, b); }

template <typename T, int CT, int WV>
__global__ void __launch_bounds__(64 * WV, 2)
cells_bwd_data_kernel(CellsParams p, const T* __restrict__ dy, const T* __restrict__ wgt, T* __restrict__ dx) {
  constexpr int OOB = (int)0x80000000;
  constexpr int CL_THREADS = 64 * WV, CL_ROWS = WV, CL_SR = WV + 3;
  constexpr int COLS = CT * 16 + 3;                                   // slab columns in use
  constexpr int P = CT * 16 + 4;                                      // slab pitch
  constexpr int CS = ((CL_SR * P - 16 + 63) / 64) * 64 + 16;          // channel pitch: 16 (mod 64) banks apart
  constexpr int TOTAL = 4 * CL_SR * P;                                // slab positions of a chunk (with the pad column)
  constexpr int NL = (TOTAL + CL_THREADS - 1) / CL_THREADS;
  extern __shared__ float lds_cells[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wc = p.wcols;
  float* const Wl = lds_cells;                                        // [K / 4][16 taps][4][wc]
  float* const slab = lds_cells + 16 * p.K * wc;                      // [4][CS]

  int b = blockIdx.x;
  const int ctb = b % p.col_tiles;
  b /= p.col_tiles;
  const int rt = b % p.row_tiles;
  const int n = b / p.row_tiles;
  const int i0 = rt * CL_ROWS, j0 = ctb * CT * 16;

  // ---- W' from the weights: column m = (c, e, f) of tap (a, b) of channel k; eight independent loads in flight
  for (int base = tid; base < p.K * 256; base += 8 * CL_THREADS) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * CL_THREADS;
      const int k = idx >> 8, tap = (idx >> 4) & 15, m = idx & 15;
      const int c = m >> 2, e = (m >> 1) & 1, f = m & 1;
      const int r = (int)((p.rpack >> (4 * (e * 4 + (tap >> 2)))) & 15u) - 1;
      const int s = (int)((p.spack >> (4 * (f * 4 + (tap & 3)))) & 15u) - 1;
      const bool ok = idx < p.K * 256 && c < p.C && r >= 0 && s >= 0;
      const float t = ld(wgt, ok ? (size_t)(((k * p.C + c) * p.KH + r) * p.KW + s) : (size_t)0);
      v[j] = ok ? t : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * CL_THREADS;
      const int k = idx >> 8, tap = (idx >> 4) & 15, m = idx & 15;
      if (idx < p.K * 256 && m < wc) Wl[(((k >> 2) * 16 + tap) * 4 + (k & 3)) * wc + m] = v[j];
    }
  }

  // ---- where this thread's slab positions lie in the output gradient (relative to channel 0 of the image)
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(dy, p.dy_bytes);
  int goff[NL], loff[NL];
#pragma unroll
  for (int q = 0; q < NL; ++q) {
    const int idx = tid + q * CL_THREADS;
    const int kk = idx / (CL_SR * P), rem = idx - kk * (CL_SR * P);
    const int row = rem / P, col = rem - row * P;
    const int oh = i0 + p.base_y + row, ow = j0 + p.base_x + col;
    const bool ok = idx < TOTAL && col < COLS && oh >= 0 && oh < p.OH && ow >= 0 && ow < p.OW;
    goff[q] = ok ? (int)((kk * p.plane + oh * p.OW + ow) * (int)sizeof(T)) : OOB;
    loff[q] = idx < TOTAL ? kk * CS + row * P + col : -1;
  }

  floatx4 acc[CT];
#pragma unroll
  for (int t = 0; t < CT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int nchunks = p.K >> 2;
  const int chunk_bytes = 4 * p.plane * (int)sizeof(T);
  int soff = n * p.K * p.plane * (int)sizeof(T);
  float stage[NL];
#pragma unroll
  for (int q = 0; q < NL; ++q) stage[q] = cells_load<T>(rsrc, goff[q], soff);

  const int g = lane >> 4, l16 = lane & 15;
  const bool acol = l16 < wc;
  const float* const bbase = slab + g * CS + wave * P + l16;
  const float* abase = Wl + g * wc + (acol ? l16 : 0);

  for (int ch = 0; ch < nchunks; ++ch) {
    __syncthreads();                       // the previous chunk has been read (first trip: W' is complete)
#pragma unroll
    for (int q = 0; q < NL; ++q)
      if (q < NL - 1 || loff[q] >= 0) slab[loff[q]] = stage[q];
    __syncthreads();
    if (ch + 1 < nchunks) {
      soff += chunk_bytes;
#pragma unroll
      for (int q = 0; q < NL; ++q) stage[q] = cells_load<T>(rsrc, goff[q], soff);
    }
    // the fragments of tap + 1 are requested between the matrix instructions of tap
    float av[2], bv[2][CT];
    auto request = [&](int set, int tap) {
      av[set] = abase[tap * 4 * wc];
#pragma unroll
      for (int t = 0; t < CT; ++t) bv[set][t] = bbase[(tap >> 2) * P + (tap & 3) + t * 16];
    };
    request(0, 0);
#pragma unroll
    for (int tap = 0; tap < 16; ++tap) {
      __builtin_amdgcn_sched_barrier(0);
      if (tap + 1 < 16) request((tap + 1) & 1, tap + 1);
      const float a_ = acol ? av[tap & 1] : 0.f;
#pragma unroll
      for (int t = 0; t < CT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_, bv[tap & 1][t], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < CT; ++t) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    abase += 16 * 4 * wc;
  }

  // ---- lane: channel g, cell (i0 + wave, j0 + 16 t + l16); its registers are (e, f) = (0,0) (0,1) (1,0) (1,1)
  const int i = i0 + wave;
  if (g < p.C) {
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      const int iw = 2 * (j0 + t * 16 + l16);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int ih = 2 * i + e;
        if (ih < p.H && iw < p.W) {
          T* const dst = dx + ((size_t)(n * p.C + g) * p.H + ih) * p.W + iw;
          if (p.vec2) {
            cells_store2(dst, acc[t][2 * e], acc[t][2 * e + 1]);
          } else {
            st(dst, 0, acc[t][2 * e]);
            if (iw + 1 < p.W) st(dst, 1, acc[t][2 * e + 1]);
          }
        }
      }
    }
  }
}

// taps of one axis: for parity e the window positions r = 2 a' + rho (rho = (e + pad) & 1) reach
// o = i + delta - a' (delta = (e + pad) >> 1).  base: the first o - i over both parities; span: how many.
struct AxisTaps {
  int base, span;
  unsigned pack;
};
AxisTaps axis_taps(int ksize, int pad) {
  int lo = 1 << 20, hi = -(1 << 20);
  for (int e = 0; e < 2; ++e) {
    const int rho = (e + pad) & 1, delta = (e + pad) >> 1, na = (ksize - rho + 1) / 2;
    if (na <= 0) continue;
    lo = std::min(lo, delta - na + 1);
    hi = std::max(hi, delta);
  }
  AxisTaps t{lo, hi - lo + 1, 0u};
  if (t.span > 4 || hi < lo) return AxisTaps{0, 99, 0u};
  for (int e = 0; e < 2; ++e) {
    const int rho = (e + pad) & 1, delta = (e + pad) >> 1;
    for (int a = 0; a < 4; ++a) {
      const int ap = delta - lo - a, r = 2 * ap + rho;
      if (ap >= 0 && r < ksize) t.pack |= (unsigned)(r + 1) << (4 * (e * 4 + a));
    }
  }
  return t;
}

// ---- forward -------------------------------------------------------------------------------------------
// The same cells the other way round: y[n][k][oh][ow] = sum over the window's taps of x[n][c][2 oh - py + r][2 ow - px + s]
// w[k][c][r][s].  Input row 2 oh - py + r = 2 (oh + base_y + a) + e: tap r is row parity e of the cell a rows below the
// first one the window touches, and the window spans at most 4 x 4 cells of 2 x 2 positions.  With the input seen as
// 4 C planes X'[(c, e, f)][i][j] = x[c][2 i + e][2 j + f] this is a stride-1 window of 16 taps over 4 C channels; a
// matrix instruction (16x16x4 fp32) contracts the four (e, f) of one (tap, c) - no padding of the contraction -, its
// M side are 16 result channels and its N side 16 result columns.  A workgroup owns 8 result rows x 16 CT columns x
// 64 result channels of one image: the input rows it needs (de-interleaved by column parity, so that consecutive result
// columns are consecutive in LDS) and W'' (16 taps x C x 4 x 64 channels) are loaded once, then every wave multiplies
// one result row: 16 C steps of 4 weight and CT input fragments for 4 CT instructions.
constexpr int CF_R = 8;             // result rows per workgroup = waves
constexpr int CF_CR = CF_R + 3;     // cell rows of the slab
constexpr int CF_LB = 32;           // loads a thread has in flight while the workgroup fills its LDS (nothing else to do then)
constexpr int CF_KP = 80;           // weights: 64 result channels of one contraction row + 16 (the rows of a fragment on distinct banks)

struct CellsFwdParams {
  int N, C, H, W, K, KH, KW, OH, OW;
  int row_tiles, col_tiles;
  int base_y, base_x;          // first cell of the window relative to the result position
  unsigned rpack, spack;       // 4 bits per (e, a) / (f, b): window row / column + 1, 0 = none
};

template <typename T, int CT>
__global__ void __launch_bounds__(64 * CF_R, 1)
cells_fwd_kernel(CellsFwdParams p, const T* __restrict__ x, const T* __restrict__ wgt, const float* __restrict__ bias,
                 T* __restrict__ y) {
  constexpr int THREADS = 64 * CF_R;
  constexpr int CC = CT * 16 + 3;                                   // cell columns of the slab
  constexpr int P = ((CC - 16 + 63) / 64) * 64 + 16;                // plane pitch: the four (e, f) planes 16 banks apart
  extern __shared__ float lds_cells[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  float* const Wl = lds_cells;                                      // [16 taps][C][4 (e, f)][CF_KP]
  float* const xs = lds_cells + 16 * p.C * 4 * CF_KP;               // [C][CF_CR][2 e][2 f][P]

  int b = blockIdx.x;
  const int ctb = b % p.col_tiles;
  b /= p.col_tiles;
  const int rt = b % p.row_tiles;
  const int n = b / p.row_tiles;
  const int k0 = blockIdx.y * 64;
  const int i0 = rt * CF_R, j0 = ctb * CT * 16;

  // ---- W'': row (tap, c, (e, f)), 64 result channels
  for (int base = tid; base < 16 * p.C * 256; base += CF_LB * THREADS) {
    float v[CF_LB];
#pragma unroll
    for (int j = 0; j < CF_LB; ++j) {
      const int idx = base + j * THREADS;
      const int m = idx & 63, kk = (idx >> 6) & 3, tc = idx >> 8;
      const int tap = tc / p.C, c = tc - tap * p.C;
      const int r = (int)((p.rpack >> (4 * ((kk >> 1) * 4 + (tap >> 2)))) & 15u) - 1;
      const int s = (int)((p.spack >> (4 * ((kk & 1) * 4 + (tap & 3)))) & 15u) - 1;
      const bool ok = idx < 16 * p.C * 256 && k0 + m < p.K && r >= 0 && s >= 0;
      const float t = ld(wgt, ok ? (size_t)((((k0 + m) * p.C + c) * p.KH + r) * p.KW + s) : (size_t)0);
      v[j] = ok ? t : 0.f;
    }
#pragma unroll
    for (int j = 0; j < CF_LB; ++j) {
      const int idx = base + j * THREADS;
      if (idx < 16 * p.C * 256) Wl[(idx >> 6) * CF_KP + (idx & 63)] = v[j];
    }
  }
  // ---- the input rows: (c, cell row, e) x 2 CC consecutive input columns, split by column parity
  {
    const int rows = p.C * CF_CR * 2, width = 2 * CC;
    const int iw0 = 2 * (j0 + p.base_x);
    for (int base = tid; base < rows * width; base += CF_LB * THREADS) {
      float v[CF_LB];
#pragma unroll
      for (int j = 0; j < CF_LB; ++j) {
        const int idx = base + j * THREADS;
        const int row = idx / width, col = idx - row * width;
        const int e = row & 1, ci = (row >> 1) % CF_CR, c = (row >> 1) / CF_CR;
        const int ih = 2 * (i0 + p.base_y + ci) + e, iw = iw0 + col;
        const bool ok = idx < rows * width && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
        const float t = ld(x, ok ? ((size_t)(n * p.C + c) * p.H + ih) * p.W + iw : (size_t)0);
        v[j] = ok ? t : 0.f;
      }
#pragma unroll
      for (int j = 0; j < CF_LB; ++j) {
        const int idx = base + j * THREADS;
        const int row = idx / width, col = idx - row * width;
        if (idx < rows * width) xs[(row * 2 + (col & 1)) * P + (col >> 1)] = v[j];
      }
    }
  }
  __syncthreads();

  floatx4 acc[4][CT];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int t = 0; t < CT; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int g = lane >> 4, l16 = lane & 15;
  // lane: contraction row (e, f) = g of a step; result channel l16 of a weight fragment, result column l16 of an input one
  const float* abase = Wl + g * CF_KP + l16;
  const float* bbase = xs + (wave * 4 + g) * P + l16;
  for (int c = 0; c < p.C; ++c) {
    float av[2][4], bv[2][CT];
    auto request = [&](int set, int tap) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) av[set][mt] = abase[(tap * p.C) * 4 * CF_KP + mt * 16];
#pragma unroll
      for (int t = 0; t < CT; ++t) bv[set][t] = bbase[(tap >> 2) * 4 * P + (tap & 3) + t * 16];
    };
    request(0, 0);
#pragma unroll
    for (int tap = 0; tap < 16; ++tap) {
      __builtin_amdgcn_sched_barrier(0);
      if (tap + 1 < 16) request((tap + 1) & 1, tap + 1);
#pragma unroll
      for (int t = 0; t < CT; ++t)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[tap & 1][mt], bv[tap & 1][t], acc[mt][t], 0, 0, 0);
#pragma unroll
      for (int q = 0; q < CT + 4; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    abase += 4 * CF_KP;
    bbase += CF_CR * 4 * P;
  }

  // ---- lane: result channels k0 + 16 mt + 4 g .. + 3, column j0 + 16 t + l16 of row i0 + wave
  const int oh = i0 + wave;
  if (oh < p.OH) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int k = k0 + mt * 16 + 4 * g + r;
        if (k < p.K) {
          const float bv0 = bias ? bias[k] : 0.f;
          T* const row = y + ((size_t)(n * p.K + k) * p.OH + oh) * p.OW;
#pragma unroll
          for (int t = 0; t < CT; ++t) {
            const int ow = j0 + t * 16 + l16;
            if (ow < p.OW) st(row, (size_t)ow, acc[mt][t][r] + bv0);
          }
        }
      }
  }
}

// forward taps of one axis: window position r reads input 2 o - pad + r = 2 (o + ia) + e; base = the smallest ia, span
// = how many; pack: 4 bits per (e, a) with r + 1
AxisTaps axis_taps_fwd(int ksize, int pad) {
  int lo = 1 << 20, hi = -(1 << 20);
  for (int r = 0; r < ksize; ++r) {
    const int d = r - pad, e = ((d % 2) + 2) % 2, ia = (d - e) / 2;
    lo = std::min(lo, ia);
    hi = std::max(hi, ia);
  }
  AxisTaps t{lo, hi - lo + 1, 0u};
  if (t.span > 4) return AxisTaps{0, 99, 0u};
  for (int r = 0; r < ksize; ++r) {
    const int d = r - pad, e = ((d % 2) + 2) % 2, ia = (d - e) / 2;
    t.pack |= (unsigned)(r + 1) << (4 * (e * 4 + (ia - lo)));
  }
  return t;
}

template <typename T, int CT>
int cells_fwd_launch(const CellsFwdParams& p, const void* x, const void* w, const float* bias, void* y, dim3 grid, hipStream_t s) {
  constexpr int P = ((CT * 16 + 3 - 16 + 63) / 64) * 64 + 16;
  const size_t shmem = ((size_t)16 * p.C * 4 * CF_KP + (size_t)p.C * CF_CR * 4 * P) * sizeof(float);
  if (!mfma_allow_lds(reinterpret_cast<const void*>(cells_fwd_kernel<T, CT>), shmem)) return -1;
  hipLaunchKernelGGL((cells_fwd_kernel<T, CT>), grid, dim3(64 * CF_R), shmem, s, p, static_cast<const T*>(x),
                     static_cast<const T*>(w), bias, static_cast<T*>(y));
  return check_launch("conv2d_fwd (mfma cells)");
}

template <typename T, int CT, int WV>
int cells_launch(const CellsParams& p, const void* dy, const void* w, void* dx, int wgs, size_t shmem, hipStream_t s) {
  if (!mfma_allow_lds(reinterpret_cast<const void*>(cells_bwd_data_kernel<T, CT, WV>), shmem)) return -1;
  hipLaunchKernelGGL((cells_bwd_data_kernel<T, CT, WV>), dim3((unsigned)wgs), dim3(64 * WV), shmem, s, p,
                     static_cast<const T*>(dy), static_cast<const T*>(w), static_cast<T*>(dx));
  return check_launch("conv2d_bwd_data (mfma cells)");
}

}  // namespace

int mfma_cells_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s) {
  if (g.groups != 1 || g.dly != 1 || g.dlx != 1 || g.sy != 2 || g.sx != 2) return -1;
  if (g.C > 4 || g.K % 4 != 0 || g.KH > 8 || g.KW > 8) return -1;
  // a single tap per parity is a plain strided 1x1 / 2x2 window: the gather kernels have no waste there
  if (g.KH * g.KW < 9) return -1;
  const AxisTaps ty = axis_taps(g.KH, g.py), tx = axis_taps(g.KW, g.px);
  if (ty.span > 4 || tx.span > 4) return -1;
  const size_t esz = dtype_size(dtype);
  const long long dybytes = (long long)g.N * g.K * g.OH * g.OW * (long long)esz;
  const long long dxelems = (long long)g.N * g.C * g.H * g.W;
  if (dybytes >= (1ll << 31) || dxelems >= (1ll << 31)) return -1;
  CellsParams p{};
  p.N = g.N; p.C = g.C; p.H = g.H; p.W = g.W; p.K = g.K; p.KH = g.KH; p.KW = g.KW; p.OH = g.OH; p.OW = g.OW;
  p.plane = g.OH * g.OW;
  p.base_y = ty.base; p.base_x = tx.base;
  p.rpack = ty.pack; p.spack = tx.pack;
  p.dy_bytes = (unsigned)dybytes;
  p.wcols = g.C <= 3 ? CL_WCOLS : 16;
  p.vec2 = g.W % 2 == 0 && reinterpret_cast<uintptr_t>(dx) % (2 * esz) == 0;
  const int cells_h = (g.H + 1) / 2, cells_w = (g.W + 1) / 2;
  const int ct_all = (cells_w + 15) / 16;
  // column tiles per workgroup: the count that wastes the fewest tiles, wider first
  int CT = 1, best = 1 << 30;
  for (int c : {7, 4, 2, 1}) {
    const int padded = (ct_all + c - 1) / c * c;
    if (padded < best) {
      best = padded;
      CT = c;
    }
  }
  constexpr int WV = 8;   // rows of cells per workgroup = its waves (4 measured the same: 137 / 234 against 134 / 240 us)
  p.row_tiles = (cells_h + WV - 1) / WV;
  p.col_tiles = (ct_all + CT - 1) / CT;
  const long long wgs = (long long)g.N * p.row_tiles * p.col_tiles;
  if (wgs >= (1ll << 31)) return -1;
  const int P = CT * 16 + 4, CS = (((WV + 3) * P - 16 + 63) / 64) * 64 + 16;
  const size_t shmem = ((size_t)16 * g.K * p.wcols + 4 * CS) * sizeof(float);
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    switch (CT) {
      case 7: return cells_launch<T, 7, WV>(p, dy, w, dx, (int)wgs, shmem, s);
      case 4: return cells_launch<T, 4, WV>(p, dy, w, dx, (int)wgs, shmem, s);
      case 2: return cells_launch<T, 2, WV>(p, dy, w, dx, (int)wgs, shmem, s);
      default: return cells_launch<T, 1, WV>(p, dy, w, dx, (int)wgs, shmem, s);
    }
  });
}

int mfma_cells_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s) {
  if (g.groups != 1 || g.dly != 1 || g.dlx != 1 || g.sy != 2 || g.sx != 2) return -1;
  if (g.C > 4 || g.KH > 8 || g.KW > 8 || g.KH * g.KW < 9) return -1;
  const AxisTaps ty = axis_taps_fwd(g.KH, g.py), tx = axis_taps_fwd(g.KW, g.px);
  if (ty.span > 4 || tx.span > 4) return -1;
  if ((long long)g.N * g.C * g.H * g.W >= (1ll << 31) || (long long)g.N * g.K * g.OH * g.OW >= (1ll << 31)) return -1;
  CellsFwdParams p{};
  p.N = g.N; p.C = g.C; p.H = g.H; p.W = g.W; p.K = g.K; p.KH = g.KH; p.KW = g.KW; p.OH = g.OH; p.OW = g.OW;
  p.base_y = ty.base; p.base_x = tx.base;
  p.rpack = ty.pack; p.spack = tx.pack;
  const int ct_all = (g.OW + 15) / 16;
  int CT = 1, best = 1 << 30;
  for (int c : {7, 4, 2, 1}) {
    const int padded = (ct_all + c - 1) / c * c;
    if (padded < best) {
      best = padded;
      CT = c;
    }
  }
  p.row_tiles = (g.OH + CF_R - 1) / CF_R;
  p.col_tiles = (ct_all + CT - 1) / CT;
  const long long wgs = (long long)g.N * p.row_tiles * p.col_tiles;
  const int kblocks = (g.K + 63) / 64;
  if (wgs >= (1ll << 31) || kblocks > 65535) return -1;
  const dim3 grid((unsigned)wgs, (unsigned)kblocks);
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    switch (CT) {
      case 7: return cells_fwd_launch<T, 7>(p, x, w, bias, y, grid, s);
      case 4: return cells_fwd_launch<T, 4>(p, x, w, bias, y, grid, s);
      case 2: return cells_fwd_launch<T, 2>(p, x, w, bias, y, grid, s);
      default: return cells_fwd_launch<T, 1>(p, x, w, bias, y, grid, s);
    }
  });
}

}  // namespace flhip
