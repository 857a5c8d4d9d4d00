// Convolutions with one-row windows (KH = 1, KW taps along the contiguous axis: the 21 x 1
// windows of a wav2letter-style speech stack) in bf16 storage on v_mfma_f32_32x32x16_bf16,
// forward and backward-data, column stride 1 or 2.
//
//   forward        y[m][o]  = sum_c sum_j w[m][c][j]  x[c][o*s + j - p]   (+ bias[m])
//   backward-data  dx[c][u] = sum_m sum_j w[m][c][j] dy[m][(u + p - j) / s]   where s divides
//
// A matrix instruction wants eight consecutive contraction channels of one position per
// lane, and every tap shifts the positions by one element: with the tensors as they lie in
// memory (channel-major rows of positions) a shifted 16-byte fragment would start on any
// 2-byte boundary.  So two small passes first bring the operands into the order the
// instruction reads:
//   rows     xr[sequence][position][Cs]: the source with its channels last, Cs = the channel
//            count padded with zeros to a multiple of 16 (tap1d16_rows_kernel; a sequence is
//            one (image, row) pair); a tap then shifts whole 16-byte cells;
//   weights  wf[block of 32 result channels][tap][k-step of 16 channels][lane][8]: the
//            fragment of every (tap, k-step) exactly as the 64 lanes hold it, in the order
//            the kernel walks (tap1d16_weights_kernel); padded channels and taps are zero.
// Backward-data over a stride of 2 is two interleaved stride-1 problems (the results of even
// and of odd index take the taps of one parity each): "phases" of one workgroup, which
// writes both so that its stores cover whole runs of dx.
//
// A workgroup (4 waves) owns 96 result positions (per phase) of one sequence x 128 result
// channels; wave w owns channels 32 w .. 32 w + 31: three (six) accumulator blocks of 32 x 32.
//   * The source rows the tile needs (96 positions + the window's reach, every channel) are
//     copied to LDS once, by buffer loads with the LDS modifier (no registers, no vector
//     instructions); a row of the slab is Cs / 8 cells + 1 unused cell, which puts the eight
//     lanes of a 16-byte read cycle on distinct banks.  With a forward stride of 2 the slab
//     keeps even and odd source positions apart, so a tap's 32 positions are consecutive rows.
//   * The weights never pass through LDS: a wave's fragment of a (tap, k-step) is 1 KiB of
//     contiguous memory, fetched straight into registers 16 stages ahead of its use.  No other
//     wave needs it, so the main loop has no barrier.
//   * Per stage (16 channels of one tap) a wave reads 3 position fragments from LDS and
//     issues 3 matrix instructions.
// Positions are the rows of the instruction tile: a lane holds 4 consecutive positions of one
// result channel (8 with two phases), stored as one piece.
#include <algorithm>
#include <cstring>

#include "conv2d_mfma.h"
#include "lds_direct.h"

namespace flhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const uintx4_t* lds_cell_t;
#else
typedef const uintx4_t* lds_cell_t;
#endif

constexpr int T1_BM = 128;       // result channels per workgroup
constexpr int T1_NB = 3;         // blocks of 32 positions per wave and phase
constexpr int T1_TP = 32 * T1_NB;
constexpr int T1_MAXTAPS = 64;   // taps over both phases, padding included
constexpr int T1_OOB = (int)0x80000000;

struct Tap1Params {
  int rows, H;           // sequences (images x rows), rows per image
  int TS, TO, TOu;       // source positions, result indices per phase, result positions per sequence
  int Cs, KS;            // padded contraction channels, Cs / 16
  int Mo;                // result channels
  int nph;               // phases (1; 2: results u = 2 o + q)
  int ntaps[2];          // taps per phase as stored (a multiple of the kernel's tap group)
  int nreal[2];          // taps per phase that exist (the others carry zero weights)
  int d0[2];             // source offset of tap 0 of a phase, relative to the slab's first position
  int smin;              // slab's first source position for result 0
  int SR, half;          // slab rows; stride 2: row of the first odd source offset
  int taps_total;        // ntaps[0] + ntaps[1]
  int ptiles, mtiles;
  unsigned src_bytes, w_bytes, dst_bytes;
};

// ---- operand passes ------------------------------------------------------------------------
// x[n][c][h][t] -> xr[n * H + h][t][Cs], channels c >= C zero.  A block transposes 32 channels x 64
// positions through LDS.
__global__ void __launch_bounds__(256)
tap1d16_rows_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ xr, int C, int H, int T, int Cs) {
  __shared__ uint16_t tile[32][66];
  const int t0 = blockIdx.x * 64, c0 = blockIdx.y * 32, row = blockIdx.z;
  const int n = row / H, h = row - n * H;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = c0 + ty + 4 * i, t = t0 + tx;
    tile[ty + 4 * i][tx] = (c < C && t < T) ? x[(((size_t)n * C + c) * H + h) * T + t] : (uint16_t)0;
  }
  __syncthreads();
  const int cx = threadIdx.x & 31, tyy = threadIdx.x >> 5;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int t = t0 + tyy + 8 * i;
    if (t < T && c0 + cx < Cs) xr[((size_t)row * T + t) * Cs + c0 + cx] = tile[cx][tyy + 8 * i];
  }
}

struct Tap1Weights {
  int Mo, Cc;            // result / contraction channels that exist
  int KS, taps_total;
  int bwd;               // 0: w[m][c][j], 1: w[c][m][j] (contraction over the filters)
  int Cw, KW;            // channels per filter and taps of the weight tensor
  int mblocks;
  signed char tapj[T1_MAXTAPS];   // weight tap of stored tap i (-1: padding)
};

__global__ void __launch_bounds__(256)
tap1d16_weights_kernel(const bf16_t* __restrict__ w, uintx4_t* __restrict__ wf, Tap1Weights p) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)p.mblocks * p.taps_total * p.KS * 64;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const long long st = idx >> 6;
  const int per_block = p.taps_total * p.KS;
  const int mblk = (int)(st / per_block), s = (int)(st - (long long)mblk * per_block);
  const int tap = s / p.KS, ks = s - tap * p.KS;
  const int m = mblk * 32 + (lane & 31), c0 = ks * 16 + (lane >> 5) * 8;
  const int j = p.tapj[tap];
  uint32_t v[4] = {0u, 0u, 0u, 0u};
  if (j >= 0 && m < p.Mo) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int c = c0 + e;
      if (c < p.Cc) {
        const size_t at = p.bwd ? ((size_t)c * p.Cw + m) * p.KW + j : ((size_t)m * p.Cw + c) * p.KW + j;
        v[e >> 1] |= (uint32_t)w[at] << (16 * (e & 1));
      }
    }
  }
  wf[idx] = uintx4_t{v[0], v[1], v[2], v[3]};
}

// ---- the convolution ---------------------------------------------------------------------
// KS k-steps per tap; DT taps per unrolled group (DT * KS >= 16 stages: the distance between a
// weight fragment's load and its use); SS source stride; NPH phases.
template <int KS, int DT, int SS, int NPH>
__global__ void __launch_bounds__(256, 1)
tap1d16_conv_kernel(Tap1Params p, const bf16_t* __restrict__ xr, const uintx4_t* __restrict__ wf,
                    const float* __restrict__ bias, bf16_t* __restrict__ dst) {
  extern __shared__ uintx4_t t1_slab[];
  constexpr int CPR = 2 * KS + 1;               // cells per slab row
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ptile = __builtin_amdgcn_readfirstlane(blockIdx.x % p.ptiles);
  const int row = __builtin_amdgcn_readfirstlane(blockIdx.x / p.ptiles);
  const int mtile = blockIdx.y;
  const int o0 = ptile * T1_TP;
  const int s0 = o0 * SS + p.smin;              // source position of slab offset 0

  // ---- the slab: load instruction ii fills cells ii * 64 .. + 63, cell L = slab row L / CPR, cell L % CPR
  {
    const intx4_t xrs = pd_rsrc(xr, p.src_bytes);
    const unsigned base = pd_lds_addr(t1_slab);
    const int ncell = p.SR * CPR, ninstr = (ncell + 63) >> 6;
    const float inv = 1.0f / (float)CPR;
    for (int ii = wave; ii < ninstr; ii += 4) {
      const int L = ii * 64 + lane;
      int c;
      const int R = fast_div(L, CPR, inv, &c);
      const int off = SS == 1 ? R : (R < p.half ? 2 * R : 2 * (R - p.half) + 1);
      const int sp = s0 + off;
      int voff = T1_OOB;
      if (R < p.SR && c < 2 * KS && (unsigned)sp < (unsigned)p.TS) voff = ((row * p.TS + sp) * p.Cs + 8 * c) * 2;
      pd_load_lds(xrs, base + ii * 1024, voff, 0);
    }
  }

  // ---- weights: this wave's stream of fragments, DT * KS stages ahead
  const __amdgpu_buffer_rsrc_t wrs = make_rsrc(wf, p.w_bytes);
  const int mblk = mtile * (T1_BM / 32) + wave;
  int wpos = mblk * p.taps_total * KS * 1024;   // byte offset of the next group's first stage
  const int wlane = lane * 16;
  uintx4_t bq[DT][KS];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) bq[dt][ks] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wlane, wpos + (dt * KS + ks) * 1024, 0);
  wpos += DT * KS * 1024;

  floatx16 acc[NPH][T1_NB];
#pragma unroll
  for (int q = 0; q < NPH; ++q)
#pragma unroll
    for (int b = 0; b < T1_NB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[q][b][r] = 0.f;

  const int fr = lane & 31, fg = lane >> 5;
  lds_cell_t ap[T1_NB];
#pragma unroll
  for (int b = 0; b < T1_NB; ++b) ap[b] = (lds_cell_t)t1_slab + ((b * 32 + fr) * CPR + fg);

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the slab (and the first weight fragments) have landed
  __syncthreads();

  auto run = [&](floatx16 (&ac)[T1_NB], int q) __attribute__((always_inline)) {
    const int groups = p.ntaps[q] / DT;
    const int dq = p.d0[q], last = p.nreal[q] - 1;
    for (int g = 0; g < groups; ++g) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        // padding taps read the rows of the last tap that exists: finite values times zero weights
        const int d = dq + min(g * DT + dt, last);
        const int trow = SS == 1 ? d : (d & 1) * p.half + (d >> 1);
        const int toff = trow * CPR;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          bf16x8 a[T1_NB];
#pragma unroll
          for (int b = 0; b < T1_NB; ++b) a[b] = __builtin_bit_cast(bf16x8, ap[b][toff + 2 * ks]);
          const bf16x8 w8 = __builtin_bit_cast(bf16x8, bq[dt][ks]);
          bq[dt][ks] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wlane, wpos + (dt * KS + ks) * 1024, 0);
#pragma unroll
          for (int b = 0; b < T1_NB; ++b) ac[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[b], w8, ac[b], 0, 0, 0);
        }
      }
      wpos += DT * KS * 1024;
    }
  };
  run(acc[0], 0);
  if (NPH == 2) run(acc[NPH - 1], 1);

  // ---- results: element r of block b: result index o0 + 32 b + 8 (r / 4) + 4 fg + r % 4 of channel m
  const int m = mtile * T1_BM + wave * 32 + fr;
  if (m >= p.Mo) return;
  const float bv = bias ? bias[m] : 0.f;
  const int n = row / p.H, h = row - n * p.H;
  const long long rbase = (((long long)n * p.Mo + m) * p.H + h) * p.TOu;     // element offset of the result row
  const __amdgpu_buffer_rsrc_t drs = make_rsrc(dst, p.dst_bytes);
  const bool even = (rbase & 1) == 0;
#pragma unroll
  for (int b = 0; b < T1_NB; ++b)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int o = o0 + b * 32 + g4 * 8 + fg * 4;
      float v[4 * NPH];
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int q = 0; q < NPH; ++q) v[e * NPH + q] = acc[q][b][4 * g4 + e] + bv;
      const int u = o * NPH;
      if (even && u + 4 * NPH <= p.TOu) {      // (u is a multiple of 4: with an even row offset the piece is 4-byte aligned)
        if (NPH == 1) {
          const uintx2_t t = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
          __builtin_amdgcn_raw_buffer_store_b64(t, drs, (int)((rbase + u) * 2), 0, 0);
        } else {
          const uintx4_t t = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4 * (NPH - 1)], v[4 * (NPH - 1) + 1]),
                              pack_bf16(v[4 * (NPH - 1) + 2], v[4 * (NPH - 1) + 3])};
          __builtin_amdgcn_raw_buffer_store_b128(t, drs, (int)((rbase + u) * 2), 0, 0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4 * NPH; ++e)
          if (u + e < p.TOu) dst[rbase + u + e] = f32_to_bf16(v[e]);
      }
    }
}

// ---- host side ---------------------------------------------------------------------------
struct Tap1Plan {
  Tap1Params p;
  Tap1Weights w;
  int SS, DT;
  size_t rows_bytes, w_bytes, lds_bytes;
  int C, H, T;           // of the source tensor, for the rows pass
};

int dt_of(int KS) { return KS >= 16 ? 1 : KS >= 8 ? 2 : KS == 6 ? 3 : KS == 4 ? 4 : KS == 2 ? 8 : 0; }

// bwd = false: forward; true: backward-data
bool tap1d_plan(const ConvGeom& g, bool bwd, Tap1Plan* pl) {
  if (g.KH != 1 || g.py != 0 || g.sy != 1 || g.dlx != 1 || g.groups != 1) return false;
  if (g.KW < 2 || g.KW > 32 || (g.sx != 1 && g.sx != 2)) return false;
  if (g.OH != g.H || (long long)g.N * g.H > 65535) return false;
  const int Cc = bwd ? g.K : g.C, Mo = bwd ? g.C : g.K;
  // contraction channels padded to a count the kernel is compiled for
  int Cs = 0;
  for (int c : {32, 64, 96, 128, 256})
    if (Cc <= c) { Cs = c; break; }
  if (!Cs || Cc < 16) return false;
  const int KS = Cs / 16, DT = dt_of(KS);
  Tap1Params& p = pl->p;
  Tap1Weights& w = pl->w;
  std::memset(&p, 0, sizeof p);
  std::memset(&w, 0, sizeof w);
  p.rows = g.N * g.H; p.H = g.H;
  p.Cs = Cs; p.KS = KS; p.Mo = Mo;
  int soff[2] = {0, 0};
  if (!bwd) {
    pl->SS = g.sx; p.nph = 1;
    p.TS = g.W; p.TO = g.OW; p.TOu = g.OW;
    p.nreal[0] = g.KW; soff[0] = -g.px;
    for (int i = 0; i < g.KW; ++i) w.tapj[i] = (signed char)i;
  } else if (g.sx == 1) {
    pl->SS = 1; p.nph = 1;
    p.TS = g.OW; p.TO = g.W; p.TOu = g.W;
    p.nreal[0] = g.KW; soff[0] = g.px - (g.KW - 1);
    for (int i = 0; i < g.KW; ++i) w.tapj[i] = (signed char)(g.KW - 1 - i);
  } else {
    // u = 2 v + q takes the taps j = jq + 2 i' with jq = (q + px) & 1, from dy[v + (q + px - jq) / 2 - i']
    pl->SS = 1; p.nph = 2;
    p.TS = g.OW; p.TO = (g.W + 1) / 2; p.TOu = g.W;
    for (int q = 0; q < 2; ++q) {
      const int jq = (q + g.px) & 1;
      p.nreal[q] = (g.KW - jq + 1) / 2;
      if (p.nreal[q] < 1) return false;
      soff[q] = (q + g.px - jq) / 2 - (p.nreal[q] - 1);
    }
  }
  int stored = 0;
  for (int q = 0; q < p.nph; ++q) {
    p.ntaps[q] = (p.nreal[q] + DT - 1) / DT * DT;
    if (bwd && g.sx == 2) {
      const int jq = (q + g.px) & 1;
      for (int i = 0; i < p.ntaps[q]; ++i) w.tapj[stored + i] = (signed char)(i < p.nreal[q] ? jq + 2 * (p.nreal[q] - 1 - i) : -1);
    } else {
      for (int i = p.nreal[q]; i < p.ntaps[q]; ++i) w.tapj[stored + i] = -1;
    }
    stored += p.ntaps[q];
  }
  if (stored > T1_MAXTAPS) return false;
  p.taps_total = stored;
  p.smin = p.nph == 2 ? std::min(soff[0], soff[1]) : soff[0];
  int span = 0;
  for (int q = 0; q < p.nph; ++q) {
    p.d0[q] = soff[q] - p.smin;
    span = std::max(span, p.d0[q] + p.nreal[q]);
  }
  if (pl->SS == 1) {
    p.SR = T1_TP + span - 1;
    p.half = 0;
  } else {
    p.half = ((2 * (T1_TP - 1) + span - 1) >> 1) + 1;
    p.SR = 2 * p.half;
  }
  const int CPR = 2 * KS + 1;
  pl->lds_bytes = (size_t)(((long long)p.SR * CPR + 63) / 64) * 1024;
  if (pl->lds_bytes > 160 * 1024) return false;
  p.ptiles = (p.TO + T1_TP - 1) / T1_TP;
  p.mtiles = (Mo + T1_BM - 1) / T1_BM;
  const long long rb = (long long)p.rows * p.TS * Cs * 2;
  const long long wb = (long long)p.mtiles * (T1_BM / 32) * stored * KS * 1024;
  const long long db = (long long)g.N * Mo * g.H * p.TOu * 2;
  if (rb >= (1ll << 31) || wb >= (1ll << 31) || db >= (1ll << 31)) return false;
  p.src_bytes = (unsigned)rb; p.w_bytes = (unsigned)wb; p.dst_bytes = (unsigned)db;
  pl->rows_bytes = ((size_t)rb + 255) & ~(size_t)255;
  pl->w_bytes = (size_t)wb;
  w.Mo = Mo; w.Cc = Cc; w.KS = KS; w.taps_total = stored; w.bwd = bwd ? 1 : 0;
  w.Cw = g.C; w.KW = g.KW; w.mblocks = p.mtiles * (T1_BM / 32);
  pl->DT = DT;
  pl->C = Cc; pl->H = g.H; pl->T = p.TS;
  return true;
}

template <int KS, int DT>
int launch_conv(const Tap1Plan& pl, const bf16_t* xr, const uintx4_t* wf, const float* bias, bf16_t* dst, hipStream_t s) {
  const dim3 grid((unsigned)(pl.p.rows * pl.p.ptiles), (unsigned)pl.p.mtiles);
  auto go = [&](auto kernel) {
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), pl.lds_bytes)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(256), pl.lds_bytes, s, pl.p, xr, wf, bias, dst);
    return check_launch("conv2d (bf16 one-row windows)");
  };
  if (pl.p.nph == 2) return go(tap1d16_conv_kernel<KS, DT, 1, 2>);
  if (pl.SS == 2) return go(tap1d16_conv_kernel<KS, DT, 2, 1>);
  return go(tap1d16_conv_kernel<KS, DT, 1, 1>);
}

int run_conv(const ConvGeom& g, bool bwd, const void* src, const void* w, const float* bias, void* dst, hipStream_t s,
             void* ws, size_t ws_bytes) {
  Tap1Plan pl;
  if (!tap1d_plan(g, bwd, &pl)) return -1;
  if (!ws || ws_bytes < pl.rows_bytes + pl.w_bytes) return -1;
  bf16_t* xr = static_cast<bf16_t*>(ws);
  uintx4_t* wf = reinterpret_cast<uintx4_t*>(static_cast<char*>(ws) + pl.rows_bytes);
  {
    const dim3 grid((unsigned)((pl.T + 63) / 64), (unsigned)(pl.p.Cs / 32), (unsigned)pl.p.rows);
    hipLaunchKernelGGL(tap1d16_rows_kernel, grid, dim3(256), 0, s, static_cast<const bf16_t*>(src), xr, pl.C, pl.H, pl.T, pl.p.Cs);
  }
  {
    const long long total = (long long)pl.w.mblocks * pl.w.taps_total * pl.w.KS * 64;
    hipLaunchKernelGGL(tap1d16_weights_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       static_cast<const bf16_t*>(w), wf, pl.w);
  }
  if (const int rc = check_launch("conv2d (bf16 one-row windows, operand passes)")) return rc;
  bf16_t* out = static_cast<bf16_t*>(dst);
  switch (pl.p.KS) {
    case 2: return launch_conv<2, 8>(pl, xr, wf, bias, out, s);
    case 4: return launch_conv<4, 4>(pl, xr, wf, bias, out, s);
    case 6: return launch_conv<6, 3>(pl, xr, wf, bias, out, s);
    case 8: return launch_conv<8, 2>(pl, xr, wf, bias, out, s);
    default: return launch_conv<16, 1>(pl, xr, wf, bias, out, s);
  }
}

}  // namespace

size_t mfma_tap1d16_conv_ws(const ConvGeom& g, bool bwd) {
  Tap1Plan pl;
  return tap1d_plan(g, bwd, &pl) ? pl.rows_bytes + pl.w_bytes : 0;
}

int mfma_tap1d16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                          void* ws, size_t ws_bytes) {
  return run_conv(g, false, x, w, bias, y, s, ws, ws_bytes);
}

int mfma_tap1d16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s, void* ws,
                               size_t ws_bytes) {
  return run_conv(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
}

}  // namespace flhip
