// Convolutions with one-row windows (KH = 1, KW taps along the contiguous axis: the 21 x 1
// windows of a wav2letter-style speech stack) on the matrix cores, forward, backward-data and
// filter gradient, column stride 1 or 2; bf16 storage on v_mfma_f32_32x32x16_bf16 and fp32 on
// v_mfma_f32_32x32x2_f32 (the same kernels compiled for either element type).
//
//   forward        y[m][o]  = sum_c sum_j w[m][c][j]  x[c][o*s + j - p]   (+ bias[m])
//   backward-data  dx[c][u] = sum_m sum_j w[m][c][j] dy[m][(u + p - j) / s]   where s divides
//
// A matrix instruction wants consecutive contraction channels of one position per lane, and
// every tap shifts the positions by one element: with the tensors as they lie in memory
// (channel-major rows of positions) a shifted 16-byte fragment would start on any element
// boundary.  So two small passes first bring the operands into the order the instruction reads:
//   rows     xr[sequence][position][Cs]: the source with its channels last, Cs = the channel
//            count padded with zeros (tap1d_rows_kernel; a sequence is one (image, row) pair); a
//            tap then shifts whole 16-byte cells (8 bf16 or 4 fp32 channels of one position);
//   weights  wf[block of 32 result channels][tap][stage of 2 cells][lane][cell]: the fragment
//            of every (tap, stage) exactly as the 64 lanes hold it, in the order the kernel walks
//            (tap1d_weights_kernel); padded channels and taps are zero.
// A stage is 16 bf16 channels (one matrix instruction per block) or 8 fp32 channels (four
// instructions of 2 channels each: lane half h holds channels 4 h .. 4 h + 3 of the stage and
// instruction e multiplies element e of both operands, so the four cover the stage).
// Backward-data over a stride of 2 is two interleaved stride-1 problems (the results of even
// and of odd index take the taps of one parity each): "phases" of one workgroup, which
// writes both so that its stores cover whole runs of dx.
//
// A workgroup (4 waves) owns 32 NB result positions (per phase; NB = 3, or 2 where the slab of 3
// would not fit) of one sequence x 128 result channels; wave w owns channels 32 w .. 32 w + 31:
// NB (2 NB) accumulator blocks of 32 x 32.
//   * The source rows the tile needs (its positions + the window's reach, every channel) are
//     copied to LDS once, by buffer loads with the LDS modifier (no registers, no vector
//     instructions); a row of the slab is its cells + 1 unused cell, which puts the eight
//     lanes of a 16-byte read cycle on distinct banks.  With a forward stride of 2 the slab
//     keeps even and odd source positions apart, so a tap's 32 positions are consecutive rows.
//   * The weights never pass through LDS: a wave's fragment of a (tap, stage) is 1 KiB of
//     contiguous memory, fetched straight into registers RW stages ahead of its use.  No other
//     wave needs it, so the main loop has no barrier.
//   * Per stage a wave reads NB position fragments from LDS (two stages ahead of their use) and
//     issues NB (bf16) or 4 NB (fp32) matrix instructions.
// Positions are the rows of the instruction tile: a lane holds 4 consecutive positions of one
// result channel (8 with two phases), stored as one piece.
#include <algorithm>
#include <cstring>

#include "conv2d_mfma.h"
#include "lds_direct.h"

namespace flhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const uintx4_t* lds_cell_t;
#else
typedef const uintx4_t* lds_cell_t;
#endif

constexpr int T1_BM = 128;       // result channels per workgroup
constexpr int T1_MAXTAPS = 64;   // taps over both phases, padding included
constexpr int T1_OOB = (int)0x80000000;

// element type -> channels per 16-byte cell; a stage is two cells
template <typename T> struct Tap1Elem;
template <> struct Tap1Elem<bf16_t> { static constexpr int CELL = 8; };
template <> struct Tap1Elem<f16_t> { static constexpr int CELL = 8; };
template <> struct Tap1Elem<float> { static constexpr int CELL = 4; };

// one stage of one block: acc += a (positions x stage channels) * w (stage channels x result channels)
__device__ __forceinline__ void tap1d_mma(floatx16& acc, const uintx4_t& a, const uintx4_t& w, const bf16_t*) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, w), acc, 0, 0, 0);
}
__device__ __forceinline__ void tap1d_mma(floatx16& acc, const uintx4_t& a, const uintx4_t& w, const f16_t*) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, w), acc, 0, 0, 0);
}
// two results rounded to the storage type, the first in the low half
__device__ __forceinline__ uint32_t tap1d_pack(float a, float b, const bf16_t*) { return pack_bf16(a, b); }
__device__ __forceinline__ uint32_t tap1d_pack(float a, float b, const f16_t*) { return pack_f16(a, b); }
__device__ __forceinline__ uint32_t tap1d_pack(float, float, const float*) { return 0u; }   // (fp32 results are not packed)
__device__ __forceinline__ void tap1d_mma(floatx16& acc, const uintx4_t& a, const uintx4_t& w, const float*) {
#pragma unroll
  for (int e = 0; e < 4; ++e)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[e]), __uint_as_float(w[e]), acc, 0, 0, 0);
}

struct Tap1Params {
  int rows, H;           // sequences (images x rows), rows per image
  int TS, TO, TOu;       // source positions, result indices per phase, result positions per sequence
  int Cs, KS;            // padded contraction channels, stages per tap
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
  // two-dimensional windows over stacked planes (tap2d_*): taps per window row, slab rows per window row = the
  // pitch of a plane's row, and the plane's geometry for the results
  int tw, tpitch, pW, pH, pN;
};

// ---- operand passes ------------------------------------------------------------------------
// x[n][c][h][t] -> xr[n * H + h][t][Cs], channels c >= C zero.  A block transposes 64 channels x 64
// positions through LDS: (bf16: pairs of positions in, where rows of an even length start on 4-byte
// boundaries;) whole 16-byte cells out.
template <typename T, bool PAIRS>
__global__ void __launch_bounds__(256)
tap1d_rows_kernel(const T* __restrict__ x, T* __restrict__ xr, int C, int H, int Tn, int Cs) {
  constexpr int CELL = Tap1Elem<T>::CELL;
  __shared__ T tile[64][sizeof(T) == 2 ? 66 : 65];
  const int t0 = blockIdx.x * 64, c0 = blockIdx.y * 64, row = blockIdx.z;
  const int n = row / H, h = row - n * H;
  if (PAIRS && sizeof(T) == 2) {
    const int tp = threadIdx.x & 31, cy = threadIdx.x >> 5;      // pair of positions, channel (+ 8 i)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = c0 + cy + 8 * i, t = t0 + 2 * tp;
      uint32_t v = 0u;
      if (c < C && t < Tn) v = *reinterpret_cast<const uint32_t*>(x + (((size_t)n * C + c) * H + h) * Tn + t);   // (Tn is even)
      *reinterpret_cast<uint32_t*>(&tile[cy + 8 * i][2 * tp]) = v;
    }
  } else {
    const int tx = threadIdx.x & 63, cy = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int c = c0 + cy + 4 * i, t = t0 + tx;
      tile[cy + 4 * i][tx] = (c < C && t < Tn) ? x[(((size_t)n * C + c) * H + h) * Tn + t] : T{};
    }
  }
  __syncthreads();
  constexpr int CPT = 64 / CELL;                // cells per position of the tile
#pragma unroll
  for (int i = 0; i < CPT * 64 / 256; ++i) {
    const int item = threadIdx.x + 256 * i, cell = item % CPT, tl = item / CPT;
    const int t = t0 + tl, c = c0 + CELL * cell;
    if (t < Tn && c < Cs) {
      __attribute__((aligned(16))) T v[CELL];
#pragma unroll
      for (int e = 0; e < CELL; ++e) v[e] = tile[CELL * cell + e][tl];
      *reinterpret_cast<uintx4_t*>(xr + ((size_t)row * Tn + t) * Cs + c) = *reinterpret_cast<const uintx4_t*>(v);
    }
  }
}

template <typename T>
static void launch_rows(const T* x, T* xr, int C, int H, int Tn, int Cs, int rows, hipStream_t s) {
  const dim3 grid((unsigned)((Tn + 63) / 64), (unsigned)((Cs + 63) / 64), (unsigned)rows);
  if (sizeof(T) == 2 && Tn % 2 == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0)
    hipLaunchKernelGGL((tap1d_rows_kernel<T, true>), grid, dim3(256), 0, s, x, xr, C, H, Tn, Cs);
  else
    hipLaunchKernelGGL((tap1d_rows_kernel<T, false>), grid, dim3(256), 0, s, x, xr, C, H, Tn, Cs);
}

struct Tap1Weights {
  int Mo, Cc;            // result / contraction channels that exist
  int KS, taps_total;
  int bwd;               // 0: w[m][c][j], 1: w[c][m][j] (contraction over the filters)
  int Cw, KW;            // channels per filter and taps of the weight tensor
  int mblocks;
  signed char tapj[T1_MAXTAPS];   // weight tap of stored tap i (-1: padding)
};

template <typename T>
__global__ void __launch_bounds__(256)
tap1d_weights_kernel(const T* __restrict__ w, uintx4_t* __restrict__ wf, Tap1Weights p) {
  constexpr int CELL = Tap1Elem<T>::CELL;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)p.mblocks * p.taps_total * p.KS * 64;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const long long st = idx >> 6;
  const int per_block = p.taps_total * p.KS;
  const int mblk = (int)(st / per_block), s = (int)(st - (long long)mblk * per_block);
  const int tap = s / p.KS, ks = s - tap * p.KS;
  const int m = mblk * 32 + (lane & 31), c0 = (2 * ks + (lane >> 5)) * CELL;
  const int j = p.tapj[tap];
  __attribute__((aligned(16))) T v[CELL];
#pragma unroll
  for (int e = 0; e < CELL; ++e) {
    const int c = c0 + e;
    v[e] = T{};
    if (j >= 0 && m < p.Mo && c < p.Cc)
      v[e] = w[p.bwd ? ((size_t)c * p.Cw + m) * p.KW + j : ((size_t)m * p.Cw + c) * p.KW + j];
  }
  wf[idx] = *reinterpret_cast<const uintx4_t*>(v);
}

// The same fragments with the tap as the index that changes fastest after the lane: the four waves of a block then read
// the same cache lines (a lane's 8 or 4 contraction channels x 9 taps are neighbours in memory), where in the order
// above - the stage fastest - every line is met once per tap by a different block.
template <typename T>
__global__ void __launch_bounds__(256)
tap_weights_by_tap_kernel(const T* __restrict__ w, uintx4_t* __restrict__ wf, Tap1Weights p) {
  constexpr int CELL = Tap1Elem<T>::CELL;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long total = (long long)p.mblocks * p.taps_total * p.KS * 64;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const long long st = idx >> 6;
  const int tap = (int)(st % p.taps_total);
  const long long r2 = st / p.taps_total;
  const int ks = (int)(r2 % p.KS), mblk = (int)(r2 / p.KS);
  const int m = mblk * 32 + (lane & 31), c0 = (2 * ks + (lane >> 5)) * CELL;
  const int j = p.tapj[tap];
  __attribute__((aligned(16))) T v[CELL];
#pragma unroll
  for (int e = 0; e < CELL; ++e) {
    const int c = c0 + e;
    v[e] = T{};
    if (j >= 0 && m < p.Mo && c < p.Cc)
      v[e] = w[p.bwd ? ((size_t)c * p.Cw + m) * p.KW + j : ((size_t)m * p.Cw + c) * p.KW + j];
  }
  wf[(((long long)mblk * p.taps_total + tap) * p.KS + ks) * 64 + lane] = *reinterpret_cast<const uintx4_t*>(v);
}

// ---- the convolution ---------------------------------------------------------------------
// KS stages per tap; DT taps per unrolled group; RW stages between a weight fragment's load and its use (RW divides
// DT * KS; a bf16 stage is one matrix instruction per block, an fp32 stage four longer ones); SS source stride;
// NPH phases; NB blocks of 32 positions.
// TD: the taps form a two-dimensional window over planes stacked in one sequence (see tap2d_plan); only the slab
// offset of a tap and the addresses of the results differ.
template <typename T, int KS, int DT, int RW, int SS, int NPH, int NB, bool TD>
__device__ __forceinline__ void
tap_conv_body(const Tap1Params& p, const T* __restrict__ xr, const uintx4_t* __restrict__ wf,
              const float* __restrict__ bias, T* __restrict__ dst) {
  extern __shared__ uintx4_t t1_slab[];
  constexpr int CELL = Tap1Elem<T>::CELL;
  constexpr int ESZ = (int)sizeof(T);
  constexpr int CPR = 2 * KS + 1;               // cells per slab row
  constexpr int TP = 32 * NB;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ptile = __builtin_amdgcn_readfirstlane(blockIdx.x % p.ptiles);
  const int row = __builtin_amdgcn_readfirstlane(blockIdx.x / p.ptiles);
  const int mtile = blockIdx.y;
  const int o0 = ptile * TP;
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
      if (R < p.SR && c < 2 * KS && (unsigned)sp < (unsigned)p.TS) voff = ((row * p.TS + sp) * p.Cs + CELL * c) * ESZ;
      pd_load_lds(xrs, base + ii * 1024, voff, 0);
    }
  }

  // ---- weights: this wave's stream of fragments, RW stages ahead
  constexpr int NS = DT * KS;
  static_assert(NS % 4 == 0 && NS % RW == 0 && KS >= 2, "fragment sets and the weight ring rotate with the unrolled group");
  const __amdgpu_buffer_rsrc_t wrs = make_rsrc(wf, p.w_bytes);
  const int mblk = mtile * (T1_BM / 32) + wave;
  int wpos = mblk * p.taps_total * KS * 1024;   // byte offset of the stage RW ahead of the group's first
  const int wlane = lane * 16;
  uintx4_t bq[RW];
#pragma unroll
  for (int i = 0; i < RW; ++i) bq[i] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wlane, wpos + i * 1024, 0);
  wpos += RW * 1024;

  floatx16 acc[NPH][NB];
#pragma unroll
  for (int q = 0; q < NPH; ++q)
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[q][b][r] = 0.f;

  const int fr = lane & 31, fg = lane >> 5;
  lds_cell_t ap[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) ap[b] = (lds_cell_t)t1_slab + ((b * 32 + fr) * CPR + fg);

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the slab (and the first weight fragments) have landed
  __syncthreads();

  // The position fragments of a stage are read two stages ahead of their use (four sets of registers in rotation;
  // a group's stage count is a multiple of four).
  auto run = [&](floatx16 (&ac)[NB], int q) __attribute__((always_inline)) {
    const int groups = p.ntaps[q] / DT;
    const int dq = p.d0[q], last = p.nreal[q] - 1;
    // slab offset (cells) of a tap's rows; padding taps read the rows of the last tap that exists: finite values
    // times zero weights
    auto toff_of = [&](int tap) {
      const int tl = min(tap, last);
      const int d = dq + (TD ? (tl / p.tw) * p.tpitch + tl % p.tw : tl);
      const int trow = SS == 1 ? d : (d & 1) * p.half + (d >> 1);
      return trow * CPR;
    };
    uintx4_t af[4][NB];
    int tcur[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) tcur[dt] = toff_of(dt);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int b = 0; b < NB; ++b) af[i][b] = ap[b][tcur[i / KS] + 2 * (i % KS)];
    for (int g = 0; g < groups; ++g) {
      int tnext[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) tnext[dt] = toff_of((g + 1) * DT + dt);
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int i2 = i + 2;
        const int o2 = i2 < NS ? tcur[(i2 % NS) / KS] : tnext[(i2 % NS) / KS];
#pragma unroll
        for (int b = 0; b < NB; ++b) af[i2 % 4][b] = ap[b][o2 + 2 * ((i2 % NS) % KS)];
        const uintx4_t w8 = bq[i % RW];
        bq[i % RW] = __builtin_amdgcn_raw_buffer_load_b128(wrs, wlane, wpos + i * 1024, 0);
#pragma unroll
        for (int b = 0; b < NB; ++b) tap1d_mma(ac[b], af[i % 4][b], w8, static_cast<const T*>(nullptr));
        __builtin_amdgcn_sched_barrier(0);     // (the scheduler would otherwise move every read down to its use)
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) tcur[dt] = tnext[dt];
      wpos += NS * 1024;
    }
  };
  run(acc[0], 0);
  if (NPH == 2) run(acc[NPH - 1], 1);

  // ---- results: element r of block b: result index o0 + 32 b + 8 (r / 4) + 4 fg + r % 4 of channel m
  const int m = mtile * T1_BM + wave * 32 + fr;
  if constexpr (TD) {
    // Results through LDS (the slab is done with): every wave parks its 32 channels x 32 NB positions at storage size,
    // then threads walk positions (consecutive lanes = consecutive positions = consecutive addresses inside a plane's
    // row, and across row ends too: the zero column has no address) with the position's plane / row / column worked
    // out once per thread.  Position o of the sequence = row o / pitch (row 0 and every (pH + 1)-th after it are the
    // zero rows between the planes), column o % pitch (the last one of a row is the zero column).
    constexpr int TPOS = 32 * NB;
    constexpr int SPT = TPOS + 4;                 // staging pitch (elements): 8-byte rows, lanes on distinct banks
    T* const stage = reinterpret_cast<T*>(t1_slab);
    const float bvt = (bias && m < p.Mo) ? bias[m] : 0.f;
    __syncthreads();
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        T* const at = stage + (wave * 32 + fr) * SPT + b * 32 + g4 * 8 + fg * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) st(at, e, acc[0][b][4 * g4 + e] + bvt);
      }
    __syncthreads();
    if (tid >= 2 * TPOS) return;
    const int pos = tid % TPOS, cg = tid / TPOS;
    const int o = o0 + pos;
    const int P = p.tpitch, H1 = p.pH + 1;
    const int prow = o / P, col = o - prow * P;
    const int n = max(prow - 1, 0) / H1, h = max(prow - 1, 0) - n * H1;
    if (!(prow >= 1 && n < p.pN && h < p.pH && col < p.pW)) return;
    const int mlim = min(T1_BM, p.Mo - mtile * T1_BM);
    const size_t plane = (size_t)p.pH * p.pW;
    T* const out = dst + ((size_t)n * p.Mo + mtile * T1_BM) * plane + (size_t)h * p.pW + col;
    for (int c = cg; c < mlim; c += 2) out[(size_t)c * plane] = stage[c * SPT + pos];
    return;
  }
  if (m >= p.Mo) return;
  const float bv = bias ? bias[m] : 0.f;
  const int n = row / p.H, h = row - n * p.H;
  const long long rbase = (((long long)n * p.Mo + m) * p.H + h) * p.TOu;     // element offset of the result row
  const __amdgpu_buffer_rsrc_t drs = make_rsrc(dst, p.dst_bytes);
  const bool aligned = ESZ == 4 || (rbase & 1) == 0;     // pieces start on 4-byte boundaries
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int o = o0 + b * 32 + g4 * 8 + fg * 4;
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int q = 0; q < NPH; ++q) v[e * NPH + q] = acc[q][b][4 * g4 + e] + bv;
      const int u = o * NPH;
      if (aligned && u + 4 * NPH <= p.TOu) {      // (u is a multiple of 4)
        const int at = (int)((rbase + u) * ESZ);
        if (ESZ == 4) {
          __builtin_amdgcn_raw_buffer_store_b128(uintx4_t{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])}, drs, at, 0, 0);
          if (NPH == 2)
            __builtin_amdgcn_raw_buffer_store_b128(uintx4_t{__float_as_uint(v[4]), __float_as_uint(v[5]), __float_as_uint(v[6]), __float_as_uint(v[7])}, drs, at + 16, 0, 0);
        } else if (NPH == 1) {
          const T* const tt = nullptr;
          const uintx2_t t = {tap1d_pack(v[0], v[1], tt), tap1d_pack(v[2], v[3], tt)};
          __builtin_amdgcn_raw_buffer_store_b64(t, drs, at, 0, 0);
        } else {
          const T* const tt = nullptr;
          const uintx4_t t = {tap1d_pack(v[0], v[1], tt), tap1d_pack(v[2], v[3], tt), tap1d_pack(v[4], v[5], tt), tap1d_pack(v[6], v[7], tt)};
          __builtin_amdgcn_raw_buffer_store_b128(t, drs, at, 0, 0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4 * NPH; ++e)
          if (u + e < p.TOu) st(dst, (size_t)(rbase + u + e), v[e]);
      }
    }
}

template <typename T, int KS, int DT, int RW, int SS, int NPH, int NB>
__global__ void __launch_bounds__(256, 1)
tap1d_conv_kernel(Tap1Params p, const T* __restrict__ xr, const uintx4_t* __restrict__ wf,
                  const float* __restrict__ bias, T* __restrict__ dst) {
  tap_conv_body<T, KS, DT, RW, SS, NPH, NB, false>(p, xr, wf, bias, dst);
}

// 3 x 3 windows of stride 1 over small planes (the 14 x 14 and 7 x 7 layers of a residual network): the same loop
// over a sequence that holds every plane of the batch, rows pH + 1 apart with a zero row between two planes, a row's
// pW positions followed by one zero column (tap2d_rows_kernel writes it so) - the window's taps are then nine fixed
// offsets into the sequence, and the zero row / column are the padding.  Results at the zero positions are not stored.
template <typename T, int KS, int DT, int RW, int NB>
__global__ void __launch_bounds__(256, 1)
tap2d_conv_kernel(Tap1Params p, const T* __restrict__ xr, const uintx4_t* __restrict__ wf,
                  const float* __restrict__ bias, T* __restrict__ dst) {
  tap_conv_body<T, KS, DT, RW, 1, 1, NB, true>(p, xr, wf, bias, dst);
}

// x[n][c][h][w] -> xr[position][Cs] with position = ((n (H + 1) + 1 + h) P + w), P = W + 1; the zero rows, the zero
// column and channels c >= C are written as zeros.  A block transposes 64 channels x 64 positions through LDS.
template <typename T>
__global__ void __launch_bounds__(256)
tap2d_rows_kernel(const T* __restrict__ x, T* __restrict__ xr, int C, int H, int W, int N, int TS, int Cs) {
  constexpr int CELL = Tap1Elem<T>::CELL;
  __shared__ T tile[64][sizeof(T) == 2 ? 66 : 65];
  const int t0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int P = W + 1, H1 = H + 1;
  {
    const int tx = threadIdx.x & 63, cy = threadIdx.x >> 6;
    const int t = t0 + tx;
    const int prow = t / P, col = t - prow * P;
    const int n = (prow - 1) / H1, h = (prow - 1) - n * H1;
    const bool ok = t < TS && prow >= 1 && n < N && h < H && col < W;
    const size_t at = ok ? ((size_t)n * C * H + h) * W + col : 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int c = c0 + cy + 4 * i;
      tile[cy + 4 * i][tx] = (ok && c < C) ? x[at + (size_t)c * H * W] : T{};
    }
  }
  __syncthreads();
  constexpr int CPT = 64 / CELL;
#pragma unroll
  for (int i = 0; i < CPT * 64 / 256; ++i) {
    const int item = threadIdx.x + 256 * i, cell = item % CPT, tl = item / CPT;
    const int t = t0 + tl, c = c0 + CELL * cell;
    if (t < TS && c < Cs) {
      __attribute__((aligned(16))) T v[CELL];
#pragma unroll
      for (int e = 0; e < CELL; ++e) v[e] = tile[CELL * cell + e][tl];
      *reinterpret_cast<uintx4_t*>(xr + (size_t)t * Cs + c) = *reinterpret_cast<const uintx4_t*>(v);
    }
  }
}

// ---- host side ---------------------------------------------------------------------------
struct Tap1Plan {
  Tap1Params p;
  Tap1Weights w;
  int SS, DT, NB;
  size_t rows_bytes, w_bytes, lds_bytes;
  int C, H, T;           // of the source tensor, for the rows pass
};

// channels of the channels-last rows: the count padded to one the convolution kernels are compiled for
int tap1d_cs(int C) {
  for (int c : {32, 64, 96, 128, 256})
    if (C <= c) return c;
  return 0;
}

// taps per unrolled group of the bf16 kernels (fp32: 1)
int dt_of(int KS) { return KS >= 16 ? 1 : KS >= 8 ? 2 : KS == 6 ? 2 : KS == 4 ? 4 : KS == 2 ? 8 : 0; }

// bwd = false: forward; true: backward-data.  esz: bytes per element (2: bf16, 4: fp32)
bool tap1d_plan(const ConvGeom& g, bool bwd, int esz, Tap1Plan* pl) {
  if (g.KH != 1 || g.py != 0 || g.sy != 1 || g.dlx != 1 || g.groups != 1) return false;
  if (g.KW < 2 || g.KW > 32 || (g.sx != 1 && g.sx != 2)) return false;
  if (g.OH != g.H || (long long)g.N * g.H > 65535) return false;
  const int Cc = bwd ? g.K : g.C, Mo = bwd ? g.C : g.K;
  // contraction channels padded to a count the kernel is compiled for
  const int Cs = tap1d_cs(Cc);
  if (!Cs || Cc < 16) return false;
  const int cell = 16 / esz;
  const int KS = Cs / (2 * cell), DT = esz == 2 ? dt_of(KS) : 1;
  Tap1Params& p = pl->p;
  Tap1Weights& w = pl->w;
  std::memset(&p, 0, sizeof p);
  std::memset(&w, 0, sizeof w);
  p.rows = g.N * g.H; p.H = g.H;
  p.Cs = Cs; p.KS = KS; p.Mo = Mo;
  int soff[2] = {0, 0};
  if (!bwd) {
    pl->SS = g.sx; p.nph = 1;
    p.TS = g.W; p.TOu = g.OW;
    p.nreal[0] = g.KW; soff[0] = -g.px;
    for (int i = 0; i < g.KW; ++i) w.tapj[i] = (signed char)i;
  } else if (g.sx == 1) {
    pl->SS = 1; p.nph = 1;
    p.TS = g.OW; p.TOu = g.W;
    p.nreal[0] = g.KW; soff[0] = g.px - (g.KW - 1);
    for (int i = 0; i < g.KW; ++i) w.tapj[i] = (signed char)(g.KW - 1 - i);
  } else {
    // u = 2 v + q takes the taps j = jq + 2 i' with jq = (q + px) & 1, from dy[v + (q + px - jq) / 2 - i']
    pl->SS = 1; p.nph = 2;
    p.TS = g.OW; p.TOu = g.W;
    for (int q = 0; q < 2; ++q) {
      const int jq = (q + g.px) & 1;
      p.nreal[q] = (g.KW - jq + 1) / 2;
      if (p.nreal[q] < 1) return false;
      soff[q] = (q + g.px - jq) / 2 - (p.nreal[q] - 1);
    }
  }
  p.TO = (p.TOu + p.nph - 1) / p.nph;
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
  const int CPR = 2 * KS + 1;
  // three blocks of positions per wave; two where the slab of three does not fit (fp32, 256 channels, forward stride 2)
  pl->NB = 0;
  for (int nb = 3; nb >= 2 && !pl->NB; --nb) {
    const int tp = 32 * nb;
    if (pl->SS == 1) {
      p.SR = tp + span - 1;
      p.half = 0;
    } else {
      p.half = ((2 * (tp - 1) + span - 1) >> 1) + 1;
      p.SR = 2 * p.half;
    }
    pl->lds_bytes = (size_t)(((long long)p.SR * CPR + 63) / 64) * 1024;
    if (pl->lds_bytes <= 160 * 1024 && (nb == 3 || (esz == 4 && KS == 32 && pl->SS == 2))) pl->NB = nb;
  }
  if (!pl->NB) return false;
  p.ptiles = (p.TO + 32 * pl->NB - 1) / (32 * pl->NB);
  p.mtiles = (Mo + T1_BM - 1) / T1_BM;
  const long long rb = (long long)p.rows * p.TS * Cs * esz;
  const long long wb = (long long)p.mtiles * (T1_BM / 32) * stored * KS * 1024;
  const long long db = (long long)g.N * Mo * g.H * p.TOu * esz;
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

template <typename T, int KS, int DT, int RW>
int launch_conv(const Tap1Plan& pl, const T* xr, const uintx4_t* wf, const float* bias, T* dst, hipStream_t s) {
  const dim3 grid((unsigned)(pl.p.rows * pl.p.ptiles), (unsigned)pl.p.mtiles);
  auto go = [&](auto kernel) {
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), pl.lds_bytes)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(256), pl.lds_bytes, s, pl.p, xr, wf, bias, dst);
    return check_launch("conv2d (one-row windows)");
  };
  if (pl.NB == 2) {
    if constexpr (sizeof(T) == 4 && KS == 32) return go(tap1d_conv_kernel<T, KS, DT, RW, 2, 1, 2>);
    return -1;
  }
  if (pl.p.nph == 2) return go(tap1d_conv_kernel<T, KS, DT, RW, 1, 2, 3>);
  if (pl.SS == 2) return go(tap1d_conv_kernel<T, KS, DT, RW, 2, 1, 3>);
  return go(tap1d_conv_kernel<T, KS, DT, RW, 1, 1, 3>);
}

template <typename T>
int run_conv(const ConvGeom& g, bool bwd, const void* src, const void* w, const float* bias, void* dst, hipStream_t s,
             void* ws, size_t ws_bytes) {
  Tap1Plan pl;
  if (!tap1d_plan(g, bwd, (int)sizeof(T), &pl)) return -1;
  if (!ws || ws_bytes < pl.rows_bytes + pl.w_bytes) return -1;
  T* xr = static_cast<T*>(ws);
  uintx4_t* wf = reinterpret_cast<uintx4_t*>(static_cast<char*>(ws) + pl.rows_bytes);
  launch_rows(static_cast<const T*>(src), xr, pl.C, pl.H, pl.T, pl.p.Cs, pl.p.rows, s);
  {
    const long long total = (long long)pl.w.mblocks * pl.w.taps_total * pl.w.KS * 64;
    hipLaunchKernelGGL(tap1d_weights_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       static_cast<const T*>(w), wf, pl.w);
  }
  if (const int rc = check_launch("conv2d (one-row windows, operand passes)")) return rc;
  T* out = static_cast<T*>(dst);
  if constexpr (sizeof(T) == 2) {
    switch (pl.p.KS) {
      case 2: return launch_conv<T, 2, 8, 16>(pl, xr, wf, bias, out, s);
      case 4: return launch_conv<T, 4, 4, 16>(pl, xr, wf, bias, out, s);
      case 6: return launch_conv<T, 6, 2, 12>(pl, xr, wf, bias, out, s);
      case 8: return launch_conv<T, 8, 2, 16>(pl, xr, wf, bias, out, s);
      default: return launch_conv<T, 16, 1, 16>(pl, xr, wf, bias, out, s);
    }
  } else {
    switch (pl.p.KS) {
      case 4: return launch_conv<T, 4, 1, 4>(pl, xr, wf, bias, out, s);
      case 8: return launch_conv<T, 8, 1, 4>(pl, xr, wf, bias, out, s);
      case 12: return launch_conv<T, 12, 1, 4>(pl, xr, wf, bias, out, s);
      case 16: return launch_conv<T, 16, 1, 4>(pl, xr, wf, bias, out, s);
      default: return launch_conv<T, 32, 1, 4>(pl, xr, wf, bias, out, s);
    }
  }
}

// ---- 3 x 3 windows over small planes -------------------------------------------------------
// The sequence of tap2d_conv_kernel: N planes of H x W, each row followed by one zero column (pitch P = W + 1), one
// zero row before every plane and one after the last: TS = (N (H + 1) + 1) P positions.  Result position o takes tap
// (r, s) from position o + (r - 1) P + (s - 1): the slab of a tile starts P + 1 positions before its first result and
// tap 3 r + s sits r P + s rows into it.  Backward-data is the same walk over dy with the taps in reverse order and
// the roles of the two channel counts exchanged.  (H + 1)(W + 1) / (H W) of the positions are computed: 1.15 for
// 14 x 14 planes, 1.31 for 7 x 7.
bool tap2d_plan(const ConvGeom& g, bool bwd, int esz, Tap1Plan* pl) {
  if (g.KH != 3 || g.KW != 3 || g.sy != 1 || g.sx != 1 || g.py != 1 || g.px != 1 || g.dly != 1 || g.dlx != 1 || g.groups != 1)
    return false;
  const int Cc = bwd ? g.K : g.C, Mo = bwd ? g.C : g.K;
  // contraction channels padded to a count the two-dimensional kernel is compiled for
  int Cs = 0;
  for (int c : {128, 256, 512})
    if (!Cs && Cc <= c && (esz == 2 || c <= 256)) Cs = c;
  if (!Cs || Cc <= Cs / 2) return false;
  const int cell = 16 / esz;
  const int KS = Cs / (2 * cell), DT = esz == 2 ? dt_of(KS) : 1;
  Tap1Params& p = pl->p;
  Tap1Weights& w = pl->w;
  std::memset(&p, 0, sizeof p);
  std::memset(&w, 0, sizeof w);
  const int P = g.W + 1;
  const long long ts = ((long long)g.N * (g.H + 1) + 1) * P;
  if (ts >= (1ll << 22) - 256) return false;
  p.rows = 1; p.H = 1;
  p.Cs = Cs; p.KS = KS; p.Mo = Mo;
  p.nph = 1;
  p.TS = (int)ts; p.TOu = p.TS; p.TO = p.TS;
  p.nreal[0] = 9;
  p.ntaps[0] = (9 + DT - 1) / DT * DT;
  p.taps_total = p.ntaps[0];
  p.d0[0] = 0;
  p.smin = -(P + 1);
  p.tw = 3; p.tpitch = P; p.pW = g.W; p.pH = g.H; p.pN = g.N;
  for (int i = 0; i < p.ntaps[0]; ++i) w.tapj[i] = (signed char)(i < 9 ? (bwd ? 8 - i : i) : -1);
  const int CPR = 2 * KS + 1;
  // three blocks of positions per wave; two where three would leave compute units without a workgroup
  // (7 x 7 x 512 at batch 64: 172 workgroups of three blocks 43.0 / 40.9 us, 256 of two 41.3 / 39.1)
  const int mt = (Mo + T1_BM - 1) / T1_BM;
  pl->SS = 1; pl->DT = DT;
  pl->NB = (long long)((ts - P + 95) / 96) * mt < mfma_num_cus() ? 2 : 3;
  p.SR = 32 * pl->NB + 2 * P + 2;
  p.half = 0;
  // the slab; the results are staged in the same memory afterwards (128 channels x 100 elements)
  pl->lds_bytes = std::max((size_t)(((long long)p.SR * CPR + 63) / 64) * 1024, (size_t)T1_BM * (32 * pl->NB + 4) * esz);
  if (pl->lds_bytes > 160 * 1024) return false;
  p.ptiles = (p.TS - P + 32 * pl->NB - 1) / (32 * pl->NB);      // (the last zero row holds no result)
  p.mtiles = (Mo + T1_BM - 1) / T1_BM;
  const long long rb = ts * Cs * esz;
  const long long wb = (long long)p.mtiles * (T1_BM / 32) * p.taps_total * KS * 1024;
  const long long db = (long long)g.N * Mo * g.H * g.W * esz;
  if (rb >= (1ll << 31) || wb >= (1ll << 31) || db >= (1ll << 31)) return false;
  p.src_bytes = (unsigned)rb; p.w_bytes = (unsigned)wb; p.dst_bytes = (unsigned)db;
  pl->rows_bytes = ((size_t)rb + 255) & ~(size_t)255;
  pl->w_bytes = (size_t)wb;
  w.Mo = Mo; w.Cc = Cc; w.KS = KS; w.taps_total = p.taps_total; w.bwd = bwd ? 1 : 0;
  w.Cw = g.C; w.KW = 9; w.mblocks = p.mtiles * (T1_BM / 32);
  pl->C = Cc; pl->H = g.H; pl->T = g.W;
  return true;
}

template <typename T, int KS, int DT, int RW>
int launch_conv2d(const Tap1Plan& pl, const T* xr, const uintx4_t* wf, const float* bias, T* dst, hipStream_t s) {
  const dim3 grid((unsigned)pl.p.ptiles, (unsigned)pl.p.mtiles);
  auto go = [&](auto kernel) {
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), pl.lds_bytes)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(256), pl.lds_bytes, s, pl.p, xr, wf, bias, dst);
    return check_launch("conv2d (3x3 windows over stacked planes)");
  };
  return pl.NB == 2 ? go(tap2d_conv_kernel<T, KS, DT, RW, 2>) : go(tap2d_conv_kernel<T, KS, DT, RW, 3>);
}

template <typename T>
int run_conv2d(const ConvGeom& g, bool bwd, const void* src, const void* w, const float* bias, void* dst, hipStream_t s,
               void* ws, size_t ws_bytes) {
  Tap1Plan pl;
  if (!tap2d_plan(g, bwd, (int)sizeof(T), &pl)) return -1;
  if (!ws || ws_bytes < pl.rows_bytes + pl.w_bytes) return -1;
  T* xr = static_cast<T*>(ws);
  uintx4_t* wf = reinterpret_cast<uintx4_t*>(static_cast<char*>(ws) + pl.rows_bytes);
  {
    const dim3 grid((unsigned)((pl.p.TS + 63) / 64), (unsigned)((pl.p.Cs + 63) / 64));
    hipLaunchKernelGGL(tap2d_rows_kernel<T>, grid, dim3(256), 0, s, static_cast<const T*>(src), xr, pl.C, g.H, g.W, g.N, pl.p.TS,
                       pl.p.Cs);
    const long long total = (long long)pl.w.mblocks * pl.w.taps_total * pl.w.KS * 64;
    hipLaunchKernelGGL(tap_weights_by_tap_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       static_cast<const T*>(w), wf, pl.w);
  }
  if (const int rc = check_launch("conv2d (3x3 windows over stacked planes, operand passes)")) return rc;
  T* out = static_cast<T*>(dst);
  if constexpr (sizeof(T) == 2) {
    switch (pl.p.KS) {
      case 8: return launch_conv2d<T, 8, 2, 16>(pl, xr, wf, bias, out, s);
      case 16: return launch_conv2d<T, 16, 1, 16>(pl, xr, wf, bias, out, s);
      default: return launch_conv2d<T, 32, 1, 16>(pl, xr, wf, bias, out, s);
    }
  } else {
    return pl.p.KS == 16 ? launch_conv2d<T, 16, 1, 4>(pl, xr, wf, bias, out, s) : launch_conv2d<T, 32, 1, 4>(pl, xr, wf, bias, out, s);
  }
}

// ---- the filter gradient -------------------------------------------------------------------
//   dw[k][c][j] = sum over sequences and positions o of dy[k][o] x[c][o*s + j - p],  db[k] = sum dy[k][o]
// The contraction runs over positions, 16 per matrix instruction.  dy is read as it lies in
// memory (a lane's 8 consecutive positions of one filter are 16 contiguous bytes, fetched
// straight into registers a few steps ahead); x comes from the channels-last rows through LDS:
// a tap shifts whole slab rows, and transposing reads (ds_read_b64_tr_b16) hand every lane its
// 8 positions of one channel.  A workgroup (4 waves) owns 64 filters x 32 channels x every tap
// over a range of positions of one sequence (or several such ranges in turn); wave w owns the
// slots w TQ .. w TQ + TQ - 1 of both filter blocks, slot g being tap g for g < KW, the bias
// gradient (dy times a tile of ones) for g = KW and unused beyond: 2 x TQ accumulator blocks
// per wave (at most 192 registers, so they stay in the accumulator file), one slab fragment
// per two matrix instructions.
// The slab of a range (its positions and the window's reach, 32 channels) is copied to LDS by
// the loads themselves before the range's first step; rows are 6 cells apart for stride 1 and
// 5 for stride 2, which keeps the four rows of a transposing read on distinct banks.
// The workgroups' tiles go to the workspace as [range set][tile][slot][64 filters][32 channels]
// and tap1d_wgrad_reduce_kernel adds them in a fixed order into dw's memory order.
typedef short shortx4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4_t* lds_tr_t;

struct Tap1WParams {
  int rows, H;          // sequences, rows per image
  int OW, TS;           // positions of dy / of the source per sequence
  int Cs;               // channels of the channels-last source rows
  int K, C, KW, px;
  int tsplit, TL;       // ranges per sequence, positions per range (a multiple of 16)
  int units, upw;       // ranges over all sequences, ranges per workgroup
  int ktiles, ctiles;
  int SRW;              // slab rows
  unsigned src_bytes, dy_bytes;
};

template <typename T, int TQ, int SS>
__global__ void __launch_bounds__(256, 1)
tap1d_wgrad_kernel(Tap1WParams p, const T* __restrict__ xr, const T* __restrict__ dy, float* __restrict__ part) {
  extern __shared__ uintx4_t t1_slab[];
  constexpr int CELL = Tap1Elem<T>::CELL;
  constexpr int ESZ = (int)sizeof(T);
  constexpr bool LO = ESZ == 2;
  constexpr int STEP = 2 * CELL;                // positions per step: a lane half holds CELL consecutive ones
  constexpr int RC = 32 / CELL;                 // cells of a slab row in use (32 channels)
  constexpr int PC = LO ? (SS == 1 ? 6 : 5) : RC + 1;   // cells per slab row
  constexpr int PE = PC * CELL;                 // the same in elements
  constexpr int RD = 4;                         // steps between a dy fragment's load and its use
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x, tile = blockIdx.y;
  const int kt = tile / p.ctiles, ct = tile - kt * p.ctiles;
  const intx4_t xrs = pd_rsrc(xr, p.src_bytes);
  const __amdgpu_buffer_rsrc_t drs = make_rsrc(dy, p.dy_bytes);
  const unsigned slab_addr = pd_lds_addr(t1_slab);
  const int fr = lane & 31, fg = lane >> 5, fq = (lane >> 4) & 1, fs = lane & 15;

  floatx16 acc[2][TQ];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int t = 0; t < TQ; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][t][r] = 0.f;
  // a tile of ones for the bias slot
  const uint32_t one = !LO ? 0x3f800000u : std::is_same<T, f16_t>::value ? 0x3c003c00u : 0x3f803f80u;
  const uintx4_t ones = {one, one, one, one};
  const int bias_slot = p.KW - wave * TQ;       // this wave's slot index of the bias gradient (outside 0 .. TQ - 1: none)

  // this lane's first read of a step at the wave's first tap.  bf16: transposing reads, row SS * (fs / 4) (+ 8 SS fg),
  // channels 16 fq + 4 (fs % 4) .. + 3.  fp32: four 4-byte reads, rows SS * (4 fg + e), channel fr.
  const T* const slabT = reinterpret_cast<const T*>(t1_slab);
  const int blane = LO ? ((8 * fg + (fs >> 2)) * SS + wave * TQ) * PE + 16 * fq + 4 * (fs & 3)
                       : (4 * fg * SS + wave * TQ) * PE + fr;

  const int u0 = split * p.upw, u1 = min(u0 + p.upw, p.units);
  for (int u = u0; u < u1; ++u) {
    const int seq = u / p.tsplit, tr = u - seq * p.tsplit;
    const int t0 = tr * p.TL, oend = min(p.OW, t0 + p.TL);
    if (t0 >= oend) continue;
    const int nsteps = (oend - t0 + STEP - 1) / STEP;
    const int tailn = (oend - t0) % STEP;       // positions of a last, partial step (0: none)
    if (u != u0) __syncthreads();                // every wave is done with the previous slab
    // ---- slab: row R holds source position t0 * SS - px + R, channels 32 ct .. + 31
    {
      const int ncell = p.SRW * PC, ninstr = (ncell + 63) >> 6;
      const float inv = 1.0f / (float)PC;
      const int sp0 = t0 * SS - p.px;
      for (int ii = wave; ii < ninstr; ii += 4) {
        const int L = ii * 64 + lane;
        int c;
        const int R = fast_div(L, PC, inv, &c);
        const int sp = sp0 + R;
        int voff = T1_OOB;
        if (R < p.SRW && c < RC && (unsigned)sp < (unsigned)p.TS) voff = ((seq * p.TS + sp) * p.Cs + ct * 32 + CELL * c) * ESZ;
        pd_load_lds(xrs, slab_addr + ii * 1024, voff, 0);
      }
    }
    // ---- dy: filters kt * 64 + 32 a + fr, positions t0 + STEP step + CELL fg .. + CELL - 1
    const int n = seq / p.H, h = seq - n * p.H;
    int aoff[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int k = kt * 64 + a * 32 + fr;
      aoff[a] = k < p.K ? ((((n * p.K + k) * p.H + h) * p.OW) + t0 + CELL * fg) * ESZ : T1_OOB;
    }
    // the partial step's mask: elements at and past oend are zero
    uint32_t tmask[4];
    {
      const int cnt = tailn ? tailn - CELL * fg : CELL;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        tmask[d] = LO ? (cnt >= 2 * d + 2 ? 0xffffffffu : cnt == 2 * d + 1 ? 0x0000ffffu : 0u) : (cnt > d ? 0xffffffffu : 0u);
    }
    uintx4_t aq[RD][2];
#pragma unroll
    for (int i = 0; i < RD; ++i)
#pragma unroll
      for (int a = 0; a < 2; ++a)
        aq[i][a] = __builtin_amdgcn_raw_buffer_load_b128(drs, i < nsteps ? aoff[a] : T1_OOB, i * 32, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                              // the slab has landed for every wave

    // the slab fragment of slot t + 1 is read while slot t is multiplied (the first slot of a step behind the last
    // of the step before)
    auto bread = [&](const T* at) __attribute__((always_inline)) {
      if constexpr (LO) {
        const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)at);
        const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)(at + 4 * SS * PE));
        const uintx2_t l2 = __builtin_bit_cast(uintx2_t, lo), h2 = __builtin_bit_cast(uintx2_t, hi);
        return uintx4_t{l2.x, l2.y, h2.x, h2.y};
      } else {
        lds_f1 f = (lds_f1)at;
        return uintx4_t{__float_as_uint(f[0]), __float_as_uint(f[SS * PE]), __float_as_uint(f[2 * SS * PE]),
                        __float_as_uint(f[3 * SS * PE])};
      }
    };
    uintx4_t bnext = bread(slabT + blane);
#define T1W_STEP(I)                                                                                       \
  {                                                                                                       \
    const int st = st0 + I;                                                                               \
    if (st < nsteps) {                                                                                    \
      uintx4_t a0 = aq[I][0], a1 = aq[I][1];                                                              \
      _Pragma("unroll") for (int a = 0; a < 2; ++a)                                                       \
        aq[I][a] = __builtin_amdgcn_raw_buffer_load_b128(drs, st + RD < nsteps ? aoff[a] : T1_OOB, (st + RD) * 32, 0); \
      if (tailn && st == nsteps - 1) {                                                                    \
        _Pragma("unroll") for (int d = 0; d < 4; ++d) { a0[d] &= tmask[d]; a1[d] &= tmask[d]; }           \
      }                                                                                                   \
      const T* bp = slabT + blane + st * (STEP * SS * PE);                                                \
      _Pragma("unroll") for (int t = 0; t < TQ; ++t) {                                                    \
        uintx4_t b4 = bnext;                                                                              \
        bnext = bread(t + 1 < TQ ? bp + (t + 1) * PE : bp + STEP * SS * PE);                              \
        if (t == bias_slot) b4 = ones;                                                                    \
        tap1d_mma(acc[0][t], a0, b4, static_cast<const T*>(nullptr));                                     \
        tap1d_mma(acc[1][t], a1, b4, static_cast<const T*>(nullptr));                                     \
        __builtin_amdgcn_sched_barrier(0);                                                                \
      }                                                                                                   \
    }                                                                                                     \
  }
    for (int st0 = 0; st0 < nsteps; st0 += RD) {
      T1W_STEP(0) T1W_STEP(1) T1W_STEP(2) T1W_STEP(3)
    }
#undef T1W_STEP
  }

  // ---- the tile: element r of block (a, t): filter 32 a + 8 (r / 4) + 4 fg + r % 4, channel fr
  float* out = part + ((size_t)(split * (p.ktiles * p.ctiles) + tile) * (4 * TQ) + wave * TQ) * 2048;
#pragma unroll
  for (int t = 0; t < TQ; ++t) {
    if (wave * TQ + t > p.KW) continue;          // an unused slot
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kl = a * 32 + (r >> 2) * 8 + fg * 4 + (r & 3);
        out[t * 2048 + kl * 32 + fr] = acc[a][t][r];
      }
  }
}

// dw[k][c][j] and db[k] from the tiles of nsplit range sets, added in the order of the sets.
// Slot g of a tile: tap g for g < KW, the bias gradient for g = KW.
__global__ void __launch_bounds__(256)
tap1d_wgrad_reduce_kernel(const float* __restrict__ part, int nsplit, int tiles, int ctiles, int slots, int K, int C, int KW,
                            float* __restrict__ dw, float* __restrict__ db) {
  const int e = blockIdx.x * 256 + threadIdx.x;   // element of a slot: filter e / 32, channel e % 32
  const int g = blockIdx.y, tile = blockIdx.z;
  const int kt = tile / ctiles, ct = tile - kt * ctiles;
  const int k = kt * 64 + (e >> 5), c = ct * 32 + (e & 31);
  const bool is_bias = g == KW;
  if (k >= K) return;
  if (is_bias ? (ct != 0 || (e & 31) != 0 || !db) : (c >= C || !dw)) return;
  const size_t stride = (size_t)tiles * slots * 2048;
  const float* src = part + ((size_t)tile * slots + g) * 2048 + e;
  float sum = 0.f;
  int s = 0;
  for (; s + 4 <= nsplit; s += 4) {
    const float v0 = src[(size_t)s * stride], v1 = src[(size_t)(s + 1) * stride], v2 = src[(size_t)(s + 2) * stride],
                v3 = src[(size_t)(s + 3) * stride];
    sum += v0; sum += v1; sum += v2; sum += v3;
  }
  for (; s < nsplit; ++s) sum += src[(size_t)s * stride];
  if (is_bias) db[k] = sum;
  else dw[((size_t)k * C + c) * KW + g] = sum;
}

struct Tap1WPlan {
  Tap1WParams p;
  int TQ, SS, nsplit;
  size_t rows_bytes, part_bytes, lds_bytes;
};

bool tap1d_wgrad_plan(const ConvGeom& g, int esz, Tap1WPlan* pl) {
  if (g.KH != 1 || g.py != 0 || g.sy != 1 || g.dlx != 1 || g.groups != 1) return false;
  if (g.KW < 6 || g.KW > 23 || (g.sx != 1 && g.sx != 2)) return false;
  if (g.OH != g.H || (long long)g.N * g.H > 65535 || g.C < 16 || g.K < 32) return false;
  if (esz == 2 && g.OW % 2 != 0) return false;   // (rows of dy start on 4-byte boundaries)
  Tap1WParams& p = pl->p;
  std::memset(&p, 0, sizeof p);
  const int TQ = (g.KW + 1 + 3) / 4;            // KW taps and the bias gradient over four waves
  pl->TQ = TQ; pl->SS = g.sx;
  p.rows = g.N * g.H; p.H = g.H; p.OW = g.OW; p.TS = g.W;
  p.Cs = tap1d_cs(g.C);
  if (!p.Cs) return false;
  p.K = g.K; p.C = g.C; p.KW = g.KW; p.px = g.px;
  p.ktiles = (g.K + 63) / 64; p.ctiles = (g.C + 31) / 32;
  const int tiles = p.ktiles * p.ctiles;
  const int PC = esz == 2 ? (g.sx == 1 ? 6 : 5) : 9;
  // ranges: enough workgroups for the chip; a range's slab must fit in LDS
  const int want = (mfma_num_cus() + tiles - 1) / tiles;
  int tsplit = std::max(1, (want + p.rows - 1) / p.rows);
  for (;; ++tsplit) {
    p.TL = ((g.OW + tsplit - 1) / tsplit + 15) / 16 * 16;
    p.SRW = (p.TL - 1) * g.sx + 4 * TQ;
    pl->lds_bytes = (size_t)(((long long)p.SRW * PC + 63) / 64) * 1024;
    if (pl->lds_bytes <= 150 * 1024) break;
    if (p.TL <= 16) return false;
  }
  p.tsplit = (g.OW + p.TL - 1) / p.TL;
  p.units = p.rows * p.tsplit;
  p.upw = std::max(1, p.units / std::max(1, want));
  pl->nsplit = (p.units + p.upw - 1) / p.upw;
  const long long rb = (long long)p.rows * p.TS * p.Cs * esz;
  const long long yb = (long long)g.N * g.K * g.H * g.OW * esz;
  if (rb >= (1ll << 31) || yb >= (1ll << 31)) return false;
  p.src_bytes = (unsigned)rb; p.dy_bytes = (unsigned)yb;
  pl->rows_bytes = ((size_t)rb + 255) & ~(size_t)255;
  pl->part_bytes = (size_t)pl->nsplit * tiles * (4 * TQ) * 2048 * sizeof(float);
  return true;
}

template <typename T, int TQ>
int launch_wgrad(const Tap1WPlan& pl, const T* xr, const T* dy, float* part, hipStream_t s) {
  const dim3 grid((unsigned)pl.nsplit, (unsigned)(pl.p.ktiles * pl.p.ctiles));
  auto go = [&](auto kernel) {
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), pl.lds_bytes)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(256), pl.lds_bytes, s, pl.p, xr, dy, part);
    return check_launch("conv2d_bwd_filter (one-row windows)");
  };
  return pl.SS == 2 ? go(tap1d_wgrad_kernel<T, TQ, 2>) : go(tap1d_wgrad_kernel<T, TQ, 1>);
}

template <typename T>
int run_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws, size_t ws_bytes, hipStream_t s,
              const void* rows) {
  Tap1WPlan pl;
  if (!tap1d_wgrad_plan(g, (int)sizeof(T), &pl)) return -1;
  if (!ws || ws_bytes < pl.rows_bytes + pl.part_bytes) return -1;
  const T* xr = static_cast<const T*>(rows ? rows : ws);
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + pl.rows_bytes);
  if (!rows) {
    launch_rows(static_cast<const T*>(x), static_cast<T*>(ws), g.C, g.H, g.W, pl.p.Cs, pl.p.rows, s);
    if (const int rc = check_launch("conv2d_bwd_filter (one-row windows, rows pass)")) return rc;
  }
  const T* dyp = static_cast<const T*>(dy);
  int rc;
  switch (pl.TQ) {
    case 2: rc = launch_wgrad<T, 2>(pl, xr, dyp, part, s); break;
    case 3: rc = launch_wgrad<T, 3>(pl, xr, dyp, part, s); break;
    case 4: rc = launch_wgrad<T, 4>(pl, xr, dyp, part, s); break;
    case 5: rc = launch_wgrad<T, 5>(pl, xr, dyp, part, s); break;
    default: rc = launch_wgrad<T, 6>(pl, xr, dyp, part, s); break;
  }
  if (rc) return rc;
  const int tiles = pl.p.ktiles * pl.p.ctiles;
  hipLaunchKernelGGL(tap1d_wgrad_reduce_kernel, dim3(8, (unsigned)(g.KW + 1), (unsigned)tiles), dim3(256), 0, s, part, pl.nsplit,
                     tiles, pl.p.ctiles, 4 * pl.TQ, g.K, g.C, g.KW, dw, db);
  return check_launch("conv2d_bwd_filter (one-row windows, sum)");
}

int esz_of(int dtype) { return dtype == FLHIP_F32 ? 4 : dtype == FLHIP_BF16 || dtype == FLHIP_F16 ? 2 : 0; }

}  // namespace

size_t mfma_tap1d_conv_ws(const ConvGeom& g, int dtype, bool bwd) {
  Tap1Plan pl;
  return esz_of(dtype) && tap1d_plan(g, bwd, esz_of(dtype), &pl) ? pl.rows_bytes + pl.w_bytes : 0;
}

int mfma_tap1d_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                        void* ws, size_t ws_bytes) {
  if (dtype == FLHIP_F32) return run_conv<float>(g, false, x, w, bias, y, s, ws, ws_bytes);
  if (dtype == FLHIP_BF16) return run_conv<bf16_t>(g, false, x, w, bias, y, s, ws, ws_bytes);
  if (dtype == FLHIP_F16) return run_conv<f16_t>(g, false, x, w, bias, y, s, ws, ws_bytes);
  return -1;
}

int mfma_tap1d_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s, void* ws,
                             size_t ws_bytes) {
  if (dtype == FLHIP_F32) return run_conv<float>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  if (dtype == FLHIP_BF16) return run_conv<bf16_t>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  if (dtype == FLHIP_F16) return run_conv<f16_t>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  return -1;
}

size_t mfma_tap2d_conv_ws(const ConvGeom& g, int dtype, bool bwd) {
  Tap1Plan pl;
  return esz_of(dtype) && tap2d_plan(g, bwd, esz_of(dtype), &pl) ? pl.rows_bytes + pl.w_bytes : 0;
}

int mfma_tap2d_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                        void* ws, size_t ws_bytes) {
  if (dtype == FLHIP_F32) return run_conv2d<float>(g, false, x, w, bias, y, s, ws, ws_bytes);
  if (dtype == FLHIP_BF16) return run_conv2d<bf16_t>(g, false, x, w, bias, y, s, ws, ws_bytes);
  if (dtype == FLHIP_F16) return run_conv2d<f16_t>(g, false, x, w, bias, y, s, ws, ws_bytes);
  return -1;
}

int mfma_tap2d_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s, void* ws,
                             size_t ws_bytes) {
  if (dtype == FLHIP_F32) return run_conv2d<float>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  if (dtype == FLHIP_BF16) return run_conv2d<bf16_t>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  if (dtype == FLHIP_F16) return run_conv2d<f16_t>(g, true, dy, w, nullptr, dx, s, ws, ws_bytes);
  return -1;
}

size_t mfma_tap1d_wgrad_ws(const ConvGeom& g, int dtype) {
  Tap1WPlan pl;
  return esz_of(dtype) && tap1d_wgrad_plan(g, esz_of(dtype), &pl) ? pl.rows_bytes + pl.part_bytes : 0;
}

size_t mfma_tap1d_rows_bytes(const ConvGeom& g, int dtype) {
  Tap1Plan f;
  Tap1WPlan w;
  const int esz = esz_of(dtype);
  return esz && tap1d_plan(g, false, esz, &f) && tap1d_wgrad_plan(g, esz, &w) && f.rows_bytes == w.rows_bytes ? w.rows_bytes : 0;
}

int mfma_tap1d_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw, float* db, void* ws, size_t ws_bytes,
                     hipStream_t s, const void* rows) {
  if (dtype == FLHIP_F32) return run_wgrad<float>(g, x, dy, dw, db, ws, ws_bytes, s, rows);
  if (dtype == FLHIP_BF16) return run_wgrad<bf16_t>(g, x, dy, dw, db, ws, ws_bytes, s, rows);
  if (dtype == FLHIP_F16) return run_wgrad<f16_t>(g, x, dy, dw, db, ws, ws_bytes, s, rows);
  return -1;
}

}  // namespace flhip
