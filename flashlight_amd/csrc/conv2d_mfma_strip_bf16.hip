// 3x3 stride-1 pad-1 convolution over 64 source channels (forward and backward-data) in
// bf16 storage on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate): the
// shape of the first ResNet stage.  At this size a pass is a few microseconds of matrix
// work and of memory traffic, so what counts is that loading, multiplying and storing
// overlap inside a workgroup:
//
//   * a workgroup owns a strip of R result rows of one image x 64 result channels and the
//     WHOLE contraction (64 channels x 9 taps).  All 512 threads first fetch the strip's
//     R + 2 source rows and the 64 x 64 x 9 weights (one unit each, everything in flight at
//     once), regroup them into 16-byte cells "8 channels of one position / of one (result
//     channel, tap)" in registers and put them in LDS.
//   * the four matrix waves (32 result channels x one block of 32 columns each) then pull
//     their 36 weight fragments out of LDS into registers, for good: the inner loop reads
//     only source fragments, and the weight area of LDS becomes the staging buffer of the
//     results.
//   * the matrix waves walk the SOURCE rows: a fragment of source row r (one of 3 column
//     shifts x 4 contraction steps) feeds the three result rows r-1, r, r+1 (window rows
//     2, 1, 0), whose accumulators rotate through three register sets.  A fragment read
//     (1 KB) is thus shared by three matrix instructions.
//   * a result row that is complete goes to the staging buffer as bf16 (bias added), and
//     after a barrier the other four waves write it to memory, 16 bytes per lane, while
//     the matrix waves are on the next row.
//
// Operand roles: A = source fragment (rows = positions), B = weights (columns = result
// channels), so a lane holds four consecutive positions of one channel per accumulator
// quad: one 8-byte staging store.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int ST_BM = 64;         // result channels per workgroup
constexpr int ST_CG = 8;          // groups of 8 source channels (64 channels)
constexpr int ST_THREADS = 512;
constexpr int ST_R = 7;           // result rows per strip
constexpr int ST_XOFF = 1;        // slab column of image column 0
// smallest value >= v that is congruent to r modulo m
constexpr int round_to_residue(int v, int r, int m) { return v + ((r - v) % m + m) % m; }
// Pitches in 16-byte cells.  A slab row holds image columns -1 .. 64 (every lane of a fragment
// read stays inside its row); row pitch = 4, plane pitches = 1 (mod 16): the 16-byte stores of
// 16 consecutive lanes (8 channel groups x 2 column groups) fall in 16 distinct bank groups.
constexpr int ST_WSP = round_to_residue(66, 4, 16);
constexpr int ST_XPL = round_to_residue((ST_R + 2) * ST_WSP, 1, 16);
constexpr int ST_APL = round_to_residue(ST_BM * 9, 1, 16);

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const uint4* lds_cell;
#else
typedef const uint4* lds_cell;
#endif

struct Strip16Params {
  int N, SC, SH, SW, DC;             // source channels / rows / columns (= result rows / columns), result channels
  int groups, SCg, DCg;
  int a_mstride, a_cstride, w_group_stride;
  int SPI;                           // staging pitch (elements)
  int mtiles;                        // 64-channel tiles per group
  int qmagic;                        // ceil(2^16 / (SW / 8)): i / (SW / 8) = (i * qmagic) >> 16 for i < 512
  unsigned src_bytes, wt_bytes;
};

template <typename E, bool BWD, int R>
__global__ void __launch_bounds__(ST_THREADS, 2)
strip16_conv_kernel(Strip16Params p, const E* __restrict__ src, const E* __restrict__ wgt,
                    const float* __restrict__ bias, E* __restrict__ dst) {
  static_assert(R == ST_R, "the slab plane pitch is laid out for ST_R result rows");
  constexpr int RS = R + 2;
  constexpr int OOB = (int)0x80000000;
  extern __shared__ uint4 lds16[];
  constexpr int WSP = ST_WSP, XPL = ST_XPL, APL = ST_APL;
  uint4* Xs = lds16;                                   // [8][XPL] + 8 spare cells
  uint4* As = lds16 + ST_CG * XPL + 8;                 // [8][APL] + 8 spare cells; later the staging buffer
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // grid = (strips, images, 64-channel tiles x groups)
  const int img = blockIdx.y, r0 = blockIdx.x * R;
  const int grp = p.mtiles == 1 ? blockIdx.z : blockIdx.z / p.mtiles;
  const int mtile = blockIdx.z - grp * p.mtiles;
  const int DW = p.SW, DH = p.SH;

  // ---------------------------------------------------------------- load (all threads)
  auto ld16 = [&](__amdgpu_buffer_rsrc_t r, int off) {
    const uintx4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    return make_uint4(v.x, v.y, v.z, v.w);
  };
  // 8x8 transpose of 16-bit values: in[k] = 8 consecutive elements of row k; cell t = the
  // 8 rows' element t
  auto transpose_store = [&](const uint4 (&in)[8], uint4* out) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      unsigned lo[4], hi[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const unsigned e = t == 0 ? in[2 * k].x : t == 1 ? in[2 * k].y : t == 2 ? in[2 * k].z : in[2 * k].w;
        const unsigned o = t == 0 ? in[2 * k + 1].x : t == 1 ? in[2 * k + 1].y : t == 2 ? in[2 * k + 1].z : in[2 * k + 1].w;
        lo[k] = __builtin_amdgcn_perm(o, e, 0x05040100u);
        hi[k] = __builtin_amdgcn_perm(o, e, 0x07060302u);
      }
      out[2 * t] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
      out[2 * t + 1] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    }
  };
  // Source unit = (channel group, 8 columns of a slab row).  The strip's rows of one channel are
  // contiguous in memory (R + 2 rows x DW / 8 pieces of 16 bytes), so pieces are numbered t along
  // that run and a lane takes (t % 2, channel group, t / 2): a load instruction reads pairs of
  // adjacent pieces, 128 contiguous bytes per channel group and wave, and the 16-byte stores of 8
  // consecutive lanes (2 pieces x 4 channel groups: +8 and +1 cells) fall in 8 different bank
  // groups.  The matrix waves take the first 256 units (slab rows 0 .. 4) and store them before
  // the first barrier; the other waves request the later rows only when their weights have
  // arrived (memory serves the early rows first) and store them while the matrix waves fetch
  // their weight fragments.  Weights are requested first: they are needed first.
  uint4 xv[8];
  int xl = ST_CG * XPL;
  {
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wt_bytes);
    const int qrow = DW >> 3;
    const int chan_bytes = DH * DW * 2;
    const int unit = tid < 256 ? tid + 256 : tid - 256;
    int xg = OOB;
    const int xt = 2 * (unit >> 4) + (unit & 1);
    if (xt < qrow * RS) {
      const int cg = (unit >> 1) & 7;
      const int rs = (xt * p.qmagic) >> 16, q = xt - rs * qrow;
      const int sr = r0 - 1 + rs;
      xl = cg * XPL + rs * WSP + ST_XOFF + 8 * q;
      if ((unsigned)sr < (unsigned)DH)
        xg = (((img * p.SC + grp * p.SCg + cg * 8) * DH + sr) * DW + 8 * q) * 2;
    }
    auto load_x = [&]() {
#pragma unroll
      for (int k = 0; k < 8; ++k) xv[k] = ld16(srsrc, xg + k * chan_bytes);
    };
    // halo columns of the slab (image columns -1 and DW .. as far as fragments of valid
    // positions reach), which no unit writes
    auto zero_halo = [&]() {
      const int nz = min(8, WSP - ST_XOFF - DW);
      for (int i = tid; i < ST_CG * RS * 9; i += ST_THREADS) {
        const int c = i % 9, t = i / 9;
        if (c <= nz)
          Xs[(t / RS) * XPL + (t % RS) * WSP + (c == 0 ? 0 : ST_XOFF + DW + c - 1)] = make_uint4(0u, 0u, 0u, 0u);
      }
    };
    const int w_base = grp * p.w_group_stride + mtile * ST_BM * p.a_mstride;
    if (!BWD) {
      // forward: thread = (result channel m, channel group); its 72 values (8 channels x 9
      // taps) are contiguous; cell `tap` takes value k * 9 + tap of each channel k
      const int m = tid & 63, cg = tid >> 6;
      const int wg = (w_base + m * p.a_mstride + cg * 72) * 2;
      uint4 wv[9];
#pragma unroll
      for (int k = 0; k < 9; ++k) wv[k] = ld16(wrsrc, wg + k * 16);
      if (wave >= 4) load_x();
      zero_halo();     // (while the loads are in flight)
      uint4* as = As + cg * APL + m * 9;
      unsigned d[36];
#pragma unroll
      for (int k = 0; k < 9; ++k) {
        d[4 * k] = wv[k].x; d[4 * k + 1] = wv[k].y; d[4 * k + 2] = wv[k].z; d[4 * k + 3] = wv[k].w;
      }
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        unsigned o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int e0 = 2 * j * 9 + tap, e1 = (2 * j + 1) * 9 + tap;   // values of channels 2j, 2j+1
          const unsigned sel = ((e0 & 1) ? 0x0302u : 0x0100u) | ((e1 & 1) ? 0x07060000u : 0x05040000u);
          o[j] = __builtin_amdgcn_perm(d[e1 >> 1], d[e0 >> 1], sel);
        }
        as[tap] = make_uint4(o[0], o[1], o[2], o[3]);
      }
      if (wave < 4) load_x();
    } else {
      // backward-data: memory is [contraction channel][(result channel, tap)]; unit =
      // (channel group, 8 consecutive (result channel, tap) values), transposed like the slab and
      // numbered like the slab's units (pairs of adjacent pieces x channel groups)
      constexpr int EG = ST_BM * 9 / 8;     // 72 units per channel group
      const int cstride_bytes = p.a_cstride * 2;
      int wg[2], wl[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int u = tid + ST_THREADS * i;
        const int cg = (u >> 1) & 7, eg = 2 * (u >> 4) + (u & 1);
        wg[i] = OOB;
        wl[i] = ST_CG * APL;
        if (eg < EG) {
          wl[i] = cg * APL + 8 * eg;
          wg[i] = (w_base + 8 * eg) * 2 + cg * 8 * cstride_bytes;
        }
      }
      uint4 wv[2][8];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) wv[i][k] = ld16(wrsrc, wg[i] + k * cstride_bytes);
      if (wave >= 4) load_x();
      zero_halo();
#pragma unroll
      for (int i = 0; i < 2; ++i) transpose_store(wv[i], As + wl[i]);
      if (wave < 4) load_x();
    }
  }
  if (wave >= 4) transpose_store(xv, Xs + xl);
  __syncthreads();                                   // weights and slab rows 0 .. 4 are in LDS

  uint16_t* const stage = reinterpret_cast<uint16_t*>(As);
  if (wave < 4) {
    // ------------------------------------------------------------ store waves
    transpose_store(xv, Xs + xl);                    // the later slab rows: visible after the next barrier,
                                                     // which the matrix waves pass before they reach them
    __syncthreads();                                 // (the matrix waves have read their weights)
    // piece = 8 columns (16 bytes) of one channel's row
    const int ppr = DW >> 3, npieces = ST_BM * ppr;
    int soff[2];
    size_t goff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = tid + 256 * i;
      const int ch = (idx * p.qmagic) >> 16, q = idx - ch * ppr;
      soff[i] = idx < npieces ? ch * p.SPI + 8 * q : -1;
      goff[i] = ((size_t)(img * p.DC + grp * p.DCg + mtile * ST_BM + ch) * DH + r0) * DW + 8 * q;
    }
    for (int o = 0; o < R; ++o) {
      __syncthreads();                               // row o is staged
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (soff[i] >= 0) {
          const uintx4_t v = *reinterpret_cast<const uintx4_t*>(stage + soff[i] + o * DW);
          __builtin_nontemporal_store(v, reinterpret_cast<uintx4_t*>(dst + goff[i] + (size_t)o * DW));
        }
    }
    return;
  }

  // ---------------------------------------------------------------- matrix waves
  const int cw = wave - 4;
  const int wm = cw & 1, blk = cw >> 1;
  const int fr = lane & 31, fh = lane >> 5;
  // weight fragments, for good: wf[t][s], t = (slab row - result row) * 3 + column shift,
  // s = contraction step (channel groups 2s and 2s + 1 for the two lane halves)
  uint4 wf[9][4];
  {
    lds_cell ap = (lds_cell)As + (fh * APL + (wm * 32 + fr) * 9);
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int s = 0; s < 4; ++s) wf[t][s] = ap[2 * s * APL + (BWD ? 8 - t : t)];
  }
  const float bv = (!BWD && bias) ? bias[grp * p.DCg + mtile * ST_BM + wm * 32 + fr] : 0.f;
  __syncthreads();                                   // the weight area may be overwritten

  // result row o accumulates in acc[o % 3]
  floatx16 acc[3];
#pragma unroll
  for (int j = 0; j < 3; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  // slab cell of (row 0, column shift 0, step 0) for this lane's position
  lds_cell xp = (lds_cell)Xs + (fh * XPL + blk * 32 + fr);
  auto frag = [](uint4 v) { return __builtin_bit_cast(bf16x8, v); };
  uint16_t* const srow = stage + (wm * 32 + fr) * p.SPI + blk * 32 + fh * 4;
  // accumulator element r is position blk*32 + (r/4)*8 + fh*4 + r%4 of channel wm*32 + fr:
  // part g = the four positions of elements 4g .. 4g+3
  auto stage_part = [&](const floatx16& a, int o, int g) {
    if (blk * 32 + g * 8 + fh * 4 < DW) {
      const uintx2_t v = {Lo16<E>::pack(a[4 * g] + bv, a[4 * g + 1] + bv), Lo16<E>::pack(a[4 * g + 2] + bv, a[4 * g + 3] + bv)};
      *reinterpret_cast<uintx2_t*>(srow + o * DW + g * 8) = v;
    }
  };
  // slab row rr, window row dr: one matrix instruction into result row rr - dr (if there is one)
  auto mma = [&](int rr, int dr, uint4 f, int j) {
    const int o = rr - dr;
    if (o >= 0 && o < R)
      acc[o % 3] = Lo16<E>::mma32(frag(f), frag(wf[dr * 3 + j % 3][j / 3]), acc[o % 3]);
  };

  // fragment i = (slab row i / 12, contraction step (i % 12) / 3, column shift i % 3); its read
  // is issued three fragments ahead into a ring of four registers.  Nothing moves across the
  // fences (the compiler would otherwise sink each read to its use).
  constexpr int NF = 12 * RS;
  auto cell = [](int i) { return (i / 12) * WSP + ((i % 12) / 3) * 2 * XPL + i % 3; };
  uint4 fq[4];
  fq[0] = xp[cell(0)];
  fq[1] = xp[cell(1)];
  fq[2] = xp[cell(2)];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int rr = 0; rr < RS; ++rr) {
#pragma unroll
    for (int j = 0; j < 10; ++j) {
      const int i = rr * 12 + j;
      if (i + 3 < NF) fq[(i + 3) & 3] = xp[cell(i + 3)];
      __builtin_amdgcn_sched_barrier(0);
      mma(rr, 0, fq[i & 3], j);
      mma(rr, 1, fq[i & 3], j);
      mma(rr, 2, fq[i & 3], j);
      __builtin_amdgcn_sched_barrier(0);
    }
    // The last two fragments complete result row rr - 2.  Its two instructions go first, the
    // other four behind them, and the conversion and staging of the finished row is spread
    // between those four: it runs while they execute.
    {
      const int i = rr * 12 + 10;
      floatx16& done = acc[(rr + 1) % 3];
      if (i + 3 < NF) fq[(i + 3) & 3] = xp[cell(i + 3)];
      __builtin_amdgcn_sched_barrier(0);
      mma(rr, 2, fq[i & 3], 10);
      mma(rr, 2, fq[(i + 1) & 3], 11);
      mma(rr, 0, fq[i & 3], 10);
      mma(rr, 1, fq[i & 3], 10);
      __builtin_amdgcn_sched_barrier(0);
      if (i + 4 < NF) fq[(i + 4) & 3] = xp[cell(i + 4)];
      __builtin_amdgcn_sched_barrier(0);
      if (rr >= 2) stage_part(done, rr - 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      mma(rr, 0, fq[(i + 1) & 3], 11);
      __builtin_amdgcn_sched_barrier(0);
      if (rr >= 2) stage_part(done, rr - 2, 1);
      __builtin_amdgcn_sched_barrier(0);
      mma(rr, 1, fq[(i + 1) & 3], 11);
      __builtin_amdgcn_sched_barrier(0);
      if (rr >= 2) {
        stage_part(done, rr - 2, 2);
        stage_part(done, rr - 2, 3);
#pragma unroll
        for (int r = 0; r < 16; ++r) done[r] = 0.f;
        __syncthreads();
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <typename E, bool BWD>
int launch(Strip16Params& p, const void* src, const void* wgt, const float* bias, void* dst, hipStream_t s) {
  constexpr int R = ST_R;
  if (p.SCg != 64 || p.DCg % ST_BM != 0 || p.SW % 8 != 0 || p.SW <= 32 || p.SW > 64 || p.SH % R != 0) return -1;
  const long long sbytes = (long long)p.N * p.SC * p.SH * p.SW * 2;
  const long long dbytes = (long long)p.N * p.DC * p.SH * p.SW * 2;
  const long long wbytes = (long long)p.groups * p.w_group_stride * 2;
  if (sbytes >= (1ll << 31) || dbytes >= (1ll << 31) || wbytes >= (1ll << 31)) return -1;
  if (reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(wgt) % 16 != 0)
    return -1;
  p.src_bytes = (unsigned)sbytes;
  p.wt_bytes = (unsigned)wbytes;
  p.SPI = (R * p.SW + 7) & ~7;
  p.mtiles = p.DCg / ST_BM;
  p.qmagic = (65536 + p.SW / 8 - 1) / (p.SW / 8);
  if (ST_CG * (p.SW / 8) * (R + 2) > ST_THREADS) return -1;
  if (p.N > 65535 || p.mtiles * p.groups > 65535) return -1;
  const size_t cells = (size_t)ST_CG * ST_XPL + 8 + (size_t)ST_CG * ST_APL + 8;
  const size_t shmem = cells * 16;
  if ((size_t)ST_BM * p.SPI * 2 > ((size_t)ST_CG * ST_APL + 8) * 16) return -1;
  auto kernel = strip16_conv_kernel<E, BWD, R>;
  if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
  const dim3 grid((unsigned)(p.SH / R), (unsigned)p.N, (unsigned)(p.mtiles * p.groups));
  hipLaunchKernelGGL(kernel, grid, dim3(ST_THREADS), shmem, s, p, static_cast<const E*>(src),
                     static_cast<const E*>(wgt), bias, static_cast<E*>(dst));
  return check_launch("conv2d (bf16 mfma strip)");
}

bool strip16_shape(const ConvGeom& g) {
  return g.KH == 3 && g.KW == 3 && g.sy == 1 && g.sx == 1 && g.dly == 1 && g.dlx == 1 && g.py == 1 && g.px == 1 &&
         g.OH == g.H && g.OW == g.W;
}

}  // namespace

int mfma_strip16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                          hipStream_t s, int dtype) {
  if (!strip16_shape(g)) return -1;
  Strip16Params p{};
  p.N = g.N; p.SC = g.C; p.SH = g.H; p.SW = g.W; p.DC = g.K;
  p.groups = g.groups; p.SCg = g.Cg; p.DCg = g.Kg;
  p.a_mstride = g.Cg * 9; p.a_cstride = 9; p.w_group_stride = g.Kg * g.Cg * 9;
  return by_lo16(dtype, [&](auto* e_) { return launch<FLHIP_T_OF(e_), false>(p, x, w, bias, y, s); });
}

int mfma_strip16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s, int dtype) {
  if (!strip16_shape(g)) return -1;
  Strip16Params p{};
  p.N = g.N; p.SC = g.K; p.SH = g.OH; p.SW = g.OW; p.DC = g.C;
  p.groups = g.groups; p.SCg = g.Kg; p.DCg = g.Cg;
  p.a_mstride = 9; p.a_cstride = g.Cg * 9; p.w_group_stride = g.Kg * g.Cg * 9;
  return by_lo16(dtype, [&](auto* e_) { return launch<FLHIP_T_OF(e_), true>(p, dy, w, nullptr, dx, s); });
}

}  // namespace flhip
