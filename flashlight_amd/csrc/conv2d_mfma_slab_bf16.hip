// Stride-1 convolution (forward and backward-data) for small windows in bf16
// storage on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//
// Same tiling as the fp32 slab kernel: a workgroup owns R whole result rows of one
// image x 64 result channels; per chunk of 32 source channels the source rows
// those results need are put in LDS once and every window tap reads them at a
// shifted address.  What differs is the operand format: an MFMA lane needs eight
// consecutive source channels of one position (16 bytes), while memory is
// channel-major.
//   slab     xs[4 channel groups][slab rows x WSP columns] of 16-byte cells (8
//            channels of one position).  A loader thread reads eight 16-byte row
//            pieces (8 channels x 8 columns), transposes them in registers
//            (v_perm_b32) and stores eight cells.  WSP = 4 (mod 16) and the plane
//            pitch = 1 (mod 16) put the 16 stores of a quarter wave in 16 distinct
//            bank groups; the 16 positions of a fragment read are contiguous.
//   weights  as[4 channel groups][64 result channels x taps] cells.  Memory order is
//            (channel, tap) per result channel (forward) or (result channel, tap)
//            per channel (backward-data).  Forward: a thread reads the 72
//            contiguous values of (result channel, 8 channels) with 16-byte loads
//            and regroups them with v_perm_b32 (3x3 windows).  Backward-data: the
//            weights look like the slab - channel-major with (result channel, tap)
//            contiguous - and go through the same 8x8 transpose.  Other shapes
//            gather a cell with eight 2-byte loads.
// 8 waves, two roles as in the fp32 kernel.  The B fragments of tap t+1 are read
// into the registers tap t has just finished with (one read behind each pair of
// MFMAs), so one set of fragment registers is enough.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int CKB = 32;          // source channels per chunk (= K of one MFMA)
constexpr int CG = CKB / 8;      // channel groups of 8
constexpr int BM = MFMA_BM;
constexpr int GTHREADS = 256;
constexpr int THREADS = 512;
constexpr int NT_MAX = 13;       // 16-position blocks per MFMA wave
constexpr int NXU_MAX = 3;       // slab units (8 channels x 8 columns) per loader thread and chunk
constexpr int NAU_MAX = 9;       // weight cells per loader thread and chunk
constexpr int KHW_MAX = 9;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const uint4* lds_cell;
#else
typedef const uint4* lds_cell;
#endif

struct Slab16Params {
  int stage_ok;          // result rows are 16-byte aligned and a half tile fits in LDS
  int wvec;              // weights are read 16 bytes at a time
  int N, SC, SH, SW, DC, DH, DW;
  int KH, KW, KHW, dly, dlx;
  int sh0, sw0;          // window shift of tap (0,0): fwd -py,-px ; bwd +py,+px
  int shs, sws;          // shift step per kh / kw: fwd +dly,+dlx ; bwd -dly,-dlx
  int min_sh, min_sw;    // smallest shifts (slab origin relative to the result origin)
  int psh, psw;          // source step per result row / column (forward: the stride; backward-data: 1)
  int groups, SCg, DCg;
  int a_mstride, a_cstride, w_group_stride;
  int R, RS;             // result rows per tile, slab rows
  int VS;                // images per tile (1: a tile is R rows of one image).  VS > 1 (3x3, stride 1, pad 1, planes
                         // that fit a tile whole): VS images stacked with one shared zero row between them; R counts
                         // the rows of the stack, of which every (DH + 1)-th is not a result
  int WSP, XOFF;         // slab row pitch (positions), slab column of image column 0
  int XPL, APL;          // plane pitches in cells: slab, weights
  int tiles_per_image, mtiles;
  int NB;                // ceil(R*DW / 16)
  int nchunks;           // ceil(SCg / 32)
  int x_cells, a_cells;  // per buffer, spare cells for idle loader lanes included
  unsigned src_bytes, wt_bytes;
};

template <typename E, bool BWD>
__global__ void __launch_bounds__(THREADS, 2)
slab16_conv_kernel(Slab16Params p, const E* __restrict__ src, const E* __restrict__ wgt,
                   const float* __restrict__ bias, E* __restrict__ dst) {
  extern __shared__ uint4 lds16[];
  uint4* Xs = lds16;                            // [2][x_cells]
  uint4* As = lds16 + 2 * p.x_cells;            // [2][a_cells]
  float* lds = reinterpret_cast<float*>(lds16);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroup-uniform values go through readfirstlane: integer division runs on the
  // vector ALU, and without it everything derived from these lives in (spilled) VGPRs
  const int img = __builtin_amdgcn_readfirstlane(blockIdx.x / p.tiles_per_image);
  const int r0 = __builtin_amdgcn_readfirstlane((blockIdx.x % p.tiles_per_image) * p.R);
  const int grp = __builtin_amdgcn_readfirstlane(blockIdx.y / p.mtiles);
  const int mtile = __builtin_amdgcn_readfirstlane(blockIdx.y % p.mtiles);
  const int m_lim = p.DCg - mtile * BM;
  const int rows = p.VS > 1 ? p.R : min(p.R, p.DH - r0);          // result rows of this tile
  const int n = p.nchunks;
  const int npos = rows * p.DW;

  // Halo columns of both slab buffers are never written by a chunk: zero them once.
  for (int i = tid; i < 2 * p.x_cells; i += THREADS) Xs[i] = make_uint4(0u, 0u, 0u, 0u);
  // bias of the tile's 64 result channels, behind the operand buffers (the epilogue
  // then needs no global loads)
  float* bias_lds = lds + 8 * (p.x_cells + p.a_cells);
  if (tid < BM) bias_lds[tid] = (bias && tid < m_lim) ? bias[grp * p.DCg + mtile * BM + tid] : 0.f;
  __syncthreads();

  // Epilogue through LDS (when rows are 16-byte aligned): the MFMA waves of one
  // channel half park their accumulators as stage[32 channels][npos] floats, then
  // all 512 threads write each channel's run of npos results, 4 at a time.
  const int SP = ((npos + 3) & ~3) + 4;                       // stage pitch (words)
  const bool staged = p.stage_ok && (npos & 3) == 0;
  auto coop_store = [&](int h) {
    const int q4 = npos >> 2;
    const float inv_q4 = 1.0f / (float)q4;
    const size_t out_base = (size_t)img * p.DC * p.DH * p.DW + (size_t)r0 * p.DW;
    const int ch0 = grp * p.DCg + mtile * BM + h * 32;
    const int lim = min(32, m_lim - h * 32) * q4;
    for (int idx = tid; idx < lim; idx += THREADS) {
      int q;
      const int ch_l = fast_div(idx, q4, inv_q4, &q);
      float4 v = *reinterpret_cast<const float4*>(lds + ch_l * SP + 4 * q);
      const float b = bias_lds[h * 32 + ch_l];
      v.x += b; v.y += b; v.z += b; v.w += b;
      st4_stream(dst, out_base + (size_t)(ch0 + ch_l) * p.DH * p.DW + 4 * q, v);
    }
  };

  if (wave < 4) {
    // ============================ loader waves ===================================
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wt_bytes);
    constexpr int OOB = (int)0x80000000;
    const int chan_bytes = p.SH * p.SW * 2;
    const int img_base = (img * p.VS * p.SC + grp * p.SCg) * p.SH * p.SW;
    // slab unit u: bits 0-1 channel group, bits 2-3 low bits of the slab row, then the
    // group of 8 image columns, then the high bits of the row (see the bank note above)
    const int qrow = (p.SW + 7) >> 3, rs_hi = (p.RS + 3) >> 2;
    const int n_units = CG * 4 * qrow * rs_hi;
    int xg[NXU_MAX], xl[NXU_MAX];                // global byte offset of channel 0 of the group, LDS cell
    int xc[NXU_MAX];                             // first channel of the unit within the chunk
    int xn[NXU_MAX];                             // columns of the unit inside the row (the last unit of a
                                                 // row of 8k+2..6 columns reads into the next row: zeroed)
#pragma unroll
    for (int i = 0; i < NXU_MAX; ++i) {
      const int u = tid + GTHREADS * i;
      xg[i] = OOB;
      xl[i] = p.x_cells - 8;
      xc[i] = 0;
      xn[i] = 8;
      if (u < n_units) {
        const int cg = u & 3, rl = (u >> 2) & 3;
        const int t = u >> 4;
        const int q = t % qrow, rh = t / qrow;
        const int rs = rh * 4 + rl;
        int sr = r0 * p.psh + p.min_sh + rs;
        int stacked = 0;                         // image of the stack this slab row belongs to
        if (p.VS > 1 && sr >= 0) {
          stacked = sr / (p.SH + 1);
          sr -= stacked * (p.SH + 1);            // sr == SH: the zero row between two images
          if (img * p.VS + stacked >= p.N) sr = -1;
        }
        xc[i] = cg * 8;
        xn[i] = min(8, p.SW - 8 * q);
        if (rs < p.RS) {
          xl[i] = cg * p.XPL + rs * p.WSP + p.XOFF + 8 * q;
          if ((unsigned)sr < (unsigned)p.SH)
            xg[i] = (img_base + stacked * p.SC * p.SH * p.SW + (cg * 8 * p.SH + sr) * p.SW + 8 * q) * 2;
        }
      }
    }
    const int APD = BM * p.KHW;                  // cells of a channel group (plane pitch is APL)
    const int w_base = grp * p.w_group_stride + mtile * BM * p.a_mstride;
    const int cstride_bytes = p.a_cstride * 2;

    // 8x8 transpose of 16-bit values: in[k] = 8 consecutive positions of channel k;
    // cell t = the 8 channels of position t.  Column 2t+s of channels 2k, 2k+1 is the
    // low (s = 0) or high (s = 1) half of dword t of the two rows.
    auto transpose_store = [&](const uint4 (&in)[8], uint4* dst, int valid = 8) {
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
        dst[2 * t] = 2 * t < valid ? make_uint4(lo[0], lo[1], lo[2], lo[3]) : make_uint4(0u, 0u, 0u, 0u);
        dst[2 * t + 1] = 2 * t + 1 < valid ? make_uint4(hi[0], hi[1], hi[2], hi[3]) : make_uint4(0u, 0u, 0u, 0u);
      }
    };
    auto ld16 = [&](__amdgpu_buffer_rsrc_t r, int off) {
      const uintx4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
      return make_uint4(v.x, v.y, v.z, v.w);
    };

    uint4 xv[NXU_MAX][8];
    auto load_x = [&](int chunk) {
      const int c0 = chunk * CKB;
      const int xbase = c0 * chan_bytes;
#pragma unroll
      for (int i = 0; i < NXU_MAX; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k)   // channels past the end of the group read zero
          xv[i][k] = ld16(srsrc, (c0 + xc[i] + k < p.SCg) ? xg[i] + xbase + k * chan_bytes : OOB);
    };
    auto store_x = [&](int buf) {
      uint4* xs = Xs + buf * p.x_cells;
#pragma unroll
      for (int i = 0; i < NXU_MAX; ++i) transpose_store(xv[i], xs + xl[i], xn[i]);
    };
    // runs the chunk pipeline with the given weight loader / storer
    auto pipeline = [&](auto&& load_w, auto&& store_w) {
      load_x(0);
      load_w(0);
      store_x(0);
      store_w(0);
      __syncthreads();
      for (int c = 0; c < n; ++c) {
        if (c + 1 < n) {
          load_x(c + 1);
          load_w(c + 1);
          store_x((c + 1) & 1);
          store_w((c + 1) & 1);
        }
        __syncthreads();
      }
    };

    if (p.wvec && !BWD) {
      // forward, 3x3: thread = (result channel m = lane, channel group = wave); the 72
      // values (8 channels x 9 taps) are contiguous; cell `tap` takes value k*9 + tap
      // of each channel k
      const int m = lane, cg = wave;
      const int wg = m < m_lim ? (w_base + m * p.a_mstride + cg * 8 * 9) * 2 : OOB;
      const int wl = cg * p.APL + m * 9;
      uint4 wv[9];
      pipeline(
          [&](int chunk) {
            const int c0 = chunk * CKB;
#pragma unroll
            for (int k = 0; k < 9; ++k)
              wv[k] = ld16(wrsrc, (c0 + cg * 8 < p.SCg) ? wg + c0 * 18 + k * 16 : OOB);
          },
          [&](int buf) {
            uint4* as = As + buf * p.a_cells + wl;
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
          });
    } else if (p.wvec) {
      // backward-data: unit = (channel group, 8 consecutive (result channel, tap) values)
      constexpr int NWU = 2;
      const int egroups = APD >> 3;
      int wg[NWU], wl[NWU], wc[NWU];
#pragma unroll
      for (int i = 0; i < NWU; ++i) {
        const int u = tid + GTHREADS * i;
        const int cg = u & 3, eg = u >> 2;
        wg[i] = OOB;
        wl[i] = p.a_cells - 8;
        wc[i] = cg * 8;
        if (eg < egroups) {
          wl[i] = cg * p.APL + 8 * eg;
          wg[i] = (w_base + 8 * eg) * 2 + cg * 8 * cstride_bytes;
        }
      }
      uint4 wv[NWU][8];
      pipeline(
          [&](int chunk) {
            const int c0 = chunk * CKB;
#pragma unroll
            for (int i = 0; i < NWU; ++i)
#pragma unroll
              for (int k = 0; k < 8; ++k)
                wv[i][k] = ld16(wrsrc, (c0 + wc[i] + k < p.SCg) ? wg[i] + (c0 + k) * cstride_bytes : OOB);
          },
          [&](int buf) {
            uint4* as = As + buf * p.a_cells;
#pragma unroll
            for (int i = 0; i < NWU; ++i) transpose_store(wv[i], as + wl[i]);
          });
    } else {
      // any layout: cell = (channel group, result channel m, tap), eight 2-byte loads
      int wg[NAU_MAX], wc[NAU_MAX], wl[NAU_MAX];
#pragma unroll
      for (int i = 0; i < NAU_MAX; ++i) {
        const int cell = tid + GTHREADS * i;
        wg[i] = OOB;
        wc[i] = 0;
        wl[i] = p.a_cells - 1;
        if (cell < CG * APD) {
          const int cg = cell / APD, rem = cell - cg * APD;
          const int m = rem / p.KHW, tap = rem - m * p.KHW;
          wl[i] = cg * p.APL + rem;
          wc[i] = cg * 8;
          if (m < m_lim) wg[i] = (w_base + m * p.a_mstride + tap) * 2 + cg * 8 * cstride_bytes;
        }
      }
      unsigned av[NAU_MAX][8];
      pipeline(
          [&](int chunk) {
            const int c0 = chunk * CKB;
#pragma unroll
            for (int i = 0; i < NAU_MAX; ++i)
#pragma unroll
              for (int k = 0; k < 8; ++k) {
                const int off = (c0 + wc[i] + k < p.SCg) ? wg[i] + (c0 + k) * cstride_bytes : OOB;
                av[i][k] = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(wrsrc, off, 0, 0);
              }
          },
          [&](int buf) {
            uint4* as = As + buf * p.a_cells;
#pragma unroll
            for (int i = 0; i < NAU_MAX; ++i)
              as[wl[i]] = make_uint4(av[i][0] | (av[i][1] << 16), av[i][2] | (av[i][3] << 16),
                                     av[i][4] | (av[i][5] << 16), av[i][6] | (av[i][7] << 16));
          });
    }
    if (staged) {
      for (int h = 0; h < 2; ++h) {
        __syncthreads();        // half h is staged
        coop_store(h);
        __syncthreads();        // stage may be overwritten
      }
    }
    return;
  }

  // =============================== MFMA waves ====================================
  // v_mfma_f32_32x32x16_bf16: a wave owns 32 result channels (lane l: channel l % 32,
  // contraction group l / 32) and NT blocks of 32 positions.  A chunk of 32 source channels
  // is two k-steps: lane half h reads the 16-byte cells of channel groups h and h + 2.
  // From one wave per SIMD the 32x32 shape issues at 2.4 PFLOP/s (measured), 16x16x32 at
  // 0.85.  Positions left over after the last whole block of 32, when there are at most 16,
  // run as one 16x16x32 block (S16) on the second wave of the pair.
  const int cw = wave - 4;
  const int wm = cw & 1, wn = cw >> 1;
  const int npos_full = p.R * p.DW;
  const int rem32 = npos_full & 31;
  const int nb32 = (npos_full >> 5) + (rem32 > 16 ? 1 : 0);
  const bool small = rem32 > 0 && rem32 <= 16;
  const int base = nb32 >> 1, odd = nb32 & 1;
  const int nt = base + (wn < odd ? 1 : 0);
  const int nb0 = wn * base + min(wn, odd);
  const bool has16 = small && wn == 1;
  const int fr = lane & 31, fh = lane >> 5;        // 32x32 fragments
  const int fr16 = lane & 15, fk16 = lane >> 4;    // 16x16 fragments of the small block
  auto run = [&](auto ntc, auto s16c) {
    constexpr int NT = decltype(ntc)::value;
    constexpr int NTA = NT > 0 ? NT : 1;
    constexpr bool S16 = decltype(s16c)::value;
    floatx16 acc[NTA];
    floatx4 acc16[2];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    acc16[0] = acc16[1] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int row_step = p.shs * p.WSP, col_step = p.sws;            // window row / column
    const int origin = (p.sh0 - p.min_sh) * p.WSP + p.sw0;           // tap (0,0)
    // 3x3 window with adjacent columns: straight-line taps, a window row walked
    // towards larger slab columns (forward kw = 0,1,2, backward kw = 2,1,0)
    const bool static33 = p.KH == 3 && p.KW == 3 && p.dlx == 1;
    const int first = origin + (static33 ? (BWD ? 2 : 0) * col_step : 0);
    const float inv_dw = 1.0f / (float)p.DW;
    const int xg2 = 2 * p.XPL, ag2 = 2 * p.APL;    // from channel group h to group h + 2
    lds_cell bp[NTA];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      int pos = (nb0 + j) * 32 + fr;
      if (pos >= npos) pos = 0;                  // padding lanes compute a discarded column
      int w;
      const int r = fast_div(pos, p.DW, inv_dw, &w);
      bp[j] = (lds_cell)Xs + (fh * p.XPL + r * p.psh * p.WSP + w * p.psw + p.XOFF + first);
    }
    lds_cell ap = (lds_cell)As + (fh * p.APL + (wm * 32 + fr) * p.KHW);
    lds_cell bq = (lds_cell)Xs, aq = (lds_cell)As + (fk16 * p.APL + (wm * 32 + fr16) * p.KHW);
    if (S16) {
      int pos = nb32 * 32 + fr16;
      if (pos >= npos) pos = 0;
      int w;
      const int r = fast_div(pos, p.DW, inv_dw, &w);
      bq += fk16 * p.XPL + r * p.psh * p.WSP + w * p.psw + p.XOFF + first;
    }

    auto frag = [](uint4 v) { return __builtin_bit_cast(bf16x8, v); };
    auto mma32 = [&](int j, uint4 a, uint4 b) {
      acc[j] = Lo16<E>::mma32(frag(a), frag(b), acc[j]);
    };
    auto mma16 = [&](uint4 a0, uint4 a1, uint4 b) {
      acc16[0] = Lo16<E>::mma16(frag(a0), frag(b), acc16[0]);
      acc16[1] = Lo16<E>::mma16(frag(a1), frag(b), acc16[1]);
    };

    __syncthreads();                             // chunk 0 is in buffer 0
    for (int c = 0; c < n; ++c) {
      if (static33) {
        constexpr int T0 = BWD ? 2 : 0, TD = BWD ? -1 : 1;   // kw of the first tap, kw step
        uint4 b[NTA][2], a0, a1, sa0, sa1, sb;
        if (NT > 0) {
          a0 = ap[T0];
          a1 = ap[ag2 + T0];
        }
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          b[j][0] = bp[j][0];
          b[j][1] = bp[j][xg2];
        }
        if (S16) {
          sa0 = aq[T0];
          sa1 = aq[16 * 9 + T0];
          sb = bq[0];
        }
        // tap t: first k-step of every block, then the second; behind each second step the
        // fragments of tap t+1 are read into the registers just used
#define FLHIP_TAP16(NEXT_TAP, NEXT_OFF)                                  \
  {                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                   \
    uint4 n0, n1, m0, m1;                                                \
    if (NT > 0) {                                                        \
      n0 = ap[NEXT_TAP];                                                 \
      n1 = ap[ag2 + (NEXT_TAP)];                                         \
    }                                                                    \
    _Pragma("unroll") for (int j = 0; j < NT; ++j) mma32(j, a0, b[j][0]); \
    _Pragma("unroll") for (int j = 0; j < NT; ++j) {                     \
      mma32(j, a1, b[j][1]);                                             \
      b[j][0] = bp[j][NEXT_OFF];                                         \
      b[j][1] = bp[j][xg2 + (NEXT_OFF)];                                 \
    }                                                                    \
    if (S16) {                                                           \
      m0 = aq[NEXT_TAP];                                                 \
      m1 = aq[16 * 9 + (NEXT_TAP)];                                      \
      mma16(sa0, sa1, sb);                                               \
      sb = bq[NEXT_OFF];                                                 \
      sa0 = m0;                                                          \
      sa1 = m1;                                                          \
    }                                                                    \
    a0 = n0;                                                             \
    a1 = n1;                                                             \
    _Pragma("unroll") for (int q = 0; q < 2 * NT + 2 + (S16 ? 3 : 0); ++q) { \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 \
    }                                                                    \
    __builtin_amdgcn_sched_barrier(0);                                   \
  }
#define FLHIP_NEXT_ROW16                                                 \
  _Pragma("unroll") for (int j = 0; j < NT; ++j) bp[j] += row_step;      \
  bq += row_step;
        FLHIP_TAP16(T0 + TD, 1)
        FLHIP_TAP16(T0 + 2 * TD, 2)
        FLHIP_NEXT_ROW16
        FLHIP_TAP16(3 + T0, 0)
        FLHIP_TAP16(3 + T0 + TD, 1)
        FLHIP_TAP16(3 + T0 + 2 * TD, 2)
        FLHIP_NEXT_ROW16
        FLHIP_TAP16(6 + T0, 0)
        FLHIP_TAP16(6 + T0 + TD, 1)
        FLHIP_TAP16(6 + T0 + 2 * TD, 2)
#undef FLHIP_NEXT_ROW16
#undef FLHIP_TAP16
#pragma unroll
        for (int j = 0; j < NT; ++j) mma32(j, a0, b[j][0]);
#pragma unroll
        for (int j = 0; j < NT; ++j) mma32(j, a1, b[j][1]);
        if (S16) mma16(sa0, sa1, sb);
      } else {
        int tap = 0;
        for (int kh = 0; kh < p.KH; ++kh) {
          for (int kw = 0; kw < p.KW; ++kw, ++tap) {
            if (NT > 0) {
              const uint4 a0 = ap[tap], a1 = ap[ag2 + tap];
#pragma unroll
              for (int j = 0; j < NT; ++j) mma32(j, a0, bp[j][0]);
#pragma unroll
              for (int j = 0; j < NT; ++j) mma32(j, a1, bp[j][xg2]);
            }
            if (S16) mma16(aq[tap], aq[16 * p.KHW + tap], bq[0]);
#pragma unroll
            for (int j = 0; j < NT; ++j) bp[j] += col_step;
            bq += col_step;
          }
#pragma unroll
          for (int j = 0; j < NT; ++j) bp[j] += row_step - p.KW * col_step;
          bq += row_step - p.KW * col_step;
        }
      }
      // back to the first tap, in the other buffer
      {
        const int sign = (c & 1) ? -1 : 1;
        const int xd = sign * p.x_cells - (p.KH - 1) * row_step - (static33 ? 0 : row_step);
#pragma unroll
        for (int j = 0; j < NT; ++j) bp[j] += xd;
        bq += xd;
        ap += sign * p.a_cells;
        aq += sign * p.a_cells;
      }
      __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------
    // accumulator element r of a 32x32 block: channel (r / 4) * 8 + fh * 4 + r % 4, position fr;
    // of a 16x16 block i: channel i * 16 + fk16 * 4 + r, position fr16
    if (staged) {
      for (int h = 0; h < 2; ++h) {
        if (wm == h) {
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            const int pos = (nb0 + j) * 32 + fr;
            if (pos < npos) {
#pragma unroll
              for (int r = 0; r < 16; ++r) lds[((r >> 2) * 8 + fh * 4 + (r & 3)) * SP + pos] = acc[j][r];
            }
          }
          if (S16) {
            const int pos = nb32 * 32 + fr16;
            if (pos < npos) {
#pragma unroll
              for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) lds[(i * 16 + fk16 * 4 + r) * SP + pos] = acc16[i][r];
            }
          }
        }
        __syncthreads();
        coop_store(h);
        __syncthreads();
      }
      return;
    }
    const size_t out_base = (size_t)img * p.VS * p.DC * p.DH * p.DW + (size_t)r0 * p.DW;
    auto put = [&](int m, int pos, float v) {
      if (m < m_lim && pos < npos) {
        const int ch = grp * p.DCg + mtile * BM + m;
        if (p.VS > 1) {
          // row of the stack -> (image, row); the row between two images is not a result
          int w;
          const int rr = fast_div(pos, p.DW, inv_dw, &w);
          const int si = rr / (p.DH + 1), row = rr - si * (p.DH + 1);
          if (row < p.DH && img * p.VS + si < p.N)
            st(dst, out_base + ((size_t)si * p.DC + ch) * p.DH * p.DW + row * p.DW + w, v + bias_lds[m]);
        } else {
          st(dst, out_base + (size_t)ch * p.DH * p.DW + pos, v + bias_lds[m]);
        }
      }
    };
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) put(wm * 32 + (r >> 2) * 8 + fh * 4 + (r & 3), (nb0 + j) * 32 + fr, acc[j][r]);
    if (S16) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) put(wm * 32 + i * 16 + fk16 * 4 + r, nb32 * 32 + fr16, acc16[i][r]);
    }
  };

  using std::integral_constant;
#define FLHIP_RUN(N)                                                                        \
  case N:                                                                                   \
    if (has16) run(integral_constant<int, N>{}, integral_constant<bool, true>{});           \
    else run(integral_constant<int, N>{}, integral_constant<bool, false>{});                \
    break;
  switch (nt) {
    FLHIP_RUN(0) FLHIP_RUN(1) FLHIP_RUN(2) FLHIP_RUN(3) FLHIP_RUN(4) FLHIP_RUN(5) FLHIP_RUN(6)
    default:
      if (has16) run(integral_constant<int, 7>{}, integral_constant<bool, true>{});
      else run(integral_constant<int, 7>{}, integral_constant<bool, false>{});
      break;
  }
#undef FLHIP_RUN
}

// smallest value >= v that is congruent to r modulo m
inline int round_to_residue(int v, int r, int m) { return v + ((r - v) % m + m) % m; }

void layout(Slab16Params* p, int R) {
  p->R = R;
  p->RS = (R - 1) * p->psh + (p->KH - 1) * p->dly + 1;
  p->XOFF = std::max(0, -p->min_sw);
  const int max_sc = p->min_sw + (p->DW - 1) * p->psw + (p->KW - 1) * p->dlx;   // last source column read
  // a row is stored in units of 8 columns: room for the last, possibly partial one
  p->WSP = round_to_residue(p->XOFF + std::max(max_sc + 1, (p->SW + 7) / 8 * 8), 4, 16);
  p->XPL = round_to_residue(p->RS * p->WSP, 1, 16);
  p->x_cells = CG * p->XPL + 8;
  // plane pitch = 2 (mod 16): the cell stores of the backward-data transpose spread
  // over the bank groups
  p->APL = round_to_residue(BM * p->KHW, 2, 16);
  p->a_cells = CG * p->APL + 8;
}

bool plan(Slab16Params* p, size_t* shmem) {
  if (p->KHW > KHW_MAX) return false;
  // rows are read 16 bytes at a time from addresses that are only 2- or 4-byte aligned when
  // the row length is not a multiple of 8 (buffer loads take any alignment in the unaligned
  // access mode the compute queues run in); the last unit of a row may run into the next
  // row or past the tensor: masked / out of range.  1x1 windows over odd rows are left to
  // the GEMM kernels.
  if (p->SW % 2 != 0 && p->KHW == 1) return false;
  const int max_pos = 2 * NT_MAX * 16;
  if (p->DW > max_pos) return false;
  const int cus = mfma_num_cus();
  int best_r = 0;
  double best_cost = 1e30;
  for (int R = 1; R <= p->DH && R * p->DW <= max_pos; ++R) {
    layout(p, R);
    const size_t bytes = (size_t)2 * (p->x_cells + p->a_cells) * 16;
    if (bytes > 156 * 1024) break;
    if (CG * 4 * ((p->SW + 7) / 8) * ((p->RS + 3) / 4) > GTHREADS * NXU_MAX) break;
    const long long tiles = (long long)p->N * ((p->DH + R - 1) / R) * p->mtiles * p->groups;
    const long long rounds = (tiles + cus - 1) / cus;
    const int nb = (R * p->DW + 15) / 16;
    const double cost = (double)rounds * ((nb + 1) / 2 + 0.5);
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best_r = R;
    }
  }
  if (best_r == 0) return false;
  p->VS = 1;
  // Planes that fit a tile whole and still make more than one round of workgroups (7x7 at batch 64): a chunk
  // of such a tile costs one trip to memory whatever it holds, so tiles of several images, stacked with one
  // shared zero row between them, take the rounds out (3x3, stride 1, pad 1: the row above an image and the
  // row below the one before it are the same zero row).
  if (best_r == p->DH && p->KH == 3 && p->psh == 1 && p->psw == 1 && p->dly == 1 && p->min_sh == -1 && p->SH == p->DH) {
    const long long tiles1 = (long long)p->N * p->mtiles * p->groups;
    int vs = 1;
    const int forced = options().conv_stack;      // measurement / test switch: this many images per tile where it fits
    while (2 * vs <= p->N && (forced ? 2 * vs <= forced : tiles1 / (2 * vs) >= cus) &&
           (2 * vs * (p->DH + 1) - 1) * p->DW <= max_pos) {
      layout(p, 2 * vs * (p->DH + 1) - 1);
      if ((size_t)2 * (p->x_cells + p->a_cells) * 16 > 156 * 1024) break;
      if (CG * 4 * ((p->SW + 7) / 8) * ((p->RS + 3) / 4) > GTHREADS * NXU_MAX) break;
      vs *= 2;
    }
    if (vs > 1) {
      p->VS = vs;
      best_r = vs * (p->DH + 1) - 1;
    }
  }
  layout(p, best_r);
  if ((CG * BM * p->KHW + GTHREADS - 1) / GTHREADS > NAU_MAX) return false;
  p->tiles_per_image = p->VS > 1 ? 1 : (p->DH + best_r - 1) / best_r;
  p->NB = (best_r * p->DW + 15) / 16;
  p->nchunks = (p->SCg + CKB - 1) / CKB;
  *shmem = (size_t)2 * (p->x_cells + p->a_cells) * 16 + BM * sizeof(float);
  {
    const int npos = best_r * p->DW, sp = ((npos + 3) & ~3) + 4;
    p->stage_ok = p->VS == 1 && p->DW % 4 == 0 && (size_t)32 * sp * sizeof(float) <= *shmem - BM * sizeof(float);
  }
  // (a whole 7x7 plane, 49 positions, is worth it for a window with several taps)
  return best_r * p->DW >= (p->KHW > 1 ? 48 : 64);
}

// Rows of odd length: a 16-byte read may start 2 bytes off a dword boundary, and the one
// whose window straddles the end of the source tensor loses the tensor's last element to
// the range check (which works on whole dwords; widening the range would read past the
// caller's buffer).  The main kernel therefore sees that one element as zero, and this
// kernel, launched behind it on the same stream, adds the element's term to the few
// results of the last image that contain it: one thread per result of the box rows
// [r0, r0+nr) x columns [c0, c0+nc) x the channels of the last group (those results are
// rounded to bf16 twice).
template <typename E, bool BWD>
__global__ void __launch_bounds__(256)
slab16_tail_fix(ConvGeom g, const E* __restrict__ src, const E* __restrict__ w,
                E* __restrict__ dst, int r0, int nr, int c0, int nc) {
  const int nch = BWD ? g.Cg : g.Kg;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= nch * nr * nc) return;
  const int col = c0 + idx % nc, row = r0 + (idx / nc) % nr, chl = idx / (nc * nr);
  const int n = g.N - 1, grp = g.groups - 1, khw = g.KH * g.KW;
  // the tap through which this result sees the last source element
  const int th = BWD ? row + g.py - (g.OH - 1) : g.H - 1 - row * g.sy + g.py;
  const int tw = BWD ? col + g.px - (g.OW - 1) : g.W - 1 - col * g.sx + g.px;
  if (th < 0 || tw < 0 || th % g.dly != 0 || tw % g.dlx != 0) return;
  const int kh = th / g.dly, kw = tw / g.dlx;
  if (kh >= g.KH || kw >= g.KW) return;
  const size_t nsrc = BWD ? (size_t)g.N * g.K * g.OH * g.OW : (size_t)g.N * g.C * g.H * g.W;
  const float last = ld(src, nsrc - 1);
  size_t o;
  float wv;
  if (!BWD) {
    const int k = grp * g.Kg + chl;
    wv = ld(w, ((size_t)k * g.Cg + (g.Cg - 1)) * khw + kh * g.KW + kw);
    o = (((size_t)n * g.K + k) * g.OH + row) * g.OW + col;
  } else {
    wv = ld(w, ((size_t)(g.K - 1) * g.Cg + chl) * khw + kh * g.KW + kw);
    o = (((size_t)n * g.C + grp * g.Cg + chl) * g.H + row) * g.W + col;
  }
  st(dst, o, ld(dst, o) + last * wv);
}

template <typename E, bool BWD>
int launch(const ConvGeom& g, Slab16Params& p, const void* src, const void* wgt, const float* bias, void* dst,
           hipStream_t s) {
  const long long sbytes = (long long)p.N * p.SC * p.SH * p.SW * 2;
  const long long wbytes = (long long)p.groups * p.w_group_stride * 2;
  if (sbytes >= (1ll << 31) || wbytes >= (1ll << 31)) return -1;
  if (reinterpret_cast<uintptr_t>(src) % 16 != 0) return -1;
  p.src_bytes = (unsigned)sbytes;
  p.wt_bytes = (unsigned)wbytes;
  size_t shmem = 0;
  if (!plan(&p, &shmem)) return -1;
  if (reinterpret_cast<uintptr_t>(dst) % 8 != 0) p.stage_ok = 0;
  // 16-byte weight loads: rows of the weight tensor start on 16-byte boundaries
  {
    const bool al = reinterpret_cast<uintptr_t>(wgt) % 16 == 0 && p.w_group_stride % 8 == 0;
    p.wvec = BWD ? (al && p.a_cstride % 8 == 0 && (BM * p.KHW) % 8 == 0 && (BM * p.a_mstride) % 8 == 0)
                 : (al && p.KHW == 9 && p.a_mstride % 8 == 0 && p.SCg % 8 == 0);
  }
  auto kernel = slab16_conv_kernel<E, BWD>;
  if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
  const dim3 grid((unsigned)(p.VS > 1 ? (p.N + p.VS - 1) / p.VS : p.N * p.tiles_per_image), (unsigned)(p.mtiles * p.groups));
  hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const E*>(src),
                     static_cast<const E*>(wgt), bias, static_cast<E*>(dst));
  if (p.SW & 1) {
    // results of the last image whose window reaches the last source element
    int r0, r1, c0, c1;
    if (!BWD) {
      r0 = (std::max(0, g.H - 1 + g.py - (g.KH - 1) * g.dly) + g.sy - 1) / g.sy; r1 = std::min(g.OH - 1, (g.H - 1 + g.py) / g.sy);
      c0 = (std::max(0, g.W - 1 + g.px - (g.KW - 1) * g.dlx) + g.sx - 1) / g.sx; c1 = std::min(g.OW - 1, (g.W - 1 + g.px) / g.sx);
    } else {
      r0 = std::max(0, g.OH - 1 - g.py); r1 = std::min(g.H - 1, g.OH - 1 - g.py + (g.KH - 1) * g.dly);
      c0 = std::max(0, g.OW - 1 - g.px); c1 = std::min(g.W - 1, g.OW - 1 - g.px + (g.KW - 1) * g.dlx);
    }
    if (r1 >= r0 && c1 >= c0) {
      const int nr = r1 - r0 + 1, nc = c1 - c0 + 1, total = (BWD ? g.Cg : g.Kg) * nr * nc;
      hipLaunchKernelGGL((slab16_tail_fix<E, BWD>), dim3((total + 255) / 256), dim3(256), 0, s, g,
                         static_cast<const E*>(src), static_cast<const E*>(wgt),
                         static_cast<E*>(dst), r0, nr, c0, nc);
    }
  }
  return check_launch("conv2d (bf16 mfma slab)");
}

void fill_fwd(const ConvGeom& g, Slab16Params* p) {
  p->N = g.N; p->SC = g.C; p->SH = g.H; p->SW = g.W; p->DC = g.K; p->DH = g.OH; p->DW = g.OW;
  p->KH = g.KH; p->KW = g.KW; p->KHW = g.KH * g.KW; p->dly = g.dly; p->dlx = g.dlx;
  p->sh0 = -g.py; p->sw0 = -g.px; p->shs = g.dly; p->sws = g.dlx;
  p->min_sh = -g.py; p->min_sw = -g.px;
  p->psh = g.sy; p->psw = g.sx;
  p->groups = g.groups; p->SCg = g.Cg; p->DCg = g.Kg;
  p->a_mstride = g.Cg * p->KHW; p->a_cstride = p->KHW; p->w_group_stride = g.Kg * g.Cg * p->KHW;
  p->mtiles = (g.Kg + BM - 1) / BM;
}

void fill_bwd(const ConvGeom& g, Slab16Params* p) {
  p->N = g.N; p->SC = g.K; p->SH = g.OH; p->SW = g.OW; p->DC = g.C; p->DH = g.H; p->DW = g.W;
  p->KH = g.KH; p->KW = g.KW; p->KHW = g.KH * g.KW; p->dly = g.dly; p->dlx = g.dlx;
  p->sh0 = g.py; p->sw0 = g.px; p->shs = -g.dly; p->sws = -g.dlx;
  p->min_sh = g.py - (g.KH - 1) * g.dly; p->min_sw = g.px - (g.KW - 1) * g.dlx;
  p->psh = 1; p->psw = 1;
  p->groups = g.groups; p->SCg = g.Kg; p->DCg = g.Cg;
  p->a_mstride = p->KHW; p->a_cstride = g.Cg * p->KHW; p->w_group_stride = g.Kg * g.Cg * p->KHW;
  p->mtiles = (g.Cg + BM - 1) / BM;
}

}  // namespace

// workgroups the forward pass below would launch (0: the shape is not this kernel's)
long long mfma_slab16_conv_fwd_workgroups(const ConvGeom& g) {
  if ((g.sy != 1 || g.sx != 1) && g.KH * g.KW == 1) return 0;
  Slab16Params p{};
  fill_fwd(g, &p);
  size_t shmem = 0;
  if (!plan(&p, &shmem)) return 0;
  return (long long)(p.VS > 1 ? (p.N + p.VS - 1) / p.VS : p.N * p.tiles_per_image) * p.mtiles * p.groups;
}

int mfma_slab16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                         hipStream_t s, int dtype) {
  // strides: results step through the slab; 1x1 windows with a stride are left to the GEMM kernels
  if ((g.sy != 1 || g.sx != 1) && g.KH * g.KW == 1) return -1;
  Slab16Params p{};
  fill_fwd(g, &p);
  return by_lo16(dtype, [&](auto* e_) { return launch<FLHIP_T_OF(e_), false>(g, p, x, w, bias, y, s); });
}

int mfma_slab16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx,
                              hipStream_t s, int dtype) {
  if (g.sy != 1 || g.sx != 1) return -1;
  Slab16Params p{};
  fill_bwd(g, &p);
  return by_lo16(dtype, [&](auto* e_) { return launch<FLHIP_T_OF(e_), true>(g, p, dy, w, nullptr, dx, s); });
}

}  // namespace flhip
