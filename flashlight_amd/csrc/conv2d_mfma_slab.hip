// Stride-1 convolution (forward and backward-data) for small windows, the shape
// class of the ResNet 3x3 layers: implicit GEMM on the matrix cores with the
// source tile resident in LDS.
//
// A workgroup owns R whole result rows of one image (all W columns) x 64 result
// channels.  The source rows those results need ("slab": R + (KH-1)*dil rows, the
// image columns plus a zero halo on both sides) are loaded ONCE per chunk of 8
// source channels and every window tap reads them at a shifted address, so
// nothing is gathered nine times.
//
// LDS layouts keep two source channels side by side, so one 8-byte read gives a
// lane its operand of both k-steps of a chunk (lane k-index fk handles channels
// 2*fk and 2*fk+1):
//   slab     xs[4 channel pairs][slab rows x WSP columns][2]
//            image column w sits at slab column w + XOFF (XOFF a multiple of 4):
//            rows are copied with 16-byte loads and stores, and the halo columns
//            are zeroed once per kernel because no chunk ever writes them;
//   weights  forward        as[64 result channels][8 channels x taps]  (memory order,
//                           copied 16 bytes at a time)
//            backward-data  as[4 channel pairs][64 result channels x taps][2]
// The plane pitches are chosen so that the 16 positions x 4 k-indices of a
// fragment read fall on distinct banks.
// 8 or 12 waves, two roles (waves w, w+4 and w+8 share a SIMD):
//   waves 0-3 load chunk c+1 (global -> registers -> the LDS buffer not in use);
//     what each thread loads is the same every chunk, so offsets are computed
//     once per kernel;
//   waves 4-7 (MW = 4) or 4-11 (MW = 8), arranged 2 (channels) x MW/2 (positions), issue
//     v_mfma_f32_16x16x4_f32 (compiled per NT = position blocks per wave).
// One barrier per chunk.  Backward-data is the same kernel with dy as the source,
// mirrored window shifts and the weights indexed [source channel][result channel].
// Shapes whose rows are not 16-byte friendly use element-wise loaders into the
// same layouts.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int CK = 8;            // source channels per chunk
constexpr int CP = CK / 2;       // channel pairs per chunk
constexpr int BM = MFMA_BM;
constexpr int GTHREADS = 256;
constexpr int THREADS = 512;      // 4 loader waves + 4 MFMA waves; the kernel compiled for 8 MFMA waves has 768
constexpr int NT_MAX = 13;       // 16-position blocks per MFMA wave
constexpr int NEX_MAX = 20;      // element-wise loader: slab elements per thread and chunk
constexpr int NEA_MAX = 20;      // element-wise loader: weight elements per thread and chunk
constexpr int NXV_MAX = 5;       // 16-byte loader: slab units (4 columns x 2 channels) per thread
constexpr int NAV_MAX = 5;       // 16-byte loader: weight units per thread
constexpr int KHW_MAX = 9;

struct SlabParams {
  int stage_ok;          // result rows are 16-byte aligned and a half tile fits in LDS
  int vec;               // 16-byte loaders apply
  int N, SC, SH, SW, DC, DH, DW;
  int KH, KW, KHW, dly, dlx;
  int sh0, sw0;          // window shift of tap (0,0): fwd -py,-px ; bwd +py,+px
  int shs, sws;          // shift step per kh / kw: fwd +dly,+dlx ; bwd -dly,-dlx
  int min_sh, min_sw;    // smallest shifts (slab origin relative to the result origin)
  int psh, psw;          // source step per result row / column (forward: the stride; backward-data: 1)
  int groups, SCg, DCg;
  int a_mstride, a_cstride, w_group_stride;
  int R, RS;             // result rows per tile, slab rows
  int WSP, XOFF;         // slab row pitch (positions), slab column of image column 0
  int XPH;               // slab plane pitch per channel pair, in positions (2 words each)
  int APW;               // weight pitch in words: fwd per result channel, bwd per channel pair
  int tiles_per_image, mtiles;
  int NB;                // ceil(R*DW / 16)
  int nchunks;           // ceil(SCg / CK)
  int x_words, a_words;  // per buffer, spare words for idle loader lanes included
  unsigned src_bytes, wgt_bytes;
};

template <typename T, bool BWD, int MW>
__global__ void __launch_bounds__(GTHREADS + 64 * MW, MW == 4 ? 2 : 1)
slab_conv_kernel(SlabParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                 const float* __restrict__ bias, T* __restrict__ dst) {
  extern __shared__ float lds[];
  float* Xs = lds;                              // [2][x_words]
  float* As = lds + 2 * p.x_words;              // [2][a_words]
  constexpr int THREADS = GTHREADS + 64 * MW;
  const int esz = (int)sizeof(T);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroup-uniform values go through readfirstlane: integer division runs on the
  // vector ALU, and without it everything derived from these lives in (spilled) VGPRs
  const int img = __builtin_amdgcn_readfirstlane(blockIdx.x / p.tiles_per_image);
  const int r0 = __builtin_amdgcn_readfirstlane((blockIdx.x % p.tiles_per_image) * p.R);
  const int grp = __builtin_amdgcn_readfirstlane(blockIdx.y / p.mtiles);
  const int mtile = __builtin_amdgcn_readfirstlane(blockIdx.y % p.mtiles);
  const int m_lim = p.DCg - mtile * BM;
  const int rows = min(p.R, p.DH - r0);          // result rows of this tile
  const int n = p.nchunks;
  const int npos = rows * p.DW;
  const int XPW = 2 * p.XPH;                     // slab plane pitch in words

  // Halo columns (and the alignment gaps) of both slab buffers are never written
  // by a chunk: zero everything once.
  for (int i = tid; i < (2 * p.x_words) >> 2; i += THREADS)
    reinterpret_cast<float4*>(Xs)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  // bias of the tile's 64 result channels, behind the operand buffers (the epilogue
  // then needs no global loads)
  float* bias_lds = lds + 2 * (p.x_words + p.a_words);
  if (tid < BM) bias_lds[tid] = (bias && tid < m_lim) ? bias[grp * p.DCg + mtile * BM + tid] : 0.f;
  __syncthreads();

  // Epilogue through LDS (when rows are 16-byte aligned): the MFMA waves of one
  // channel half park their accumulators as stage[32 channels][npos] in the LDS
  // that held the operands, then all 512 threads write each channel's run of
  // npos results with 16-byte stores.
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
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wgt_bytes);
    // A slot that has nothing to load carries the byte offset 2^31, which stays out
    // of range after the chunk offset is added, so its buffer load returns zero
    // without a branch; it stores to spare words behind the buffer.
    constexpr int OOB = (int)0x80000000;
    const int xdummy = p.x_words - 8, adummy = p.a_words - 8;
    const int img_base = (img * p.SC + grp * p.SCg) * p.SH * p.SW;
    const int w_base = grp * p.w_group_stride + mtile * BM * p.a_mstride;
    const int chan_bytes = p.SH * p.SW * esz;

    if (p.vec) {
      // ---- 16-byte loaders -------------------------------------------------------
      // slab unit u over (channel pair, slab row, group of 4 image columns)
      const int qrow = p.SW >> 2, per_pair = p.RS * qrow;
      const float inv_pp = 1.0f / (float)per_pair, inv_q = 1.0f / (float)qrow;
      int xg[NXV_MAX], xl[NXV_MAX];              // global byte offset, LDS word offset
#pragma unroll
      for (int i = 0; i < NXV_MAX; ++i) {
        const int u = tid + GTHREADS * i;
        xg[i] = OOB;
        xl[i] = xdummy;
        if (u < CP * per_pair) {
          int rem, q;
          const int cp = fast_div(u, per_pair, inv_pp, &rem);
          const int rs = fast_div(rem, qrow, inv_q, &q);
          const int sr = r0 * p.psh + p.min_sh + rs;
          xl[i] = cp * XPW + (rs * p.WSP + p.XOFF + 4 * q) * 2;
          if ((unsigned)sr < (unsigned)p.SH)
            xg[i] = (img_base + (2 * cp * p.SH + sr) * p.SW + 4 * q) * esz;
        }
      }
      // weight unit u: forward (result channel m, 4 consecutive (channel, tap) words);
      // backward (channel pair, 4 consecutive (result channel, tap) words)
      const int per_row = BWD ? (BM * p.KHW) >> 2 : (CK * p.KHW) >> 2;
      const float inv_row = 1.0f / (float)per_row;
      const int n_units = (BWD ? CP : BM) * per_row;
      int ag[NAV_MAX], al[NAV_MAX];
#pragma unroll
      for (int i = 0; i < NAV_MAX; ++i) {
        const int u = tid + GTHREADS * i;
        ag[i] = OOB;
        al[i] = adummy;
        if (u < n_units) {
          int q;
          const int row = fast_div(u, per_row, inv_row, &q);
          if (!BWD) {
            al[i] = row * p.APW + 4 * q;
            ag[i] = (w_base + row * p.a_mstride + 4 * q) * esz;
          } else {
            al[i] = row * p.APW + 8 * q;
            ag[i] = (w_base + 2 * row * p.a_cstride + 4 * q) * esz;
          }
        }
      }
      const int a_pair_bytes = p.a_cstride * esz;
      constexpr int AV2 = BWD ? 2 : 1;

      float4 xv[NXV_MAX][2], av[NAV_MAX][AV2];
      auto load_chunk = [&](int chunk) {
        const int c0 = chunk * CK;
        const int xbase = c0 * chan_bytes, abase = c0 * p.a_cstride * esz;
#pragma unroll
        for (int i = 0; i < NXV_MAX; ++i) {
          xv[i][0] = buf_ld4(srsrc, xg[i] + xbase, src);
          xv[i][1] = buf_ld4(srsrc, xg[i] + xbase + chan_bytes, src);
        }
#pragma unroll
        for (int i = 0; i < NAV_MAX; ++i) {
          av[i][0] = buf_ld4(wrsrc, ag[i] + abase, wgt);
          if (BWD) av[i][AV2 - 1] = buf_ld4(wrsrc, ag[i] + abase + a_pair_bytes, wgt);
        }
      };
      auto store_chunk = [&](int buf) {
        float* xs = Xs + buf * p.x_words;
        float* as = As + buf * p.a_words;
#pragma unroll
        for (int i = 0; i < NXV_MAX; ++i) {
          const float4 a = xv[i][0], b = xv[i][1];
          *reinterpret_cast<float4*>(xs + xl[i]) = make_float4(a.x, b.x, a.y, b.y);
          *reinterpret_cast<float4*>(xs + xl[i] + 4) = make_float4(a.z, b.z, a.w, b.w);
        }
#pragma unroll
        for (int i = 0; i < NAV_MAX; ++i) {
          if (!BWD) {
            *reinterpret_cast<float4*>(as + al[i]) = av[i][0];
          } else {
            const float4 a = av[i][0], b = av[i][AV2 - 1];
            *reinterpret_cast<float4*>(as + al[i]) = make_float4(a.x, b.x, a.y, b.y);
            *reinterpret_cast<float4*>(as + al[i] + 4) = make_float4(a.z, b.z, a.w, b.w);
          }
        }
      };
      load_chunk(0);
      store_chunk(0);
      __syncthreads();
      for (int c = 0; c < n; ++c) {
        if (c + 1 < n) {
          load_chunk(c + 1);
          store_chunk((c + 1) & 1);
        }
        __syncthreads();
      }
    } else {
      // ---- element-wise loaders ------------------------------------------------------
      // slab elements e = tid + 256*i over (channel, slab row, image column)
      const int per_chan = p.RS * p.SW;
      const float inv_pc = 1.0f / (float)per_chan, inv_sw = 1.0f / (float)p.SW;
      const float inv_khw = 1.0f / (float)p.KHW;
      const int tail = p.SCg - (n - 1) * CK;     // channels of the last chunk (1..8)
      int xg[NEX_MAX], xl[NEX_MAX];
      unsigned xlive = 0, alive = 0;             // bit i: slot i is a channel of the last chunk
#pragma unroll
      for (int i = 0; i < NEX_MAX; ++i) {
        const int e = tid + GTHREADS * i;
        xg[i] = OOB;
        xl[i] = xdummy;
        if (e < CK * per_chan) {
          int q, sc;
          const int c = fast_div(e, per_chan, inv_pc, &q);
          const int rs = fast_div(q, p.SW, inv_sw, &sc);
          const int sr = r0 * p.psh + p.min_sh + rs;
          xl[i] = (c >> 1) * XPW + (rs * p.WSP + p.XOFF + sc) * 2 + (c & 1);
          if ((unsigned)sr < (unsigned)p.SH) xg[i] = (img_base + (c * p.SH + sr) * p.SW + sc) * esz;
          if (c < tail) xlive |= 1u << i;
        }
      }
      // weight elements: e over (result channel m, chunk channel c, tap), memory order
      const int per_m = CK * p.KHW;
      int ag[NEA_MAX], al[NEA_MAX];
#pragma unroll
      for (int i = 0; i < NEA_MAX; ++i) {
        const int e = tid + GTHREADS * i;
        ag[i] = OOB;
        al[i] = adummy;
        if (e < BM * per_m) {
          int m, c, tap, q;
          if (!BWD) {        // w[m][c][tap]: (c, tap) contiguous per m
            m = fast_div(e, per_m, 1.0f / (float)per_m, &q);
            c = fast_div(q, p.KHW, inv_khw, &tap);
            al[i] = m * p.APW + c * p.KHW + tap;
          } else {           // w[c][m][tap]: (m, tap) contiguous per c
            c = fast_div(e, BM * p.KHW, 1.0f / (float)(BM * p.KHW), &q);
            m = fast_div(q, p.KHW, inv_khw, &tap);
            al[i] = (c >> 1) * p.APW + (m * p.KHW + tap) * 2 + (c & 1);
          }
          if (m < m_lim) ag[i] = (w_base + m * p.a_mstride + c * p.a_cstride + tap) * esz;
          if (c < tail) alive |= 1u << i;
        }
      }

      float xv[NEX_MAX], av[NEA_MAX];
      auto load_chunk = [&](int chunk) {
        const int c0 = chunk * CK;
        const int xbase = c0 * chan_bytes, abase = c0 * p.a_cstride * esz;
        if (c0 + CK <= p.SCg) {
#pragma unroll
          for (int i = 0; i < NEX_MAX; ++i) xv[i] = buf_ld(srsrc, xg[i] + xbase, src);
#pragma unroll
          for (int i = 0; i < NEA_MAX; ++i) av[i] = buf_ld(wrsrc, ag[i] + abase, wgt);
        } else {
          // last chunk of a channel count that is not a multiple of 8: channels past
          // the end read zero
#pragma unroll
          for (int i = 0; i < NEX_MAX; ++i)
            xv[i] = buf_ld(srsrc, (xlive >> i) & 1 ? xg[i] + xbase : OOB, src);
#pragma unroll
          for (int i = 0; i < NEA_MAX; ++i)
            av[i] = buf_ld(wrsrc, (alive >> i) & 1 ? ag[i] + abase : OOB, wgt);
        }
      };
      auto store_chunk = [&](int buf) {
        float* xs = Xs + buf * p.x_words;
        float* as = As + buf * p.a_words;
#pragma unroll
        for (int i = 0; i < NEX_MAX; ++i) xs[xl[i]] = xv[i];
#pragma unroll
        for (int i = 0; i < NEA_MAX; ++i) as[al[i]] = av[i];
      };
      load_chunk(0);
      store_chunk(0);
      __syncthreads();
      for (int c = 0; c < n; ++c) {
        if (c + 1 < n) {
          load_chunk(c + 1);
          store_chunk((c + 1) & 1);
        }
        __syncthreads();
      }
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
  const int cw = wave - 4;
  constexpr int PW = MW / 2;                     // waves over the positions
  const int wm = cw & 1, wn = cw >> 1;
  const int base = p.NB / PW, rem = p.NB % PW;
  const int nt = base + (wn < rem ? 1 : 0);
  const int nb0 = wn * base + min(wn, rem);
  const int fr = lane & 15, fk = lane >> 4;
  auto run = [&](auto ntc) {
    constexpr int NT = decltype(ntc)::value;
    floatx4 acc[2][NT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // LDS address (buffer 0) of this lane's result position in block j at the first
    // window tap.  The addresses walk the window inside a chunk, return to the first
    // tap, and switch buffers between chunks.
    const int row_step = p.shs * p.WSP, col_step = p.sws;            // window row / column
    const int origin = (p.sh0 - p.min_sh) * p.WSP + p.sw0;           // tap (0,0)
    // 3x3 window with adjacent columns: the nine taps are straight-line code.  A
    // window row is walked towards larger slab columns (forward kw = 0,1,2, backward
    // kw = 2,1,0) so that its three taps differ by immediate offsets, and the
    // fragments of tap t+1 are read while the MFMAs of tap t run.
    const bool static33 = p.KH == 3 && p.KW == 3 && p.dlx == 1;
    const int first = origin + (static33 ? (BWD ? 2 : 0) * col_step : 0);
    const float inv_dw = 1.0f / (float)p.DW;
    lds_f2 bp[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      int pos = (nb0 + j) * 16 + fr;
      if (pos >= npos) pos = 0;                  // padding lanes compute a discarded column
      int w;
      const int r = fast_div(pos, p.DW, inv_dw, &w);
      bp[j] = (lds_f2)(reinterpret_cast<const float2*>(Xs)) +
              (fk * p.XPH + r * p.psh * p.WSP + w * p.psw + p.XOFF + first);
    }
    // weights of this lane: rows wm*32 + fr (+16), channels 2*fk and 2*fk+1
    lds_f1 a1 = (lds_f1)As + ((wm * 32 + fr) * p.APW + 2 * fk * p.KHW);       // forward
    lds_f1 a1b = a1 + 16 * p.APW;
    lds_f2 a2 = (lds_f2)(reinterpret_cast<const float2*>(As)) +               // backward
                (fk * (p.APW >> 1) + (wm * 32 + fr) * p.KHW);

    // Fragments of one tap: both k-steps (.x, .y) of 2 weight rows and NT positions.
    struct Frag {
      float2 a[2];
      float2 b[NT];
    };
    // tap: window tap index of the weights; boff: slab shift on top of bp[] (float2 units)
    auto read_frags = [&](Frag& f, auto khw, int tap, int boff) {
      const int k = khw;
      if (BWD) {
        f.a[0] = a2[tap];
        f.a[1] = a2[16 * k + tap];
      } else {
        f.a[0] = make_float2(a1[tap], a1[k + tap]);
        f.a[1] = make_float2(a1b[tap], a1b[k + tap]);
      }
#pragma unroll
      for (int j = 0; j < NT; ++j) f.b[j] = bp[j][boff];
    };
    auto mma = [&](const Frag& f) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[0].x, f.b[j].x, acc[0][j], 0, 0, 0);
        acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[1].x, f.b[j].x, acc[1][j], 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[0].y, f.b[j].y, acc[0][j], 0, 0, 0);
        acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[1].y, f.b[j].y, acc[1][j], 0, 0, 0);
      }
    };
    const int xhalf = p.x_words >> 1, ahalf = p.a_words >> 1;        // buffer size in float2

    __syncthreads();                             // chunk 0 is in buffer 0
    for (int c = 0; c < n; ++c) {
      if (static33) {
        constexpr std::integral_constant<int, 9> K9{};
        constexpr int T0 = BWD ? 2 : 0, TD = BWD ? -1 : 1;   // kw of the first tap, kw step
        constexpr int REST = 3 * NT - 4 > 0 ? 3 * NT - 4 : 0;
        Frag f0, f1;
        read_frags(f0, K9, T0, 0);
        // One LDS read is slotted behind each of the first MFMAs of the tap, so the
        // reads issue in the shadow of the matrix pipe instead of ahead of it.
#define FLHIP_TAP(CUR, NXT, TAP, BOFF)                                \
  __builtin_amdgcn_sched_barrier(0);                                  \
  read_frags(NXT, K9, TAP, BOFF);                                     \
  mma(CUR);                                                           \
  _Pragma("unroll") for (int q = 0; q < NT + 4; ++q) {                \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
  }                                                                   \
  __builtin_amdgcn_sched_group_barrier(0x008, REST, 0);               \
  __builtin_amdgcn_sched_barrier(0);
#define FLHIP_NEXT_ROW _Pragma("unroll") for (int j = 0; j < NT; ++j) bp[j] += row_step;
        FLHIP_TAP(f0, f1, T0 + TD, 1)
        FLHIP_TAP(f1, f0, T0 + 2 * TD, 2)
        FLHIP_NEXT_ROW
        FLHIP_TAP(f0, f1, 3 + T0, 0)
        FLHIP_TAP(f1, f0, 3 + T0 + TD, 1)
        FLHIP_TAP(f0, f1, 3 + T0 + 2 * TD, 2)
        FLHIP_NEXT_ROW
        FLHIP_TAP(f1, f0, 6 + T0, 0)
        FLHIP_TAP(f0, f1, 6 + T0 + TD, 1)
        FLHIP_TAP(f1, f0, 6 + T0 + 2 * TD, 2)
#undef FLHIP_NEXT_ROW
#undef FLHIP_TAP
        mma(f0);
      } else {
        int tap = 0;
        for (int kh = 0; kh < p.KH; ++kh) {
          for (int kw = 0; kw < p.KW; ++kw, ++tap) {
            Frag f;
            read_frags(f, p.KHW, tap, 0);
            mma(f);
#pragma unroll
            for (int j = 0; j < NT; ++j) bp[j] += col_step;
          }
#pragma unroll
          for (int j = 0; j < NT; ++j) bp[j] += row_step - p.KW * col_step;
        }
      }
      // back to the first tap, in the other buffer
      {
        const int sign = (c & 1) ? -1 : 1;
        const int xd = sign * xhalf - (p.KH - 1) * row_step - (static33 ? 0 : row_step);
#pragma unroll
        for (int j = 0; j < NT; ++j) bp[j] += xd;
        a1 += sign * p.a_words;
        a1b += sign * p.a_words;
        a2 += sign * ahalf;
      }
      __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------
    if (staged) {
      for (int h = 0; h < 2; ++h) {
        if (wm == h) {
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            const int pos = (nb0 + j) * 16 + fr;
            if (pos < npos) {
#pragma unroll
              for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) lds[(i * 16 + fk * 4 + r) * SP + pos] = acc[i][j][r];
            }
          }
        }
        __syncthreads();
        coop_store(h);
        __syncthreads();
      }
      return;
    }
    float bv[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) bv[i][r] = bias_lds[wm * 32 + i * 16 + fk * 4 + r];
    const size_t out_base = (size_t)img * p.DC * p.DH * p.DW + (size_t)r0 * p.DW;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int pos = (nb0 + j) * 16 + fr;
      if (pos < npos) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = wm * 32 + i * 16 + fk * 4 + r;
            if (m < m_lim) {
              const int ch = grp * p.DCg + mtile * BM + m;
              st(dst, out_base + (size_t)ch * p.DH * p.DW + pos, acc[i][j][r] + bv[i][r]);
            }
          }
      }
    }
  };

  auto run_small = [&]() {
    switch (nt) {
      case 0: case 1: run(std::integral_constant<int, 1>{}); break;
      case 2: run(std::integral_constant<int, 2>{}); break;
      case 3: run(std::integral_constant<int, 3>{}); break;
      case 4: run(std::integral_constant<int, 4>{}); break;
      case 5: run(std::integral_constant<int, 5>{}); break;
      case 6: run(std::integral_constant<int, 6>{}); break;
      default: run(std::integral_constant<int, 7>{}); break;
    }
  };
  if constexpr (MW == 8) {
    run_small();                                 // 26 blocks over 4 waves: 7 at most
  } else {
    if (nt <= 7) {
      run_small();
    } else {
      switch (nt) {
        case 8: run(std::integral_constant<int, 8>{}); break;
        case 9: run(std::integral_constant<int, 9>{}); break;
        case 10: run(std::integral_constant<int, 10>{}); break;
        case 11: run(std::integral_constant<int, 11>{}); break;
        case 12: run(std::integral_constant<int, 12>{}); break;
        default: run(std::integral_constant<int, 13>{}); break;
      }
    }
  }
}

// smallest value >= v that is congruent to r modulo m
inline int round_to_residue(int v, int r, int m) { return v + ((r - v) % m + m) % m; }

// LDS layout of a tile of R result rows.
void layout(SlabParams* p, int R, bool bwd) {
  p->R = R;
  p->RS = (R - 1) * p->psh + (p->KH - 1) * p->dly + 1;
  p->XOFF = (std::max(0, -p->min_sw) + 3) & ~3;
  const int max_sc = p->min_sw + (p->DW - 1) * p->psw + (p->KW - 1) * p->dlx;   // last source column read
  p->WSP = (p->XOFF + std::max(max_sc + 1, p->SW) + 3) & ~3;
  // pair-plane pitch = 16 (mod 32) positions: the four k-indices of a fragment read
  // start 32 banks apart
  p->XPH = round_to_residue(p->RS * p->WSP, 16, 32);
  p->x_words = CP * 2 * p->XPH + 8;
  if (!bwd) {
    p->APW = round_to_residue(CK * p->KHW + 4, 12, 64);
    p->a_words = BM * p->APW + 8;
  } else {
    p->APW = round_to_residue(2 * BM * p->KHW, 32, 64);
    p->a_words = CP * p->APW + 8;
  }
}

// Picks the rows per tile: as many as fit 26 position blocks and the LDS budget,
// preferring a tile count that fills the CUs evenly.  Returns false when the
// shape is outside this kernel.
bool plan(SlabParams* p, size_t* shmem, bool bwd, bool aligned) {
  if (p->KHW > KHW_MAX) return false;
  const int max_pos = 2 * NT_MAX * 16;
  if (p->DW > max_pos) return false;
  // 16-byte loaders: rows, channel planes and weight rows start on 16-byte
  // boundaries (8-byte for bf16 storage) and the channel count has no tail
  p->vec = aligned && p->SW % 4 == 0 && p->SCg % CK == 0 && p->w_group_stride % 4 == 0 &&
           (bwd ? p->a_cstride : p->a_mstride) % 4 == 0;
  const int cus = mfma_num_cus();
  int best_r = 0;
  double best_cost = 1e30;
  for (int R = 1; R <= p->DH && R * p->DW <= max_pos; ++R) {
    layout(p, R, bwd);
    const size_t bytes = (size_t)2 * (p->x_words + p->a_words) * sizeof(float);
    if (bytes > 150 * 1024) break;
    if (p->vec ? CP * p->RS * (p->SW / 4) > GTHREADS * NXV_MAX
               : CK * p->RS * p->SW > GTHREADS * NEX_MAX)
      break;
    const long long tiles = (long long)p->N * ((p->DH + R - 1) / R) * p->mtiles * p->groups;
    const long long rounds = (tiles + cus - 1) / cus;
    const int nb = (R * p->DW + 15) / 16;
    // time ~ rounds x (blocks of the busier MFMA wave pair) ; small fixed cost per round
    double cost = (double)rounds * ((nb + 1) / 2 + 0.5);
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best_r = R;
    }
  }
  if (best_r == 0) return false;
  if (p->vec ? (bwd ? CP * (BM * p->KHW / 4) : BM * (CK * p->KHW / 4)) > GTHREADS * NAV_MAX
             : BM * CK * p->KHW > GTHREADS * NEA_MAX)
    return false;
  layout(p, best_r, bwd);
  p->tiles_per_image = (p->DH + best_r - 1) / best_r;
  p->NB = (best_r * p->DW + 15) / 16;
  p->nchunks = (p->SCg + CK - 1) / CK;
  *shmem = (size_t)2 * (p->x_words + p->a_words) * sizeof(float) + BM * sizeof(float);
  {
    const int npos = best_r * p->DW, sp = ((npos + 3) & ~3) + 4;
    p->stage_ok = p->DW % 4 == 0 && (size_t)32 * sp * sizeof(float) <= *shmem - BM * sizeof(float);
  }
  // a tile with few positions would leave the matrix cores idle: not worth it
  return best_r * p->DW >= 48;
}

template <typename T, bool BWD>
int launch(SlabParams& p, const void* src, const void* wgt, const float* bias, void* dst,
           hipStream_t s) {
  const long long sbytes = (long long)p.N * p.SC * p.SH * p.SW * (long long)sizeof(T);
  const long long wbytes = (long long)p.groups * p.w_group_stride * (long long)sizeof(T);
  if (sbytes >= (1ll << 31) || wbytes >= (1ll << 31)) return -1;
  p.src_bytes = (unsigned)sbytes;
  p.wgt_bytes = (unsigned)wbytes;
  size_t shmem = 0;
  const uintptr_t align = 4 * sizeof(T);
  const bool aligned = reinterpret_cast<uintptr_t>(src) % align == 0 &&
                       reinterpret_cast<uintptr_t>(wgt) % align == 0;
  if (!plan(&p, &shmem, BWD, aligned)) return -1;
  if (reinterpret_cast<uintptr_t>(dst) % 16 != 0) p.stage_ok = 0;
  const dim3 grid((unsigned)(p.N * p.tiles_per_image), (unsigned)(p.mtiles * p.groups));
  // eight MFMA waves (four over the positions per channel half, two per SIMD) instead of four: measured 1 to 8 %
  // faster on every ResNet 3x3 layer (56x56: 66.5 -> 65.0 us forward; 7x7 planes: 118 -> 108 us backward-data)
  const int mw = options().slab_waves ? options().slab_waves : (p.NB >= 8 ? 8 : 4);
  if (mw == 8) {
    auto kernel = slab_conv_kernel<T, BWD, 8>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(GTHREADS + 64 * 8), shmem, s, p, static_cast<const T*>(src),
                       static_cast<const T*>(wgt), bias, static_cast<T*>(dst));
  } else {
    auto kernel = slab_conv_kernel<T, BWD, 4>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const T*>(src),
                       static_cast<const T*>(wgt), bias, static_cast<T*>(dst));
  }
  return check_launch("conv2d (mfma slab)");
}

}  // namespace

int mfma_slab_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                       const float* bias, void* y, hipStream_t s) {
  // strides: results step through the slab; 1x1 windows with a stride are left to the GEMM kernels
  if ((g.sy != 1 || g.sx != 1) && g.KH * g.KW == 1) return -1;
  SlabParams p{};
  p.N = g.N; p.SC = g.C; p.SH = g.H; p.SW = g.W; p.DC = g.K; p.DH = g.OH; p.DW = g.OW;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW; p.dly = g.dly; p.dlx = g.dlx;
  p.sh0 = -g.py; p.sw0 = -g.px; p.shs = g.dly; p.sws = g.dlx;
  p.min_sh = -g.py; p.min_sw = -g.px;
  p.psh = g.sy; p.psw = g.sx;
  p.groups = g.groups; p.SCg = g.Cg; p.DCg = g.Kg;
  p.a_mstride = g.Cg * p.KHW; p.a_cstride = p.KHW; p.w_group_stride = g.Kg * g.Cg * p.KHW;
  p.mtiles = (g.Kg + BM - 1) / BM;
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch<T, false>(p, x, w, bias, y, s);
  });
}

int mfma_slab_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                            hipStream_t s) {
  if (g.sy != 1 || g.sx != 1) return -1;
  SlabParams p{};
  p.N = g.N; p.SC = g.K; p.SH = g.OH; p.SW = g.OW; p.DC = g.C; p.DH = g.H; p.DW = g.W;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW; p.dly = g.dly; p.dlx = g.dlx;
  p.sh0 = g.py; p.sw0 = g.px; p.shs = -g.dly; p.sws = -g.dlx;
  p.min_sh = g.py - (g.KH - 1) * g.dly; p.min_sw = g.px - (g.KW - 1) * g.dlx;
  p.psh = 1; p.psw = 1;
  p.groups = g.groups; p.SCg = g.Kg; p.DCg = g.Cg;
  p.a_mstride = p.KHW; p.a_cstride = g.Cg * p.KHW; p.w_group_stride = g.Kg * g.Cg * p.KHW;
  p.mtiles = (g.Cg + BM - 1) / BM;
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch<T, true>(p, dy, w, nullptr, dx, s);
  });
}

}  // namespace flhip
