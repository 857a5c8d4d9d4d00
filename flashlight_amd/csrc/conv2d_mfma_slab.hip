// Stride-1 convolution (forward and backward-data) for small windows, the shape
// class of the ResNet 3x3 layers: implicit GEMM on the matrix cores with the
// source tile resident in LDS.
//
// A workgroup owns R whole result rows of one image (all W columns) x 64 result
// channels.  The source rows those results need ("slab": R + (KH-1)*dil rows,
// W + (KW-1)*dil columns, zero where outside the image) are loaded ONCE per
// chunk of 8 source channels and every window tap reads them at a shifted
// address, so nothing is gathered nine times.  LDS layouts put the channel
// innermost with an odd pitch (9 words): the k index of an MFMA fragment is then
// a compile-time immediate offset and consecutive lanes hit distinct banks.
//   slab   xs[position (row-major rows x cols)][9]   (8 channels + pad)
//   weights as[64 result channels][9 tap slots][9]   (8 channels + pad)
// 8 waves, two roles (wave w and w+4 share a SIMD):
//   waves 0-3 load chunk c+1 (global -> registers -> the LDS buffer not in use);
//     what each thread loads is the same every chunk, so offsets are computed
//     once per kernel;
//   waves 4-7, arranged 2 (channels) x 2 (positions), issue
//     v_mfma_f32_16x16x4_f32: per tap, NT+1 address adds, then straight-line
//     fragment reads and MFMAs (compiled per NT).
// One barrier per chunk (taps x 2 k-steps x 2*NT MFMAs apart).  Backward-data is
// the same kernel with dy as the source, mirrored window shifts and the weights
// indexed [source channel][result channel].
#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int CK = 8;            // source channels per chunk
constexpr int PP = 9;            // LDS pitch per position / per weight row (words)
constexpr int BM = MFMA_BM;
constexpr int GTHREADS = 256;
constexpr int THREADS = 512;
constexpr int NT_MAX = 13;       // 16-position blocks per MFMA wave
constexpr int NEX_MAX = 20;      // slab elements per loader thread and chunk
constexpr int NEA_MAX = 20;      // weight elements per loader thread and chunk
constexpr int KHW_MAX = 9;

struct SlabParams {
  int stage_ok;          // result rows are 16-byte aligned and a half tile fits in LDS
  int N, SC, SH, SW, DC, DH, DW;
  int KH, KW, KHW, dly, dlx;
  int sh0, sw0;          // window shift of tap (0,0): fwd -py,-px ; bwd +py,+px
  int shs, sws;          // shift step per kh / kw: fwd +dly,+dlx ; bwd -dly,-dlx
  int min_sh, min_sw;    // smallest shifts (slab origin relative to the result origin)
  int groups, SCg, DCg;
  int a_mstride, a_cstride, w_group_stride;
  int R, RS, WS;         // result rows per tile, slab rows, slab columns
  int tiles_per_image, mtiles;
  int NB;                // ceil(R*DW / 16)
  int nchunks;           // ceil(SCg / CK)
  int slab_words, a_words;   // per buffer
  unsigned src_bytes, wgt_bytes;
};

template <typename T, bool BWD>
__global__ void __launch_bounds__(THREADS, 2)
slab_conv_kernel(SlabParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                 const float* __restrict__ bias, T* __restrict__ dst) {
  extern __shared__ float lds[];
  float* Xs = lds;                              // [2][slab_words]
  float* As = lds + 2 * p.slab_words;           // [2][a_words]
  const int esz = (int)sizeof(T);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int img = blockIdx.x / p.tiles_per_image;
  const int r0 = (blockIdx.x % p.tiles_per_image) * p.R;
  const int grp = blockIdx.y / p.mtiles, mtile = blockIdx.y % p.mtiles;
  const int m_lim = p.DCg - mtile * BM;
  const int rows = min(p.R, p.DH - r0);          // result rows of this tile
  const int n = p.nchunks;
  const int npos = rows * p.DW;

  // Epilogue through LDS (when rows are 16-byte aligned): the MFMA waves of one
  // channel half park their accumulators as stage[32 channels][npos] in the LDS
  // that held the operands, then all 512 threads write each channel's run of
  // npos results with 16-byte stores.
  const int SP = ((npos + 3) & ~3) + 4;                       // stage pitch (words)
  const bool staged = p.stage_ok && (npos & 3) == 0;
  auto coop_store = [&](int h) {
    const int q4 = npos >> 2;
    const size_t out_base = (size_t)img * p.DC * p.DH * p.DW + (size_t)r0 * p.DW;
    for (int idx = tid; idx < 32 * q4; idx += THREADS) {
      const int ch_l = idx / q4, q = idx - ch_l * q4;
      const int m = h * 32 + ch_l;
      if (m < m_lim) {
        const int ch = grp * p.DCg + mtile * BM + m;
        const float b = bias ? bias[ch] : 0.f;
        float4 v = *reinterpret_cast<const float4*>(lds + ch_l * SP + 4 * q);
        v.x += b; v.y += b; v.z += b; v.w += b;
        st4_stream(dst, out_base + (size_t)ch * p.DH * p.DW + 4 * q, v);
      }
    }
  };

  if (wave < 4) {
    // ============================ loader waves ===================================
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wgt_bytes);
    // slab elements of this thread: e = tid + 256*i over (channel, slab row, slab col).
    // Offsets are fixed for the kernel; an element that is padding (outside the
    // image) or past the slab gets the byte offset 2^31, which stays out of range
    // after the chunk offset is added, so its buffer load returns zero.
    constexpr int OOB = (int)0x80000000;
    const int slab_pos = p.RS * p.WS;
    const float inv_slab = 1.0f / (float)slab_pos, inv_ws = 1.0f / (float)p.WS;
    const float inv_khw = 1.0f / (float)p.KHW;
    const int nex = (CK * slab_pos + GTHREADS - 1) / GTHREADS;
    const int xdummy = p.slab_words - 1, adummy = p.a_words - 1;   // spare words of each buffer
    int xg[NEX_MAX], xl[NEX_MAX];                // global byte offset, LDS word offset
    const int img_base = (img * p.SC + grp * p.SCg) * p.SH * p.SW;
    int xcmax = 0;
#pragma unroll
    for (int i = 0; i < NEX_MAX; ++i) {
      const int e = tid + GTHREADS * i;
      xg[i] = OOB;
      xl[i] = xdummy;
      if (i < nex && e < CK * slab_pos) {
        int q, ws;
        const int c = fast_div(e, slab_pos, inv_slab, &q);
        const int rs = fast_div(q, p.WS, inv_ws, &ws);
        const int sr = r0 + p.min_sh + rs, sc = p.min_sw + ws;
        xl[i] = q * PP + c;
        if ((unsigned)sr < (unsigned)p.SH && (unsigned)sc < (unsigned)p.SW)
          xg[i] = (img_base + (c * p.SH + sr) * p.SW + sc) * esz;
        xcmax = c;    // ascending in i
      }
    }
    // weight elements: e over (result channel m, chunk channel c, tap), memory order
    const int per_m = CK * p.KHW;
    const int nea = (BM * per_m + GTHREADS - 1) / GTHREADS;
    int ag[NEA_MAX], al[NEA_MAX];                // global byte offset, LDS word offset
    const int w_base = grp * p.w_group_stride + mtile * BM * p.a_mstride;
#pragma unroll
    for (int i = 0; i < NEA_MAX; ++i) {
      const int e = tid + GTHREADS * i;
      ag[i] = OOB;
      al[i] = adummy;
      if (i < nea && e < BM * per_m) {
        int m, c, tap, q;
        if (!BWD) {        // w[m][c][tap]: (c, tap) contiguous per m
          m = fast_div(e, per_m, 1.0f / (float)per_m, &q);
          c = fast_div(q, p.KHW, inv_khw, &tap);
        } else {           // w[c][m][tap]: (m, tap) contiguous per c
          c = fast_div(e, BM * p.KHW, 1.0f / (float)(BM * p.KHW), &q);
          m = fast_div(q, p.KHW, inv_khw, &tap);
        }
        al[i] = (m * KHW_MAX + tap) * PP + c;
        if (m < m_lim) ag[i] = (w_base + m * p.a_mstride + c * p.a_cstride + tap) * esz;
      }
    }
    const int chan_bytes = p.SH * p.SW * esz;
    (void)xcmax;

    float xv[NEX_MAX], av[NEA_MAX];
    auto load_chunk = [&](int chunk) {
      const int c0 = chunk * CK;
      const int xbase = c0 * chan_bytes, abase = c0 * p.a_cstride * esz;
      if (c0 + CK <= p.SCg) {
        // unused slots carry the out-of-range offset: no branch, no memory access
#pragma unroll
        for (int i = 0; i < NEX_MAX; ++i) xv[i] = buf_ld(srsrc, xg[i] + xbase, src);
#pragma unroll
        for (int i = 0; i < NEA_MAX; ++i) av[i] = buf_ld(wrsrc, ag[i] + abase, wgt);
      } else {
        // last chunk of a channel count that is not a multiple of 8: channels past
        // the end read zero
#pragma unroll
        for (int i = 0; i < NEX_MAX; ++i) {
          const int c = xl[i] - (xl[i] / PP) * PP;
          xv[i] = buf_ld(srsrc, c0 + c < p.SCg ? xg[i] + xbase : OOB, src);
        }
#pragma unroll
        for (int i = 0; i < NEA_MAX; ++i)
          av[i] = buf_ld(wrsrc, c0 + (al[i] - (al[i] / PP) * PP) < p.SCg ? ag[i] + abase : OOB, wgt);
      }
    };
    auto store_chunk = [&](int buf) {
      float* xs = Xs + buf * p.slab_words;
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
  const int wm = cw & 1, wn = cw >> 1;
  const int base = p.NB >> 1, rem = p.NB & 1;
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

    // slab word offset of this lane's position in block j (tap shift excluded)
    const float inv_dw = 1.0f / (float)p.DW;
    int pbase[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      int pos = (nb0 + j) * 16 + fr;
      if (pos >= npos) pos = 0;                  // padding lanes compute a discarded column
      int w;
      const int r = fast_div(pos, p.DW, inv_dw, &w);
      pbase[j] = (r * p.WS + w) * PP + fk;
    }
    const int abase0 = (wm * 32 + fr) * KHW_MAX * PP + fk;

    // Fragments of one tap: 2 k-steps x (2 A + NT B).  Every offset inside is a
    // compile-time immediate on top of the per-block address ba[j].
    struct Frag {
      float a[CK / 4][2];
      float b[CK / 4][NT];
    };
    auto read_frags = [&](Frag& f, const float* at, const int (&ba)[NT], const float* xs, int boff) {
#pragma unroll
      for (int ks = 0; ks < CK / 4; ++ks) {
        f.a[ks][0] = at[ks * 4];
        f.a[ks][1] = at[16 * KHW_MAX * PP + ks * 4];
#pragma unroll
        for (int j = 0; j < NT; ++j) f.b[ks][j] = xs[ba[j] + boff + ks * 4];
      }
    };
    auto mma = [&](const Frag& f) {
#pragma unroll
      for (int ks = 0; ks < CK / 4; ++ks)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[ks][0], f.b[ks][j], acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[ks][1], f.b[ks][j], acc[1][j], 0, 0, 0);
        }
    };
    const int row_step = p.shs * p.WS * PP, col_step = p.sws * PP;   // window row / column
    const int origin = ((p.sh0 - p.min_sh) * p.WS + (p.sw0 - p.min_sw)) * PP;   // tap (0,0)
    // 3x3 window whose columns are one apart: the nine taps are straight-line code,
    // the three taps of a window row differ by immediate offsets (forward walks kw
    // upwards, backward-data downwards), and the fragments of tap t+1 are read
    // while the MFMAs of tap t run.
    const bool static33 = p.KH == 3 && p.KW == 3 && (p.sws == 1 || p.sws == -1);
    const int kw_first = p.sws == 1 ? 0 : 2, kw_dir = p.sws == 1 ? 1 : -1;

    __syncthreads();                             // chunk 0 is in buffer 0
    for (int c = 0; c < n; ++c) {
      const float* xs = Xs + (c & 1) * p.slab_words;
      const float* as = As + (c & 1) * p.a_words + abase0;
      if (static33) {
        int ba[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) ba[j] = pbase[j] + origin + kw_first * col_step;
        const float* a0 = as + kw_first * PP;
        const int ad = kw_dir * PP;
        Frag f0, f1;
        read_frags(f0, a0, ba, xs, 0);
        // One LDS read is slotted behind each of the first MFMAs of the tap, so the
        // reads issue in the shadow of the matrix pipe instead of ahead of it.
#define FLHIP_TAP(CUR, NXT, AT, BA, BOFF)                     \
  __builtin_amdgcn_sched_barrier(0);                          \
  read_frags(NXT, AT, BA, xs, BOFF);                          \
  mma(CUR);                                                   \
  _Pragma("unroll") for (int q = 0; q < (CK / 4) * (2 + NT); ++q) { \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        \
  }                                                           \
  __builtin_amdgcn_sched_group_barrier(0x008, (CK / 4) * (2 * NT - 2), 0); \
  __builtin_amdgcn_sched_barrier(0);
#define FLHIP_NEXT_ROW _Pragma("unroll") for (int j = 0; j < NT; ++j) ba[j] += row_step;
        FLHIP_TAP(f0, f1, a0 + ad, ba, PP)
        FLHIP_TAP(f1, f0, a0 + 2 * ad, ba, 2 * PP)
        FLHIP_NEXT_ROW
        FLHIP_TAP(f0, f1, a0 + 3 * PP, ba, 0)
        FLHIP_TAP(f1, f0, a0 + 3 * PP + ad, ba, PP)
        FLHIP_TAP(f0, f1, a0 + 3 * PP + 2 * ad, ba, 2 * PP)
        FLHIP_NEXT_ROW
        FLHIP_TAP(f1, f0, a0 + 6 * PP, ba, 0)
        FLHIP_TAP(f0, f1, a0 + 6 * PP + ad, ba, PP)
        FLHIP_TAP(f1, f0, a0 + 6 * PP + 2 * ad, ba, 2 * PP)
#undef FLHIP_NEXT_ROW
#undef FLHIP_TAP
        mma(f0);
      } else {
        int ba[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) ba[j] = pbase[j] + origin;
        int tap = 0;
        for (int kh = 0; kh < p.KH; ++kh) {
          for (int kw = 0; kw < p.KW; ++kw, ++tap) {
            Frag f;
            read_frags(f, as + tap * PP, ba, xs, 0);
            mma(f);
#pragma unroll
            for (int j = 0; j < NT; ++j) ba[j] += col_step;
          }
#pragma unroll
          for (int j = 0; j < NT; ++j) ba[j] += row_step - p.KW * col_step;
        }
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
    // this lane's eight result channels and their bias
    float bv[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = wm * 32 + i * 16 + fk * 4 + r;
        bv[i][r] = (bias && m < m_lim) ? bias[grp * p.DCg + mtile * BM + m] : 0.f;
      }
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

  switch (nt) {
    case 0: case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 6: run(std::integral_constant<int, 6>{}); break;
    case 7: run(std::integral_constant<int, 7>{}); break;
    case 8: run(std::integral_constant<int, 8>{}); break;
    case 9: run(std::integral_constant<int, 9>{}); break;
    case 10: run(std::integral_constant<int, 10>{}); break;
    case 11: run(std::integral_constant<int, 11>{}); break;
    case 12: run(std::integral_constant<int, 12>{}); break;
    default: run(std::integral_constant<int, 13>{}); break;
  }
}

// Picks the rows per tile: as many as fit 26 position blocks and the LDS budget,
// preferring a tile count that fills the CUs evenly.  Returns false when the
// shape is outside this kernel.
bool plan(SlabParams* p, size_t* shmem) {
  if (p->KHW > KHW_MAX) return false;
  const int max_pos = 2 * NT_MAX * 16;
  if (p->DW > max_pos) return false;
  const int cus = mfma_num_cus();
  int best_r = 0;
  double best_cost = 1e30;
  for (int R = 1; R <= p->DH && R * p->DW <= max_pos; ++R) {
    const int RS = R + (p->KH - 1) * p->dly, WS = p->DW + (p->KW - 1) * p->dlx;
    const int slab_words = RS * WS * PP + 8, a_words = KHW_MAX * BM * PP + 8;
    const size_t bytes = (size_t)2 * (slab_words + a_words) * sizeof(float);
    if (bytes > 150 * 1024) break;
    if ((CK * RS * WS + GTHREADS - 1) / GTHREADS > NEX_MAX) break;
    const long long tiles = (long long)p->N * ((p->DH + R - 1) / R) * p->mtiles * p->groups;
    const long long rounds = (tiles + cus - 1) / cus;
    const int nb = (R * p->DW + 15) / 16;
    // time ~ rounds x (blocks of the busier MFMA wave pair) ; small fixed cost per round
    const double cost = (double)rounds * ((nb + 1) / 2 + 0.5);
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best_r = R;
    }
  }
  if (best_r == 0) return false;
  if ((BM * CK * p->KHW + GTHREADS - 1) / GTHREADS > NEA_MAX) return false;
  p->R = best_r;
  p->RS = best_r + (p->KH - 1) * p->dly;
  p->WS = p->DW + (p->KW - 1) * p->dlx;
  p->tiles_per_image = (p->DH + best_r - 1) / best_r;
  p->NB = (best_r * p->DW + 15) / 16;
  p->nchunks = (p->SCg + CK - 1) / CK;
  p->slab_words = p->RS * p->WS * PP + 8;   // + spare words for out-of-slab loader lanes
  p->a_words = KHW_MAX * BM * PP + 8;
  *shmem = (size_t)2 * (p->slab_words + p->a_words) * sizeof(float);
  {
    const int npos = best_r * p->DW, sp = ((npos + 3) & ~3) + 4;
    p->stage_ok = p->DW % 4 == 0 && (size_t)32 * sp * sizeof(float) <= *shmem;
  }
  // a tile with few positions would leave the matrix cores idle: not worth it
  return best_r * p->DW >= 64;
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
  if (!plan(&p, &shmem)) return -1;
  if (reinterpret_cast<uintptr_t>(dst) % 16 != 0) p.stage_ok = 0;
  auto kernel = slab_conv_kernel<T, BWD>;
  if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
  const dim3 grid((unsigned)(p.N * p.tiles_per_image), (unsigned)(p.mtiles * p.groups));
  hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const T*>(src),
                     static_cast<const T*>(wgt), bias, static_cast<T*>(dst));
  return check_launch("conv2d (mfma slab)");
}

}  // namespace

int mfma_slab_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                       const float* bias, void* y, hipStream_t s) {
  if (g.sy != 1 || g.sx != 1) return -1;
  SlabParams p{};
  p.N = g.N; p.SC = g.C; p.SH = g.H; p.SW = g.W; p.DC = g.K; p.DH = g.OH; p.DW = g.OW;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW; p.dly = g.dly; p.dlx = g.dlx;
  p.sh0 = -g.py; p.sw0 = -g.px; p.shs = g.dly; p.sws = g.dlx;
  p.min_sh = -g.py; p.min_sw = -g.px;
  p.groups = g.groups; p.SCg = g.Cg; p.DCg = g.Kg;
  p.a_mstride = g.Cg * p.KHW; p.a_cstride = p.KHW; p.w_group_stride = g.Kg * g.Cg * p.KHW;
  p.mtiles = (g.Kg + BM - 1) / BM;
  return dtype == FLHIP_F32 ? launch<float, false>(p, x, w, bias, y, s)
                            : launch<bf16_t, false>(p, x, w, bias, y, s);
}

int mfma_slab_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                            hipStream_t s) {
  if (g.sy != 1 || g.sx != 1) return -1;
  SlabParams p{};
  p.N = g.N; p.SC = g.K; p.SH = g.OH; p.SW = g.OW; p.DC = g.C; p.DH = g.H; p.DW = g.W;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW; p.dly = g.dly; p.dlx = g.dlx;
  p.sh0 = g.py; p.sw0 = g.px; p.shs = -g.dly; p.sws = -g.dlx;
  p.min_sh = g.py - (g.KH - 1) * g.dly; p.min_sw = g.px - (g.KW - 1) * g.dlx;
  p.groups = g.groups; p.SCg = g.Kg; p.DCg = g.Cg;
  p.a_mstride = p.KHW; p.a_cstride = g.Cg * p.KHW; p.w_group_stride = g.Kg * g.Cg * p.KHW;
  p.mtiles = (g.Cg + BM - 1) / BM;
  return dtype == FLHIP_F32 ? launch<float, true>(p, dy, w, nullptr, dx, s)
                            : launch<bf16_t, true>(p, dy, w, nullptr, dx, s);
}

}  // namespace flhip
