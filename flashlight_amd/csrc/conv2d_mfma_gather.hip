// Implicit-GEMM convolution on the gfx950 matrix cores: forward and
// backward-data.
//
// Both are one "gather" kernel.  The result tensor D [N, DC, DH, DW] is a GEMM
//   D[m, P] = sum_kk A[m, kk] * B[kk, P]
//   m  = result channel inside its group,
//   P  = flattened result position (n, h, w),
//   kk = (source channel, kh, kw) in the weights' own memory order,
//   A  = weights, read in place (no reordering pass),
//   B  = source values gathered on the fly (im2col never exists in memory).
// A workgroup owns a 64 x (16*NB) tile of D and has 8 waves with two roles:
//   waves 0-3 ("gather"): one result position per thread; per K-chunk of 16 rows
//     each thread fetches its position's 16 values (coalesced along W,
//     branch-free: out-of-image taps become out-of-range buffer loads, which
//     return zero) plus its share of the weight tile, two chunks ahead of the
//     matrix cores, and stores the chunk that arrived into the LDS buffer the
//     MFMA waves are not reading;
//   waves 4-7 ("mfma"): arranged 2 (M) x 2 (N); wave (wm, wn) owns 32 x (16*nt)
//     of the tile, nt = floor or ceil of NB/2, reads its LDS fragments and issues
//     the chunk's MFMAs back to back (the loop is compiled per nt so that it is
//     straight-line code).
// Wave w and wave w+4 sit on the same SIMD, so the hardware overlaps address
// arithmetic, loads and LDS stores of one with the MFMAs of the other; the two
// roles meet at one barrier per chunk (double-buffered LDS).  Two workgroups
// share a CU.  What a K row means (channel offset, window shift) is decoded once
// per kernel into an LDS table that the gather waves read 16 rows at a time.
// NB is chosen per launch so that the tile count fills 2 slots per CU with as
// little tail as possible (NB = 13 for 32x64x56x56: 483 workgroups, 512 slots).
//
// v_mfma_f32_16x16x4_f32 operand layout (lane l of 64):
//   A operand: A[i = l%16][k = l/16]     B operand: B[k = l/16][j = l%16]
//   result   : D[i = 4*(l/16) + r][j = l%16], r = 0..3
#include <map>
#include <mutex>
#include <utility>
#include "conv2d_mfma.h"

namespace flhip {

static int g_num_cus = 0;
int mfma_num_cus() {
  if (g_num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_num_cus = n;
    else
      g_num_cus = 256;
  }
  return g_num_cus;
}

bool mfma_allow_lds(const void* func, size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  if (bytes > 160 * 1024) return false;
  // the limit is kept per (kernel, device): raised once, not on every launch
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, size_t> raised;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = raised[std::make_pair(func, dev)];
  if (bytes <= have) return true;
  if (hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return false;
  have = bytes;
  return true;
}

namespace {

constexpr int KC = 16;        // K rows per chunk
constexpr int BM = MFMA_BM;
constexpr int APITCH = 80;    // LDS pitch of the A tile (== 16 mod 32 banks)
constexpr int NT_MAX = 8;     // 16-wide position blocks per wave
constexpr int NB_MAX = 2 * NT_MAX;
constexpr int GTHREADS = 256;              // gather threads (waves 0-3)
constexpr int THREADS = 2 * GTHREADS;      // plus the four MFMA waves
constexpr int AROWS = BM * KC / GTHREADS;  // A elements per gather thread and chunk

enum { MODE_FWD = 0, MODE_BWD_S1 = 1, MODE_BWD_GEN = 2 };

struct GatherParams {
  int N, SC, SH, SW, DC, DH, DW;  // source [N,SC,SH,SW], result [N,DC,DH,DW]
  int KH, KW, KHW;
  int sy, sx, py, px, dly, dlx;
  int groups, SCg, DCg;
  int Ktot;             // SCg*KH*KW
  int nchunks;          // ceil(Ktot / KC)
  int a_mstride;        // weight stride between result channels
  int w_group_stride;   // weight stride between groups
  int a_bwd_kstride;    // bwd: weight stride between source channels (Cg*KHW)
  int q16, r16;         // KC = q16*KHW + r16
  int NB;               // position blocks per workgroup
  int BNP;              // LDS pitch of the B tile
  int mtiles;
  int Ptotal;           // N*DH*DW
  int DHW, SHW;
  unsigned src_bytes, wgt_bytes;
};

// K-row table in LDS, tabA[kk] = {x, y}, tabB[kk] = z:
//   stride-1 modes: x = byte offset contributed by the row (channel and window
//     shift), y / z = low / high word of (1 << tap).  Whether a tap falls inside
//     the image depends on the position only, so every gather thread keeps a
//     64-bit validity mask over the taps and tests one bit per element;
//   general backward mode: x = byte offset of the channel, y = dh, z = dw
//     (dh = -2^20 marks a row past Ktot) and validity is computed per element.
constexpr int ROW_INVALID = -(1 << 20);

template <typename T, int MODE>
__global__ void __launch_bounds__(THREADS, 4)
gather_conv_kernel(GatherParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                   const float* __restrict__ bias, T* __restrict__ dst) {
  extern __shared__ float lds[];
  const int bstride = KC * p.BNP, astride = KC * APITCH;
  float* Bs = lds;                                   // [2][KC][BNP]
  float* As = lds + 2 * bstride;                     // [2][KC][APITCH]
  const int nrows = (p.nchunks + 2) * KC;              // two chunks of padding rows
  int2* tabA = reinterpret_cast<int2*>(As + 2 * astride);   // [nrows]
  int* tabB = reinterpret_cast<int*>(tabA + nrows);           // [nrows]
  const int esz = (int)sizeof(T);
  const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
  const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wgt_bytes);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = blockIdx.y / p.mtiles, mtile = blockIdx.y % p.mtiles;
  const int BN = p.NB * 16;
  const int tile_p0 = blockIdx.x * BN;
  const int m_lim = p.DCg - mtile * BM;               // valid result channels in the tile
  const int n = p.nchunks;

  // ---- K-row table, once per kernel -------------------------------------------
  for (int kk = tid; kk < nrows; kk += THREADS) {
    int2 ra = make_int2(0, ROW_INVALID);
    int rb = 0;
    if (kk < p.Ktot) {
      const int c = kk / p.KHW, t = kk - c * p.KHW;
      const int kh = t / p.KW, kw = t - kh * p.KW;
      const int dh = (MODE == MODE_FWD ? kh : -kh) * p.dly;
      const int dw = (MODE == MODE_FWD ? kw : -kw) * p.dlx;
      if (MODE == MODE_BWD_GEN) {
        ra.x = c * p.SHW * esz;
        ra.y = dh;
        rb = dw;
      } else {
        ra.x = (c * p.SHW + dh * p.SW + dw) * esz;
        ra.y = t < 32 ? (int)(1u << t) : 0;
        rb = t >= 32 ? (int)(1u << (t - 32)) : 0;
      }
    } else if (MODE != MODE_BWD_GEN) {
      ra.y = 0;
    }
    tabA[kk] = ra;
    tabB[kk] = rb;
  }
  __syncthreads();

  if (wave < 4) {
    // =========================== gather waves ==================================
    const int P = tile_p0 + tid;
    const bool pvalid = tid < BN && P < p.Ptotal;
    int hb, wb, pixbase;
    {
      const int Pc = pvalid ? P : 0;
      const int ni = Pc / p.DHW, q = Pc - ni * p.DHW;
      const int h = q / p.DW, w = q - h * p.DW;
      if (MODE == MODE_FWD) {
        hb = h * p.sy - p.py;
        wb = w * p.sx - p.px;
      } else {
        hb = h + p.py;
        wb = w + p.px;
      }
      pixbase = (ni * p.SC + grp * p.SCg) * p.SHW;
      if (MODE != MODE_BWD_GEN) pixbase += hb * p.SW + wb;
      pixbase *= esz;                                  // byte offset
      if (!pvalid) hb = 4 * ROW_INVALID;               // every tap fails the bounds test
    }
    unsigned mask_lo = 0, mask_hi = 0;                 // taps that fall inside the image
    if (MODE != MODE_BWD_GEN) {
      for (int t = 0; t < p.KHW; ++t) {
        const int kh = t / p.KW, kw = t - kh * p.KW;
        const int ih = hb + (MODE == MODE_FWD ? kh : -kh) * p.dly;
        const int iw = wb + (MODE == MODE_FWD ? kw : -kw) * p.dlx;
        const unsigned ok = ((unsigned)ih < (unsigned)p.SH) & ((unsigned)iw < (unsigned)p.SW);
        if (t < 32)
          mask_lo |= ok << t;
        else
          mask_hi |= ok << (t - 32);
      }
    }
    const bool taps64 = p.KHW > 32;
    // share of the A tile: row ar = tid%16, m = tid/16 + 16*i
    const int ar = tid & 15, am = tid >> 4;
    const int wbase = grp * p.w_group_stride + mtile * BM * p.a_mstride;   // elements
    int a_kk = ar, a_c = 0, a_t = ar;                  // row of the chunk being fetched
    if (MODE != MODE_FWD) {
      a_c = ar / p.KHW;
      a_t = ar - a_c * p.KHW;
    }

    auto load_chunk = [&](int chunk, float (&breg)[KC], float (&areg)[AROWS]) {
      int goff[KC], dh[KC], dw[KC];
      {
        const int4* ta = reinterpret_cast<const int4*>(tabA + chunk * KC);
        const int4* tb = reinterpret_cast<const int4*>(tabB + chunk * KC);
#pragma unroll
        for (int i = 0; i < KC / 2; ++i) {
          const int4 v = ta[i];
          goff[2 * i] = v.x; dh[2 * i] = v.y; goff[2 * i + 1] = v.z; dh[2 * i + 1] = v.w;
        }
        if (MODE == MODE_BWD_GEN || taps64) {
#pragma unroll
          for (int i = 0; i < KC / 4; ++i) {
            const int4 v = tb[i];
            dw[4 * i] = v.x; dw[4 * i + 1] = v.y; dw[4 * i + 2] = v.z; dw[4 * i + 3] = v.w;
          }
        }
      }
#pragma unroll
      for (int r = 0; r < KC; ++r) {
        bool ok;
        int off;
        if (MODE == MODE_BWD_GEN) {
          const int th = hb + dh[r], tw = wb + dw[r];
          const int ih = th / p.sy, iw = tw / p.sx;
          ok = (th >= 0) & (tw >= 0) & (ih * p.sy == th) & (iw * p.sx == tw) & (ih < p.SH) &
               (iw < p.SW);
          off = pixbase + goff[r] + (ih * p.SW + iw) * esz;
        } else {
          unsigned m = mask_lo & (unsigned)dh[r];
          if (taps64) m |= mask_hi & (unsigned)dw[r];
          ok = m != 0;
          off = pixbase + goff[r];
        }
        breg[r] = buf_ld(srsrc, ok ? off : -1, src);
      }
      const int arow = wbase + (MODE == MODE_FWD ? a_kk : a_c * p.a_bwd_kstride + a_t);
      const bool kok = a_kk < p.Ktot;
#pragma unroll
      for (int i = 0; i < AROWS; ++i) {
        const int m = am + 16 * i;
        const bool ok = kok & (m < m_lim);
        areg[i] = buf_ld(wrsrc, ok ? (m * p.a_mstride + arow) * esz : -1, wgt);
      }
      a_kk += KC;
      if (MODE != MODE_FWD) {
        a_c += p.q16;
        a_t += p.r16;
        if (a_t >= p.KHW) {
          a_t -= p.KHW;
          ++a_c;
        }
      }
    };
    auto store_chunk = [&](int buf, const float (&breg)[KC], const float (&areg)[AROWS]) {
      float* bs = Bs + buf * bstride;
      float* as = As + buf * astride;
#pragma unroll
      for (int r = 0; r < KC; ++r) bs[r * p.BNP + tid] = breg[r];
#pragma unroll
      for (int i = 0; i < AROWS; ++i) as[ar * APITCH + am + 16 * i] = areg[i];
    };

    // Two register sets: chunk c+1 waits in one while chunk c+2 is being fetched
    // into the other, so a fetch has two MFMA phases to come back from HBM.  The
    // table has two chunks of padding rows, so fetching past the end is harmless.
    float bregA[KC], aregA[AROWS], bregB[KC], aregB[AROWS];
    load_chunk(0, bregA, aregA);
    store_chunk(0, bregA, aregA);
    load_chunk(1, bregB, aregB);
    __syncthreads();
    for (int c = 0; c < n; c += 2) {
      load_chunk(c + 2, bregA, aregA);
      store_chunk(1, bregB, aregB);              // chunk c+1
      __syncthreads();
      if (c + 1 >= n) break;
      load_chunk(c + 3, bregB, aregB);
      store_chunk(0, bregA, aregA);              // chunk c+2
      __syncthreads();
    }
    return;
  }

  // ============================= MFMA waves ====================================
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

    __syncthreads();                             // chunk 0 is in LDS buffer 0
    for (int c = 0; c < n; ++c) {
      const float* as = As + (c & 1) * astride + wm * 32 + fr;
      const float* bs = Bs + (c & 1) * bstride + nb0 * 16 + fr;
      float a[KC / 4][2], b[KC / 4][NT];
#pragma unroll
      for (int ks = 0; ks < KC / 4; ++ks) {
        const int krow = ks * 4 + fk;
        a[ks][0] = as[krow * APITCH];
        a[ks][1] = as[krow * APITCH + 16];
#pragma unroll
        for (int j = 0; j < NT; ++j) b[ks][j] = bs[krow * p.BNP + j * 16];
      }
      __builtin_amdgcn_sched_barrier(0);         // all fragment reads ahead of the MFMAs
#pragma unroll
      for (int ks = 0; ks < KC / 4; ++ks) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ks][0], b[ks][j], acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ks][1], b[ks][j], acc[1][j], 0, 0, 0);
        }
      }
      __syncthreads();
    }

    // ---- epilogue: bias and store ---------------------------------------------
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int Pj = tile_p0 + (nb0 + j) * 16 + fr;
      if (Pj < p.Ptotal) {
        const int ni = Pj / p.DHW, q = Pj - ni * p.DHW;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = wm * 32 + i * 16 + fk * 4 + r;
            if (m < m_lim) {
              const int ch = grp * p.DCg + mtile * BM + m;
              float v = acc[i][j][r];
              if (bias) v += bias[ch];
              st(dst, (size_t)(ni * p.DC + ch) * p.DHW + q, v);
            }
          }
        }
      }
    }
  };

  switch (nt) {
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 6: run(std::integral_constant<int, 6>{}); break;
    case 7: run(std::integral_constant<int, 7>{}); break;
    default: run(std::integral_constant<int, 8>{}); break;
  }
}

// Chooses the number of 16-position blocks per workgroup so that the tile count
// wastes as little of the last pass of workgroups over the CUs as possible.
int choose_nb(long long pblocks, int mtiles_total, int slots) {
  int best = 8;
  double best_cost = 1e30;
  for (int nb = 8; nb <= NB_MAX; ++nb) {
    const long long tiles = ((pblocks + nb - 1) / nb) * mtiles_total;
    const long long rounds = (tiles + slots - 1) / slots;
    // time ~ rounds * nb (+ a small fixed cost per round for prologue/epilogue)
    const double cost = (double)rounds * (nb + 1.0);
    if (cost < best_cost - 1e-9 || (cost < best_cost + 1e-9 && nb > best)) {
      best_cost = cost;
      best = nb;
    }
  }
  return best;
}

template <typename T, int MODE>
int launch_gather(const GatherParams& p0, const void* src, const void* wgt, const float* bias,
                  void* dst, hipStream_t s) {
  GatherParams p = p0;
  // byte offsets are 32-bit; rows past Ktot rely on |shift| < 2^20
  const long long sbytes = (long long)p.N * p.SC * p.SHW * (long long)sizeof(T);
  const long long wbytes = (long long)p.groups * p.w_group_stride * (long long)sizeof(T);
  const int hmax = MODE == MODE_FWD ? p.DH * p.sy : p.DH + p.py;
  if (sbytes >= (1ll << 31) || wbytes >= (1ll << 31) || hmax >= (1 << 19) ||
      (p.KH - 1) * p.dly >= (1 << 19) || (MODE != MODE_BWD_GEN && p.KHW > 64))
    return -1;
  p.src_bytes = (unsigned)sbytes;
  p.wgt_bytes = (unsigned)wbytes;
  p.nchunks = (p.Ktot + KC - 1) / KC;
  p.q16 = KC / p.KHW;
  p.r16 = KC % p.KHW;
  const long long pblocks = ((long long)p.Ptotal + 15) / 16;
  p.NB = choose_nb(pblocks, p.mtiles * p.groups, 2 * mfma_num_cus());
  const int BN = p.NB * 16;
  (void)BN;
  p.BNP = GTHREADS + 16;                     // every gather thread owns a column; == 16 mod 32
  const size_t shmem = (size_t)2 * (KC * p.BNP + KC * APITCH) * sizeof(float) +
                       (size_t)(p.nchunks + 2) * KC * 3 * sizeof(int);
  auto kernel = gather_conv_kernel<T, MODE>;
  if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
  const dim3 grid((unsigned)((pblocks + p.NB - 1) / p.NB), (unsigned)(p.mtiles * p.groups));
  hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const T*>(src),
                     static_cast<const T*>(wgt), bias, static_cast<T*>(dst));
  return check_launch("conv2d (mfma)");
}

}  // namespace

int mfma_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias,
                  void* y, hipStream_t s) {
  GatherParams p{};
  p.N = g.N; p.SC = g.C; p.SH = g.H; p.SW = g.W; p.DC = g.K; p.DH = g.OH; p.DW = g.OW;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW;
  p.sy = g.sy; p.sx = g.sx; p.py = g.py; p.px = g.px; p.dly = g.dly; p.dlx = g.dlx;
  p.groups = g.groups; p.SCg = g.Cg; p.DCg = g.Kg;
  p.Ktot = g.Cg * p.KHW;
  p.a_mstride = p.Ktot;
  p.w_group_stride = g.Kg * p.Ktot;
  p.a_bwd_kstride = 0;
  p.mtiles = (g.Kg + BM - 1) / BM;
  p.Ptotal = g.N * g.OH * g.OW;
  p.DHW = g.OH * g.OW; p.SHW = g.H * g.W;
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch_gather<T, MODE_FWD>(p, x, w, bias, y, s);
  });
}

int mfma_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                       hipStream_t s) {
  GatherParams p{};
  p.N = g.N; p.SC = g.K; p.SH = g.OH; p.SW = g.OW; p.DC = g.C; p.DH = g.H; p.DW = g.W;
  p.KH = g.KH; p.KW = g.KW; p.KHW = g.KH * g.KW;
  p.sy = g.sy; p.sx = g.sx; p.py = g.py; p.px = g.px; p.dly = g.dly; p.dlx = g.dlx;
  p.groups = g.groups; p.SCg = g.Kg; p.DCg = g.Cg;
  p.Ktot = g.Kg * p.KHW;
  p.a_mstride = p.KHW;
  p.w_group_stride = g.Kg * g.Cg * p.KHW;
  p.a_bwd_kstride = g.Cg * p.KHW;
  p.mtiles = (g.Cg + BM - 1) / BM;
  p.Ptotal = g.N * g.H * g.W;
  p.DHW = g.H * g.W; p.SHW = g.OH * g.OW;
  const bool s1 = g.sy == 1 && g.sx == 1;
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return s1 ? launch_gather<T, MODE_BWD_S1>(p, dy, w, nullptr, dx, s)
              : launch_gather<T, MODE_BWD_GEN>(p, dy, w, nullptr, dx, s);
  });
}

}  // namespace flhip
