// Implicit-GEMM convolution on the gfx950 matrix cores.
//
// Forward and backward-data share one "gather" kernel: the result tensor D
// [N, DC, DH, DW] is a GEMM  D[m, P] = sum_kk A[m, kk] * B[kk, P]  with
//   m  = result channel inside its group,
//   P  = flattened result position (n, h, w),
//   kk = (source channel, kh, kw) in the weights' own memory order,
//   A  = weights (read in place, no reordering pass),
//   B  = source values gathered on the fly (im2col never exists in memory).
// A workgroup of 8 waves owns a 64 x (16*NB) tile of D.  Per K-chunk of 16 rows
// the B tile is gathered with one thread per result position (coalesced along
// W) into registers while the matrix cores work on the previous chunk out of
// LDS; the per-row decoding of kk (channel offset, window shift) is done once
// per chunk by 16 threads into a small LDS table, so the per-element cost is an
// add, a bounds test, a load and an LDS store.  Waves are arranged 2 (M) x 4 (N);
// each owns 32 x (16*nt) of the tile with nt in {ceil, floor}(NB/4), which lets NB
// be chosen so that the tile count just fills the 256 CUs in one round (NB = 25
// for 32x64x56x56: 251 workgroups).
//
// v_mfma_f32_16x16x4_f32 operand layout (lane l of 64):
//   A operand: A[i = l%16][k = l/16]     B operand: B[k = l/16][j = l%16]
//   result   : D[i = 4*(l/16) + r][j = l%16], r = 0..3
#include "conv2d.h"

namespace flhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int KC = 16;        // K rows per chunk
constexpr int BM = 64;        // result channels per workgroup
constexpr int APITCH = 80;    // LDS pitch of the A tile (== 16 mod 32 banks)
constexpr int NT_MAX = 7;     // 16-wide position blocks per wave
constexpr int NB_MAX = 4 * NT_MAX;
constexpr int THREADS = 512;

enum { MODE_FWD = 0, MODE_BWD_S1 = 1, MODE_BWD_GEN = 2 };

struct GatherParams {
  int N, SC, SH, SW, DC, DH, DW;  // source [N,SC,SH,SW], result [N,DC,DH,DW]
  int KH, KW, KHW;
  int sy, sx, py, px, dly, dlx;
  int groups, SCg, DCg;
  int Ktot;             // SCg*KH*KW
  int a_mstride;        // weight stride between result channels
  int w_group_stride;   // weight stride between groups
  int a_bwd_kstride;    // bwd: weight stride between source channels (Cg*KHW)
  int NB;               // position blocks per workgroup
  int BNP;              // LDS pitch of the B tile
  int mtiles;
  int Ptotal;           // N*DH*DW
  int DHW, SHW;
};

struct RowInfo {
  int goff;   // source offset contributed by the row (channel and window shift)
  int dh, dw; // signed window shift
  int aoff;   // weight offset contributed by the row
};

template <typename T, int MODE>
__global__ void __launch_bounds__(THREADS)
gather_conv_kernel(GatherParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                   const float* __restrict__ bias, T* __restrict__ dst) {
  extern __shared__ float lds[];
  float* Bs = lds;                                  // [KC][BNP]
  float* As = lds + KC * p.BNP;                     // [KC][APITCH]
  RowInfo* tab = reinterpret_cast<RowInfo*>(As + KC * APITCH);  // [2][KC]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;          // waves w and w+4 share a SIMD
  const int grp = blockIdx.y / p.mtiles, mtile = blockIdx.y % p.mtiles;
  const int BN = p.NB * 16;
  const int tile_p0 = blockIdx.x * BN;

  // this wave's share of the NB position blocks
  const int base = p.NB >> 2, rem = p.NB & 3;
  const int nt = base + (wn < rem ? 1 : 0);
  const int nb0 = wn * base + min(wn, rem);

  // ---- per-thread gather position (one result position per thread) --------
  const bool loader = tid < BN;
  const int P = tile_p0 + tid;
  bool pvalid = loader && P < p.Ptotal;
  int hb = 0, wb = 0, pixbase = 0;
  {
    const int Pc = pvalid ? P : 0;
    const int n = Pc / p.DHW, q = Pc - n * p.DHW;
    const int h = q / p.DW, w = q - h * p.DW;
    if (MODE == MODE_FWD) {
      hb = h * p.sy - p.py;
      wb = w * p.sx - p.px;
    } else {
      hb = h + p.py;
      wb = w + p.px;
    }
    pixbase = (n * p.SC + grp * p.SCg) * p.SHW;
    if (MODE != MODE_BWD_GEN) pixbase += hb * p.SW + wb;
  }

  // ---- per-thread share of the A tile: rows r = tid%16, m = tid/16 (+32) ---
  const int ar = tid & 15, am = tid >> 4;
  const int m_lim = p.DCg - mtile * BM;             // valid result channels in tile
  const T* wbase = wgt + (size_t)grp * p.w_group_stride + (size_t)(mtile * BM) * p.a_mstride;

  auto fill_table = [&](int chunk, int slot) {
    if (tid < KC) {
      const int kk = chunk * KC + tid;
      RowInfo ri;
      if (kk < p.Ktot) {
        const int c = kk / p.KHW, t = kk - c * p.KHW;
        const int kh = t / p.KW, kw = t - kh * p.KW;
        if (MODE == MODE_FWD) {
          ri.dh = kh * p.dly;
          ri.dw = kw * p.dlx;
          ri.aoff = kk;
        } else {
          ri.dh = -kh * p.dly;
          ri.dw = -kw * p.dlx;
          ri.aoff = c * p.a_bwd_kstride + t;
        }
        ri.goff = c * p.SHW;
        if (MODE != MODE_BWD_GEN) ri.goff += ri.dh * p.SW + ri.dw;
      } else {
        ri.goff = 0;
        ri.dh = -(1 << 28);   // forces the bounds test to fail
        ri.dw = 0;
        ri.aoff = -1;
      }
      tab[slot * KC + tid] = ri;
    }
  };

  float breg[KC];
  float areg[2];

  auto load_chunk = [&](int slot) {
    const RowInfo* tb = tab + slot * KC;
#pragma unroll
    for (int r = 0; r < KC; ++r) {
      const RowInfo ri = tb[r];
      float v = 0.f;
      if (MODE == MODE_BWD_GEN) {
        const int th = hb + ri.dh, tw = wb + ri.dw;
        const int ih = th / p.sy, iw = tw / p.sx;
        if (pvalid && th >= 0 && tw >= 0 && ih * p.sy == th && iw * p.sx == tw && ih < p.SH &&
            iw < p.SW)
          v = ld(src, (size_t)(pixbase + ri.goff + ih * p.SW + iw));
      } else {
        const int ih = hb + ri.dh, iw = wb + ri.dw;
        if (pvalid && (unsigned)ih < (unsigned)p.SH && (unsigned)iw < (unsigned)p.SW)
          v = ld(src, (size_t)(pixbase + ri.goff));
      }
      breg[r] = v;
    }
    const int aoff = tb[ar].aoff;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = am + 32 * i;
      areg[i] = (aoff >= 0 && m < m_lim) ? ld(wbase, (size_t)m * p.a_mstride + aoff) : 0.f;
    }
  };

  auto store_chunk = [&]() {
    if (loader) {
#pragma unroll
      for (int r = 0; r < KC; ++r) Bs[r * p.BNP + tid] = breg[r];
    }
    As[ar * APITCH + am] = areg[0];
    As[ar * APITCH + am + 32] = areg[1];
  };

  floatx4 acc[2][NT_MAX];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NT_MAX; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int nchunks = (p.Ktot + KC - 1) / KC;
  fill_table(0, 0);
  __syncthreads();
  load_chunk(0);
  fill_table(1, 1);
  store_chunk();
  __syncthreads();

  const int fr = lane & 15, fk = lane >> 4;
  for (int c = 0; c < nchunks; ++c) {
    const bool more = c + 1 < nchunks;
    if (more) load_chunk((c + 1) & 1);
    fill_table(c + 2, c & 1);
#pragma unroll
    for (int ks = 0; ks < KC / 4; ++ks) {
      const int krow = ks * 4 + fk;
      const float a0 = As[krow * APITCH + wm * 32 + fr];
      const float a1 = As[krow * APITCH + wm * 32 + 16 + fr];
      const float* brow = Bs + krow * p.BNP + nb0 * 16 + fr;
#pragma unroll
      for (int j = 0; j < NT_MAX; ++j) {
        if (j < nt) {
          const float b = brow[j * 16];
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b, acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b, acc[1][j], 0, 0, 0);
        }
      }
    }
    __syncthreads();
    if (more) store_chunk();
    __syncthreads();
  }

  // ---- epilogue: bias and store ---------------------------------------------
#pragma unroll
  for (int j = 0; j < NT_MAX; ++j) {
    if (j < nt) {
      const int Pj = tile_p0 + (nb0 + j) * 16 + fr;
      if (Pj < p.Ptotal) {
        const int n = Pj / p.DHW, q = Pj - n * p.DHW;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = wm * 32 + i * 16 + fk * 4 + r;
            if (m < m_lim) {
              const int ch = grp * p.DCg + mtile * BM + m;
              float v = acc[i][j][r];
              if (bias) v += bias[ch];
              st(dst, (size_t)(n * p.DC + ch) * p.DHW + q, v);
            }
          }
        }
      }
    }
  }
}

// Chooses the number of 16-position blocks per workgroup so that the tile count
// wastes as little of the last round over the CUs as possible.
int choose_nb(long long pblocks, int mtiles_total, int num_cus) {
  int best = 8;
  double best_cost = 1e30;
  for (int nb = 8; nb <= NB_MAX; ++nb) {
    const long long tiles = ((pblocks + nb - 1) / nb) * mtiles_total;
    const long long rounds = (tiles + num_cus - 1) / num_cus;
    // time ~ rounds * nb (+ a small fixed cost per round for prologue/epilogue)
    const double cost = (double)rounds * (nb + 1.0);
    if (cost < best_cost - 1e-9 || (cost < best_cost + 1e-9 && nb > best)) {
      best_cost = cost;
      best = nb;
    }
  }
  return best;
}

int num_cus() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}

template <typename T, int MODE>
int launch_gather(const GatherParams& p0, const void* src, const void* wgt, const float* bias,
                  void* dst, hipStream_t s) {
  GatherParams p = p0;
  const long long pblocks = ((long long)p.Ptotal + 15) / 16;
  p.NB = choose_nb(pblocks, p.mtiles * p.groups, num_cus());
  const int BN = p.NB * 16;
  p.BNP = BN + ((16 - BN % 32) + 32) % 32;   // == 16 mod 32
  const size_t shmem = (size_t)(KC * p.BNP + KC * APITCH) * sizeof(float) + 2 * KC * sizeof(RowInfo);
  const dim3 grid((unsigned)((pblocks + p.NB - 1) / p.NB), (unsigned)(p.mtiles * p.groups));
  hipLaunchKernelGGL((gather_conv_kernel<T, MODE>), grid, dim3(THREADS), shmem, s, p,
                     static_cast<const T*>(src), static_cast<const T*>(wgt), bias,
                     static_cast<T*>(dst));
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
  return dtype == FLHIP_F32 ? launch_gather<float, MODE_FWD>(p, x, w, bias, y, s)
                            : launch_gather<bf16_t, MODE_FWD>(p, x, w, bias, y, s);
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
  if (dtype == FLHIP_F32)
    return s1 ? launch_gather<float, MODE_BWD_S1>(p, dy, w, nullptr, dx, s)
              : launch_gather<float, MODE_BWD_GEN>(p, dy, w, nullptr, dx, s);
  return s1 ? launch_gather<bf16_t, MODE_BWD_S1>(p, dy, w, nullptr, dx, s)
            : launch_gather<bf16_t, MODE_BWD_GEN>(p, dy, w, nullptr, dx, s);
}

// ---------------------------------------------------------------------------
// Filter gradient: dw[m, j] = sum_P dy[m, P] * x_gathered[P, j] per group, with
// m = output channel, j = (input channel, kh, kw) in dw's own memory order and
// P = (n, oh, ow).  The long reduction over P is split over `nsplit`
// workgroups per output tile; each writes an fp32 partial tile to the workspace
// and a second kernel adds the partials in a fixed order (deterministic, no
// atomics).  The bias gradient rides along: the dy tile is already in LDS, so
// the workgroups of the first column tile also sum it per channel.
// ---------------------------------------------------------------------------
namespace {

constexpr int WKC = 16;         // positions per K-chunk
constexpr int WKP = 17;         // LDS pitch of both tiles (positions contiguous)
constexpr int WNT_MAX = 9;      // 16-column blocks per wave
constexpr int WNB_MAX = 4 * WNT_MAX;

struct WgradParams {
  int N, C, H, W, K, OH, OW;
  int KH, KW, KHW, sy, sx, py, px, dly, dlx;
  int groups, Cg, Kg;
  int ncols;        // Cg*KHW
  int NBW;          // 16-column blocks per workgroup tile
  int ntiles_n, mtiles;
  int nsplit, pps;  // K-splits and positions per split (multiple of WKC)
  int Ptotal, OHW, HW;
  int E;            // K*Cg*KHW: elements of dw
  int want_db;
};

struct ColInfo {
  int coff;   // c*HW + kh*dly*W + kw*dlx, or -1 for a padding column
  int dhw;    // (kh*dly) << 16 | (kw*dlx)
};

template <typename T>
__global__ void __launch_bounds__(THREADS)
wgrad_kernel(WgradParams p, const T* __restrict__ x, const T* __restrict__ dy,
             float* __restrict__ out /* dw when nsplit == 1, else partials */,
             float* __restrict__ db_out) {
  extern __shared__ float lds[];
  const int BNW = p.NBW * 16;
  float* Bs = lds;                                  // [BNW][WKP]
  float* As = lds + BNW * WKP;                      // [BM][WKP]
  ColInfo* ctab = reinterpret_cast<ColInfo*>(As + BM * WKP);   // [BNW]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int split = blockIdx.x;
  const int ntile = blockIdx.y % p.ntiles_n, mtile = blockIdx.y / p.ntiles_n;
  const int grp = blockIdx.z;
  const int col0 = ntile * BNW;

  const int base = p.NBW >> 2, rem = p.NBW & 3;
  const int nt = base + (wn < rem ? 1 : 0);
  const int nb0 = wn * base + min(wn, rem);

  for (int j = tid; j < BNW; j += THREADS) {
    const int col = col0 + j;
    ColInfo ci;
    if (col < p.ncols) {
      const int c = col / p.KHW, t = col - c * p.KHW;
      const int kh = t / p.KW, kw = t - kh * p.KW;
      ci.coff = c * p.HW + kh * p.dly * p.W + kw * p.dlx;
      ci.dhw = ((kh * p.dly) << 16) | (kw * p.dlx);
    } else {
      ci.coff = -1;
      ci.dhw = 0;
    }
    ctab[j] = ci;
  }
  __syncthreads();

  const int pl = tid & 15, cl = tid >> 4;            // position lane, column/channel lane
  const int m_lim = p.Kg - mtile * BM;
  const int P_begin = split * p.pps, P_end = min(P_begin + p.pps, p.Ptotal);
  const int nchunks = (P_end - P_begin + WKC - 1) / WKC;
  const int ncl = (BNW + 31) / 32;                   // columns per thread (<= 18)

  float breg[2 * WNT_MAX];
  float areg[2];

  auto load_chunk = [&](int chunk) {
    const int P = P_begin + chunk * WKC + pl;
    const bool pv = P < P_end;
    const int Pc = pv ? P : 0;
    const int n = Pc / p.OHW, q = Pc - n * p.OHW;
    const int oh = q / p.OW, ow = q - oh * p.OW;
    const int ihb = oh * p.sy - p.py, iwb = ow * p.sx - p.px;
    const int xbase = (n * p.C + grp * p.Cg) * p.HW + ihb * p.W + iwb;
#pragma unroll
    for (int i = 0; i < 2 * WNT_MAX; ++i) {
      float v = 0.f;
      const int j = cl + 32 * i;
      if (i < ncl && j < BNW) {
        const ColInfo ci = ctab[j];
        const int ih = ihb + (ci.dhw >> 16), iw = iwb + (ci.dhw & 0xffff);
        if (pv && ci.coff >= 0 && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W)
          v = ld(x, (size_t)(xbase + ci.coff));
      }
      breg[i] = v;
    }
    const int ybase = (n * p.K + grp * p.Kg + mtile * BM) * p.OHW + q;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = cl + 32 * i;
      areg[i] = (pv && m < m_lim) ? ld(dy, (size_t)(ybase + m * p.OHW)) : 0.f;
    }
  };

  auto store_chunk = [&]() {
#pragma unroll
    for (int i = 0; i < 2 * WNT_MAX; ++i) {
      const int j = cl + 32 * i;
      if (i < ncl && j < BNW) Bs[j * WKP + pl] = breg[i];
    }
    As[cl * WKP + pl] = areg[0];
    As[(cl + 32) * WKP + pl] = areg[1];
  };

  floatx4 acc[2][WNT_MAX];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < WNT_MAX; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float dbacc = 0.f;
  const bool do_db = p.want_db && ntile == 0 && tid < BM;

  if (nchunks > 0) {
    load_chunk(0);
    store_chunk();
  }
  __syncthreads();

  const int fr = lane & 15, fk = lane >> 4;
  for (int c = 0; c < nchunks; ++c) {
    const bool more = c + 1 < nchunks;
    if (more) load_chunk(c + 1);
#pragma unroll
    for (int ks = 0; ks < WKC / 4; ++ks) {
      const int kcol = ks * 4 + fk;
      const float a0 = As[(wm * 32 + fr) * WKP + kcol];
      const float a1 = As[(wm * 32 + 16 + fr) * WKP + kcol];
      const float* bcol = Bs + (nb0 * 16 + fr) * WKP + kcol;
#pragma unroll
      for (int j = 0; j < WNT_MAX; ++j) {
        if (j < nt) {
          const float b = bcol[j * 16 * WKP];
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b, acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b, acc[1][j], 0, 0, 0);
        }
      }
    }
    if (do_db) {
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < WKC; ++k) s += As[tid * WKP + k];
      dbacc += s;
    }
    __syncthreads();
    if (more) store_chunk();
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------
  float* o = out + (p.nsplit > 1 ? (size_t)split * (p.E + p.K) : 0);
#pragma unroll
  for (int j = 0; j < WNT_MAX; ++j) {
    if (j < nt) {
      const int col = col0 + (nb0 + j) * 16 + fr;
      if (col < p.ncols) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = wm * 32 + i * 16 + fk * 4 + r;
            if (m < m_lim)
              o[(size_t)(grp * p.Kg + mtile * BM + m) * p.ncols + col] = acc[i][j][r];
          }
      }
    }
  }
  if (do_db && tid < m_lim) {
    const int ch = grp * p.Kg + mtile * BM + tid;
    if (p.nsplit > 1)
      o[p.E + ch] = dbacc;
    else
      db_out[ch] = dbacc;
  }
}

// out[e] = sum over s of part[s][e]; elements past E go to db.
__global__ void __launch_bounds__(256)
wgrad_reduce_kernel(const float* __restrict__ part, int nsplit, int E, int K, int want_db,
                    float* __restrict__ dw, float* __restrict__ db) {
  __shared__ float red[4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int e = blockIdx.x * 64 + tx;
  const int total = E + (want_db ? K : 0);
  const size_t stride = (size_t)E + K;
  float s0 = 0.f, s1 = 0.f;
  if (e < total) {
    int s = ty;
    for (; s + 4 < nsplit; s += 8) {
      s0 += part[(size_t)s * stride + e];
      s1 += part[(size_t)(s + 4) * stride + e];
    }
    if (s < nsplit) s0 += part[(size_t)s * stride + e];
  }
  red[ty][tx] = s0 + s1;
  __syncthreads();
  if (ty == 0 && e < total) {
    const float v = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
    if (e < E)
      dw[e] = v;
    else
      db[e - E] = v;
  }
}

bool wgrad_plan(const ConvGeom& g, WgradParams* p) {
  p->N = g.N; p->C = g.C; p->H = g.H; p->W = g.W; p->K = g.K; p->OH = g.OH; p->OW = g.OW;
  p->KH = g.KH; p->KW = g.KW; p->KHW = g.KH * g.KW;
  p->sy = g.sy; p->sx = g.sx; p->py = g.py; p->px = g.px; p->dly = g.dly; p->dlx = g.dlx;
  p->groups = g.groups; p->Cg = g.Cg; p->Kg = g.Kg;
  p->ncols = g.Cg * p->KHW;
  const int nblocks = (p->ncols + 15) / 16;
  p->ntiles_n = (nblocks + WNB_MAX - 1) / WNB_MAX;
  p->NBW = (nblocks + p->ntiles_n - 1) / p->ntiles_n;
  p->mtiles = (g.Kg + BM - 1) / BM;
  p->Ptotal = g.N * g.OH * g.OW;
  p->OHW = g.OH * g.OW; p->HW = g.H * g.W;
  p->E = g.K * p->ncols;
  // window shifts are packed into 16 bits each
  if ((g.KH - 1) * g.dly >= 32768 || (g.KW - 1) * g.dlx >= 32768) return false;
  const long long base_wgs = (long long)p->ntiles_n * p->mtiles * g.groups;
  if (p->ntiles_n * p->mtiles > 65535 || g.groups > 65535) return false;
  long long ns = num_cus() / base_wgs;
  const long long max_ns = (p->Ptotal + 255) / 256;
  if (ns > max_ns) ns = max_ns;
  if (ns < 1) ns = 1;
  long long pps = (p->Ptotal + ns - 1) / ns;
  pps = (pps + WKC - 1) / WKC * WKC;
  p->pps = (int)pps;
  p->nsplit = (int)((p->Ptotal + pps - 1) / pps);
  return true;
}

}  // namespace

size_t mfma_conv_bwd_filter_ws(const ConvGeom& g, int) {
  WgradParams p{};
  if (!wgrad_plan(g, &p)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
}

int mfma_conv_bwd_filter(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                         float* db, void* ws, size_t ws_bytes, hipStream_t s) {
  if (!dw) return -1;   // bias gradient alone: the plain reduction kernel
  WgradParams p{};
  if (!wgrad_plan(g, &p)) return -1;
  p.want_db = db != nullptr;
  if (p.nsplit > 1 && (!ws || ws_bytes < (size_t)p.nsplit * (p.E + p.K) * sizeof(float)))
    return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  const int BNW = p.NBW * 16;
  const size_t shmem = (size_t)(BNW * WKP + BM * WKP) * sizeof(float) + BNW * sizeof(ColInfo);
  const dim3 grid(p.nsplit, p.ntiles_n * p.mtiles, g.groups);
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  if (dtype == FLHIP_F32)
    hipLaunchKernelGGL((wgrad_kernel<float>), grid, dim3(THREADS), shmem, s, p,
                       static_cast<const float*>(x), static_cast<const float*>(dy), out, db);
  else
    hipLaunchKernelGGL((wgrad_kernel<bf16_t>), grid, dim3(THREADS), shmem, s, p,
                       static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(dy), out, db);
  if (p.nsplit > 1) {
    const int total = p.E + (p.want_db ? p.K : 0);
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((total + 63) / 64), dim3(256), 0, s,
                       static_cast<const float*>(ws), p.nsplit, p.E, p.K, p.want_db, dw, db);
  }
  return check_launch("conv2d_bwd_filter (mfma)");
}

}  // namespace flhip
