// Filter (and bias) gradient on the gfx950 matrix cores.
//
// Per group: dw[m, j] = sum_P dy[m, P] * xg[P, j], with m = output channel,
// j = (input channel, kh, kw) in dw's own memory order, P = (n, oh, ow) and xg
// the input gathered through the window (never materialised).  The long
// reduction over P is split over `nsplit` workgroups per output tile; each
// writes an fp32 partial tile to the workspace and a second kernel adds the
// partials in a fixed order, so the result is deterministic and uses no
// atomics.  The bias gradient rides along: the dy tile is already in LDS, so
// the workgroups of the first column tile also sum it per channel.
//
// A workgroup of 4 waves (2 along m x 2 along j) owns 64 x (16*NBW) of dw, two
// workgroups share a CU; P is
// walked in chunks of 16 positions through double-buffered LDS tiles stored
// [row][position] with pitch 17.  What a column j means (channel offset, window
// shift) is decoded once per kernel; every thread keeps the entries of its own
// columns in registers.  Padding is fetched as out-of-range buffer loads (zero).
#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int THREADS = 256;    // 4 waves
constexpr int BM = MFMA_BM;
constexpr int WKC = 16;         // positions per K-chunk
constexpr int WKP = 17;         // LDS pitch of both tiles (positions contiguous)
constexpr int WNT_MAX = 8;      // 16-column blocks per wave
constexpr int WNB_MAX = 2 * WNT_MAX;
constexpr int WCL_MAX = WNB_MAX;        // columns gathered per thread (16 per block / 16 lanes)
constexpr int WAR = BM / 16;            // dy rows per thread

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
  int q16, r16;     // WKC = q16*OW + r16
  unsigned x_bytes, dy_bytes;
};

constexpr int COL_INVALID = -(1 << 20);

template <typename T>
__global__ void __launch_bounds__(THREADS, 2)
wgrad_kernel(WgradParams p, const T* __restrict__ x, const T* __restrict__ dy,
             float* __restrict__ out /* dw when nsplit == 1, else partials */,
             float* __restrict__ db_out) {
  extern __shared__ float lds[];
  const int BNW = p.NBW * 16;
  const int bstride = BNW * WKP, astride = BM * WKP;
  float* Bs = lds;                                   // [2][BNW][WKP]
  float* As = lds + 2 * bstride;                     // [2][BM][WKP]
  const int esz = (int)sizeof(T);
  const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(x, p.x_bytes);
  const __amdgpu_buffer_rsrc_t yrsrc = make_rsrc(dy, p.dy_bytes);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int split = blockIdx.x;
  const int ntile = blockIdx.y % p.ntiles_n, mtile = blockIdx.y / p.ntiles_n;
  const int grp = blockIdx.z;
  const int col0 = ntile * BNW;

  const int base = p.NBW >> 1, rem = p.NBW & 1;
  const int nt = base + (wn < rem ? 1 : 0);
  const int nb0 = nt > 0 ? wn * base + min(wn, rem) : 0;

  const int pl = tid & 15, cl = tid >> 4;            // position lane, column/channel lane
  const int m_lim = p.Kg - mtile * BM;
  const int P_begin = split * p.pps, P_end = min(P_begin + p.pps, p.Ptotal);
  const int nchunks = (P_end - P_begin + WKC - 1) / WKC;
  const int ncl = p.NBW;                             // columns per thread: BNW / 16

  // this thread's columns: byte offset and window shift, fixed for the kernel
  int coff[WCL_MAX], cdh[WCL_MAX], cdw[WCL_MAX];
#pragma unroll
  for (int i = 0; i < WCL_MAX; ++i) {
    const int j = cl + 16 * i, col = col0 + j;
    coff[i] = 0; cdh[i] = COL_INVALID; cdw[i] = 0;
    if (i < ncl && col < p.ncols) {
      const int c = col / p.KHW, t = col - c * p.KHW;
      const int kh = t / p.KW, kw = t - kh * p.KW;
      coff[i] = (c * p.HW + kh * p.dly * p.W + kw * p.dlx) * esz;
      cdh[i] = kh * p.dly;
      cdw[i] = kw * p.dlx;
    }
  }

  // position of this thread in the chunk being loaded, advanced by WKC per chunk
  int ld_P = P_begin + pl, ld_n, ld_oh, ld_ow;
  {
    const int Pc = min(ld_P, p.Ptotal - 1);
    ld_n = Pc / p.OHW;
    const int q = Pc - ld_n * p.OHW;
    ld_oh = q / p.OW;
    ld_ow = q - ld_oh * p.OW;
  }

  // two register sets: chunk c+1 waits in one while chunk c+2 is being fetched
  float bregA[WCL_MAX], aregA[WAR], bregB[WCL_MAX], aregB[WAR];

  auto load_chunk = [&](float (&breg)[WCL_MAX], float (&areg)[WAR]) {
    const bool pv = ld_P < P_end;
    const int ihb = pv ? ld_oh * p.sy - p.py : 4 * COL_INVALID, iwb = ld_ow * p.sx - p.px;
    const int xbase = ((ld_n * p.C + grp * p.Cg) * p.HW + ihb * p.W + iwb) * esz;
#pragma unroll
    for (int i = 0; i < WCL_MAX; ++i) {
      if (i < ncl) {
        const int ih = ihb + cdh[i], iw = iwb + cdw[i];
        const bool ok = ((unsigned)ih < (unsigned)p.H) & ((unsigned)iw < (unsigned)p.W);
        breg[i] = buf_ld(xrsrc, ok ? xbase + coff[i] : -1, x);
      }
    }
    const int ybase = (ld_n * p.K + grp * p.Kg + mtile * BM + cl) * p.OHW + ld_oh * p.OW + ld_ow;
#pragma unroll
    for (int i = 0; i < WAR; ++i) {
      const bool ok = pv & (cl + 16 * i < m_lim);
      areg[i] = buf_ld(yrsrc, ok ? (ybase + 16 * i * p.OHW) * esz : -1, dy);
    }
    // advance to the same lane of the next chunk
    ld_P += WKC;
    ld_ow += p.r16;
    ld_oh += p.q16;
    if (ld_ow >= p.OW) {
      ld_ow -= p.OW;
      ++ld_oh;
    }
    while (ld_oh >= p.OH) {
      ld_oh -= p.OH;
      ++ld_n;
    }
  };

  auto store_chunk = [&](int buf, const float (&breg)[WCL_MAX], const float (&areg)[WAR]) {
    float* bs = Bs + buf * bstride;
    float* as = As + buf * astride;
#pragma unroll
    for (int i = 0; i < WCL_MAX; ++i)
      if (i < ncl) bs[(cl + 16 * i) * WKP + pl] = breg[i];
#pragma unroll
    for (int i = 0; i < WAR; ++i) as[(cl + 16 * i) * WKP + pl] = areg[i];
  };

  load_chunk(bregA, aregA);
  store_chunk(0, bregA, aregA);
  if (nchunks > 1) load_chunk(bregB, aregB);
  __syncthreads();

  const int fr = lane & 15, fk = lane >> 4;
  const bool do_db = p.want_db && ntile == 0 && tid < BM;
  float dbacc = 0.f;
  float* o = out + (p.nsplit > 1 ? (size_t)split * (p.E + p.K) : 0);

  auto run = [&](auto ntc) {
    constexpr int NT = decltype(ntc)::value;
    floatx4 acc[2][NT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](int c) {
      const float* as = As + (c & 1) * astride + (wm * 32 + fr) * WKP + fk;
      const float* bs = Bs + (c & 1) * bstride + (nb0 * 16 + fr) * WKP + fk;
      float a[WKC / 4][2], b[WKC / 4][NT];
#pragma unroll
      for (int ks = 0; ks < WKC / 4; ++ks) {
        a[ks][0] = as[ks * 4];
        a[ks][1] = as[16 * WKP + ks * 4];
#pragma unroll
        for (int j = 0; j < NT; ++j) b[ks][j] = bs[j * 16 * WKP + ks * 4];
      }
      __builtin_amdgcn_sched_barrier(0);   // keep the fragment reads ahead of the MFMAs
#pragma unroll
      for (int ks = 0; ks < WKC / 4; ++ks) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ks][0], b[ks][j], acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ks][1], b[ks][j], acc[1][j], 0, 0, 0);
        }
      }
      if (do_db) {
        const float* ar = As + (c & 1) * astride + tid * WKP;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < WKC; ++k) s += ar[k];
        dbacc += s;
      }
    };

    const int n = nchunks;
    for (int c = 0; c < n; c += 2) {
      if (c + 2 < n) load_chunk(bregA, aregA);
      compute(c);
      if (c + 1 < n) store_chunk(1, bregB, aregB);
      __syncthreads();
      if (c + 1 >= n) break;
      if (c + 3 < n) load_chunk(bregB, aregB);
      compute(c + 1);
      if (c + 2 < n) store_chunk(0, bregA, aregA);
      __syncthreads();
    }

    if (nt > 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
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
  };

  switch (nt) {
    case 0:
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 6: run(std::integral_constant<int, 6>{}); break;
    case 7: run(std::integral_constant<int, 7>{}); break;
    default: run(std::integral_constant<int, 8>{}); break;
  }

  if (do_db && tid < min(m_lim, BM)) {
    const int ch = grp * p.Kg + mtile * BM + tid;
    if (p.nsplit > 1)
      o[p.E + ch] = dbacc;
    else
      db_out[ch] = dbacc;
  }
}

// out[e] = sum over s of part[s][e]; elements past E go to db.  A block covers 64
// groups of four consecutive elements with 16 threads each; a thread adds every 16th
// partial, all of its 16-byte loads in flight together, and the 16 sums of a group
// are added in a fixed order (deterministic).  (E + K) % 4 == 0 is required.
constexpr int RED_TY = 16;
__global__ void __launch_bounds__(64 * RED_TY)
wgrad_reduce_kernel(const float* __restrict__ part, int nsplit, int E, int K, int want_db,
                    float* __restrict__ dw, float* __restrict__ db) {
  __shared__ float4 red[RED_TY][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int e = (blockIdx.x * 64 + tx) * 4;
  const int total = E + (want_db ? K : 0);
  const size_t stride = (size_t)E + K;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (e < total) {
    for (int s0 = ty; s0 < nsplit; s0 += 8 * RED_TY) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int s = s0 + u * RED_TY;
        v[u] = s < nsplit ? *reinterpret_cast<const float4*>(part + (size_t)s * stride + e)
                          : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w;
      }
    }
  }
  red[ty][tx] = acc;
  __syncthreads();
  if (ty == 0 && e < total) {
    float4 r = red[0][tx];
#pragma unroll
    for (int k = 1; k < RED_TY; ++k) {
      const float4 t = red[k][tx];
      r.x += t.x; r.y += t.y; r.z += t.z; r.w += t.w;
    }
    const float rv[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int ek = e + k;
      if (ek < E)
        dw[ek] = rv[k];
      else if (ek < total)
        db[ek - E] = rv[k];
    }
  }
}

// Few partial streams (at most 16) of a large gradient: a thread owns four elements and adds the splits in order, eight
// loads in flight at a time (the kernel above spreads the splits over 16 rows of threads: with 8 splits half of a
// workgroup idles and every thread has one load in flight - 512 x 2048 filters in 8 splits: 16.9 us).
__global__ void __launch_bounds__(256)
wgrad_reduce_few_kernel(const float* __restrict__ part, int nsplit, int E, int K, int want_db,
                        float* __restrict__ dw, float* __restrict__ db) {
  const int e = (blockIdx.x * 256 + threadIdx.x) * 4;
  const int total = E + (want_db ? K : 0);
  const size_t stride = (size_t)E + K;
  if (e >= total) return;
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < nsplit; s0 += 8) {
    float4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = s0 + u < nsplit ? *reinterpret_cast<const float4*>(part + (size_t)(s0 + u) * stride + e)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      r.x += v[u].x; r.y += v[u].y; r.z += v[u].z; r.w += v[u].w;
    }
  }
  const float rv[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int ek = e + k;
    if (ek < E)
      dw[ek] = rv[k];
    else if (ek < total)
      db[ek - E] = rv[k];
  }
}

// element-wise variant for sizes that are not multiples of four
__global__ void __launch_bounds__(256)
wgrad_reduce_kernel1(const float* __restrict__ part, int nsplit, int E, int K, int want_db,
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
  p->q16 = WKC / g.OW;
  p->r16 = WKC % g.OW;
  return true;
}

// Byte offsets are 32-bit and padding columns rely on |shift| < 2^20.
template <typename T>
bool wgrad_fits(const ConvGeom& g, WgradParams* p) {
  const long long xb = (long long)g.N * g.C * g.H * g.W * (long long)sizeof(T);
  const long long yb = (long long)g.N * g.K * g.OH * g.OW * (long long)sizeof(T);
  if (xb >= (1ll << 31) || yb >= (1ll << 31) || g.OH * g.sy >= (1 << 19) ||
      (g.KH - 1) * g.dly >= (1 << 19))
    return false;
  p->x_bytes = (unsigned)xb;
  p->dy_bytes = (unsigned)yb;
  return true;
}

bool wgrad_split(WgradParams* p, const ConvGeom& g) {
  const long long base_wgs = (long long)p->ntiles_n * p->mtiles * g.groups;
  if (p->ntiles_n * p->mtiles > 65535 || g.groups > 65535) return false;
  long long ns = 2 * mfma_num_cus() / base_wgs;
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

void wgrad_reduce_launch(const float* part, int nsplit, int E, int K, int want_db, float* dw,
                         float* db, hipStream_t s) {
  const int total = E + (want_db ? K : 0);
  if ((E + K) % 4 == 0 && reinterpret_cast<uintptr_t>(part) % 16 == 0 && nsplit <= 16 && total >= (1 << 18))
    hipLaunchKernelGGL(wgrad_reduce_few_kernel, dim3((total + 1023) / 1024), dim3(256), 0, s, part, nsplit, E, K, want_db, dw, db);
  else if ((E + K) % 4 == 0 && reinterpret_cast<uintptr_t>(part) % 16 == 0)
    hipLaunchKernelGGL(wgrad_reduce_kernel, dim3((total + 255) / 256), dim3(64 * RED_TY), 0, s, part,
                       nsplit, E, K, want_db, dw, db);
  else
    hipLaunchKernelGGL(wgrad_reduce_kernel1, dim3((total + 63) / 64), dim3(256), 0, s, part, nsplit,
                       E, K, want_db, dw, db);
}

size_t mfma_conv_bwd_filter_ws(const ConvGeom& g, int) {
  WgradParams p{};
  if (!wgrad_plan(g, &p) || !wgrad_split(&p, g)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
}

int mfma_conv_bwd_filter(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                         float* db, void* ws, size_t ws_bytes, hipStream_t s) {
  if (!dw) return -1;   // bias gradient alone: the plain reduction kernel
  WgradParams p{};
  if (!wgrad_plan(g, &p) || !wgrad_split(&p, g)) return -1;
  if (!by_dtype(dtype, [&](auto* t_) { return wgrad_fits<FLHIP_T_OF(t_)>(g, &p); })) return -1;
  p.want_db = db != nullptr;
  if (p.nsplit > 1 && (!ws || ws_bytes < (size_t)p.nsplit * (p.E + p.K) * sizeof(float)))
    return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  const int BNW = p.NBW * 16;
  const size_t shmem = (size_t)2 * (BNW * WKP + BM * WKP) * sizeof(float);
  const dim3 grid(p.nsplit, p.ntiles_n * p.mtiles, g.groups);
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  const int rc_ = by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    auto kernel = wgrad_kernel<T>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const T*>(x),
                       static_cast<const T*>(dy), out, db);
    return 0;
  });
  if (rc_) return rc_;
  if (p.nsplit > 1)
    wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.K, p.want_db, dw, db, s);
  return check_launch("conv2d_bwd_filter (mfma)");
}

}  // namespace flhip
