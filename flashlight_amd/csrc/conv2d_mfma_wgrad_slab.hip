// Filter (and bias) gradient for 3x3 stride-1 convolutions with the operands
// resident in LDS.
//
// dw[m, (c,tap)] = sum over positions of dy[m, pos] * x[c, pos + shift(tap)].
// A workgroup owns 64 output channels x 32 input channels (288 columns) over a
// range of (image, output row) pairs; per output row it stages that row of dy
// ([64][W]) and the three input rows the window touches ([32][3][W+2*dil], zero
// where outside the image) in LDS once, and every tap reads the same rows at a
// shifted address - nothing is gathered per tap.  8 waves, two roles (wave w and
// w+4 share a SIMD): waves 0-3 stage row r+1 while waves 4-7 (2 along m x 2
// along the columns, 32 x 144 each) run v_mfma_f32_16x16x4_f32 over row r, four
// positions per instruction.  One barrier per row.  Partial tiles go to the
// workspace and are added in a fixed order by wgrad_reduce_kernel
// (deterministic); the bias gradient is summed from the dy rows in LDS.
#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int BM = MFMA_BM;
constexpr int CB = 32;           // input channels per workgroup
constexpr int GTHREADS = 256;
constexpr int THREADS = 512;
constexpr int NTW = 9;           // 16-column blocks per MFMA wave (CB*9/16/2)
constexpr int NXE = 8;           // x elements per loader thread and window row
constexpr int NDE = 16;          // dy elements per loader thread and row

struct WSlabParams {
  int N, C, H, W, K, OH, OW;
  int py, px, dly, dlx;
  int groups, Cg, Kg;
  int WS;              // staged row width: OW + 2*dlx
  int CP, DP;          // LDS pitches: per input channel (3 rows), per dy row
  int nhalves, mtiles;
  int nsplit, rps;     // K-splits, (image,row) pairs per split
  int total_rows;
  int E;               // K*Cg*9
  int want_db;
  int xs_words, ds_words;
  unsigned x_bytes, dy_bytes;
};

template <typename T>
__global__ void __launch_bounds__(THREADS, 2)
wgrad_slab_kernel(WSlabParams p, const T* __restrict__ x, const T* __restrict__ dy,
                  float* __restrict__ out, float* __restrict__ db_out) {
  extern __shared__ float lds[];
  float* Xs = lds;                          // [2][CB][3][WS] with channel pitch CP
  float* Ds = lds + 2 * p.xs_words;         // [2][BM][DP]
  constexpr int OOB = (int)0x80000000;
  const int esz = (int)sizeof(T);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x;
  const int half = blockIdx.y % p.nhalves, mtile = blockIdx.y / p.nhalves;
  const int grp = blockIdx.z;
  const int m_lim = p.Kg - mtile * BM;
  const int row_begin = split * p.rps, row_end = min(row_begin + p.rps, p.total_rows);
  const int nrows = row_end - row_begin;
  const int HW = p.H * p.W, OHW = p.OH * p.OW;

  if (wave < 4) {
    // ============================== loader waves ================================
    const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t yrsrc = make_rsrc(dy, p.dy_bytes);
    // x: per window row kh, elements e = tid + 256*i over (channel, staged column)
    const int nxe = (CB * p.WS + GTHREADS - 1) / GTHREADS;
    int xg[NXE], xl[NXE];
#pragma unroll
    for (int i = 0; i < NXE; ++i) {
      const int e = tid + GTHREADS * i;
      xg[i] = OOB;
      xl[i] = CB * p.CP;                      // spare words past the tile (kh*WS is added)
      if (i < nxe && e < CB * p.WS) {
        const int c = e / p.WS, ws = e - c * p.WS;
        const int iw = ws - p.px;
        xl[i] = c * p.CP + ws;
        if ((unsigned)iw < (unsigned)p.W) xg[i] = ((grp * p.Cg + half * CB + c) * HW + iw) * esz;
      }
    }
    // dy: elements over (output channel m, column)
    const int nde = (BM * p.OW + GTHREADS - 1) / GTHREADS;
    int yg[NDE], yl[NDE];
#pragma unroll
    for (int i = 0; i < NDE; ++i) {
      const int e = tid + GTHREADS * i;
      yg[i] = OOB;
      yl[i] = p.ds_words - 1;
      if (i < nde && e < BM * p.OW) {
        const int m = e / p.OW, ow = e - m * p.OW;
        yl[i] = m * p.DP + ow;
        if (m < m_lim) yg[i] = ((grp * p.Kg + mtile * BM + m) * OHW + ow) * esz;
      }
    }
    // two register sets: row r+2 is in flight while row r+1 is written to LDS
    float xvA[3][NXE], yvA[NDE], xvB[3][NXE], yvB[NDE];
    auto load_row = [&](int row, float (&xv)[3][NXE], float (&yv)[NDE]) {
      const int img = row / p.OH, oh = row - img * p.OH;
#pragma unroll
      for (int kh = 0; kh < 3; ++kh) {
        const int ih = oh - p.py + kh * p.dly;
        const int rb = (img * p.C * HW + ih * p.W) * esz;
        if ((unsigned)ih < (unsigned)p.H) {           // uniform: the whole window row exists
#pragma unroll
          for (int i = 0; i < NXE; ++i) xv[kh][i] = buf_ld(xrsrc, xg[i] + rb, x);
        } else {
#pragma unroll
          for (int i = 0; i < NXE; ++i) xv[kh][i] = 0.f;
        }
      }
      const int yb = (img * p.K * OHW + oh * p.OW) * esz;
#pragma unroll
      for (int i = 0; i < NDE; ++i) yv[i] = buf_ld(yrsrc, yg[i] + yb, dy);
    };
    auto store_row = [&](int buf, const float (&xv)[3][NXE], const float (&yv)[NDE]) {
      float* xs = Xs + buf * p.xs_words;
      float* ds = Ds + buf * p.ds_words;
#pragma unroll
      for (int kh = 0; kh < 3; ++kh)
#pragma unroll
        for (int i = 0; i < NXE; ++i) xs[xl[i] + kh * p.WS] = xv[kh][i];
#pragma unroll
      for (int i = 0; i < NDE; ++i) ds[yl[i]] = yv[i];
    };

    const bool do_db = p.want_db && half == 0 && tid < BM;
    float dbacc = 0.f;
    auto sum_db = [&](int r) {
      if (do_db) {
        const float* drow = Ds + (r & 1) * p.ds_words + tid * p.DP;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        for (int w = 0; w < p.OW; w += 4) {      // OW % 4 == 0
          s0 += drow[w]; s1 += drow[w + 1]; s2 += drow[w + 2]; s3 += drow[w + 3];
        }
        dbacc += (s0 + s1) + (s2 + s3);
      }
    };
    if (nrows > 0) {
      load_row(row_begin, xvA, yvA);
      store_row(0, xvA, yvA);
    }
    if (nrows > 1) load_row(row_begin + 1, xvB, yvB);
    __syncthreads();
    for (int r = 0; r < nrows; r += 2) {
      // even row r: row r+1 waits in set B, row r+2 goes to set A
      if (r + 2 < nrows) load_row(row_begin + r + 2, xvA, yvA);
      if (r + 1 < nrows) store_row(1, xvB, yvB);
      sum_db(r);
      __syncthreads();
      if (r + 1 >= nrows) break;
      if (r + 3 < nrows) load_row(row_begin + r + 3, xvB, yvB);
      if (r + 2 < nrows) store_row(0, xvA, yvA);
      sum_db(r + 1);
      __syncthreads();
    }
    if (do_db && tid < m_lim) {
      const int ch = grp * p.Kg + mtile * BM + tid;
      if (p.nsplit > 1)
        out[(size_t)split * (p.E + p.K) + p.E + ch] = dbacc;
      else
        db_out[ch] = dbacc;
    }
    return;
  }

  // ================================ MFMA waves ===================================
  const int cw = wave - 4;
  const int wm = cw & 1, wn = cw >> 1;
  const int fr = lane & 15, fk = lane >> 4;
  floatx4 acc[2][NTW];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NTW; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this lane's column in block j: local column -> (channel, kh, kw) -> LDS offset
  int colbase[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int col = (wn * NTW + j) * 16 + fr;
    const int c = col / 9, t = col - c * 9;
    const int kh = t / 3, kw = t - kh * 3;
    colbase[j] = c * p.CP + kh * p.WS + kw * p.dlx + fk;
  }
  const int abase = (wm * 32 + fr) * p.DP + fk;
  const int ksteps = p.OW / 4;

  // Fragments of two k-steps (8 positions): 2x2 dy values and 2xNTW x values.
  struct Frag {
    float a[2][2];
    float b[2][NTW];
  };
  const float* ds_row;
  const float* bp[NTW];
  auto read_frags = [&](Frag& f, int ks) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      f.a[u][0] = ds_row[(ks + u) * 4];
      f.a[u][1] = ds_row[16 * p.DP + (ks + u) * 4];
#pragma unroll
      for (int j = 0; j < NTW; ++j) f.b[u][j] = bp[j][(ks + u) * 4];
    }
  };
  auto mma = [&](const Frag& f) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < NTW; ++j) {
        acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[u][0], f.b[u][j], acc[0][j], 0, 0, 0);
        acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[u][1], f.b[u][j], acc[1][j], 0, 0, 0);
      }
  };

  __syncthreads();
  for (int r = 0; r < nrows; ++r) {
    const float* xs = Xs + (r & 1) * p.xs_words;
    ds_row = Ds + (r & 1) * p.ds_words + abase;
#pragma unroll
    for (int j = 0; j < NTW; ++j) bp[j] = xs + colbase[j];
    if ((ksteps & 1) == 0) {
      // pairs of k-steps, fragments of the next pair read while this pair's MFMAs
      // run.  The read past the last pair stays inside the LDS tile and is unused.
      Frag f0, f1;
      read_frags(f0, 0);
      int ks = 0;
      for (; ks + 4 <= ksteps; ks += 4) {
        read_frags(f1, ks + 2);
        __builtin_amdgcn_sched_barrier(0);
        mma(f0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(f0, ks + 4);
        __builtin_amdgcn_sched_barrier(0);
        mma(f1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (ks < ksteps) mma(f0);      // ksteps == 2 (mod 4)
    } else {
      for (int ks = 0; ks < ksteps; ++ks) {
        const float a0 = ds_row[ks * 4];
        const float a1 = ds_row[16 * p.DP + ks * 4];
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
          const float b = bp[j][ks * 4];
          acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b, acc[0][j], 0, 0, 0);
          acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b, acc[1][j], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  float* o = out + (p.nsplit > 1 ? (size_t)split * (p.E + p.K) : 0);
  const int ncols = p.Cg * 9;
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int col = half * CB * 9 + (wn * NTW + j) * 16 + fr;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int m = wm * 32 + i * 16 + fk * 4 + rr;
        if (m < m_lim) o[(size_t)(grp * p.Kg + mtile * BM + m) * ncols + col] = acc[i][j][rr];
      }
  }
}

bool plan(const ConvGeom& g, WSlabParams* p) {
  if (g.KH != 3 || g.KW != 3 || g.sy != 1 || g.sx != 1) return false;
  if (g.Cg % CB != 0 || g.OW % 4 != 0) return false;
  p->N = g.N; p->C = g.C; p->H = g.H; p->W = g.W; p->K = g.K; p->OH = g.OH; p->OW = g.OW;
  p->py = g.py; p->px = g.px; p->dly = g.dly; p->dlx = g.dlx;
  p->groups = g.groups; p->Cg = g.Cg; p->Kg = g.Kg;
  p->WS = g.OW + 2 * g.dlx;
  if ((CB * p->WS + GTHREADS - 1) / GTHREADS > NXE) return false;
  if ((BM * g.OW + GTHREADS - 1) / GTHREADS > NDE) return false;
  p->CP = 3 * p->WS + 1;
  if (p->CP % 2 == 0) ++p->CP;                     // odd channel pitch spreads the banks
  p->DP = g.OW + ((2 - g.OW % 32) + 32) % 32;      // == 2 mod 32: dy fragments conflict-free
  p->xs_words = CB * p->CP + 2 * p->WS + 8;   // + spare words for unused loader slots
  p->ds_words = BM * p->DP + 16;
  p->nhalves = g.Cg / CB;
  p->mtiles = (g.Kg + BM - 1) / BM;
  p->total_rows = g.N * g.OH;
  p->E = g.K * g.Cg * 9;
  const long long base_wgs = (long long)p->nhalves * p->mtiles * g.groups;
  if (p->nhalves * p->mtiles > 65535 || g.groups > 65535) return false;
  long long ns = mfma_num_cus() / base_wgs;
  if (ns > p->total_rows) ns = p->total_rows;
  if (ns < 1) ns = 1;
  p->rps = (int)((p->total_rows + ns - 1) / ns);
  p->nsplit = (p->total_rows + p->rps - 1) / p->rps;
  return true;
}

// defined in conv2d_mfma_wgrad.hip
}  // namespace

void wgrad_reduce_launch(const float* part, int nsplit, int E, int K, int want_db, float* dw,
                         float* db, hipStream_t s);

size_t mfma_slab_wgrad_ws(const ConvGeom& g, int) {
  WSlabParams p{};
  if (!plan(g, &p)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
}

bool mfma_slab_wgrad_applies(const ConvGeom& g) {
  WSlabParams p{};
  return plan(g, &p);
}

int mfma_slab_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                    float* db, void* ws, size_t ws_bytes, hipStream_t s) {
  if (!dw) return -1;
  WSlabParams p{};
  if (!plan(g, &p)) return -1;
  const size_t esz = dtype == FLHIP_F32 ? 4 : 2;
  const long long xb = (long long)g.N * g.C * g.H * g.W * (long long)esz;
  const long long yb = (long long)g.N * g.K * g.OH * g.OW * (long long)esz;
  if (xb >= (1ll << 31) || yb >= (1ll << 31)) return -1;
  p.x_bytes = (unsigned)xb;
  p.dy_bytes = (unsigned)yb;
  p.want_db = db != nullptr;
  const size_t need = p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
  if (need && (!ws || ws_bytes < need))
    return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  const size_t shmem = (size_t)2 * (p.xs_words + p.ds_words) * sizeof(float);
  const dim3 grid(p.nsplit, p.nhalves * p.mtiles, g.groups);
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  if (dtype == FLHIP_F32) {
    auto kernel = wgrad_slab_kernel<float>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const float*>(x),
                       static_cast<const float*>(dy), out, db);
  } else {
    auto kernel = wgrad_slab_kernel<bf16_t>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(dy), out, db);
  }
  if (p.nsplit > 1)
    wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.K, p.want_db, dw, db, s);
  return check_launch("conv2d_bwd_filter (mfma slab)");
}

}  // namespace flhip
