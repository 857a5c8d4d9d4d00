// Filter (and bias) gradient for 3x3 stride-1 convolutions with the operands
// resident in LDS.
//
// dw[m, (c,tap)] = sum over positions of dy[m, pos] * x[c, pos + shift(tap)].
// A workgroup owns 64 output channels x 32 input channels (288 columns) over a
// range of (image, output row) pairs; per output row it stages that row of dy
// ([64][OW]) and the three input rows the window touches ([32][3][WS], image
// column w at staged column w + XOFF, zero halo) in LDS once, and every tap reads
// the same rows at a shifted address - nothing is gathered per tap.  8 waves, two
// roles (wave w and w+4 share a SIMD): waves 0-3 stage row r+1 (16-byte loads and
// LDS stores when the rows allow it) while waves 4-7 (2 along m x 2 along the
// columns, 32 x 144 each) run v_mfma_f32_16x16x4_f32 over row r.  A lane's two
// k-steps of a group of 8 positions are the adjacent positions 2*fk and 2*fk+1, so
// one 8-byte LDS read feeds both.  One barrier per row.  The finished 64 x 288
// tile is parked in LDS and written with 16-byte stores; partial tiles go to the
// workspace and are added in a fixed order by wgrad_reduce_kernel
// (deterministic).  The bias gradient is summed from the dy values on their way
// through the loader registers.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int BM = MFMA_BM;
constexpr int CB = 32;           // input channels per workgroup
constexpr int GTHREADS = 256;
constexpr int THREADS = 512;
constexpr int NTW = 9;           // 16-column blocks per MFMA wave (CB*9/16/2)
constexpr int NXE = 8;           // element-wise loader: x elements per thread and window row
constexpr int NDE = 16;          // element-wise loader: dy elements per thread and row
constexpr int NXV = 2;           // 16-byte loader: x units per thread and window row
constexpr int NDV = 4;           // 16-byte loader: dy units per thread and row
constexpr int SPW = CB * 9 + 4;  // pitch of the parked result tile (words)

struct WSlabParams {
  int N, C, H, W, K, OH, OW;
  int py, px, dly, dlx;
  int groups, Cg, Kg;
  int WS, XOFF;        // staged row pitch, staged column of image column 0
  int CP, DP;          // LDS pitches: per input channel (3 rows), per dy row
  int vec;             // 16-byte loaders apply
  int stage_ok;        // the result tile (and the bias partials) fit in LDS
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
  // readfirstlane: the division runs on the vector ALU, the results are uniform
  const int half = __builtin_amdgcn_readfirstlane(blockIdx.y % p.nhalves);
  const int mtile = __builtin_amdgcn_readfirstlane(blockIdx.y / p.nhalves);
  const int grp = blockIdx.z;
  const int m_lim = p.Kg - mtile * BM;
  const int row_begin = split * p.rps, row_end = min(row_begin + p.rps, p.total_rows);
  const int nrows = row_end - row_begin;
  const int HW = p.H * p.W, OHW = p.OH * p.OW;
  float* o = out + (p.nsplit > 1 ? (size_t)split * (p.E + p.K) : 0);
  const int ncols = p.Cg * 9;
  float* stage = lds;                       // [BM][SPW], after the last row
  float* dbpart = lds + (p.stage_ok ? BM * SPW : 0);   // [BM][OW/4] bias partials (16-byte loader)

  // The halo columns of the staged rows are never written: zero the buffers once.
  for (int i = tid; i < (2 * (p.xs_words + p.ds_words)) >> 2; i += THREADS)
    reinterpret_cast<float4*>(lds)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();

  // 16-byte stores of the parked tile, all 512 threads
  auto store_tile = [&]() {
    constexpr int Q = CB * 9 / 4;
    for (int idx = tid; idx < BM * Q; idx += THREADS) {
      const int m = idx / Q, q = idx - m * Q;
      if (m < m_lim) {
        const float4 v = *reinterpret_cast<const float4*>(stage + m * SPW + 4 * q);
        *reinterpret_cast<float4*>(o + (size_t)(grp * p.Kg + mtile * BM + m) * ncols +
                                   half * CB * 9 + 4 * q) = v;
      }
    }
  };

  if (wave < 4) {
    // ============================== loader waves ================================
    const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t yrsrc = make_rsrc(dy, p.dy_bytes);
    const bool do_db = p.want_db && half == 0;
    const int db_ch = grp * p.Kg + mtile * BM + tid;     // for tid < BM
    auto write_db = [&](float v) {
      if (p.nsplit > 1)
        o[p.E + db_ch] = v;
      else
        db_out[db_ch] = v;
    };

    if (p.vec) {
      // ---- 16-byte loaders -------------------------------------------------------
      // x units per window row: (channel, group of 4 image columns); dy units:
      // (output channel, group of 4 columns)
      const int qx = p.W >> 2, qy = p.OW >> 2;
      int xg[NXV], xl[NXV], yg[NDV], yl[NDV];
#pragma unroll
      for (int i = 0; i < NXV; ++i) {
        const int u = tid + GTHREADS * i;
        xg[i] = OOB;
        xl[i] = CB * p.CP;                    // spare words past the tile (kh*WS is added)
        if (u < CB * qx) {
          const int c = u / qx, q = u - c * qx;
          xl[i] = c * p.CP + p.XOFF + 4 * q;
          xg[i] = ((grp * p.Cg + half * CB + c) * HW + 4 * q) * esz;
        }
      }
#pragma unroll
      for (int i = 0; i < NDV; ++i) {
        const int u = tid + GTHREADS * i;
        yg[i] = OOB;
        yl[i] = p.ds_words - 8;
        if (u < BM * qy) {
          const int m = u / qy, q = u - m * qy;
          yl[i] = m * p.DP + 4 * q;
          if (m < m_lim) yg[i] = ((grp * p.Kg + mtile * BM + m) * OHW + 4 * q) * esz;
        }
      }
      // two register sets: row r+2 is in flight while row r+1 is written to LDS
      float4 xvA[3][NXV], yvA[NDV], xvB[3][NXV], yvB[NDV];
      float dbp[NDV];
#pragma unroll
      for (int i = 0; i < NDV; ++i) dbp[i] = 0.f;
      auto load_row = [&](int row, float4 (&xv)[3][NXV], float4 (&yv)[NDV]) {
        const int img = row / p.OH, oh = row - img * p.OH;
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
          const int ih = oh - p.py + kh * p.dly;
          const int rb = (img * p.C * HW + ih * p.W) * esz;
          if ((unsigned)ih < (unsigned)p.H) {           // uniform: the whole window row exists
#pragma unroll
            for (int i = 0; i < NXV; ++i) xv[kh][i] = buf_ld4(xrsrc, xg[i] + rb, x);
          } else {
#pragma unroll
            for (int i = 0; i < NXV; ++i) xv[kh][i] = make_float4(0.f, 0.f, 0.f, 0.f);
          }
        }
        const int yb = (img * p.K * OHW + oh * p.OW) * esz;
#pragma unroll
        for (int i = 0; i < NDV; ++i) yv[i] = buf_ld4(yrsrc, yg[i] + yb, dy);
      };
      auto store_row = [&](int buf, const float4 (&xv)[3][NXV], const float4 (&yv)[NDV]) {
        float* xs = Xs + buf * p.xs_words;
        float* ds = Ds + buf * p.ds_words;
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
          for (int i = 0; i < NXV; ++i)
            *reinterpret_cast<float4*>(xs + xl[i] + kh * p.WS) = xv[kh][i];
#pragma unroll
        for (int i = 0; i < NDV; ++i) {
          *reinterpret_cast<float4*>(ds + yl[i]) = yv[i];
          dbp[i] += (yv[i].x + yv[i].y) + (yv[i].z + yv[i].w);
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
        __syncthreads();
        if (r + 1 >= nrows) break;
        if (r + 3 < nrows) load_row(row_begin + r + 3, xvB, yvB);
        if (r + 2 < nrows) store_row(0, xvA, yvA);
        __syncthreads();
      }
      // bias: the partials of a channel sit in qy consecutive units; they go
      // through LDS behind the parked tile (or, when nothing is parked, at its start:
      // the MFMA waves are done with LDS after the last row)
      if (do_db) {
#pragma unroll
        for (int i = 0; i < NDV; ++i) {
          const int u = tid + GTHREADS * i;
          if (u < BM * qy) dbpart[u] = dbp[i];
        }
      }
      __syncthreads();                      // tile parked, partials written
      if (do_db && tid < min(m_lim, BM)) {
        float s = 0.f;
        for (int q = 0; q < qy; ++q) s += dbpart[tid * qy + q];
        write_db(s);
      }
      if (p.stage_ok) store_tile();
      return;
    }

    // ---- element-wise loaders ------------------------------------------------------
    int xg[NXE], xl[NXE];
#pragma unroll
    for (int i = 0; i < NXE; ++i) {
      const int e = tid + GTHREADS * i;
      xg[i] = OOB;
      xl[i] = CB * p.CP;
      if (e < CB * p.W) {
        const int c = e / p.W, iw = e - c * p.W;
        xl[i] = c * p.CP + p.XOFF + iw;
        xg[i] = ((grp * p.Cg + half * CB + c) * HW + iw) * esz;
      }
    }
    int yg[NDE], yl[NDE];
#pragma unroll
    for (int i = 0; i < NDE; ++i) {
      const int e = tid + GTHREADS * i;
      yg[i] = OOB;
      yl[i] = p.ds_words - 8;
      if (e < BM * p.OW) {
        const int m = e / p.OW, ow = e - m * p.OW;
        yl[i] = m * p.DP + ow;
        if (m < m_lim) yg[i] = ((grp * p.Kg + mtile * BM + m) * OHW + ow) * esz;
      }
    }
    float xvA[3][NXE], yvA[NDE], xvB[3][NXE], yvB[NDE];
    auto load_row = [&](int row, float (&xv)[3][NXE], float (&yv)[NDE]) {
      const int img = row / p.OH, oh = row - img * p.OH;
#pragma unroll
      for (int kh = 0; kh < 3; ++kh) {
        const int ih = oh - p.py + kh * p.dly;
        const int rb = (img * p.C * HW + ih * p.W) * esz;
        if ((unsigned)ih < (unsigned)p.H) {
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
    // bias: thread m < 64 adds up its dy row while it sits in LDS
    const bool sum_rows = do_db && tid < BM;
    float dbacc = 0.f;
    auto sum_db = [&](int r) {
      if (sum_rows) {
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
    if (sum_rows && tid < min(m_lim, BM)) write_db(dbacc);
    __syncthreads();                        // tile parked
    if (p.stage_ok) store_tile();
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

  const int ksteps = p.OW >> 2;
  const int ngroups = ksteps >> 1;          // groups of 8 positions, 2 per lane
  // this lane's column in block j: local column -> (channel, kh, kw) -> LDS address
  lds_f1 bp[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    const int col = (wn * NTW + j) * 16 + fr;
    const int c = col / 9, t = col - c * 9;
    const int kh = t / 3, kw = t - kh * 3;
    bp[j] = (lds_f1)Xs + (c * p.CP + kh * p.WS + kw * p.dlx + p.XOFF - p.px + 2 * fk);
  }
  lds_f1 ap0 = (lds_f1)Ds + ((wm * 32 + fr) * p.DP + 2 * fk);
  lds_f1 ap1 = ap0 + 16 * p.DP;

  // Fragments of a group of 8 positions: .x and .y are the two k-steps.
  struct Frag {
    float2 a[2];
    float2 b[NTW];
  };
  auto read_frags = [&](Frag& f, int off) {
    f.a[0] = make_float2(ap0[off], ap0[off + 1]);
    f.a[1] = make_float2(ap1[off], ap1[off + 1]);
#pragma unroll
    for (int j = 0; j < NTW; ++j) f.b[j] = make_float2(bp[j][off], bp[j][off + 1]);
  };
  auto mma = [&](const Frag& f) {
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
      acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[0].x, f.b[j].x, acc[0][j], 0, 0, 0);
      acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[1].x, f.b[j].x, acc[1][j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
      acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[0].y, f.b[j].y, acc[0][j], 0, 0, 0);
      acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.a[1].y, f.b[j].y, acc[1][j], 0, 0, 0);
    }
  };
  auto advance = [&](int words_x, int words_d) {
#pragma unroll
    for (int j = 0; j < NTW; ++j) bp[j] += words_x;
    ap0 += words_d;
    ap1 += words_d;
  };

  __syncthreads();
  for (int r = 0; r < nrows; ++r) {
    int walked = 0;
    if (ngroups > 0) {
      // Fragments of the next group are read while this group's MFMAs run, one LDS
      // read slotted behind each of the first MFMAs.  The read past the last group
      // stays inside the LDS tile and is not used.
      Frag f0, f1;
      read_frags(f0, 0);
#define FLHIP_GROUP(CUR, NXT, OFF)                                    \
  __builtin_amdgcn_sched_barrier(0);                                  \
  read_frags(NXT, OFF);                                               \
  mma(CUR);                                                           \
  _Pragma("unroll") for (int q = 0; q < 2 * NTW + 4; ++q) {           \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
  }                                                                   \
  __builtin_amdgcn_sched_group_barrier(0x008, 2 * NTW - 4, 0);        \
  __builtin_amdgcn_sched_barrier(0);
      int g = 0;
      for (; g + 2 <= ngroups; g += 2) {
        FLHIP_GROUP(f0, f1, 8)
        FLHIP_GROUP(f1, f0, 16)
        advance(16, 16);
        walked += 16;
      }
#undef FLHIP_GROUP
      if (g < ngroups) mma(f0);
    }
    if (ksteps & 1) {
      // last four positions of a row whose length is not a multiple of 8: one
      // k-step, lane fk takes position 8*ngroups + fk
      const int off = 8 * ngroups - walked - fk;
      const float a0 = ap0[off];
      const float a1 = ap1[off];
#pragma unroll
      for (int j = 0; j < NTW; ++j) {
        const float b = bp[j][off];
        acc[0][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b, acc[0][j], 0, 0, 0);
        acc[1][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b, acc[1][j], 0, 0, 0);
      }
    }
    // back to the row start, in the other buffer
    const int sign = (r & 1) ? -1 : 1;
    advance(sign * p.xs_words - walked, sign * p.ds_words - walked);
    __syncthreads();
  }

  if (p.stage_ok) {
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
      const int col = (wn * NTW + j) * 16 + fr;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
          stage[(wm * 32 + i * 16 + fk * 4 + rr) * SPW + col] = acc[i][j][rr];
    }
    __syncthreads();
    store_tile();
    return;
  }
  __syncthreads();                          // the loader waves' last barrier
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

// smallest value >= v that is congruent to r modulo m
inline int round_to_residue(int v, int r, int m) { return v + ((r - v) % m + m) % m; }

bool plan(const ConvGeom& g, WSlabParams* p, bool aligned) {
  if (g.KH != 3 || g.KW != 3 || g.sy != 1 || g.sx != 1) return false;
  if (g.Cg % CB != 0 || g.OW % 4 != 0) return false;
  p->N = g.N; p->C = g.C; p->H = g.H; p->W = g.W; p->K = g.K; p->OH = g.OH; p->OW = g.OW;
  p->py = g.py; p->px = g.px; p->dly = g.dly; p->dlx = g.dlx;
  p->groups = g.groups; p->Cg = g.Cg; p->Kg = g.Kg;
  p->vec = aligned && g.W % 4 == 0;
  if (p->vec ? (CB * (g.W / 4) > GTHREADS * NXV || BM * (g.OW / 4) > GTHREADS * NDV)
             : (CB * g.W > GTHREADS * NXE || BM * g.OW > GTHREADS * NDE))
    return false;
  p->XOFF = (g.px + 3) & ~3;
  // staged columns: the image, and whatever the rightmost tap of the last position
  // (plus the unused read-ahead of 8 positions) touches
  const int need = p->XOFF + std::max(g.W, g.OW - g.px + 2 * g.dlx);
  const int ws_min = (need + 3) & ~3;
  // dy pitch: a multiple of 4 with DP/4 odd puts the 16 rows x 4 k-indices of a
  // fragment read on distinct banks
  p->DP = round_to_residue(g.OW + 4, 4, 8);
  p->ds_words = BM * p->DP + 24;
  // row pitch = 8 (mod 32): the three window rows of a channel land 8 banks apart;
  // fall back to the smallest pitch when LDS is short
  const size_t lds_cap = 150 * 1024;
  for (int attempt = 0; attempt < 2; ++attempt) {
    p->WS = attempt == 0 ? round_to_residue(ws_min, 8, 32) : ws_min;
    p->CP = 3 * p->WS;
    p->xs_words = CB * p->CP + 2 * p->WS + 24;   // + spare words for idle loader slots / read-ahead
    if ((size_t)2 * (p->xs_words + p->ds_words) * sizeof(float) <= lds_cap) break;
    if (attempt == 1) return false;
  }
  p->stage_ok = (size_t)(BM * SPW + BM * (g.OW / 4)) <= (size_t)2 * (p->xs_words + p->ds_words);
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

}  // namespace

// defined in conv2d_mfma_wgrad.hip
void wgrad_reduce_launch(const float* part, int nsplit, int E, int K, int want_db, float* dw,
                         float* db, hipStream_t s);

size_t mfma_slab_wgrad_ws(const ConvGeom& g, int) {
  WSlabParams p{};
  if (!plan(g, &p, false)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
}

bool mfma_slab_wgrad_applies(const ConvGeom& g) {
  WSlabParams p{};
  return plan(g, &p, false);
}

int mfma_slab_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                    float* db, void* ws, size_t ws_bytes, hipStream_t s) {
  if (!dw) return -1;
  WSlabParams p{};
  const size_t esz = dtype == FLHIP_F32 ? 4 : 2;
  const bool aligned = reinterpret_cast<uintptr_t>(x) % (4 * esz) == 0 &&
                       reinterpret_cast<uintptr_t>(dy) % (4 * esz) == 0;
  if (!plan(g, &p, aligned)) return -1;
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
  if (reinterpret_cast<uintptr_t>(out) % 16 != 0) p.stage_ok = 0;
  const int rc_ = by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    auto kernel = wgrad_slab_kernel<T>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const T*>(x),
                       static_cast<const T*>(dy), out, db);
    return 0;
  });
  if (rc_) return rc_;
  if (p.nsplit > 1)
    wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.K, p.want_db, dw, db, s);
  return check_launch("conv2d_bwd_filter (mfma slab)");
}

}  // namespace flhip
