// Filter (and bias) gradient for 3x3 stride-1 pad-1 convolutions in bf16 storage on
// the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate and fp32 result).
//
// dw[m, (c,kh,kw)] = sum over positions of dy[m, pos] * x[c, pos + shift].  The
// contraction index is the position, which is contiguous in memory for both
// operands, so the fragments (8 consecutive positions per lane) need no transpose.
// A workgroup owns 64 output channels x 32 input channels (288 columns) over a
// range of (image, output row) pairs, as the fp32 row kernel does.  Per output row
// LDS holds
//   ds[64 output channels][OWp]            the dy row, zero past OW
//   xs[288 columns = (c,kh,kw)][OWp]       input row ih(kh) of channel c shifted by
//                                          kw-1 columns: x[p + kw - 1], zero outside
// (bf16, OWp = OW rounded up to 32, row pitch OWp*2+16 bytes so that the 16 rows of a
// fragment read fall on distinct banks).  The three shifted copies are made in
// registers from one aligned 16-byte load per 8 columns: the neighbouring columns
// come from the adjacent lanes, v_alignbit_b32 shifts by one element.
// A step is one output row, or - rows of at most 16 (8) columns, images of an even (multiple of
// four) number of rows - two (four) consecutive rows of an image side by side in the 32 positions
// of a k-step: a step costs about 0.6 us whatever it holds (barrier, loader instructions), so a
// 14x14 layer runs twice as fast two rows to a step.
// 8 waves, two roles: waves 0-3 keep four steps in flight in registers (a step of
// MFMA work is far shorter than memory latency) and write step r+2 while waves 4-7
// (2 along m x 2 along the columns, 32 x 144 each) work on step r out of three LDS
// buffers; fragments of the next k-step - or of the next step, which is complete one
// barrier earlier - are read into the registers just used.  One barrier per step.  The loader
// loops are compiled for the units per thread a shape needs (2 + 1 for rows up to 32 columns).
// Partial tiles go to the workspace and are added in a fixed order by
// wgrad_reduce_kernel; the bias gradient is summed from the dy values as they pass
// through the loader registers.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int BM = MFMA_BM;
constexpr int CB = 32;           // input channels per workgroup
constexpr int NCOL = CB * 9;     // columns of the tile
constexpr int THREADS = 512;
constexpr int NTW = 9;           // 16-column blocks per MFMA wave
constexpr int NXI_MAX = 3;       // x units (one (c,kh) row piece of 8 columns) per loader thread and step
constexpr int NDI_MAX = 2;       // dy units per loader thread and step
constexpr int NSET = 4;          // steps in flight in loader registers
constexpr int SPW = NCOL + 4;    // pitch of the parked result tile (words)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const uint4* lds_cell;
#else
typedef const uint4* lds_cell;
#endif

struct W16Params {
  int N, C, H, W, K, OH, OW;
  int py, dly;
  int groups, Cg, Kg;
  int G;               // output rows per step: rows of at most 16 (8) columns go two (four) at a
                       // time, side by side in the 32 positions of a k-step
  int Qr;              // 8-column groups per output row
  int Q;               // 8-column groups per step (G * Qr)
  int OHG;             // steps per image (OH / G)
  int RPW;             // rows per loader wave pass (64 / Q)
  int nks;             // k-steps of 32 positions per step
  int PB;              // LDS row pitch in bytes
  int buf_cells;       // 16-byte cells per LDS buffer (xs then ds)
  int nhalves, mtiles;
  int nsplit, rps;     // K-splits, steps per split
  int total_rows;      // steps in all (N * OH / G)
  int E;               // K*Cg*9
  int want_db;
  int tail;            // dwords (column pairs) of a row's last 8-column unit that lie inside the row
  unsigned x_bytes, dy_bytes;
};

template <typename E, int NXI, int NDI>
__global__ void __launch_bounds__(THREADS, 2)
wgrad16_kernel(W16Params p, const E* __restrict__ x, const E* __restrict__ dy,
               float* __restrict__ out, float* __restrict__ db_out) {
  extern __shared__ uint4 lds16[];
  float* lds = reinterpret_cast<float*>(lds16);
  constexpr int OOB = (int)0x80000000;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x;
  const int half = __builtin_amdgcn_readfirstlane(blockIdx.y % p.nhalves);
  const int mtile = __builtin_amdgcn_readfirstlane(blockIdx.y / p.nhalves);
  const int grp = blockIdx.z;
  const int m_lim = p.Kg - mtile * BM;
  const int row_begin = split * p.rps, row_end = min(row_begin + p.rps, p.total_rows);
  const int nrows = row_end - row_begin;
  const int HW = p.H * p.W, OHW = p.OH * p.OW;
  float* o = out + (p.nsplit > 1 ? (size_t)split * (p.E + p.K) : 0);
  const int ncols = p.Cg * 9;
  const int pcells = p.PB >> 4;             // row pitch in cells
  const int ds_cell0 = NCOL * pcells;       // dy rows follow the 288 x rows of a buffer
  float* stage = lds;                       // [BM][SPW] after the last row
  float* dbpart = lds + BM * SPW;           // [BM][Q] bias partials

  // Positions past OW and the columns outside the image are never written: zero all
  // three buffers once.
  for (int i = tid; i < 3 * p.buf_cells; i += THREADS) lds16[i] = make_uint4(0u, 0u, 0u, 0u);
  __syncthreads();

  auto store_tile = [&]() {
    constexpr int QT = NCOL / 4;
    for (int idx = tid; idx < BM * QT; idx += THREADS) {
      const int m = idx / QT, q = idx - m * QT;
      if (m < m_lim) {
        const float4 v = *reinterpret_cast<const float4*>(stage + m * SPW + 4 * q);
        *reinterpret_cast<float4*>(o + (size_t)(grp * p.Kg + mtile * BM + m) * ncols +
                                   half * NCOL + 4 * q) = v;
      }
    }
  };

  if (wave < 4) {
    // ============================== loader waves ================================
    const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t yrsrc = make_rsrc(dy, p.dy_bytes);
    const bool do_db = p.want_db && half == 0;
    // A wave pass covers RPW rows of Q units; lane = row_in_pass * Q + q, so the
    // columns next to a unit's eight are in the adjacent lanes.
    // (q = the unit's cell in the step: output row q / Qr of the step, columns 8 * (q % Qr)...)
    const int rl = lane / p.Q, q = lane - rl * p.Q;
    const int rsub = q / p.Qr, qq = q - rsub * p.Qr;
    const bool lane_ok = rl < p.RPW;
    const bool first_q = qq == 0, last_q = qq == p.Qr - 1;
    // x rows: index xr = c*3 + kh (96 per tile); dy rows: m (64 per tile)
    int xg[NXI], xl[NXI], xkh[NXI];
#pragma unroll
    for (int i = 0; i < NXI; ++i) {
      const int xr = (i * 4 + wave) * p.RPW + rl;
      xg[i] = OOB;
      xl[i] = -1;
      xkh[i] = 0;
      if (lane_ok && xr < CB * 3) {
        const int c = xr / 3, kh = xr - c * 3;
        xkh[i] = kh;
        xl[i] = xr * 3 * pcells + q;           // cell of the kw = 0 copy; kw copies are pcells apart
        xg[i] = ((grp * p.Cg + half * CB + c) * HW + rsub * p.W + 8 * qq) * 2;
      }
    }
    int yg[NDI], yl[NDI];
#pragma unroll
    for (int i = 0; i < NDI; ++i) {
      const int m = (i * 4 + wave) * p.RPW + rl;
      yg[i] = OOB;
      yl[i] = -1;
      if (lane_ok && m < BM) {
        yl[i] = ds_cell0 + m * pcells + q;
        if (m < m_lim) yg[i] = ((grp * p.Kg + mtile * BM + m) * OHW + rsub * p.OW + 8 * qq) * 2;
      }
    }
    float dbp[NDI];
#pragma unroll
    for (int i = 0; i < NDI; ++i) dbp[i] = 0.f;

    struct RowRegs {
      uintx4_t xv[NXI], yv[NDI];
    };
    auto load_row = [&](int row, RowRegs& r) {
      const bool live = row < row_end;
      const int img = row / p.OHG, oh = (row - img * p.OHG) * p.G + rsub;
#pragma unroll
      for (int i = 0; i < NXI; ++i) {
        const int ih = oh - p.py + xkh[i] * p.dly;
        const bool ok = live && (unsigned)ih < (unsigned)p.H;
        r.xv[i] = __builtin_amdgcn_raw_buffer_load_b128(
            xrsrc, ok ? xg[i] + (img * p.C * HW + (ih - rsub) * p.W) * 2 : OOB, 0, 0);
      }
      const int yb = (img * p.K * OHW + (oh - rsub) * p.OW) * 2;
#pragma unroll
      for (int i = 0; i < NDI; ++i)
        r.yv[i] = __builtin_amdgcn_raw_buffer_load_b128(yrsrc, live ? yg[i] + yb : OOB, 0, 0);
    };
    // the last unit of a row of 8k+2..6 columns has read into the next row: zero that part
    auto in_row = [&](uintx4_t v) {
      if (last_q) {
        v.y = p.tail > 1 ? v.y : 0u;
        v.z = p.tail > 2 ? v.z : 0u;
        v.w = p.tail > 3 ? v.w : 0u;
      }
      return v;
    };
    auto store_row = [&](int buf, const RowRegs& r) {
      uint4* b = lds16 + buf * p.buf_cells;
#pragma unroll
      for (int i = 0; i < NXI; ++i) {
        const uintx4_t v = in_row(r.xv[i]);
        // element left of the eight (high half of the left lane's last dword) and
        // right of them (low half of the right lane's first dword); zero at row ends
        unsigned left = __shfl_up(v.w, 1, 64), right = __shfl_down(v.x, 1, 64);
        left = first_q ? 0u : left;
        right = last_q ? 0u : right;
        const unsigned s1 = __builtin_amdgcn_alignbit(v.y, v.x, 16);
        const unsigned s2 = __builtin_amdgcn_alignbit(v.z, v.y, 16);
        const unsigned s3 = __builtin_amdgcn_alignbit(v.w, v.z, 16);
        if (xl[i] >= 0) {
          b[xl[i]] = make_uint4(__builtin_amdgcn_alignbit(v.x, left, 16), s1, s2, s3);   // x[p-1]
          b[xl[i] + pcells] = make_uint4(v.x, v.y, v.z, v.w);                            // x[p]
          b[xl[i] + 2 * pcells] =
              make_uint4(s1, s2, s3, __builtin_amdgcn_alignbit(right, v.w, 16));         // x[p+1]
        }
      }
#pragma unroll
      for (int i = 0; i < NDI; ++i) {
        const uintx4_t v = in_row(r.yv[i]);
        if (yl[i] >= 0) b[yl[i]] = make_uint4(v.x, v.y, v.z, v.w);
        if (do_db) {
          float s = 0.f;
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const unsigned d = k == 0 ? v.x : k == 1 ? v.y : k == 2 ? v.z : v.w;
            s += Lo16<E>::lo(d) + Lo16<E>::hi(d);
          }
          dbp[i] += s;
        }
      }
    };

    // steps r..r+1 in LDS before the first barrier, r+2..r+1+NSET in registers
    RowRegs set[NSET];
#pragma unroll
    for (int u = 0; u < NSET; ++u) load_row(row_begin + u, set[u]);
    if (nrows > 0) store_row(0, set[0]);
    load_row(row_begin + NSET, set[0]);
    if (nrows > 1) store_row(1, set[1]);
    load_row(row_begin + NSET + 1, set[1]);
    __syncthreads();
    // iteration r: the MFMA waves work on step r; step r+2 (register set (r+2)%NSET) goes
    // to buffer (r+2)%3 and the set is refilled with step r+2+NSET
    for (int r4 = 0; r4 < nrows; r4 += NSET) {
#pragma unroll
      for (int u = 0; u < NSET; ++u) {
        const int r = r4 + u;
        if (r < nrows) {
          if (r + 2 < nrows) store_row((r + 2) % 3, set[(u + 2) % NSET]);
          load_row(row_begin + r + 2 + NSET, set[(u + 2) % NSET]);
          __syncthreads();
        }
      }
    }
    // bias: partials of a channel sit in Q consecutive slots behind the parked tile
    if (do_db) {
#pragma unroll
      for (int i = 0; i < NDI; ++i) {
        const int m = (i * 4 + wave) * p.RPW + rl;
        if (lane_ok && m < BM) dbpart[m * p.Q + q] = dbp[i];
      }
    }
    __syncthreads();                        // tile parked, partials written
    if (do_db && tid < min(m_lim, BM)) {
      float s = 0.f;
      for (int k = 0; k < p.Q; ++k) s += dbpart[tid * p.Q + k];
      const int ch = grp * p.Kg + mtile * BM + tid;
      if (p.nsplit > 1)
        o[p.E + ch] = s;
      else
        db_out[ch] = s;
    }
    store_tile();
    return;
  }

  // ================================ MFMA waves ===================================
  // v_mfma_f32_32x32x16_bf16: a wave owns 32 output channels (A: lane l holds channel l % 32,
  // position group l / 32) and 144 columns as four blocks of 32 plus one block of 16 (the
  // latter through v_mfma_f32_16x16x32_bf16).  A k-step of 32 positions is two 32x32x16
  // steps: lane half h reads cells h and h + 2 of the step's four.  The 32x32 shape issues
  // 2.8 times faster from one wave per SIMD than 16x16x32 (measured).
  const int cw = wave - 4;
  const int wm = cw & 1, wn = cw >> 1;
  const int fr = lane & 31, fh = lane >> 5;
  const int fr16 = lane & 15, fk16 = lane >> 4;
  constexpr int NB32 = 4;
  floatx16 acc[NB32];
  floatx4 acc16[2];
#pragma unroll
  for (int j = 0; j < NB32; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  acc16[0] = acc16[1] = floatx4{0.f, 0.f, 0.f, 0.f};

  // cell addresses in buffer 0
  lds_cell bp[NB32];
#pragma unroll
  for (int j = 0; j < NB32; ++j)
    bp[j] = (lds_cell)lds16 + ((wn * (NTW * 16) + j * 32 + fr) * pcells + fh);
  lds_cell ap = (lds_cell)lds16 + (ds_cell0 + (wm * 32 + fr) * pcells + fh);
  lds_cell bq = (lds_cell)lds16 + ((wn * (NTW * 16) + NB32 * 32 + fr16) * pcells + fk16);
  lds_cell aq0 = (lds_cell)lds16 + (ds_cell0 + (wm * 32 + fr16) * pcells + fk16);
  lds_cell aq1 = aq0 + 16 * pcells;
  auto advance = [&](int cells) {
#pragma unroll
    for (int j = 0; j < NB32; ++j) bp[j] += cells;
    ap += cells;
    bq += cells;
    aq0 += cells;
    aq1 += cells;
  };
  auto frag = [](uint4 v) { return __builtin_bit_cast(bf16x8, v); };

  uint4 a[2], b[NB32][2], sa0, sa1, sb;
  // One k-step: MFMAs on the fragments in registers; behind them the fragments at cell
  // offset OFF (next k-step of this row, or k-step 0 of the next row after the pointers
  // moved) are read into the registers just used.
#define FLHIP_KSTEP(OFF)                                                 \
  {                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                   \
    const uint4 n0 = ap[OFF], n1 = ap[(OFF) + 2];                        \
    const uint4 m0 = aq0[OFF], m1 = aq1[OFF];                            \
    _Pragma("unroll") for (int j = 0; j < NB32; ++j)                     \
      acc[j] = Lo16<E>::mma32(frag(a[0]), frag(b[j][0]), acc[j]); \
    _Pragma("unroll") for (int j = 0; j < NB32; ++j) {                   \
      acc[j] = Lo16<E>::mma32(frag(a[1]), frag(b[j][1]), acc[j]); \
      b[j][0] = bp[j][OFF];                                              \
      b[j][1] = bp[j][(OFF) + 2];                                        \
    }                                                                    \
    acc16[0] = Lo16<E>::mma16(frag(sa0), frag(sb), acc16[0]); \
    acc16[1] = Lo16<E>::mma16(frag(sa1), frag(sb), acc16[1]); \
    sb = bq[OFF];                                                        \
    a[0] = n0;                                                           \
    a[1] = n1;                                                           \
    sa0 = m0;                                                            \
    sa1 = m1;                                                            \
    _Pragma("unroll") for (int q = 0; q < 2 * NB32 + 5; ++q) {           \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 \
    }                                                                    \
    __builtin_amdgcn_sched_barrier(0);                                   \
  }

  __syncthreads();                          // rows 0 and 1 are in buffers 0 and 1
  a[0] = ap[0];
  a[1] = ap[2];
  sa0 = aq0[0];
  sa1 = aq1[0];
  sb = bq[0];
#pragma unroll
  for (int j = 0; j < NB32; ++j) {
    b[j][0] = bp[j][0];
    b[j][1] = bp[j][2];
  }
  for (int r = 0; r < nrows; ++r) {
    for (int ks = 0; ks + 1 < p.nks; ++ks) {
      FLHIP_KSTEP(4)
      advance(4);
    }
    // last k-step of the row: the next fragments are k-step 0 of row r+1, in the
    // next buffer (written one barrier ago)
    advance(((r % 3 == 2) ? -2 : 1) * p.buf_cells - 4 * (p.nks - 1));
    FLHIP_KSTEP(0)
    __syncthreads();
  }
#undef FLHIP_KSTEP

  // accumulator element r of a 32x32 block: channel (r / 4) * 8 + fh * 4 + r % 4, column fr
#pragma unroll
  for (int j = 0; j < NB32; ++j) {
    const int col = wn * (NTW * 16) + j * 32 + fr;
#pragma unroll
    for (int rr = 0; rr < 16; ++rr)
      stage[(wm * 32 + (rr >> 2) * 8 + fh * 4 + (rr & 3)) * SPW + col] = acc[j][rr];
  }
  {
    const int col = wn * (NTW * 16) + NB32 * 32 + fr16;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
        stage[(wm * 32 + i * 16 + fk16 * 4 + rr) * SPW + col] = acc16[i][rr];
  }
  __syncthreads();
  store_tile();
}

bool plan(const ConvGeom& g, W16Params* p) {
  if (g.KH != 3 || g.KW != 3 || g.sy != 1 || g.sx != 1 || g.px != 1 || g.dlx != 1) return false;
  // rows are read in units of 8 columns from 4-byte aligned addresses
  if (g.Cg % CB != 0 || g.OW % 2 != 0 || g.W != g.OW || g.OW > 64) return false;
  p->N = g.N; p->C = g.C; p->H = g.H; p->W = g.W; p->K = g.K; p->OH = g.OH; p->OW = g.OW;
  p->py = g.py; p->dly = g.dly;
  p->groups = g.groups; p->Cg = g.Cg; p->Kg = g.Kg;
  p->Qr = (g.OW + 7) / 8;
  p->tail = (g.OW - 8 * (p->Qr - 1)) / 2;
  // short rows share a step (the images' row count permitting): four rows of 8 columns or two of at most 16
  // side by side in the 32 positions of a k-step, two rows of at most 32 columns as two k-steps
  p->G = (p->Qr == 1 && g.OH % 4 == 0) ? 4 : (p->Qr <= 4 && g.OH % 2 == 0) ? 2 : 1;
  p->Q = p->G * p->Qr;
  p->OHG = g.OH / p->G;
  p->RPW = 64 / p->Q;
  if (CB * 3 > NXI_MAX * 4 * p->RPW || BM > NDI_MAX * 4 * p->RPW) return false;
  const int owp = (8 * p->Q + 31) & ~31;
  p->nks = owp / 32;
  p->PB = owp * 2 + 16;
  p->buf_cells = (NCOL + BM) * (p->PB / 16) + 1;   // + one cell: the read-ahead past the last row
  if ((size_t)3 * p->buf_cells * 16 > 158 * 1024) return false;
  if ((size_t)(BM * SPW + BM * p->Q) * sizeof(float) > (size_t)3 * p->buf_cells * 16) return false;
  p->nhalves = g.Cg / CB;
  p->mtiles = (g.Kg + BM - 1) / BM;
  p->total_rows = g.N * p->OHG;
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

size_t mfma_wgrad16_ws(const ConvGeom& g) {
  W16Params p{};
  if (!plan(g, &p)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
}

int mfma_wgrad16(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws,
                 size_t ws_bytes, hipStream_t s, int dtype) {
  if (!dw) return -1;
  W16Params p{};
  if (!plan(g, &p)) return -1;
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(dy) % 16 != 0) return -1;
  const long long xb = (long long)g.N * g.C * g.H * g.W * 2;
  const long long yb = (long long)g.N * g.K * g.OH * g.OW * 2;
  if (xb >= (1ll << 31) || yb >= (1ll << 31)) return -1;
  p.x_bytes = (unsigned)xb;
  p.dy_bytes = (unsigned)yb;
  p.want_db = db != nullptr;
  const size_t need = p.nsplit > 1 ? (size_t)p.nsplit * (p.E + p.K) * sizeof(float) : 0;
  if (need && (!ws || ws_bytes < need))
    return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  if (reinterpret_cast<uintptr_t>(out) % 16 != 0) return -1;
  const size_t shmem = (size_t)3 * p.buf_cells * 16;
  // loader units per thread and step the shape needs (fewer = fewer loader instructions)
  const bool small = CB * 3 <= 2 * 4 * p.RPW && BM <= 4 * p.RPW;
  const dim3 grid(p.nsplit, p.nhalves * p.mtiles, g.groups);
  const int rc = by_lo16(dtype, [&](auto* e_) {
    using E = FLHIP_T_OF(e_);
    auto kernel = small ? wgrad16_kernel<E, 2, 1> : wgrad16_kernel<E, NXI_MAX, NDI_MAX>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, grid, dim3(THREADS), shmem, s, p, static_cast<const E*>(x), static_cast<const E*>(dy), out, db);
    return 0;
  });
  if (rc) return rc;
  if (p.nsplit > 1)
    wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.K, p.want_db, dw, db, s);
  return check_launch("conv2d_bwd_filter (bf16 mfma)");
}

}  // namespace flhip
