// Filter (and bias) gradient of 3x3 stride-1 pad-1 convolutions in bf16 storage on
// v_mfma_f32_32x32x16_bf16, with the operand rows copied into LDS by the memory pipeline
// itself (buffer loads with the LDS modifier): no wave spends vector instructions on loading,
// all eight waves multiply.
//
//   dw[m][c][kh][kw] = sum over images n and positions (oh, ow) of
//                      dy[n][m][oh][ow] * x[n][c][oh + kh - 1][ow + kw - 1]
//
// The contraction runs over positions, which are contiguous in memory in both operands.  A
// stage is 64 position slots: one output row of 33 to 64 positions (described here; groups of
// shorter rows and whole small images: at the kernel), i.e. the dy row of 64 result channels
// and ONE new input row (n, oh + 1) of 64 input channels; the input rows oh - 1 and oh are
// still in LDS from the two stages before (a ring of rows), so every row of both tensors is
// fetched once per tile.  The vertical taps kh are those three input rows; the horizontal taps
// kw are taken on the dy side, where they cost a third of the rows: with iw = ow + kw - 1,
//   sum_ow dy[ow] x[ow + kw - 1] = sum_iw D_kw[iw] x[iw],   D_kw[iw] = dy[iw - kw + 1]
// (zero outside the row).  D_1 is the dy row as loaded; D_0 and D_2 are made from it by an
// LDS -> LDS pass (a 16-byte cell and one element of its neighbour, shifted by v_alignbit), two
// stages ahead of the multiplications.  The tile is 2 (result channels) x 2 (input channels)
// blocks of 32 x 32 with nine accumulator tiles (kh, kw) each; two waves per block take
// alternate 16-position steps of a stage and add their accumulators through LDS at the end.
//
// Rows of W positions are cut into cells of 8 (16 bytes); when W is not a multiple of 8 the
// last cell ENDS at the row's last position and repeats positions of the cell before it; the
// repeated positions are zeroed in the input rows (by the lanes that loaded them), so every
// product is counted once.  Cells past the row are loaded from an offset beyond the tensor:
// the range check of the buffer descriptor writes zeros.  So are whole input rows above and
// below an image.  A row of LDS is 128 bytes; cell c of row r sits at cell c ^ (r & 7), so
// the 32 rows of a fragment read spread over the banks (a lane fetches the cell that belongs
// where it writes).
//
// A workgroup owns a 64 x 64 tile of (result, input) channels over a range of stages; with one
// row per stage two stages only load at the start of the range and of every image (rows oh - 1
// and oh).  One barrier per stage; while stage t multiplies, the loads of stage t + 1 + WD_D
// are issued, the shifted copies of stage t + 2 are made and the first fragments of stage
// t + 1 are fetched.  Partial tiles go to the workspace as [tap][result channel][input channel]
// (so a lane's 16 values of a tap leave as coalesced rows) and are added in a fixed order by
// wgrad_taps_reduce_kernel, which writes [result channel][input channel][tap].  The bias
// gradient is summed from the dy cells as they pass through the registers of the shifting
// pass (the positions a last cell repeats left out), in the workgroups of the first tile
// column.
#include <algorithm>

#include "conv2d_mfma.h"
#include "lds_direct.h"

namespace flhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int WD_T = 64;                 // tile side (channels)
constexpr int WD_D = 3;                  // the loads of stage t + 1 + D are issued while stage t multiplies
constexpr int WD_NSD = WD_D + 2;         // dy rows in the ring
constexpr int WD_NSX = WD_D + 4;         // input rows in the ring
constexpr int WD_NSH = 3;                // buffers of shifted copies: read (t), waiting (t + 1), being written (t + 2)
constexpr int WD_SLOT = WD_T * 128;      // bytes of a slot: 64 rows of 8 cells
constexpr int WD_LDS = (WD_NSD + WD_NSX + 2 * WD_NSH) * WD_SLOT;

struct WdParams {
  int N, C, K, H, W;
  int ncell;              // cells per row
  int dup;                // positions the last cell repeats
  int keep;               // positions of a cell that belong to the row (8; W in whole-image stages over rows of W < 8)
  int img;                // a stage is a whole image
  int G;                  // output rows per stage (0: whole image)
  int ctiles, mtiles;
  int total_rows, rps, nsplit;
  int E;                  // K * C * 9
  int want_db;
  unsigned x_bytes, dy_bytes;
};

// The stages of a workgroup's range of rows, in order: at the start of the range and of each
// image, two stages that only load input rows (oh - 1, oh); then one per output row.
struct WdStages {
  int n, oh, phase, left;   // image, row, 0 / 1: loading stages, 2: rows; output rows left
  __device__ __forceinline__ void start(int row, int H, int rows) {
    n = row / H;
    oh = row - n * H;
    phase = 0;
    left = rows;
  }
  // the next stage: input row to load (-1 or H: outside the image) and whether it multiplies
  __device__ __forceinline__ bool next(int H, int* img, int* ih) {
    *img = n;
    if (phase == 0) { *ih = oh - 1; phase = 1; return false; }
    if (phase == 1) { *ih = oh; phase = 2; return false; }
    *ih = oh + 1;
    --left;
    if (++oh == H) { oh = 0; ++n; phase = 0; }
    return true;
  }
};

// NK16: steps of 16 positions per row (2 or 4).  Eight waves: two per 32 x 32 block of the tile (and per SIMD), which
// take alternate steps of a row and add their accumulators through LDS at the end: while one of them shifts,
// computes addresses or waits for LDS, the other one's matrix instructions run (one wave per block: 1.3 us per row
// of 56 positions instead of 1.15).
//
// IMG: planes of at most 7 rows of at most 8 positions (7x7): a stage is a whole image, row j in cell j of the 64
// position slots, cell 7 (and every row past the image) zero.  The three input rows of output row j are cells
// (j + kh - 1) mod 8 of the same slot - row -1 and row H both land on a zero cell - so there is no ring of rows and
// no stage that only loads.  A cell of a row of W < 8 positions ends with positions of the next row: they are zeroed in
// the input cells and masked out of the shifted dy copies.  The one cell of each tensor that would reach past its
// end is loaded as zeros and filled in by its lane with plain loads.
//
// G = 2, 4 (rows of at most 32 / 16 positions): a stage is a group of G output rows, row j of the group in cells
// j * 8 / G ... of the 64 position slots.  Its input slot holds the rows G g - 1 ... G g + G - 2; the two rows below
// them are the first two of the NEXT stage's slot, which the loads have brought in already (they run ahead), so
// the first group of an image needs no stage before it (row -1 is loaded as zeros); after the last group of an
// image or of the workgroup's range one stage only loads (the rows below the last group).
constexpr int NW = 8;
template <typename E, int NK16, int G>
__global__ void __launch_bounds__(64 * NW, 1)
wgrad_dma_kernel(WdParams p, const E* __restrict__ x, const E* __restrict__ dy, float* __restrict__ out) {
  constexpr bool IMG = G == 0;          // a stage is a whole image
  constexpr bool GRP = G >= 2;          // a stage is a group of G rows
  constexpr int CPR = GRP ? 8 / G : 8;  // cells of a row in a slot
  static_assert((NK16 == 2 || NK16 == 4) && (G == 1 || NK16 == 4) && (G == 0 || G == 1 || G == 2 || G == 4), "shapes in use");
  extern __shared__ __align__(16) char wd_lds[];
  char* const dring = wd_lds;                                   // [WD_NSD] dy rows
  char* const xring = wd_lds + WD_NSD * WD_SLOT;                // [WD_NSX] input rows
  char* const shift = wd_lds + (WD_NSD + WD_NSX) * WD_SLOT;     // [WD_NSH buffers][D_0, D_2]
  constexpr int OOB = (int)0x80000000;
  constexpr int THREADS = 64 * NW;
  constexpr int NCU = 2 * NK16;                                 // cells of a row that the multiplications read
  constexpr int NLB = 8 / NW;                                   // 8-row blocks of a slot that a wave loads
  constexpr int NSW = NK16 * 4 / NW;                            // steps of a row per wave
  const int split = blockIdx.x, mtile = blockIdx.y / p.ctiles, ctile = blockIdx.y - mtile * p.ctiles;
  const int m0 = mtile * WD_T, c0 = ctile * WD_T;
  const int tid = threadIdx.x, lane = tid & 63, fr = lane & 31, fh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = wave & 3, half = wave >> 2;                   // block of the tile; which steps of a row
  const int wm = blk >> 1, wn = blk & 1;
  const int row_begin = split * p.rps, nrows = min(row_begin + p.rps, p.total_rows) - row_begin;
  const intx4_t drs = pd_rsrc(dy, p.dy_bytes), xrs = pd_rsrc(x, p.x_bytes);
  const int P = p.H * p.W;

  // ---- loads: instruction i of a wave fills rows 8 (NW i + wave) .. + 7 of a slot; lane -> row + lane / 8, LDS
  // cell lane % 8, i.e. the row's cell (lane % 8) ^ (lane / 8)
  const int lrow = lane >> 3, lcell = (lane & 7) ^ lrow;
  // (IMG: cell = row of the image; GRP: cell = (row of the group, cell of the row))
  const int lj = GRP ? lcell / CPR : 0, lcq = GRP ? lcell % CPR : lcell;
  const bool cell_ok = IMG ? lcell < p.H : lcq < p.ncell;
  // first position of the lane's cell (GRP: in its row)
  const int lpos = IMG ? lcell * p.W : (lcq == p.ncell - 1 ? p.W - 8 : 8 * lcq);
  int xoff[NLB], doff[NLB];
#pragma unroll
  for (int i = 0; i < NLB; ++i) {
    const int r = 8 * (NW * i + wave) + lrow;
    xoff[i] = cell_ok ? ((c0 + r) * P + lpos) * 2 : OOB;
    doff[i] = cell_ok ? ((m0 + r) * P + lpos) * 2 : OOB;
  }
  const unsigned lds0 = pd_lds_addr(wd_lds);
  // stage `st` of the range: its loads into dy slot st % NSD and input slot st % NSX
  WdStages gi, gc;
  gi.start(row_begin, p.H, nrows);
  gc.start(row_begin, p.H, nrows);
  int nstages = 0;
  const int GH = GRP ? (p.H + G - 1) / G : 1;          // groups per image; a "row" of the range is a group
  // GRP: the groups of the range in order, one loading stage after the last group of an image and of the range
  struct { int n, g, left; bool post; } qi{row_begin / GH, row_begin % GH, nrows, false}, qc = qi;
  auto grp_next = [&](auto& q, int* img, int* grp) -> bool {
    *img = q.n;
    *grp = q.g;
    if (q.post) {                       // the rows below the group before
      q.post = false;
      if (q.g == GH) { q.g = 0; ++q.n; }
      return false;
    }
    --q.left;
    ++q.g;
    if (q.g == GH || q.left == 0) q.post = true;
    return true;
  };
  if (GRP) {
    const int n_first = row_begin / GH, n_last = (row_begin + nrows - 1) / GH;
    // one loading stage per image the range ends in or passes the end of (the range's own end included)
    nstages = nrows + (n_last - n_first + 1);
  } else if (IMG) {
    nstages = nrows;                    // a "row" of the range is an image
  } else {
    const int n_first = row_begin / p.H, n_last = (row_begin + nrows - 1) / p.H;
    nstages = nrows + 2 * (n_last - n_first + 1);
  }
  int islot_d = 0, islot_x = 0, issued = 0;
  auto issue = [&]() {
    int img, ih = 0, oh = 0;
    bool rows = true;
    if (GRP) {
      int grp;
      rows = grp_next(qi, &img, &grp);
      ih = G * grp - 1 + lj;            // the lane's input row, and its output row
      oh = G * grp + lj;
    } else if (IMG) {
      img = row_begin + issued;
    } else {
      oh = gi.oh;
      rows = gi.next(p.H, &img, &ih);
    }
    ++issued;
    const bool x_in = ih >= 0 && ih < p.H, d_in = rows && oh < p.H;
    const int xs = (img * p.C * p.H + ih) * p.W * 2, ds = (img * p.K * p.H + oh) * p.W * 2;
#pragma unroll
    for (int i = 0; i < NLB; ++i) {
      pd_load_lds(xrs, lds0 + (WD_NSD + islot_x) * WD_SLOT + (NW * i + wave) * 1024,
                  (x_in && xoff[i] != OOB) ? xoff[i] + xs : OOB, 0);
      pd_load_lds(drs, lds0 + islot_d * WD_SLOT + (NW * i + wave) * 1024, (d_in && doff[i] != OOB) ? doff[i] + ds : OOB, 0);
    }
    islot_d = islot_d + 1 == WD_NSD ? 0 : islot_d + 1;
    islot_x = islot_x + 1 == WD_NSX ? 0 : islot_x + 1;
  };
  // After this lane's loads of a stage have landed: zeros over the repeated positions (the first p.dup of the row's
  // last cell) of the input cells it loaded into slot xs.  IMG (stage = image `img`, dy slot ds): zeros over the
  // positions past the row in its input cells, and the cell at the very end of either tensor, which was loaded as
  // zeros (the last two bytes of its 16 lie past the tensor), is filled in with plain loads.
  auto fix_tail = [&](int xs, int ds, int img) {
    if (IMG) {
      if (p.keep < 8 && cell_ok) {
#pragma unroll
        for (int i = 0; i < NLB; ++i) {
          uint16_t* q = reinterpret_cast<uint16_t*>(xring + xs * WD_SLOT + (NW * i + wave) * 1024 + lane * 16);
          uint16_t* qd = reinterpret_cast<uint16_t*>(dring + ds * WD_SLOT + (NW * i + wave) * 1024 + lane * 16);
          const int ox = xoff[i] + img * p.C * P * 2, od = doff[i] + img * p.K * P * 2;
          if ((unsigned)ox + 16u > p.x_bytes)
            for (int e = 0; e < p.keep; ++e) q[e] = reinterpret_cast<const uint16_t*>(x)[(ox >> 1) + e];
          if ((unsigned)od + 16u > p.dy_bytes)
            for (int e = 0; e < p.keep; ++e) qd[e] = reinterpret_cast<const uint16_t*>(dy)[(od >> 1) + e];
          for (int e = p.keep; e < 8; ++e) q[e] = 0;
        }
      }
      return;
    }
    if (p.dup != 0 && lcq == p.ncell - 1) {
#pragma unroll
      for (int i = 0; i < NLB; ++i) {
        char* q = xring + xs * WD_SLOT + (NW * i + wave) * 1024 + lane * 16;
        int d = p.dup, at = 0;
        if (d >= 4) {
          *reinterpret_cast<uintx2_t*>(q) = uintx2_t{0u, 0u};
          d -= 4;
          at = 8;
        }
        if (d >= 2) {
          *reinterpret_cast<uint32_t*>(q + at) = 0u;
          d -= 2;
          at += 4;
        }
        if (d) *reinterpret_cast<uint16_t*>(q + at) = 0;
      }
    }
  };

  // ---- the two shifted copies of a dy row: a thread makes cells (row, cell) = (idx / NCU, idx % NCU),
  // idx = tid + THREADS i.  D_0 = positions + 1 (the element after the cell comes from the next cell, zero past the
  // row), D_2 = positions - 1 (the element before it from the cell before, zero before the row).  The reads of
  // a stage are issued in one go and the results written later, so the multiplications in between hide them.
  constexpr int NSH = (WD_T * NCU + THREADS - 1) / THREADS;
  int sh_cell[NSH], sh_nx[NSH], sh_pv[NSH];      // byte offsets in a slot: the cell, the element after it, the one before
  unsigned sh_skip[NSH], sh_keep[NSH];            // elements [skip, keep) of the cell count: the head may repeat positions,
                                                  // the tail may belong to the next row (IMG)
  uint32_t sh_mask[NSH][4];                       // the same tail as a mask over the cell's four words
  bool sh_on[NSH], sh_has_nx[NSH], sh_has_pv[NSH];
#pragma unroll
  for (int i = 0; i < NSH; ++i) {
    const int idx = tid + THREADS * i;
    const int r = (idx / NCU) & (WD_T - 1), c = idx % NCU, sw = r & 7;
    const int cq = GRP ? c % CPR : c;            // the cell inside its row; the neighbours are cells of the same row
    const bool in = IMG ? c < p.H : cq < p.ncell;
    const int pos = cq == p.ncell - 1 ? p.W - 8 : 8 * cq;
    const int cn = min(c + 1, 7), start = cq + 1 == p.ncell - 1 ? p.W - 8 : 8 * (cq + 1);
    const int cp = max(c - 1, 0);                 // starts at 8 (cq - 1) (only the last cell of a row is moved)
    sh_on[i] = idx < WD_T * NCU;
    sh_cell[i] = r * 128 + ((c ^ sw) << 4);
    sh_has_nx[i] = !IMG && in && pos + 8 < p.W;
    sh_has_pv[i] = !IMG && in && pos > 0;
    sh_nx[i] = r * 128 + ((cn ^ sw) << 4) + (sh_has_nx[i] ? 2 * (pos + 8 - start) : 0);
    sh_pv[i] = r * 128 + ((cp ^ sw) << 4) + (sh_has_pv[i] ? 2 * (pos - 1 - 8 * (cq - 1)) : 0);
    sh_skip[i] = !in ? 8u : (!IMG && cq == p.ncell - 1 ? (unsigned)p.dup : 0u);
    sh_keep[i] = IMG ? (unsigned)p.keep : 8u;
#pragma unroll
    for (int k = 0; k < 4; ++k)
      sh_mask[i][k] = (2u * k < sh_keep[i] ? 0xffffu : 0u) | (2u * k + 1 < sh_keep[i] ? 0xffff0000u : 0u);
  }
  uintx4_t sh_v[NSH];
  uint32_t sh_a[NSH], sh_b[NSH];
  float dbsum[NSH];
#pragma unroll
  for (int i = 0; i < NSH; ++i) dbsum[i] = 0.f;
  const bool do_db = p.want_db && ctile == 0;
  auto shift_reads = [&](int ds_slot) {
    const char* src = dring + ds_slot * WD_SLOT;
#pragma unroll
    for (int i = 0; i < NSH; ++i) {
      sh_v[i] = *reinterpret_cast<const uintx4_t*>(src + sh_cell[i]);
      sh_a[i] = *reinterpret_cast<const uint16_t*>(src + sh_nx[i]);
      sh_b[i] = *reinterpret_cast<const uint16_t*>(src + sh_pv[i]);
    }
  };
  auto shift_writes = [&](int buf) {
    char* dst = shift + buf * 2 * WD_SLOT;
#pragma unroll
    for (int i = 0; i < NSH; ++i) {
      // cells past the row hold zeros (the loads wrote them), so do their copies
      const uintx4_t v = uintx4_t{sh_v[i].x & sh_mask[i][0], sh_v[i].y & sh_mask[i][1], sh_v[i].z & sh_mask[i][2],
                                  sh_v[i].w & sh_mask[i][3]};
      const uint32_t nx = sh_has_nx[i] ? sh_a[i] : 0u, pv = sh_has_pv[i] ? sh_b[i] : 0u;
      if (sh_on[i]) {
        char* o = dst + sh_cell[i];
        *reinterpret_cast<uintx4_t*>(o) =
            uintx4_t{(v.x >> 16) | (v.y << 16), (v.y >> 16) | (v.z << 16), (v.z >> 16) | (v.w << 16), (v.w >> 16) | (nx << 16)};
        *reinterpret_cast<uintx4_t*>(o + WD_SLOT) =
            uintx4_t{pv | (v.x << 16), (v.x >> 16) | (v.y << 16), (v.y >> 16) | (v.z << 16), (v.z >> 16) | (v.w << 16)};
      }
      if (do_db) {
        // bias gradient: the row's dy values pass through here once; positions that the last cell repeats are left out
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          t += 2u * k >= sh_skip[i] ? Lo16<E>::lo(w[k]) : 0.f;                    // (the tail is masked already)
          t += 2u * k + 1 >= sh_skip[i] ? Lo16<E>::hi(w[k]) : 0.f;
        }
        dbsum[i] += sh_on[i] ? t : 0.f;
      }
    }
  };

  // ---- fragments: lane -> row fr of a 32-row block, k-octet fh of a 16-position step; the wave's step j of a row
  // is step half + 2 j
  int foff[NSW];                        // byte offset of the lane's cell of step j in its row
#pragma unroll
  for (int j = 0; j < NSW; ++j) {
    const int sstep = half + 2 * j;
    foff[j] = ((2 * sstep + fh) ^ (fr & 7)) * 16;
  }
  // input rows: the same cell of three slots (rows of a ring); IMG: the cells (row + kh - 1) mod 8 of one slot;
  // GRP: row j + kh of this stage's slot, or row j + kh - G of the next stage's (bnext)
  int boff[NSW][3];
  bool bnext[NSW][3];
#pragma unroll
  for (int j = 0; j < NSW; ++j)
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
      const int cell = 2 * (half + 2 * j) + fh;
      bnext[j][kh] = false;
      if (GRP) {
        const int rho = cell / CPR + kh;          // the same for both halves of the wave: a row has at least 2 cells
        bnext[j][kh] = __builtin_amdgcn_readfirstlane(rho >= G ? 1 : 0) != 0;
        boff[j][kh] = ((((rho % G) * CPR + cell % CPR)) ^ (fr & 7)) * 16;
      } else {
        boff[j][kh] = IMG ? ((((cell + kh - 1) & 7) ^ (fr & 7)) * 16) : foff[j];
      }
    }
  const int arow = (wm * 32 + fr) * 128, brow = (wn * 32 + fr) * 128;
  floatx16 acc[3][3];
#pragma unroll
  for (int r = 0; r < 16; ++r)
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int b = 0; b < 3; ++b) acc[a][b][r] = 0.f;

  if (nrows > 0) {
    // Stage t multiplies while: the loads of stage t + 1 + D are issued, the shifted copies of stage t + 2 are made
    // (its loads are waited for before the barrier of iteration t), and the fragments of stage t + 1's first step
    // are fetched behind the last products of stage t.  Every wave issues 2 NLB loads per stage.
    static_assert(WD_D == 3, "the load counts below");
#pragma unroll
    for (int st = 0; st <= WD_D; ++st)
      if (st < nstages) issue();
    static_assert(NLB == 1, "two loads per stage and wave");
    if (WD_D + 1 <= nstages) PD_WAIT_VM(4);           // stages 2 .. D may be outstanding: 0 and 1 have landed
    else PD_WAIT_VM(0);
    fix_tail(0, 0, row_begin);
    if (nstages > 1) fix_tail(1, 1, row_begin + 1);
    int sd = 0, sx = 0, sb = 0;          // slots of stage t: dy ring, input ring, shifted copies
    bool m0_ = false, m1_ = false, m2_ = false;   // whether stages t, t + 1, t + 2 multiply
    if (GRP) {
      int img, grp;
      m0_ = grp_next(qc, &img, &grp);
      m1_ = grp_next(qc, &img, &grp);
    } else if (IMG) {
      m0_ = true;
      m1_ = nstages > 1;
    } else {
      // (stages 0 and 1 only load: no shifted copies to make, no fragments to fetch)
      int img, ih;
      m0_ = gc.next(p.H, &img, &ih);
      if (nstages > 1) m1_ = gc.next(p.H, &img, &ih);
    }
    bf16x8 fa[2][3], fb[2][3];
#define WD_FRAGS(SET, J, D0, D1, B0, B1, B2)                                                           \
  {                                                                                                    \
    fa[SET][0] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((D0) + foff[J]));       \
    fa[SET][1] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((D1) + foff[J]));       \
    fa[SET][2] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((D0) + WD_SLOT + foff[J])); \
    fb[SET][0] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((B0) + boff[J][0]));    \
    fb[SET][1] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((B1) + boff[J][1]));    \
    fb[SET][2] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>((B2) + boff[J][2]));    \
  }
#define WD_MULT(SET)                                                                                   \
  _Pragma("unroll") for (int kh = 0; kh < 3; ++kh)                                                     \
    _Pragma("unroll") for (int kw = 0; kw < 3; ++kw)                                                   \
      acc[kh][kw] = Lo16<E>::mma32(fa[SET][kw], fb[SET][kh], acc[kh][kw]);
    if (IMG || GRP) {
      // the first two stages multiply too: their shifted copies, and the first fragments of stage 0
      __syncthreads();
      shift_reads(0);
      shift_writes(0);
      if (nstages > 1) {
        shift_reads(1);
        shift_writes(1);
      }
      __syncthreads();
      const char* xs0 = xring + brow;
      const char* xs1 = xring + WD_SLOT + brow;
      WD_FRAGS(0, 0, shift + arow, dring + arow, (bnext[0][0] ? xs1 : xs0), (bnext[0][1] ? xs1 : xs0), (bnext[0][2] ? xs1 : xs0))
    }
    for (int t = 0; t < nstages; ++t) {
      const int nd = sd + 1 == WD_NSD ? 0 : sd + 1, nx = sx + 1 == WD_NSX ? 0 : sx + 1, nb = sb + 1 == WD_NSH ? 0 : sb + 1;
      const int nd2 = nd + 1 == WD_NSD ? 0 : nd + 1, nx2 = nx + 1 == WD_NSX ? 0 : nx + 1, nb2 = nb + 1 == WD_NSH ? 0 : nb + 1;
      m2_ = false;
      if (t + 2 < nstages) {
        if (t + 1 + WD_D <= nstages) PD_WAIT_VM(2);     // stages t + 3 .. t + D may be outstanding
        else PD_WAIT_VM(0);
        fix_tail(nx2, nd2, row_begin + t + 2);
        if (GRP) {
          int img, grp;
          m2_ = grp_next(qc, &img, &grp);
        } else if (IMG) {
          m2_ = true;
        } else {
          int img, ih;
          m2_ = gc.next(p.H, &img, &ih);
        }
      }
      __syncthreads();
      if (t + 1 + WD_D < nstages) issue();
      if (m2_) shift_reads(nd2);
      // operands of stage t and of stage t + 1 (for its first fragments)
      const char* d1 = dring + sd * WD_SLOT + arow;
      const char* d0 = shift + sb * 2 * WD_SLOT + arow;
      const int x1 = sx == 0 ? WD_NSX - 1 : sx - 1, x0 = x1 == 0 ? WD_NSX - 1 : x1 - 1;
      const char* bc = xring + sx * WD_SLOT + brow;       // this stage's input slot, the next stage's, the one after
      const char* bn = xring + nx * WD_SLOT + brow;
      const char* bn2 = xring + nx2 * WD_SLOT + brow;
      const char* br1 = xring + x1 * WD_SLOT + brow;      // the rows of the two stages before (ring of single rows)
      const char* br0 = xring + x0 * WD_SLOT + brow;
      const char* e1 = dring + nd * WD_SLOT + arow;
      const char* e0 = shift + nb * 2 * WD_SLOT + arow;
      // input rows of tap row kh for the wave's step J of stage t (T = 0) or t + 1 (T = 1)
#define WD_B(T, J, KH)                                                                                     \
  (GRP ? (bnext[J][KH] ? ((T) ? bn2 : bn) : ((T) ? bn : bc))                                               \
       : IMG ? ((T) ? bn : bc)                                                                             \
             : ((KH) == 2 ? ((T) ? bn : bc) : (KH) == 1 ? ((T) ? bc : br1) : ((T) ? br1 : br0)))
      if (NSW == 1) {
        // one step per row and wave: no second register set to fetch ahead into; the other wave of the SIMD covers the wait
        if (m0_) {
          WD_FRAGS(0, 0, d0, d1, WD_B(0, 0, 0), WD_B(0, 0, 1), WD_B(0, 0, 2))
          WD_MULT(0)
        }
        if (m2_) shift_writes(nb2);
      } else {
        if (m0_) {
          // (set 0 holds the first step: fetched at the end of the iteration before)
          WD_FRAGS(1, 1, d0, d1, WD_B(0, 1, 0), WD_B(0, 1, 1), WD_B(0, 1, 2))
          WD_MULT(0)
        }
        if (m2_) shift_writes(nb2);
        if (m0_) {
#pragma unroll
          for (int j = 1; j < NSW; ++j) {
            if (j + 1 < NSW) WD_FRAGS((j + 1) & 1, (j + 1 < NSW ? j + 1 : 0), d0, d1, WD_B(0, (j + 1 < NSW ? j + 1 : 0), 0), WD_B(0, (j + 1 < NSW ? j + 1 : 0), 1), WD_B(0, (j + 1 < NSW ? j + 1 : 0), 2))
            else if (m1_) WD_FRAGS(0, 0, e0, e1, WD_B(1, 0, 0), WD_B(1, 0, 1), WD_B(1, 0, 2))
            WD_MULT(j & 1)
          }
        } else if (m1_) {
          WD_FRAGS(0, 0, e0, e1, WD_B(1, 0, 0), WD_B(1, 0, 1), WD_B(1, 0, 2))
        }
      }
      sd = nd;
      sx = nx;
      sb = nb;
      m0_ = m1_;
      m1_ = m2_;
    }
#undef WD_B
#undef WD_MULT
#undef WD_FRAGS
  }

  // element r of a tile: result channel m0 + wm*32 + (r/4)*8 + fh*4 + r%4, input channel c0 + wn*32 + fr
  float* o = out + (size_t)split * ((size_t)p.E + p.K);
  const size_t KC = (size_t)p.K * p.C;
  const int c = c0 + wn * 32 + fr;
  {
    // The two waves of a block add their accumulators through LDS: taps 0..4 end up in the first wave, taps 5..8 in
    // the second (the other wave's values parked as [block][tap][4 registers][lane] cells of 16 bytes: 80 KB from the
    // second waves, then 64 KB from the first), then each stores its share.
    static_assert(WD_LDS >= 4 * 9 * 4 * 64 * 16, "the parked accumulators fit");
    uintx4_t* park = reinterpret_cast<uintx4_t*>(wd_lds);
    auto parked = [&](int tap, int q) {
      return tap < 5 ? ((blk * 5 + tap) * 4 + q) * 64 + lane : 4 * 5 * 4 * 64 + ((blk * 4 + tap - 5) * 4 + q) * 64 + lane;
    };
    __syncthreads();
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        const int tap = kh * 3 + kw;
        const bool mine = (tap < 5) == (half == 0);          // this wave keeps the tap
        if (!mine) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            park[parked(tap, q)] =
                uintx4_t{__float_as_uint(acc[kh][kw][4 * q]), __float_as_uint(acc[kh][kw][4 * q + 1]),
                         __float_as_uint(acc[kh][kw][4 * q + 2]), __float_as_uint(acc[kh][kw][4 * q + 3])};
        }
      }
    __syncthreads();
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        const int tap = kh * 3 + kw;
        const bool mine = (tap < 5) == (half == 0);
        if (mine) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uintx4_t v = park[parked(tap, q)];
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int r = 4 * q + k;
              const int m = m0 + wm * 32 + (r >> 2) * 8 + fh * 4 + (r & 3);
              // the first wave's value first: the same order of the two terms in both shares
              const float lo = half == 0 ? acc[kh][kw][r] : __uint_as_float(w[k]);
              const float hi = half == 0 ? __uint_as_float(w[k]) : acc[kh][kw][r];
              o[tap * KC + (size_t)m * p.C + c] = lo + hi;
            }
          }
        }
      }
  }
  if (do_db) {
    // a row's sums sit in the threads idx = row * NCU .. + NCU - 1: through LDS, added in a fixed order
    float* sums = reinterpret_cast<float*>(wd_lds);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NSH; ++i)
      if (sh_on[i]) sums[tid + THREADS * i] = dbsum[i];
    __syncthreads();
    if (tid < WD_T) {
      float t = 0.f;
      for (int k = 0; k < NCU; ++k) t += sums[tid * NCU + k];
      o[p.E + m0 + tid] = t;
    }
  }
}

// ---- the same pass on 32 x 32 tiles -----------------------------------------------------------
// A 64 x 64 tile per workgroup leaves few tiles (ONE for 64 -> 64 channels), so the positions are cut
// into as many slices as there are CUs and every slice writes a whole partial gradient: 256 x 147 KB
// written and read again by the reduce kernel, three times the bytes of the operands.  Here a
// workgroup owns a 32 x 32 tile of (result, input) channels: four times the tiles, a quarter of the
// slices, a quarter of the partial bytes; a slice is four times longer, so its start-up and its
// final exchange weigh a quarter.  Each operand row is then fetched by two (K / 32, C / 32) tiles
// instead of one: the tiles of a slice are numbered so that they run on one XCD at the same time and
// the second fetch comes out of its L2.
//
// Slots are 32 rows (4 KB), a stage is one 16-byte load per lane: waves 0-3 copy the 32 dy rows,
// waves 4-7 the 32 input rows, into two rings of W3_NS slots (stage st lives in slot st % W3_NS of
// both).  One 32 x 32 block has 4 steps of 16 positions per stage for 8 waves, so an iteration of
// the main loop (one barrier) covers TWO stages: wave (half, step) multiplies step `step` of stage
// 2u + half.  Everything else a wave does in the iteration runs under its own matrix instructions:
// the loads of the two stages W3_D ahead, the shifted dy copies of the stage four ahead (one cell
// per thread) and the fragments of its next stage, fetched into each fragment register as soon
// as the last product that reads it has been issued.
// What bounds an iteration is the number of instructions a wave issues in it (a wave issues one
// every four or five cycles, whatever their kind), so the loop is written to have few:
//  * it is unrolled over the W3_NS / 2 positions of the rings and compiled once per half, so every LDS
//    address is a constant plus a lane's fixed offset;
//  * what a stage loads (image, rows) comes from a table of 64 stages that a wave keeps in the lanes of two
//    registers (entry i in lane i, fetched with v_readlane) and refills every 32 iterations;
//  * every stage multiplies, also the ones that only bring input rows in (the two at the head of an
//    image when rows are long, the one below a group of short rows) and the stage of zeros that
//    pads an odd count: their dy rows are loaded as zeros, so their products are zeros (slots of the
//    input ring that no load has filled yet are cleared when the workgroup starts);
//  * the bias gradient is one more matrix instruction per stage - the dy fragment times a
//    fragment of ones with zeros at the positions a row's last cell repeats - in place of sixteen
//    vector instructions per cell of the shifting pass.
// At the end the eight waves' accumulators are added through LDS, three taps at a time, in a fixed order.
constexpr int W3_T = 32;
constexpr int W3_NS = 16;                 // slots per ring
constexpr int W3_D = 12;                  // the loads of stages 2u + 2 + D, 2u + 3 + D are issued in iteration u
constexpr int W3_NSH = 4;                 // shifted copies of stages 2u + 2, 2u + 3 (read in iteration u), 2u + 4, 2u + 5 (written)
constexpr int W3_SLOT = W3_T * 128;
constexpr int W3_LDS = (2 * W3_NS + 2 * W3_NSH) * W3_SLOT;     // all 160 KB of a CU
static_assert(W3_D % 2 == 0 && W3_D >= 6 && W3_NS >= W3_D + 4 && W3_NS % 4 == 0, "stages are issued in pairs; a stage's input rows stay for two more stages");
#define W3_WAIT_VM(N) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory")

// What stage `st` of a workgroup's range loads: {byte offset of input row ih0 of the image in x (channel 0), ih0,
// byte offset of dy row oh0 (channel 0), oh0 or a negative number when the stage has no dy rows (it only loads
// input rows and does not multiply)}.  In the modes with several rows per stage a lane adds its row of the group
// to ih0 / oh0 (and that row's bytes to the offsets); rows outside the image are loaded as zeros.
//   G == 1: at the start of the range and of every image two stages load the input rows oh - 1 and oh, then one
//           stage per output row oh loads dy row oh and input row oh + 1;
//   G >= 2: a "row" of the range is a group of G output rows; a group's stage loads dy rows G g .. and input rows
//           G g - 1 ..; after the last group of an image or of the range one stage loads the input rows below it;
//   G == 0: a "row" of the range is an image, a stage loads it whole.
template <int G>
__device__ __forceinline__ int4 w3_stage(const WdParams& p, int row_begin, int nrows, int st) {
  const int GH = G >= 2 ? (p.H + G - 1) / G : p.H;          // "rows" per image
  int img, ih0, oh0;
  if (G == 0) {
    img = row_begin + st;
    ih0 = 0;
    oh0 = 0;
  } else {
    const int extra = G == 1 ? 2 : 1;                          // stages of a segment that only load
    const int n0 = row_begin / GH, f0 = row_begin - n0 * GH;
    const int r0 = min(GH - f0, nrows);                        // rows of the range in its first image
    int seg, local, first, count;
    if (st < r0 + extra) {
      seg = 0; local = st; first = f0; count = r0;
    } else {
      const int s2 = st - (r0 + extra);
      seg = 1 + s2 / (GH + extra);
      local = s2 - (seg - 1) * (GH + extra);
      first = 0;
      count = min(GH, nrows - r0 - (seg - 1) * GH);
    }
    img = n0 + seg;
    if (G == 1) {
      const int oh = first + local - 2;                        // (local < 2: the two loading stages)
      ih0 = local == 0 ? first - 1 : local == 1 ? first : oh + 1;
      oh0 = local < 2 ? -1 : oh;
    } else {
      const int grp = first + min(local, count);
      ih0 = G * grp - 1;
      oh0 = local < count ? G * grp : -1;
    }
  }
  return make_int4((img * p.C * p.H + ih0) * p.W * 2, ih0, (img * p.K * p.H + max(oh0, 0)) * p.W * 2, oh0);
}

template <typename E, int G>
__global__ void __launch_bounds__(512, 1)
wgrad_dma32_kernel(WdParams p, const E* __restrict__ x, const E* __restrict__ dy, float* __restrict__ out) {
  constexpr bool IMG = G == 0;          // a stage is a whole image
  constexpr bool GRP = G >= 2;          // a stage is a group of G rows
  constexpr int CPR = GRP ? 8 / G : 8;  // cells of a row in a slot
  static_assert(G == 0 || G == 1 || G == 2 || G == 4, "shapes in use");
  extern __shared__ __align__(16) char wd_lds[];
  // LDS as 32-bit addresses: a lane's fixed offset plus a constant, which the instruction carries
  typedef __attribute__((address_space(3))) char lchar;
  typedef __attribute__((address_space(3))) uintx4_t lu4;
  typedef __attribute__((address_space(3))) uint16_t lu16;
  lchar* const L = (lchar*)wd_lds;
  constexpr int DRING = 0, XRING = W3_NS * W3_SLOT, SHIFT = 2 * W3_NS * W3_SLOT;   // byte offsets: dy rows, input rows, [buffer][D_0, D_2]
  constexpr int OOB = (int)0x80000000;
  // workgroup -> (slice, tile): consecutive workgroup numbers go to the 8 XCDs in turn; the tiles of a slice get
  // numbers 8 apart, so they share an L2
  const int ntiles = p.ctiles * p.mtiles;
  const int per = (int)gridDim.x >> 3;
  const int lin = ((int)blockIdx.x & 7) * per + ((int)blockIdx.x >> 3);
  if (lin >= p.nsplit * ntiles) return;
  const int split = lin / ntiles, tile = lin - split * ntiles;
  const int mtile = tile / p.ctiles, ctile = tile - mtile * p.ctiles;
  const int m0 = mtile * W3_T, c0 = ctile * W3_T;
  const int tid = threadIdx.x, lane = tid & 63, fr = lane & 31, fh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kstep = wave & 3, half = wave >> 2;                 // step of a stage; which stages
  const bool ldx = wave >= 4;                                   // this wave copies input rows (else dy rows)
  const int lblk = wave & 3;                                    // ... rows 8 lblk .. + 7 of the slot
  const int row_begin = split * p.rps, nrows = min(row_begin + p.rps, p.total_rows) - row_begin;
  const intx4_t drs = pd_rsrc(dy, p.dy_bytes), xrs = pd_rsrc(x, p.x_bytes);
  const int P = p.H * p.W;
  int nstages = 0;
  if (nrows > 0) {
    if (GRP) {
      const int GH = (p.H + G - 1) / G;
      nstages = nrows + ((row_begin + nrows - 1) / GH - row_begin / GH + 1);
    } else if (IMG) {
      nstages = nrows;
    } else {
      nstages = nrows + 2 * ((row_begin + nrows - 1) / p.H - row_begin / p.H + 1);
    }
  }
  // (an odd count gets one stage more that loads zeros: stages go in pairs)
  const int nst2 = (nstages + 1) & ~1;
  // the wave's table of stages tbase .. tbase + 63 (lane i: stage tbase + i): offset and first row of the tensor
  // this wave loads; stages past the last load zeros
  int tab_base = 0, tab_row = 0;
  auto fill_table = [&](int tbase) __attribute__((always_inline)) {
    const int st = tbase + lane;
    const int4 e = st < nstages ? w3_stage<G>(p, row_begin, nrows, st) : make_int4(0, -(1 << 20), 0, -1);
    tab_base = ldx ? e.x : e.z;
    tab_row = ldx ? e.y : e.w;
  };
  fill_table(0);
  // ---- loads: lane -> row 8 lblk + lane / 8, LDS cell lane % 8, i.e. the row's cell (lane % 8) ^ (lane / 8)
  const int lrow = lane >> 3, lcell = (lane & 7) ^ lrow;
  const int lj = GRP ? lcell / CPR : 0, lcq = GRP ? lcell % CPR : lcell;
  const bool cell_ok = IMG ? lcell < p.H : lcq < p.ncell;
  const int lpos = IMG ? lcell * p.W : (lcq == p.ncell - 1 ? p.W - 8 : 8 * lcq);
  // the lane's offset in the stage's row of channel 0 of its tensor (its row of a group included)
  const int loff = cell_ok ? (((ldx ? c0 : m0) + 8 * lblk + lrow) * P + lpos + lj * p.W) * 2 : OOB;
  const unsigned lds0 = pd_lds_addr(wd_lds) + (ldx ? XRING : DRING) + lblk * 1024;   // this wave's part of slot 0 of its ring
  // stage st (in the wave's table) into slot `slot` of the wave's ring
  auto issue = [&](int st, int slot) __attribute__((always_inline)) {
    const int base = __builtin_amdgcn_readlane(tab_base, st & 63), row0 = __builtin_amdgcn_readlane(tab_row, st & 63);
    if (ldx) {
      const bool in = (unsigned)(row0 + lj) < (unsigned)p.H && loff != OOB;
      pd_load_lds(xrs, lds0 + slot * W3_SLOT, in ? loff + base : OOB, 0);
    } else {
      const bool in = row0 >= 0 && row0 + lj < p.H && loff != OOB;
      pd_load_lds(drs, lds0 + slot * W3_SLOT, in ? loff + base : OOB, 0);
    }
  };
  // after this lane's load of a stage has landed (see the kernel above): zeros over the repeated positions of the
  // input cell it loaded; IMG: zeros over the positions past the row in its input cell, and the cell at the very end
  // of its tensor, which was loaded as zeros, is filled in with plain loads
  const bool any_fix = IMG ? p.keep < 8 : (ldx && p.dup != 0);      // (the same for all lanes of a wave)
  const int my_cell = (ldx ? XRING : DRING) + lblk * 1024 + lane * 16;
  auto fix_tail = [&](int slot, int img) __attribute__((always_inline)) {
    char* cellp = wd_lds + my_cell + slot * W3_SLOT;
    if (IMG) {
      if (cell_ok) {
        uint16_t* q = reinterpret_cast<uint16_t*>(cellp);
        const int o = loff + img * (ldx ? p.C : p.K) * P * 2;
        if ((unsigned)o + 16u > (ldx ? p.x_bytes : p.dy_bytes)) {
          const uint16_t* src = reinterpret_cast<const uint16_t*>(ldx ? x : dy);
          for (int e = 0; e < p.keep; ++e) q[e] = src[(o >> 1) + e];
        }
        if (ldx)
          for (int e = p.keep; e < 8; ++e) q[e] = 0;
      }
      return;
    }
    if (lcq == p.ncell - 1) {
      int d = p.dup, at = 0;
      if (d >= 4) {
        *reinterpret_cast<uintx2_t*>(cellp) = uintx2_t{0u, 0u};
        d -= 4;
        at = 8;
      }
      if (d >= 2) {
        *reinterpret_cast<uint32_t*>(cellp + at) = 0u;
        d -= 2;
        at += 4;
      }
      if (d) *reinterpret_cast<uint16_t*>(cellp + at) = 0;
    }
  };

  // ---- the two shifted copies of a dy row: the 256 threads of a half make one cell each, (row, cell) = (idx / 8, idx % 8).
  // D_0 = positions + 1 (the element after the cell comes from the next cell, zero past the row), D_2 = positions - 1.
  int sh_cell, sh_nx, sh_pv;      // LDS offsets: the thread's cell in dy slot 0, the element after it, the one before
  uint32_t sh_mask[4];      // IMG: the positions of the cell that belong to its row
  bool sh_has_nx, sh_has_pv;
  {
    const int idx = tid & 255;
    const int r = idx >> 3, c = idx & 7, sw = r & 7;
    const int cq = GRP ? c % CPR : c;
    const bool in = IMG ? c < p.H : cq < p.ncell;
    const int pos = cq == p.ncell - 1 ? p.W - 8 : 8 * cq;
    const int cn = min(c + 1, 7), start = cq + 1 == p.ncell - 1 ? p.W - 8 : 8 * (cq + 1);
    const int cp = max(c - 1, 0);
    sh_has_nx = !IMG && in && pos + 8 < p.W;
    sh_has_pv = !IMG && in && pos > 0;
    sh_cell = DRING + r * 128 + ((c ^ sw) << 4);
    sh_nx = DRING + r * 128 + ((cn ^ sw) << 4) + (sh_has_nx ? 2 * (pos + 8 - start) : 0);
    sh_pv = DRING + r * 128 + ((cp ^ sw) << 4) + (sh_has_pv ? 2 * (pos - 1 - 8 * (cq - 1)) : 0);
    const unsigned keep = IMG ? (unsigned)p.keep : 8u;
#pragma unroll
    for (int k = 0; k < 4; ++k) sh_mask[k] = (2u * k < keep ? 0xffffu : 0u) | (2u * k + 1 < keep ? 0xffff0000u : 0u);
  }
  uintx4_t sh_v;
  uint32_t sh_a, sh_b;
  auto shift_reads = [&](int ds_slot) __attribute__((always_inline)) {
    sh_v = *(const lu4*)(L + sh_cell + ds_slot * W3_SLOT);
    sh_a = *(const lu16*)(L + sh_nx + ds_slot * W3_SLOT);
    sh_b = *(const lu16*)(L + sh_pv + ds_slot * W3_SLOT);
  };
  auto shift_writes = [&](int buf) __attribute__((always_inline)) {
    lchar* o = L + sh_cell + (SHIFT - DRING) + buf * 2 * W3_SLOT;
    uintx4_t v = sh_v;
    if (IMG) v = uintx4_t{v.x & sh_mask[0], v.y & sh_mask[1], v.z & sh_mask[2], v.w & sh_mask[3]};
    const uint32_t nx = sh_has_nx ? sh_a : 0u, pv = sh_has_pv ? sh_b : 0u;
    *(lu4*)o =
        uintx4_t{__builtin_amdgcn_alignbit(v.y, v.x, 16), __builtin_amdgcn_alignbit(v.z, v.y, 16),
                 __builtin_amdgcn_alignbit(v.w, v.z, 16), __builtin_amdgcn_alignbit(nx, v.w, 16)};
    *(lu4*)(o + W3_SLOT) =
        uintx4_t{__builtin_amdgcn_alignbit(v.x, pv << 16, 16), __builtin_amdgcn_alignbit(v.y, v.x, 16),
                 __builtin_amdgcn_alignbit(v.z, v.y, 16), __builtin_amdgcn_alignbit(v.w, v.z, 16)};
  };

  // ---- fragments: lane -> row fr of the block, k-octet fh of the wave's step
  const int cellf = 2 * kstep + fh;                 // the lane's cell of a row of 8
  const int fa_d = DRING + fr * 128 + ((cellf ^ (fr & 7)) * 16);      // LDS offsets: dy row of slot 0
  const int fa_s = fa_d + (SHIFT - DRING);                             // D_0 of buffer 0 (D_2: + W3_SLOT)
  int fb_p[3];                              // input rows of tap row kh in slot 0 ...
  bool bnext[3];                                    // ... of the stage itself or (groups of rows) of the next stage
#pragma unroll
  for (int kh = 0; kh < 3; ++kh) {
    bnext[kh] = false;
    int cell = cellf;
    if (GRP) {
      const int rho = cellf / CPR + kh;
      bnext[kh] = __builtin_amdgcn_readfirstlane(rho >= G ? 1 : 0) != 0;
      cell = (rho % G) * CPR + cellf % CPR;
    } else if (IMG) {
      cell = (cellf + kh - 1) & 7;
    }
    fb_p[kh] = XRING + fr * 128 + ((cell ^ (fr & 7)) * 16);
  }
  // bias gradient: the lane's eight positions as ones, zeros where the row's last cell repeats positions, where a
  // cell lies past the row and (IMG) where its positions belong to the next row
  const bool do_db = p.want_db && ctile == 0;
  bf16x8 ones;
  {
    const int cq = GRP ? cellf % CPR : cellf;
    const bool in = IMG ? cellf < p.H : cq < p.ncell;
    const int skip = !in ? 8 : (!IMG && cq == p.ncell - 1 ? p.dup : 0), keep = IMG ? p.keep : 8;
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      w[k] = ((2 * k >= skip && 2 * k < keep) ? (Lo16<E>::ONE2 & 0xffffu) : 0u) | ((2 * k + 1 >= skip && 2 * k + 1 < keep) ? (Lo16<E>::ONE2 & 0xffff0000u) : 0u);
    ones = __builtin_bit_cast(bf16x8, uintx4_t{w[0], w[1], w[2], w[3]});
  }
  floatx16 acc[3][3], accb;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    accb[r] = 0.f;
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int b = 0; b < 3; ++b) acc[a][b][r] = 0.f;
  }

  auto finish = [&]() __attribute__((always_inline)) {
    // element r of a wave's tile: result channel m0 + (r/4)*8 + fh*4 + r%4, input channel c0 + fr.  The eight waves'
    // tiles are added through LDS three taps (one kh) at a time: every wave parks its three tiles as 16-byte cells
    // [wave][kw][r / 4][lane], then thread `cell` adds the eight copies of its cells in wave order and stores.
    float* o = out + (size_t)split * ((size_t)p.E + p.K);
    const size_t KC = (size_t)p.K * p.C;
    static_assert(W3_LDS >= 8 * 3 * 4 * 64 * 16, "the parked accumulators fit");
    uintx4_t* park = reinterpret_cast<uintx4_t*>(wd_lds);
  #pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
      __syncthreads();
  #pragma unroll
      for (int kw = 0; kw < 3; ++kw)
  #pragma unroll
        for (int q = 0; q < 4; ++q)
          park[((wave * 3 + kw) * 4 + q) * 64 + lane] =
              uintx4_t{__float_as_uint(acc[kh][kw][4 * q]), __float_as_uint(acc[kh][kw][4 * q + 1]),
                       __float_as_uint(acc[kh][kw][4 * q + 2]), __float_as_uint(acc[kh][kw][4 * q + 3])};
      __syncthreads();
  #pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int cell = tid + 512 * i;
        if (cell < 768) {
          uintx4_t v[8];
  #pragma unroll
          for (int w = 0; w < 8; ++w) v[w] = park[w * 768 + cell];
          float sum[4];
  #pragma unroll
          for (int k = 0; k < 4; ++k) {
            float t = __uint_as_float(v[0][k]);
  #pragma unroll
            for (int w = 1; w < 8; ++w) t += __uint_as_float(v[w][k]);
            sum[k] = t;
          }
          const int kw = cell >> 8, q = (cell >> 6) & 3, ln = cell & 63;
          const int tap = kh * 3 + kw, c = c0 + (ln & 31);
  #pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int m = m0 + q * 8 + (ln >> 5) * 4 + k;
            o[tap * KC + (size_t)m * p.C + c] = sum[k];
          }
        }
      }
    }
    if (do_db) {
      // every column of a wave's bias tile holds the same 32 sums: column 0 (lanes 0 and 32) goes through LDS as
      // [wave][result channel], and the eight waves' sums are added in wave order
      float* sums = reinterpret_cast<float*>(wd_lds);
      __syncthreads();
      if (fr == 0) {
  #pragma unroll
        for (int r = 0; r < 16; ++r) sums[wave * 32 + (r >> 2) * 8 + fh * 4 + (r & 3)] = accb[r];
      }
      __syncthreads();
      if (tid < W3_T) {
        float t = sums[tid];
        for (int w = 1; w < 8; ++w) t += sums[w * 32 + tid];
        o[p.E + m0 + tid] = t;
      }
    }
  };

  if (nstages > 0) {
    // every wave issues one load per stage; stages 0 .. D + 1 before the loop
#pragma unroll
    for (int st = 0; st < W3_D + 2; ++st)
      if (st < nst2) issue(st, st);
    // The slots of the input ring that these loads do not fill start as zeros: the first stages take "the rows of the
    // stages before them" from the last two slots, and the last stage of groups of rows takes the rows below it from
    // the slot of a stage that does not exist.  Their dy rows are zeros, but zero times whatever LDS held is not
    // always zero.  (Slots that have been loaded once hold rows of the tensor from then on.)
    {
      typedef __attribute__((address_space(3))) uintx4_t lu4z;
      const int first = min(nst2, W3_D + 2);
      lu4z* z = (lu4z*)(wd_lds + XRING + first * W3_SLOT);
      for (int i = tid; i < (W3_NS - first) * (W3_SLOT / 16); i += 512) z[i] = uintx4_t{0u, 0u, 0u, 0u};
    }
    if (W3_D + 2 <= nst2) W3_WAIT_VM(W3_D - 2);        // stages 4 .. D + 1 may be outstanding: 0 .. 3 have landed
    else W3_WAIT_VM(0);
    if (any_fix) {
#pragma unroll
      for (int st = 0; st < 4; ++st)
        if (st < nstages) fix_tail(st, row_begin + st);
    }
    const int niter = nst2 >> 1;
    // Compiled once per half: this wave's stages are s = 2u + HALF.
    auto run = [&](auto half_c) __attribute__((always_inline)) {
      constexpr int HALF = decltype(half_c)::value;
      bf16x8 fa[3], fb[3];
      // fragments of the stage in ring slot SL (its shifted copies in buffer SL % 4): its dy row (D_1), D_0, D_2 and its
      // three input rows.  Ring of single rows (G == 1): the stage's own slot holds row oh + 1, the two slots before
      // it rows oh and oh - 1.
      auto load_fa = [&](auto sl_c) __attribute__((always_inline)) {
        constexpr int SL = decltype(sl_c)::value;
        fa[0] = __builtin_bit_cast(bf16x8, *(const lu4*)(L + fa_s + (SL & 3) * 2 * W3_SLOT));
        fa[1] = __builtin_bit_cast(bf16x8, *(const lu4*)(L + fa_d + SL * W3_SLOT));
        fa[2] = __builtin_bit_cast(bf16x8, *(const lu4*)(L + fa_s + ((SL & 3) * 2 + 1) * W3_SLOT));
      };
      auto load_fb = [&](auto sl_c, auto kh_c) __attribute__((always_inline)) {
        constexpr int SL = decltype(sl_c)::value, KH = decltype(kh_c)::value;
        constexpr int NEXT = (SL + 1) % W3_NS, PREV = (SL + W3_NS - 1) % W3_NS, PREV2 = (SL + W3_NS - 2) % W3_NS;
        const int slot = GRP ? (bnext[KH] ? NEXT : SL) : IMG ? SL : (KH == 2 ? SL : KH == 1 ? PREV : PREV2);
        fb[KH] = __builtin_bit_cast(bf16x8, *(const lu4*)(L + fb_p[KH] + slot * W3_SLOT));
      };
      using I0 = std::integral_constant<int, 0>;
      using I1 = std::integral_constant<int, 1>;
      using I2 = std::integral_constant<int, 2>;
      {
        // the shifted copies of stages 0 .. 3 (half h: stages h and 2 + h), then this wave's fragments of its first stage
        __syncthreads();
        shift_reads(HALF);
        shift_writes(HALF);
        if (2 + HALF < nst2) {
          shift_reads(2 + HALF);
          shift_writes(2 + HALF);
        }
        __syncthreads();
        load_fa(std::integral_constant<int, HALF>{});
        load_fb(std::integral_constant<int, HALF>{}, I0{});
        load_fb(std::integral_constant<int, HALF>{}, I1{});
        load_fb(std::integral_constant<int, HALF>{}, I2{});
      }
      // one iteration; u = PH (mod W3_NS / 2), so stage 2u + HALF + k lives in slot (2 PH + HALF + k) % W3_NS
      auto body = [&](auto ph_c, const int u) __attribute__((always_inline)) {
        constexpr int PH = decltype(ph_c)::value;
        constexpr int S2 = (2 * PH + HALF + 2) % W3_NS, S4 = (2 * PH + HALF + 4) % W3_NS;      // slots of stages s + 2, s + 4
        constexpr int F4 = (2 * PH + 4) % W3_NS, F5 = (2 * PH + 5) % W3_NS;                    // of stages 2u + 4, 2u + 5
        constexpr int L0 = (2 * PH + 2 + W3_D) % W3_NS, L1 = (2 * PH + 3 + W3_D) % W3_NS;      // of the stages to load
        const int sl = 2 * u + 2 + W3_D;
        const bool more4 = 2 * u + 4 < nst2, morel = sl < nst2;
        if (more4) {
          if (2 * u + 2 + W3_D <= nst2) W3_WAIT_VM(W3_D - 4);   // stages 2u + 6 .. 2u + 1 + D may be outstanding
          else W3_WAIT_VM(0);
          if (any_fix) {
            fix_tail(F4, row_begin + 2 * u + 4);
            if (2 * u + 5 < nstages) fix_tail(F5, row_begin + 2 * u + 5);       // (not the stage of zeros that pads an odd count)
          }
        }
        __syncthreads();
        if (morel) {
          if ((sl & 63) == 0) fill_table(sl);      // (sl is even: a pair of stages never straddles two tables)
          issue(sl, L0);
          issue(sl + 1, L1);
        }
        // (past the last stages these read and write slots that nobody reads any more)
        shift_reads(S4);
        // the products of stage s; each fragment register is refilled with stage s + 2's as soon as its last reader has issued
        {
#pragma unroll
          for (int kw = 0; kw < 3; ++kw) acc[0][kw] = Lo16<E>::mma32(fa[kw], fb[0], acc[0][kw]);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_fb(std::integral_constant<int, S2>{}, I0{});
        __builtin_amdgcn_sched_barrier(0);
        {
#pragma unroll
          for (int kw = 0; kw < 3; ++kw) acc[1][kw] = Lo16<E>::mma32(fa[kw], fb[1], acc[1][kw]);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_fb(std::integral_constant<int, S2>{}, I1{});
        shift_writes(S4 & 3);
        __builtin_amdgcn_sched_barrier(0);
        {
#pragma unroll
          for (int kw = 0; kw < 3; ++kw) acc[2][kw] = Lo16<E>::mma32(fa[kw], fb[2], acc[2][kw]);
          if (do_db) accb = Lo16<E>::mma32(fa[1], ones, accb);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_fb(std::integral_constant<int, S2>{}, I2{});
        load_fa(std::integral_constant<int, S2>{});
      };
      body(std::integral_constant<int, 0>{}, 0);
      // (one way out of the loop: the accumulators have one live range)
#pragma unroll 1
      for (int u = 1; u < niter; u += 8) {
        body(std::integral_constant<int, 1>{}, u);
        if (u + 1 < niter) {
          body(std::integral_constant<int, 2>{}, u + 1);
          if (u + 2 < niter) {
            body(std::integral_constant<int, 3>{}, u + 2);
            if (u + 3 < niter) {
              body(std::integral_constant<int, 4>{}, u + 3);
              if (u + 4 < niter) {
                body(std::integral_constant<int, 5>{}, u + 4);
                if (u + 5 < niter) {
                  body(std::integral_constant<int, 6>{}, u + 5);
                  if (u + 6 < niter) {
                    body(std::integral_constant<int, 7>{}, u + 6);
                    if (u + 7 < niter) body(std::integral_constant<int, 0>{}, u + 7);
                  }
                }
              }
            }
          }
        }
      }
      finish();
    };
    static_assert(W3_NS == 16, "the loop above is unrolled over the eight positions of the rings");
    // (each branch ends in the final exchange: the two copies of the loop never meet)
    if (half == 0) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});
  } else {
    finish();
  }
}

// part[split][tap][K][C] (+ [K] bias sums) -> dw[K][C][tap], db[K]; the splits are added in a fixed order.
// A workgroup of 16 x 16 threads owns 64 consecutive elements (16 threads x 4), its 16 rows of threads share the
// splits: small workgroups, so that a gradient of 36864 elements still spreads over every CU.
constexpr int WD_RTX = 16, WD_RTY = 16;
__global__ void __launch_bounds__(WD_RTX * WD_RTY)
wgrad_taps_reduce_kernel(const float* __restrict__ part, int nsplit, int K, int C, int want_db,
                         float* __restrict__ dw, float* __restrict__ db) {
  __shared__ float4 red[WD_RTY][WD_RTX];
  const int tx = threadIdx.x % WD_RTX, ty = threadIdx.x / WD_RTX;
  const int E = K * C * 9;
  const int e = (blockIdx.x * WD_RTX + tx) * 4;
  const int total = E + (want_db ? K : 0);
  const size_t stride = (size_t)E + K;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (e < total) {
    for (int s0 = ty; s0 < nsplit; s0 += 8 * WD_RTY) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int s = s0 + u * WD_RTY;
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
    for (int k = 1; k < WD_RTY; ++k) {
      const float4 t = red[k][tx];
      r.x += t.x; r.y += t.y; r.z += t.z; r.w += t.w;
    }
    const float rv[4] = {r.x, r.y, r.z, r.w};
    if (e < E) {
      // four consecutive input channels of one (tap, result channel)
      const int KC = K * C;
      const int tap = e / KC, mc = e - tap * KC;
#pragma unroll
      for (int k = 0; k < 4; ++k) dw[(size_t)(mc + k) * 9 + tap] = rv[k];
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) db[e - E + k] = rv[k];
    }
  }
}

// The same reduction for few splits of a large gradient (512 x 512 filters over 7x7 planes: 4 splits of 9.4 MB): a
// thread owns four input channels of a result channel, adds its nine taps over the splits in order and writes the
// 36 values as they lie in dw (the kernel above would write them as 4-byte pieces 36 bytes apart).
__global__ void __launch_bounds__(64)
wgrad_taps_gather_reduce_kernel(const float* __restrict__ part, int nsplit, int K, int C, int want_db,
                                float* __restrict__ dw, float* __restrict__ db) {
  const int KC = K * C, E = KC * 9;
  const size_t stride = (size_t)E + K;
  const int item = blockIdx.x * 64 + threadIdx.x;       // (result channel, group of four input channels)
  if (item * 4 < KC) {
    float4 acc[9];
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) acc[tap] = make_float4(0.f, 0.f, 0.f, 0.f);
    // two splits' loads in flight at a time (18 of 16 bytes per thread)
    for (int sp = 0; sp < nsplit; sp += 2) {
      float4 v[2][9];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int tap = 0; tap < 9; ++tap)
          v[u][tap] = sp + u < nsplit
                          ? *reinterpret_cast<const float4*>(part + (size_t)(sp + u) * stride + (size_t)tap * KC + (size_t)item * 4)
                          : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) {
          acc[tap].x += v[u][tap].x; acc[tap].y += v[u][tap].y; acc[tap].z += v[u][tap].z; acc[tap].w += v[u][tap].w;
        }
    }
    // dw[(m * C + c) * 9 + tap], c = 4 consecutive channels: 36 consecutive values
    float o[36];
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      o[tap] = acc[tap].x;
      o[9 + tap] = acc[tap].y;
      o[18 + tap] = acc[tap].z;
      o[27 + tap] = acc[tap].w;
    }
    float4* dst = reinterpret_cast<float4*>(dw + (size_t)item * 36);
#pragma unroll
    for (int q = 0; q < 9; ++q) dst[q] = make_float4(o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]);
  }
  if (want_db && item < K) {
    float t = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) t += part[(size_t)sp * stride + E + item];
    db[item] = t;
  }
}

// T: tile side (64: wgrad_dma_kernel, 32: wgrad_dma32_kernel)
bool wd_plan(const ConvGeom& g, WdParams* p, int T) {
  if (!(g.KH == 3 && g.KW == 3 && g.sy == 1 && g.sx == 1 && g.py == 1 && g.px == 1 && g.dly == 1 && g.dlx == 1 &&
        g.groups == 1 && g.OH == g.H && g.OW == g.W))
    return false;
  const bool img = g.H <= 7 && g.W <= 8 && g.W >= 2;       // whole images per stage
  if (g.C % T != 0 || g.K % T != 0 || (!img && g.W < 8) || g.W > 64) return false;
  const long long xb = (long long)g.N * g.C * g.H * g.W * 2, db = (long long)g.N * g.K * g.H * g.W * 2;
  if (xb >= (1ll << 31) || db >= (1ll << 31)) return false;
  p->N = g.N; p->C = g.C; p->K = g.K; p->H = g.H; p->W = g.W;
  p->ncell = img ? 1 : (g.W + 7) / 8;
  p->dup = img ? 0 : 8 * p->ncell - g.W;
  p->keep = img ? g.W : 8;
  p->img = img;
  p->G = img ? 0 : g.W <= 16 ? 4 : g.W <= 32 ? 2 : 1;
  p->x_bytes = (unsigned)xb;
  p->dy_bytes = (unsigned)db;
  p->ctiles = g.C / T;
  p->mtiles = g.K / T;
  p->total_rows = img ? g.N : g.N * ((g.H + (p->G - 1)) / (p->G > 1 ? p->G : 1));        // stages: images, rows or groups of rows
  p->E = g.K * g.C * 9;
  const long long tiles = (long long)p->ctiles * p->mtiles;
  if (tiles > 65535) return false;
  // one workgroup per CU; every slice writes and re-reads the whole gradient
  long long ns = mfma_num_cus() / tiles;
  if (ns > p->total_rows / 4) ns = p->total_rows / 4;     // at least four rows per slice
  if (ns < 1) ns = 1;
  p->rps = (int)((p->total_rows + ns - 1) / ns);
  p->nsplit = (p->total_rows + p->rps - 1) / p->rps;
  return true;
}

// Which tile a geometry gets.  32 x 32 tiles quarter the partial gradients that the slices write and the reduce
// kernel reads back, and double the fetches of every operand row (from L2 when the tiles of a slice run together).
// Measured on the 3x3 layers of ResNet-50 (us per call with the bias gradient, 32 x 32 against 64 x 64 tiles): at batch
// 32 every layer gains (56x56 23.2 / 27.0, 28x28 25.5 / 28.9, 14x14 31.3 / 34.9, 7x7 31.0 / 36.2: the slices of 64 x 64
// tiles are 7 or 8 stages long there, mostly start-up); at batch 64 the first layer gains (30.3 / 34.5) and the
// others, whose operands are then fetched 4 to 16 times, lose or draw (36.8 / 35.2, 46.0 / 43.2, 42.6 / 42.3).
bool wd_use32(const ConvGeom& g, WdParams* p) {
  if (options().conv_skip & Options::SKIP_WD32) return false;
  if (!wd_plan(g, p, W3_T)) return false;
  WdParams q{};
  if (!wd_plan(g, &q, WD_T)) return true;               // channel counts that only the small tiles divide
  return p->ctiles * p->mtiles <= 4 || q.rps < 12;
}

size_t wd_ws_bytes(const WdParams& p) { return (size_t)p.nsplit * ((size_t)p.E + p.K) * sizeof(float); }

}  // namespace

size_t mfma_wgrad_dma16_ws(const ConvGeom& g) {
  // the larger of the two plans, so that either kernel can run whatever the switches say at the time of the call
  WdParams p{}, q{};
  const size_t a = wd_plan(g, &p, WD_T) ? wd_ws_bytes(p) : 0, b = wd_plan(g, &q, W3_T) ? wd_ws_bytes(q) : 0;
  return a > b ? a : b;
}

// -1 when the shape is not this kernel's
template <typename E>
static int wgrad_dma16_run(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws, size_t ws_bytes,
                           hipStream_t s, int tile) {
  WdParams p{};
  if (!dw) return -1;
  const bool t32 = tile == 0 ? wd_use32(g, &p) : tile == W3_T && wd_plan(g, &p, W3_T);
  if (tile == W3_T && !t32) return -1;
  if (!t32 && !wd_plan(g, &p, WD_T)) return -1;
  if (!ws || ws_bytes < wd_ws_bytes(p) || reinterpret_cast<uintptr_t>(ws) % 16 != 0) return -1;   // (the reduce kernels read 16 bytes at a time)
  p.want_db = db != nullptr;
  float* part = static_cast<float*>(ws);
  const E* xp = static_cast<const E*>(x);
  const E* dyp = static_cast<const E*>(dy);
  if (t32) {
    const unsigned wgs = (unsigned)(p.nsplit * p.ctiles * p.mtiles);
    const dim3 grid((wgs + 7) / 8 * 8);
#define W3_LAUNCH(GR)                                                                                      \
  {                                                                                                        \
    if (!mfma_allow_lds(reinterpret_cast<const void*>(wgrad_dma32_kernel<E, GR>), W3_LDS)) return -1;      \
    hipLaunchKernelGGL((wgrad_dma32_kernel<E, GR>), grid, dim3(512), W3_LDS, s, p, xp, dyp, part);         \
  }
    if (p.G == 0) W3_LAUNCH(0)
    else if (p.G == 1) W3_LAUNCH(1)
    else if (p.G == 2) W3_LAUNCH(2)
    else W3_LAUNCH(4)
#undef W3_LAUNCH
  } else {
  // measured on the ResNet-50 layers at batch 64 against the kernel with register staging: 56x56 planes 36 against
  // 42 us, 28x28 (two rows per stage) 36 against 40, 14x14 (four rows) 43 against 52, 7x7 (whole images) 47 against 94
  // through gathered taps
  const dim3 grid((unsigned)p.nsplit, (unsigned)(p.ctiles * p.mtiles));
#define WD_LAUNCH(NK, GR)                                                                                      \
  {                                                                                                            \
    if (!mfma_allow_lds(reinterpret_cast<const void*>(wgrad_dma_kernel<E, NK, GR>), WD_LDS)) return -1;        \
    hipLaunchKernelGGL((wgrad_dma_kernel<E, NK, GR>), grid, dim3(64 * NW), WD_LDS, s, p, xp, dyp, part);       \
  }
  if (p.G == 0) WD_LAUNCH(4, 0)
  else if (p.G == 1) WD_LAUNCH(4, 1)
  else if (p.G == 2) WD_LAUNCH(4, 2)
  else WD_LAUNCH(4, 4)
#undef WD_LAUNCH
  }
  const int total = p.E + (p.want_db ? p.K : 0);
  // (a thread of it walks all splits and taps: it needs a gradient large enough for a few waves per CU;
  // 256 x 256 filters in 16 splits: 40 us against 7 us of the kernel below)
  if (p.nsplit <= 8 && p.K * p.C >= 256 * 512 && reinterpret_cast<uintptr_t>(dw) % 16 == 0) {
    hipLaunchKernelGGL(wgrad_taps_gather_reduce_kernel, dim3((p.K * p.C / 4 + 63) / 64), dim3(64), 0, s, part, p.nsplit,
                       p.K, p.C, p.want_db, dw, db);
    return check_launch("conv2d_bwd_filter 3x3 (bf16 mfma, direct-to-LDS)");
  }
  hipLaunchKernelGGL(wgrad_taps_reduce_kernel, dim3((total + 4 * WD_RTX - 1) / (4 * WD_RTX)), dim3(WD_RTX * WD_RTY), 0, s, part, p.nsplit, p.K,
                     p.C, p.want_db, dw, db);
  return check_launch("conv2d_bwd_filter 3x3 (bf16 mfma, direct-to-LDS)");
}

int mfma_wgrad_dma16(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws, size_t ws_bytes,
                     hipStream_t s, int tile, int dtype) {
  return by_lo16(dtype, [&](auto* e_) { return wgrad_dma16_run<FLHIP_T_OF(e_)>(g, x, dy, dw, db, ws, ws_bytes, s, tile); });
}

}  // namespace flhip
