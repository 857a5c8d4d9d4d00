// 1x1 stride-1 convolutions in bf16 storage, forward and backward-data, on
// v_mfma_f32_32x32x16_bf16 with operand tiles that the memory pipeline itself copies into
// LDS (buffer loads with the LDS modifier, 16 bytes per lane): no wave spends vector
// instructions on loading, all four waves multiply, and up to seven stages of 32 contraction
// channels are in flight per workgroup.  Made for the layers whose planes are small
// (14x14, 7x7): few workgroups, long contractions, where a stage must not cost a trip to
// memory and a pass over a loader's registers.
//
//   forward        y[m][q]  = sum_c w[m][c]  x[c][q]  (+ bias[m])
//   backward-data  dx[c][q] = sum_m w[m][c] dy[m][q]
//
// Positions: a plane of P positions is cut into cells of 8 (16 bytes); the last cell of a
// plane ENDS at the plane's last position (it starts at P - 8 and repeats positions of the
// cell before it when P is not a multiple of 8), so no cell reaches into the next row of
// the tensor and every cell is loaded and stored whole.  Cells are numbered over the batch
// (image * cells-per-plane + cell); a workgroup owns 16 of them (128 position slots) x 128
// result channels.  Repeated positions are computed twice from the same operands in the same
// order and stored twice with the same value.
//
// LDS ring of 4 or 8 stages.  The loads into LDS are written as inline assembly: for the builtin
// the compiler inserts its own waits in front of the transposing reads, and those wait for
// every load in flight, which would leave nothing in flight.  The kernel counts its loads
// itself (s_waitcnt vmcnt(n) before the barrier that publishes a stage).
//   source   [32 channels][128 slots], pitch 288 bytes: as in memory, fetched by lanes as
//            8 channels of one position with transposing reads (ds_read_b64_tr_b16)
//   weights  forward [128 result channels][32 contraction], pitch 80 bytes, 16-byte reads;
//            backward-data [32 contraction][128 result channels] like the source
// A load instruction fills 64 consecutive 16-byte cells of LDS, one per lane; the lanes that
// fall on the unused cells of a pitch, on result channels past the last or on cells past the
// batch pass an offset beyond the tensor (the range check of the buffer descriptor then
// returns zeros without a fetch); those rows only reach results that are not stored.
// Positions are the rows of the instruction tile: a lane holds 4 consecutive positions of a
// result channel; results go through LDS and leave as whole cells.
#include <algorithm>

#include "conv2d_mfma.h"
#include "lds_direct.h"

namespace flhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short shortx4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4_t* lds_tr_t;

constexpr int PD_KC = 32;                          // contraction channels per stage
constexpr int PD_BM = 128;                         // result channels per workgroup (64 for grids that would leave CUs idle)
constexpr int PD_CELLS = 16;                       // position cells per workgroup
constexpr int PD_XC = PD_CELLS + 2;                // cells per row of a [32][128] tile
constexpr int PD_XP = PD_XC * 8;                   // the same in elements
constexpr int PD_WC = 5;                           // cells per row of the forward weight tile (4 + 1)
constexpr int PD_WP = PD_WC * 8;
constexpr int PD_XCELLS = PD_KC * PD_XC;           // 576 = 9 load instructions
// weight tile of BM result channels: forward [BM][32] (10 / 5 load instructions), backward-data [32][BM] with two
// unused cells per row (9 / 5 load instructions)
constexpr int pd_wcells(bool bwd, int bm) { return bwd ? PD_KC * (bm / 8 + 2) : bm * PD_WC; }
constexpr int pd_stage(int bm) { return PD_XCELLS + bm * PD_WC; }   // cells per stage (the forward tile is the larger one)
// Stages in the ring, NS: 4 (76 KiB, two workgroups per CU: one multiplies while the other starts
// or stores) for grids that fill the chip more than once, 8 (152 KiB) for grids of at most one
// workgroup per CU, where only the depth of the ring hides the way to memory.  Loads run
// NS - 2 stages ahead of the stage being read.
constexpr int PD_YP = 8 * PD_CELLS + 8;            // result staging pitch (elements)

struct PwdParams {
  int Kc, Mo;           // contraction channels, result channels
  int P, Pc;            // positions and cells per plane
  int ncells;           // cells over the batch
  int nstages, mtiles, ctiles;
  unsigned src_bytes, w_bytes, dst_bytes;
  const float* pos_bias;   // one value per position, added to every result channel (matrix products: one image), or null
  // matrix products with the contraction cut into slices (blockIdx.y): sps stages per slice (nstages: one slice), and
  // where slice k leaves its fp32 partial product, [result channel][position], Mo * P floats per slice (null: one slice,
  // results in the element type at dst)
  int sps;
  float* part;
};

// rows r0 .. r0+7 of column c0 + s of a 16-bit tile stored [row][column] (see the 1x1 kernels
// with register staging for the lane map of the transposing read)
__device__ __forceinline__ bf16x8 pd_gather8(const uint16_t* tile, int pitch, int r0, int c0, int s) {
  const uint16_t* t = tile + (r0 + (s >> 2)) * pitch + c0 + 4 * (s & 3);
  const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)t);
  const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_t)(t + 4 * pitch));
  const uintx2_t l = __builtin_bit_cast(uintx2_t, lo), h = __builtin_bit_cast(uintx2_t, hi);
  const uintx4_t v = {l.x, l.y, h.x, h.y};
  return __builtin_bit_cast(bf16x8, v);
}

// two packed elements plus two packed elements, each sum rounded once
template <typename E>
__device__ __forceinline__ uint32_t pd_add_x2(uint32_t a, uint32_t b) {
  return Lo16<E>::pack(Lo16<E>::lo(a) + Lo16<E>::lo(b), Lo16<E>::hi(a) + Lo16<E>::hi(b));
}

// at most N of this wave's loads outstanding
template <int N>
__device__ __forceinline__ void pd_wait_loads() {
  static_assert(N == 0 || N == 3 || N == 4 || N == 6 || N == 8 || N == 15 || N == 18 || N == 20 || N == 24, "counts in use");
  if (N == 0) PD_WAIT_VM(0);
  if (N == 3) PD_WAIT_VM(3);
  if (N == 4) PD_WAIT_VM(4);
  if (N == 6) PD_WAIT_VM(6);
  if (N == 8) PD_WAIT_VM(8);
  if (N == 15) PD_WAIT_VM(15);
  if (N == 18) PD_WAIT_VM(18);
  if (N == 20) PD_WAIT_VM(20);
  if (N == 24) PD_WAIT_VM(24);
}

template <typename E, bool BWD, int PD_NS, int BM>
__global__ void __launch_bounds__(256, PD_NS == 4 ? 2 : 1)
pwd16_conv_kernel(PwdParams p, const E* __restrict__ src, const E* __restrict__ wgt,
                  const float* __restrict__ bias, E* __restrict__ dst, const E* __restrict__ addend) {
  static_assert(BM == 128 || BM == 64, "tile heights in use");
  constexpr int PD_D = PD_NS - 2;
  constexpr int PD_STAGE = pd_stage(BM);
  constexpr int WXC = BM / 8 + 2, WXP = WXC * 8;               // backward-data weight tile: cells / elements per row
  __shared__ __align__(16) uint4 ring[PD_NS * PD_STAGE];
  uint16_t* const ys = reinterpret_cast<uint16_t*>(ring);      // result staging, once the ring is done with
  static_assert(BM * PD_YP * 2 <= PD_NS * PD_STAGE * 16, "the staged results fit in the ring");
  constexpr int NXI = PD_XCELLS / 64, NWI = pd_wcells(BWD, BM) / 64, NI = NXI + NWI;
  static_assert(PD_XCELLS % 64 == 0 && pd_wcells(BWD, BM) % 64 == 0, "whole load instructions");
  static_assert(NI <= 20 && NI >= 12, "five load instructions per wave at most, three at least");
  constexpr int MINL = NI / 4;                                  // loads every wave issues per stage at least
  static_assert(PD_NS == 4 || PD_NS == 8, "the ring slot is the stage number modulo a power of two");

  // consecutive workgroups go to different XCDs: the channel tiles that share a source tile
  // run back to back on one XCD
  const int id = blockIdx.x, xcd = id & 7, seq = id >> 3;
  const int mtile = seq % p.mtiles, ctile = (seq / p.mtiles) * 8 + xcd;
  if (ctile >= p.ctiles) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m0 = mtile * BM, cell0 = ctile * PD_CELLS;
  const intx4_t xrs = pd_rsrc(src, p.src_bytes), wrs = pd_rsrc(wgt, p.w_bytes);

  // ---- load roles: instruction ii = wave + 4 n of a stage; lane -> LDS cell ii * 64 + lane.
  // Per instruction, the same for all lanes: descriptor, LDS offset, bytes to advance per stage.
  int voff[5], klim[5];      // klim: contraction channels from the lane's cell to the end of its row (forward weights)
  intx4_t lrs[5];
  int loff[5], lstep[5];
#pragma unroll
  for (int n = 0; n < 5; ++n) {
    const int ii = wave + 4 * n;
    const bool isx = ii < NXI;
    lrs[n] = isx ? xrs : wrs;
    loff[n] = (isx ? ii * 64 : PD_XCELLS + (ii - NXI) * 64) * 16;
    lstep[n] = isx ? PD_KC * 2 * p.P : BWD ? PD_KC * 2 * p.Mo : PD_KC * 2;
    voff[n] = (int)0x80000000;      // past every tensor: such a lane fetches nothing and its cell gets zeros
    klim[n] = 0x7fffffff;
    if (ii < NXI) {
      const int L = ii * 64 + lane, row = L / PD_XC, c = L - row * PD_XC;
      const int cell = cell0 + c;
      if (c < PD_CELLS && cell < p.ncells) {
        const int img = cell / p.Pc, j = cell - img * p.Pc;
        voff[n] = ((img * p.Kc + row) * p.P + min(8 * j, p.P - 8)) * 2;
      }
    } else if (ii < NI) {
      const int L = (ii - NXI) * 64 + lane;
      if (BWD) {
        const int row = L / WXC, c = L - row * WXC, mo = m0 + 8 * c;
        if (c < BM / 8 && mo < p.Mo) voff[n] = (row * p.Mo + mo) * 2;
      } else {
        const int m = L / PD_WC, c = L - m * PD_WC;
        if (c < 4 && m0 + m < p.Mo) voff[n] = ((m0 + m) * p.Kc + 8 * c) * 2;
        klim[n] = p.Kc - 8 * c;     // a last stage of fewer than 32 channels: the cells past the row's end fetch nothing
      }
    }
  }
  const bool fourth = wave + 12 < NI, fifth = wave + 16 < NI;
  const int sbeg = blockIdx.y * p.sps;      // this slice's first stage
  const int n = min(p.nstages - sbeg, p.sps), n2 = (n + 1) & ~1;
  // stages are multiplied in pairs: with an odd number the stage past the contraction fetches nothing and fills its
  // slot with zeros (both operands: it adds 0)
  auto issue = [&](int t, uint4* ring) {
    const unsigned base = (unsigned)reinterpret_cast<uintptr_t>((lds_void_t)ring);
    const bool live = t < n;
    const int tg = sbeg + t;
#pragma unroll
    for (int k = 0; k < 3; ++k)
      pd_load_lds(lrs[k], base + loff[k], (live && tg * PD_KC < klim[k]) ? voff[k] : (int)0x80000000, tg * lstep[k]);
    if (fourth) pd_load_lds(lrs[3], base + loff[3], (live && tg * PD_KC < klim[3]) ? voff[3] : (int)0x80000000, tg * lstep[3]);
    if (fifth) pd_load_lds(lrs[4], base + loff[4], (live && tg * PD_KC < klim[4]) ? voff[4] : (int)0x80000000, tg * lstep[4]);
  };

  // ---- fragments: 128 result channels: wave = (position half, channel half), 2 x 2 blocks of 32 x 32;
  // 64 result channels: wave = position quarter, 1 x 2 blocks
  constexpr int NA = BM == 128 ? 2 : 1;
  const int pos0 = BM == 128 ? (wave & 1) * 64 : wave * 32, mw0 = BM == 128 ? (wave >> 1) * 64 : 0;
  const int fh = lane >> 5, fq = (lane >> 4) & 1, fs = lane & 15, fr = lane & 31;
  bf16x8 fa[2][2][NA], fb[2][2][2];      // [register set][k-step of 16][block]
  floatx16 acc[NA][2];
#pragma unroll
  for (int i = 0; i < NA; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#define PD_READ(RING, SET)                                                                              \
  {                                                                                                     \
    const uint16_t* X_ = reinterpret_cast<const uint16_t*>(RING);                                       \
    const uint16_t* W_ = reinterpret_cast<const uint16_t*>(RING + PD_XCELLS);                           \
    _Pragma("unroll") for (int ks = 0; ks < 2; ++ks) {                                                  \
      _Pragma("unroll") for (int i = 0; i < NA; ++i)                                                    \
        fa[SET][ks][i] = pd_gather8(X_, PD_XP, ks * 16 + 8 * fh, pos0 + i * 32 + 16 * fq, fs);          \
      _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                     \
        fb[SET][ks][j] = BWD ? pd_gather8(W_, WXP, ks * 16 + 8 * fh, mw0 + j * 32 + 16 * fq, fs)        \
                             : __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(           \
                                   &W_[(mw0 + j * 32 + fr) * PD_WP + ks * 16 + 8 * fh]));               \
    }                                                                                                   \
  }
#define PD_MULT(SET)                                                                                    \
  _Pragma("unroll") for (int ks = 0; ks < 2; ++ks)                                                      \
    _Pragma("unroll") for (int i = 0; i < NA; ++i)                                                      \
      _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                     \
        acc[i][j] = Lo16<E>::mma32(fa[SET][ks][i], fb[SET][ks][j], acc[i][j]);

  // stages 0 .. D in flight, stage 0 in registers
#pragma unroll
  for (int st = 0; st <= PD_D; ++st)
    if (st < n2) issue(st, ring + st * PD_STAGE);
  if (PD_D < n2) pd_wait_loads<MINL * PD_D>();      // stages 1 .. D may be outstanding
  else pd_wait_loads<0>();
  __syncthreads();
  PD_READ(ring, 0)

  // iteration t: the stage t + 1 has landed for every wave (wait for this wave's loads, then the
  // barrier); the loads of stage t + 1 + D go to the slot whose fragments were multiplied in
  // iteration t - 1; the fragments of stage t + 1 are read while those of stage t are multiplied.
  // Only the wait and the loads depend on the stage number; the reads of one register set and the
  // matrix instructions on the other are one block of code without branches, which the scheduler
  // interleaves: with a branch on the stage number around them every wave waited for its reads
  // before its first matrix instruction, and reads and products took turns.
  constexpr int NREAD = (BWD ? 4 * NA + 8 : 4 * NA + 4), NMULT = 4 * NA;
#define PD_ITER(U)                                                                                  \
  {                                                                                                 \
    if (t0 + U + PD_D < n2) pd_wait_loads<MINL * (PD_D - 1)>();                                     \
    else pd_wait_loads<0>();                                                                        \
    __syncthreads();                                                                                \
    if (t0 + U + 1 + PD_D < n2) issue(t0 + U + 1 + PD_D, ring + ((s0 + U + 1 + PD_D) & (PD_NS - 1)) * PD_STAGE); \
    PD_READ((ring + ((s0 + U + 1) & (PD_NS - 1)) * PD_STAGE), (U + 1) % 2)                          \
    PD_MULT(U % 2)                                                                                  \
    _Pragma("unroll") for (int q = 0; q < NMULT; ++q) {                                             \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                            \
      __builtin_amdgcn_sched_group_barrier(0x100, (NREAD + NMULT - 1) / NMULT, 0);                  \
    }                                                                                               \
  }
  // two stages per trip (the register sets alternate); the ring slot is the stage number modulo the ring
  for (int t0 = 0; t0 < n2; t0 += 2) {
    const int s0 = t0 & (PD_NS - 1);
    PD_ITER(0) PD_ITER(1)
  }
#undef PD_ITER
#undef PD_MULT
#undef PD_READ

  if (p.part) {
    // a slice's partial product leaves in fp32 straight from the accumulators (one image): a lane's four consecutive
    // positions of a result channel; the positions a plane's last cell repeats are written twice with the same value
    float* const part = p.part + (size_t)blockIdx.y * p.Mo * p.P;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ch = m0 + mw0 + j * 32 + fr;
      if (ch >= p.Mo) continue;
#pragma unroll
      for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int cell = cell0 + (pos0 + i * 32) / 8 + g;
          if (cell >= p.ncells) continue;
          float* q = part + (size_t)ch * p.P + min(8 * cell, p.P - 8) + fh * 4;
#pragma unroll
          for (int e = 0; e < 4; ++e) q[e] = acc[i][j][4 * g + e];
        }
    }
    return;
  }
  __syncthreads();      // every wave has read its last fragments: the ring becomes the staging tile
  // ---- results: element r of block (i, j): slot pos0 + i*32 + (r/4)*8 + fh*4 + r%4 of channel
  // mw0 + j*32 + fr.  [channel][slot] in LDS, then whole cells to memory.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int ml = mw0 + j * 32 + fr;
    const float bv = (!BWD && bias && m0 + ml < p.Mo) ? bias[m0 + ml] : 0.f;
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (p.pos_bias) {      // one image: slot 8 c + e of the tile is position min(8 (cell0 + c), P - 8) + e
          const int cell = cell0 + (pos0 + i * 32) / 8 + g;
          if (cell < p.ncells) {
            const float* pb = p.pos_bias + min(8 * cell, p.P - 8) + fh * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * g + e] += pb[e];
          }
        }
        const uintx2_t o = {Lo16<E>::pack(acc[i][j][4 * g] + bv, acc[i][j][4 * g + 1] + bv),
                            Lo16<E>::pack(acc[i][j][4 * g + 2] + bv, acc[i][j][4 * g + 3] + bv)};
        *reinterpret_cast<uintx2_t*>(&ys[ml * PD_YP + pos0 + i * 32 + g * 8 + fh * 4]) = o;
      }
  }
  __syncthreads();
  {
    const int c = tid & 15, cell = cell0 + c;
    if (cell < p.ncells) {
      const int img = cell / p.Pc, j = cell - img * p.Pc;
      const int base = (img * p.Mo + m0) * p.P + min(8 * j, p.P - 8);
      const __amdgpu_buffer_rsrc_t drs = make_rsrc(dst, p.dst_bytes);
      const __amdgpu_buffer_rsrc_t ars = make_rsrc(addend ? addend : dst, p.dst_bytes);
      for (int ml = tid >> 4; ml < BM && m0 + ml < p.Mo; ml += 16) {
        uintx4_t v = *reinterpret_cast<const uintx4_t*>(&ys[ml * PD_YP + 8 * c]);
        const int off = (base + ml * p.P) * 2;
        if (addend) {
          const uintx4_t a = __builtin_amdgcn_raw_buffer_load_b128(ars, off, 0, 0);
          v = uintx4_t{pd_add_x2<E>(v.x, a.x), pd_add_x2<E>(v.y, a.y), pd_add_x2<E>(v.z, a.z),
                       pd_add_x2<E>(v.w, a.w)};
        }
        __builtin_amdgcn_raw_buffer_store_b128(v, drs, off, 0, 0);
      }
    }
  }
}

bool pwd16_applies(const ConvGeom& g, bool bwd) {
  if (!(g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1 && g.sy == 1 && g.sx == 1 &&
        g.OH == g.H && g.OW == g.W && g.C % 8 == 0 && g.K % 8 == 0))
    return false;
  const int kc = bwd ? g.K : g.C, mo = bwd ? g.C : g.K;
  if (kc % PD_KC != 0 || g.H * g.W < 8) return false;
  // measured on the ResNet-50 layers at batch 32 and 64: ahead of the kernels with register staging
  // on planes up to 28x28 (by 10 to 45 %), behind them on 56x56 planes (those layers run at the
  // speed of memory there, several workgroups per CU); a tile of 128 result channels wants more than 64.
  // FLHIP_PW16_PF set lifts the rule (tests, measurements).
  return options().pw16_pf != 0 || (g.H * g.W <= 1024 && mo > 64);
}

// slices of the contraction for a matrix product of ctiles x mtiles tiles over nstages stages: as many as it takes to
// give every CU a workgroup, at least eight stages each; *sps = stages per slice
int pwd16_slices(int ctiles, int mtiles, int nstages, int* sps, int cap = 32) {
  long long ns = mfma_num_cus() / std::max(1ll, (long long)ctiles * mtiles);
  if (ns > nstages / 8) ns = nstages / 8;
  if (ns > cap) ns = cap;
  if (ns < 1) ns = 1;
  *sps = (int)((nstages + ns - 1) / ns);
  return (*sps > 0) ? (nstages + *sps - 1) / *sps : 1;
}

// result channels per tile
int pwd16_bm(const PwdParams& p) {
  const int pf = options().pw16_pf;
  bool small = (long long)p.ctiles * ((p.Mo + PD_BM - 1) / PD_BM) <= mfma_num_cus() / 2;
  if (pf) small = pf == 2 || pf == 8;
  return small ? 64 : PD_BM;
}

// grid and kernel variant for a filled-in PwdParams (Kc, Mo, P, Pc, ncells, nstages, ctiles and the byte sizes)
// slices > 1 (matrix products): the contraction in that many slices at most, their fp32 partial products at p.part
template <typename E, bool BWD>
int pwd16_go(PwdParams p, const void* src, const void* w, const float* bias, void* dst, const void* addend,
             hipStream_t s, const char* what, int* slices = nullptr) {
  // tiles of 64 result channels when tiles of 128 would leave half of the CUs without a workgroup (7x7 planes
  // with 512 result channels at batch 64: 112 workgroups of 64 stages); the deep ring for grids of at most one
  // workgroup per CU.  FLHIP_PW16_PF = 1 / 4 forces the shallow / deep ring with tiles of 128, 2 / 8 with tiles of 64.
  const int cus = mfma_num_cus(), pf = options().pw16_pf;
  const int bm = pwd16_bm(p);
  const bool small = bm == 64;
  p.mtiles = (p.Mo + bm - 1) / bm;
  const long long grid = (long long)((p.ctiles + 7) / 8) * 8 * p.mtiles;
  if (grid > 0x7fffffffll) return -1;
  int ns = 1;
  p.sps = p.nstages;
  if (slices) {
    ns = pwd16_slices(p.ctiles, p.mtiles, p.nstages, &p.sps, *slices);      // at most what the caller's workspace holds
    *slices = ns;
    if (ns <= 1) p.part = nullptr;
  }
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid, (unsigned)ns), dim3(256), 0, s, p, static_cast<const E*>(src),
                       static_cast<const E*>(w), bias, static_cast<E*>(dst), static_cast<const E*>(addend));
  };
  bool deep = (long long)p.ctiles * p.mtiles * ns <= (long long)cus;
  if (pf) deep = pf >= 4;
  if (small) {
    if (deep) go(pwd16_conv_kernel<E, BWD, 8, 64>);
    else go(pwd16_conv_kernel<E, BWD, 4, 64>);
  } else {
    if (deep) go(pwd16_conv_kernel<E, BWD, 8, 128>);
    else go(pwd16_conv_kernel<E, BWD, 4, 128>);
  }
  return check_launch(what);
}

// byte sizes as 32-bit offsets, with room for the rows of a last tile that lie past the tensor
bool pwd16_sizes(PwdParams* p, long long images) {
  const long long sb = images * p->Kc * p->P * 2, db = images * p->Mo * p->P * 2;
  const long long wb = (long long)p->Kc * p->Mo * 2;
  if (std::max(sb, db) + (long long)(PD_BM + PD_KC) * p->P * 2 >= (1ll << 31) || wb + PD_BM * p->Kc * 2ll >= (1ll << 31))
    return false;
  p->src_bytes = (unsigned)sb;
  p->dst_bytes = (unsigned)db;
  p->w_bytes = (unsigned)wb;
  p->Pc = (p->P + 7) / 8;
  p->ncells = (int)(images * p->Pc);
  p->nstages = (p->Kc + PD_KC - 1) / PD_KC;
  p->ctiles = (p->ncells + PD_CELLS - 1) / PD_CELLS;
  return images * p->Pc <= 0x7fffffffll;
}

template <typename E, bool BWD>
int launch_pwd16(const ConvGeom& g, const void* src, const void* w, const float* bias, void* dst, const void* addend,
                 hipStream_t s) {
  if (!pwd16_applies(g, BWD)) return -1;
  PwdParams p{};
  p.Kc = BWD ? g.K : g.C;
  p.Mo = BWD ? g.C : g.K;
  p.P = g.H * g.W;
  if (!pwd16_sizes(&p, g.N)) return -1;
  return pwd16_go<E, BWD>(p, src, w, bias, dst, addend, s,
                          BWD ? "conv2d_bwd_data 1x1 (bf16 mfma, direct-to-LDS)" : "conv2d_fwd 1x1 (bf16 mfma, direct-to-LDS)");
}


// ---- filter gradient ---------------------------------------------------------------------
//   dw[m][c] = sum over (image, position) of dy[m][q] x[c][q]
// Both operands are contiguous along the contraction, so a fragment (one row, 8 consecutive
// positions) is a 16-byte cell as it lies in memory: no transposing reads.  A workgroup owns
// dw[128 m][128 c] and a slice of the contraction; a stage is 8 cells (64 position slots, cells
// numbered over the batch as above) of the 128 dy rows and the 128 x rows: 32 KiB, one load
// instruction per 8 rows, ring of 4 stages.  A row of a tile is 128 bytes; cell c of row r sits
// at cell c ^ (r & 7), so the 32 rows of a fragment read spread over the banks without padding
// (a lane fetches the cell that belongs where it writes).
// Planes that are not a multiple of 8 positions: the last cell of a plane ends at its last
// position and repeats up to 7 positions of the cell before it; in the dy tile those repeated
// positions are overwritten with zeros (by the lanes that loaded them, between the wait for
// their loads and the barrier), so every product is counted once.
// Partial tiles go to the workspace and are added in a fixed order by the reduce kernel the other
// filter-gradient kernels use.  No bias gradient (layers with one take the kernels with register
// staging, which sum it from the loader's registers).
constexpr int PWG_T = 128;                 // tile side
constexpr int PWG_CH = 8;                  // cells per stage
constexpr int PWG_STAGE = 2 * PWG_T * PWG_CH;   // cells per stage: dy rows 0..127, x rows 128..255
constexpr int PWG_NS = 4;
constexpr int PWG_D = PWG_NS - 2;

struct PwdWgradParams {
  int C, Mo, P, Pc, N;
  int ncells, nstages, sps, nsplit;   // cells and stages over the batch, stages per slice, slices
  int ctiles, mtiles;
  int E;
  int dup;                            // positions the last cell of a plane repeats (0: planes of 8k positions)
  unsigned x_bytes, dy_bytes;
};

// DIRECT (matrix products: one slice): the tile leaves in the element type, at out16, with bias[column] added
template <typename E, bool DIRECT>
__global__ void __launch_bounds__(256, 1)
pwd16_wgrad_kernel(PwdWgradParams p, const E* __restrict__ x, const E* __restrict__ dy, float* __restrict__ out,
                   uint16_t* __restrict__ out16, const float* __restrict__ bias) {
  __shared__ __align__(16) uint4 ring[PWG_NS * PWG_STAGE];
  const int slice = blockIdx.x, mtile = blockIdx.y / p.ctiles, ctile = blockIdx.y - mtile * p.ctiles;
  const int m0 = mtile * PWG_T, c0 = ctile * PWG_T;
  const int tid = threadIdx.x, lane = tid & 63, fr = lane & 31, fh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int sbeg = slice * p.sps, n = min(p.nstages, sbeg + p.sps) - sbeg;      // this slice's stages
  const int n2 = (n + 1) & ~1;          // stages are multiplied in pairs: with an odd number one stage of zeros more
  const intx4_t drs = pd_rsrc(dy, p.dy_bytes), xrs = pd_rsrc(x, p.x_bytes);
  constexpr int OOB = (int)0x80000000;

  // ---- load roles: instruction ii = wave + 4 k (k = 0..7) fills rows 8 ii .. 8 ii + 7 of a stage (k < 4: dy rows,
  // k >= 4: x rows); lane -> row 8 ii + lane / 8, LDS cell lane % 8, i.e. the stage's cell (lane % 8) ^ (lane / 8)
  const int lrow = lane >> 3, lcell = (lane & 7) ^ lrow;
  int rowoff[8];                        // byte offset of the lane's row inside an image, or OOB past the last channel
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int r = 8 * ((wave + 4 * k) & 15) + lrow;      // row of the dy (k < 4) or x tile
    if (k < 4) rowoff[k] = m0 + r < p.Mo ? (m0 + r) * p.P * 2 : OOB;
    else rowoff[k] = c0 + r < p.C ? (c0 + r) * p.P * 2 : OOB;
  }
  // the lane's cell of the next stage to load: image, cell inside the plane
  int cell = (sbeg * PWG_CH + lcell);
  int img = cell / p.Pc, j = cell - img * p.Pc;
  const int dimg = PWG_CH / p.Pc, dj = PWG_CH - dimg * p.Pc;
  const int dy_img = p.Mo * p.P * 2, x_img = p.C * p.P * 2;
  unsigned tailq = 0;                   // bit u: the cell this lane loaded into ring slot u is the last of its plane
  int left = n;                         // stages of this slice not yet issued: a stage past the slice fetches nothing (zeros)
  auto issue = [&](int slot) {
    const unsigned base = (unsigned)reinterpret_cast<uintptr_t>((lds_void_t)(ring + slot * PWG_STAGE));
    const bool live = img < p.N && left > 0;
    --left;
    const int col = min(8 * j, p.P - 8) * 2;
    const int od = live ? img * dy_img + col : OOB, ox = live ? img * x_img + col : OOB;
    const bool tail = live && p.dup != 0 && j == p.Pc - 1;
    tailq = tail ? tailq | (1u << slot) : tailq & ~(1u << slot);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int ro = rowoff[k], o = k < 4 ? od : ox;
      pd_load_lds(k < 4 ? drs : xrs, base + (wave + 4 * k) * 1024, (ro == OOB || o == OOB) ? OOB : ro + o, 0);
    }
    // on to the same cell of the next stage
    j += dj;
    img += dimg;
    if (j >= p.Pc) {
      j -= p.Pc;
      img += 1;
    }
  };
  // zeros over the repeated positions of the dy cells this lane loaded into ring slot `slot` (its four dy loads
  // have landed): the first p.dup positions of the cell
  auto fix_tail = [&](int slot) {
    if (tailq & (1u << slot)) {
      char* cellp = reinterpret_cast<char*>(ring + slot * PWG_STAGE) + lane * 16;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        char* q = cellp + (wave + 4 * k) * 1024;
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

  // ---- fragments: wave = (m half, c half), 2 x 2 blocks; lane: row fr of a block, k-octet fh
  int aoff[4];                         // byte offset of the cell of k-step s in the lane's row (the swizzle is the row's)
#pragma unroll
  for (int sk = 0; sk < 4; ++sk) aoff[sk] = ((2 * sk + fh) ^ (fr & 7)) * 16;
  const int arow = (wm * 64 + fr) * 128, brow = (PWG_T + wn * 64 + fr) * 128;
  bf16x8 fa[2][4][2], fb[2][4][2];     // [register set][k-step][block]
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][jj][r] = 0.f;

#define PWG_READ(SLOT, SET)                                                                                  \
  {                                                                                                          \
    const char* st_ = reinterpret_cast<const char*>(ring + (SLOT) * PWG_STAGE);                              \
    _Pragma("unroll") for (int sk = 0; sk < 4; ++sk)                                                         \
      _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                        \
        fa[SET][sk][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(st_ + arow + i * 32 * 128 + aoff[sk])); \
        fb[SET][sk][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(st_ + brow + i * 32 * 128 + aoff[sk])); \
      }                                                                                                      \
  }
#define PWG_MULT(SET)                                                                                        \
  _Pragma("unroll") for (int sk = 0; sk < 4; ++sk)                                                           \
    _Pragma("unroll") for (int i = 0; i < 2; ++i)                                                            \
      _Pragma("unroll") for (int jj = 0; jj < 2; ++jj)                                                       \
        acc[i][jj] = Lo16<E>::mma32(fa[SET][sk][i], fb[SET][sk][jj], acc[i][jj]);

  // stages 0 .. D in flight; every wave issues 8 loads per stage.  Only the wait and the loads depend on the
  // stage number: the reads of one register set and the matrix instructions on the other are one block of
  // code without branches, interleaved one matrix instruction to one read.
  if (n > 0) {
#pragma unroll
    for (int st = 0; st <= PWG_D; ++st)
      if (st < n2) issue(st);
    if (PWG_D < n2) PD_WAIT_VM(16);
    else PD_WAIT_VM(0);
    fix_tail(0);
    __syncthreads();
    PWG_READ(0, 0)
#define PWG_ITER(U)                                                                    \
  {                                                                                    \
    if (t0 + U + PWG_D < n2) PD_WAIT_VM(8);                                            \
    else PD_WAIT_VM(0);                                                                \
    fix_tail((s0 + U + 1) & (PWG_NS - 1));                                             \
    __syncthreads();                                                                   \
    if (t0 + U + 1 + PWG_D < n2) issue((s0 + U + 1 + PWG_D) & (PWG_NS - 1));           \
    PWG_READ((s0 + U + 1) & (PWG_NS - 1), (U + 1) % 2)                                 \
    PWG_MULT(U % 2)                                                                    \
    _Pragma("unroll") for (int q = 0; q < 16; ++q) {                                   \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                               \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                               \
    }                                                                                  \
  }
    // two stages per trip (the register sets alternate); the ring slot is the stage number modulo the ring
    for (int t0 = 0; t0 < n2; t0 += 2) {
      const int s0 = t0 & (PWG_NS - 1);
      PWG_ITER(0) PWG_ITER(1)
    }
#undef PWG_ITER
  }
#undef PWG_MULT
#undef PWG_READ

  // element r of acc[i][jj]: row m0 + wm*64 + i*32 + (r/4)*8 + fh*4 + r%4, column c0 + wn*64 + jj*32 + fr
  float* o = out + (size_t)slice * (p.nsplit > 1 ? (size_t)p.E + p.Mo : 0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int c = c0 + wn * 64 + jj * 32 + fr;
      if (c >= p.C) continue;
      const float bv = (DIRECT && bias) ? bias[c] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + fh * 4 + (r & 3);
        if (m >= p.Mo) continue;
        if (DIRECT) out16[(size_t)m * p.C + c] = Lo16<E>::narrow(acc[i][jj][r] + bv);
        else o[(size_t)m * p.C + c] = acc[i][jj][r];
      }
    }
}

bool pwd16_wgrad_plan(const ConvGeom& g, PwdWgradParams* p) {
  if (!(g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1 && g.sy == 1 && g.sx == 1 &&
        g.OH == g.H && g.OW == g.W && g.C % 8 == 0 && g.K % 8 == 0))
    return false;
  // (a side of 64 channels fills half of a tile: twice the matrix work for a pass that waits for memory, 41 -> 31 us
  // on the 64 <-> 256 channel layers over 56x56 planes at batch 64)
  if (g.C < 64 || g.K < 64 || g.H * g.W < 8) return false;
  p->C = g.C; p->Mo = g.K; p->P = g.H * g.W; p->N = g.N;
  p->Pc = (p->P + 7) / 8;
  p->dup = (8 - p->P % 8) % 8;
  const long long xb = (long long)g.N * g.C * p->P * 2, db = (long long)g.N * g.K * p->P * 2;
  if (xb >= (1ll << 31) || db >= (1ll << 31)) return false;
  p->x_bytes = (unsigned)xb;
  p->dy_bytes = (unsigned)db;
  p->ncells = g.N * p->Pc;
  p->nstages = (p->ncells + PWG_CH - 1) / PWG_CH;
  p->ctiles = (g.C + PWG_T - 1) / PWG_T;
  p->mtiles = (g.K + PWG_T - 1) / PWG_T;
  p->E = g.K * g.C;
  const long long tiles = (long long)p->ctiles * p->mtiles;
  if (tiles > 65535) return false;
  // one workgroup per CU (128 KiB of LDS); every slice writes and re-reads the whole gradient
  long long ns = mfma_num_cus() / tiles;
  if (ns > p->nstages / 4) ns = p->nstages / 4;      // at least four stages per slice
  if (ns < 1) ns = 1;
  p->sps = (int)((p->nstages + ns - 1) / ns);
  p->nsplit = (p->nstages + p->sps - 1) / p->sps;
  return true;
}

}  // namespace

int mfma_pwd16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y, hipStream_t s, int dtype) {
  return by_lo16(dtype, [&](auto* e_) { return launch_pwd16<FLHIP_T_OF(e_), false>(g, x, w, bias, y, nullptr, s); });
}

int mfma_pwd16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, const void* addend, void* dx,
                             hipStream_t s, int dtype) {
  return by_lo16(dtype, [&](auto* e_) { return launch_pwd16<FLHIP_T_OF(e_), true>(g, dy, w, nullptr, dx, addend, s); });
}

}  // namespace flhip

namespace flhip {

// defined in conv2d_mfma_wgrad.hip
void wgrad_reduce_launch(const float* part, int nsplit, int E, int K, int want_db, float* dw,
                         float* db, hipStream_t s);

size_t mfma_pwd16_wgrad_ws(const ConvGeom& g) {
  PwdWgradParams p{};
  if (!pwd16_wgrad_plan(g, &p)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float) : 0;
}

// -1 when the shape (or a bias gradient) is not this kernel's
int mfma_pwd16_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, void* ws, size_t ws_bytes, hipStream_t s,
                     int dtype) {
  PwdWgradParams p{};
  if (!dw || !pwd16_wgrad_plan(g, &p)) return -1;
  // measured on the ResNet-50 layers at batch 64: 7 to 20 % ahead of the kernel with register staging on planes of
  // 14x14 and more (both move the same 100 MB through L2 for 30 MB of operands: 128 x 128 tiles); on 7x7 planes ahead
  // where dy is the large operand (512 -> 2048 channels: 28.6 against 31.2 us), level the other way round.
  // FLHIP_PW16_PF set lifts the rule (tests).
  if (!options().pw16_pf && p.P < 64 && g.K < 4 * g.C) return -1;
  const size_t need = p.nsplit > 1 ? (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float) : 0;
  if (need && (!ws || ws_bytes < need)) return -1;
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  by_lo16(dtype, [&](auto* e_) {
    using E = FLHIP_T_OF(e_);
    hipLaunchKernelGGL((pwd16_wgrad_kernel<E, false>), dim3((unsigned)p.nsplit, (unsigned)(p.ctiles * p.mtiles)), dim3(256), 0,
                       s, p, static_cast<const E*>(x), static_cast<const E*>(dy), out, (uint16_t*)nullptr, (const float*)nullptr);
  });
  if (p.nsplit > 1) wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.Mo, 0, dw, nullptr, s);
  return check_launch("conv2d_bwd_filter 1x1 (bf16 mfma, direct-to-LDS)");
}

// out[i] = the sum of `slices` fp32 partial products, n floats apart, added in slice order and rounded once
template <typename E>
__global__ void __launch_bounds__(256) gemm16_sum_slices_kernel(const float* __restrict__ part, uint16_t* __restrict__ out,
                                                                size_t n, int slices) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    float v = part[i];
    for (int k = 1; k < slices; ++k) v += part[(size_t)k * n + i];
    out[i] = Lo16<E>::narrow(v);
  }
}

bool gemm16_plan(int mode, int M, int N, int K, const float* bias_rows, PwdParams* p) {
  if (M < 8 || (mode == 0 && K % 8 != 0) || (mode == 2 && (bias_rows || N % 2 != 0))) return false;
  p->Kc = K; p->Mo = N; p->P = M;
  return pwd16_sizes(p, 1);
}

// bytes of workspace with which A B^T (mode 2) cuts its contraction into slices (0: one slice, or not these kernels')
size_t mfma_gemm16_ws_bytes(int dtype, int mode, int M, int N, int K) {
  PwdParams p{};
  if (!is_lo16(dtype) || mode != 2 || M <= 0 || N <= 0 || K <= 0 || !gemm16_plan(mode, M, N, K, nullptr, &p)) return 0;
  const int bm = pwd16_bm(p);
  int sps;
  const int ns = pwd16_slices(p.ctiles, (N + bm - 1) / bm, p.nstages, &sps);
  return ns > 1 ? (size_t)ns * M * N * sizeof(float) : 0;
}

// Column-major matrix products in 16-bit storage on the kernels above (C is M x N, stored [n][m]):
//   mode 0, C = A B    : A (M x K) is stored [k][m]: the source of a forward 1x1 layer over ONE image whose plane is the
//                        M rows; B stored [n][k] are its weights; bias_rows (one per row of C) is a bias per position
//   mode 1, C = A^T B  : A stored [m][k] and B stored [n][k] are both contiguous along the contraction: the filter
//                        gradient's tile, written in the element type; bias_rows is a bias per column of that tile
//   mode 2, C = A B^T  : A stored [k][m], B stored [k][n]: a backward-data 1x1 layer with B as the weights
// One rounding per element, after the fp32 sum (and the bias).  -1 when the shape is not these kernels':
// fewer than 8 rows (modes 0, 2) or a contraction shorter than 8 (mode 1), a contraction that is not a multiple
// of 8 in mode 0 (a 16-byte cell of B would straddle two rows), a bias or an odd number of columns in mode 2 (the
// range check of a buffer load works on 4-byte words: the word that holds the last element of B's last row would
// lie half past the tensor and come back as zero), operands of 2 GiB.
// With a workspace of mfma_gemm16_ws_bytes, A B^T over a long contraction and few tiles (the weight gradient of a
// layer over many frames) cuts the contraction into slices, one workgroup per tile and slice; their fp32 partial
// products are added in slice order.
int mfma_gemm16(int dtype, int mode, const void* A, const void* B, void* C, int M, int N, int K,
                const float* bias_rows, hipStream_t s, void* ws, size_t ws_bytes) {
  if (!is_lo16(dtype) || M <= 0 || N <= 0 || K <= 0) return -1;
  if (mode == 1) {
    if (K < 8) return -1;
    PwdWgradParams p{};
    p.C = M; p.Mo = N; p.P = K; p.N = 1;
    p.Pc = (K + 7) / 8;
    p.dup = (8 - K % 8) % 8;
    const long long xb = (long long)M * K * 2, db = (long long)N * K * 2;
    if (xb >= (1ll << 31) || db >= (1ll << 31)) return -1;
    p.x_bytes = (unsigned)xb;
    p.dy_bytes = (unsigned)db;
    p.ncells = p.Pc;
    p.nstages = (p.ncells + PWG_CH - 1) / PWG_CH;
    p.ctiles = (M + PWG_T - 1) / PWG_T;
    p.mtiles = (N + PWG_T - 1) / PWG_T;
    p.E = 0;
    p.sps = p.nstages;
    p.nsplit = 1;
    if ((long long)p.ctiles * p.mtiles > 65535) return -1;
    by_lo16(dtype, [&](auto* e_) {
      using E = FLHIP_T_OF(e_);
      hipLaunchKernelGGL((pwd16_wgrad_kernel<E, true>), dim3(1u, (unsigned)(p.ctiles * p.mtiles)), dim3(256), 0, s, p,
                         static_cast<const E*>(A), static_cast<const E*>(B), (float*)nullptr, static_cast<uint16_t*>(C),
                         bias_rows);
      return 0;
    });
    return check_launch("matmul (A^T * B, 16-bit mfma)");
  }
  if (mode != 0 && mode != 2) return -1;
  PwdParams p{};
  if (!gemm16_plan(mode, M, N, K, bias_rows, &p)) return -1;
  p.pos_bias = bias_rows;
  return by_lo16(dtype, [&](auto* e_) {
    using E = FLHIP_T_OF(e_);
    if (mode == 0) return pwd16_go<E, false>(p, A, B, nullptr, C, nullptr, s, "matmul (A * B, 16-bit mfma)");
    const size_t per = (size_t)M * N * sizeof(float);
    int slices = ws ? (int)std::min<size_t>(ws_bytes / per, 32) : 1;
    if (slices <= 1) return pwd16_go<E, true>(p, A, B, nullptr, C, nullptr, s, "matmul (A * B^T, 16-bit mfma)");
    p.part = static_cast<float*>(ws);
    const int rc = pwd16_go<E, true>(p, A, B, nullptr, C, nullptr, s, "matmul (A * B^T, 16-bit mfma)", &slices);
    if (rc != 0 || slices <= 1) return rc;
    const size_t n = (size_t)M * N;
    hipLaunchKernelGGL(gemm16_sum_slices_kernel<E>, dim3((unsigned)std::min<size_t>((n + 255) / 256, 4096)), dim3(256), 0, s,
                       static_cast<const float*>(ws), static_cast<uint16_t*>(C), n, slices);
    return check_launch("matmul (A * B^T, 16-bit mfma, slices added)");
  });
}

}  // namespace flhip
