// 1x1 stride-1 convolutions in bf16 storage on the bf16 matrix cores
// (v_mfma_f32_16x16x32_bf16, fp32 accumulate): forward, backward-data and the filter
// gradient.  Per image the tensors are [channels][positions] with positions contiguous.
//
//   forward        y[m][q]  = sum_c w[m][c]  x[c][q]  (+ bias[m])
//   backward-data  dx[c][q] = sum_m w[m][c] dy[m][q]
// contract over the ROW index of the source, but an MFMA lane wants eight consecutive
// contraction indices of one position.  The source tile goes to LDS as it is in memory
// ([32 channels][128 positions]) and a lane fetches its eight channels with two
// transposing reads (ds_read_b64_tr_b16: 16 lanes pass the addresses of four channel rows
// x four 8-byte pieces and each receives four channels of one position); a pitch of 288
// bytes keeps the four rows of a read in disjoint banks.
// Weights: forward [m][c] is contraction-contiguous (16-byte LDS reads), backward-data
// contracts over m: its tile is copied as it is and read like the source.  Positions are the rows of the
// instruction tile, so a lane ends up with four consecutive positions of one result
// channel: one 8-byte store.  Positions are flattened over the batch (a plane of 14x14
// would waste a quarter of a 128-wide tile per image).  When a plane is not a multiple
// of 4 positions (7x7) a 4-position run starts at any even byte and may begin in one
// image and end in the next: the ODD variants load such a run as the last four positions
// of the first image and the first four of the second and shift the two together, and
// store it element by element.
//
//   filter gradient  dw[m][c] = sum_{n,q} dy[m][q] x[c][q]   (+ db[m] = sum dy)
// contracts over positions, contiguous in both operands: both tiles are read from LDS
// 16 bytes at a time.  The contraction (batch x positions) is cut into slices that a
// fixed-order kernel adds.
//
// 256 threads; every thread loads, then computes (global -> registers -> the LDS buffer
// not in use, one barrier per chunk).
#include "conv2d_mfma.h"

namespace flhip {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int PB_BP = 128;    // positions per workgroup
constexpr int PB_KC = 32;     // contraction per chunk = K of one instruction
constexpr int PB_XP = PB_BP + 16;  // source tile pitch (elements): 288 bytes, four rows' 32-byte pieces in disjoint banks
constexpr int PB_WP = PB_KC + 8;   // weight tile pitch, forward ([result channel][contraction])
constexpr int PB_WPB = 64 + 8;     // weight tile pitch, backward-data ([contraction][64 result channels])

struct Pw16Params {
  int Kc, Mo;        // contraction channels, result channels
  int P, Ptot;       // positions per image, over the batch
  int nchunks, mtiles, ptiles;
};

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uintx4_t v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}

// Eight elements of one column of a 16-bit LDS tile stored [row][column]: rows r0 .. r0+7
// of column c0 + s for lane s of each group of 16 lanes, by two transposing reads
// (ds_read_b64_tr_b16).  In such a read lane s of a group passes the address of four
// consecutive elements ("row slot" s) and receives element s % 4 of the row slots
// s / 4, s / 4 + 4, s / 4 + 8, s / 4 + 12.  With row slot s pointing at columns
// c0 + 4 * (s % 4) .. + 3 of tile row r0 + s / 4, lane s receives rows r0 .. r0 + 3 of
// column c0 + s.  c0 and the pitch are multiples of 4 elements (8-byte addresses).
typedef short shortx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 gather8_tr(const uint16_t* tile, int pitch, int r0, int c0, int s) {
  typedef __attribute__((address_space(3))) shortx4_t* lds_ptr;
  const uint16_t* t = tile + (r0 + (s >> 2)) * pitch + c0 + 4 * (s & 3);
  const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)t);
  const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(t + 4 * pitch));
  const uintx2_t l = __builtin_bit_cast(uintx2_t, lo), h = __builtin_bit_cast(uintx2_t, hi);
  return as_bf16x8(l.x, l.y, h.x, h.y);
}

// 8 bytes at any 2-byte boundary
__device__ __forceinline__ uintx2_t load8_any(const bf16_t* p) {
  uintx2_t v;
  __builtin_memcpy(&v, p, 8);
  return v;
}
__device__ __forceinline__ void store8_any(bf16_t* p, uintx2_t v) { __builtin_memcpy(p, &v, 8); }
// a: the last four positions of an image's row, b: the first four of the next image's;
// result: the last rem (1..3) of a followed by the first 4 - rem of b
__device__ __forceinline__ uintx2_t merge_runs(uintx2_t a, uintx2_t b, int rem) {
  const uint64_t A = ((uint64_t)a.y << 32) | a.x, B = ((uint64_t)b.y << 32) | b.x;
  const uint64_t v = (A >> (16 * (4 - rem))) | (B << (16 * rem));
  return uintx2_t{(uint32_t)v, (uint32_t)(v >> 32)};
}

// a + b on two bf16 values per dword, each sum rounded to bf16 (what an element-wise add of the
// two tensors would give)
template <typename E>
__device__ __forceinline__ uint32_t add_x2(uint32_t a, uint32_t b) {
  return Lo16<E>::pack(Lo16<E>::lo(a) + Lo16<E>::lo(b), Lo16<E>::hi(a) + Lo16<E>::hi(b));
}

// BWD = false: forward (weights [Mo][Kc]); true: backward-data (weights [Kc][Mo]).
// addend (or null): a tensor of the result's shape that is added to the rounded result (the
// gradient a variable already holds, when this pass delivers its second one).
// MT = 16-channel result tiles per workgroup (4: 64 result channels; 8 was measured and
// is slower on every ResNet-50 layer, as is loading two chunks ahead instead of one).
// ODD: planes that are not a multiple of 4 positions (at least 4).
// PF = chunks whose global loads are in flight while one is multiplied: 1 when the grid
// fills the chip several times over (other workgroups hide the latency), 4 for small grids
// with long contractions (7x7 planes: about 100 workgroups of up to 64 chunks each, one
// wave per SIMD), where a chunk otherwise costs one trip to memory.
template <typename E, bool BWD, int MT, bool ODD, int PF>
__global__ void __launch_bounds__(256)
pw16_conv_kernel(Pw16Params p, const bf16_t* __restrict__ src, const bf16_t* __restrict__ wgt,
                 const float* __restrict__ bias, bf16_t* __restrict__ dst, const bf16_t* __restrict__ addend) {
  constexpr int BM = MT * 16, WQ = BM / 64;      // result channels; 16-byte weight pieces per thread
  static_assert(!BWD || BM == 64, "the backward-data weight tile is [contraction][64 result channels]");
  static_assert(PB_KC * PB_WPB <= 64 * PB_WP, "both weight layouts share one buffer size");
  constexpr int XSZ = PB_KC * PB_XP;             // elements per source buffer
  constexpr int WSZ = BM * PB_WP;                // per weight buffer, [m][k] in both directions
  constexpr int YP = PB_BP + 8;                  // result staging pitch
  constexpr int LDS_ELEMS = 2 * (XSZ + WSZ) > BM * YP ? 2 * (XSZ + WSZ) : BM * YP;
  __shared__ __align__(16) uint16_t lds16[LDS_ELEMS];
  uint16_t* const Xs0 = lds16;
  uint16_t* const Ws0 = lds16 + 2 * XSZ;
  // consecutive workgroups go to different XCDs: the channel tiles that share a source
  // tile run back to back on one XCD
  const int id = blockIdx.x, xcd = id & 7, seq = id >> 3;
  const int mtile = seq % p.mtiles, ptile = (seq / p.mtiles) * 8 + xcd;
  if (ptile >= p.ptiles) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fg = lane >> 4;
  const int m0 = mtile * BM, q0 = ptile * PB_BP;

  // ---- loader roles: a 4-position run of rows lr, lr+8, lr+16, lr+24 of the source tile
  const int lq = (tid & 31) * 4, lr = tid >> 5;
  const int q = q0 + lq;
  const bool qv = q < p.Ptot;
  const int img = qv ? q / p.P : 0, pos = qv ? q - img * p.P : 0;
  // ODD: a run with fewer than 4 positions left in its image continues in the next one
  const int rem = p.P - pos;
  const bool cross = ODD && qv && rem < 4, nextv = cross && q + rem < p.Ptot;
  const bf16_t* sp = src + (size_t)img * p.Kc * p.P + (cross ? p.P - 4 : pos);
  const bf16_t* sp2 = nextv ? src + (size_t)(img + 1) * p.Kc * p.P : sp;
  // LATE: every load issues, from an address inside its tensor, and what lies outside the
  // tile is zeroed when the registers go to LDS (nothing between a load and the next one
  // depends on loaded data)
  constexpr bool LATE = ODD || PF > 1;
  struct Stage {
    uintx2_t x[4];
    uintx2_t xb[ODD ? 4 : 1];   // ODD: the same rows of the next image
    uintx4_t w[WQ];
  };
  // weights: forward rows m = tid / 4 (+ 64), 8 contraction elements (tid % 4) * 8;
  // backward-data row k = tid / 8, 8 result channels (tid % 8) * 8 (+ 64)
  const int wr = BWD ? tid >> 3 : tid >> 2, wc = BWD ? (tid & 7) * 8 : (tid & 3) * 8;
  auto gload = [&](int c, Stage& st) {
    const int k0 = c * PB_KC;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lr + 8 * i;
      // LATE: row clamped into the tensor (no branch, no select on the way to the load)
      const uint32_t off = (uint32_t)min(k, p.Kc - 1) * (uint32_t)p.P;
      if (ODD) {
        st.x[i] = load8_any(sp + off);
        st.xb[i] = load8_any(sp2 + off);
      } else if (LATE) {
        st.x[i] = *reinterpret_cast<const uintx2_t*>(sp + off);
      } else {
        st.x[i] = (qv && k < p.Kc) ? *reinterpret_cast<const uintx2_t*>(sp + (size_t)k * p.P) : uintx2_t{0u, 0u};
      }
    }
#pragma unroll
    for (int h = 0; h < WQ; ++h) {
      const int k = BWD ? k0 + wr : k0 + wc, m = BWD ? m0 + wc + 64 * h : m0 + wr + 64 * h;
      const bool in = k < p.Kc && m < p.Mo;
      const size_t off = BWD ? (size_t)k * p.Mo + m : (size_t)m * p.Kc + k;
      // LATE: the 8-element piece clamped into the matrix (both dimensions are multiples of 8)
      const uint32_t offc = BWD ? (uint32_t)min(k, p.Kc - 1) * (uint32_t)p.Mo + (uint32_t)min(m, p.Mo - 8)
                                : (uint32_t)min(m, p.Mo - 1) * (uint32_t)p.Kc + (uint32_t)min(k, p.Kc - 8);
      if (LATE) st.w[h] = *reinterpret_cast<const uintx4_t*>(wgt + offc);
      else st.w[h] = in ? *reinterpret_cast<const uintx4_t*>(wgt + off) : uintx4_t{0u, 0u, 0u, 0u};
    }
  };
  // Forward weights live in LDS as [result channel m][contraction k], 8-element contraction
  // groups g stored at group slot g ^ ((m >> 3) & 3); backward-data weights as in memory,
  // [contraction k][result channel m], read by transposing reads like the source.
  auto wslot = [](int m, int g) { return m * PB_WP + 8 * (g ^ ((m >> 3) & 3)); };
  auto sstore = [&](int c, const Stage& st) {
    const int buf = c & 1;
    uint16_t* X = Xs0 + buf * XSZ;
    uint16_t* Wt = Ws0 + buf * WSZ;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uintx2_t v = st.x[i];
      if (ODD) {   // no branch: every lane shifts, lanes whose run crosses keep the result
        const uintx2_t mr = merge_runs(v, nextv ? st.xb[i] : uintx2_t{0u, 0u}, cross ? rem : 1);
        v = cross ? mr : v;
      }
      if (LATE && !(qv && c * PB_KC + lr + 8 * i < p.Kc)) v = uintx2_t{0u, 0u};
      uint32_t* d = reinterpret_cast<uint32_t*>(&X[(lr + 8 * i) * PB_XP + lq]);
      d[0] = v.x;
      d[1] = v.y;
    }
#pragma unroll
    for (int h = 0; h < WQ; ++h) {
      uintx4_t wv = st.w[h];
      if (LATE) {
        const int k = BWD ? c * PB_KC + wr : c * PB_KC + wc, m = BWD ? m0 + wc + 64 * h : m0 + wr + 64 * h;
        if (!(k < p.Kc && m < p.Mo)) wv = uintx4_t{0u, 0u, 0u, 0u};
      }
      if (BWD) {
        *reinterpret_cast<uintx4_t*>(&Wt[wr * PB_WPB + wc]) = wv;
      } else {
        *reinterpret_cast<uintx4_t*>(&Wt[wslot(wr + 64 * h, wc >> 3)]) = wv;
      }
    }
  };

  floatx4 acc[2][MT];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](int buf) {
    const uint16_t* X = Xs0 + buf * XSZ;
    const uint16_t* Wt = Ws0 + buf * WSZ;
    bf16x8 a[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = gather8_tr(X, PB_XP, 8 * fg, wave * 32 + i * 16, fr);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const bf16x8 b = BWD ? gather8_tr(Wt, PB_WPB, 8 * fg, j * 16, fr)
                           : __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(&Wt[wslot(j * 16 + fr, fg)]));
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i][j] = Lo16<E>::mma16(a[i], b, acc[i][j]);
    }
  };

  const int n = p.nchunks;
  if (PF == 1) {
    Stage st;
    gload(0, st);
    sstore(0, st);
    __syncthreads();
    for (int c = 0; c < n; ++c) {
      if (c + 1 < n) gload(c + 1, st);
      compute(c & 1);
      if (c + 1 < n) sstore(c + 1, st);
      __syncthreads();
    }
  } else {
    // st[c % PF] holds chunk c from its load until it is copied to LDS one iteration
    // before its product; then the register set takes chunk c + PF
    Stage st[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j)
      if (j < n) gload(j, st[j]);
    sstore(0, st[0]);
    __syncthreads();
    // while every chunk of a round has a successor PF on: no conditions, so the waits for
    // a register set's loads can be counted exactly; then the last one or two rounds
    int c0 = 0;
    for (; c0 + 2 * PF <= n; c0 += PF) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int c = c0 + j;
        gload(c + PF, st[j]);
        compute(c & 1);
        sstore(c + 1, st[(j + 1) % PF]);
        __syncthreads();
      }
    }
    for (; c0 < n; c0 += PF) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int c = c0 + j;
        if (c < n) {
          if (c + PF < n) gload(c + PF, st[j]);
          compute(c & 1);
          if (c + 1 < n) sstore(c + 1, st[(j + 1) % PF]);
          __syncthreads();
        }
      }
    }
  }

  // ---- results: a lane holds positions wave*32 + i*16 + 4*fg .. +3 of channel j*16 + fr.
  // They go to LDS as [channel][position] (the operand buffers are free: the loop ended
  // with a barrier), then every channel's run of positions leaves in 16-byte (planes of
  // 8k positions) or 8-byte pieces, 256 contiguous bytes per channel.
  uint16_t* Ys = lds16;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int ml = j * 16 + fr;
      const float bv = (!BWD && bias && m0 + ml < p.Mo) ? bias[m0 + ml] : 0.f;
      const uintx2_t o = {(uint32_t)Lo16<E>::narrow(acc[i][j][0] + bv) | ((uint32_t)Lo16<E>::narrow(acc[i][j][1] + bv) << 16),
                          (uint32_t)Lo16<E>::narrow(acc[i][j][2] + bv) | ((uint32_t)Lo16<E>::narrow(acc[i][j][3] + bv) << 16)};
      *reinterpret_cast<uintx2_t*>(&Ys[ml * YP + wave * 32 + i * 16 + 4 * fg]) = o;
    }
  __syncthreads();
  if (ODD) {
    const int pc = (tid & 31) * 4, qo = q0 + pc;
    if (qo < p.Ptot) {
      const int im = qo / p.P, po = qo - im * p.P, left = p.P - po;
      bf16_t* dp = dst + (size_t)im * p.Mo * p.P + po;
      bf16_t* dp2 = dst + (size_t)(im + 1) * p.Mo * p.P - left;   // element e >= left: position e - left of the next image
      for (int ml = tid >> 5; ml < BM && m0 + ml < p.Mo; ml += 8) {
        uintx2_t v = *reinterpret_cast<const uintx2_t*>(&Ys[ml * YP + pc]);
        const size_t row = (size_t)(m0 + ml) * p.P;
        if (left >= 4) {
          if (addend) {
            const uintx2_t a = load8_any(addend + (dp - dst) + row);
            v = uintx2_t{add_x2<E>(v.x, a.x), add_x2<E>(v.y, a.y)};
          }
          store8_any(dp + row, v);
        } else {
          const uint32_t e4[4] = {v.x & 0xffffu, v.x >> 16, v.y & 0xffffu, v.y >> 16};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (qo + e < p.Ptot) {
              bf16_t* o = (e < left ? dp : dp2) + row + e;
              *o = addend ? Lo16<E>::narrow(Lo16<E>::widen((uint16_t)e4[e]) + Lo16<E>::widen(addend[o - dst])) : (bf16_t)e4[e];
            }
        }
      }
    }
  } else if ((p.P & 7) == 0) {
    const int pc = (tid & 15) * 8, qo = q0 + pc;
    if (qo < p.Ptot) {
      const int im = qo / p.P, po = qo - im * p.P;
      bf16_t* dp = dst + (size_t)im * p.Mo * p.P + po;
      for (int ml = tid >> 4; ml < BM && m0 + ml < p.Mo; ml += 16) {
        uintx4_t v = *reinterpret_cast<const uintx4_t*>(&Ys[ml * YP + pc]);
        if (addend) {
          const uintx4_t a = *reinterpret_cast<const uintx4_t*>(addend + (dp - dst) + (size_t)(m0 + ml) * p.P);
          v = uintx4_t{add_x2<E>(v.x, a.x), add_x2<E>(v.y, a.y), add_x2<E>(v.z, a.z), add_x2<E>(v.w, a.w)};
        }
        *reinterpret_cast<uintx4_t*>(dp + (size_t)(m0 + ml) * p.P) = v;
      }
    }
  } else {
    const int pc = (tid & 31) * 4, qo = q0 + pc;
    if (qo < p.Ptot) {
      const int im = qo / p.P, po = qo - im * p.P;
      bf16_t* dp = dst + (size_t)im * p.Mo * p.P + po;
      for (int ml = tid >> 5; ml < BM && m0 + ml < p.Mo; ml += 8) {
        uintx2_t v = *reinterpret_cast<const uintx2_t*>(&Ys[ml * YP + pc]);
        if (addend) {
          const uintx2_t a = *reinterpret_cast<const uintx2_t*>(addend + (dp - dst) + (size_t)(m0 + ml) * p.P);
          v = uintx2_t{add_x2<E>(v.x, a.x), add_x2<E>(v.y, a.y)};
        }
        *reinterpret_cast<uintx2_t*>(dp + (size_t)(m0 + ml) * p.P) = v;
      }
    }
  }
}

bool pw16_applies(const ConvGeom& g) {
  return g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1 && g.sy == 1 && g.sx == 1 &&
         g.OH == g.H && g.OW == g.W && g.H * g.W >= 4 && g.C % 8 == 0 && g.K % 8 == 0;
}

template <typename E, bool BWD>
int launch_pw16(const ConvGeom& g, const void* src, const void* w, const float* bias, void* dst, hipStream_t s,
                const void* addend = nullptr) {
  Pw16Params p{};
  p.Kc = BWD ? g.K : g.C;
  p.Mo = BWD ? g.C : g.K;
  p.P = g.H * g.W;
  const long long ptot = (long long)g.N * p.P;
  if (ptot * std::max(p.Kc, p.Mo) >= (1ll << 31)) return -1;
  p.Ptot = (int)ptot;
  p.nchunks = (p.Kc + PB_KC - 1) / PB_KC;
  p.ptiles = (p.Ptot + PB_BP - 1) / PB_BP;
  p.mtiles = (p.Mo + 63) / 64;
  const long long grid = (long long)((p.ptiles + 7) / 8) * 8 * p.mtiles;
  if (grid > 0x7fffffffll) return -1;
  // deep prefetch for grids of at most one workgroup per CU with at least 8 chunks (measured
  // on the ResNet-50 layers: 20 to 30 % faster there, slower on every larger grid);
  // FLHIP_PW16_PF = 1 / 4 forces one or the other
  bool deep = grid <= (long long)mfma_num_cus() && p.nchunks >= 8;
  if (options().pw16_pf) deep = options().pw16_pf >= 4;
  const bool odd = p.P % 4 != 0;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), 0, s, p, static_cast<const bf16_t*>(src),
                       static_cast<const bf16_t*>(w), bias, static_cast<bf16_t*>(dst), static_cast<const bf16_t*>(addend));
  };
  if (odd) {
    if (deep) go(pw16_conv_kernel<E, BWD, 4, true, 4>);
    else go(pw16_conv_kernel<E, BWD, 4, true, 1>);
  } else {
    if (deep) go(pw16_conv_kernel<E, BWD, 4, false, 4>);
    else go(pw16_conv_kernel<E, BWD, 4, false, 1>);
  }
  return check_launch(BWD ? "conv2d_bwd_data 1x1 (bf16 mfma)" : "conv2d_fwd 1x1 (bf16 mfma)");
}

// ---- filter gradient -------------------------------------------------------------------
constexpr int PG_KC = 64;          // positions per chunk (two instructions deep)
constexpr int PG_P = PG_KC + 8;    // LDS pitch (elements): 16-byte reads, rows 144 bytes apart

struct Pw16WgradParams {
  int C, Mo, P, Ptot;
  int ctiles, mtiles;
  int nchunks, cps, nsplit;   // chunks of 64 positions over the batch, per slice, slices
  int E, want_db;
};

// grid (slice, channel-tile pair).  A workgroup owns dw[64 m][64 c] and one slice of the
// positions of the whole batch; per chunk thread t loads one 8-byte run of 4 positions (inside
// one image; ODD: planes not a multiple of 4 positions, where a run may end in the next
// image) of rows t / 16 + 16 g, g = 0..3, of both operands.  out: slice-major partial results
// [nsplit][E + Mo] (dw tile values, then the bias sums), or dw / db themselves when there
// is one slice.
template <typename E, bool ODD>
__global__ void __launch_bounds__(256)
pw16_wgrad_kernel(Pw16WgradParams p, const bf16_t* __restrict__ x, const bf16_t* __restrict__ dy,
                  float* __restrict__ out, float* __restrict__ db_direct) {
  __shared__ __align__(16) uint16_t Ds[2][64 * PG_P];
  __shared__ __align__(16) uint16_t Xs[2][64 * PG_P];
  const int slice = blockIdx.x, mtile = blockIdx.y / p.ctiles, ctile = blockIdx.y - mtile * p.ctiles;
  const int m0 = mtile * 64, c0 = ctile * 64;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fg = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int cbeg = slice * p.cps, cend = min(p.nchunks, cbeg + p.cps);

  // loader roles: 16 lanes cover the 64 positions of a chunk row (128 contiguous bytes), so a
  // wave's load touches 4 rows (with 4 lanes per row it touched 16 for the same bytes, and the
  // kernel ran at the rate of those requests); a thread loads rows lrow + 16 g, g = 0..3
  const int lrow = tid >> 4, lpos = (tid & 15) * 4;
  bool mv[4], cv[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    mv[g] = m0 + lrow + 16 * g < p.Mo;
    cv[g] = c0 + lrow + 16 * g < p.C;
  }
  // the thread's run of chunk c: positions Q = c*64 + lpos .. + 3 of the batch; q = Q's offset
  // in its image, od / ox = element offsets of (image, row 0) + q in dy / x
  int q;
  long long od, ox;
  {
    const long long Q = (long long)cbeg * PG_KC + lpos;
    const int n = (int)(Q / p.P);
    q = (int)(Q - (long long)n * p.P);
    od = (long long)n * p.Mo * p.P + q;
    ox = (long long)n * p.C * p.P + q;
  }
  const long long drow = (long long)(m0 + lrow) * p.P, xrow = (long long)(c0 + lrow) * p.P, rstep = 16ll * p.P;
  const long long dlim = (long long)(p.Ptot / p.P) * p.Mo * p.P;   // == N * Mo * P
  uintx2_t sd[4], sx[4];
  float bsum[4] = {0.f, 0.f, 0.f, 0.f};
  const bool do_bias = p.want_db && ctile == 0;
  auto gload = [&]() {
    const bool in = od < dlim;     // past the last image: nothing left
    // ODD: a run with fewer than 4 positions left in its image continues in the next one
    // (if there is one); all loads issue, from addresses inside the tensors
    const int rem = p.P - q;
    const bool cross = ODD && rem < 4;
    const int back = cross ? 4 - rem : 0;
    const long long nd = od - q + (long long)p.Mo * p.P, nx = ox - q + (long long)p.C * p.P;
    const bool nin = cross && nd < dlim;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (ODD) {
        uintx2_t a = load8_any(dy + ((in && mv[g]) ? od - back + drow + g * rstep : 0));
        uintx2_t b = load8_any(dy + ((nin && mv[g]) ? nd + drow + g * rstep : 0));
        if (cross) a = merge_runs(a, nin ? b : uintx2_t{0u, 0u}, rem);
        sd[g] = (in && mv[g]) ? a : uintx2_t{0u, 0u};
        a = load8_any(x + ((in && cv[g]) ? ox - back + xrow + g * rstep : 0));
        b = load8_any(x + ((nin && cv[g]) ? nx + xrow + g * rstep : 0));
        if (cross) a = merge_runs(a, nin ? b : uintx2_t{0u, 0u}, rem);
        sx[g] = (in && cv[g]) ? a : uintx2_t{0u, 0u};
      } else {
        sd[g] = (in && mv[g]) ? *reinterpret_cast<const uintx2_t*>(dy + od + drow + g * rstep) : uintx2_t{0u, 0u};
        sx[g] = (in && cv[g]) ? *reinterpret_cast<const uintx2_t*>(x + ox + xrow + g * rstep) : uintx2_t{0u, 0u};
      }
    }
    // next chunk: 64 positions on, possibly into the following images
    q += PG_KC; od += PG_KC; ox += PG_KC;
    while (q >= p.P) {
      q -= p.P;
      od += (long long)(p.Mo - 1) * p.P;
      ox += (long long)(p.C - 1) * p.P;
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      *reinterpret_cast<uintx2_t*>(&Ds[buf][(lrow + 16 * g) * PG_P + lpos]) = sd[g];
      *reinterpret_cast<uintx2_t*>(&Xs[buf][(lrow + 16 * g) * PG_P + lpos]) = sx[g];
      if (do_bias) {
        bsum[g] += Lo16<E>::widen((uint16_t)(sd[g].x & 0xffffu)) + Lo16<E>::widen((uint16_t)(sd[g].x >> 16));
        bsum[g] += Lo16<E>::widen((uint16_t)(sd[g].y & 0xffffu)) + Lo16<E>::widen((uint16_t)(sd[g].y >> 16));
      }
    }
  };

  floatx4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  if (cbeg < cend) {
    gload();
    sstore(0);
  }
  __syncthreads();
  for (int c = cbeg; c < cend; ++c) {
    const int buf = (c - cbeg) & 1;
    if (c + 1 < cend) gload();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(&Ds[buf][((2 * wm + i) * 16 + fr) * PG_P + ks * 32 + 8 * fg]));
        b[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(&Xs[buf][((2 * wn + i) * 16 + fr) * PG_P + ks * 32 + 8 * fg]));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Lo16<E>::mma16(a[i], b[j], acc[i][j]);
    }
    if (c + 1 < cend) sstore(buf ^ 1);
    __syncthreads();
  }

  float* o = out + (size_t)slice * (p.nsplit > 1 ? (size_t)p.E + p.Mo : 0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = c0 + (2 * wn + j) * 16 + fr;
      if (c >= p.C) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + (2 * wm + i) * 16 + 4 * fg + r;
        if (m < p.Mo) o[(size_t)m * p.C + c] = acc[i][j][r];
      }
    }
  if (do_bias) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float b = bsum[g];
      b += __shfl_xor(b, 1, 64);
      b += __shfl_xor(b, 2, 64);
      b += __shfl_xor(b, 4, 64);
      b += __shfl_xor(b, 8, 64);
      if ((tid & 15) == 0 && mv[g]) {
        if (p.nsplit > 1) o[p.E + m0 + lrow + 16 * g] = b;
        else db_direct[m0 + lrow + 16 * g] = b;
      }
    }
  }
}

bool pw16_wgrad_plan(const ConvGeom& g, Pw16WgradParams* p) {
  if (!pw16_applies(g)) return false;
  p->C = g.C; p->Mo = g.K; p->P = g.H * g.W;
  const long long ptot = (long long)g.N * p->P;
  if (ptot * std::max(g.C, g.K) >= (1ll << 31)) return false;
  p->Ptot = (int)ptot;
  p->ctiles = (g.C + 63) / 64;
  p->mtiles = (g.K + 63) / 64;
  p->nchunks = (int)((ptot + PG_KC - 1) / PG_KC);
  p->E = g.K * g.C;
  const long long tiles = (long long)p->ctiles * p->mtiles;
  if (tiles > 65535) return false;
  // every slice costs a write and a read of the whole gradient: fewer slices for large ones
  // (measured on the ResNet-50 layers)
  const int mult = p->E >= 100000 ? 3 : 4;
  long long ns = (long long)mult * mfma_num_cus() / tiles;
  if (ns > p->nchunks / 4) ns = p->nchunks / 4;    // at least four chunks per slice
  if (ns < 1) ns = 1;
  p->cps = (int)((p->nchunks + ns - 1) / ns);
  p->nsplit = (p->nchunks + p->cps - 1) / p->cps;
  return true;
}

// ---- filter gradient, 128 x 128 tiles -------------------------------------------------------
// For layers with at least 128 channels on both sides.  dw[m][c] = sum over (image, position) of
// dy[m][q] x[c][q]: both operands are contiguous along the contraction, so a fragment (one row,
// 8 consecutive positions) is 16 bytes of memory and 16 bytes of LDS - no transposes anywhere.
// A workgroup (4 waves, each 64 x 64 results on v_mfma_f32_32x32x16_bf16) owns dw[128 m][128 c]
// and a slice of the chunks; a chunk = up to 64 positions of ONE image (planes of 49 positions are
// one chunk of four steps, the last with one position; 196 = 3 chunks + one of one step), so a
// row piece never leaves its image.  Thread t loads the 16-byte piece t % 8 of rows t / 8 + 32 g
// (g = 0..3) of both tiles: 8 lanes cover a row's 128 bytes.  A piece that reaches past the end
// of its row is masked in registers (it reads the first bytes of the next row; the very last
// row of a tensor instead reads the 16 bytes that END at the row's end and shifts them down).
constexpr int PG2_T = 128;         // tile side
constexpr int PG2_P = 64 + 8;      // LDS pitch (elements)

struct Pw16Wgrad2Params {
  int C, Mo, P, N;
  int ctiles, mtiles;
  int cpi;                    // chunks per image
  int nchunks, cps, nsplit;   // chunks over the batch, per slice, slices
  int E, want_db;
  unsigned x_bytes, dy_bytes;
};

template <typename E>
__global__ void __launch_bounds__(256, 2)
pw16_wgrad2_kernel(Pw16Wgrad2Params p, const bf16_t* __restrict__ x, const bf16_t* __restrict__ dy,
                   float* __restrict__ out, float* __restrict__ db_direct) {
  extern __shared__ __align__(16) uint16_t lds_pg2[];     // [2 buffers][dy rows 0..127, x rows 128..255][PG2_P]
  constexpr int OOB = (int)0x80000000;
  const int slice = blockIdx.x, mtile = blockIdx.y / p.ctiles, ctile = blockIdx.y - mtile * p.ctiles;
  const int m0 = mtile * PG2_T, c0 = ctile * PG2_T;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 31, fh = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  const int cbeg = slice * p.cps, cend = min(p.nchunks, cbeg + p.cps);
  const __amdgpu_buffer_rsrc_t drsrc = make_rsrc(dy, p.dy_bytes), xrsrc = make_rsrc(x, p.x_bytes);

  const int piece = tid & 7, lrow = tid >> 3;
  int drow[4], xrow[4];        // element offset of the row inside an image, or -1
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int m = m0 + lrow + 32 * g, c = c0 + lrow + 32 * g;
    drow[g] = m < p.Mo ? m * p.P : -1;
    xrow[g] = c < p.C ? c * p.P : -1;
  }
  const float inv_cpi = 1.0f / (float)p.cpi;
  uintx4_t sd[4], sx[4];
  float bsum[4] = {0.f, 0.f, 0.f, 0.f};
  const bool do_bias = p.want_db && ctile == 0;

  // one operand's four pieces of chunk ch; v = positions of the piece inside the row (<= 0: none)
  auto load4 = [&](__amdgpu_buffer_rsrc_t rsrc, const int (&row)[4], int img_elems, unsigned total_bytes, int n, int q,
                   int v, uintx4_t (&dst)[4]) {
    // elements of the piece inside the row -> dword masks
    unsigned mk[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) mk[d] = (v > 2 * d ? 0x0000ffffu : 0u) | (v > 2 * d + 1 ? 0xffff0000u : 0u);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int off = (n * img_elems + row[g] + q) * 2;
      const bool live = row[g] >= 0 && v > 0;
      // the last row of the tensor: a piece that would pass its end
      const bool last = live && v < 8 && (unsigned)(off + 16) > total_bytes;
      uintx4_t t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, live && !last ? off : OOB, 0, 0);
      if (__builtin_amdgcn_ballot_w64(last) != 0) {
        if (last) {
          const uintx4_t u = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off - 2 * (8 - v), 0, 0);
          const unsigned long long lo = ((unsigned long long)u.y << 32) | u.x, hi = ((unsigned long long)u.w << 32) | u.z;
          const int sh = 16 * (8 - v);
          const unsigned long long rl = sh >= 64 ? hi >> (sh - 64) : (lo >> sh) | (hi << (64 - sh));
          const unsigned long long rh = sh >= 64 ? 0ull : hi >> sh;
          t = uintx4_t{(unsigned)rl, (unsigned)(rl >> 32), (unsigned)rh, (unsigned)(rh >> 32)};
        }
      }
      dst[g] = uintx4_t{t.x & mk[0], t.y & mk[1], t.z & mk[2], t.w & mk[3]};
    }
  };
  auto gload = [&](int ch) {
    int k;
    const int n = fast_div(ch, p.cpi, inv_cpi, &k);
    const int q = k * 64 + 8 * piece;
    const int v = p.P - q;
    load4(drsrc, drow, p.Mo * p.P, p.dy_bytes, n, q, v, sd);
    load4(xrsrc, xrow, p.C * p.P, p.x_bytes, n, q, v, sx);
  };
  auto sstore = [&](int buf) {
    uint16_t* b = lds_pg2 + buf * (2 * PG2_T * PG2_P);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      *reinterpret_cast<uintx4_t*>(b + (lrow + 32 * g) * PG2_P + 8 * piece) = sd[g];
      *reinterpret_cast<uintx4_t*>(b + (PG2_T + lrow + 32 * g) * PG2_P + 8 * piece) = sx[g];
      if (do_bias) {
        const unsigned w4[4] = {sd[g].x, sd[g].y, sd[g].z, sd[g].w};
#pragma unroll
        for (int d = 0; d < 4; ++d)
          bsum[g] += Lo16<E>::widen((uint16_t)(w4[d] & 0xffffu)) + Lo16<E>::widen((uint16_t)(w4[d] >> 16));
      }
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  if (cbeg < cend) {
    gload(cbeg);
    sstore(0);
  }
  __syncthreads();
  for (int ch = cbeg; ch < cend; ++ch) {
    const int buf = (ch - cbeg) & 1;
    if (ch + 1 < cend) gload(ch + 1);
    // steps of 16 positions that hold any: the chunk's positions are P - 64 k
    int k;
    fast_div(ch, p.cpi, inv_cpi, &k);
    const int nks = min(4, (p.P - 64 * k + 15) >> 4);
    const uint16_t* b = lds_pg2 + buf * (2 * PG2_T * PG2_P);
    const uint16_t* ap = b + (wm * 64 + fr) * PG2_P + 8 * fh;
    const uint16_t* bp = b + (PG2_T + wn * 64 + fr) * PG2_P + 8 * fh;
    for (int ks = 0; ks < nks; ++ks) {
      bf16x8 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(ap + i * 32 * PG2_P + 16 * ks));
        bf[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(bp + i * 32 * PG2_P + 16 * ks));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Lo16<E>::mma32(af[i], bf[j], acc[i][j]);
    }
    if (ch + 1 < cend) sstore(buf ^ 1);
    __syncthreads();
  }

  // element r of acc[i][j]: row m0 + wm*64 + i*32 + (r/4)*8 + fh*4 + r%4, column c0 + wn*64 + j*32 + fr
  float* o = out + (size_t)slice * (p.nsplit > 1 ? (size_t)p.E + p.Mo : 0);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = c0 + wn * 64 + j * 32 + fr;
      if (c >= p.C) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + fh * 4 + (r & 3);
        if (m < p.Mo) o[(size_t)m * p.C + c] = acc[i][j][r];
      }
    }
  if (do_bias) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float bsm = bsum[g];
      bsm += __shfl_xor(bsm, 1, 64);
      bsm += __shfl_xor(bsm, 2, 64);
      bsm += __shfl_xor(bsm, 4, 64);
      const int m = m0 + lrow + 32 * g;
      if (piece == 0 && m < p.Mo) {
        if (p.nsplit > 1) o[p.E + m] = bsm;
        else db_direct[m] = bsm;
      }
    }
  }
}

bool pw16_wgrad2_plan(const ConvGeom& g, Pw16Wgrad2Params* p) {
  if (!pw16_applies(g) || g.C < PG2_T || g.K < PG2_T || g.H * g.W < 8) return false;
  p->C = g.C; p->Mo = g.K; p->P = g.H * g.W; p->N = g.N;
  const long long xb = (long long)g.N * g.C * p->P * 2, db = (long long)g.N * g.K * p->P * 2;
  if (xb >= (1ll << 31) || db >= (1ll << 31)) return false;
  p->x_bytes = (unsigned)xb;
  p->dy_bytes = (unsigned)db;
  p->ctiles = (g.C + PG2_T - 1) / PG2_T;
  p->mtiles = (g.K + PG2_T - 1) / PG2_T;
  p->cpi = (p->P + 63) / 64;
  p->nchunks = g.N * p->cpi;
  p->E = g.K * g.C;
  const long long tiles = (long long)p->ctiles * p->mtiles;
  if (tiles > 65535) return false;
  // every slice writes and re-reads the whole gradient
#ifndef PG2_MULT
#define PG2_MULT 2
#endif
  long long ns = (long long)PG2_MULT * mfma_num_cus() / tiles;
  if (ns > p->nchunks / 4) ns = p->nchunks / 4;    // at least four chunks per slice
  if (ns < 1) ns = 1;
  p->cps = (int)((p->nchunks + ns - 1) / ns);
  p->nsplit = (p->nchunks + p->cps - 1) / p->cps;
  return true;
}

// ---- strided 1x1 windows ---------------------------------------------------------------
// A 1x1 window with strides reads the input on a lattice.  With room for the lattice
// points as a tensor of their own ([N][C][OH][OW]) the three passes become the stride-1
// passes above plus one copy: gather the lattice (forward, filter gradient) or spread the
// compact gradient over a zeroed dx (backward-data).
__global__ void __launch_bounds__(256)
lattice_gather_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ xc, int H, int W, int OH, int OW,
                      int sy, int sx, uint32_t total) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t ow = i % OW, t = i / OW, oh = t % OH, plane = t / OH;
  xc[i] = x[((size_t)plane * H + (size_t)oh * sy) * W + (size_t)ow * sx];
}

// thread = VEC consecutive elements of a row of dx (W a multiple of VEC)
template <int VEC>
__global__ void __launch_bounds__(256)
lattice_scatter_kernel(const bf16_t* __restrict__ dxc, bf16_t* __restrict__ dx, int H, int W, int OH, int OW,
                       int sy, int sx, uint32_t total) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t per_row = W / VEC, w0 = (i % per_row) * VEC, t = i / per_row, h = t % H, plane = t / H;
  const bool rowv = h % sy == 0;
  const bf16_t* src = dxc + ((size_t)plane * OH + h / sy) * OW;
  uint16_t v[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const uint32_t w = w0 + e;
    v[e] = (rowv && w % sx == 0) ? src[w / sx] : (uint16_t)0;
  }
  bf16_t* d = dx + ((size_t)plane * H + h) * W + w0;
  if constexpr (VEC == 8) {
    *reinterpret_cast<uintx4_t*>(d) = uintx4_t{v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16),
                                               v[4] | ((uint32_t)v[5] << 16), v[6] | ((uint32_t)v[7] << 16)};
  } else if constexpr (VEC == 4) {
    *reinterpret_cast<uintx2_t*>(d) = uintx2_t{v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16)};
  } else if constexpr (VEC == 2) {
    *reinterpret_cast<uint32_t*>(d) = v[0] | ((uint32_t)v[1] << 16);
  } else {
    d[0] = v[0];
  }
}

// the stride-1 problem over the lattice points, if the kernels above take it
bool pw16_strided_plan(const ConvGeom& g, ConvGeom* c) {
  if (!(g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1 && (g.sy > 1 || g.sx > 1))) return false;
  *c = g;
  c->H = g.OH; c->W = g.OW; c->sy = 1; c->sx = 1;
  return pw16_applies(*c);
}
size_t lattice_bytes(const ConvGeom& c) {   // the gathered input / compact dx, rounded for what follows it
  return (((size_t)c.N * c.C * c.H * c.W * sizeof(bf16_t)) + 255) & ~(size_t)255;
}
bool taps_gather(const ConvGeom& g, const void* x, void* xc, hipStream_t s);
void lattice_gather(const ConvGeom& g, const void* x, void* xc, hipStream_t s) {
  // the gather kernel of the windows with several taps (T = 1 here) is the faster copy
  // (11 / 7 us against 15 / 9 us on the 56x56 / 28x28 downsample layers of ResNet-50)
  if (taps_gather(g, x, xc, s)) return;
  const uint32_t total = (uint32_t)((size_t)g.N * g.C * g.OH * g.OW);
  hipLaunchKernelGGL(lattice_gather_kernel, dim3((total + 255) / 256), dim3(256), 0, s, static_cast<const bf16_t*>(x),
                     static_cast<bf16_t*>(xc), g.H, g.W, g.OH, g.OW, g.sy, g.sx, total);
}
void lattice_scatter(const ConvGeom& g, const void* dxc, void* dx, hipStream_t s) {
  const int vec = ((uintptr_t)dx & 15) ? 1 : g.W % 8 == 0 ? 8 : g.W % 4 == 0 ? 4 : g.W % 2 == 0 ? 2 : 1;
  const uint32_t total = (uint32_t)((size_t)g.N * g.C * g.H * g.W / vec);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((total + 255) / 256), dim3(256), 0, s, static_cast<const bf16_t*>(dxc),
                       static_cast<bf16_t*>(dx), g.H, g.W, g.OH, g.OW, g.sy, g.sx, total);
  };
  if (vec == 8) go(lattice_scatter_kernel<8>);
  else if (vec == 4) go(lattice_scatter_kernel<4>);
  else if (vec == 2) go(lattice_scatter_kernel<2>);
  else go(lattice_scatter_kernel<1>);
}


// ---- strided windows with several taps (backward passes), odd rows (filter gradient) ------
// The same idea one step further: with the window's taps gathered next to the channels,
//   xc[n][c * T + tap][oh][ow] = x[n][c][oh sy + kh dly - py][ow sx + kw dlx - px]  (0 outside),
// a strided 3x3 convolution is a 1x1 stride-1 one over C * T channels whose weight matrix is
// the OIHW filter as it lies in memory.  The filter gradient gathers xc and runs the 1x1
// filter-gradient kernel; backward-data runs the 1x1 kernel into the workspace (one bf16
// plane per channel and tap) and sums the taps that reach each element of dx in fp32.
// A workgroup handles the T planes of one (image, channel): contiguous in xc.
// PAIR: a thread makes two neighbouring columns (rows of even length) and stores 4 bytes
// Both kernels below: a workgroup per (image, channel) with threads laid out (columns, rows) over
// the plane - the first dimension is the next power of two that covers a row - so that no index
// needs a division (with a flat index the divisions, not memory, set the pace of these copies).
template <bool PAIR>
__global__ void __launch_bounds__(256)
taps_gather_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ xc, ConvGeom g) {
  constexpr int V = PAIR ? 2 : 1;
  const int P = g.OH * g.OW, T = g.KH * g.KW;
  const int tx = threadIdx.x, ow = tx * V;
  const unsigned plane = blockIdx.x * blockDim.z + threadIdx.z;   // small planes: several per workgroup
  if (ow >= g.OW || plane >= (unsigned)(g.N * g.C)) return;
  const bf16_t* xp = x + (size_t)plane * g.H * g.W;
  bf16_t* op = xc + (size_t)plane * T * P;
  for (int tap = 0; tap < T; ++tap) {
    const int kh = tap / g.KW, kw = tap - kh * g.KW;
    const int dh = kh * g.dly - g.py, dw = kw * g.dlx - g.px;
    for (int oh = threadIdx.y; oh < g.OH; oh += blockDim.y) {
      const int ih = oh * g.sy + dh;
      const bool rv = (unsigned)ih < (unsigned)g.H;
      uint32_t v[V];
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const int iw = (ow + e) * g.sx + dw;
        v[e] = (rv && (unsigned)iw < (unsigned)g.W) ? xp[ih * g.W + iw] : (bf16_t)0;
      }
      bf16_t* o = op + tap * P + oh * g.OW + ow;
      if constexpr (PAIR) *reinterpret_cast<uint32_t*>(o) = v[0] | (v[1] << 16);
      else *o = (bf16_t)v[0];
    }
  }
}

// S2: strides 2, no dilation (parity picks the taps that reach an element, no division by a
// stride); PAIR as above, over the columns of dx
template <typename E, bool S2, bool PAIR>
__global__ void __launch_bounds__(256)
taps_spread_kernel(const bf16_t* __restrict__ dxc, bf16_t* __restrict__ dx, ConvGeom g) {
  constexpr int V = PAIR ? 2 : 1;
  const int P = g.OH * g.OW, T = g.KH * g.KW;
  const int w0 = threadIdx.x * V;
  const unsigned plane = blockIdx.x * blockDim.z + threadIdx.z;
  if (w0 >= g.W || plane >= (unsigned)(g.N * g.C)) return;
  const bf16_t* cp = dxc + (size_t)plane * T * P;
  bf16_t* dp = dx + (size_t)plane * g.H * g.W;
  for (int h = threadIdx.y; h < g.H; h += blockDim.y) {
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const int w = w0 + e;
      acc[e] = 0.f;
      if (S2) {
        // the taps with h + py - kh and w + px - kw even: kh = ((h + py) & 1) + 2a, kw likewise
        // (windows of at most 4 x 4); the four loads are issued together
        const int kh0 = (h + g.py) & 1, kw0 = (w + g.px) & 1;
        uint32_t ld[2][2];
        bool ok[2][2];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            const int kh = kh0 + 2 * a, kw = kw0 + 2 * b;
            const int dh = h + g.py - kh, dw = w + g.px - kw;
            ok[a][b] = kh < g.KH && kw < g.KW && dh >= 0 && dw >= 0 && (dh >> 1) < g.OH && (dw >> 1) < g.OW;
            ld[a][b] = cp[ok[a][b] ? (kh * g.KW + kw) * P + (dh >> 1) * g.OW + (dw >> 1) : 0];
          }
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[e] += ok[a][b] ? Lo16<E>::widen((uint16_t)ld[a][b]) : 0.f;
      } else {
        for (int kh = 0; kh < g.KH; ++kh) {
          const int a = h + g.py - kh * g.dly;
          if (a < 0 || a % g.sy != 0 || a / g.sy >= g.OH) continue;
          for (int kw = 0; kw < g.KW; ++kw) {
            const int b = w + g.px - kw * g.dlx;
            if (b < 0 || b % g.sx != 0 || b / g.sx >= g.OW) continue;
            acc[e] += Lo16<E>::widen(cp[(kh * g.KW + kw) * P + (a / g.sy) * g.OW + b / g.sx]);
          }
        }
      }
    }
    bf16_t* o = dp + h * g.W + w0;
    if constexpr (PAIR) *reinterpret_cast<uint32_t*>(o) = (uint32_t)Lo16<E>::narrow(acc[0]) | ((uint32_t)Lo16<E>::narrow(acc[1]) << 16);
    else *o = Lo16<E>::narrow(acc[0]);
  }
}

// (columns, rows, planes) threads for planes of cols x rows work items: 256 in all, the first
// dimension the next power of two >= cols; rows wider than 256 items do not get here
inline bool plane_block(int cols, int rows, dim3* b) {
  unsigned bx = 1;
  while ((int)bx < cols) bx <<= 1;
  if (bx > 256) return false;
  unsigned by = 256 / bx;
  while (by > 1 && (int)(by / 2) >= rows) by >>= 1;
  *b = dim3(bx, by, 256 / (bx * by));   // planes smaller than 256 items share a workgroup
  return true;
}

bool taps_gather(const ConvGeom& g, const void* x, void* xc, hipStream_t s) {
  const bool pair = g.OW % 2 == 0 && ((uintptr_t)xc & 3) == 0;
  dim3 block;
  if (!plane_block(g.OW / (pair ? 2 : 1), g.OH, &block)) return false;
  const dim3 grid((unsigned)((g.N * g.C + block.z - 1) / block.z));
  if (pair) hipLaunchKernelGGL(taps_gather_kernel<true>, grid, block, 0, s, static_cast<const bf16_t*>(x), static_cast<bf16_t*>(xc), g);
  else hipLaunchKernelGGL(taps_gather_kernel<false>, grid, block, 0, s, static_cast<const bf16_t*>(x), static_cast<bf16_t*>(xc), g);
  return true;
}
template <typename E>
bool taps_spread(const ConvGeom& g, const void* dxc, void* dx, hipStream_t s) {
  const bool pair = g.W % 2 == 0 && ((uintptr_t)dx & 3) == 0;
  const bool s2 = g.sy == 2 && g.sx == 2 && g.dly == 1 && g.dlx == 1 && g.KH <= 4 && g.KW <= 4;
  dim3 block;
  if (!plane_block(g.W / (pair ? 2 : 1), g.H, &block)) return false;
  const dim3 grid((unsigned)((g.N * g.C + block.z - 1) / block.z));
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, static_cast<const bf16_t*>(dxc), static_cast<bf16_t*>(dx), g);
  };
  if (s2) { if (pair) go(taps_spread_kernel<E, true, true>); else go(taps_spread_kernel<E, true, false>); }
  else { if (pair) go(taps_spread_kernel<E, false, true>); else go(taps_spread_kernel<E, false, false>); }
  return true;
}

bool pw16_taps_plan(const ConvGeom& g, ConvGeom* c, bool wgrad = false) {
  const int T = g.KH * g.KW;
  // stride 1: only the filter gradient over rows of odd length, which the row kernel for bf16
  // storage does not take (7x7 planes: 84 us through the taps, 138 us converting; over even rows
  // the row kernel is as fast or faster)
  const bool s1ok = wgrad && g.OW % 2 != 0;
  if (!(g.groups == 1 && T > 1 && T <= 9 && (g.sy > 1 || g.sx > 1 || s1ok))) return false;
  if ((long long)g.N * g.C * T * g.OH * g.OW >= (1ll << 31)) return false;
  if (g.W > 256 || g.OW > 256) return false;   // a row of the plane per row of threads
  *c = g;
  c->C = g.C * T; c->Cg = c->C;
  c->H = g.OH; c->W = g.OW;
  c->KH = 1; c->KW = 1; c->sy = 1; c->sx = 1; c->py = 0; c->px = 0; c->dly = 1; c->dlx = 1;
  return pw16_applies(*c);
}

// Forward through gathered taps (the gather writes 9/4 of the input for a 3x3 stride-2 window, the product
// then runs as a 1x1 layer over C * T channels): where the product goes to the kernels that load straight to LDS
// this beats the slab kernel's strided forward pass (whose loader moves 2.5 times the bytes per product there)
// when that pass would need two rounds of workgroups or more: the stride-2 3x3 layers of ResNet-50 at batch 64
// take 110 / 65 / 102 us on the slab kernel and 73 / 58 / 77 us this way; at batch 32 (one round, two for the
// first) 37 / 33 / 55 against 42 / 45 / 67.
bool pw16_taps_forward(const ConvGeom& g, const ConvGeom& c) {
  if (!((g.sy > 1 || g.sx > 1) && !(options().conv_skip & Options::SKIP_PWDMA) && c.H * c.W <= 1024 && c.K > 64 &&
        c.C % 32 == 0))
    return false;
  const long long slab = mfma_slab16_conv_fwd_workgroups(g);
  return slab == 0 || slab >= 2 * (long long)mfma_num_cus();
}

}  // namespace

size_t mfma_pointwise16_lattice_ws(const ConvGeom& g, bool bwd) {
  ConvGeom c;
  if (pw16_strided_plan(g, &c)) return lattice_bytes(c);
  if (!options().pw16_no_taps && pw16_taps_plan(g, &c) && (bwd || pw16_taps_forward(g, c))) return lattice_bytes(c);
  return 0;
}

// Bytes of the gathered input that the forward pass of this geometry leaves at the start of its workspace and
// that the filter gradient would otherwise gather again (the same kernel, the same layout); 0 when the forward
// pass does not gather.
size_t mfma_pointwise16_gathered_bytes(const ConvGeom& g) {
  ConvGeom c;
  Pw16WgradParams p{};
  if (pw16_strided_plan(g, &c)) return pw16_wgrad_plan(c, &p) ? lattice_bytes(c) : 0;
  if (!options().pw16_no_taps && pw16_taps_plan(g, &c) && pw16_taps_forward(g, c)) {
    ConvGeom cw;
    if (pw16_taps_plan(g, &cw, true) && pw16_wgrad_plan(cw, &p) && lattice_bytes(cw) == lattice_bytes(c)) return lattice_bytes(c);
  }
  return 0;
}

// the compact 1x1 problem of a strided layer: on the kernels that load straight to LDS where those
// are ahead, else on the ones above
template <typename E, bool BWD>
int launch_compact(const ConvGeom& c, const void* src, const void* w, const float* bias, void* dst, hipStream_t s) {
  if (!(options().conv_skip & Options::SKIP_PWDMA)) {
    const int r = BWD ? mfma_pwd16_conv_bwd_data(c, src, w, nullptr, dst, s, Lo16<E>::TAG)
                      : mfma_pwd16_conv_fwd(c, src, w, bias, dst, s, Lo16<E>::TAG);
    if (r >= 0) return r;
  }
  return launch_pw16<E, BWD>(c, src, w, bias, dst, s);
}

template <typename E>
static int pointwise16_conv_fwd_impl(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                                     hipStream_t s, void* ws, size_t ws_bytes) {
  ConvGeom c;
  if (pw16_strided_plan(g, &c)) {
    if (!ws || ws_bytes < lattice_bytes(c)) return -1;
    lattice_gather(g, x, ws, s);
    return launch_compact<E, false>(c, ws, w, bias, y, s);
  }
  if (!options().pw16_no_taps && pw16_taps_plan(g, &c) && pw16_taps_forward(g, c) && ws && ws_bytes >= lattice_bytes(c) &&
      taps_gather(g, x, ws, s))
    return launch_compact<E, false>(c, ws, w, bias, y, s);
  if (!pw16_applies(g)) return -1;
  return launch_pw16<E, false>(g, x, w, bias, y, s);
}

template <typename E>
static int pointwise16_conv_bwd_data_impl(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s,
                                          void* ws, size_t ws_bytes) {
  ConvGeom c;
  if (pw16_strided_plan(g, &c)) {
    if (!ws || ws_bytes < lattice_bytes(c)) return -1;
    const int rc = launch_compact<E, true>(c, dy, w, nullptr, ws, s);
    if (rc != FLHIP_OK) return rc;
    lattice_scatter(g, ws, dx, s);
    return check_launch("conv2d_bwd_data strided 1x1 (bf16 mfma)");
  }
  if (!options().pw16_no_taps && pw16_taps_plan(g, &c)) {
    if (!ws || ws_bytes < lattice_bytes(c)) return -1;
    const int rc = launch_compact<E, true>(c, dy, w, nullptr, ws, s);
    if (rc != FLHIP_OK) return rc;
    if (!taps_spread<E>(g, ws, dx, s)) return fail(FLHIP_RUNTIME_ERROR, "conv2d_bwd_data: plane too wide for the spread kernel");
    return check_launch("conv2d_bwd_data strided window (bf16 mfma)");
  }
  if (!pw16_applies(g)) return -1;
  return launch_pw16<E, true>(g, dy, w, nullptr, dx, s);
}

// dx = addend + backward-data, in the kernel's own result pass; -1 when this geometry's
// backward-data pass is not the plain 1x1 kernel
int mfma_pointwise16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                              hipStream_t s, void* ws, size_t ws_bytes, int dtype) {
  return by_lo16(dtype, [&](auto* e_) { return pointwise16_conv_fwd_impl<FLHIP_T_OF(e_)>(g, x, w, bias, y, s, ws, ws_bytes); });
}

int mfma_pointwise16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s,
                                   void* ws, size_t ws_bytes, int dtype) {
  return by_lo16(dtype, [&](auto* e_) { return pointwise16_conv_bwd_data_impl<FLHIP_T_OF(e_)>(g, dy, w, dx, s, ws, ws_bytes); });
}

int mfma_pointwise16_conv_bwd_data_add(const ConvGeom& g, const void* dy, const void* w, const void* addend, void* dx,
                                       hipStream_t s, int dtype) {
  ConvGeom c;
  if (pw16_strided_plan(g, &c) || (!options().pw16_no_taps && pw16_taps_plan(g, &c)) || !pw16_applies(g)) return -1;
  if (reinterpret_cast<uintptr_t>(addend) % 16 != 0) return -1;
  return by_lo16(dtype, [&](auto* e_) { return launch_pw16<FLHIP_T_OF(e_), true>(g, dy, w, nullptr, dx, s, addend); });
}

size_t mfma_pointwise16_wgrad_ws(const ConvGeom& g0) {
  ConvGeom g = g0;
  size_t lattice = 0;
  if (pw16_strided_plan(g0, &g) || (!options().pw16_no_taps && pw16_taps_plan(g0, &g, true))) lattice = lattice_bytes(g);
  else g = g0;
  Pw16WgradParams p{};
  if (!pw16_wgrad_plan(g, &p)) return 0;
  size_t need = p.nsplit > 1 ? (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float) : 0;
  Pw16Wgrad2Params p2{};
  if (pw16_wgrad2_plan(g, &p2) && p2.nsplit > 1)
    need = std::max(need, (size_t)p2.nsplit * ((size_t)p2.E + p2.Mo) * sizeof(float));
  need = std::max(need, mfma_pwd16_wgrad_ws(g));
  return lattice + need;
}

// (gathered: the gathered input a forward pass left behind - mfma_pointwise16_gathered_bytes() of it -, taken in
// place of x; -1 when this geometry has none)
template <typename E>
static int pointwise16_wgrad_impl(const ConvGeom& g0, const void* x, const void* dy, float* dw, float* db, void* ws,
                                  size_t ws_bytes, hipStream_t s, const void* gathered) {
  if (!dw) return -1;
  ConvGeom g = g0;
  const bool strided = pw16_strided_plan(g0, &g);
  const bool taps = !strided && !options().pw16_no_taps && pw16_taps_plan(g0, &g, true);
  if (!strided && !taps) g = g0;
  Pw16WgradParams p{};
  if (!pw16_wgrad_plan(g, &p)) return -1;
  if (gathered) {
    if (!(strided || taps) || mfma_pointwise16_gathered_bytes(g0) == 0) return -1;
    x = gathered;
  } else if (strided || taps) {
    // the gathered input first, the slices of the gradient behind it
    const size_t lb = lattice_bytes(g);
    if (!ws || ws_bytes < lb) return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
    if (strided) lattice_gather(g0, x, ws, s);
    else if (!taps_gather(g0, x, ws, s)) return fail(FLHIP_RUNTIME_ERROR, "conv2d_bwd_filter: plane too wide for the gather kernel");
    x = ws;
    ws = static_cast<char*>(ws) + lb;
    ws_bytes -= lb;
  }
  if (!db && !(options().conv_skip & Options::SKIP_PWDMA)) {
    const int r = mfma_pwd16_wgrad(g, x, dy, dw, ws, ws_bytes, s, Lo16<E>::TAG);
    if (r >= 0) return r;
  }
  Pw16Wgrad2Params p2{};
  if (!(options().conv_skip & Options::SKIP_WGRAD128) && pw16_wgrad2_plan(g, &p2) && reinterpret_cast<uintptr_t>(x) % 4 == 0 &&
      reinterpret_cast<uintptr_t>(dy) % 4 == 0) {
    p2.want_db = db != nullptr;
    const size_t need2 = p2.nsplit > 1 ? (size_t)p2.nsplit * ((size_t)p2.E + p2.Mo) * sizeof(float) : 0;
    const size_t shmem = (size_t)2 * 2 * PG2_T * PG2_P * sizeof(uint16_t);
    if ((!need2 || (ws && ws_bytes >= need2)) && mfma_allow_lds(reinterpret_cast<const void*>(pw16_wgrad2_kernel<E>), shmem)) {
      float* out2 = p2.nsplit > 1 ? static_cast<float*>(ws) : dw;
      hipLaunchKernelGGL(pw16_wgrad2_kernel<E>, dim3((unsigned)p2.nsplit, (unsigned)(p2.ctiles * p2.mtiles)), dim3(256), shmem, s,
                         p2, static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(dy), out2, db);
      if (p2.nsplit > 1) wgrad_reduce_launch(static_cast<const float*>(ws), p2.nsplit, p2.E, p2.Mo, p2.want_db, dw, db, s);
      return check_launch("conv2d_bwd_filter 1x1 (bf16 mfma, 128 x 128 tiles)");
    }
  }
  p.want_db = db != nullptr;
  const size_t need = p.nsplit > 1 ? (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float) : 0;
  if (need && (!ws || ws_bytes < need)) return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  const dim3 grid((unsigned)p.nsplit, (unsigned)(p.ctiles * p.mtiles));
  if (p.P % 4 == 0)
    hipLaunchKernelGGL((pw16_wgrad_kernel<E, false>), grid, dim3(256), 0, s, p, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(dy), out, db);
  else
    hipLaunchKernelGGL((pw16_wgrad_kernel<E, true>), grid, dim3(256), 0, s, p, static_cast<const bf16_t*>(x),
                       static_cast<const bf16_t*>(dy), out, db);
  if (p.nsplit > 1) wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.Mo, p.want_db, dw, db, s);
  return check_launch("conv2d_bwd_filter 1x1 (bf16 mfma)");
}

int mfma_pointwise16_wgrad(const ConvGeom& g0, const void* x, const void* dy, float* dw, float* db, void* ws,
                           size_t ws_bytes, hipStream_t s, const void* gathered, int dtype) {
  return by_lo16(dtype, [&](auto* e_) {
    return pointwise16_wgrad_impl<FLHIP_T_OF(e_)>(g0, x, dy, dw, db, ws, ws_bytes, s, gathered);
  });
}

}  // namespace flhip
