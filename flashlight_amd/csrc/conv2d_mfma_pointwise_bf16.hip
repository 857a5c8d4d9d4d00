// 1x1 stride-1 convolutions in bf16 storage on the bf16 matrix cores
// (v_mfma_f32_16x16x32_bf16, fp32 accumulate): forward, backward-data and the filter
// gradient.  Per image the tensors are [channels][positions] with positions contiguous.
//
//   forward        y[m][q]  = sum_c w[m][c]  x[c][q]  (+ bias[m])
//   backward-data  dx[c][q] = sum_m w[m][c] dy[m][q]
// contract over the ROW index of the source, but an MFMA lane wants eight consecutive
// contraction indices of one position.  The source tile goes to LDS as it is in memory
// ([32 channels][128 positions]) and a lane gathers its eight channels with eight 16-bit
// LDS reads (a pitch of 130 elements puts the four lane groups of a read in disjoint
// banks); eight matrix instructions per wave and chunk pay for 16 + 4 such reads.
// Weights: forward [m][c] is contraction-contiguous (16-byte LDS reads), backward-data
// contracts over m and gathers like the source.  Positions are the rows of the
// instruction tile, so a lane ends up with four consecutive positions of one result
// channel: one 8-byte store.  Positions are flattened over the batch (a plane of 14x14
// would waste a quarter of a 128-wide tile per image); planes must be a multiple of 4
// positions so that a 4-position run stays inside one image and is 8-byte aligned.
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
constexpr int PB_XP = PB_BP + 2;   // source tile pitch (elements)
constexpr int PB_WP = PB_KC + 8;   // weight tile pitch ([result channel][contraction])

struct Pw16Params {
  int Kc, Mo;        // contraction channels, result channels
  int P, Ptot;       // positions per image, over the batch
  int nchunks, mtiles, ptiles;
};

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uintx4_t v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}

// eight elements of one column, rows r0 .. r0+7, of a 16-bit LDS tile
__device__ __forceinline__ bf16x8 gather8(const uint16_t* tile, int pitch, int r0, int col) {
  const uint16_t* t = tile + r0 * pitch + col;
  const uint32_t a = (uint32_t)t[0] | ((uint32_t)t[pitch] << 16);
  const uint32_t b = (uint32_t)t[2 * pitch] | ((uint32_t)t[3 * pitch] << 16);
  const uint32_t c = (uint32_t)t[4 * pitch] | ((uint32_t)t[5 * pitch] << 16);
  const uint32_t d = (uint32_t)t[6 * pitch] | ((uint32_t)t[7 * pitch] << 16);
  return as_bf16x8(a, b, c, d);
}

// BWD = false: forward (weights [Mo][Kc]); true: backward-data (weights [Kc][Mo]).
// MT = 16-channel result tiles per workgroup (4: 64 result channels; 8 was measured and
// is slower on every ResNet-50 layer, as is loading two chunks ahead instead of one).
template <bool BWD, int MT>
__global__ void __launch_bounds__(256)
pw16_conv_kernel(Pw16Params p, const bf16_t* __restrict__ src, const bf16_t* __restrict__ wgt,
                 const float* __restrict__ bias, bf16_t* __restrict__ dst) {
  constexpr int BM = MT * 16, WQ = BM / 64;      // result channels; 16-byte weight pieces per thread
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
  const bf16_t* sp = src + (size_t)img * p.Kc * p.P + pos;
  struct Stage {
    uintx2_t x[4];
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
      st.x[i] = (qv && k < p.Kc) ? *reinterpret_cast<const uintx2_t*>(sp + (size_t)k * p.P) : uintx2_t{0u, 0u};
    }
#pragma unroll
    for (int h = 0; h < WQ; ++h) {
      if (BWD) {
        const int k = k0 + wr, m = m0 + wc + 64 * h;
        st.w[h] = (k < p.Kc && m < p.Mo) ? *reinterpret_cast<const uintx4_t*>(wgt + (size_t)k * p.Mo + m)
                                         : uintx4_t{0u, 0u, 0u, 0u};
      } else {
        const int m = m0 + wr + 64 * h, k = k0 + wc;
        st.w[h] = (m < p.Mo && k < p.Kc) ? *reinterpret_cast<const uintx4_t*>(wgt + (size_t)m * p.Kc + k)
                                         : uintx4_t{0u, 0u, 0u, 0u};
      }
    }
  };
  // Weights live in LDS as [result channel m][contraction k], 8-element contraction groups
  // g stored at group slot g ^ ((m >> 3) & 3).  Forward copies 16-byte pieces; backward-data
  // holds eight result channels of one k per piece and scatters them (the swizzle spreads
  // those 16-bit stores over the banks).
  auto wslot = [](int m, int g) { return m * PB_WP + 8 * (g ^ ((m >> 3) & 3)); };
  auto sstore = [&](int buf, const Stage& st) {
    uint16_t* X = Xs0 + buf * XSZ;
    uint16_t* Wt = Ws0 + buf * WSZ;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t* d = reinterpret_cast<uint32_t*>(&X[(lr + 8 * i) * PB_XP + lq]);
      d[0] = st.x[i].x;
      d[1] = st.x[i].y;
    }
#pragma unroll
    for (int h = 0; h < WQ; ++h) {
      if (BWD) {
        const uint32_t v[4] = {st.w[h].x, st.w[h].y, st.w[h].z, st.w[h].w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int m = wc + 64 * h + e;
          Wt[wslot(m, wr >> 3) + (wr & 7)] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
        }
      } else {
        *reinterpret_cast<uintx4_t*>(&Wt[wslot(wr + 64 * h, wc >> 3)]) = st.w[h];
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
    for (int i = 0; i < 2; ++i) a[i] = gather8(X, PB_XP, 8 * fg, wave * 32 + i * 16 + fr);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(&Wt[wslot(j * 16 + fr, fg)]));
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b, acc[i][j], 0, 0, 0);
    }
  };

  const int n = p.nchunks;
  Stage st;
  gload(0, st);
  sstore(0, st);
  __syncthreads();
  for (int c = 0; c < n; ++c) {
    if (c + 1 < n) gload(c + 1, st);
    compute(c & 1);
    if (c + 1 < n) sstore((c + 1) & 1, st);
    __syncthreads();
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
      const uintx2_t o = {(uint32_t)f32_to_bf16(acc[i][j][0] + bv) | ((uint32_t)f32_to_bf16(acc[i][j][1] + bv) << 16),
                          (uint32_t)f32_to_bf16(acc[i][j][2] + bv) | ((uint32_t)f32_to_bf16(acc[i][j][3] + bv) << 16)};
      *reinterpret_cast<uintx2_t*>(&Ys[ml * YP + wave * 32 + i * 16 + 4 * fg]) = o;
    }
  __syncthreads();
  if ((p.P & 7) == 0) {
    const int pc = (tid & 15) * 8, qo = q0 + pc;
    if (qo < p.Ptot) {
      const int im = qo / p.P, po = qo - im * p.P;
      bf16_t* dp = dst + (size_t)im * p.Mo * p.P + po;
      for (int ml = tid >> 4; ml < BM && m0 + ml < p.Mo; ml += 16)
        *reinterpret_cast<uintx4_t*>(dp + (size_t)(m0 + ml) * p.P) = *reinterpret_cast<const uintx4_t*>(&Ys[ml * YP + pc]);
    }
  } else {
    const int pc = (tid & 31) * 4, qo = q0 + pc;
    if (qo < p.Ptot) {
      const int im = qo / p.P, po = qo - im * p.P;
      bf16_t* dp = dst + (size_t)im * p.Mo * p.P + po;
      for (int ml = tid >> 5; ml < BM && m0 + ml < p.Mo; ml += 8)
        *reinterpret_cast<uintx2_t*>(dp + (size_t)(m0 + ml) * p.P) = *reinterpret_cast<const uintx2_t*>(&Ys[ml * YP + pc]);
    }
  }
}

bool pw16_applies(const ConvGeom& g) {
  return g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1 && g.sy == 1 && g.sx == 1 &&
         g.OH == g.H && g.OW == g.W && (g.H * g.W) % 4 == 0 && g.C % 8 == 0 && g.K % 8 == 0;
}

template <bool BWD>
int launch_pw16(const ConvGeom& g, const void* src, const void* w, const float* bias, void* dst, hipStream_t s) {
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
  hipLaunchKernelGGL((pw16_conv_kernel<BWD, 4>), dim3((unsigned)grid), dim3(256), 0, s, p,
                     static_cast<const bf16_t*>(src), static_cast<const bf16_t*>(w), bias,
                     static_cast<bf16_t*>(dst));
  return check_launch(BWD ? "conv2d_bwd_data 1x1 (bf16 mfma)" : "conv2d_fwd 1x1 (bf16 mfma)");
}

}  // namespace

int mfma_pointwise16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                              hipStream_t s) {
  if (!pw16_applies(g)) return -1;
  return launch_pw16<false>(g, x, w, bias, y, s);
}

int mfma_pointwise16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s) {
  if (!pw16_applies(g)) return -1;
  return launch_pw16<true>(g, dy, w, nullptr, dx, s);
}

}  // namespace flhip
