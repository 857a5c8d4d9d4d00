// 1x1 convolutions without padding as GEMMs on the gfx950 fp32 matrix cores:
// forward and backward-data, any stride.
//
// With a 1x1 window the result is, per image n,
//   D[n][m][map_d(q)] = sum_k A[m][k] * S[n][k][map_s(q)],   q = 0 .. P-1,
//   forward : S = x, A = w [K][C] (k contiguous), P = OH*OW, map_s = the stride
//             lattice of the input, map_d = identity;
//   backward: S = dy, A = w^T (m contiguous), P = OH*OW, map_s = identity,
//             map_d = the stride lattice of dx (the other elements of dx are zero
//             and are cleared by a fill kernel first).
// For stride 1 both maps are the identity and a channel plane is one contiguous row
// of the GEMM, so operands and results move as 16-byte vectors.
//
// A workgroup owns 64 result channels x BN = 32*PT positions (positions run across
// image boundaries; PT = 2 by default) and has 8 waves with two roles, as the other MFMA
// kernels here:
//   waves 0-3 (loaders) fetch chunk c+2 (32 contraction channels of the source tile
//     and of the weight tile) into registers while chunk c+1 waits in a second
//     register set, and store it into the LDS buffer the MFMA waves are not reading;
//   waves 4-7 (MFMA), arranged 2 (positions) x 2 (channels), own 16*PT positions x 32
//     channels each and issue the chunk's MFMAs from 8-byte LDS fragment reads.
// One barrier per chunk; two LDS buffers.
//
// LDS layouts (one buffer): source xs[16 pairs][XPS] with float2 {channel 2j, 2j+1} per
// position, so one 8-byte read feeds two MFMAs (the k index of v_mfma_f32_16x16x4_f32
// is the lane group; the first MFMA takes the even channels of a pair-step, the
// second the odd ones).  Weights: forward as[64 m][APW] (k contiguous, the memory
// order), backward as[16 pairs][APS] with float2 per result channel.  Pitches are
// chosen so that the 32 lanes of one read pass touch distinct banks.
//
// The matrix-core operands are swapped against the usual convention: the source
// tile is the A operand (rows = positions), the weights the B operand, so that a
// lane's four accumulator values are four consecutive positions of one channel and
// leave as one 16-byte store.
#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int KC = 32;                 // contraction channels per chunk
constexpr int NPAIR = KC / 2;
constexpr int BM = MFMA_BM;            // result channels per workgroup
constexpr int APW = KC + 4;            // forward weight pitch: 16 channels x 2 lane groups hit 64 banks
constexpr int APS = 2 * BM + 32;       // backward weight pair stride (== 32 mod 64)
constexpr int LTHREADS = 256;
constexpr int OOB = (int)0x80000000;

struct PwParams {
  int Kc, Mo;            // contraction / result channels
  int SP, DP;            // elements per source / result channel plane
  int P, Ptot;           // GEMM positions per image, over all images
  int OW;                // positions per row of the strided lattice
  int rowstep, colstep;  // lattice: element (q / OW) * rowstep + (q % OW) * colstep
  int src_map, dst_map;  // 1 = that side goes through the lattice
  int vec_w;             // weight tile by 16-byte loads
  int nchunks, mtiles, ptiles;
  int cps;               // chunks per contraction slice (blockIdx.y); == nchunks without split-K
  unsigned dst_slice;    // elements between the partial results of consecutive slices
  unsigned src_bytes, wgt_bytes, dst_bytes;
};

__device__ __forceinline__ int lattice(const PwParams& p, int q) {
  const int r = q / p.OW;
  return r * p.rowstep + (q - r * p.OW) * p.colstep;
}

template <typename T>
__device__ __forceinline__ void buf_st1(__amdgpu_buffer_rsrc_t r, int byte_off, float v, T*);
template <>
__device__ __forceinline__ void buf_st1<float>(__amdgpu_buffer_rsrc_t r, int byte_off, float v, float*) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, byte_off, 0, 0);
}
template <>
__device__ __forceinline__ void buf_st1<bf16_t>(__amdgpu_buffer_rsrc_t r, int byte_off, float v, bf16_t*) {
  __builtin_amdgcn_raw_buffer_store_b16(f32_to_bf16(v), r, byte_off, 0, 0);
}
template <>
__device__ __forceinline__ void buf_st1<f16_t>(__amdgpu_buffer_rsrc_t r, int byte_off, float v, f16_t*) {
  __builtin_amdgcn_raw_buffer_store_b16(f32_to_f16(v).bits, r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st4v(__amdgpu_buffer_rsrc_t r, int byte_off, floatx4 v, f16_t*) {
  const uintx2_t t = {pack_f16(v[0], v[1]), pack_f16(v[2], v[3])};
  __builtin_amdgcn_raw_buffer_store_b64(t, r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st4v(__amdgpu_buffer_rsrc_t r, int byte_off, floatx4 v, float*) {
  const uintx4_t t = {__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]),
                      __float_as_uint(v[3])};
  __builtin_amdgcn_raw_buffer_store_b128(t, r, byte_off, 0, 0);
}
__device__ __forceinline__ void buf_st4v(__amdgpu_buffer_rsrc_t r, int byte_off, floatx4 v, bf16_t*) {
  const uintx2_t t = {(uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16),
                      (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16)};
  __builtin_amdgcn_raw_buffer_store_b64(t, r, byte_off, 0, 0);
}

// The MFMA waves' share of one chunk (32 contraction channels = 4 pair-steps): wave
// (wp, wc) multiplies positions wp*16*PT .. by channels wc*32 .. out of the LDS buffer
// `buf` (source tile, then weight tile) into its PT x 2 accumulator tiles.
template <bool BWD, int PT>
__device__ __forceinline__ void mfma_chunk(const float* buf, int wp, int wc, int fr, int fg,
                                           floatx4 (&acc)[PT][2]) {
  constexpr int XPS = 2 * 32 * PT + 32;
  const float* xs = buf + fg * XPS + (wp * PT * 16 + fr) * 2;
  const float* as = buf + NPAIR * XPS + (BWD ? fg * APS + (wc * 32 + fr) * 2 : (wc * 32 + fr) * APW + 2 * fg);
#pragma unroll
  for (int s = 0; s < KC / 8; ++s) {
    float2 a[PT], b[2];
#pragma unroll
    for (int i = 0; i < PT; ++i) a[i] = *reinterpret_cast<const float2*>(xs + 4 * s * XPS + i * 32);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      b[j] = *reinterpret_cast<const float2*>(as + (BWD ? 4 * s * APS + j * 32 : j * 16 * APW + 8 * s));
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // .x / .y: the even / odd channel of the lane group's pair = two k-steps
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].x, b[j].x, acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].y, b[j].y, acc[i][j], 0, 0, 0);
      }
  }
}

template <typename T, bool BWD, int PT, bool VEC>
__global__ void __launch_bounds__(MFMA_THREADS)
pointwise_conv_kernel(PwParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                      const float* __restrict__ bias, T* __restrict__ dst) {
  constexpr int BN = 32 * PT;               // positions per workgroup
  constexpr int XPS = 2 * BN + 32;          // source pair stride in words (== 32 mod 64)
  constexpr int QN = BN / 4;                // position quads per tile
  constexpr int JSTEP = LTHREADS / QN;      // pairs covered by one sweep of the loader threads
  constexpr int NJ = NPAIR / JSTEP;         // sweeps per chunk
  constexpr int ASZ = BWD ? NPAIR * APS : BM * APW;
  constexpr int BUF = NPAIR * XPS + ASZ;
  constexpr int esz = (int)sizeof(T);
  static_assert(NJ >= 1 && NJ * JSTEP == NPAIR, "tile shape");
  extern __shared__ float lds[];            // [2][BUF]: source tile, then weight tile

  // XCD-aware tile order: consecutive workgroups go to different XCDs, so the tiles
  // that share a source tile (all channel tiles of one position tile) are put on
  // one XCD, back to back
  const int id = blockIdx.x, xcd = id & 7, seq = id >> 3;
  const int mtile = __builtin_amdgcn_readfirstlane(seq % p.mtiles);
  const int ptile = __builtin_amdgcn_readfirstlane((seq / p.mtiles) * 8 + xcd);
  if (ptile >= p.ptiles) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tileP0 = ptile * BN;
  // split-K: slice blockIdx.y takes chunks [c0, c0 + n) and writes its own partial result
  const int c0 = blockIdx.y * p.cps;
  const int n = min(p.nchunks - c0, p.cps);

  if (wave < 4) {
    // ================================ loaders ====================================
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wgt_bytes);
    const int pq = tid % QN, j0 = tid / QN;
    const int SPb = p.SP * esz;
    // 16-byte path: byte offset of channel 0 at this thread's four positions; element-wise
    // path: a lane owns one position of the tile (a wave's load of one channel is then a
    // contiguous run wherever the map allows) and the wave the channel pairs 4*wave .. +3
    static_assert(VEC || PT == 2, "the element-wise loaders assume 64 positions per tile");
    int sb;
    {
      const int Pg = VEC ? tileP0 + 4 * pq : tileP0 + lane;
      const int ni = Pg / p.P, q = Pg - ni * p.P;
      sb = Pg < p.Ptot ? (ni * p.Kc * p.SP + ((!VEC && p.src_map) ? lattice(p, q) : q)) * esz : OOB;
    }
    // weight tile shares: forward (m, 4 consecutive k), backward (pair, 4 consecutive m)
    const int wm = BWD ? (tid & 15) * 4 : tid >> 3;       // backward: first of 4 channels
    const int wk = BWD ? (tid >> 4) * 2 : (tid & 7) * 4;  // first contraction index inside the chunk
    const int m0 = mtile * BM;

    auto load = [&](int c, float4 (&sr)[NJ][2], float4 (&wr)[2]) {
      const int k0 = (c0 + c) * KC;
      if (VEC) {
#pragma unroll
        for (int i = 0; i < NJ; ++i) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int k = k0 + 2 * (j0 + i * JSTEP) + h;
            sr[i][h] = buf_ld4(srsrc, (k < p.Kc && sb != OOB) ? sb + k * SPb : OOB, src);
          }
        }
      } else {
        // sr[0][h] = channels k0 + 8*wave + 4h .. +3 at this lane's position
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int k = k0 + 8 * wave + 4 * h + e;
            v[e] = buf_ld(srsrc, (k < p.Kc && sb != OOB) ? sb + k * SPb : OOB, src);
          }
          sr[0][h] = make_float4(v[0], v[1], v[2], v[3]);
        }
      }
      if (!BWD) {
        // rows m = wm and wm + 32, columns k0 + wk .. +3 of w[m][k]
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int m = m0 + wm + 32 * i, k = k0 + wk;
          const int off = (m * p.Kc + k) * esz;
          if (p.vec_w) {
            wr[i] = buf_ld4(wrsrc, (m < p.Mo && k < p.Kc) ? off : OOB, wgt);
          } else {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              v[e] = buf_ld(wrsrc, (m < p.Mo && k + e < p.Kc) ? off + e * esz : OOB, wgt);
            wr[i] = make_float4(v[0], v[1], v[2], v[3]);
          }
        }
      } else {
        // rows k = k0 + wk and +1, columns m0 + wm .. +3 of w[k][m]
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int k = k0 + wk + h, m = m0 + wm;
          const int off = (k * p.Mo + m) * esz;
          if (p.vec_w) {
            wr[h] = buf_ld4(wrsrc, (k < p.Kc && m < p.Mo) ? off : OOB, wgt);
          } else {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              v[e] = buf_ld(wrsrc, (k < p.Kc && m + e < p.Mo) ? off + e * esz : OOB, wgt);
            wr[h] = make_float4(v[0], v[1], v[2], v[3]);
          }
        }
      }
    };
    auto store = [&](int buf, const float4 (&sr)[NJ][2], const float4 (&wr)[2]) {
      float* xs = lds + buf * BUF;
      float* as = xs + NPAIR * XPS;
      if (VEC) {
#pragma unroll
        for (int i = 0; i < NJ; ++i) {
          float4* d = reinterpret_cast<float4*>(xs + (j0 + i * JSTEP) * XPS + 8 * pq);
          d[0] = make_float4(sr[i][0].x, sr[i][1].x, sr[i][0].y, sr[i][1].y);
          d[1] = make_float4(sr[i][0].z, sr[i][1].z, sr[i][0].w, sr[i][1].w);
        }
      } else {
        float* d = xs + 4 * wave * XPS + 2 * lane;
        *reinterpret_cast<float2*>(d) = make_float2(sr[0][0].x, sr[0][0].y);
        *reinterpret_cast<float2*>(d + XPS) = make_float2(sr[0][0].z, sr[0][0].w);
        *reinterpret_cast<float2*>(d + 2 * XPS) = make_float2(sr[0][1].x, sr[0][1].y);
        *reinterpret_cast<float2*>(d + 3 * XPS) = make_float2(sr[0][1].z, sr[0][1].w);
      }
      if (!BWD) {
        *reinterpret_cast<float4*>(as + wm * APW + wk) = wr[0];
        *reinterpret_cast<float4*>(as + (wm + 32) * APW + wk) = wr[1];
      } else {
        float4* d = reinterpret_cast<float4*>(as + (wk >> 1) * APS + 2 * wm);
        d[0] = make_float4(wr[0].x, wr[1].x, wr[0].y, wr[1].y);
        d[1] = make_float4(wr[0].z, wr[1].z, wr[0].w, wr[1].w);
      }
    };

    float4 srA[NJ][2], wrA[2], srB[NJ][2], wrB[2];
    load(0, srA, wrA);
    store(0, srA, wrA);
    load(1, srB, wrB);
    __syncthreads();
    for (int c = 0; c < n; c += 2) {
      load(c + 2, srA, wrA);
      store(1, srB, wrB);                      // chunk c+1
      __syncthreads();
      if (c + 1 >= n) break;
      load(c + 3, srB, wrB);
      store(0, srA, wrA);                      // chunk c+2
      __syncthreads();
    }
    return;
  }

  // ================================ MFMA waves ===================================
  const int cw = wave - 4;
  const int wp = cw & 1, wc = cw >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  floatx4 acc[PT][2];
#pragma unroll
  for (int i = 0; i < PT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  __syncthreads();                             // chunk 0 is in buffer 0
  for (int c = 0; c < n; ++c) {
    mfma_chunk<BWD, PT>(lds + (c & 1) * BUF, wp, wc, fr, fg, acc);
    __syncthreads();
  }

  // ---- epilogue: a lane holds positions Pg .. Pg+3 of channel ch per accumulator ----
  const __amdgpu_buffer_rsrc_t drsrc = make_rsrc(dst + (size_t)blockIdx.y * p.dst_slice, p.dst_bytes);
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const int Pg = tileP0 + (wp * PT + i) * 16 + 4 * fg;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ch = mtile * BM + wc * 32 + j * 16 + fr;
      floatx4 v = acc[i][j];
      if (bias && ch < p.Mo && blockIdx.y == 0) {
        const float bv = bias[ch];
        v[0] += bv; v[1] += bv; v[2] += bv; v[3] += bv;
      }
      if (VEC) {
        const int ni = Pg / p.P, q = Pg - ni * p.P;
        const bool ok = Pg < p.Ptot && ch < p.Mo;
        buf_st4v(drsrc, ok ? ((ni * p.Mo + ch) * p.DP + q) * esz : OOB, v, dst);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int Pe = Pg + e;
          const int ni = Pe / p.P, q = Pe - ni * p.P;
          const bool ok = Pe < p.Ptot && ch < p.Mo;
          const int off = ((ni * p.Mo + ch) * p.DP + (p.dst_map ? lattice(p, q) : q)) * esz;
          buf_st1<T>(drsrc, ok ? off : OOB, v[e], dst);
        }
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) zero_kernel(T* __restrict__ p, size_t n16, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  uint4* q = reinterpret_cast<uint4*>(p);
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride)
    q[i] = make_uint4(0, 0, 0, 0);
  constexpr size_t per = 16 / sizeof(T);
  for (size_t i = n16 * per + (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = T{};
}

template <typename T, bool BWD, int PT, bool VEC>
int launch_tile(const PwParams& p0, const void* src, const void* wgt, const float* bias, void* dst,
                hipStream_t s) {
  PwParams p = p0;
  constexpr int BN = 32 * PT;
  p.ptiles = (p.Ptot + BN - 1) / BN;
  const size_t shmem = (size_t)2 * (NPAIR * (2 * BN + 32) + (BWD ? NPAIR * APS : BM * APW)) * sizeof(float);
  auto kernel = pointwise_conv_kernel<T, BWD, PT, VEC>;
  if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
  const unsigned grid = (unsigned)(((p.ptiles + 7) / 8) * 8 * p.mtiles);
  if (p.cps <= 0 || p.cps > p.nchunks) p.cps = p.nchunks;
  const unsigned slices = (unsigned)((p.nchunks + p.cps - 1) / p.cps);
  hipLaunchKernelGGL(kernel, dim3(grid, slices), dim3(MFMA_THREADS), shmem, s, p, static_cast<const T*>(src),
                     static_cast<const T*>(wgt), bias, static_cast<T*>(dst));
  return check_launch("conv2d 1x1 (mfma)");
}

template <typename T, bool BWD>
int launch_pw(const PwParams& p, bool vec, const void* src, const void* wgt, const float* bias,
              void* dst, hipStream_t s) {
  // 64 x 64 tiles: four workgroups share a CU (39 KB of LDS each), so the load
  // latency at the start of one tile and the stores at its end overlap the MFMA phase
  // of the others; measured faster than 64 x 128 and 64 x 256 on every ResNet-50 1x1
  // layer (the switch PW_PT=4|8 selects those, a measurement aid)
  const int pt = options().pw_pt;
  if (vec) {
    if (pt == 8) return launch_tile<T, BWD, 8, true>(p, src, wgt, bias, dst, s);
    if (pt == 4) return launch_tile<T, BWD, 4, true>(p, src, wgt, bias, dst, s);
    return launch_tile<T, BWD, 2, true>(p, src, wgt, bias, dst, s);
  }
  return launch_tile<T, BWD, 2, false>(p, src, wgt, bias, dst, s);
}

// ---- windows with several taps, any stride, padding and dilation ------------------------
// The same GEMM with the contraction running over (channel chunk, tap): for a tap the
// source position of a result position is shifted by the tap's (dh, dw) and is
// outside the image for some positions (padding), which the loaders turn into
// out-of-range offsets (zero).  Positions are enumerated per "class":
//   forward : one class, the whole result grid, every tap;
//   backward: one class per residue ((ih + py) mod sy, (iw + px) mod sx) of the dx
//             grid.  Only the taps with kh*dil_y = that residue (mod sy) reach a class,
//             and for those (ih + py - kh*dil_y) / sy is exact, so a class is a stride-1
//             problem over dy whose results land on a lattice of dx.  Every element of dx
//             belongs to exactly one class (a class without taps stores zeros), and no
//             multiplication is spent on taps that cannot contribute.
// Tiles are 64 channels x 64 positions of one class; loads and stores are element-wise.
constexpr int MAX_CLASSES = 16;
constexpr int MAX_TAPS = 128;          // over all classes
constexpr int DEPTH = 2;               // chunks in flight per loader thread (even); 4 measured no faster

struct TapClass {
  int tile0;             // first position tile of the class
  int Hc, Wc;            // class grid
  int h0, w0;            // result coordinates of class grid (0, 0)
  int bh, bw;            // source coordinates of class grid (0, 0) at shift (0, 0)
  int tap0, ntaps;
};
struct Tap {
  short dh, dw;          // source shift
  int tmem;              // tap index in the weights (kh * KW + kw)
};
struct TapParams {
  int N, Kc, Mo;
  int SH, SW, DH, DW;    // source / result planes
  int KHW;
  int ssh, ssw;          // source step per class grid step
  int rsh, rsw;          // result step per class grid step
  int kchunks, mtiles, ptiles, nclasses;
  int wre;               // weights were reordered to [tap][row][column] (see reorder_taps_kernel)
  unsigned src_bytes, wgt_bytes, dst_bytes;
  TapClass cls[MAX_CLASSES];
  Tap taps[MAX_TAPS];
};

template <typename T, bool BWD>
__global__ void __launch_bounds__(MFMA_THREADS)
tapped_conv_kernel(TapParams p, const T* __restrict__ src, const T* __restrict__ wgt,
                   const float* __restrict__ bias, T* __restrict__ dst) {
  constexpr int PT = 2, BN = 32 * PT;
  constexpr int XPS = 2 * BN + 32;
  constexpr int ASZ = BWD ? NPAIR * APS : BM * APW;
  constexpr int BUF = NPAIR * XPS + ASZ;
  constexpr int esz = (int)sizeof(T);
  static_assert(BN == 64 && NPAIR == 16, "a loader wave covers 64 positions x 4 channel pairs");
  __shared__ float lds[2 * BUF];

  const int id = blockIdx.x, xcd = id & 7, seq = id >> 3;
  const int mtile = __builtin_amdgcn_readfirstlane(seq % p.mtiles);
  const int ptile = __builtin_amdgcn_readfirstlane((seq / p.mtiles) * 8 + xcd);
  if (ptile >= p.ptiles) return;
  int cl = 0;
  while (cl + 1 < p.nclasses && ptile >= p.cls[cl + 1].tile0) ++cl;
  cl = __builtin_amdgcn_readfirstlane(cl);
  const int Hc = p.cls[cl].Hc, Wc = p.cls[cl].Wc, ntaps = p.cls[cl].ntaps, tap0 = p.cls[cl].tap0;
  const int Pc = Hc * Wc, Pctot = p.N * Pc;
  const int tileP0 = (ptile - p.cls[cl].tile0) * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = p.kchunks * ntaps;

  if (wave < 4) {
    // ================================ loaders ====================================
    // A thread owns one position of the tile (lane = position, so a wave's load of one
    // channel is one contiguous run wherever the source step is 1) and the four channel
    // pairs 4*wave .. 4*wave+3 of a chunk.
    const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
    const __amdgpu_buffer_rsrc_t wrsrc = make_rsrc(wgt, p.wgt_bytes);
    const int SPb = p.SH * p.SW * esz;
    int nb, sh0, sw0;
    {
      const int Pe = tileP0 + lane;
      const int ni = Pe / Pc, r = Pe - ni * Pc;
      const int hc = r / Wc, wcl = r - hc * Wc;
      nb = ni * p.Kc * SPb;
      // a position past the class gets a row that fails every bounds test
      sh0 = Pe < Pctot ? hc * p.ssh + p.cls[cl].bh : -(1 << 24);
      sw0 = wcl * p.ssw + p.cls[cl].bw;
    }
    // weight tile: lanes run along the dimension whose stride is one tap group (KHW
    // elements); forward (k = tid % 32, m = tid / 32 + 8i), backward (m = tid % 64,
    // k = tid / 64 + 4i)
    const int wl = BWD ? tid & 63 : tid & 31;
    const int wo = BWD ? tid >> 6 : tid >> 5;
    const int m0 = mtile * BM;
    int kc = 0, ti = 0;                        // chunk = (channel chunk kc, tap ti), taps inner

    auto load = [&](float (&sr)[8], float (&wr)[8]) {
      const Tap tp = p.taps[min(tap0 + ti, MAX_TAPS - 1)];
      const int k0 = kc * KC;
      const int ih = sh0 + tp.dh, iw = sw0 + tp.dw;
      const bool ok = (unsigned)ih < (unsigned)p.SH && (unsigned)iw < (unsigned)p.SW && ntaps > 0;
      const int so = nb + (ih * p.SW + iw) * esz + (k0 + 8 * wave) * SPb;
#pragma unroll
      for (int h = 0; h < 8; ++h)
        sr[h] = buf_ld(srsrc, (ok && k0 + 8 * wave + h < p.Kc) ? so + h * SPb : OOB, src);
      if (!BWD) {
        const int k = k0 + wl;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int m = m0 + wo + 8 * i;
          const int wo_ = p.wre ? (tp.tmem * p.Mo + m) * p.Kc + k : (m * p.Kc + k) * p.KHW + tp.tmem;
          wr[i] = buf_ld(wrsrc, (m < p.Mo && k < p.Kc && ntaps > 0) ? wo_ * esz : OOB, wgt);
        }
      } else {
        const int m = m0 + wl;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int k = k0 + wo + 4 * i;
          const int wo_ = p.wre ? (tp.tmem * p.Kc + k) * p.Mo + m : (k * p.Mo + m) * p.KHW + tp.tmem;
          wr[i] = buf_ld(wrsrc, (m < p.Mo && k < p.Kc && ntaps > 0) ? wo_ * esz : OOB, wgt);
        }
      }
      if (++ti >= ntaps) {
        ti = 0;
        ++kc;                                   // chunks past the end read channels >= Kc: zeros
      }
    };
    auto store = [&](int buf, const float (&sr)[8], const float (&wr)[8]) {
      float* xs = lds + buf * BUF;
      float* as = xs + NPAIR * XPS;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<float2*>(xs + (4 * wave + j) * XPS + 2 * lane) = make_float2(sr[2 * j], sr[2 * j + 1]);
      if (!BWD) {
#pragma unroll
        for (int i = 0; i < 8; ++i) as[(wo + 8 * i) * APW + wl] = wr[i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int k = wo + 4 * i;
          as[(k >> 1) * APS + 2 * wl + (k & 1)] = wr[i];
        }
      }
    };

    // DEPTH register sets: the loads of chunk c+DEPTH are issued while chunk c+1 is
    // stored, so a load has DEPTH-1 chunk periods to come back
    float sr[DEPTH][8], wr[DEPTH][8];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load(sr[d], wr[d]);
    store(0, sr[0], wr[0]);
    __syncthreads();
    for (int c = 0; c < n; c += DEPTH) {
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) {
        if (c + u >= n) break;
        load(sr[u], wr[u]);                                          // chunk c+u+DEPTH
        store((u + 1) & 1, sr[(u + 1) % DEPTH], wr[(u + 1) % DEPTH]);  // chunk c+u+1
        __syncthreads();
      }
    }
    return;
  }

  // ================================ MFMA waves ===================================
  const int cw = wave - 4;
  const int wp = cw & 1, wc = cw >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  floatx4 acc[PT][2];
#pragma unroll
  for (int i = 0; i < PT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  __syncthreads();                             // chunk 0 is in buffer 0
  for (int c = 0; c < n; ++c) {
    mfma_chunk<BWD, PT>(lds + (c & 1) * BUF, wp, wc, fr, fg, acc);
    __syncthreads();
  }

  const __amdgpu_buffer_rsrc_t drsrc = make_rsrc(dst, p.dst_bytes);
  const int h0 = p.cls[cl].h0, w0 = p.cls[cl].w0;
#pragma unroll
  for (int i = 0; i < PT; ++i) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int Pe = tileP0 + (wp * PT + i) * 16 + 4 * fg + e;
      const int ni = Pe / Pc, r = Pe - ni * Pc;
      const int hc = r / Wc, wcl = r - hc * Wc;
      const int pix = (h0 + hc * p.rsh) * p.DW + w0 + wcl * p.rsw;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int ch = mtile * BM + wc * 32 + j * 16 + fr;
        const bool ok = Pe < Pctot && ch < p.Mo;
        float v = acc[i][j][e];
        if (bias && ch < p.Mo) v += bias[ch];
        buf_st1<T>(drsrc, ok ? ((ni * p.Mo + ch) * p.DH * p.DW + pix) * esz : OOB, v, dst);
      }
    }
  }
}

template <bool BWD>
bool tapped_plan(const ConvGeom& g, TapParams* p) {
  if (g.groups != 1 || g.KH * g.KW > MAX_TAPS) return false;
  // a chunk is 32 contraction channels of one tap: with few channels most of it is
  // padding, and the kernel that flattens (channel, tap) into one contraction does better
  const int kc = BWD ? g.K : g.C;
  if ((kc + KC - 1) / KC * KC * 2 > 3 * kc) return false;
  p->N = g.N;
  p->KHW = g.KH * g.KW;
  p->nclasses = 0;
  int ntaps = 0, tiles = 0;
  auto add_class = [&](TapClass c) {
    c.tile0 = tiles;
    const long long pos = (long long)g.N * c.Hc * c.Wc;
    tiles += (int)((pos + 63) / 64);
    p->cls[p->nclasses++] = c;
  };
  if (!BWD) {
    p->Kc = g.C; p->Mo = g.K; p->SH = g.H; p->SW = g.W; p->DH = g.OH; p->DW = g.OW;
    p->ssh = g.sy; p->ssw = g.sx; p->rsh = 1; p->rsw = 1;
    TapClass c{};
    c.Hc = g.OH; c.Wc = g.OW; c.h0 = 0; c.w0 = 0; c.bh = -g.py; c.bw = -g.px;
    c.tap0 = 0; c.ntaps = p->KHW;
    for (int kh = 0; kh < g.KH; ++kh)
      for (int kw = 0; kw < g.KW; ++kw)
        p->taps[ntaps++] = Tap{(short)(kh * g.dly), (short)(kw * g.dlx), kh * g.KW + kw};
    add_class(c);
  } else {
    p->Kc = g.K; p->Mo = g.C; p->SH = g.OH; p->SW = g.OW; p->DH = g.H; p->DW = g.W;
    p->ssh = 1; p->ssw = 1; p->rsh = g.sy; p->rsw = g.sx;
    if (g.sy * g.sx > MAX_CLASSES) return false;
    for (int a = 0; a < g.sy; ++a)
      for (int b = 0; b < g.sx; ++b) {
        TapClass c{};
        c.h0 = ((a - g.py) % g.sy + g.sy) % g.sy;
        c.w0 = ((b - g.px) % g.sx + g.sx) % g.sx;
        c.Hc = c.h0 < g.H ? (g.H - 1 - c.h0) / g.sy + 1 : 0;
        c.Wc = c.w0 < g.W ? (g.W - 1 - c.w0) / g.sx + 1 : 0;
        if (c.Hc == 0 || c.Wc == 0) continue;
        c.bh = (c.h0 + g.py - a) / g.sy;
        c.bw = (c.w0 + g.px - b) / g.sx;
        c.tap0 = ntaps;
        for (int kh = 0; kh < g.KH; ++kh)
          for (int kw = 0; kw < g.KW; ++kw) {
            if ((kh * g.dly) % g.sy != a || (kw * g.dlx) % g.sx != b) continue;
            if (ntaps >= MAX_TAPS) return false;
            p->taps[ntaps++] = Tap{(short)(-(kh * g.dly - a) / g.sy), (short)(-(kw * g.dlx - b) / g.sx),
                                   kh * g.KW + kw};
          }
        c.ntaps = ntaps - c.tap0;
        add_class(c);
      }
  }
  if (p->nclasses == 0) return false;
  p->ptiles = tiles;
  p->kchunks = (p->Kc + KC - 1) / KC;
  p->mtiles = (p->Mo + BM - 1) / BM;
  if ((g.KH - 1) * g.dly >= (1 << 14) || (g.KW - 1) * g.dlx >= (1 << 14)) return false;
  return true;
}

// The weights of one tap are KHW elements apart in memory ([filter][channel][tap]): a
// wave's load of a weight tile touches one 4-byte element per 4*KHW bytes.  With a
// workspace the weights are first copied to [tap][filter][channel] (a transpose of a
// (filter*channel) x KHW matrix, a few microseconds), where the same loads are contiguous.
template <typename T>
__global__ void __launch_bounds__(256) reorder_taps_kernel(const T* __restrict__ in, T* __restrict__ out, int rows,
                                                           int khw) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)rows * khw) return;
  const int t = (int)(i / rows), r = (int)(i - (long long)t * rows);
  out[i] = in[(long long)r * khw + t];
}

template <bool BWD>
int launch_tapped(const ConvGeom& g, int dtype, const void* src, const void* wgt, const float* bias,
                  void* dst, hipStream_t s, void* ws, size_t ws_bytes) {
  TapParams p{};
  if (!tapped_plan<BWD>(g, &p)) return -1;
  const long long esz = dtype == FLHIP_F32 ? 4 : 2;
  const long long xb = (long long)g.N * g.C * g.H * g.W * esz, yb = (long long)g.N * g.K * g.OH * g.OW * esz;
  const long long wb = (long long)g.K * g.C * g.KH * g.KW * esz;
  if (xb >= (1ll << 31) || yb >= (1ll << 31) || wb >= (1ll << 31)) return -1;
  p.src_bytes = (unsigned)(BWD ? yb : xb);
  p.dst_bytes = (unsigned)(BWD ? xb : yb);
  p.wgt_bytes = (unsigned)wb;
  const bool no_reorder = options().tapped_no_reorder;
  if (ws && ws_bytes >= (size_t)wb && p.KHW > 1 && !no_reorder) {
    const int rows = g.K * g.C;
    const long long total = (long long)rows * p.KHW;
    by_dtype(dtype, [&](auto* t_) {
      using T = FLHIP_T_OF(t_);
      hipLaunchKernelGGL((reorder_taps_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                         static_cast<const T*>(wgt), static_cast<T*>(ws), rows, p.KHW);
    });
    wgt = ws;
    p.wre = 1;
  }
  const unsigned grid = (unsigned)(((p.ptiles + 7) / 8) * 8 * p.mtiles);
  by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    hipLaunchKernelGGL((tapped_conv_kernel<T, BWD>), dim3(grid), dim3(MFMA_THREADS), 0, s, p,
                       static_cast<const T*>(src), static_cast<const T*>(wgt), bias,
                       static_cast<T*>(dst));
  });
  return check_launch("conv2d (tapped mfma)");
}

bool pw_applies(const ConvGeom& g) {
  return g.KH == 1 && g.KW == 1 && g.py == 0 && g.px == 0 && g.groups == 1;
}


// ---- filter gradient of a 1x1 convolution ---------------------------------------------
//   dw[m][c] = sum over (n, q) of dy[n][m][q] * x[n][c][map(q)]   (+ db[m] = sum of dy)
// is a GEMM whose contraction runs over positions, which are contiguous in memory in
// both operands, so the tiles go to LDS in memory order [row][position] (pitch 36: the
// 32 lanes of one 8-byte read pass hit distinct banks) and a lane's float2 holds two
// consecutive positions = the k index of two MFMAs.  A workgroup owns 64 (m) x 64 (c)
// of dw and one slice of the positions; it writes its tile (and, for the first column
// tile, the bias sums collected by the loader threads) to the workspace, and the
// fixed-order reduction kernel shared with the other filter-gradient kernels adds the
// slices.  Same wave roles and barrier scheme as above; four workgroups per CU.
constexpr int PC = 32;                 // positions per chunk
constexpr int WPITCH = PC + 4;

struct PwWgradParams {
  int Mo, C;             // channels of dy / of x
  int P, Ptot, SP;       // positions per image (dy), over all images; elements per x plane
  int OW, x_map;         // x_map: x goes through the window geometry below
  int H, W, KW, KHW, sy, sx, py, px, dly, dlx;
  int pps, nsplit;       // positions per slice (multiple of PC), slices
  int ctiles, mtiles;
  int E;                 // Mo * C
  int want_db;
  unsigned x_bytes, dy_bytes;
};

template <typename T, bool VEC>
__global__ void __launch_bounds__(MFMA_THREADS)
pointwise_wgrad_kernel(PwWgradParams p, const T* __restrict__ x, const T* __restrict__ dy,
                       float* __restrict__ out) {
  constexpr int TILE = BM * WPITCH;
  constexpr int esz = (int)sizeof(T);
  __shared__ float lds[2][2][TILE];          // [buffer][dy tile, x tile]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x;
  const int ctile = __builtin_amdgcn_readfirstlane(blockIdx.y % p.ctiles);
  const int mtile = __builtin_amdgcn_readfirstlane(blockIdx.y / p.ctiles);
  const int tap = blockIdx.z;                            // one window tap per workgroup
  const int pos0 = split * p.pps;
  const int pos1 = min(pos0 + p.pps, p.Ptot);
  const int n = (pos1 - pos0 + PC - 1) / PC;
  float* part = out + (size_t)split * (p.nsplit > 1 ? (size_t)p.E + p.Mo : 0);

  if (wave < 4) {
    // ================================ loaders ====================================
    const __amdgpu_buffer_rsrc_t xrsrc = make_rsrc(x, p.x_bytes);
    const __amdgpu_buffer_rsrc_t yrsrc = make_rsrc(dy, p.dy_bytes);
    const bool do_db = p.want_db && ctile == 0 && tap == 0;
    if (VEC) {
      // ---- 16-byte loads: a thread owns rows `row` and `row + 32`, positions 4kq .. 4kq+3 ----
      const int row = tid >> 3, kq = tid & 7;
      int ni = (pos0 + 4 * kq) / p.P, qi = (pos0 + 4 * kq) - ni * p.P;
      float dbs[2] = {0.f, 0.f};
      const int mrow = mtile * BM + row, crow = ctile * BM + row;
      auto load = [&](int c, float4 (&yr)[2], float4 (&xr)[2]) {
        const bool ok = pos0 + c * PC + 4 * kq < pos1;
        const int yo = ni * p.Mo * p.P + qi, xo = ni * p.C * p.SP + qi;
        qi += PC;
        while (qi >= p.P) {
          qi -= p.P;
          ++ni;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int m = mrow + 32 * i, ch = crow + 32 * i;
          yr[i] = buf_ld4(yrsrc, (ok && m < p.Mo) ? (yo + m * p.P) * esz : OOB, dy);
          xr[i] = buf_ld4(xrsrc, (ok && ch < p.C) ? (xo + ch * p.SP) * esz : OOB, x);
        }
      };
      auto store = [&](int buf, const float4 (&yr)[2], const float4 (&xr)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          *reinterpret_cast<float4*>(&lds[buf][0][(row + 32 * i) * WPITCH + 4 * kq]) = yr[i];
          *reinterpret_cast<float4*>(&lds[buf][1][(row + 32 * i) * WPITCH + 4 * kq]) = xr[i];
          if (do_db) dbs[i] += (yr[i].x + yr[i].y) + (yr[i].z + yr[i].w);
        }
      };
      float4 yA[2], xA[2], yB[2], xB[2];
      load(0, yA, xA);
      store(0, yA, xA);
      load(1, yB, xB);
      __syncthreads();
      for (int c = 0; c < n; c += 2) {
        load(c + 2, yA, xA);
        store(1, yB, xB);                        // chunk c+1 (zeros past the slice)
        __syncthreads();
        if (c + 1 >= n) break;
        load(c + 3, yB, xB);
        store(0, yA, xA);                        // chunk c+2
        __syncthreads();
      }
      if (do_db) {
        // the 8 threads that share a row are neighbours in the wave
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          float v = dbs[i];
          v += __shfl_xor(v, 1, 64);
          v += __shfl_xor(v, 2, 64);
          v += __shfl_xor(v, 4, 64);
          const int m = mrow + 32 * i;
          if (kq == 0 && m < p.Mo) part[p.E + m] = v;
        }
      }
    } else {
      // ---- element-wise loads: a lane owns one position of the chunk (so a wave's load
      // of a row is a contiguous run wherever the geometry allows) and rows r0 + 8i ----
      const int pl = tid & 31, r0 = tid >> 5;
      int ni = (pos0 + pl) / p.P, qi = (pos0 + pl) - ni * p.P;
      const int tdh = (tap / p.KW) * p.dly - p.py, tdw = (tap % p.KW) * p.dlx - p.px;
      float dbs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      const int mrow = mtile * BM + r0, crow = ctile * BM + r0;
      auto load = [&](int c, float (&yr)[8], float (&xr)[8]) {
        const bool ok = pos0 + c * PC + pl < pos1;
        const int yo = ni * p.Mo * p.P + qi;
        int xq = qi;
        bool okx = ok;
        if (p.x_map) {
          const int oh = qi / p.OW, ow = qi - oh * p.OW;
          const int ih = oh * p.sy + tdh, iw = ow * p.sx + tdw;
          okx = ok && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
          xq = ih * p.W + iw;
        }
        const int xo = ni * p.C * p.SP + xq;
        qi += PC;
        while (qi >= p.P) {
          qi -= p.P;
          ++ni;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int m = mrow + 8 * i, ch = crow + 8 * i;
          yr[i] = buf_ld(yrsrc, (ok && m < p.Mo) ? (yo + m * p.P) * esz : OOB, dy);
          xr[i] = buf_ld(xrsrc, (okx && ch < p.C) ? (xo + ch * p.SP) * esz : OOB, x);
        }
      };
      auto store = [&](int buf, const float (&yr)[8], const float (&xr)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          lds[buf][0][(r0 + 8 * i) * WPITCH + pl] = yr[i];
          lds[buf][1][(r0 + 8 * i) * WPITCH + pl] = xr[i];
          if (do_db) dbs[i] += yr[i];
        }
      };
      float yA[8], xA[8], yB[8], xB[8];
      load(0, yA, xA);
      store(0, yA, xA);
      load(1, yB, xB);
      __syncthreads();
      for (int c = 0; c < n; c += 2) {
        load(c + 2, yA, xA);
        store(1, yB, xB);
        __syncthreads();
        if (c + 1 >= n) break;
        load(c + 3, yB, xB);
        store(0, yA, xA);
        __syncthreads();
      }
      if (do_db) {
        // the 32 lanes that share a row are one half of a wave
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float v = dbs[i];
#pragma unroll
          for (int o = 1; o < 32; o <<= 1) v += __shfl_xor(v, o, 64);
          const int m = mrow + 8 * i;
          if (pl == 0 && m < p.Mo) part[p.E + m] = v;
        }
      }
    }
    return;
  }

  // ================================ MFMA waves ===================================
  const int cw = wave - 4;
  const int wm = cw & 1, wn = cw >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  floatx4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  __syncthreads();
  for (int c = 0; c < n; ++c) {
    const float* ys = &lds[c & 1][0][(wm * 32 + fr) * WPITCH + 2 * fg];
    const float* xs = &lds[c & 1][1][(wn * 32 + fr) * WPITCH + 2 * fg];
#pragma unroll
    for (int s = 0; s < PC / 8; ++s) {
      float2 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = *reinterpret_cast<const float2*>(ys + i * 16 * WPITCH + 8 * s);
        b[i] = *reinterpret_cast<const float2*>(xs + i * 16 * WPITCH + 8 * s);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].x, b[j].x, acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i].y, b[j].y, acc[i][j], 0, 0, 0);
        }
    }
    __syncthreads();
  }
  // lane: rows m0 + 4*fg + r, column c0 + fr of each accumulator
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ch = ctile * BM + wn * 32 + j * 16 + fr;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = mtile * BM + wm * 32 + i * 16 + 4 * fg + r;
        if (m < p.Mo && ch < p.C) part[((size_t)m * p.C + ch) * p.KHW + tap] = acc[i][j][r];
      }
    }
}

bool pw_wgrad_plan(const ConvGeom& g, PwWgradParams* p, int max_slices = 0) {
  if (g.groups != 1) return false;
  // 64-channel column tiles: with few input channels the kernel that flattens
  // (channel, tap) into the columns wastes less
  if (!pw_applies(g) && (g.C + BM - 1) / BM * BM * 2 > 3 * g.C) return false;
  p->Mo = g.K; p->C = g.C;
  p->P = g.OH * g.OW; p->Ptot = g.N * p->P; p->SP = g.H * g.W;
  p->OW = g.OW;
  p->H = g.H; p->W = g.W; p->KW = g.KW; p->KHW = g.KH * g.KW;
  p->sy = g.sy; p->sx = g.sx; p->py = g.py; p->px = g.px; p->dly = g.dly; p->dlx = g.dlx;
  p->x_map = (g.sy != 1 || g.sx != 1 || !pw_applies(g)) ? 1 : 0;
  p->ctiles = (g.C + BM - 1) / BM;
  p->mtiles = (g.K + BM - 1) / BM;
  p->E = g.K * g.C * p->KHW;
  const long long base = (long long)p->ctiles * p->mtiles * p->KHW;
  if ((long long)p->ctiles * p->mtiles > 65535 || p->KHW > 65535) return false;
  long long ns = 4ll * mfma_num_cus() / base;
  const long long max_ns = (p->Ptot + 255) / 256;
  if (ns > max_ns) ns = max_ns;
  if (max_slices > 0 && ns > max_slices) ns = max_slices;
  if (ns < 1) ns = 1;
  long long pps = (p->Ptot + ns - 1) / ns;
  pps = (pps + PC - 1) / PC * PC;
  p->pps = (int)pps;
  p->nsplit = (int)((p->Ptot + pps - 1) / pps);
  return true;
}

}  // namespace

int mfma_pointwise_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                            const float* bias, void* y, hipStream_t s, int ksplit) {
  if (!pw_applies(g)) return -1;
  const long long esz = dtype == FLHIP_F32 ? 4 : 2;
  const long long sb = (long long)g.N * g.C * g.H * g.W * esz, db = (long long)g.N * g.K * g.OH * g.OW * esz;
  const long long wb = (long long)g.K * g.C * esz;
  if (sb >= (1ll << 31) || db >= (1ll << 31) || wb >= (1ll << 31)) return -1;
  PwParams p{};
  p.Kc = g.C; p.Mo = g.K; p.SP = g.H * g.W; p.DP = g.OH * g.OW;
  p.P = g.OH * g.OW; p.Ptot = g.N * p.P; p.OW = g.OW;
  p.rowstep = g.sy * g.W; p.colstep = g.sx;
  p.src_map = (g.sy != 1 || g.sx != 1) ? 1 : 0;
  p.dst_map = 0;
  p.vec_w = (g.C % 4 == 0) ? 1 : 0;
  p.nchunks = (g.C + KC - 1) / KC;
  p.mtiles = (g.K + BM - 1) / BM;
  p.src_bytes = (unsigned)sb; p.wgt_bytes = (unsigned)wb; p.dst_bytes = (unsigned)db;
  const bool vec = !p.src_map && p.P % 4 == 0;
  if (ksplit > 1) {
    if (dtype != FLHIP_F32 || db * ksplit >= (1ll << 31)) return -1;
    p.cps = (p.nchunks + ksplit - 1) / ksplit;
    p.dst_slice = (unsigned)(db / esz);
    p.dst_bytes = (unsigned)db;
  }
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch_pw<T, false>(p, vec, x, w, bias, y, s);
  });
}

int mfma_pointwise_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                                 hipStream_t s, const float* bias, int ksplit) {
  if (!pw_applies(g)) return -1;
  const long long esz = dtype == FLHIP_F32 ? 4 : 2;
  const long long sb = (long long)g.N * g.K * g.OH * g.OW * esz, db = (long long)g.N * g.C * g.H * g.W * esz;
  const long long wb = (long long)g.K * g.C * esz;
  if (sb >= (1ll << 31) || db >= (1ll << 31) || wb >= (1ll << 31)) return -1;
  PwParams p{};
  p.Kc = g.K; p.Mo = g.C; p.SP = g.OH * g.OW; p.DP = g.H * g.W;
  p.P = g.OH * g.OW; p.Ptot = g.N * p.P; p.OW = g.OW;
  p.rowstep = g.sy * g.W; p.colstep = g.sx;
  p.src_map = 0;
  // dx covers more than the lattice when a stride skips elements or the last rows /
  // columns are never reached; those elements are zero
  const bool full = g.sy == 1 && g.sx == 1 && g.OH == g.H && g.OW == g.W;
  p.dst_map = full ? 0 : 1;
  p.vec_w = (g.C % 4 == 0) ? 1 : 0;
  p.nchunks = (g.K + KC - 1) / KC;
  p.mtiles = (g.C + BM - 1) / BM;
  p.src_bytes = (unsigned)sb; p.wgt_bytes = (unsigned)wb; p.dst_bytes = (unsigned)db;
  if (!full) {
    const size_t nel = (size_t)g.N * g.C * g.H * g.W;
    const size_t n16 = (size_t)db / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (blocks < 1) blocks = 1;
    by_dtype(dtype, [&](auto* t_) {
      using T = FLHIP_T_OF(t_);
      hipLaunchKernelGGL((zero_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, static_cast<T*>(dx), n16, nel);
    });
  }
  const bool vec = full && p.P % 4 == 0;
  if (ksplit > 1) {
    if (dtype != FLHIP_F32 || !full || db * ksplit >= (1ll << 31)) return -1;
    p.cps = (p.nchunks + ksplit - 1) / ksplit;
    p.dst_slice = (unsigned)(db / esz);
  }
  return by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    return launch_pw<T, true>(p, vec, dy, w, bias, dx, s);
  });
}

// ---- split contraction for 1x1 stride-1 fp32 layers with few tiles ----------------------
// 7x7 planes with 2048 channels to contract: 200 tiles of 64 chunks each on 256 CUs.  With
// workspace for the partial results the contraction is cut into slices (blockIdx.y of the
// kernel above; the bias goes with slice 0) that the fixed-order reduction kernel adds.
// The dispatch uses it for backward-data only (512 -> 2048 channels over 7x7: 91 -> 68 us);
// forward over the same shapes measured no faster with it (54 -> 56 us).
// Returns the request to pass as ksplit (1: no split); *slices = partial results written.
static int pw_split_request(const ConvGeom& g, bool bwd, int* slices) {
  *slices = 1;
  if (!pw_applies(g) || g.sy != 1 || g.sx != 1 || g.OH != g.H || g.OW != g.W) return 1;
  const int Kc = bwd ? g.K : g.C, Mo = bwd ? g.C : g.K;
  const long long tiles = (((long long)g.N * g.H * g.W + 63) / 64) * ((Mo + BM - 1) / BM);
  const int chunks = (Kc + KC - 1) / KC;
  if (chunks < 32 || tiles > mfma_num_cus()) return 1;
  long long ks = 2ll * mfma_num_cus() / tiles;
  if (ks > 8) ks = 8;
  if (ks > chunks / 8) ks = chunks / 8;      // at least 8 chunks per slice
  if (ks < 2) return 1;
  *slices = mfma_gemm_slices(Kc, (int)ks);
  return (int)ks;
}

size_t mfma_pointwise_split_ws(const ConvGeom& g, int dtype, bool bwd) {
  int slices;
  if (dtype != FLHIP_F32 || pw_split_request(g, bwd, &slices) <= 1) return 0;
  return (size_t)slices * g.N * (bwd ? g.C : g.K) * g.H * g.W * sizeof(float);
}

int mfma_pointwise_conv_split(const ConvGeom& g, int dtype, bool bwd, const void* src, const void* w,
                              const float* bias, void* dst, void* ws, size_t ws_bytes, hipStream_t s) {
  int slices;
  if (dtype != FLHIP_F32) return -1;
  const int ks = pw_split_request(g, bwd, &slices);
  const size_t E = (size_t)g.N * (bwd ? g.C : g.K) * g.H * g.W;
  if (ks <= 1 || slices <= 1 || !ws || ws_bytes < slices * E * sizeof(float) || E >= (1ull << 31)) return -1;
  const int rc = bwd ? mfma_pointwise_conv_bwd_data(g, dtype, src, w, ws, s, nullptr, ks)
                     : mfma_pointwise_conv_fwd(g, dtype, src, w, bias, ws, s, ks);
  if (rc != FLHIP_OK) return rc;
  wgrad_reduce_launch(static_cast<const float*>(ws), slices, (int)E, 0, 0, static_cast<float*>(dst), nullptr, s);
  return check_launch("conv2d 1x1 (split contraction)");
}

size_t mfma_pointwise_wgrad_ws(const ConvGeom& g) {
  PwWgradParams p{};
  if (!pw_wgrad_plan(g, &p)) return 0;
  return p.nsplit > 1 ? (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float) : 0;
}

int mfma_pointwise_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                         float* db, void* ws, size_t ws_bytes, bool windows, hipStream_t s, int max_slices) {
  if (!dw) return -1;   // bias gradient alone: the plain reduction kernel
  if (!windows && !pw_applies(g)) return -1;
  PwWgradParams p{};
  if (!pw_wgrad_plan(g, &p, max_slices)) return -1;
  const long long esz = dtype == FLHIP_F32 ? 4 : 2;
  const long long xb = (long long)g.N * g.C * g.H * g.W * esz, yb = (long long)g.N * g.K * g.OH * g.OW * esz;
  if (xb >= (1ll << 31) || yb >= (1ll << 31)) return -1;
  p.x_bytes = (unsigned)xb;
  p.dy_bytes = (unsigned)yb;
  p.want_db = db != nullptr;
  if (p.nsplit > 1 && (!ws || ws_bytes < (size_t)p.nsplit * ((size_t)p.E + p.Mo) * sizeof(float)))
    return fail(FLHIP_INVALID_ARGUMENT, "conv2d_bwd_filter: workspace too small");
  // a single slice writes dw in place; its bias sums need a home of their own
  if (p.nsplit == 1 && db) return -1;
  float* out = p.nsplit > 1 ? static_cast<float*>(ws) : dw;
  const dim3 grid((unsigned)p.nsplit, (unsigned)(p.ctiles * p.mtiles), (unsigned)p.KHW);
  const bool vec = !p.x_map && p.P % 4 == 0;
  const int rc_ = by_dtype(dtype, [&](auto* t_) {
    using T = FLHIP_T_OF(t_);
    if (vec)
      hipLaunchKernelGGL((pointwise_wgrad_kernel<T, true>), grid, dim3(MFMA_THREADS), 0, s, p,
                         static_cast<const T*>(x), static_cast<const T*>(dy), out);
    else
      hipLaunchKernelGGL((pointwise_wgrad_kernel<T, false>), grid, dim3(MFMA_THREADS), 0, s, p,
                         static_cast<const T*>(x), static_cast<const T*>(dy), out);
    return 0;
  });
  if (rc_) return rc_;
  if (const int rc = check_launch("conv2d_bwd_filter 1x1 (mfma)")) return rc;
  if (p.nsplit > 1) {
    wgrad_reduce_launch(static_cast<const float*>(ws), p.nsplit, p.E, p.Mo, p.want_db, dw, db, s);
    return check_launch("conv2d_bwd_filter 1x1 (reduce)");
  }
  return FLHIP_OK;
}

int mfma_tapped_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias,
                         void* y, hipStream_t s, void* ws, size_t ws_bytes) {
  return launch_tapped<false>(g, dtype, x, w, bias, y, s, ws, ws_bytes);
}

int mfma_tapped_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                              hipStream_t s, void* ws, size_t ws_bytes) {
  return launch_tapped<true>(g, dtype, dy, w, nullptr, dx, s, ws, ws_bytes);
}

// bytes of workspace with which the tapped kernels read reordered weights (0: not their shape)
size_t mfma_tapped_ws(const ConvGeom& g, int dtype, bool bwd) {
  TapParams p{};
  if (g.KH * g.KW <= 1 || !(bwd ? tapped_plan<true>(g, &p) : tapped_plan<false>(g, &p))) return 0;
  return (size_t)g.K * g.C * g.KH * g.KW * (dtype == FLHIP_F32 ? 4 : 2);
}

// Column-major matrix products on the same kernels: a matrix with its columns as
// "images" of one position each is a 1x1-convolution operand.
//   mode 0, C = A B    : A (M x K) is stored [k][m] = backward-data weights, B [n][k], C [n][m]
//   mode 1, C = A^T B  : A stored (K x M) = [m][k] = forward weights
//   mode 2, C = A B^T  : B stored (N x K) = [k][n]; C[n][m] = sum_k B[k][n] A[k][m] is the filter
//                        gradient with the rows of B as dy and of A as x (fp32 only: that kernel
//                        writes fp32; single slice only: there is no workspace here)
// bias_rows (fp32[M] or null) is added to every column in modes 0 and 1.  ksplit > 1 (modes
// 0 and 1, fp32): the contraction is cut into that many slices at most, slice s writes its
// partial product at C + s*M*N and the caller adds them (the number of slices written is
// ceil(chunks / ceil(chunks / ksplit)) with chunks = ceil(K / 32): see mfma_gemm_slices).
// Returns -1 when the product does not fit these kernels.
int mfma_gemm(int dtype, int mode, const void* A, const void* B, void* C, int M, int N, int K,
              const float* bias_rows, hipStream_t s, int ksplit) {
  ConvGeom g{};
  g.H = g.W = g.OH = g.OW = g.KH = g.KW = 1;
  g.sy = g.sx = g.dly = g.dlx = g.groups = 1;
  if (mode == 0) {
    g.N = N; g.C = M; g.K = K; g.Cg = M; g.Kg = K;
    return mfma_pointwise_conv_bwd_data(g, dtype, B, A, C, s, bias_rows, ksplit);
  }
  if (mode == 1) {
    g.N = N; g.C = K; g.K = M; g.Cg = K; g.Kg = M;
    return mfma_pointwise_conv_fwd(g, dtype, B, A, bias_rows, C, s, ksplit);
  }
  if (mode == 2 && dtype == FLHIP_F32 && !bias_rows && ksplit <= 1) {
    g.N = K; g.C = M; g.K = N; g.Cg = M; g.Kg = N;
    // no workspace here, so one slice of the contraction per tile: fine when there are
    // enough 64 x 64 tiles to occupy the machine or the contraction is short
    const long long tiles = (long long)((M + BM - 1) / BM) * ((N + BM - 1) / BM);
    if (tiles < 64 && mfma_pointwise_wgrad_ws(g) != 0) return -1;
    return mfma_pointwise_wgrad(g, dtype, A, B, static_cast<float*>(C), nullptr, nullptr, 0, false, s, 1);
  }
  return -1;
}

// C[n][m] += bias[m]
__global__ void __launch_bounds__(256) add_row_bias_kernel(float* __restrict__ C, const float* __restrict__ bias, int M,
                                                           size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) C[i] += bias[i % M];
}

// The same products (fp32) with a matrix as ONE image whose plane is its contiguous dimension, so that the kernels
// fetch their operand tiles as on the planes of a convolution (positions contiguous) instead of gathering one
// position per image:
//   mode 0, C = A B    : forward layer, x = A ([k][m]: K channels over a plane of M), weights B ([n][k]); the bias
//                        per row of C is a bias per position: added by a pass of its own
//   mode 1, C = A^T B  : filter gradient, x = A ([m][k]), dy = B ([n][k]), plane = the contraction (one slice)
//   mode 2, C = A B^T  : backward-data layer, dy = A ([k][m]), weights B ([k][n])
int mfma_gemm_planes(int mode, const void* A, const void* B, void* C, int M, int N, int K, const float* bias_rows,
                     hipStream_t s) {
  ConvGeom g{};
  g.N = 1;
  g.H = g.OH = g.KH = g.KW = 1;
  g.sy = g.sx = g.dly = g.dlx = g.groups = 1;
  int rc = -1;
  if (mode == 0) {
    g.W = g.OW = M; g.C = g.Cg = K; g.K = g.Kg = N;
    rc = mfma_pointwise_conv_fwd(g, FLHIP_F32, A, B, nullptr, C, s, 1);
  } else if (mode == 2 && !bias_rows) {
    g.W = g.OW = M; g.C = g.Cg = N; g.K = g.Kg = K;
    rc = mfma_pointwise_conv_bwd_data(g, FLHIP_F32, A, B, C, s, nullptr, 1);
  } else if (mode == 1) {
    g.W = g.OW = K; g.C = g.Cg = M; g.K = g.Kg = N;
    const long long tiles = (long long)((M + BM - 1) / BM) * ((N + BM - 1) / BM);
    if (tiles < 64) return -1;
    rc = mfma_pointwise_wgrad(g, FLHIP_F32, A, B, static_cast<float*>(C), nullptr, nullptr, 0, false, s, 1);
  }
  if (rc != 0 || !bias_rows) return rc;
  const size_t n = (size_t)M * N;
  hipLaunchKernelGGL(add_row_bias_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 8192)), dim3(256), 0, s,
                     static_cast<float*>(C), bias_rows, M, n);
  return check_launch("matmul (bias)");
}

// number of partial products mfma_gemm writes for a contraction of length K cut into at
// most ksplit slices
int mfma_gemm_slices(int K, int ksplit) {
  const int chunks = (K + KC - 1) / KC;
  if (ksplit <= 1) return 1;
  const int cps = (chunks + ksplit - 1) / ksplit;
  return (chunks + cps - 1) / cps;
}

}  // namespace flhip
