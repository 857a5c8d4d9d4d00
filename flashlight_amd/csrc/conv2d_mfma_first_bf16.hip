// Forward convolution of a first layer (few input channels, wide window, even column stride:
// the 7x7 stride-2 stem of ResNet over 3 channels) in bf16 storage on the bf16 matrix cores
// (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//
// The contraction runs over (channel, window row) pairs; each pair is one group of 8
// contraction values = the window row itself, which is contiguous in memory: the 16 bytes
// that start at column ow * sx - px (rounded down to an even column, so that every load is
// dword-aligned; the window's columns then sit at elements sh .. sh + KW - 1 of the group,
// sh = px & 1, and the other elements are zeroed).  A lane of the A operand is one result
// position and fetches its groups straight from memory - neighbouring positions read
// overlapping bytes, which the vector cache serves - so the source never passes through LDS.
// The weights of a wave (64 result channels x up to 22 groups) stay in registers for the
// whole kernel.  A wave owns runs of 64 consecutive positions (two blocks of 32): results are
// staged in LDS per wave and leave as whole 128-byte lines per channel.
#include <algorithm>

#include "conv2d_mfma.h"

namespace flhip {
namespace {

constexpr int F1_NS = 11;          // contraction steps (2 groups each): up to 22 (channel, window row) pairs
constexpr int F1_SP = 64 + 8;      // staging pitch (elements)
constexpr int F1_WAVES = 4;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct First16Params {
  int N, C, H, W, K, OH, OW;
  int KH, KW, sy, sx, py, px;
  int P;                 // OH * OW
  int NO;                // C * KH groups
  int sh;                // element of a group that holds window column 0
  int runs_per_image;    // ceil(P / 64)
  int total_runs;
  int mtiles;            // ceil(K / 64)
  unsigned src_bytes;
};

template <typename E>
__global__ void __launch_bounds__(64 * F1_WAVES, 2)
first16_conv_kernel(First16Params p, const bf16_t* __restrict__ src, const bf16_t* __restrict__ wgt,
                    const float* __restrict__ bias, bf16_t* __restrict__ dst) {
  constexpr int OOB = (int)0x80000000;
  extern __shared__ uint16_t lds_first[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 31, fh = lane >> 5;
  const int mtile = blockIdx.y;
  const int wrow = p.NO * p.KW;                        // weights per result channel

  // ---- weights: the tile's 64 x wrow values through LDS, then every lane builds its groups
  {
    const int m0 = mtile * 64;
    const int nw = min(64, p.K - m0) * wrow;
    const bf16_t* wsrc = wgt + (size_t)m0 * wrow;
    for (int i = tid; i < 64 * wrow; i += 64 * F1_WAVES) lds_first[i] = i < nw ? wsrc[i] : (uint16_t)0;
  }
  __syncthreads();
  uint4 wf[2][F1_NS];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int s = 0; s < F1_NS; ++s) {
      const int o = 2 * s + fh;
      unsigned e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int kw = i - p.sh;
        e[i] = (o < p.NO && kw >= 0 && kw < p.KW) ? lds_first[(mb * 32 + fr) * wrow + o * p.KW + kw] : 0u;
      }
      wf[mb][s] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
    }
  const float bv0 = (bias && mtile * 64 + fr < p.K) ? bias[mtile * 64 + fr] : 0.f;
  const float bv1 = (bias && mtile * 64 + 32 + fr < p.K) ? bias[mtile * 64 + 32 + fr] : 0.f;
  __syncthreads();                                     // the weight area becomes the staging buffers

  // ---- per lane: byte offset of (channel, window row) of each of its groups, window rows packed 4 bits each
  int ooff[F1_NS];
  unsigned khlo = 0, khhi = 0;
#pragma unroll
  for (int s = 0; s < F1_NS; ++s) {
    const int o = 2 * s + fh;
    const int c = o / p.KH, kh = o - c * p.KH;
    ooff[s] = (c * p.H + kh) * p.W * 2;
    if (s < 8) khlo |= (unsigned)kh << (4 * s);
    else khhi |= (unsigned)kh << (4 * (s - 8));
  }
  const __amdgpu_buffer_rsrc_t srsrc = make_rsrc(src, p.src_bytes);
  uint16_t* const stage = lds_first + wave * (64 * F1_SP);
  const float inv_ow = 1.0f / (float)p.OW;
  const float inv_rpi = 1.0f / (float)p.runs_per_image;
  auto frag = [](uint4 v) { return __builtin_bit_cast(bf16x8, v); };

  for (int run = blockIdx.x * F1_WAVES + wave; run < p.total_runs; run += gridDim.x * F1_WAVES) {
    int rin;
    const int n = fast_div(run, p.runs_per_image, inv_rpi, &rin);
    const int pos0 = rin * 64;
    floatx16 acc[2][2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][mb][r] = 0.f;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int pos = pos0 + b * 32 + fr;
      int ow;
      const int oh = fast_div(pos, p.OW, inv_ow, &ow);
      const int ih0 = oh * p.sy - p.py, iw0 = ow * p.sx - p.px - p.sh;
      const int base = pos < p.P ? ((n * p.C * p.H + ih0) * p.W + iw0) * 2 : OOB;
      // elements of a group that lie inside the window and inside the row
      unsigned mk[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int i0 = 2 * d, i1 = 2 * d + 1;
        const bool v0 = i0 >= p.sh && i0 < p.sh + p.KW && (unsigned)(iw0 + i0) < (unsigned)p.W;
        const bool v1 = i1 >= p.sh && i1 < p.sh + p.KW && (unsigned)(iw0 + i1) < (unsigned)p.W;
        mk[d] = (v0 ? 0x0000ffffu : 0u) | (v1 ? 0xffff0000u : 0u);
      }
      uintx4_t a[F1_NS];
#pragma unroll
      for (int s = 0; s < F1_NS; ++s) {
        const int kh = (int)(((s < 8 ? khlo : khhi) >> (4 * (s & 7))) & 15u);
        const bool ok = (unsigned)(ih0 + kh) < (unsigned)p.H && base != OOB && 2 * s + fh < p.NO;
        const int off = base + ooff[s];
        // (a row, group or position that does not exist reads beyond the range: zero)
        const bool neg = ok && off < 0;
        a[s] = __builtin_amdgcn_raw_buffer_load_b128(srsrc, ok && !neg ? off : OOB, 0, 0);
        if (__builtin_amdgcn_ballot_w64(neg) != 0) {
          // the first row of the tensor with window columns left of it: the 16 bytes would start
          // before the tensor; its elements inside the row one by one (a few lanes of one wave)
          if (neg) {
            unsigned e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
              e[i] = iw0 + i >= 0 ? (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(srsrc, off + 2 * i, 0, 0) : 0u;
            a[s] = uintx4_t{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
          }
        }
      }
#pragma unroll
      for (int s = 0; s < F1_NS; ++s) {
        const uint4 av = make_uint4(a[s].x & mk[0], a[s].y & mk[1], a[s].z & mk[2], a[s].w & mk[3]);
        acc[b][0] = Lo16<E>::mma32(frag(av), frag(wf[0][s]), acc[b][0]);
        acc[b][1] = Lo16<E>::mma32(frag(av), frag(wf[1][s]), acc[b][1]);
      }
    }
    // ---- results: element r of an accumulator is position b*32 + (r/4)*8 + fh*4 + r%4 of channel
    // mb*32 + fr; staged as [channel][64 positions], then 16 bytes per lane, 128 per channel
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const float bv = mb ? bv1 : bv0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const floatx16& c = acc[b][mb];
          const uintx2_t v = {Lo16<E>::pack(c[4 * g] + bv, c[4 * g + 1] + bv), Lo16<E>::pack(c[4 * g + 2] + bv, c[4 * g + 3] + bv)};
          *reinterpret_cast<uintx2_t*>(stage + (mb * 32 + fr) * F1_SP + b * 32 + g * 8 + fh * 4) = v;
        }
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's staged results are in LDS
    const size_t obase = ((size_t)n * p.K + mtile * 64) * p.P + pos0;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = it * 64 + lane, ch = idx >> 3, q = idx & 7;
      const uintx4_t v = *reinterpret_cast<const uintx4_t*>(stage + ch * F1_SP + 8 * q);
      if (mtile * 64 + ch < p.K && pos0 + 8 * q < p.P)
        __builtin_nontemporal_store(v, reinterpret_cast<uintx4_t*>(dst + obase + (size_t)ch * p.P + 8 * q));
    }
    asm volatile("" ::: "memory");                       // (the next run's staging stores stay behind these reads)
  }
}


// ---------------------------------------------------------------------------------------------
// Filter (and bias) gradient of the same layers, column stride 2:
//   dw[m][c][kh][kw] = sum over (n, oh, ow) of dy[n][m][oh][ow] * x[n][c][oh*sy - py + kh][2*ow - px + kw]
// contracts over positions.  Per result row oh, D[m][j] += dy[m][ow] * B[ow][j] with one column j per
// (group = (c, kh), element i = kw + sh): B[ow][(c, kh, i)] = x[c][ih][2*ow - px - sh + i], the same
// 16-byte windows as in the forward pass.  A lane of the B operand needs 8 consecutive ow of ONE
// column: transposing LDS reads (ds_read_b64_tr_b16) deliver exactly that from rows stored as they
// are in memory - lane s of a group of 16 passes the address of the 8-byte half window of position
// k0 + s / 4 in group (s % 4) / 2 and receives, for column s, the four positions k0 .. k0 + 3.
// Those reads need 8-byte addresses and a window starts every 4 bytes, so LDS holds each row twice:
// copy p (for odd / even ow) is the row shifted by 2p elements.  One more row of ones makes column
// (C*KH)*8 the bias gradient.  A workgroup takes bands of 4 result rows of one image: the band's
// source rows go to LDS once, dy rows are double-buffered, and every wave accumulates its 32 x 96
// part of the 64 x 192 tile in registers over all its bands; the partial tiles are added in a
// fixed order by first16_wgrad_reduce.
constexpr int FW_RB = 4;            // result rows per band
constexpr int FW_CP = 232;          // elements per row copy (two copies per row)
constexpr int FW_DP = 120;          // dy row pitch (elements)
constexpr int FW_NJ = 192;          // columns of the tile

struct First16WgradParams {
  int N, C, H, W, K, OH, OW;
  int KH, KW, sy, py, px;
  int P, NO, sh;
  int NR;                  // source rows of a band: (FW_RB - 1) * sy + KH
  int bands_per_image, total_bands;
  int mtiles;
};

// KS = steps of 16 positions per result row when known at compile time (the loop is then
// unrolled and its fragment reads run ahead of the matrix instructions), 0 = any
template <typename E, int KS>
__global__ void __launch_bounds__(256, 2)
first16_wgrad_kernel(First16WgradParams p, const bf16_t* __restrict__ x, const bf16_t* __restrict__ dy,
                     float* __restrict__ partial) {
  extern __shared__ uint16_t lds_first[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 31, fh = lane >> 5;
  const int mtile = blockIdx.y;
  const int nrows = p.C * p.NR;                        // then the row of ones and the row of zeros
  uint16_t* const xs = lds_first;                      // [nrows + 2][2 copies][FW_CP]
  uint16_t* const dys = lds_first + (nrows + 2) * 2 * FW_CP;   // [2][64][FW_DP]
  for (int i = tid; i < 2 * FW_CP; i += 256) {
    xs[nrows * 2 * FW_CP + i] = (uint16_t)(Lo16<E>::ONE2 & 0xffffu);   // 1.0
    xs[(nrows + 1) * 2 * FW_CP + i] = 0;
  }

  // ---- B operand: this lane's part of the transposing reads, per block of 32 columns
  // (4 groups): slot s = lane % 16 -> position k0 + 8 * fh + s / 4 (copy = its parity), group
  // 4 * jb + 2 * ((lane / 16) & 1) + (s % 4) / 2, half (s % 2)
  const int mb = wave & 1, jset = wave >> 1;
  int baddr[3], bstep[3];
  {
    const int sl = lane & 15, r = sl >> 2, cq = sl & 3;
    const int owl = 8 * fh + r;                        // position within a step of 16
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const int o = 4 * (3 * jset + t) + 2 * ((lane >> 4) & 1) + (cq >> 1);
      int row, step;
      if (o < p.NO) {
        const int c = o / p.KH, kh = o - c * p.KH;
        row = c * p.NR + kh;
        step = p.sy * 2 * FW_CP;
      } else {
        row = o == p.NO ? nrows : nrows + 1;
        step = 0;
      }
      baddr[t] = (row * 2 + (owl & 1)) * FW_CP + 4 * (owl >> 1) + 4 * (cq & 1);
      bstep[t] = step;
    }
  }
  typedef short shortx4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) shortx4_t* lds_tr;
  auto bfrag = [&](const uint16_t* a) {
    const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)a);
    const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr)(a + 8));   // positions + 4
    const uintx2_t l = __builtin_bit_cast(uintx2_t, lo), h = __builtin_bit_cast(uintx2_t, hi);
    const uintx4_t v = {l.x, l.y, h.x, h.y};
    return __builtin_bit_cast(bf16x8, v);
  };

  floatx16 acc[3];
#pragma unroll
  for (int t = 0; t < 3; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  // dy row: 64 channels x OW positions as 16-byte pieces, 4 per thread
  const int ppr = p.OW >> 3;                           // pieces per channel row
  const float inv_ppr = 1.0f / (float)ppr;
  int dsrc[4], ddst[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i;
    int q;
    const int m = fast_div(idx, ppr, inv_ppr, &q);
    const bool ok = m < 64 && mtile * 64 + m < p.K;
    dsrc[i] = ok ? (mtile * 64 + m) * p.P + 8 * q : -1;
    ddst[i] = m < 64 ? m * FW_DP + 8 * q : -1;
  }
  const int hw = p.W >> 1, shd = (p.px + p.sh) >> 1;   // dwords per source row; window shift in dwords
  const float inv_bpi = 1.0f / (float)p.bands_per_image;
  const uint32_t* const x32 = reinterpret_cast<const uint32_t*>(x);
  uint32_t* const xs32 = reinterpret_cast<uint32_t*>(xs);
  constexpr int xcdw = FW_CP / 2;                      // dwords per row copy
  const int xcp = tid >= xcdw ? 1 : 0;
  const int xsd = tid - xcp * xcdw + xcp - shd;        // source dword of this thread's dword of a row
  const bool xcol_ok = tid < 2 * xcdw && (unsigned)xsd < (unsigned)hw;

  for (int band = blockIdx.x; band < p.total_bands; band += gridDim.x) {
    int bi;
    const int n = fast_div(band, p.bands_per_image, inv_bpi, &bi);
    const int oh0 = bi * FW_RB;
    const int rows = min(FW_RB, p.OH - oh0);
    const bf16_t* const dyn = dy + (size_t)n * p.K * p.P;
    uintx4_t dv[4];
    auto load_dy = [&](int oh) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dv[i] = dsrc[i] >= 0 ? *reinterpret_cast<const uintx4_t*>(dyn + dsrc[i] + oh * p.OW) : uintx4_t{0u, 0u, 0u, 0u};
    };
    auto store_dy = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (ddst[i] >= 0) *reinterpret_cast<uintx4_t*>(dys + buf * 64 * FW_DP + ddst[i]) = dv[i];
    };
    __syncthreads();                                   // the previous band's reads are done
    load_dy(oh0);
    // the band's source rows, both copies: thread = dword of a row (dword d of copy cp is source
    // dword d + cp - shd), eight rows in flight
    for (int c = 0; c < p.C; ++c)
      for (int rl0 = 0; rl0 < p.NR; rl0 += 8) {
        uint32_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const int ih = oh0 * p.sy - p.py + rl0 + k;
          v[k] = (xcol_ok && rl0 + k < p.NR && (unsigned)ih < (unsigned)p.H)
                     ? x32[(((size_t)n * p.C + c) * p.H + ih) * hw + xsd] : 0u;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (tid < 2 * xcdw && rl0 + k < p.NR) xs32[(c * p.NR + rl0 + k) * (2 * xcdw) + tid] = v[k];
      }
    store_dy(0);
    __syncthreads();
    for (int r = 0; r < rows; ++r) {
      if (r + 1 < rows) load_dy(oh0 + r + 1);
      const uint16_t* const da = dys + (r & 1) * 64 * FW_DP + (mb * 32 + fr) * FW_DP + 8 * fh;
      auto step = [&](int ks) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4_t*>(da + 16 * ks));
#pragma unroll
        for (int t = 0; t < 3; ++t) {
          const bf16x8 b = bfrag(xs + baddr[t] + r * bstep[t] + 32 * ks);
          acc[t] = Lo16<E>::mma32(a, b, acc[t]);
        }
      };
      if (KS > 0) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) step(ks);
      } else {
        for (int ks = 0; ks < (p.OW >> 4); ++ks) step(ks);
      }
      if (r + 1 < rows) store_dy((r + 1) & 1);
      __syncthreads();
    }
  }
  // ---- partial tile of this workgroup: element r of acc[t] is row mb*32 + (r/4)*8 + fh*4 + r%4,
  // column (3*jset + t)*32 + fr
  float* const out = partial + ((size_t)blockIdx.x * p.mtiles + mtile) * 64 * FW_NJ;
#pragma unroll
  for (int t = 0; t < 3; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      out[(mb * 32 + (r >> 2) * 8 + fh * 4 + (r & 3)) * FW_NJ + (3 * jset + t) * 32 + fr] = acc[t][r];
}

// dw[m][c][kh][kw] and db[m]: the workgroups' partial tiles added in a fixed order (eight
// slices of the workgroup range, each summed in launch order by one thread, then the eight sums)
__global__ void __launch_bounds__(256)
first16_wgrad_reduce(First16WgradParams p, const float* __restrict__ partial, int nwg, float* __restrict__ dw,
                     float* __restrict__ db) {
  __shared__ float part[8][32];
  const int wrow = p.NO * p.KW;
  const int el = threadIdx.x & 31, slice = threadIdx.x >> 5;
  const int t = blockIdx.x * 32 + el;
  const bool live = t < p.K * (wrow + 1);
  int m = 0, e = 0;
  float sum = 0.f;
  if (live) {
    m = t / (wrow + 1);
    e = t - m * (wrow + 1);
    int col = p.NO * 8;
    if (e < wrow) {
      const int o = e / p.KW, kw = e - o * p.KW;
      col = o * 8 + kw + p.sh;
    }
    const float* src = partial + ((size_t)(m >> 6) * 64 + (m & 63)) * FW_NJ + col;
    const size_t stride = (size_t)p.mtiles * 64 * FW_NJ;
    const int w0 = slice * nwg / 8, w1 = (slice + 1) * nwg / 8;
#pragma unroll 8
    for (int w = w0; w < w1; ++w) sum += src[w * stride];
  }
  part[slice][el] = sum;
  __syncthreads();
  if (slice == 0 && live) {
    float total = part[0][el];
#pragma unroll
    for (int i = 1; i < 8; ++i) total += part[i][el];
    if (e < wrow) {
      if (dw) dw[(size_t)m * wrow + e] = total;
    } else if (db) {
      db[m] = total;
    }
  }
}

bool first16_wgrad_plan(const ConvGeom& g, First16WgradParams* p, int* nwg, size_t* shmem) {
  if (g.groups != 1 || g.dly != 1 || g.dlx != 1 || g.sx != 2 || g.W % 2 != 0) return false;
  const int sh = g.px & 1;
  if (g.KW + sh > 8 || g.C > 4 || g.KH > 15) return false;
  if (g.C * g.KH + 1 > FW_NJ / 8) return false;
  if (g.OW % 16 != 0 || g.OW > 112 || g.K % 32 != 0) return false;
  if ((long long)g.N * g.K * g.OH * g.OW * 2 >= (1ll << 31) || (long long)g.N * g.C * g.H * g.W * 2 >= (1ll << 31)) return false;
  p->N = g.N; p->C = g.C; p->H = g.H; p->W = g.W; p->K = g.K; p->OH = g.OH; p->OW = g.OW;
  p->KH = g.KH; p->KW = g.KW; p->sy = g.sy; p->py = g.py; p->px = g.px;
  p->P = g.OH * g.OW; p->NO = g.C * g.KH; p->sh = sh;
  p->NR = (FW_RB - 1) * g.sy + g.KH;
  p->bands_per_image = (g.OH + FW_RB - 1) / FW_RB;
  p->total_bands = g.N * p->bands_per_image;
  p->mtiles = (g.K + 63) / 64;
  *nwg = std::min(p->total_bands, 2 * mfma_num_cus());
  *shmem = ((size_t)(g.C * p->NR + 2) * 2 * FW_CP + 2 * 64 * FW_DP) * sizeof(uint16_t);
  return *shmem <= 80 * 1024;
}

}  // namespace

size_t mfma_first16_wgrad_ws(const ConvGeom& g) {
  First16WgradParams p{};
  int nwg;
  size_t shmem;
  if (!first16_wgrad_plan(g, &p, &nwg, &shmem)) return 0;
  return (size_t)nwg * p.mtiles * 64 * FW_NJ * sizeof(float);
}

int mfma_first16_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws,
                       size_t ws_bytes, hipStream_t s, int dtype) {
  First16WgradParams p{};
  int nwg;
  size_t shmem;
  if (!first16_wgrad_plan(g, &p, &nwg, &shmem)) return -1;
  if (!ws || ws_bytes < (size_t)nwg * p.mtiles * 64 * FW_NJ * sizeof(float)) return -1;
  if (reinterpret_cast<uintptr_t>(x) % 4 != 0 || reinterpret_cast<uintptr_t>(dy) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(ws) % 16 != 0 || (g.OH * g.OW) % 8 != 0)
    return -1;
  float* partial = static_cast<float*>(ws);
  const int rc = by_lo16(dtype, [&](auto* e_) {
    using E = FLHIP_T_OF(e_);
    auto kernel = g.OW == 112 ? first16_wgrad_kernel<E, 7> : first16_wgrad_kernel<E, 0>;
    if (!mfma_allow_lds(reinterpret_cast<const void*>(kernel), shmem)) return -1;
    hipLaunchKernelGGL(kernel, dim3((unsigned)nwg, (unsigned)p.mtiles), dim3(256), shmem, s, p,
                       static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(dy), partial);
    return 0;
  });
  if (rc) return rc;
  const int total = g.K * (p.NO * g.KW + 1);
  hipLaunchKernelGGL(first16_wgrad_reduce, dim3((unsigned)((total + 31) / 32)), dim3(256), 0, s, p, partial, nwg, dw, db);
  return check_launch("conv2d_bwd_filter (bf16 mfma first layer)");
}


int mfma_first16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                          hipStream_t s, int dtype) {
  if (g.groups != 1 || g.dly != 1 || g.dlx != 1) return -1;
  const int sh = g.px & 1;
  // every 16-byte read starts on a dword: even column stride, even rows, window inside 8 elements
  if (g.sx % 2 != 0 || g.W % 2 != 0 || g.KW + sh > 8) return -1;
  if (g.C * g.KH > 2 * F1_NS || g.KH > 15) return -1;
  const int P = g.OH * g.OW;
  if (P % 8 != 0 || g.K % 32 != 0) return -1;
  // few input channels: otherwise the slab kernels make better use of every byte they read
  if (g.C > 4) return -1;
  const long long sbytes = (long long)g.N * g.C * g.H * g.W * 2, dbytes = (long long)g.N * g.K * P * 2;
  if (sbytes >= (1ll << 30) || dbytes >= (1ll << 31)) return -1;
  if (reinterpret_cast<uintptr_t>(x) % 4 != 0 || reinterpret_cast<uintptr_t>(y) % 16 != 0) return -1;
  First16Params p{};
  p.N = g.N; p.C = g.C; p.H = g.H; p.W = g.W; p.K = g.K; p.OH = g.OH; p.OW = g.OW;
  p.KH = g.KH; p.KW = g.KW; p.sy = g.sy; p.sx = g.sx; p.py = g.py; p.px = g.px;
  p.P = P; p.NO = g.C * g.KH; p.sh = sh;
  p.runs_per_image = (P + 63) / 64;
  p.total_runs = g.N * p.runs_per_image;
  p.mtiles = (g.K + 63) / 64;
  p.src_bytes = (unsigned)sbytes;
  const size_t shmem = std::max((size_t)64 * p.NO * g.KW, (size_t)F1_WAVES * 64 * F1_SP) * sizeof(uint16_t);
  const int wgs = std::min((p.total_runs + F1_WAVES - 1) / F1_WAVES, 2 * mfma_num_cus());
  const int rc = by_lo16(dtype, [&](auto* e_) {
    using E = FLHIP_T_OF(e_);
    if (!mfma_allow_lds(reinterpret_cast<const void*>(first16_conv_kernel<E>), shmem)) return -1;
    hipLaunchKernelGGL(first16_conv_kernel<E>, dim3((unsigned)wgs, (unsigned)p.mtiles), dim3(64 * F1_WAVES), shmem, s, p,
                       static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), bias, static_cast<bf16_t*>(y));
    return 0;
  });
  if (rc) return rc;
  return check_launch("conv2d (bf16 mfma first layer)");
}

}  // namespace flhip
