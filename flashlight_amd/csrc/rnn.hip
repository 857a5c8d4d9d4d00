// rnn / rnnBackward: ReLU / tanh RNN, LSTM and GRU, stacked and bidirectional, with the
// semantics and the flat weight order of the cuDNN calls the reference makes
// (flashlight/fl/autograd/tensor/backend/cudnn/RNN.cpp:62-375): per pseudo-layer
// (layer-major, forward direction first) the input matrices of every gate
// ([hidden][in], row-major) then the recurrent ones; after all matrices, per
// pseudo-layer the input biases then the recurrent biases.  Gates: LSTM i, f, g, o;
// GRU r, z, n with n = tanh(W_n x + b_Wn + r * (R_n h + b_Rn)), h' = (1-z)*n + z*h.
//
// Structure: the input projections of all time steps of a pseudo-layer are one matrix
// product; the recurrence is a loop over time of (recurrent product, gate kernel).
// The products go through flhip_matmul (matrix cores where the shapes allow).  The
// forward pass keeps, per pseudo-layer and in step order, the state before every step,
// the gate activations and (GRU) R_n h + b_Rn in the reserve buffer; the backward pass
// walks the steps in reverse, writes the pre-activation gradients of all steps, and
// turns them into dx, dW, dR and the bias gradients with four products / reductions.
// Layouts follow Flashlight: x [input, B, T] column-major = memory [T][B][input], etc.
// fp32 only; no dropout between layers (the closure's dropProb must be 0).
#include <algorithm>

#include "common.h"
#include "conv2d.h"

extern "C" int flhip_matmul(const void* A, const void* B, void* C, int32_t M, int32_t N, int32_t K,
                            int trans_a, int trans_b, const float* bias_rows, int dtype, void* stream);
extern "C" int flhip_sum_columns(const void* x, float* out, int32_t rows, int32_t cols, int dtype,
                                 void* stream);

namespace flhip {
namespace {

enum { RNN_RELU = 0, RNN_TANH = 1, RNN_LSTM = 2, RNN_GRU = 3 };

struct RnnGeom {
  int I, H, L, D, mode, T, B, G;
  size_t BH, GH;
  size_t nparams;
  float dropout;
  uint32_t seed_lo, seed_hi;
};

inline int gates_of(int mode) { return mode == RNN_LSTM ? 4 : mode == RNN_GRU ? 3 : 1; }

int make_geom(const flhip_rnn_desc* d, RnnGeom* g) {
  FLHIP_REQUIRE(d, "rnn: null descriptor");
  FLHIP_REQUIRE(d->input_size > 0 && d->hidden_size > 0 && d->num_layers > 0 && d->seq_len > 0 &&
                    d->batch > 0,
                "rnn: sizes must be positive");
  FLHIP_REQUIRE(d->mode >= RNN_RELU && d->mode <= RNN_GRU, "rnn: unknown mode");
  FLHIP_REQUIRE(d->dtype == FLHIP_F32, "rnn: f32 only");
  FLHIP_REQUIRE(d->dropout >= 0.f && d->dropout < 1.f, "rnn: dropout must be in [0, 1)");
  g->dropout = d->dropout; g->seed_lo = d->seed_lo; g->seed_hi = d->seed_hi;
  g->I = d->input_size; g->H = d->hidden_size; g->L = d->num_layers; g->D = d->bidirectional ? 2 : 1;
  g->mode = d->mode; g->T = d->seq_len; g->B = d->batch; g->G = gates_of(d->mode);
  g->BH = (size_t)g->B * g->H;
  g->GH = (size_t)g->G * g->H;
  size_t n = 0;
  for (int l = 0; l < g->L; ++l) {
    const size_t in = l == 0 ? g->I : (size_t)g->D * g->H;
    n += g->D * (g->GH * (in + g->H) + 2 * g->GH);
  }
  g->nparams = n;
  FLHIP_REQUIRE((size_t)g->T * g->B * std::max<size_t>(g->GH, (size_t)g->D * g->H) < (1u << 30) &&
                    n < (1u << 30),
                "rnn: problem too large for 32-bit indices");
  return FLHIP_OK;
}

struct Offsets {
  size_t W, R, bW, bR;
};
Offsets offsets(const RnnGeom& g, int pl) {
  Offsets o{};
  size_t off = 0;
  for (int p = 0; p < g.L * g.D; ++p) {
    const size_t in = p / g.D == 0 ? g.I : (size_t)g.D * g.H;
    if (p == pl) {
      o.W = off;
      o.R = off + g.GH * in;
    }
    off += g.GH * (in + g.H);
  }
  o.bW = off + (size_t)pl * 2 * g.GH;
  o.bR = o.bW + g.GH;
  return o;
}

// reserve buffer, in floats: per pseudo-layer {HP [(T+1)*BH], CP [(T+1)*BH] (LSTM),
// GT [T*B*GH], RN [T*BH] (GRU)}, then the outputs of layers 0 .. L-2 ([T*B*D*H] each)
struct Reserve {
  size_t per_pl, hp, cp, gt, rn, acts, total;
};
Reserve reserve_layout(const RnnGeom& g) {
  Reserve r{};
  size_t o = 0;
  r.hp = o; o += (size_t)(g.T + 1) * g.BH;
  r.cp = o; if (g.mode == RNN_LSTM) o += (size_t)(g.T + 1) * g.BH;
  r.gt = o; o += (size_t)g.T * g.B * g.GH;
  r.rn = o; if (g.mode == RNN_GRU) o += (size_t)g.T * g.BH;
  r.per_pl = o;
  r.acts = r.per_pl * g.L * g.D;
  r.total = r.acts + (size_t)(g.L - 1) * g.T * g.B * g.D * g.H;
  return r;
}

// workspace, in floats (one call): forward {XP [T*B*GH], RP [B*GH], bias [GH]};
// backward {dGW [T*B*GH], dGR [T*B*GH], gout [T*B*D*H], gin [T*B*inmax], tmp [T*B*inmax],
// dh_dir [2*BH], dc [BH], dh_rec [slices*BH]}
// The recurrent products of one time step are small (batch columns): their contraction is
// cut into slices so that enough workgroups run, and the gate kernels add the partial
// products.  Slices for a product with M rows, N columns, contraction K:
int step_slices(size_t M, size_t N, size_t K, int* ksplit) {
  const long long tiles = (long long)((M + 63) / 64) * ((N + 63) / 64), chunks = (long long)(K + 31) / 32;
  // from 32 tiles on, one step is bound by its two launches, not by the product
  long long k = tiles >= 32 ? 1 : 256 / tiles;
  if (k > chunks / 4) k = chunks / 4;   // at least four chunks of 32 per slice
  if (k > 32) k = 32;
  if (k < 1) k = 1;
  *ksplit = (int)k;
  return mfma_gemm_slices((int)K, (int)k);
}

// The fused path (one launch per time step for both directions) keeps the projections
// and gradients of both directions at once: forward {XP [D][T*B*GH], bias [D][GH]};
// backward = the layout above, then for the second direction {dGW, dGR, dh_dir [2*BH], dc [BH]}.
// slices of the contraction for the weight-gradient products (A * B^T over all time steps
// and batch columns): enough 64 x 64 tiles times slices to fill the machine several
// times over, at least eight chunks of 32 per slice
int wgrad_slices(size_t M, size_t N, size_t K) {
  const long long tiles = (long long)((M + 63) / 64) * ((N + 63) / 64), chunks = (long long)(K + 31) / 32;
  long long ns = 1024 / tiles;
  if (ns > chunks / 8) ns = chunks / 8;
  if (ns > 16) ns = 16;
  if (ns < 1) ns = 1;
  const long long cps = (chunks + ns - 1) / ns;
  return (int)((chunks + cps - 1) / cps);
}

int mm(const float* A, const float* B, float* C, size_t M, size_t N, size_t K, int ta, int tb,
       const float* bias, hipStream_t s) {
  return flhip_matmul(A, B, C, (int32_t)M, (int32_t)N, (int32_t)K, ta, tb, bias, FLHIP_F32, s);
}

// C = op(A) B in `*slices` partial products at C + k*M*N (see step_slices)
int mm_sliced(const float* A, const float* B, float* C, size_t M, size_t N, size_t K, int ta, int* slices,
              hipStream_t s) {
  int ksplit;
  const int ns = step_slices(M, N, K, &ksplit);
  if (ns > 1 && mfma_gemm(FLHIP_F32, ta ? 1 : 0, A, B, C, (int)M, (int)N, (int)K, nullptr, s, ksplit) >= 0) {
    *slices = ns;
    return check_launch("rnn (recurrent product)");
  }
  *slices = 1;
  return mm(A, B, C, M, N, K, ta, 0, nullptr, s);
}


// ... and at the end the partial products of the sliced weight-gradient products
size_t wgrad_scratch(const RnnGeom& g) {
  const size_t TB = (size_t)g.T * g.B, inmax = std::max<size_t>(g.I, (size_t)g.D * g.H);
  size_t n = 0;
  for (size_t M : {(size_t)g.I, inmax, (size_t)g.H}) {
    const int ns = wgrad_slices(M, g.GH, TB);
    if (ns > 1) n = std::max(n, (size_t)ns * M * g.GH);
  }
  return n;
}

size_t wgrad_scratch_offset(const RnnGeom& g) {
  const size_t TB = (size_t)g.T * g.B, inmax = std::max<size_t>(g.I, (size_t)g.D * g.H);
  int k;
  const size_t sb = step_slices(g.H, g.B, g.GH, &k);
  return 2 * TB * g.GH + TB * g.D * g.H + 2 * TB * inmax + (3 + sb) * g.BH +
         (size_t)(g.D - 1) * (2 * TB * g.GH + 3 * g.BH);
}

size_t workspace_floats(const RnnGeom& g) {
  const size_t TB = (size_t)g.T * g.B;
  int k;
  const size_t sf = step_slices(g.GH, g.B, g.H, &k);
  const size_t fwd = std::max(TB * g.GH + sf * g.B * g.GH + g.GH, (size_t)g.D * (TB * g.GH + g.GH));
  const size_t bwd = wgrad_scratch_offset(g) + wgrad_scratch(g);
  return std::max(fwd, bwd) + 64;
}

// the fused step kernels tile the hidden state by 16 and hold at most 64 batch columns
bool fused_applies(const RnnGeom& g) {
  return !options().rnn_unfused && g.H % 16 == 0 && g.B <= 64;
}

__device__ __forceinline__ float sigm(float v) { return 1.f / (1.f + expf(-v)); }

// bsum[q] = bW[q] + bR[q], except the GRU n gate, whose recurrent bias stays inside
// r * (R_n h + b_Rn)
__global__ void __launch_bounds__(256) rnn_bias_kernel(const float* __restrict__ bW, const float* __restrict__ bR,
                                                       float* __restrict__ bsum, int GH, int H, int mode) {
  const int q = blockIdx.x * 256 + threadIdx.x;
  if (q >= GH) return;
  bsum[q] = (mode == RNN_GRU && q >= 2 * H) ? bW[q] : bW[q] + bR[q];
}

// Dropout between layers: x[i] *= keep(i) / (1 - p) over the output sequence of `layer`, with the
// counter-based mask of (seed, layer, i): two rounds of a 32-bit finaliser, the top 24 bits as
// a uniform number in [0, 1).  The backward pass applies the same mask to the gradient.
__global__ void __launch_bounds__(256) rnn_dropout_kernel(float* __restrict__ x, size_t n, uint32_t seed_lo,
                                                          uint32_t seed_hi, uint32_t layer, float p, float scale) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  uint32_t h = (uint32_t)i * 0x9E3779B1u ^ seed_lo;
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  h += seed_hi + layer * 0x632BE5ABu;
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  const bool keep = (float)(h >> 8) * (1.0f / 16777216.0f) >= p;
  x[i] = keep ? x[i] * scale : 0.f;
}

__global__ void __launch_bounds__(256) rnn_init_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src ? src[i] : 0.f;
}

// out = a + sum of nb slices of b (either may be null); out may be a
__global__ void __launch_bounds__(256) rnn_add2_kernel(const float* a, const float* __restrict__ b, int nb,
                                                       float* out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = a ? a[i] : 0.f;
  if (b)
    for (int k = 0; k < nb; ++k) v += b[(size_t)k * n + i];
  out[i] = v;
}

struct CellFwd {
  const float* xp;    // [B][GH] input projection (+ biases) of this time step
  const float* rp;    // [nrp][B][GH] recurrent projection, in nrp partial products (two-kernel path)
  int nrp;
  const float* R;     // [GH][H] recurrent matrices (fused path)
  const float* bRn;   // GRU: recurrent bias of the n gate [H]
  const float* hp;    // [B][H] state before the step
  const float* cp;    // LSTM
  float* hn;          // [B][H] state after the step
  float* cn;
  float* gt;          // [B][GH] gate activations kept for the backward pass
  float* rn;          // GRU: R_n h + b_Rn
  float* out;         // layer output at this time step, this direction's slice; row pitch ldo
  float* hy;          // final state of the pseudo-layer (written at the last step) or null
  float* cy;
  int ldo;
};

// gate math of one (batch b, hidden h) element, in two halves so that a kernel can issue
// the loads before it computes the recurrent projections rp (one per gate)
template <int MODE>
struct CellFwdIn {
  float xp[MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1];
  float prev;   // LSTM: c before the step; GRU: h before the step
  float bRn;
};

template <int MODE>
__device__ __forceinline__ CellFwdIn<MODE> cell_fwd_load(const CellFwd& a, int b, int h, int H) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1;
  const size_t e = (size_t)b * H + h, q = (size_t)b * G * H + h;
  CellFwdIn<MODE> in;
#pragma unroll
  for (int gq = 0; gq < G; ++gq) in.xp[gq] = a.xp[q + (size_t)gq * H];
  in.prev = MODE == RNN_LSTM ? a.cp[e] : MODE == RNN_GRU ? a.hp[e] : 0.f;
  in.bRn = MODE == RNN_GRU ? a.bRn[h] : 0.f;
  return in;
}

template <int MODE>
__device__ __forceinline__ void cell_fwd_finish(const CellFwd& a, int b, int h, int H, const CellFwdIn<MODE>& in,
                                                const float* rp) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1;
  const size_t e = (size_t)b * H + h, q = (size_t)b * G * H + h;
  float hv;
  if (MODE == RNN_RELU || MODE == RNN_TANH) {
    const float pre = in.xp[0] + rp[0];
    hv = MODE == RNN_RELU ? (pre > 0.f ? pre : 0.f) : tanhf(pre);
    a.gt[q] = hv;
  } else if (MODE == RNN_LSTM) {
    const float ig = sigm(in.xp[0] + rp[0]), fg = sigm(in.xp[G > 1 ? 1 : 0] + rp[G > 1 ? 1 : 0]);
    const float gg = tanhf(in.xp[G > 2 ? 2 : 0] + rp[G > 2 ? 2 : 0]), og = sigm(in.xp[G > 3 ? 3 : 0] + rp[G > 3 ? 3 : 0]);
    const float c = fg * in.prev + ig * gg;
    a.cn[e] = c;
    if (a.cy) a.cy[e] = c;
    hv = og * tanhf(c);
    a.gt[q] = ig; a.gt[q + H] = fg; a.gt[q + 2 * H] = gg; a.gt[q + 3 * H] = og;
  } else {
    const float rg = sigm(in.xp[0] + rp[0]), zg = sigm(in.xp[G > 1 ? 1 : 0] + rp[G > 1 ? 1 : 0]);
    const float rn = rp[G > 2 ? 2 : 0] + in.bRn;
    const float ng = tanhf(in.xp[G > 2 ? 2 : 0] + rg * rn);
    a.rn[e] = rn;
    hv = (1.f - zg) * ng + zg * in.prev;
    a.gt[q] = rg; a.gt[q + H] = zg; a.gt[q + 2 * H] = ng;
  }
  a.hn[e] = hv;
  a.out[(size_t)b * a.ldo + h] = hv;
  if (a.hy) a.hy[e] = hv;
}

template <int MODE>
__global__ void __launch_bounds__(256) rnn_cell_fwd(CellFwd a, int B, int H) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= B * H) return;
  const int b = e / H, h = e - b * H;
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1;
  const size_t q = (size_t)b * G * H + h;
  const CellFwdIn<MODE> in = cell_fwd_load<MODE>(a, b, h, H);
  float rp[G];
#pragma unroll
  for (int gq = 0; gq < G; ++gq) rp[gq] = 0.f;
  for (int k = 0; k < a.nrp; ++k) {
    const float* r = a.rp + (size_t)k * B * G * H + q;
#pragma unroll
    for (int gq = 0; gq < G; ++gq) rp[gq] += r[gq * H];
  }
  cell_fwd_finish<MODE>(a, b, h, H, in, rp);
}

// One time step of up to two directions in one launch: recurrent product and gate math.
// A workgroup owns four hidden units (blockIdx.x) of one direction (blockIdx.y): its
// 16-row matrix-core tile is {gate g, unit hh} = row 4*g + hh of the recurrent
// matrices, its columns are the batch (NBT tiles of 16, batch <= 64), and the four
// waves split the contraction over the hidden state in interleaved chunks of 16.  A
// lane's 16-byte load supplies the operands of four 16x16x4 products (the k index of a
// lane group is permuted the same way on both operands).  The partial tiles meet in
// LDS, then one thread per (batch, unit) applies the gates; those threads issue the
// loads of their gate inputs before the product, so that the two latencies overlap.
// Needs H % 16 == 0.
struct StepFwd {
  CellFwd d[2];
  int B, H;
};
constexpr int STEP_FWD_WAVES = 4;

template <int MODE, int NBT>
__global__ void __launch_bounds__(64 * STEP_FWD_WAVES) rnn_step_fwd(StepFwd p) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1, NB = NBT * 16, W = STEP_FWD_WAVES;
  __shared__ float red[W][16][NB + 1];
  const CellFwd& a = p.d[blockIdx.y];
  const int H = p.H, B = p.B, h0 = blockIdx.x * 4;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fg = lane >> 4;
  const bool cell = tid < 4 * B;
  const int cb = tid >> 2, ch = h0 + (tid & 3);
  CellFwdIn<MODE> cin{};
  if (cell) cin = cell_fwd_load<MODE>(a, cb, ch, H);
  const int gate = fr >> 2;
  const bool av = gate < G;
  const float* ap = a.R + ((size_t)(av ? gate : 0) * H + h0 + (fr & 3)) * H + 4 * fg;
  const float* bp[NBT];
  bool bv[NBT];
#pragma unroll
  for (int nt = 0; nt < NBT; ++nt) {
    const int b = nt * 16 + fr;
    bv[nt] = b < B;
    bp[nt] = a.hp + (size_t)(bv[nt] ? b : 0) * H + 4 * fg;
  }
  floatx4_t acc[NBT];
#pragma unroll
  for (int nt = 0; nt < NBT; ++nt) acc[nt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  // U chunks are in flight per wave at a time: the loop is bound by the latency of
  // its loads, not by the products
  constexpr int U = NBT == 4 ? 4 : 8;
  const int chunks = H >> 4;
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int c0 = wave; c0 < chunks; c0 += W * U) {
    float4 ra[U], rb[U][NBT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // every load is issued (from a clamped, valid address) before any is used
      const int c = min(c0 + W * u, chunks - 1);
      ra[u] = *reinterpret_cast<const float4*>(ap + c * 16);
#pragma unroll
      for (int nt = 0; nt < NBT; ++nt) rb[u][nt] = *reinterpret_cast<const float4*>(bp[nt] + c * 16);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool in = c0 + W * u < chunks;
      if (!(in && av)) ra[u] = zero4;
#pragma unroll
      for (int nt = 0; nt < NBT; ++nt)
        if (!(in && bv[nt])) rb[u][nt] = zero4;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float av4[4] = {ra[u].x, ra[u].y, ra[u].z, ra[u].w};
#pragma unroll
      for (int nt = 0; nt < NBT; ++nt) {
        const float bv4[4] = {rb[u][nt].x, rb[u][nt].y, rb[u][nt].z, rb[u][nt].w};
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(av4[m], bv4[m], acc[nt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int nt = 0; nt < NBT; ++nt)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * fg + r][nt * 16 + fr] = acc[nt][r];
  __syncthreads();
  if (cell) {
    const int hh = tid & 3;
    float rp[G];
#pragma unroll
    for (int gq = 0; gq < G; ++gq) {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < W; ++wv) v += red[wv][gq * 4 + hh][cb];
      rp[gq] = v;
    }
    cell_fwd_finish<MODE>(a, cb, ch, H, cin, rp);
  }
}

struct CellBwd {
  const float* gout;  // gradient of the layer output at this time step, this direction's slice; pitch ldo (may be null)
  const float* dh_a;  // gradient reaching h through the recurrence: direct part ...
  const float* dh_b;  // ... and the part through the recurrent matrices, in ndhb partial products
  int ndhb;           //     (either pointer may be null)
  const float* R;         // fused path: recurrent matrices [GH][H] and the recurrent-side
  const float* dgr_next;  // pre-activation gradients [B][GH] of the step walked before (or null)
  float* dc;          // LSTM: in = gradient of c after the step, out = of c before it
  const float* gt;    // gate activations of the step
  const float* cp;    // LSTM: c before the step
  const float* cn;    //       c after the step
  const float* hp;    // state before the step
  const float* rn;    // GRU
  float* dgw;         // [B][GH] pre-activation gradients seen by the input side
  float* dgr;         // [B][GH] ... by the recurrent side
  float* dh_dir;      // [B][H] direct gradient towards the previous state (GRU: go * z, else 0)
  int ldo;
};

// gradient math of one (batch b, hidden h) element in two halves (loads, then math and
// stores); rec = gradient arriving through the recurrent matrices
template <int MODE>
struct CellBwdIn {
  float go;     // gradient of the output + direct recurrent part
  float gt[MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1];
  float cn, cp, dc;   // LSTM
  float hp, rn;       // GRU
};

template <int MODE>
__device__ __forceinline__ CellBwdIn<MODE> cell_bwd_load(const CellBwd& a, int b, int h, int H) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1;
  const size_t e = (size_t)b * H + h, q = (size_t)b * G * H + h;
  CellBwdIn<MODE> in{};
  in.go = a.gout ? a.gout[(size_t)b * a.ldo + h] : 0.f;
  if (a.dh_a) in.go += a.dh_a[e];
#pragma unroll
  for (int gq = 0; gq < G; ++gq) in.gt[gq] = a.gt[q + (size_t)gq * H];
  if (MODE == RNN_LSTM) {
    in.cn = a.cn[e]; in.cp = a.cp[e]; in.dc = a.dc[e];
  }
  if (MODE == RNN_GRU) {
    in.hp = a.hp[e]; in.rn = a.rn[e];
  }
  return in;
}

template <int MODE>
__device__ __forceinline__ void cell_bwd_finish(const CellBwd& a, int b, int h, int H, const CellBwdIn<MODE>& in,
                                                float rec) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1;
  const size_t e = (size_t)b * H + h, q = (size_t)b * G * H + h;
  const float go = in.go + rec;
  float direct = 0.f;
  if (MODE == RNN_RELU || MODE == RNN_TANH) {
    const float hv = in.gt[0];
    const float gp = MODE == RNN_RELU ? (hv > 0.f ? go : 0.f) : go * (1.f - hv * hv);
    a.dgw[q] = gp;
    a.dgr[q] = gp;
  } else if (MODE == RNN_LSTM) {
    const float ig = in.gt[0], fg = in.gt[G > 1 ? 1 : 0], gg = in.gt[G > 2 ? 2 : 0], og = in.gt[G > 3 ? 3 : 0];
    const float tc = tanhf(in.cn);
    const float dc = in.dc + go * og * (1.f - tc * tc);
    const float v0 = dc * gg * ig * (1.f - ig), v1 = dc * in.cp * fg * (1.f - fg);
    const float v2 = dc * ig * (1.f - gg * gg), v3 = go * tc * og * (1.f - og);
    a.dgw[q] = v0; a.dgw[q + H] = v1; a.dgw[q + 2 * H] = v2; a.dgw[q + 3 * H] = v3;
    a.dgr[q] = v0; a.dgr[q + H] = v1; a.dgr[q + 2 * H] = v2; a.dgr[q + 3 * H] = v3;
    a.dc[e] = dc * fg;
  } else {
    const float rg = in.gt[0], zg = in.gt[G > 1 ? 1 : 0], ng = in.gt[G > 2 ? 2 : 0], rn = in.rn;
    const float dn = go * (1.f - zg) * (1.f - ng * ng);
    const float v0 = dn * rn * rg * (1.f - rg), v1 = go * (in.hp - ng) * zg * (1.f - zg);
    a.dgw[q] = v0; a.dgw[q + H] = v1; a.dgw[q + 2 * H] = dn;
    a.dgr[q] = v0; a.dgr[q + H] = v1; a.dgr[q + 2 * H] = dn * rg;
    direct = go * zg;
  }
  a.dh_dir[e] = direct;
}

template <int MODE>
__global__ void __launch_bounds__(256) rnn_cell_bwd(CellBwd a, int B, int H) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= B * H) return;
  const int b = e / H, h = e - b * H;
  const CellBwdIn<MODE> in = cell_bwd_load<MODE>(a, b, h, H);
  float rec = 0.f;
  if (a.dh_b)
    for (int k = 0; k < a.ndhb; ++k) rec += a.dh_b[(size_t)k * B * H + e];
  cell_bwd_finish<MODE>(a, b, h, H, in, rec);
}

// One backward time step of up to two directions in one launch.  A workgroup owns 16
// hidden units of one direction: rows of its matrix-core tile are the units (columns
// of the recurrent matrices, 64 contiguous bytes per contraction index), columns the
// batch.  Its sixteen waves split the contraction over the gate rows (G*H) in
// interleaved chunks of 16 (with four batch tiles: eight groups of two waves, each wave
// two of the tiles); the partial tiles meet in LDS and one thread per (unit, batch)
// applies the gate gradients of the step, which become the next launch's operand.
// Those threads issue their loads before the product.  H % 16 == 0.
struct StepBwd {
  CellBwd d[2];
  int B, H;
};

template <int MODE, int NBT>
__global__ void __launch_bounds__(1024) rnn_step_bwd(StepBwd p) {
  constexpr int G = MODE == RNN_LSTM ? 4 : MODE == RNN_GRU ? 3 : 1, NB = NBT * 16;
  constexpr int NW = NBT == 4 ? 2 : NBT;      // batch tiles per wave
  constexpr int KG = 16 / (NBT / NW);         // wave groups along the contraction
  __shared__ float red[KG][16][NB + 1];
  const CellBwd& a = p.d[blockIdx.y];
  const int H = p.H, B = p.B, h0 = blockIdx.x * 16, GH = G * H;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fg = lane >> 4;
  const bool cell = tid < 16 * B;
  const int cb = tid >> 4, ch = h0 + (tid & 15);
  CellBwdIn<MODE> cin{};
  if (cell) cin = cell_bwd_load<MODE>(a, cb, ch, H);
  const bool have = a.dgr_next != nullptr;
  if (have) {
    const int kg = wave % KG, nt0 = (wave / KG) * NW;
    const float* ap = a.R + (size_t)(4 * fg) * H + h0 + fr;
    const float* bp[NW];
    bool bv[NW];
#pragma unroll
    for (int nt = 0; nt < NW; ++nt) {
      const int b = (nt0 + nt) * 16 + fr;
      bv[nt] = b < B;
      bp[nt] = a.dgr_next + (size_t)(bv[nt] ? b : 0) * GH + 4 * fg;
    }
    floatx4_t acc[NW];
#pragma unroll
    for (int nt = 0; nt < NW; ++nt) acc[nt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    constexpr int U = NW == 2 ? 4 : 8;   // chunks in flight per wave (registers: 128 per thread)
    const int chunks = GH >> 4;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int c0 = kg; c0 < chunks; c0 += KG * U) {
      float ra[U][4];
      float4 rb[U][NW];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = min(c0 + KG * u, chunks - 1);
#pragma unroll
        for (int m = 0; m < 4; ++m) ra[u][m] = ap[((size_t)c * 16 + m) * H];
#pragma unroll
        for (int nt = 0; nt < NW; ++nt) rb[u][nt] = *reinterpret_cast<const float4*>(bp[nt] + c * 16);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool in = c0 + KG * u < chunks;
#pragma unroll
        for (int m = 0; m < 4; ++m)
          if (!in) ra[u][m] = 0.f;
#pragma unroll
        for (int nt = 0; nt < NW; ++nt)
          if (!(in && bv[nt])) rb[u][nt] = zero4;
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int nt = 0; nt < NW; ++nt) {
          const float bv4[4] = {rb[u][nt].x, rb[u][nt].y, rb[u][nt].z, rb[u][nt].w};
#pragma unroll
          for (int m = 0; m < 4; ++m)
            acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[u][m], bv4[m], acc[nt], 0, 0, 0);
        }
    }
#pragma unroll
    for (int nt = 0; nt < NW; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[kg][4 * fg + r][(nt0 + nt) * 16 + fr] = acc[nt][r];
  }
  __syncthreads();
  if (cell) {
    float rec = 0.f;
    if (have) {
#pragma unroll
      for (int k = 0; k < KG; ++k) rec += red[k][tid & 15][cb];
    }
    cell_bwd_finish<MODE>(a, cb, ch, H, cin, rec);
  }
}

inline unsigned nblocks(size_t n) { return (unsigned)((n + 255) / 256); }

// dst [M x N] = A [M x K] * B^T, through `scratch` when the contraction is cut into slices
int mm_nt(const float* A, const float* B, float* dst, size_t M, size_t N, size_t K, float* scratch, hipStream_t s) {
  const int ns = wgrad_slices(M, N, K);
  if (ns <= 1) return gemm_nt(FLHIP_F32, A, B, dst, (int)M, (int)N, (int)K, 1, s);
  if (const int rc = gemm_nt(FLHIP_F32, A, B, scratch, (int)M, (int)N, (int)K, ns, s)) return rc;
  hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(M * N)), dim3(256), 0, s, (const float*)nullptr, scratch, ns, dst,
                     M * N);
  return FLHIP_OK;
}

template <int MODE>
int forward_pl(const RnnGeom& g, int pl, const float* in, size_t inl, const float* w, const float* hx,
               const float* cx, float* out, float* hy, float* cy, float* res, float* ws, hipStream_t s) {
  const Reserve r = reserve_layout(g);
  const Offsets o = offsets(g, pl);
  const int dir = pl % g.D;
  const size_t TB = (size_t)g.T * g.B;
  float* HP = res + (size_t)pl * r.per_pl + r.hp;
  float* CP = res + (size_t)pl * r.per_pl + r.cp;
  float* GT = res + (size_t)pl * r.per_pl + r.gt;
  float* RN = res + (size_t)pl * r.per_pl + r.rn;
  float* XP = ws;
  float* RP = XP + TB * g.GH;
  int kdummy;
  float* bsum = RP + (size_t)step_slices(g.GH, g.B, g.H, &kdummy) * g.B * g.GH;
  hipLaunchKernelGGL(rnn_bias_kernel, dim3(nblocks(g.GH)), dim3(256), 0, s, w + o.bW, w + o.bR, bsum,
                     (int)g.GH, g.H, g.mode);
  // XP [GH x TB] = W [GH x in] (row-major = a column-major in x GH matrix, transposed) * IN [in x TB]
  if (const int rc = mm(w + o.W, in, XP, g.GH, TB, inl, 1, 0, bsum, s)) return rc;
  hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s, hx ? hx + (size_t)pl * g.BH : nullptr,
                     HP, g.BH);
  if (MODE == RNN_LSTM)
    hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s,
                       cx ? cx + (size_t)pl * g.BH : nullptr, CP, g.BH);
  for (int st = 0; st < g.T; ++st) {
    const int t = dir ? g.T - 1 - st : st;
    int nrp = 1;
    if (const int rc = mm_sliced(w + o.R, HP + (size_t)st * g.BH, RP, g.GH, g.B, g.H, 1, &nrp, s)) return rc;
    CellFwd a{};
    a.xp = XP + (size_t)t * g.B * g.GH;
    a.rp = RP;
    a.nrp = nrp;
    a.bRn = w + o.bR + 2 * g.H;
    a.hp = HP + (size_t)st * g.BH;
    a.cp = CP + (size_t)st * g.BH;
    a.hn = HP + (size_t)(st + 1) * g.BH;
    a.cn = CP + (size_t)(st + 1) * g.BH;
    a.gt = GT + (size_t)st * g.B * g.GH;
    a.rn = RN + (size_t)st * g.BH;
    a.ldo = g.D * g.H;
    a.out = out + (size_t)t * g.B * a.ldo + (size_t)dir * g.H;
    const bool last = st == g.T - 1;
    a.hy = last ? hy + (size_t)pl * g.BH : nullptr;
    a.cy = (last && cy && MODE == RNN_LSTM) ? cy + (size_t)pl * g.BH : nullptr;
    hipLaunchKernelGGL((rnn_cell_fwd<MODE>), dim3(nblocks(g.BH)), dim3(256), 0, s, a, g.B, g.H);
  }
  return check_launch("rnn_fwd");
}

template <int MODE, int NBT>
void launch_step_fwd(const StepFwd& p, int D, hipStream_t s) {
  hipLaunchKernelGGL((rnn_step_fwd<MODE, NBT>), dim3(p.H / 4, D), dim3(64 * STEP_FWD_WAVES), 0, s, p);
}

// one layer, all directions: per direction the input projection of all steps, then one
// launch per time step for both directions
template <int MODE>
int forward_layer_fused(const RnnGeom& g, int l, const float* in, size_t inl, const float* w, const float* hx,
                        const float* cx, float* out, float* hy, float* cy, float* res, float* ws, hipStream_t s) {
  const Reserve r = reserve_layout(g);
  const size_t TB = (size_t)g.T * g.B;
  for (int dir = 0; dir < g.D; ++dir) {
    const int pl = l * g.D + dir;
    const Offsets o = offsets(g, pl);
    float* XP = ws + (size_t)dir * TB * g.GH;
    float* bsum = ws + (size_t)g.D * TB * g.GH + (size_t)dir * g.GH;
    hipLaunchKernelGGL(rnn_bias_kernel, dim3(nblocks(g.GH)), dim3(256), 0, s, w + o.bW, w + o.bR, bsum,
                       (int)g.GH, g.H, g.mode);
    if (const int rc = mm(w + o.W, in, XP, g.GH, TB, inl, 1, 0, bsum, s)) return rc;
    hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s,
                       hx ? hx + (size_t)pl * g.BH : nullptr, res + (size_t)pl * r.per_pl + r.hp, g.BH);
    if (MODE == RNN_LSTM)
      hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s,
                         cx ? cx + (size_t)pl * g.BH : nullptr, res + (size_t)pl * r.per_pl + r.cp, g.BH);
  }
  for (int st = 0; st < g.T; ++st) {
    StepFwd p{};
    p.B = g.B;
    p.H = g.H;
    for (int dir = 0; dir < g.D; ++dir) {
      const int pl = l * g.D + dir, t = dir ? g.T - 1 - st : st;
      const Offsets o = offsets(g, pl);
      float* base = res + (size_t)pl * r.per_pl;
      CellFwd& a = p.d[dir];
      a.xp = ws + (size_t)dir * TB * g.GH + (size_t)t * g.B * g.GH;
      a.R = w + o.R;
      a.bRn = w + o.bR + 2 * g.H;
      a.hp = base + r.hp + (size_t)st * g.BH;
      a.cp = base + r.cp + (size_t)st * g.BH;
      a.hn = base + r.hp + (size_t)(st + 1) * g.BH;
      a.cn = base + r.cp + (size_t)(st + 1) * g.BH;
      a.gt = base + r.gt + (size_t)st * g.B * g.GH;
      a.rn = base + r.rn + (size_t)st * g.BH;
      a.ldo = g.D * g.H;
      a.out = out + (size_t)t * g.B * a.ldo + (size_t)dir * g.H;
      const bool last = st == g.T - 1;
      a.hy = last ? hy + (size_t)pl * g.BH : nullptr;
      a.cy = (last && cy && MODE == RNN_LSTM) ? cy + (size_t)pl * g.BH : nullptr;
    }
    if (g.B <= 16) launch_step_fwd<MODE, 1>(p, g.D, s);
    else if (g.B <= 32) launch_step_fwd<MODE, 2>(p, g.D, s);
    else launch_step_fwd<MODE, 4>(p, g.D, s);
  }
  return check_launch("rnn_fwd");
}

template <int MODE>
int backward_pl(const RnnGeom& g, int pl, const float* in, size_t inl, const float* w, const float* gout,
                const float* dhy, const float* dcy, float* gin, bool first_dir, float* dhx, float* dcx,
                float* dw, const float* res, float* ws, hipStream_t s) {
  const Reserve r = reserve_layout(g);
  const Offsets o = offsets(g, pl);
  const int dir = pl % g.D;
  const size_t TB = (size_t)g.T * g.B, inmax = std::max<size_t>(g.I, (size_t)g.D * g.H);
  const float* HP = res + (size_t)pl * r.per_pl + r.hp;
  const float* CP = res + (size_t)pl * r.per_pl + r.cp;
  const float* GT = res + (size_t)pl * r.per_pl + r.gt;
  const float* RN = res + (size_t)pl * r.per_pl + r.rn;
  float* dGW = ws;
  float* dGR = dGW + TB * g.GH;
  float* tmp = dGR + TB * g.GH + TB * g.D * g.H + TB * inmax;   // behind gout and gin
  float* dh_dir = tmp + TB * inmax;                               // two buffers, alternating
  float* dc = dh_dir + 2 * g.BH;
  float* dh_rec = dc + g.BH;                                      // as many slices as step_slices says
  if (MODE == RNN_LSTM)
    hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s,
                       dcy ? dcy + (size_t)pl * g.BH : nullptr, dc, g.BH);
  const float* dha = dhy ? dhy + (size_t)pl * g.BH : nullptr;   // direct part for the first step walked
  const float* dhb = nullptr;
  int ndhb = 1;
  for (int st = g.T - 1; st >= 0; --st) {
    const int t = dir ? g.T - 1 - st : st;
    CellBwd a{};
    a.ldo = g.D * g.H;
    a.gout = gout ? gout + (size_t)t * g.B * a.ldo + (size_t)dir * g.H : nullptr;
    a.dh_a = dha;
    a.dh_b = dhb;
    a.ndhb = ndhb;
    a.dc = dc;
    a.gt = GT + (size_t)st * g.B * g.GH;
    a.cp = CP + (size_t)st * g.BH;
    a.cn = CP + (size_t)(st + 1) * g.BH;
    a.hp = HP + (size_t)st * g.BH;
    a.rn = RN + (size_t)st * g.BH;
    a.dgw = dGW + (size_t)t * g.B * g.GH;
    a.dgr = dGR + (size_t)st * g.B * g.GH;
    a.dh_dir = dh_dir + (size_t)(st & 1) * g.BH;
    hipLaunchKernelGGL((rnn_cell_bwd<MODE>), dim3(nblocks(g.BH)), dim3(256), 0, s, a, g.B, g.H);
    // gradient through the recurrent matrices: dh_rec [H x B] = R^T [H x GH] * dGR[st] [GH x B]
    if (const int rc = mm_sliced(w + o.R, a.dgr, dh_rec, g.H, g.B, g.GH, 0, &ndhb, s)) return rc;
    dha = a.dh_dir;
    dhb = dh_rec;
  }
  if (dhx)
    hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s, dha, dhb, ndhb, dhx + (size_t)pl * g.BH,
                       g.BH);
  if (dcx && MODE == RNN_LSTM)
    hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s, dc, dcx + (size_t)pl * g.BH, g.BH);
  // gradient of the layer input: gin [in x TB] (+)= W^T [in x GH] * dGW [GH x TB]
  float* gdst = first_dir ? gin : tmp;
  if (const int rc = mm(w + o.W, dGW, gdst, inl, TB, g.GH, 0, 0, nullptr, s)) return rc;
  if (!first_dir)
    hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(TB * inl)), dim3(256), 0, s, gin, tmp, 1, gin, TB * inl);
  // dW [GH][in] row-major = column-major in x GH = IN [in x TB] * dGW^T; dR likewise with the
  // states before each step; the bias gradients are the row sums
  float* scratch = ws + wgrad_scratch_offset(g);
  if (const int rc = mm_nt(in, dGW, dw + o.W, inl, g.GH, TB, scratch, s)) return rc;
  if (const int rc = mm_nt(HP, dGR, dw + o.R, g.H, g.GH, TB, scratch, s)) return rc;
  if (const int rc = flhip_sum_columns(dGW, dw + o.bW, (int32_t)g.GH, (int32_t)TB, FLHIP_F32, s)) return rc;
  if (const int rc = flhip_sum_columns(dGR, dw + o.bR, (int32_t)g.GH, (int32_t)TB, FLHIP_F32, s)) return rc;
  return check_launch("rnn_bwd");
}

template <int MODE, int NBT>
void launch_step_bwd(const StepBwd& p, int D, hipStream_t s) {
  hipLaunchKernelGGL((rnn_step_bwd<MODE, NBT>), dim3(p.H / 16, D), dim3(1024), 0, s, p);
}

template <int MODE>
int backward_layer_fused(const RnnGeom& g, int l, const float* in, size_t inl, const float* w, const float* gout,
                         const float* dhy, const float* dcy, float* gin, float* dhx, float* dcx, float* dw,
                         const float* res, float* ws, hipStream_t s) {
  const Reserve r = reserve_layout(g);
  const size_t TB = (size_t)g.T * g.B, inmax = std::max<size_t>(g.I, (size_t)g.D * g.H);
  int kdummy;
  const size_t sb = step_slices(g.H, g.B, g.GH, &kdummy);
  float* tmp = ws + 2 * TB * g.GH + TB * g.D * g.H + TB * inmax;
  float* dh_rec = tmp + TB * inmax + 3 * g.BH;
  float* second = dh_rec + sb * g.BH;
  float *dGW[2], *dGR[2], *dh_dir[2], *dc[2];
  dGW[0] = ws; dGR[0] = ws + TB * g.GH; dh_dir[0] = tmp + TB * inmax; dc[0] = dh_dir[0] + 2 * g.BH;
  dGW[1] = second; dGR[1] = second + TB * g.GH; dh_dir[1] = second + 2 * TB * g.GH; dc[1] = dh_dir[1] + 2 * g.BH;
  if (MODE == RNN_LSTM)
    for (int dir = 0; dir < g.D; ++dir)
      hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s,
                         dcy ? dcy + (size_t)(l * g.D + dir) * g.BH : nullptr, dc[dir], g.BH);
  for (int st = g.T - 1; st >= 0; --st) {
    StepBwd p{};
    p.B = g.B;
    p.H = g.H;
    for (int dir = 0; dir < g.D; ++dir) {
      const int pl = l * g.D + dir, t = dir ? g.T - 1 - st : st;
      const Offsets o = offsets(g, pl);
      const float* base = res + (size_t)pl * r.per_pl;
      CellBwd& a = p.d[dir];
      a.ldo = g.D * g.H;
      a.gout = gout ? gout + (size_t)t * g.B * a.ldo + (size_t)dir * g.H : nullptr;
      const bool first = st == g.T - 1;
      a.dh_a = first ? (dhy ? dhy + (size_t)pl * g.BH : nullptr) : dh_dir[dir] + (size_t)((st + 1) & 1) * g.BH;
      a.R = w + o.R;
      a.dgr_next = first ? nullptr : dGR[dir] + (size_t)(st + 1) * g.B * g.GH;
      a.dc = dc[dir];
      a.gt = base + r.gt + (size_t)st * g.B * g.GH;
      a.cp = base + r.cp + (size_t)st * g.BH;
      a.cn = base + r.cp + (size_t)(st + 1) * g.BH;
      a.hp = base + r.hp + (size_t)st * g.BH;
      a.rn = base + r.rn + (size_t)st * g.BH;
      a.dgw = dGW[dir] + (size_t)t * g.B * g.GH;
      a.dgr = dGR[dir] + (size_t)st * g.B * g.GH;
      a.dh_dir = dh_dir[dir] + (size_t)(st & 1) * g.BH;
    }
    if (g.B <= 16) launch_step_bwd<MODE, 1>(p, g.D, s);
    else if (g.B <= 32) launch_step_bwd<MODE, 2>(p, g.D, s);
    else launch_step_bwd<MODE, 4>(p, g.D, s);
  }
  for (int dir = 0; dir < g.D; ++dir) {
    const int pl = l * g.D + dir;
    const Offsets o = offsets(g, pl);
    const float* HP = res + (size_t)pl * r.per_pl + r.hp;
    if (dhx) {
      int ndhb = 1;
      if (const int rc = mm_sliced(w + o.R, dGR[dir], dh_rec, g.H, g.B, g.GH, 0, &ndhb, s)) return rc;
      hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s, dh_dir[dir], dh_rec, ndhb,
                         dhx + (size_t)pl * g.BH, g.BH);
    }
    if (dcx && MODE == RNN_LSTM)
      hipLaunchKernelGGL(rnn_init_kernel, dim3(nblocks(g.BH)), dim3(256), 0, s, dc[dir], dcx + (size_t)pl * g.BH,
                         g.BH);
    float* gdst = dir == 0 ? gin : tmp;
    if (const int rc = mm(w + o.W, dGW[dir], gdst, inl, TB, g.GH, 0, 0, nullptr, s)) return rc;
    if (dir)
      hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(TB * inl)), dim3(256), 0, s, gin, tmp, 1, gin, TB * inl);
    float* scratch = ws + wgrad_scratch_offset(g);
    if (const int rc = mm_nt(in, dGW[dir], dw + o.W, inl, g.GH, TB, scratch, s)) return rc;
    if (const int rc = mm_nt(HP, dGR[dir], dw + o.R, g.H, g.GH, TB, scratch, s)) return rc;
    if (const int rc = flhip_sum_columns(dGW[dir], dw + o.bW, (int32_t)g.GH, (int32_t)TB, FLHIP_F32, s)) return rc;
    if (const int rc = flhip_sum_columns(dGR[dir], dw + o.bR, (int32_t)g.GH, (int32_t)TB, FLHIP_F32, s)) return rc;
  }
  return check_launch("rnn_bwd");
}

}  // namespace
}  // namespace flhip

using namespace flhip;

extern "C" size_t flhip_rnn_param_count(const flhip_rnn_desc* d) {
  RnnGeom g;
  return make_geom(d, &g) == FLHIP_OK ? g.nparams : 0;
}
extern "C" size_t flhip_rnn_reserve_bytes(const flhip_rnn_desc* d) {
  RnnGeom g;
  return make_geom(d, &g) == FLHIP_OK ? reserve_layout(g).total * sizeof(float) : 0;
}
extern "C" size_t flhip_rnn_workspace_bytes(const flhip_rnn_desc* d) {
  RnnGeom g;
  return make_geom(d, &g) == FLHIP_OK ? workspace_floats(g) * sizeof(float) : 0;
}

extern "C" int flhip_rnn_fwd(const flhip_rnn_desc* d, const void* x, const void* hx, const void* cx,
                             const void* w, void* y, void* hy, void* cy, void* reserve,
                             size_t reserve_bytes, void* ws, size_t ws_bytes, void* stream) {
  RnnGeom g;
  const int rc0 = make_geom(d, &g);
  if (rc0 != FLHIP_OK) return rc0;
  FLHIP_REQUIRE(x && w && y && hy, "rnn_fwd: null argument");
  FLHIP_REQUIRE(reserve && reserve_bytes >= flhip_rnn_reserve_bytes(d), "rnn_fwd: reserve buffer too small");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_rnn_workspace_bytes(d), "rnn_fwd: workspace too small");
  hipStream_t s = as_stream(stream);
  const Reserve r = reserve_layout(g);
  float* res = static_cast<float*>(reserve);
  const float* wf = static_cast<const float*>(w);
  const size_t act = (size_t)g.T * g.B * g.D * g.H;
  for (int l = 0; l < g.L; ++l) {
    const float* in = l == 0 ? static_cast<const float*>(x) : res + r.acts + (size_t)(l - 1) * act;
    float* out = l == g.L - 1 ? static_cast<float*>(y) : res + r.acts + (size_t)l * act;
    const size_t inl = l == 0 ? g.I : (size_t)g.D * g.H;
    if (fused_applies(g)) {
      int rc;
      auto args = [&](auto fn) {
        return fn(g, l, in, inl, wf, static_cast<const float*>(hx), static_cast<const float*>(cx), out,
                  static_cast<float*>(hy), static_cast<float*>(cy), res, static_cast<float*>(ws), s);
      };
      switch (g.mode) {
        case RNN_RELU: rc = args(forward_layer_fused<RNN_RELU>); break;
        case RNN_TANH: rc = args(forward_layer_fused<RNN_TANH>); break;
        case RNN_LSTM: rc = args(forward_layer_fused<RNN_LSTM>); break;
        default: rc = args(forward_layer_fused<RNN_GRU>);
      }
      if (rc != FLHIP_OK) return rc;
    } else {
      for (int dir = 0; dir < g.D; ++dir) {
        const int pl = l * g.D + dir;
        int rc;
        auto args = [&](auto fn) {
          return fn(g, pl, in, inl, wf, static_cast<const float*>(hx), static_cast<const float*>(cx), out,
                    static_cast<float*>(hy), static_cast<float*>(cy), res, static_cast<float*>(ws), s);
        };
        switch (g.mode) {
          case RNN_RELU: rc = args(forward_pl<RNN_RELU>); break;
          case RNN_TANH: rc = args(forward_pl<RNN_TANH>); break;
          case RNN_LSTM: rc = args(forward_pl<RNN_LSTM>); break;
          default: rc = args(forward_pl<RNN_GRU>);
        }
        if (rc != FLHIP_OK) return rc;
      }
    }
    // what the next layer reads (and the backward pass reads again as that layer's input); the
    // layer's own recurrence and hy / cy used the states kept beside it in the reserve buffer
    if (g.dropout > 0.f && l + 1 < g.L)
      hipLaunchKernelGGL(rnn_dropout_kernel, dim3(nblocks(act)), dim3(256), 0, s, out, act, g.seed_lo, g.seed_hi,
                         (uint32_t)l, g.dropout, 1.0f / (1.0f - g.dropout));
  }
  return check_launch("rnn_fwd");
}

extern "C" int flhip_rnn_bwd(const flhip_rnn_desc* d, const void* x, const void* w, const void* dy,
                             const void* dhy, const void* dcy, const void* reserve,
                             size_t reserve_bytes, void* dx, void* dhx, void* dcx, void* dw, void* ws,
                             size_t ws_bytes, void* stream) {
  RnnGeom g;
  const int rc0 = make_geom(d, &g);
  if (rc0 != FLHIP_OK) return rc0;
  FLHIP_REQUIRE(x && w && dx && dw, "rnn_bwd: null argument");
  FLHIP_REQUIRE(reserve && reserve_bytes >= flhip_rnn_reserve_bytes(d),
                "rnn_bwd: needs the reserve buffer of the forward pass");
  FLHIP_REQUIRE(ws && ws_bytes >= flhip_rnn_workspace_bytes(d), "rnn_bwd: workspace too small");
  hipStream_t s = as_stream(stream);
  const Reserve r = reserve_layout(g);
  const float* res = static_cast<const float*>(reserve);
  const float* wf = static_cast<const float*>(w);
  float* wsf = static_cast<float*>(ws);
  const size_t TB = (size_t)g.T * g.B, act = TB * g.D * g.H, inmax = std::max<size_t>(g.I, (size_t)g.D * g.H);
  float* goutbuf = wsf + 2 * TB * g.GH;
  float* ginbuf = goutbuf + act;
  const float* gout = static_cast<const float*>(dy);   // gradient of the top layer's output (may be null)
  for (int l = g.L - 1; l >= 0; --l) {
    const float* in = l == 0 ? static_cast<const float*>(x) : res + r.acts + (size_t)(l - 1) * act;
    const size_t inl = l == 0 ? g.I : (size_t)g.D * g.H;
    float* gin = l == 0 ? static_cast<float*>(dx) : ginbuf;
    if (fused_applies(g)) {
      int rc;
      auto args = [&](auto fn) {
        return fn(g, l, in, inl, wf, gout, static_cast<const float*>(dhy), static_cast<const float*>(dcy), gin,
                  static_cast<float*>(dhx), static_cast<float*>(dcx), static_cast<float*>(dw), res, wsf, s);
      };
      switch (g.mode) {
        case RNN_RELU: rc = args(backward_layer_fused<RNN_RELU>); break;
        case RNN_TANH: rc = args(backward_layer_fused<RNN_TANH>); break;
        case RNN_LSTM: rc = args(backward_layer_fused<RNN_LSTM>); break;
        default: rc = args(backward_layer_fused<RNN_GRU>);
      }
      if (rc != FLHIP_OK) return rc;
    } else {
      for (int dir = 0; dir < g.D; ++dir) {
        const int pl = l * g.D + dir;
        int rc;
        auto args = [&](auto fn) {
          return fn(g, pl, in, inl, wf, gout, static_cast<const float*>(dhy), static_cast<const float*>(dcy),
                    gin, dir == 0, static_cast<float*>(dhx), static_cast<float*>(dcx), static_cast<float*>(dw),
                    res, wsf, s);
        };
        switch (g.mode) {
          case RNN_RELU: rc = args(backward_pl<RNN_RELU>); break;
          case RNN_TANH: rc = args(backward_pl<RNN_TANH>); break;
          case RNN_LSTM: rc = args(backward_pl<RNN_LSTM>); break;
          default: rc = args(backward_pl<RNN_GRU>);
        }
        if (rc != FLHIP_OK) return rc;
      }
    }
    if (l > 0) {
      // the gradient of this layer's input is the gradient of the output of the layer below
      hipLaunchKernelGGL(rnn_add2_kernel, dim3(nblocks(TB * inl)), dim3(256), 0, s, ginbuf, (const float*)nullptr, 0,
                         goutbuf, TB * inl);
      gout = goutbuf;
      if (g.dropout > 0.f)
        hipLaunchKernelGGL(rnn_dropout_kernel, dim3(nblocks(act)), dim3(256), 0, s, goutbuf, act, g.seed_lo, g.seed_hi,
                           (uint32_t)(l - 1), g.dropout, 1.0f / (1.0f - g.dropout));
    }
  }
  (void)inmax;
  return FLHIP_OK;
}
