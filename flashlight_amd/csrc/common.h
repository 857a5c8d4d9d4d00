// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <type_traits>

#include "flhip.h"

namespace flhip {

// ---- errors ---------------------------------------------------------------
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);

#define FLHIP_REQUIRE(cond, msg)                                    \
  do {                                                              \
    if (!(cond)) return ::flhip::fail(FLHIP_INVALID_ARGUMENT, msg); \
  } while (0)

// Checks the launch itself; execution errors surface at the caller's next sync.
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(FLHIP_RUNTIME_ERROR,
                std::string(what) + ": " + hipGetErrorString(e));
  return FLHIP_OK;
}

// ---- storage types --------------------------------------------------------
typedef uint16_t bf16_t;  // raw bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}
// round to nearest even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32, two
// values per instruction when neighbours are converted together); the host pass of the
// compiler only parses this.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
}

// two values in one instruction: a in the low half of the result, b in the high half
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  typedef float pack_f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 pack_bf16x2 __attribute__((ext_vector_type(2)));
  const pack_f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, pack_bf16x2));
}

// IEEE half storage (Flashlight's f16): a type of its own, so that the element-wise helpers below can be
// overloaded on it.  Kernels that are templates on the storage type convert on load and store; sums are fp32.
struct f16_t {
  uint16_t bits;
};
__device__ __forceinline__ float f16_to_f32(f16_t v) { return (float)__builtin_bit_cast(_Float16, v.bits); }
// round to nearest even (v_cvt_f16_f32)
__device__ __forceinline__ f16_t f32_to_f16(float f) { return f16_t{__builtin_bit_cast(uint16_t, (_Float16)f)}; }
__device__ __forceinline__ uint32_t pack_f16(float a, float b) {
  return (uint32_t)f32_to_f16(a).bits | ((uint32_t)f32_to_f16(b).bits << 16);
}
__device__ __forceinline__ float f16lo(uint32_t w) { return f16_to_f32(f16_t{(uint16_t)(w & 0xffffu)}); }
__device__ __forceinline__ float f16hi(uint32_t w) { return f16_to_f32(f16_t{(uint16_t)(w >> 16)}); }

__device__ __forceinline__ float ld(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float ld(const f16_t* p, size_t i) { return f16_to_f32(p[i]); }
__device__ __forceinline__ void st(f16_t* p, size_t i, float v) { p[i] = f32_to_f16(v); }
__device__ __forceinline__ float ld(const bf16_t* p, size_t i) {
  return bf16_to_f32(p[i]);
}
__device__ __forceinline__ void st(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st(bf16_t* p, size_t i, float v) {
  p[i] = f32_to_bf16(v);
}

// four consecutive elements, 16-byte (f32) / 8-byte (bf16) aligned
__device__ __forceinline__ float4 ld4(const float* p, size_t i) {
  return *reinterpret_cast<const float4*>(p + i);
}
__device__ __forceinline__ float4 ld4(const bf16_t* p, size_t i) {
  uint2 r = *reinterpret_cast<const uint2*>(p + i);
  return make_float4(__uint_as_float(r.x << 16),
                     __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16),
                     __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ float4 ld4(const f16_t* p, size_t i) {
  uint2 r = *reinterpret_cast<const uint2*>(p + i);
  return make_float4(f16lo(r.x), f16hi(r.x), f16lo(r.y), f16hi(r.y));
}
__device__ __forceinline__ void st4(f16_t* p, size_t i, float4 v) {
  uint2 r;
  r.x = pack_f16(v.x, v.y);
  r.y = pack_f16(v.z, v.w);
  *reinterpret_cast<uint2*>(p + i) = r;
}
__device__ __forceinline__ void st4(float* p, size_t i, float4 v) {
  *reinterpret_cast<float4*>(p + i) = v;
}
__device__ __forceinline__ void st4(bf16_t* p, size_t i, float4 v) {
  uint2 r;
  r.x = pack_bf16(v.x, v.y);
  r.y = pack_bf16(v.z, v.w);
  *reinterpret_cast<uint2*>(p + i) = r;
}

// Streaming stores: the result is not read again by the kernel that writes it, so
// it should not displace re-used input lines from the caches.
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uintx2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void st4_stream(float* p, size_t i, float4 v) {
  const floatx4_t t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<floatx4_t*>(p + i));
}
__device__ __forceinline__ void st4_stream(bf16_t* p, size_t i, float4 v) {
  const uintx2_t t = {pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
  __builtin_nontemporal_store(t, reinterpret_cast<uintx2_t*>(p + i));
}

__device__ __forceinline__ void st4_stream(f16_t* p, size_t i, float4 v) {
  const uintx2_t t = {pack_f16(v.x, v.y), pack_f16(v.z, v.w)};
  __builtin_nontemporal_store(t, reinterpret_cast<uintx2_t*>(p + i));
}

// ---- buffer loads ------------------------------------------------------------
// Raw buffer descriptor over `bytes` bytes at p: loads at a byte offset at or
// past `bytes` return zero, which is how the gathers fetch padding.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ float buf_ld(__amdgpu_buffer_rsrc_t r, int byte_off, const float*) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 0));
}
__device__ __forceinline__ float buf_ld(__amdgpu_buffer_rsrc_t r, int byte_off, const bf16_t*) {
  return bf16_to_f32((bf16_t)__builtin_amdgcn_raw_buffer_load_b16(r, byte_off, 0, 0));
}

__device__ __forceinline__ float buf_ld(__amdgpu_buffer_rsrc_t r, int byte_off, const f16_t*) {
  return f16_to_f32(f16_t{(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, byte_off, 0, 0)});
}

// four consecutive elements at a byte offset (16-byte aligned for float, 8 for bf16)
typedef unsigned uintx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 buf_ld4(__amdgpu_buffer_rsrc_t r, int byte_off, const f16_t*) {
  const uintx2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 0);
  return make_float4(f16lo(v.x), f16hi(v.x), f16lo(v.y), f16hi(v.y));
}
__device__ __forceinline__ float4 buf_ld4(__amdgpu_buffer_rsrc_t r, int byte_off, const float*) {
  const uintx4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z),
                     __uint_as_float(v.w));
}
__device__ __forceinline__ float4 buf_ld4(__amdgpu_buffer_rsrc_t r, int byte_off, const bf16_t*) {
  const uintx2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 0);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                     __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}

// pointers into LDS (the host pass of the compiler only parses the kernels)
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) const float2* lds_f2;
typedef __attribute__((address_space(3))) const float* lds_f1;
#else
typedef const float2* lds_f2;
typedef const float* lds_f1;
#endif

// ---- small-integer division ------------------------------------------------------
// e / d for 0 <= e < 2^22 with inv = 1.0f / d: a float estimate corrected to the
// exact quotient (a handful of VALU operations instead of the ~30 of an integer
// division).  *rem receives e - q*d.
__device__ __forceinline__ int fast_div(int e, int d, float inv, int* rem) {
  int q = (int)((float)e * inv);
  int r = e - q * d;
  if (r < 0) {
    --q;
    r += d;
  }
  if (r >= d) {
    ++q;
    r -= d;
  }
  *rem = r;
  return q;
}

// ---- reductions -----------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum of `v` over the block; result valid in every thread.  `smem` holds at
// least blockDim.x/64 floats and may be reused after the call returns.
// (NW: the number of waves when the caller knows it at compile time - the loop over the waves' sums is then
// unrolled and its LDS reads go out together; 0: taken from blockDim)
template <int NW = 0>
__device__ __forceinline__ float block_sum(float v, float* smem) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = NW ? NW : (int)((blockDim.x + 63) >> 6);
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) smem[wid] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < nw; ++i) r += smem[i];
  return r;
}

// Two sums at once: the additions of two block_sum calls in the same order, with half the barriers.
// smem holds 2 * (number of waves) floats.
template <int NW = 0>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* smem) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = NW ? NW : (int)((blockDim.x + 63) >> 6);
  a = wave_sum(a);
  b = wave_sum(b);
  __syncthreads();
  if (lane == 0) {
    smem[wid] = a;
    smem[nw + wid] = b;
  }
  __syncthreads();
  float ra = 0.f, rb = 0.f;
#pragma unroll
  for (int i = 0; i < nw; ++i) {
    ra += smem[i];
    rb += smem[nw + i];
  }
  a = ra;
  b = rb;
}

// ---- elementwise kernels ------------------------------------------------------------
// out[i] = op(a[i], b[i]) (b may be null for a unary op), four elements per thread through
// 16-byte (float) / 8-byte (bf16) accesses; launch_elementwise handles tails and pointers
// that are not aligned for that with the element-wise kernel.  out may alias a or b.
template <typename T, typename Op>
__global__ void __launch_bounds__(256) ew_vec_kernel(const T* a, const T* b,
                                                     T* out, size_t nvec, Op op) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
    const float4 va = ld4(a, 4 * i);
    const float4 vb = b ? ld4(b, 4 * i) : va;
    st4(out, 4 * i, make_float4(op(va.x, vb.x), op(va.y, vb.y), op(va.z, vb.z), op(va.w, vb.w)));
  }
}
template <typename T, typename Op>
__global__ void __launch_bounds__(256) ew_kernel(const T* a, const T* b,
                                                 T* out, size_t n, Op op) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const float va = ld(a, i);
    st(out, i, op(va, b ? ld(b, i) : va));
  }
}
template <typename T, typename Op>
inline void launch_elementwise(const T* a, const T* b, T* out, size_t n, Op op, hipStream_t s) {
  auto blocks = [](size_t work) {
    size_t k = (work + 255) / 256;
    return (unsigned)(k > 65536 ? 65536 : k < 1 ? 1 : k);
  };
  const uintptr_t al = 4 * sizeof(T);
  const bool aligned = reinterpret_cast<uintptr_t>(a) % al == 0 && reinterpret_cast<uintptr_t>(out) % al == 0 &&
                       (!b || reinterpret_cast<uintptr_t>(b) % al == 0);
  const size_t nvec = aligned ? n / 4 : 0;
  if (nvec) hipLaunchKernelGGL((ew_vec_kernel<T, Op>), dim3(blocks(nvec)), dim3(256), 0, s, a, b, out, nvec, op);
  const size_t done = nvec * 4;
  if (done < n)
    hipLaunchKernelGGL((ew_kernel<T, Op>), dim3(blocks(n - done)), dim3(256), 0, s, a + done, b ? b + done : b,
                       out + done, n - done, op);
}

// ---- process-wide switches ---------------------------------------------------------
// Measurement / debugging aids.  They are read from the environment (FLHIP_<NAME>) once,
// when the library first needs them, and can be changed afterwards only through
// flhip_set_option(); no entry point calls getenv on its per-call path.
struct Options {
  enum { ALGO_AUTO = 0, ALGO_DIRECT, ALGO_GATHER, ALGO_TAPPED, ALGO_CONVERT };
  enum { SKIP_BF16 = 1, SKIP_GEMM1X1 = 2, SKIP_SLAB = 4, SKIP_TAPPED = 8, SKIP_STRIP = 16, SKIP_FIRST = 32, SKIP_WGRAD128 = 64, SKIP_PWDMA = 128, SKIP_WD32 = 256, SKIP_TAP1D = 512, SKIP_CELLS = 1024, SKIP_TAP2D = 2048 };
  int conv_algo = ALGO_AUTO;      // CONV_ALGO = direct | gather | tapped | convert
  unsigned conv_skip = 0;         // CONV_SKIP = comma list of bf16, gemm1x1, slab, tapped, strip, first, wgrad128, pwdma, wd32, tap1d, cells, tap2d
  int pw_pt = 2;                  // PW_PT = 2 | 4 | 8: position-tile width of the fp32 1x1 kernels / 32
  int pw16_pf = 0;                // PW16_PF = 1 / 4: one / four chunks (shallow / deep ring) in flight in the bf16 1x1 kernels, 2 / 8: the same with
                                  // tiles of 64 result channels in the direct-to-LDS kernels (0: by grid size)
  int conv_stack = 0;             // CONV_STACK = 1 | 2 | 4 | 8: images per tile of the bf16 3x3 kernel over planes that fit a tile (0: by grid size)
  int slab_waves = 0;             // SLAB_WAVES = 4 | 8: MFMA waves per workgroup of the fp32 3x3 kernels (0: by tile size)
  bool pw16_no_taps = false;      // PW16_NO_TAPS: bf16 windows with several taps stay off the gathered-taps path
  bool tapped_no_reorder = false; // TAPPED_NO_REORDER: tapped kernels read the original weight layout
  bool matmul_valu = false;       // MATMUL_VALU: flhip_matmul stays off the matrix cores
  int matmul_planes = -1;         // MATMUL_PLANES: bit m set = fp32 product of mode m (0: A B, 1: A^T B, 2: A B^T) with a
                                  // matrix as one image's plane whatever its shape; 0: never; -1: by shape
  bool matmul_fp32_cores = false; // MATMUL_FP32_CORES: 16-bit products stay on the fp32 matrix instructions
  bool rnn_unfused = false;       // RNN_UNFUSED: two-kernel rnn steps
  bool tap2d_all = false;         // TAP2D_ALL: the kernel for 3x3 windows over stacked planes takes every geometry it can, not only those of its measured rule
  int bn_algo = 0;                // BN_ALGO = split (1) | resident (2)
};
const Options& options();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

inline bool dtype_ok(int32_t dt) { return dt == FLHIP_F32 || dt == FLHIP_BF16 || dt == FLHIP_F16; }
inline size_t dtype_size(int32_t dt) { return dt == FLHIP_F32 ? 4 : 2; }
// the two 16-bit storage types (bf16 and IEEE half share the 16-bit matrix-core kernels)
inline bool is_lo16(int32_t dt) { return dt == FLHIP_BF16 || dt == FLHIP_F16; }

// Calls f with a null pointer of the storage type of `dt`:
//   by_dtype(dt, [&](auto* t) { using T = std::remove_pointer_t<decltype(t)>; return launch<T>(...); })
template <typename F>
inline auto by_dtype(int32_t dt, F&& f) {
  if (dt == FLHIP_F32) return f(static_cast<float*>(nullptr));
  if (dt == FLHIP_F16) return f(static_cast<f16_t*>(nullptr));
  return f(static_cast<bf16_t*>(nullptr));
}
#define FLHIP_T_OF(t) std::remove_pointer_t<decltype(t)>

}  // namespace flhip
