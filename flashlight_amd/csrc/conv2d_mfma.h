// Shared pieces of the MFMA convolution kernels.
#pragma once
#include <type_traits>

#include "conv2d.h"

namespace flhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// The two 16-bit storage types on their matrix instructions (same shapes, same fp32 accumulators): the kernels hold
// operand fragments as 128 raw bits (bf16x8 registers whatever the type) and are templates on the element type E.
typedef __bf16 lo16_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 lo16_f16x8 __attribute__((ext_vector_type(8)));
template <typename E> struct Lo16;
template <> struct Lo16<bf16_t> {
  static constexpr int TAG = FLHIP_BF16;
  static constexpr uint32_t ONE2 = 0x3f803f80u;            // two ones
  template <typename V> static __device__ __forceinline__ floatx16 mma32(const V& a, const V& b, const floatx16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(lo16_bf16x8, a), __builtin_bit_cast(lo16_bf16x8, b), c, 0, 0, 0);
  }
  template <typename V> static __device__ __forceinline__ floatx4 mma16(const V& a, const V& b, const floatx4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lo16_bf16x8, a), __builtin_bit_cast(lo16_bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_bf16(a, b); }
  static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  static __device__ __forceinline__ float widen(uint16_t bits) { return __uint_as_float((uint32_t)bits << 16); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return f32_to_bf16(f); }
};
template <> struct Lo16<f16_t> {
  static constexpr int TAG = FLHIP_F16;
  static constexpr uint32_t ONE2 = 0x3c003c00u;
  template <typename V> static __device__ __forceinline__ floatx16 mma32(const V& a, const V& b, const floatx16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(lo16_f16x8, a), __builtin_bit_cast(lo16_f16x8, b), c, 0, 0, 0);
  }
  template <typename V> static __device__ __forceinline__ floatx4 mma16(const V& a, const V& b, const floatx4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(lo16_f16x8, a), __builtin_bit_cast(lo16_f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_f16(a, b); }
  static __device__ __forceinline__ float lo(uint32_t w) { return f16lo(w); }
  static __device__ __forceinline__ float hi(uint32_t w) { return f16hi(w); }
  static __device__ __forceinline__ float widen(uint16_t bits) { return f16_to_f32(f16_t{bits}); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return f32_to_f16(f).bits; }
};
// f(null pointer of the 16-bit element type of `dtype`)
template <typename F>
inline auto by_lo16(int dtype, F&& f) {
  if (dtype == FLHIP_F16) return f(static_cast<f16_t*>(nullptr));
  return f(static_cast<bf16_t*>(nullptr));
}

constexpr int MFMA_THREADS = 512;   // 8 waves: 2 per SIMD
constexpr int MFMA_BM = 64;         // result rows (channels) per workgroup

// Number of compute units of the current device (256 on MI355X).
int mfma_num_cus();

// Raises the dynamic-LDS limit of `func` when a launch needs more than the
// default 64 KiB.  Returns false when the device cannot provide `bytes`.
bool mfma_allow_lds(const void* func, size_t bytes);

}  // namespace flhip
