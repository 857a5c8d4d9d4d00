// Shared pieces of the MFMA convolution kernels.
#pragma once
#include <type_traits>

#include "conv2d.h"

namespace flhip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int MFMA_THREADS = 512;   // 8 waves: 2 per SIMD
constexpr int MFMA_BM = 64;         // result rows (channels) per workgroup

// Number of compute units of the current device (256 on MI355X).
int mfma_num_cus();

// Raises the dynamic-LDS limit of `func` when a launch needs more than the
// default 64 KiB.  Returns false when the device cannot provide `bytes`.
bool mfma_allow_lds(const void* func, size_t bytes);

}  // namespace flhip
