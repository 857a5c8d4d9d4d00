// Global memory -> LDS without a trip through vector registers: buffer loads with the LDS
// modifier (16 bytes per lane), written as inline assembly so that the kernels count their
// own loads in flight (for the compiler's LDS-load builtin the compiler inserts waits that
// drain every load).
#pragma once
#include <stdint.h>

namespace flhip {

typedef int intx4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_void_t;

// at most N of this wave's vector-memory operations outstanding (N a literal)
#define PD_WAIT_VM(N) asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory")

// raw buffer descriptor (the words of make_rsrc) as four scalars for the inline assembly below
__device__ __forceinline__ intx4_t pd_rsrc(const void* ptr, unsigned bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(ptr);
  return intx4_t{__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                 __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
                 __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
}
// 64 lanes x 16 bytes from rsrc + voff (per lane) + soff to the 1 KiB of LDS at lds_addr (workgroup
// address, the same for all lanes): lane l lands at lds_addr + 16 l.  m0 is not declared as clobbered (the
// compiler reserves it and warns); nothing else in these kernels uses it: no LDS-load builtin, no
// relative register moves, no messages.
__device__ __forceinline__ void pd_load_lds(intx4_t rsrc, unsigned lds_addr, int voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// workgroup-relative address of an LDS object, as the M0 value of pd_load_lds
__device__ __forceinline__ unsigned pd_lds_addr(const void* p) {
  return (unsigned)reinterpret_cast<uintptr_t>((lds_void_t)p);
}

}  // namespace flhip
