// Direct global-memory-to-LDS transfers (gfx950 global_load_lds_dwordx4) and the waits that order their readers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace nnvhip {

#pragma clang diagnostic ignored "-Winline-asm"
// 64 lanes x 16 bytes from global memory straight into LDS: lane l's 16 bytes at gbase + voff land at
// lds_addr + 16 * l.  The compiler does not see the LDS write; the caller orders readers behind it with
// wait_vm + block_barrier.  (m0 carries the LDS address of the transfer.)
__device__ __forceinline__ void lds_dma16(const double* gbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(gbase)
               : "memory", "m0");
}
__device__ __forceinline__ unsigned lds_addr_of(const void* p) {
  return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
__device__ __forceinline__ void block_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  // vmcnt <= N and nothing else (gfx9 encoding: vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8])
  __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

}  // namespace nnvhip
