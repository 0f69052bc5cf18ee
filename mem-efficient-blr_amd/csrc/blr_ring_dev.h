// Device helpers of the kernels that copy operand tiles global -> LDS directly (no registers in between).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace blr {

constexpr int ring_vmcnt(int n) { return (n & 0xf) | ((n >> 4) << 14) | (7 << 4) | (0xf << 8); }   // s_waitcnt immediate: vmcnt = n only
typedef short s16x4 __attribute__((ext_vector_type(4)));
// 16 bytes per lane from base + off into LDS at lds + 16 * lane (base and lds are wave-uniform; lds goes through M0)
__device__ __forceinline__ void ring_load_lds(const void* base, uint32_t off, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ uint32_t ring_lds_addr(const void* p) {
  return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)((void __attribute__((address_space(3)))*)(p)));
}

}  // namespace blr
