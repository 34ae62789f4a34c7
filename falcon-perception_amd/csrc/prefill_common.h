// Shared by the prefill kernels: loads from global memory straight into LDS (no staging registers)
// and an exchange between the two halves of a wavefront.
#ifndef FP_PREFILL_COMMON_H
#define FP_PREFILL_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fp {

// 16 bytes per lane from global memory to LDS at `lds` + lane * 16 (`lds` wavefront-uniform).
// Written as inline assembly on purpose: while the compiler knows of such a load in flight it turns
// every wait for an LDS read into a wait for all of them, which serialises the operand reads of a
// main loop against its MFMAs.  The code that issues these loads waits for them itself (vmcnt(0)
// before the barrier that publishes a tile).  Nothing else in these kernels uses M0.
__device__ __forceinline__ void load_to_lds(const char* src, char* lds) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds)));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(base), "v"(src) : "memory");
}

// The same with the address split into a wavefront-uniform base (scalar registers) and a 32-bit offset per lane.
__device__ __forceinline__ void load_to_lds(const char* base, uint32_t offset, char* lds) {
  const uint32_t m0v = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds)));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(m0v), "v"(offset), "s"(base) : "memory");
}

// max(x of lane l, x of lane l ^ 32) in both lanes, without the trip through LDS a shuffle takes:
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second, so
// from (x, x) it leaves the lower halves' values in one register and the upper halves' in the other.
// (Inline assembly: the compiler's builtin returned the first register for both results.)  The no-ops
// cover the wait states between a vector write, the swap and the next vector read.
__device__ __forceinline__ float max_across_lane_halves(float x) {
  float lo = x, hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
  return fmaxf(lo, hi);
}

}  // namespace fp
#endif
