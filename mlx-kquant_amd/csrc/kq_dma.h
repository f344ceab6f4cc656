// Direct-to-LDS loads (global_load_lds_*) and the explicit waits that go with them.
//
// The compiler does not track when such a load has landed in LDS (it either ignores the dependence or waits for
// every outstanding load), so the loads are issued from inline assembly and every wait is an explicit
// s_waitcnt vmcnt(n): loads of a wave return in order, n = number of load instructions issued after the one
// whose data is needed.  Stores of the same wave also count in vmcnt; a store between two loads can only make
// such a wait last longer, never end it early.
#pragma once

#include <stdint.h>

#include <hip/hip_runtime.h>

namespace kqdma {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// LDS address of lane l: lds (wave-uniform) + 16 l (4 l for the 2-byte form, which writes a zero-extended dword).
__device__ __forceinline__ void dma16(const uint8_t* sbase, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
// 4-byte form: LDS address of lane l = lds + 4 l
__device__ __forceinline__ void dma4(const uint8_t* sbase, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
__device__ __forceinline__ void dma2(const uint8_t* sbase, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2" ::"s"(lds), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
__device__ __forceinline__ u32x4 gload16(const void* p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
typedef uint32_t u32x2_dma __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x2_dma gload8(const void* p) {
  u32x2_dma v;
  asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
template <int N>
__device__ __forceinline__ void vmwait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void lgkm_drain() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t*)p;
}

}  // namespace kqdma
