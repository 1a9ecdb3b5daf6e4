// Building blocks shared by the matrix-core kernels: compile-time loops, the LDS
// swizzle, and memory operations issued as assembly with hand-counted waits.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>
#include "quant.h"

namespace ztvm {

template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), fully unrolled
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
template <int V>
using ic = std::integral_constant<int, V>;

// LDS rows of 64 f16 = eight 16-byte chunks. A 128-bit read serves 16 lanes per cycle = two
// 128-byte rows of banks, and rows of equal parity share a bank half, so the chunk index is
// XOR-ed with bits 1..3 of the row (measured conflict-free, 560 B/ns per CU).
__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row >> 1) & 7u; }

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// ---- memory operations as assembly. The compiler treats a global->LDS transfer as an LDS
// access of unknown order and from then on drains every counter at each wait it inserts; issued
// this way the transfers and register fetches are invisible to it and the kernel places exact
// s_waitcnt counts itself (vmcnt retires in issue order). A fetched register must pass through
// settle() before its first use: the empty dependency keeps the compiler from reading it early.
//
// 16 bytes per lane: global (base + voff + OFF) -> LDS (lds_base + 16*lane). The instruction
// adds its immediate offset to the LDS address as well, so M0 carries lds_base - OFF; callers
// keep lds_base >= OFF.
template <int OFF>
__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
               :
               : "v"(voff), "s"(base), "s"(lds_base - OFF), "n"(OFF)
               : "memory", "m0");
}
template <int OFF>
__device__ __forceinline__ void fetch32(uint32_t& v, const void* base, uint32_t voff) {
  asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void fetch64(u32x2& v, const void* base, uint32_t voff) {
  asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void fetch96(u32x3& v, const void* base, uint32_t voff) {
  asm volatile("global_load_dwordx3 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void fetch128(u32x4& v, const void* base, uint32_t voff) {
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void fetch16(uint32_t& v, const void* base, uint32_t voff) {
  asm volatile("global_load_ushort %0, %1, %2 offset:%3" : "=v"(v) : "v"(voff), "s"(base), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_lgkm() {
  asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(N));
}
// wait until at most N younger fetches are in flight, then release v
template <int N, class T>
__device__ __forceinline__ void settle(T& v) {
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N));
}
template <class T>
__device__ __forceinline__ void release(T& v) {
  asm volatile("" : "+v"(v));
}
__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" : : : "memory"); }

}  // namespace ztvm
