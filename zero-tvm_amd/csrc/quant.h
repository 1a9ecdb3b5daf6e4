// Device-side unpack of 4-bit and 3-bit group-quantized weights into exact
// f16 integers, two values per 32-bit register, without integer->float
// conversion instructions.
//
// Trick: OR-ing a small integer field into the mantissa of a suitable f16
// constant yields (offset + q) exactly; one packed f16 subtract removes the
// offset. A field at mantissa bit r needs the constant whose ulp is 2^-r:
// 1024 (r=0), 128 (r=3), 64 (r=4), 8 (r=7).
//
// Both formats are consumed in blocks of 8 consecutive values and both come
// out in the same slot order  [v0,v4 | v1,v5 | v2,v6 | v3,v7]  so activations
// staged once in that order serve 4-bit and 3-bit rows alike.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ztvm {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// f32 -> f16 of a value that must first exist as an f32. Without the empty dependency the
// compiler folds the producing multiply / fused multiply-add into a mixed-precision
// instruction that rounds once, straight to f16 (and adds +0, which loses the sign of a zero
// product); the formats here are defined as round to f32, then round to f16.
__device__ __forceinline__ _Float16 narrow_f32(float v) {
  asm volatile("" : "+v"(v));
  return (_Float16)v;
}

__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ uint32_t as_u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// Position of value i (0..7) of an 8-value block in the slot order above.
__host__ __device__ constexpr int slot_of(int i) { return (i & 3) * 2 + (i >> 2); }
// Inverse: which value sits in slot s.
__host__ __device__ constexpr int value_in_slot(int s) { return (s >> 1) + (s & 1) * 4; }

// (a & mask) | c in ONE instruction. A VOP3 instruction of this ISA may read a
// single scalar operand, so the OR constant is kept in a vector register
// (callers hoist it out of their loops); left to itself the compiler emits a
// separate AND and OR, each with its own literal.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t c_vgpr) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(c_vgpr));
  return d;
}

// OR constants of the unpackers, materialised once per kernel in VGPRs.
struct UnpackConsts {
  uint32_t c4_lo, c4_hi;  // 4-bit: 1024|1024 and 64|64
  uint32_t c3_a, c3_b;    // 3-bit: 64|1024 and 8|128
  __device__ __forceinline__ void init() {
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(c4_lo));
    asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(c4_hi));
    asm volatile("v_mov_b32 %0, 0x64005400" : "=v"(c3_a));
    asm volatile("v_mov_b32 %0, 0x58004800" : "=v"(c3_b));
  }
};

// One u32 of eight 4-bit values (value i at bits [4i,4i+4)) -> 4 x h2 holding
// the exact integers 0..15 in slot order.
__device__ __forceinline__ void unpack4_block(uint32_t w, h2 q[4], const UnpackConsts& k) {
  const h2 k1024 = {(_Float16)1024.f, (_Float16)1024.f};
  const h2 k64 = {(_Float16)64.f, (_Float16)64.f};
  const uint32_t w8 = w >> 8;
  q[0] = as_h2(and_or(w, 0x000F000Fu, k.c4_lo)) - k1024;   // v0, v4
  q[1] = as_h2(and_or(w, 0x00F000F0u, k.c4_hi)) - k64;     // v1, v5
  q[2] = as_h2(and_or(w8, 0x000F000Fu, k.c4_lo)) - k1024;  // v2, v6
  q[3] = as_h2(and_or(w8, 0x00F000F0u, k.c4_hi)) - k64;    // v3, v7
}

// Two pre-shifted views of a 24-bit window of eight 3-bit values:
//   lo_view = window << 4  (v0 at bit 4, v1 at bit 7, v4 at bit 16, v5 at bit 19)
//   hi_view = window >> 2  (v2 at bit 4, v3 at bit 7, v6 at bit 16, v7 at bit 19)
// Bits outside the four fields may hold anything.
__device__ __forceinline__ void unpack3_views(uint32_t lo_view, uint32_t hi_view, h2 q[4], const UnpackConsts& k) {
  const h2 ka = {(_Float16)64.f, (_Float16)1024.f};  // fields at r=4 (lo half) and r=0 (hi half)
  const h2 kb = {(_Float16)8.f, (_Float16)128.f};    // fields at r=7 (lo half) and r=3 (hi half)
  q[0] = as_h2(and_or(lo_view, 0x00070070u, k.c3_a)) - ka;  // v0, v4
  q[1] = as_h2(and_or(lo_view, 0x00380380u, k.c3_b)) - kb;  // v1, v5
  q[2] = as_h2(and_or(hi_view, 0x00070070u, k.c3_a)) - ka;  // v2, v6
  q[3] = as_h2(and_or(hi_view, 0x00380380u, k.c3_b)) - kb;  // v3, v7
}

// 32 consecutive 3-bit values = 96 bits = three words (the row bitstream is
// LSB-first and 32-value chunks are word aligned). Block b is the 24-bit
// window at stream bit 24b; the views are taken straight from the stream with
// funnel shifts. q[4*b + j] is pair j of block b.
__device__ __forceinline__ void unpack3_chunk(uint32_t w0, uint32_t w1, uint32_t w2, h2 q[16], const UnpackConsts& k) {
  unpack3_views(w0 << 4, w0 >> 2, q + 0, k);                                                        // bits  0..23
  unpack3_views(__builtin_amdgcn_alignbit(w1, w0, 20), __builtin_amdgcn_alignbit(w1, w0, 26), q + 4, k);   // bits 24..47
  unpack3_views(__builtin_amdgcn_alignbit(w2, w1, 12), __builtin_amdgcn_alignbit(w2, w1, 18), q + 8, k);   // bits 48..71
  unpack3_views(w2 >> 4, w2 >> 10, q + 12, k);                                                      // bits 72..95
}

__device__ __forceinline__ void unpack4_chunk(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3, h2 q[16], const UnpackConsts& k) {
  unpack4_block(w0, q + 0, k);
  unpack4_block(w1, q + 4, k);
  unpack4_block(w2, q + 8, k);
  unpack4_block(w3, q + 12, k);
}

// 8-bit values, four per word (value i at bits [8i, 8i+8)): the byte goes into the mantissa of
// 1024, whose ulp is 1, so 1024 + q is exact for q < 1024. One word gives the pairs (v0,v2) and
// (v1,v3); an 8-value block (two words) comes out in the slot order [v0,v2 | v1,v3 | v4,v6 | v5,v7].
__host__ __device__ constexpr int value_in_slot8(int s) { return ((s >> 2) << 2) + ((s >> 1) & 1) + ((s & 1) << 1); }

__device__ __forceinline__ void unpack8_word(uint32_t w, h2 q[2], const UnpackConsts& k) {
  const h2 k1024 = {(_Float16)1024.f, (_Float16)1024.f};
  q[0] = as_h2(and_or(w, 0x00FF00FFu, k.c4_lo)) - k1024;       // v0, v2
  q[1] = as_h2(and_or(w >> 8, 0x00FF00FFu, k.c4_lo)) - k1024;  // v1, v3
}

// 32 consecutive 8-bit values = eight words
__device__ __forceinline__ void unpack8_chunk(const uint32_t w[8], h2 q[16], const UnpackConsts& k) {
#pragma unroll
  for (int i = 0; i < 8; i++) unpack8_word(w[i], q + 2 * i, k);
}

// Sum over all 64 lanes (LANES=64), or over each aligned group of LANES lanes,
// with DPP row operations. After the call the LAST lane of each group holds
// the group's sum.
template <int LANES>
__device__ __forceinline__ float group_sum_to_last_lane(float v) {
  static_assert(LANES == 16 || LANES == 32 || LANES == 64, "lane group");
  // within each row of 16 lanes
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
  if (LANES >= 32)  // rows 1 and 3 += lane 15 of the row before
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
  if (LANES == 64)  // rows 2 and 3 += lane 31
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
  return v;
}

}  // namespace ztvm
