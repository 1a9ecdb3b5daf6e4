// Load-time repacking of MLX safetensors records into the buffers the kernels
// bind: element conversion of one part of a concatenation plan straight into
// its place in the destination buffer, whole-row permutation, and the fused
// dequantize + split + transpose of the MLA kv_b projection
// (src/zero-tvm/mlx-weights.ts:100-135, :490-543, :558-667). The records are
// uploaded as they sit in the file; everything after that happens in HBM, so a
// checkpoint crosses PCIe once and is never touched by the host again.
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

// bf16 -> f16 bit pattern (mlx-weights.ts:100-127): exponent rebias by 112, f16
// subnormals rounded to nearest even, |x| past 65504 clamped to 0x7bff and reported,
// inf kept, nan made quiet, bf16 below 2^-25 flushed to signed zero.
__device__ __forceinline__ uint32_t bf16_to_f16_bits(uint32_t b, uint32_t& overflow) {
  const uint32_t sign = b & 0x8000u;
  const int raw = (int)((b >> 7) & 0xffu);
  const uint32_t mant0 = (b & 0x7fu) << 16;
  if (raw == 0xff) return sign | 0x7c00u | (mant0 ? 0x200u : 0u);
  const int exp = raw - 112;
  if (exp >= 0x1f) {
    overflow++;
    return sign | 0x7bffu;
  }
  if (exp <= 0) {
    if (exp < -10) return sign;
    const uint32_t mant = mant0 | 0x800000u;
    const int sh = 14 - exp;
    uint32_t h = mant >> sh;
    const uint32_t rem = mant & ((1u << sh) - 1u);
    const uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return sign | h;
  }
  return sign | ((uint32_t)exp << 10) | (mant0 >> 13);
}

// one wave adds its lanes' counts with a single vector atomic
__device__ __forceinline__ void report(uint32_t* counter, uint32_t n) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) n += __shfl_xor(n, m, 64);
  if (n && (threadIdx.x & 63u) == 0 && counter) atomicAdd(counter, n);
}

// 8 values per thread: 16 bytes in, 16 bytes out
__global__ __launch_bounds__(256) void bf16_f16_vec_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, size_t n16,
                                                           uint32_t* counter) {
  const size_t stride = (size_t)gridDim.x * 256u;
  uint32_t over = 0;
  for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += stride) {
    const u32x4 v = src[i];
    const uint32_t in[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
      o[j] = bf16_to_f16_bits(in[j] & 0xffffu, over) | (bf16_to_f16_bits(in[j] >> 16, over) << 16);
    dst[i] = u32x4{o[0], o[1], o[2], o[3]};
  }
  report(counter, over);
}

// any alignment, any count: one value per thread
__global__ __launch_bounds__(256) void bf16_f16_kernel(uint16_t* __restrict__ dst, const uint16_t* __restrict__ src, size_t n,
                                                       uint32_t* counter) {
  const size_t stride = (size_t)gridDim.x * 256u;
  uint32_t over = 0;
  for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n; i += stride) dst[i] = (uint16_t)bf16_to_f16_bits(src[i], over);
  report(counter, over);
}

// bf16 -> f32 is a shift (mlx-weights.ts:130-135)
__global__ __launch_bounds__(256) void bf16_f32_kernel(uint32_t* __restrict__ dst, const uint16_t* __restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256u;
  for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n; i += stride) dst[i] = (uint32_t)src[i] << 16;
}

__global__ __launch_bounds__(256) void copy1_kernel(unsigned char* __restrict__ dst, const unsigned char* __restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256u;
  for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// Destination row j takes source row map[j]; UNIT bytes per thread step (mlx-weights.ts:558-576).
// The map is validated on the host before it is uploaded.
template <typename T>
__global__ __launch_bounds__(256) void permute_rows_kernel(T* __restrict__ dst, const T* __restrict__ src,
                                                           const uint32_t* __restrict__ map, uint32_t rows, uint32_t units) {
  const uint64_t total = (uint64_t)rows * units;
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < total; i += stride) {
    const uint32_t j = (uint32_t)(i / units), u = (uint32_t)(i % units);
    dst[i] = src[(size_t)map[j] * units + u];
  }
}

// MLX-affine 4-bit group-64 [heads*(nope+v), k] -> f16 [heads][k][nope] then [heads][v][k]
// (mlx-weights.ts:598-667). One thread dequantizes one packed word (8 values) of one row:
// w = fl16(fl32(q*s + b)). For the K half the row index is the fastest-varying thread
// coordinate, so the eight strided stores of a wave each cover 64 consecutive f16 of the
// transposed matrix; for the V half the word index is fastest and a thread stores 16 bytes.
struct SplitParams {
  uint16_t* out;
  const uint32_t* w;
  const _Float16* s;
  const _Float16* b;
  uint32_t k, heads, nope, v, wpr, gpr;
  uint32_t* counter;
};

__device__ __forceinline__ void dequant_word(const SplitParams& p, size_t r, uint32_t word_idx, _Float16 out[8], uint32_t& over) {
  const uint32_t word = p.w[r * p.wpr + word_idx];
  const uint32_t g = word_idx >> 3;
  const float s = (float)p.s[r * p.gpr + g], b = (float)p.b[r * p.gpr + g];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    float val = __builtin_fmaf((float)((word >> (4 * j)) & 15u), s, b);
    if (__builtin_fabsf(val) > 65504.f) over++;
    out[j] = narrow_f32(val);  // two roundings, as the format defines
  }
}

__global__ __launch_bounds__(256) void split_k_kernel(const SplitParams p) {
  // thread -> (head, word, i) with i fastest
  const uint64_t total = (uint64_t)p.heads * p.wpr * p.nope;
  const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  uint32_t over = 0;
  if (idx < total) {
    const uint32_t i = (uint32_t)(idx % p.nope);
    const uint32_t word_idx = (uint32_t)((idx / p.nope) % p.wpr);
    const uint32_t h = (uint32_t)(idx / ((uint64_t)p.nope * p.wpr));
    _Float16 val[8];
    dequant_word(p, (size_t)h * (p.nope + p.v) + i, word_idx, val, over);
    uint16_t* o = p.out + (size_t)h * p.k * p.nope + (size_t)word_idx * 8u * p.nope + i;
#pragma unroll
    for (int j = 0; j < 8; j++) o[(size_t)j * p.nope] = __builtin_bit_cast(uint16_t, val[j]);
  }
  report(p.counter, over);
}

__global__ __launch_bounds__(256) void split_v_kernel(const SplitParams p) {
  // thread -> (head, i, word) with word fastest
  const uint64_t total = (uint64_t)p.heads * p.v * p.wpr;
  const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  uint32_t over = 0;
  if (idx < total) {
    const uint32_t word_idx = (uint32_t)(idx % p.wpr);
    const uint32_t i = (uint32_t)((idx / p.wpr) % p.v);
    const uint32_t h = (uint32_t)(idx / ((uint64_t)p.wpr * p.v));
    _Float16 val[8];
    dequant_word(p, (size_t)h * (p.nope + p.v) + p.nope + i, word_idx, val, over);
    h8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = val[j];
    uint16_t* o = p.out + (size_t)p.heads * p.k * p.nope + ((size_t)h * p.v + i) * p.k + (size_t)word_idx * 8u;
    *reinterpret_cast<h8*>(o) = r;
  }
  report(p.counter, over);
}

uint32_t blocks_for(uint64_t threads, uint32_t cap = 8192) {
  uint64_t b = (threads + 255) / 256;
  return (uint32_t)(b > cap ? cap : (b ? b : 1));
}

}  // namespace

hipError_t launch_repack_convert(void* dst, const void* src, size_t src_bytes, int convert, uint32_t* counter, hipStream_t s) {
  const uintptr_t d = reinterpret_cast<uintptr_t>(dst), a = reinterpret_cast<uintptr_t>(src);
  if (convert == 0) {  // raw bytes
    if (!((d | a | src_bytes) & 15u)) return launch_copy(dst, src, src_bytes, s);
    hipLaunchKernelGGL(copy1_kernel, dim3(blocks_for(src_bytes)), dim3(256), 0, s, reinterpret_cast<unsigned char*>(dst),
                       reinterpret_cast<const unsigned char*>(src), src_bytes);
  } else if (convert == 1) {  // bf16 -> f16
    if (!((d | a | src_bytes) & 15u))
      hipLaunchKernelGGL(bf16_f16_vec_kernel, dim3(blocks_for(src_bytes / 16)), dim3(256), 0, s, reinterpret_cast<u32x4*>(dst),
                         reinterpret_cast<const u32x4*>(src), src_bytes / 16, counter);
    else
      hipLaunchKernelGGL(bf16_f16_kernel, dim3(blocks_for(src_bytes / 2)), dim3(256), 0, s, reinterpret_cast<uint16_t*>(dst),
                         reinterpret_cast<const uint16_t*>(src), src_bytes / 2, counter);
  } else {  // bf16 -> f32
    hipLaunchKernelGGL(bf16_f32_kernel, dim3(blocks_for(src_bytes / 2)), dim3(256), 0, s, reinterpret_cast<uint32_t*>(dst),
                       reinterpret_cast<const uint16_t*>(src), src_bytes / 2);
  }
  return hipGetLastError();
}

hipError_t launch_permute_rows(void* dst, const void* src, const uint32_t* map, uint32_t rows, size_t row_bytes, hipStream_t s) {
  const uintptr_t d = reinterpret_cast<uintptr_t>(dst), a = reinterpret_cast<uintptr_t>(src);
  if (!((d | a | row_bytes) & 15u)) {
    const uint32_t units = (uint32_t)(row_bytes / 16);
    hipLaunchKernelGGL(permute_rows_kernel<u32x4>, dim3(blocks_for((uint64_t)rows * units)), dim3(256), 0, s,
                       reinterpret_cast<u32x4*>(dst), reinterpret_cast<const u32x4*>(src), map, rows, units);
  } else if (!((d | a | row_bytes) & 1u)) {
    const uint32_t units = (uint32_t)(row_bytes / 2);
    hipLaunchKernelGGL(permute_rows_kernel<uint16_t>, dim3(blocks_for((uint64_t)rows * units)), dim3(256), 0, s,
                       reinterpret_cast<uint16_t*>(dst), reinterpret_cast<const uint16_t*>(src), map, rows, units);
  } else {
    const uint32_t units = (uint32_t)row_bytes;
    hipLaunchKernelGGL(permute_rows_kernel<unsigned char>, dim3(blocks_for((uint64_t)rows * units)), dim3(256), 0, s,
                       reinterpret_cast<unsigned char*>(dst), reinterpret_cast<const unsigned char*>(src), map, rows, units);
  }
  return hipGetLastError();
}

hipError_t launch_dequant_split(void* out, const void* w, const void* scales, const void* biases, uint32_t k, uint32_t heads,
                                uint32_t nope, uint32_t v, uint32_t* counter, hipStream_t s) {
  SplitParams p{};
  p.out = reinterpret_cast<uint16_t*>(out);
  p.w = reinterpret_cast<const uint32_t*>(w);
  p.s = reinterpret_cast<const _Float16*>(scales);
  p.b = reinterpret_cast<const _Float16*>(biases);
  p.k = k; p.heads = heads; p.nope = nope; p.v = v; p.wpr = k / 8; p.gpr = k / 64;
  p.counter = counter;
  const uint64_t tk = (uint64_t)heads * p.wpr * nope, tv = (uint64_t)heads * v * p.wpr;
  if (tk) hipLaunchKernelGGL(split_k_kernel, dim3((uint32_t)((tk + 255) / 256)), dim3(256), 0, s, p);
  if (tv) hipLaunchKernelGGL(split_v_kernel, dim3((uint32_t)((tv + 255) / 256)), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace ztvm
