// The small dispatches either side of the quantized matmuls in a MoE / FFN
// block: the SiLU-gate epilogue, the router (logits + softmax top-k), the
// weighted sum over expert slots and the expert-id -> pool-slot translation.
// All of them are bandwidth- or latency-bound; they are written for 64-wide
// waves with 16-byte accesses and in-wave reductions (no LDS, no barriers).
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

// Wave-wide f32 reductions as a six-step scan over data-parallel-primitive moves (shifts within
// rows of 16 lanes, then the two row broadcasts); lane 63 ends up with the result, which is
// read back to every lane. The order of the additions is fixed, so results repeat exactly.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float v, float identity) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity), __builtin_bit_cast(int, v),
                                                               CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f32<0x111, 0xF>(v, 0.f);  // row_shr:1
  v += dpp_f32<0x112, 0xF>(v, 0.f);  // row_shr:2
  v += dpp_f32<0x114, 0xF>(v, 0.f);  // row_shr:4
  v += dpp_f32<0x118, 0xF>(v, 0.f);  // row_shr:8
  v += dpp_f32<0x142, 0xA>(v, 0.f);  // row_bcast:15
  v += dpp_f32<0x143, 0xC>(v, 0.f);  // row_bcast:31
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
  constexpr float LOW = -3.4e38f;
  v = fmaxf(v, dpp_f32<0x111, 0xF>(v, LOW));
  v = fmaxf(v, dpp_f32<0x112, 0xF>(v, LOW));
  v = fmaxf(v, dpp_f32<0x114, 0xF>(v, LOW));
  v = fmaxf(v, dpp_f32<0x118, 0xF>(v, LOW));
  v = fmaxf(v, dpp_f32<0x142, 0xA>(v, LOW));
  v = fmaxf(v, dpp_f32<0x143, 0xC>(v, LOW));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---------------------------------------------------------------- silu_mul ----
// out[t*F + i] = f16( up * (gate * (1 / (1 + exp(-gate)))) ), gate_up = [rows][2F],
// all in f32 (src/compiler/shaders/silu_mul.wgsl:27-44).
__device__ __forceinline__ float silu_gate(float g, float u) {
  const float sg = g * (1.0f / (1.0f + expf(-g)));
  return u * sg;
}

// VEC = 8: one 16-byte chunk of gate and of up per thread; VEC = 1: any F.
template <int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(_Float16* __restrict__ out, const _Float16* __restrict__ gu,
                                                       uint32_t rows, uint32_t ffn) {
  const uint32_t per_row = ffn / VEC;
  const uint64_t total = (uint64_t)rows * per_row;
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += stride) {
    const uint32_t t = (uint32_t)(idx / per_row), c = (uint32_t)(idx % per_row);
    const _Float16* g = gu + (size_t)t * 2 * ffn + (size_t)c * VEC;
    _Float16* o = out + (size_t)t * ffn + (size_t)c * VEC;
    if (VEC == 8) {
      const h8 gv = *reinterpret_cast<const h8*>(g);
      const h8 uv = *reinterpret_cast<const h8*>(g + ffn);
      h8 r;
#pragma unroll
      for (int j = 0; j < 8; j++) r[j] = narrow_f32(silu_gate((float)gv[j], (float)uv[j]));
      *reinterpret_cast<h8*>(o) = r;
    } else {
      o[0] = narrow_f32(silu_gate((float)g[0], (float)g[ffn]));
    }
  }
}

// ------------------------------------------------------------- moe_combine ----
// out[t,i] = f16( sum_s score[t*S+s] * slots[(t*S+s)*N + i] ), f32 accumulation in
// slot order, one fused multiply-add per slot (src/compiler/shaders/moe_combine.wgsl:33-44).
template <int VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(_Float16* __restrict__ out, const _Float16* __restrict__ slots,
                                                          const float* __restrict__ score, uint32_t N, uint32_t S) {
  const uint32_t t = blockIdx.y;
  const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * VEC;
  if (i >= N) return;
  const float* sc = score + (size_t)t * S;
  const _Float16* base = slots + (size_t)t * S * N + i;
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; j++) acc[j] = 0.f;
  for (uint32_t s = 0; s < S; s++) {
    const float w = sc[s];
    if (VEC == 8) {
      const h8 v = *reinterpret_cast<const h8*>(base + (size_t)s * N);
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] = __builtin_fmaf(w, (float)v[j], acc[j]);
    } else {
      acc[0] = __builtin_fmaf(w, (float)base[(size_t)s * N], acc[0]);
    }
  }
  _Float16* o = out + (size_t)t * N + i;
  if (VEC == 8) {
    h8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = narrow_f32(acc[j]);
    *reinterpret_cast<h8*>(o) = r;
  } else {
    o[0] = narrow_f32(acc[0]);
  }
}

// ----------------------------------------------------------- router logits ----
// logit[t,e] = sum_g ( s[e,g] * sum_i x[t,i]*q[e,i] + b[e,g] * sum_i x[t,i] ), groups of 64,
// q unsigned 8-bit (4 per word) or 4-bit (8 per word), LSB first; BITS == 16: plain
// f16 rows (src/compiler/shaders/moe_router_logits.wgsl:45-140, moe_router_logits_f16.wgsl:33-57).
//
// One wave per router row and per block of TT tokens: a lane reads 16 bytes of the row
// once and uses them for every token of its block, so the row crosses L2 once per TT
// tokens instead of once per token. Small dispatches take TT = 1 (more waves, the work
// is latency-bound), chunked prefill TT = 8. Partial sums are f32; the 64 lanes are summed with
// a butterfly, so every lane (and every launch) sees the same order.
template <int BITS, int ROUTER_TT>
__global__ __launch_bounds__(256) void router_logits_kernel(float* __restrict__ logits, const _Float16* __restrict__ x,
                                                            const void* __restrict__ w, const _Float16* __restrict__ scales,
                                                            const _Float16* __restrict__ biases, uint32_t D, uint32_t rows,
                                                            uint32_t tokens) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t e = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (e >= rows) return;  // whole waves leave together; nothing below synchronises across waves
  const uint32_t t0 = blockIdx.y * ROUTER_TT;
  const uint32_t nt = tokens - t0 < ROUTER_TT ? tokens - t0 : ROUTER_TT;
  constexpr uint32_t VALS = BITS == 16 ? 8u : 128u / BITS;  // values per 16-byte chunk: 8 | 16 | 32
  const uint32_t chunks = D / VALS;
  const uint32_t gpr = D / 64u;
  float acc[ROUTER_TT];
#pragma unroll
  for (int t = 0; t < ROUTER_TT; t++) acc[t] = 0.f;

  for (uint32_t c = lane; c < chunks; c += 64u) {
    float q[VALS];
    float s = 1.f, b = 0.f;
    if constexpr (BITS == 16) {
      const h8 v = *reinterpret_cast<const h8*>(reinterpret_cast<const _Float16*>(w) + (size_t)e * D + (size_t)c * 8u);
#pragma unroll
      for (int j = 0; j < 8; j++) q[j] = (float)v[j];
    } else {
      constexpr uint32_t PER = 32u / BITS;
      const u32x4 v = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint32_t*>(w) + ((size_t)e * chunks + c) * 4u);
      const uint32_t word[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (uint32_t j = 0; j < VALS; j++) q[j] = (float)((word[j / PER] >> (BITS * (j % PER))) & ((1u << BITS) - 1u));
      const uint32_t g = c * VALS / 64u;
      s = (float)scales[(size_t)e * gpr + g];
      b = (float)biases[(size_t)e * gpr + g];
    }
#pragma unroll
    for (int t = 0; t < ROUTER_TT; t++) {
      if ((uint32_t)t < nt) {
        const _Float16* xp = x + (size_t)(t0 + t) * D + (size_t)c * VALS;
        float dot = 0.f, xs = 0.f;
#pragma unroll
        for (uint32_t j = 0; j < VALS; j += 8) {
          const h8 xv = *reinterpret_cast<const h8*>(xp + j);
#pragma unroll
          for (int k = 0; k < 8; k++) {
            dot = __builtin_fmaf((float)xv[k], q[j + k], dot);
            xs += (float)xv[k];
          }
        }
        acc[t] = BITS == 16 ? acc[t] + dot : __builtin_fmaf(s, dot, __builtin_fmaf(b, xs, acc[t]));
      }
    }
  }
#pragma unroll
  for (int t = 0; t < ROUTER_TT; t++) {
    if ((uint32_t)t < nt) {
      const float r = wave_sum(acc[t]);
      if (lane == 0) logits[(size_t)(t0 + t) * rows + e] = r;
    }
  }
}

// ------------------------------------------------------------ router top-k ----
// Softmax over all E routed experts, then the K largest in descending order (ties to
// the lower index), renormalised over the survivors when norm_topk; the shared expert,
// when present, is slot K with index E and sigmoid(logit[E])
// (src/compiler/shaders/moe_router_topk.wgsl:67-136). One wave per token; lane l
// holds experts l, l+64, ... (coalesced reads); nothing leaves registers.
//
// The K arg-max rounds are a serial chain, so each round is kept short: two six-step scans over
// data-parallel-primitive moves on 32-bit values (the largest probability, then the lowest index
// holding it) instead of cross-lane LDS permutes or 64-bit keys, and only as many registers per
// lane as the expert count needs.
constexpr int TOPK_PER = 8;  // 64 lanes x 8 = 512 experts at most

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v, uint32_t identity) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)identity, (int)v, CTRL, ROW_MASK, 0xF, false);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, dpp_u32<0x111, 0xF>(v, 0u));
  v = max(v, dpp_u32<0x112, 0xF>(v, 0u));
  v = max(v, dpp_u32<0x114, 0xF>(v, 0u));
  v = max(v, dpp_u32<0x118, 0xF>(v, 0u));
  v = max(v, dpp_u32<0x142, 0xA>(v, 0u));
  v = max(v, dpp_u32<0x143, 0xC>(v, 0u));
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  v = min(v, dpp_u32<0x111, 0xF>(v, ~0u));
  v = min(v, dpp_u32<0x112, 0xF>(v, ~0u));
  v = min(v, dpp_u32<0x114, 0xF>(v, ~0u));
  v = min(v, dpp_u32<0x118, 0xF>(v, ~0u));
  v = min(v, dpp_u32<0x142, 0xA>(v, ~0u));
  v = min(v, dpp_u32<0x143, 0xC>(v, ~0u));
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// PER = experts per lane (E <= 64 * PER). A candidate is the bit pattern of its probability plus one
// (probabilities are non-negative floats, so their bit patterns order like the values; zero marks
// "none" and "already taken", and an underflowed probability of exactly 0 is still a candidate). Each
// of the K rounds takes the wave's largest candidate, then the lowest expert index holding it.
template <int PER>
__global__ __launch_bounds__(256) void router_topk_kernel(uint32_t* __restrict__ out_idx, float* __restrict__ out_score,
                                                          const float* __restrict__ logits, uint32_t E, uint32_t K,
                                                          uint32_t norm_topk, uint32_t has_shared, uint32_t tokens) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t tok = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (tok >= tokens) return;  // whole waves leave together
  const float* l = logits + (size_t)tok * (E + has_shared);
  const size_t obase = (size_t)tok * (K + has_shared);

  float pv[PER];
  float m = -3.0e38f;
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t e = lane + 64u * i;
    pv[i] = e < E ? l[e] : -3.0e38f;
    m = fmaxf(m, pv[i]);
  }
  const float shared_logit = has_shared ? l[E] : 0.f;
  const float peak = wave_max(m);
  float s = 0.f;
  uint32_t cand[PER];
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t e = lane + 64u * i;
    const float p = e < E ? expf(pv[i] - peak) : 0.f;
    s += p;
    cand[i] = e < E ? __builtin_bit_cast(uint32_t, p) + 1u : 0u;
  }
  const float denom = wave_sum(s);

  float total = 0.f, mine = 0.f;
  uint32_t mine_idx = 0;
  for (uint32_t k = 0; k < K; k++) {
    uint32_t best = cand[0];
#pragma unroll
    for (int i = 1; i < PER; i++) best = max(best, cand[i]);
    best = wave_max_u32(best);
    uint32_t holder = ~0u;  // this lane's lowest expert index holding `best`
#pragma unroll
    for (int i = PER - 1; i >= 0; i--) holder = cand[i] == best ? lane + 64u * i : holder;
    const uint32_t win = wave_min_u32(holder);
    const float bv = __builtin_bit_cast(float, best - 1u);
    total += bv;
    if (lane == k) {
      mine = bv;
      mine_idx = win;
    }
#pragma unroll
    for (int i = 0; i < PER; i++)
      if (lane + 64u * i == win) cand[i] = 0u;
  }
  const float scale = norm_topk ? 1.0f / total : 1.0f / denom;
  if (lane < K) {
    out_idx[obase + lane] = mine_idx;
    out_score[obase + lane] = mine * scale;
  }
  if (has_shared && lane == 0) {
    out_idx[obase + K] = E;
    out_score[obase + K] = 1.0f / (1.0f + expf(-shared_logit));
  }
}

// ---------------------------------------------------------- slot translate ----
// ids_out[i] = slot_map[ids_in[i]], a miss (0xffffffff) or an id past the map -> slot 0
// (src/compiler/shaders/moe_slot_translate.wgsl:32-36).
__global__ __launch_bounds__(64) void slot_translate_kernel(uint32_t* __restrict__ ids_out, const uint32_t* __restrict__ ids_in,
                                                            const uint32_t* __restrict__ slot_map, uint32_t n, uint32_t map_len) {
  const uint32_t i = blockIdx.x * 64u + threadIdx.x;
  if (i >= n) return;
  const uint32_t e = ids_in[i];
  const uint32_t s = e < map_len ? slot_map[e] : 0xffffffffu;
  ids_out[i] = s == 0xffffffffu ? 0u : s;
}

// ---------------------------------------------------------------- kv_quantize_int8 ----
// One wave per (token, kv head, side): max |x| over the head's row, scale = max / 127 (at least
// 1e-8), q = clamp(round-half-even(x / scale)) packed four to a word, and the f16 scale
// (src/compiler/shaders/kv_quantize_int8.wgsl:47-164). Page layout, in words:
// page . head . slot . side(K|V) . dim/4; scales: page . head . slot . side.
struct KvqParams {
  uint32_t kv_heads, head_dim, page_size, tokens, pos_off, pages_word_off, scales_off;
  uint64_t pages_capacity_words, scales_capacity;
};
constexpr int KVQ_TURNS = 4;  // words of a row per lane: head_dim <= 4 * 64 * KVQ_TURNS

__global__ __launch_bounds__(256) void kv_quantize_int8_kernel(uint32_t* __restrict__ pages, _Float16* __restrict__ scales,
                                                               const _Float16* __restrict__ k_slot, const _Float16* __restrict__ v_slot,
                                                               const int32_t* __restrict__ position_map, const KvqParams p) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t unit = blockIdx.x * 4u + (threadIdx.x >> 6);  // uniform per wave
  if (unit >= p.tokens * p.kv_heads * 2u) return;
  const uint32_t tok = unit / (p.kv_heads * 2u), rest = unit - tok * p.kv_heads * 2u;
  const uint32_t head = rest >> 1, side = rest & 1u;
  const uint32_t row_words = p.head_dim / 4u;
  const _Float16* src = (side ? v_slot : k_slot) + (size_t)tok * p.kv_heads * p.head_dim + (size_t)head * p.head_dim;
  float v[KVQ_TURNS][4];
  float m = 0.f;
#pragma unroll
  for (int t = 0; t < KVQ_TURNS; t++) {
    const uint32_t w = lane + t * 64u;
#pragma unroll
    for (int i = 0; i < 4; i++) v[t][i] = 0.f;
    if (w < row_words) {
      const h4 x = *reinterpret_cast<const h4*>(src + 4u * w);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        v[t][i] = (float)x[i];
        m = fmaxf(m, fabsf(v[t][i]));
      }
    }
  }
  m = wave_max(m);
  float scale = m / 127.0f;
  if (scale < 1e-8f) scale = 1e-8f;
  const float inv_scale = 1.0f / scale;
  const int32_t position = position_map[p.pos_off + tok];
  if (position < 0) return;  // uniform per wave
  const uint32_t page_no = (uint32_t)position / p.page_size, slot = (uint32_t)position - page_no * p.page_size;
  const uint64_t scale_idx = (uint64_t)page_no * p.kv_heads * p.page_size * 2u + (uint64_t)head * p.page_size * 2u + slot * 2u + side + p.scales_off;
  if (lane == 0 && (!p.scales_capacity || scale_idx < p.scales_capacity)) scales[scale_idx] = (_Float16)scale;
  const uint64_t base = (uint64_t)page_no * p.kv_heads * p.page_size * 2u * row_words + (uint64_t)head * p.page_size * 2u * row_words +
                        (uint64_t)slot * 2u * row_words + (uint64_t)side * row_words + p.pages_word_off;
#pragma unroll
  for (int t = 0; t < KVQ_TURNS; t++) {
    const uint32_t w = lane + t * 64u;
    if (w < row_words && (!p.pages_capacity_words || base + w < p.pages_capacity_words)) {
      uint32_t packed = 0;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float q = __builtin_rintf(v[t][i] * inv_scale);
        q = fminf(fmaxf(q, -127.f), 127.f);
        packed |= ((uint32_t)(int32_t)q & 0xffu) << (8 * i);
      }
      pages[base + w] = packed;
    }
  }
}

uint32_t grid_for(uint64_t threads) {
  uint64_t blocks = (threads + 255) / 256;
  return (uint32_t)(blocks > 16384 ? 16384 : (blocks ? blocks : 1));
}

}  // namespace

hipError_t launch_silu_mul(void* out, const void* gate_up, uint32_t rows, uint32_t ffn, hipStream_t s) {
  const bool vec = ffn % 8 == 0 && !((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(gate_up)) & 15u);
  _Float16* o = reinterpret_cast<_Float16*>(out);
  const _Float16* g = reinterpret_cast<const _Float16*>(gate_up);
  if (vec) hipLaunchKernelGGL(silu_mul_kernel<8>, dim3(grid_for((uint64_t)rows * (ffn / 8))), dim3(256), 0, s, o, g, rows, ffn);
  else hipLaunchKernelGGL(silu_mul_kernel<1>, dim3(grid_for((uint64_t)rows * ffn)), dim3(256), 0, s, o, g, rows, ffn);
  return hipGetLastError();
}

hipError_t launch_moe_combine(void* out, const void* slots, const void* score, uint32_t tokens, uint32_t N, uint32_t S,
                              hipStream_t s) {
  const bool vec = N % 8 == 0 && !((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(slots)) & 15u);
  _Float16* o = reinterpret_cast<_Float16*>(out);
  const _Float16* sl = reinterpret_cast<const _Float16*>(slots);
  const float* sc = reinterpret_cast<const float*>(score);
  if (vec) hipLaunchKernelGGL(moe_combine_kernel<8>, dim3((N / 8 + 255) / 256, tokens), dim3(256), 0, s, o, sl, sc, N, S);
  else hipLaunchKernelGGL(moe_combine_kernel<1>, dim3((N + 255) / 256, tokens), dim3(256), 0, s, o, sl, sc, N, S);
  return hipGetLastError();
}

template <int TT>
void launch_router_tt(float* lg, const _Float16* xx, const void* w, const _Float16* sc, const _Float16* bi, uint32_t bits,
                      uint32_t D, uint32_t rows, uint32_t tokens, hipStream_t s) {
  const dim3 grid((rows + 3) / 4, (tokens + TT - 1) / TT);
  if (bits == 8) hipLaunchKernelGGL((router_logits_kernel<8, TT>), grid, dim3(256), 0, s, lg, xx, w, sc, bi, D, rows, tokens);
  else if (bits == 4) hipLaunchKernelGGL((router_logits_kernel<4, TT>), grid, dim3(256), 0, s, lg, xx, w, sc, bi, D, rows, tokens);
  else hipLaunchKernelGGL((router_logits_kernel<16, TT>), grid, dim3(256), 0, s, lg, xx, w, sc, bi, D, rows, tokens);
}

hipError_t launch_router_logits(void* logits, const void* x, const void* w, const void* scales, const void* biases,
                                uint32_t bits, uint32_t D, uint32_t rows, uint32_t tokens, hipStream_t s) {
  float* lg = reinterpret_cast<float*>(logits);
  const _Float16* xx = reinterpret_cast<const _Float16*>(x);
  const _Float16* sc = reinterpret_cast<const _Float16*>(scales);
  const _Float16* bi = reinterpret_cast<const _Float16*>(biases);
  // enough waves to cover the chip first, weight reuse second
  const uint64_t waves1 = (uint64_t)rows * tokens;
  if (waves1 >= 8u * 4096u) launch_router_tt<8>(lg, xx, w, sc, bi, bits, D, rows, tokens, s);
  else if (waves1 >= 2u * 4096u) launch_router_tt<2>(lg, xx, w, sc, bi, bits, D, rows, tokens, s);
  else launch_router_tt<1>(lg, xx, w, sc, bi, bits, D, rows, tokens, s);
  return hipGetLastError();
}

uint32_t router_topk_max_experts() { return 64u * TOPK_PER; }

hipError_t launch_router_topk(void* out_idx, void* out_score, const void* logits, uint32_t E, uint32_t K, uint32_t norm_topk,
                              uint32_t has_shared, uint32_t tokens, hipStream_t s) {
  auto go = [&](auto k) {
    hipLaunchKernelGGL(k, dim3((tokens + 3) / 4), dim3(256), 0, s, reinterpret_cast<uint32_t*>(out_idx),
                       reinterpret_cast<float*>(out_score), reinterpret_cast<const float*>(logits), E, K, norm_topk, has_shared, tokens);
  };
  if (E <= 64) go(router_topk_kernel<1>);
  else if (E <= 128) go(router_topk_kernel<2>);
  else if (E <= 256) go(router_topk_kernel<4>);
  else go(router_topk_kernel<TOPK_PER>);
  return hipGetLastError();
}

hipError_t launch_kv_quantize_int8(void* pages_i8, void* scales, const void* k_slot, const void* v_slot, const int32_t* position_map,
                                   uint32_t kv_heads, uint32_t head_dim, uint32_t page_size, uint32_t tokens, uint32_t pos_off,
                                   uint32_t pages_word_off, uint32_t scales_off, uint64_t pages_capacity_words, uint64_t scales_capacity,
                                   hipStream_t s) {
  if (head_dim > 4u * 64u * KVQ_TURNS) return hipErrorInvalidValue;  // rejected by the entry point
  const KvqParams p{kv_heads, head_dim, page_size, tokens, pos_off, pages_word_off, scales_off, pages_capacity_words, scales_capacity};
  const uint32_t units = tokens * kv_heads * 2u;
  hipLaunchKernelGGL(kv_quantize_int8_kernel, dim3((units + 3) / 4), dim3(256), 0, s, reinterpret_cast<uint32_t*>(pages_i8),
                     reinterpret_cast<_Float16*>(scales), reinterpret_cast<const _Float16*>(k_slot), reinterpret_cast<const _Float16*>(v_slot),
                     position_map, p);
  return hipGetLastError();
}

hipError_t launch_slot_translate(void* ids_out, const void* ids_in, const void* slot_map, uint32_t n, uint32_t map_len,
                                 hipStream_t s) {
  hipLaunchKernelGGL(slot_translate_kernel, dim3((n + 63) / 64), dim3(64), 0, s, reinterpret_cast<uint32_t*>(ids_out),
                     reinterpret_cast<const uint32_t*>(ids_in), reinterpret_cast<const uint32_t*>(slot_map), n, map_len);
  return hipGetLastError();
}

}  // namespace ztvm
