/*
 * CPU oracle, second part: the loader-side conversions of MLX checkpoints and
 * the small dispatches either side of the quantized matmuls in a MoE block.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only the test-suite, the
 * smoke check and the bench's cpu_baseline leg may link or call it; the
 * shipped library (libztvm_hip.so) never does and has no CPU fallback.
 *
 * Every function restates arithmetic of the reference (abgnydn/zero-tvm);
 * citations are paths relative to the reference's root.
 *
 * Parity pins (tests/test_oracle_block_pins.py):
 *   zo_bf16_to_f16          all 65536 bit patterns against numpy's
 *                           float32 -> float16 cast (equal wherever the value
 *                           fits f16; clamp + count where it does not; quiet
 *                           NaN), and the reference test's own value list
 *                           (tests/kernels/mlx-repack.mjs:87-136: one overflow,
 *                           subnormals kept, 1e-40 flushed)
 *   zo_bf16_to_f32          all 65536 patterns against a numpy shift
 *   zo_permute_rows         numpy fancy indexing; the de-interleave map and
 *                           its inverse differ
 *   zo_dequant_affine_split the already pinned zo_dequant_matrix + numpy
 *                           reshape/transposes
 *   zo_silu_mul             scipy.special.expit in float64
 *   zo_moe_combine          numpy einsum in float64; one-hot scores
 *   zo_router_logits        numpy float64 on independently unpacked bytes /
 *                           nibbles; a width mix-up is off by O(1)
 *   zo_router_topk          scipy softmax + stable argsort; ties, K == E,
 *                           shared slot == expit(logit[E])
 *   zo_slot_translate       numpy take + where
 *   zo_qkv_fused            the pinned dequant + a numpy matmul, the rotation as a complex
 *                           multiplication by exp(i*freq), the cache as a reshaped
 *                           [page][K|V][kv_head][slot][dim] array; swapping the pair or the
 *                           sign of the sine, or writing V rotated, fails it
 *   zo_kv_quantize_int8     numpy float32 formulation (np.rint, true division); the bound
 *                           |q*scale - x| <= scale/2 + |x|*2^-11 on every element; an all-zero
 *                           row; the reference test's own float64 reference within its +-1 count
 *                           (tests/kernels/compile-qwen.mjs:720-747)
 *   zo_add_rmsnorm          numpy formulation (float64 sum of squares rounded once, float32 after:
 *                           equal bit for bit); a constant row (closed form
 *                           c / sqrt(c^2 + eps) * gamma); zero input; gamma = 1 gives unit RMS
 * The reference's byte-exact repack fixtures (.weights-local/kernel-refs) are
 * git-ignored and absent, so fidelity of the plans to a real MLX checkpoint is
 * "parity unpinned"; what is pinned is each conversion against numpy.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ZO_API __attribute__((visibility("default")))

uint16_t zo_f32_to_f16(float val);
float zo_f16_to_f32(uint16_t h);

/* ------------------------------------------------------- bf16 at load -- */

/* bf16 -> f16 with overflow counting (src/zero-tvm/mlx-weights.ts:100-127):
 * exponent rebias by 112, subnormals rounded to nearest even, values past
 * 65504 clamped to 0x7bff and counted, inf/nan kept (nan made quiet), bf16
 * below 2^-25 flushed to signed zero. Returns the overflow count. */
ZO_API uint64_t zo_bf16_to_f16(const uint16_t* src, uint16_t* out, size_t n) {
  uint64_t overflow = 0;
  for (size_t i = 0; i < n; i++) {
    uint32_t b = src[i];
    uint32_t sign = b & 0x8000u;
    int32_t raw = (int32_t)((b >> 7) & 0xffu);
    uint32_t mant0 = (b & 0x7fu) << 16;
    if (raw == 0xff) { out[i] = (uint16_t)(sign | 0x7c00u | (mant0 ? 0x200u : 0u)); continue; }
    int32_t exp = raw - 112;
    if (exp >= 0x1f) { out[i] = (uint16_t)(sign | 0x7bffu); overflow++; continue; }
    if (exp <= 0) {
      if (exp < -10) { out[i] = (uint16_t)sign; continue; }
      uint32_t mant = mant0 | 0x800000u;
      int sh = 14 - exp;
      uint32_t h = mant >> sh;
      uint32_t rem = mant & ((1u << sh) - 1u);
      uint32_t half = 1u << (sh - 1);
      if (rem > half || (rem == half && (h & 1u))) h++;
      out[i] = (uint16_t)(sign | h);
      continue;
    }
    out[i] = (uint16_t)(sign | ((uint32_t)exp << 10) | (mant0 >> 13));
  }
  return overflow;
}

/* bf16 -> f32 bits: a shift (src/zero-tvm/mlx-weights.ts:130-135). */
ZO_API void zo_bf16_to_f32(const uint16_t* src, uint32_t* out, size_t n) {
  for (size_t i = 0; i < n; i++) out[i] = (uint32_t)src[i] << 16;
}

/* Whole-row permutation: destination row j takes source row src[j]
 * (src/zero-tvm/mlx-weights.ts:558-576). Returns 0, or -1 when the map length,
 * the divisibility or an index is wrong (the reference throws). */
ZO_API int zo_permute_rows(const uint8_t* data, uint8_t* out, size_t bytes, uint32_t rows, const uint32_t* src,
                           uint32_t src_len) {
  if (src_len != rows || rows == 0 || bytes % rows) return -1;
  size_t rb = bytes / rows;
  for (uint32_t j = 0; j < rows; j++) {
    if (src[j] >= rows) return -1;
    memcpy(out + (size_t)j * rb, data + (size_t)src[j] * rb, rb);
  }
  return 0;
}

/* The de-interleave map of the rotary rows, row j takes original row deint(j):
 * even indices first, then the odd ones (src/zero-tvm/mlx-weights.ts:310). */
ZO_API uint32_t zo_deint(uint32_t j, uint32_t R) { return j < R / 2 ? 2 * j : 2 * (j - R / 2) + 1; }

/* MLX-affine 4-bit group-64 [heads*(nope+v), k] -> f16 [heads][k][nope] (K
 * transposed) followed by [heads][v][k] (src/zero-tvm/mlx-weights.ts:598-667).
 * value = fl16(fl32(q*s + b)); returns how many |values| exceed 65504. */
ZO_API uint64_t zo_dequant_affine_split(const uint32_t* w, const uint16_t* s, const uint16_t* b, uint32_t k,
                                        uint32_t heads, uint32_t nope, uint32_t v, uint16_t* out) {
  const uint32_t wpr = k / 8, gpr = k / 64;
  const size_t kblock = (size_t)heads * k * nope;
  uint64_t overflow = 0;
  float* row = (float*)malloc(sizeof(float) * k);
  for (uint32_t h = 0; h < heads; h++) {
    for (uint32_t i = 0; i < nope + v; i++) {
      size_t r = (size_t)h * (nope + v) + i;
      for (uint32_t g = 0; g < gpr; g++) {
        double sc = (double)zo_f16_to_f32(s[r * gpr + g]);
        double bi = (double)zo_f16_to_f32(b[r * gpr + g]);
        for (uint32_t c = g * 64; c < (g + 1) * 64; c++) {
          uint32_t word = w[r * wpr + (c >> 3)];
          /* a JS number expression stored into a Float32Array: one rounding from f64 */
          row[c] = (float)((double)((word >> ((c & 7u) * 4u)) & 15u) * sc + bi);
        }
      }
      if (i < nope) {
        size_t base = (size_t)h * k * nope + i;
        for (uint32_t c = 0; c < k; c++) {
          if (fabsf(row[c]) > 65504.f) overflow++;
          out[base + (size_t)c * nope] = zo_f32_to_f16(row[c]);
        }
      } else {
        size_t base = kblock + (size_t)h * v * k + (size_t)(i - nope) * k;
        for (uint32_t c = 0; c < k; c++) {
          if (fabsf(row[c]) > 65504.f) overflow++;
          out[base + c] = zo_f32_to_f16(row[c]);
        }
      }
    }
  }
  free(row);
  return overflow;
}

/* ------------------------------------------------------------ silu_mul -- */

/* out[t*F+i] = up * silu(gate) over gate_up [rows][2F]
 * (src/compiler/shaders/silu_mul.wgsl:27-44).
 *   out64: the reference test's own float64 form, unrounded
 *          (tests/kernels/compile-qwen35.mjs:1588-1592: up * (g / (1 + exp(-g))))
 *   out16: the shader's float32 form, gate * (1/(1+exp(-gate))) then * up, stored as f16 */
ZO_API void zo_silu_mul(const uint16_t* gu, uint32_t rows, uint32_t ffn, double* out64, uint16_t* out16) {
  for (uint32_t t = 0; t < rows; t++)
    for (uint32_t i = 0; i < ffn; i++) {
      float g = zo_f16_to_f32(gu[(size_t)t * 2 * ffn + i]);
      float u = zo_f16_to_f32(gu[(size_t)t * 2 * ffn + ffn + i]);
      if (out64) out64[(size_t)t * ffn + i] = (double)u * ((double)g / (1.0 + exp(-(double)g)));
      if (out16) {
        float sg = g * (1.0f / (1.0f + expf(-g)));
        out16[(size_t)t * ffn + i] = zo_f32_to_f16(u * sg);
      }
    }
}

/* ---------------------------------------------------------- moe_combine -- */

/* out[t,i] = sum_s score[t*S+s] * slots[(t*S+s)*N+i], slot order, f32
 * accumulate (src/compiler/shaders/moe_combine.wgsl:33-44).
 *   out64: float64 sum, unrounded
 *   out16: float32 accumulation in slot order with a fused multiply-add per slot, stored as f16 */
ZO_API void zo_moe_combine(const uint16_t* slots, const float* score, uint32_t tokens, uint32_t N, uint32_t S,
                           double* out64, uint16_t* out16) {
  for (uint32_t t = 0; t < tokens; t++)
    for (uint32_t i = 0; i < N; i++) {
      double a64 = 0.0;
      float a32 = 0.f;
      for (uint32_t s = 0; s < S; s++) {
        float v = zo_f16_to_f32(slots[((size_t)t * S + s) * N + i]);
        float sc = score[(size_t)t * S + s];
        a64 += (double)sc * (double)v;
        a32 = fmaf(sc, v, a32);
      }
      if (out64) out64[(size_t)t * N + i] = a64;
      if (out16) out16[(size_t)t * N + i] = zo_f32_to_f16(a32);
    }
}

/* -------------------------------------------------------- router logits -- */

/* logit[t,e] of the MoE router (src/compiler/shaders/moe_router_logits.wgsl:45-87
 * for 8 bits, :101-140 for 4 bits, moe_router_logits_f16.wgsl:33-57 for f16 rows).
 * The float64 form follows the reference test's formula
 * (tests/kernels/run.mjs:218-237):
 *   logit[e] = sum_g ( s[e,g] * sum_i x[i]*q[e,i] + b[e,g] * sum_i x[i] ), groups of 64;
 *   bits == 16: plain dot product of f16 rows.
 * w is u32 words (8/4 bits, LSB first) or f16 bit patterns (16). */
ZO_API void zo_router_logits(uint32_t bits, uint32_t D, uint32_t rows, uint32_t tokens, const uint16_t* x,
                             const void* w, const uint16_t* scales, const uint16_t* biases, double* logits) {
  for (uint32_t t = 0; t < tokens; t++)
    for (uint32_t e = 0; e < rows; e++) {
      double acc = 0.0;
      if (bits == 16) {
        const uint16_t* w16 = (const uint16_t*)w;
        for (uint32_t i = 0; i < D; i++)
          acc += (double)zo_f16_to_f32(x[(size_t)t * D + i]) * (double)zo_f16_to_f32(w16[(size_t)e * D + i]);
      } else {
        const uint32_t* ww = (const uint32_t*)w;
        const uint32_t per = 32 / bits, mask = (1u << bits) - 1u, gpr = D / 64;
        for (uint32_t g = 0; g < gpr; g++) {
          double dot = 0.0, xs = 0.0;
          for (uint32_t j = 0; j < 64; j++) {
            uint32_t i = g * 64 + j;
            uint32_t word = ww[((size_t)e * D + i) / per];
            uint32_t q = (word >> (bits * (i % per))) & mask;
            double xv = (double)zo_f16_to_f32(x[(size_t)t * D + i]);
            dot += xv * (double)q;
            xs += xv;
          }
          acc += (double)zo_f16_to_f32(scales[(size_t)e * gpr + g]) * dot +
                 (double)zo_f16_to_f32(biases[(size_t)e * gpr + g]) * xs;
        }
      }
      logits[(size_t)t * rows + e] = acc;
    }
}

/* ---------------------------------------------------------- router top-k -- */

/* Softmax over the E routed experts, then the K largest in descending order,
 * ties to the lower index, renormalised over the survivors when norm_topk, and
 * the shared expert (index E, sigmoid of logit E) as slot K when has_shared
 * (src/compiler/shaders/moe_router_topk.wgsl:67-136; float64 reference
 * tests/kernels/run.mjs:290-306). Strides: E+has_shared logits and
 * K+has_shared slots per token. Slots past the block are not written. */
ZO_API void zo_router_topk(const float* logits, uint32_t tokens, uint32_t E, uint32_t K, int norm_topk, int has_shared,
                           uint32_t* out_idx, double* out_score) {
  double* p = (double*)malloc(sizeof(double) * E);
  for (uint32_t t = 0; t < tokens; t++) {
    const float* l = logits + (size_t)t * (E + (has_shared ? 1 : 0));
    uint32_t* oi = out_idx + (size_t)t * (K + (has_shared ? 1 : 0));
    double* os = out_score + (size_t)t * (K + (has_shared ? 1 : 0));
    double peak = -INFINITY, denom = 0.0, total = 0.0;
    for (uint32_t e = 0; e < E; e++) if ((double)l[e] > peak) peak = (double)l[e];
    for (uint32_t e = 0; e < E; e++) { p[e] = exp((double)l[e] - peak); denom += p[e]; }
    for (uint32_t k = 0; k < K; k++) {
      double bv = -1.0;
      uint32_t bi = 0;
      for (uint32_t e = 0; e < E; e++) if (p[e] > bv) { bv = p[e]; bi = e; }
      oi[k] = bi;
      os[k] = bv;
      total += bv;
      p[bi] = -1.0;
    }
    double scale = norm_topk ? 1.0 / total : 1.0 / denom;
    for (uint32_t k = 0; k < K; k++) os[k] *= scale;
    if (has_shared) {
      oi[K] = E;
      os[K] = 1.0 / (1.0 + exp(-(double)l[E]));
    }
  }
  free(p);
}

/* Expert id -> pool slot through a resident map; a miss (0xffffffff) becomes
 * slot 0 (src/compiler/shaders/moe_slot_translate.wgsl:32-36). */
ZO_API void zo_slot_translate(const uint32_t* ids_in, const uint32_t* slot_map, uint32_t n, uint32_t* ids_out) {
  for (uint32_t i = 0; i < n; i++) {
    uint32_t s = slot_map[ids_in[i]];
    ids_out[i] = s == 0xffffffffu ? 0u : s;
  }
}

/* ------------------------------------------------------------ qkv_fused -- */

/* QKV matmul + RoPE + paged KV append for one token (src/compiler/shaders/qkv_fused.wgsl:41-193),
 * following the reference test's float64 form (tests/kernels/run.mjs:797-806, :836-860):
 * row dot products in float64 over per-element (q-7)*s (or q*s+b), freq = pos / theta^(2*dim/head_dim),
 * rot_lo = c*lo - s*hi, rot_hi = c*hi + s*lo, everything rounded to f16 only at the store.
 * q_out [heads*head_dim] and pages (already holding the cache's previous contents) are f16 bit patterns. */
ZO_API void zo_qkv_fused(uint32_t affine, uint32_t K, uint32_t heads, uint32_t kv_heads, uint32_t head_dim,
                         uint32_t page_size, uint32_t kv_page_stride, uint32_t head_page_stride, uint32_t v_page_offset,
                         uint32_t pages_elem_offset, double theta, int32_t position, const uint16_t* hidden,
                         const uint32_t* weights, const uint16_t* scales, const uint16_t* biases, uint16_t* q_out,
                         uint16_t* pages) {
  const uint32_t half = head_dim / 2, KP = K / 8, G = affine ? 64 : 32, SPR = K / G;
  const uint32_t q_dim = heads * head_dim, kv_dim = kv_heads * head_dim;
  const uint32_t page_no = (uint32_t)position / page_size, slot = (uint32_t)position % page_size;
  for (uint32_t group = 0; group < 3; group++) {
    const uint32_t nheads = group == 0 ? heads : kv_heads;
    const uint32_t row_base = group == 0 ? 0 : group == 1 ? q_dim : q_dim + kv_dim;
    for (uint32_t h = 0; h < nheads; h++)
      for (uint32_t d = 0; d < half; d++) {
        double v[2];
        for (int part = 0; part < 2; part++) {
          const size_t row = (size_t)row_base + (size_t)h * head_dim + d + (part ? half : 0);
          double acc = 0;
          for (uint32_t k = 0; k < K; k++) {
            const uint32_t q = (weights[row * KP + (k >> 3)] >> (4 * (k & 7))) & 15u;
            const double s = zo_f16_to_f32(scales[row * SPR + k / G]);
            const double w = affine ? (double)q * s + (double)zo_f16_to_f32(biases[row * SPR + k / G]) : ((double)q - 7.0) * s;
            acc += (double)zo_f16_to_f32(hidden[k]) * w;
          }
          v[part] = acc;
        }
        double lo = v[0], hi = v[1];
        if (group != 2) {
          const double freq = (double)position / pow(theta, (double)(d * 2) / (double)head_dim);
          const double c = cos(freq), s = sin(freq);
          lo = c * v[0] - s * v[1];
          hi = c * v[1] + s * v[0];
        }
        uint16_t* dst = group == 0 ? q_out + (size_t)h * head_dim + d
                                   : pages + (size_t)page_no * kv_page_stride + (size_t)h * head_page_stride +
                                         (size_t)slot * head_dim + pages_elem_offset + d + (group == 2 ? v_page_offset : 0);
        dst[0] = zo_f32_to_f16((float)lo);
        dst[half] = zo_f32_to_f16((float)hi);
      }
  }
}

/* ----------------------------------------------------- kv_quantize_int8 -- */

/* int8 quantisation of one token's K and V rows into the paged int8 cache
 * (src/compiler/shaders/kv_quantize_int8.wgsl:47-164), in the shader's f32 operations:
 * per (kv head, side) scale = max|x| / 127, at least 1e-8, stored as f16;
 * q = clamp(round-half-even(x * (1 / scale)), -127, 127), four to a word, low byte first.
 * k_slot / v_slot are [tokens][kv_heads*head_dim] f16 bit patterns; pages and scales already
 * hold the cache's previous contents. Layout: words page.head.slot.side.dim/4, scales
 * page.head.slot.side (src/compiler/model-spec.ts:652-658). */
ZO_API void zo_kv_quantize_int8(uint32_t kv_heads, uint32_t head_dim, uint32_t page_size, uint32_t tokens, const int32_t* positions,
                                uint32_t pages_word_offset, uint32_t scales_elem_offset, const uint16_t* k_slot, const uint16_t* v_slot,
                                uint32_t* pages, uint16_t* scales) {
  const uint32_t row_words = head_dim / 4, kv_dim = kv_heads * head_dim;
  for (uint32_t t = 0; t < tokens; t++) {
    if (positions[t] < 0) continue;
    const uint32_t page_no = (uint32_t)positions[t] / page_size, slot = (uint32_t)positions[t] % page_size;
    for (uint32_t h = 0; h < kv_heads; h++)
      for (uint32_t side = 0; side < 2; side++) {
        const uint16_t* src = (side ? v_slot : k_slot) + (size_t)t * kv_dim + (size_t)h * head_dim;
        float m = 0.f;
        for (uint32_t d = 0; d < head_dim; d++) m = fmaxf(m, fabsf(zo_f16_to_f32(src[d])));
        volatile float scale = m / 127.0f;
        if (scale < 1e-8f) scale = 1e-8f;
        volatile float inv = 1.0f / scale;
        scales[(size_t)page_no * kv_heads * page_size * 2 + (size_t)h * page_size * 2 + slot * 2 + side + scales_elem_offset] =
            zo_f32_to_f16(scale);
        const size_t base = (size_t)page_no * kv_heads * page_size * 2 * row_words + (size_t)h * page_size * 2 * row_words +
                            (size_t)slot * 2 * row_words + (size_t)side * row_words + pages_word_offset;
        for (uint32_t w = 0; w < row_words; w++) {
          uint32_t packed = 0;
          for (int i = 0; i < 4; i++) {
            volatile float prod = zo_f16_to_f32(src[4 * w + i]) * inv;
            float q = nearbyintf(prod);  /* default rounding mode: ties to even */
            q = q < -127.f ? -127.f : (q > 127.f ? 127.f : q);
            packed |= ((uint32_t)(int32_t)q & 0xffu) << (8 * i);
          }
          pages[base + w] = packed;
        }
      }
  }
}

/* ------------------------------------------------------- add + RMSNorm -- */

/* The FFN-entry add + RMSNorm as the fused-FFN prologue computes it
 * (src/compiler/shaders/fused_ffn_prologue.wgsl:62-97, the numerics of add_norm.wgsl):
 * val = f16(residual + delta); sum of f32(val)^2 in f32; rms_inv = 1 / sqrt(sum / K + eps);
 * out = f16(f32(val) * rms_inv * f32(gamma)). The order of the f32 sum is the implementation's (a
 * 64-lane tree in the shader, a wave-then-workgroup tree in the HIP kernel); every such order lies
 * within a few f32 steps of the exactly rounded sum, which is what this function uses (the squares
 * are exact in f32, so the double sum rounded once is that value). rms_inv may therefore differ from
 * a kernel's in its last bits, and out by one f16 step on the rare element at a rounding boundary. */
ZO_API void zo_add_rmsnorm(const uint16_t* residual, const uint16_t* delta, const uint16_t* gamma, uint32_t K, float eps,
                           uint16_t* out) {
  double exact = 0.0;
  for (uint32_t k = 0; k < K; k++) {
    const float val = zo_f16_to_f32(zo_f32_to_f16(zo_f16_to_f32(residual[k]) + zo_f16_to_f32(delta[k])));
    exact += (double)val * (double)val;
  }
  volatile float ss = (float)exact;
  volatile float mean = ss / (float)K;
  const float rms_inv = 1.0f / sqrtf(mean + eps);
  for (uint32_t k = 0; k < K; k++) {
    const float val = zo_f16_to_f32(zo_f32_to_f16(zo_f16_to_f32(residual[k]) + zo_f16_to_f32(delta[k])));
    volatile float t = val * rms_inv;
    volatile float u = t * zo_f16_to_f32(gamma[k]);
    out[k] = zo_f32_to_f16(u);
  }
}
