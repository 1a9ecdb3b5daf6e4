/*
 * CPU oracle for the int4/int3 group-quantized dequant-matmul family.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only the test-suite, the
 * smoke check and the bench's cpu_baseline leg may link or call it; the
 * shipped library (libztvm_hip.so) never does and has no CPU fallback.
 *
 * Every function restates, in plain C, arithmetic that the reference
 * (abgnydn/zero-tvm, TypeScript + WGSL) holds in its kernel generator and in
 * the JS references of its own kernel tests. Citations are paths relative to
 * the reference's root.
 *
 * Parity pins (what a plausible mistake would break):
 *   zo_f32_to_f16 / zo_f16_to_f32  exhaustive 65536-pattern round trip and
 *                                  comparison against numpy float16 casts
 *   zo_mulberry32                  closed-form re-derivation in Python ints
 *   zo_unpack4                     byte-wise even/odd formulation
 *                                  (int4_matmul.gen.ts:1175-1180) + numpy
 *   zo_unpack8                     numpy's little-endian byte view of the words
 *   zo_unpack3 / zo_unpack3_window numpy.unpackbits(bitorder='little') and
 *                                  the two forms against each other for
 *                                  every block shift {0,24,16,8}
 *   zo_dequant_*                   brute force over all q x all finite f16
 *                                  scales x sampled biases against numpy
 *                                  float32 arithmetic
 *   zo_gemv_* / zo_gemm_*          one-hot activations (y == W[n,k]),
 *                                  constant nibbles, zero scale, float64
 *                                  matmul on the dequantized matrix
 *   zo_moe_gemv                    equality with dense calls on the
 *                                  gathered expert slab
 * The reference commits no golden vectors for this path (its real-weight
 * bundles are git-ignored), so nothing here is checked against a
 * reference-held output; the vendor (MLX) on-disk format fidelity is
 * therefore "parity unpinned" and rests on the documented bit layout.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ZO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ f16 -- */

/* f32 -> f16 bits, round to nearest even, subnormals kept.
 * Follows tests/kernels/half.mjs:13-36 (same as
 * src/zero-tvm/mlx-weights.ts:157-180). */
ZO_API uint16_t zo_f32_to_f16(float val) {
  uint32_t x;
  memcpy(&x, &val, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  int32_t exp = (int32_t)((x >> 23) & 0xffu);
  uint32_t mant = x & 0x7fffffu;
  if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0u));
  exp = exp - 127 + 15;
  if (exp >= 0x1f) return (uint16_t)(sign | 0x7c00u);
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    mant |= 0x800000u;
    int sh = 14 - exp;
    uint32_t h = mant >> sh;
    uint32_t rem = mant & ((1u << sh) - 1u);
    uint32_t half = 1u << (sh - 1);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((uint32_t)exp << 10) | (mant >> 13);
  uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

/* f16 bits -> f32. Follows tests/kernels/half.mjs:39-63. */
ZO_API float zo_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t mant = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (mant == 0) {
      bits = sign;
    } else {
      int e = -1;
      uint32_t m = mant;
      do {
        e++;
        m <<= 1;
      } while (!(m & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (exp == 0x1f) {
    bits = sign | 0x7f800000u | (mant << 13);
  } else {
    bits = sign | ((exp - 15 + 127) << 23) | (mant << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

ZO_API void zo_f32_to_f16_array(const float* src, uint16_t* dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = zo_f32_to_f16(src[i]);
}
ZO_API void zo_f16_to_f32_array(const uint16_t* src, float* dst, size_t n) {
  for (size_t i = 0; i < n; i++) dst[i] = zo_f16_to_f32(src[i]);
}

/* ------------------------------------------------------------------ rng -- */

/* mulberry32, the PRNG of the reference's kernel tests
 * (tests/kernels/run.mjs:44-52). `state` is the JS closure's `seed`;
 * returns a double in [0,1). */
ZO_API double zo_mulberry32(uint32_t* state) {
  uint32_t seed = *state + 0x6d2b79f5u;
  *state = seed;
  uint32_t t = (seed ^ (seed >> 15)) * (1u | seed);
  t = (t + ((t ^ (t >> 7)) * (61u | t))) ^ t;
  return (double)(t ^ (t >> 14)) / 4294967296.0;
}

/* The reference's seeded GEMV test vector (tests/kernels/run.mjs:77-104):
 * toF16 is f64 -> f32 -> f16 (tests/kernels/half.mjs:66).
 * rng(1); input[K] = toF16(r*2-1); scales[N*SPR] = toF16(r*0.05+0.01);
 * affine: biases[N*SPR] = toF16(r*0.1-0.05); then q3 values floor(r*8)
 * packed bit-serially (:90-100), or int4 words (r*0xffffffff)>>>0 (:103).
 * Outputs are f16 bit patterns and packed words. */
ZO_API void zo_reference_gemv_case(uint32_t seed, uint32_t N, uint32_t K, int affine, int q3, uint16_t* input,
                                   uint16_t* scales, uint16_t* biases, uint32_t* weights) {
  uint32_t st = seed;
  uint32_t KP = q3 ? (K * 3) / 32 : K / 8;
  uint32_t SPR = K / (affine ? 64 : 32);
  for (uint32_t i = 0; i < K; i++) input[i] = zo_f32_to_f16((float)(zo_mulberry32(&st) * 2 - 1));
  for (uint32_t i = 0; i < N * SPR; i++) scales[i] = zo_f32_to_f16((float)(zo_mulberry32(&st) * 0.05 + 0.01));
  if (affine)
    for (uint32_t i = 0; i < N * SPR; i++) biases[i] = zo_f32_to_f16((float)(zo_mulberry32(&st) * 0.1 - 0.05));
  if (q3) {
    uint8_t* q = (uint8_t*)malloc((size_t)N * K);
    for (size_t i = 0; i < (size_t)N * K; i++) q[i] = (uint8_t)floor(zo_mulberry32(&st) * 8);
    memset(weights, 0, (size_t)N * KP * 4);
    for (uint32_t row = 0; row < N; row++)
      for (uint32_t i = 0; i < K; i++) {
        uint32_t v = q[(size_t)row * K + i];
        uint32_t bit = 3 * i, w = row * KP + (bit >> 5), sh = bit & 31;
        weights[w] |= v << sh;
        if (sh > 29) weights[w + 1] |= v >> (32 - sh);
      }
    free(q);
  } else {
    for (size_t i = 0; i < (size_t)N * KP; i++) {
      double d = zo_mulberry32(&st) * 4294967295.0; /* (r*0xffffffff)>>>0 */
      weights[i] = (uint32_t)d;
    }
  }
}

/* --------------------------------------------------------------- unpack -- */

/* 4-bit: value k of a row is (W[k>>3] >> 4*(k&7)) & 15, LSB-first
 * (src/compiler/shaders/int4_matmul.gen.ts:157-167;
 * tests/kernels/compile-qwen35.mjs:1065). */
ZO_API uint32_t zo_unpack4(const uint32_t* row, uint32_t k) { return (row[k >> 3] >> (4 * (k & 7))) & 15u; }

/* 3-bit, closed form: each row is one LSB-first bitstream and value k owns
 * bits [3k, 3k+3) (src/compiler/shaders/int4_matmul.gen.ts:115-133; packer
 * tests/kernels/run.mjs:90-100; scripts/make-kernel-ref.py:55-63). */
ZO_API uint32_t zo_unpack3(const uint32_t* row, uint32_t k) {
  uint32_t bit = 3 * k, w = bit >> 5, sh = bit & 31;
  uint64_t two = row[w];
  if (sh > 29) two |= (uint64_t)row[w + 1] << 32;
  return (uint32_t)(two >> sh) & 7u;
}

/* 3-bit, the kernel's own form: 8-value blocks read through a 24-bit window
 * whose in-word shift cycles {0,24,16,8}; the second word is OR-ed in only
 * when sh > 8 (src/compiler/shaders/int4_matmul.gen.ts:409-448). */
ZO_API uint32_t zo_unpack3_window(const uint32_t* row, uint32_t k) {
  uint32_t block = k >> 3, i = k & 7;
  uint32_t bit = block * 24, sh = bit & 31, wi = bit >> 5;
  uint32_t win = row[wi] >> sh;
  if (sh > 8) win |= row[wi + 1] << (32 - sh);
  return (win >> (3 * i)) & 7u;
}

/* Bit-serial 3-bit packer (tests/kernels/run.mjs:90-100). `words` must hold
 * 3K/32 entries and is overwritten. */
ZO_API void zo_pack3(const uint8_t* values, uint32_t K, uint32_t* words) {
  memset(words, 0, (size_t)(3 * K / 32) * 4);
  for (uint32_t i = 0; i < K; i++) {
    uint32_t v = values[i] & 7u, bit = 3 * i, w = bit >> 5, sh = bit & 31;
    words[w] |= v << sh;
    if (sh > 29) words[w + 1] |= v >> (32 - sh);
  }
}

ZO_API void zo_pack4(const uint8_t* values, uint32_t K, uint32_t* words) {
  memset(words, 0, (size_t)(K / 8) * 4);
  for (uint32_t i = 0; i < K; i++) words[i >> 3] |= (uint32_t)(values[i] & 15u) << (4 * (i & 7));
}

/* 8-bit (MLX affine): four unsigned bytes per word, value k at bits [8(k&3), 8(k&3)+8) of word k>>2
 * (src/compiler/shaders/int8_affine_matvec.wgsl:57-66; tests/kernels/int8-affine.mjs:76-78). */
ZO_API uint32_t zo_unpack8(const uint32_t* row, uint32_t k) { return (row[k >> 2] >> (8u * (k & 3u))) & 255u; }

ZO_API void zo_pack8(const uint8_t* values, uint32_t K, uint32_t* words) {
  memset(words, 0, (size_t)(K / 4) * 4);
  for (uint32_t i = 0; i < K; i++) words[i >> 2] |= (uint32_t)values[i] << (8 * (i & 3));
}

static inline uint32_t unpack_q(const uint32_t* row, uint32_t k, uint32_t bits) {
  return bits == 3 ? zo_unpack3(row, k) : bits == 8 ? zo_unpack8(row, k) : zo_unpack4(row, k);
}

/* -------------------------------------------------------------- dequant -- */

/* Affine (MLX, group 64): w = q*s + b evaluated once in f32
 * (src/zero-tvm/mlx-weights.ts:637-648 stores `nibble*s + b`, computed in
 * f64, into a Float32Array; q*s is exact, so this is one f32 rounding).
 * Symmetric (MLC q4f16_1, group 32): w = (q-7)*s
 * (src/compiler/shaders/int4_matmul.gen.ts:17-19). */
ZO_API float zo_dequant_f32(uint32_t q, uint16_t s16, uint16_t b16, int affine) {
  double s = zo_f16_to_f32(s16);
  if (affine) return (float)((double)q * s + (double)zo_f16_to_f32(b16));
  return (float)(((double)q - 7.0) * s);
}

/* The f16 a kernel stages: RNE of the f32 value
 * (src/compiler/shaders/int4_matmul.gen.ts:1111-1113;
 * src/zero-tvm/mlx-weights.ts:651-660). */
ZO_API uint16_t zo_dequant_f16(uint32_t q, uint16_t s16, uint16_t b16, int affine) {
  return zo_f32_to_f16(zo_dequant_f32(q, s16, b16, affine));
}

/* Whole matrix [N,K]: out_f32 and/or out_f16 may be NULL. */
ZO_API void zo_dequant_matrix(uint32_t bits, int affine, uint32_t N, uint32_t K, const uint32_t* weights,
                              const uint16_t* scales, const uint16_t* biases, float* out_f32, uint16_t* out_f16) {
  uint32_t KP = K * bits / 32, G = affine ? 64 : 32, SPR = K / G;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < (int64_t)N; n++) {
    const uint32_t* row = weights + (size_t)n * KP;
    for (uint32_t k = 0; k < K; k++) {
      uint32_t g = k / G;
      uint16_t s = scales[(size_t)n * SPR + g], b = affine ? biases[(size_t)n * SPR + g] : 0;
      float w = zo_dequant_f32(unpack_q(row, k, bits), s, b, affine);
      if (out_f32) out_f32[(size_t)n * K + k] = w;
      if (out_f16) out_f16[(size_t)n * K + k] = zo_f32_to_f16(w);
    }
  }
}

/* ----------------------------------------------------------- GEMV / GEMM -- */

/* One output element, the reference test's own factored arithmetic
 * (tests/kernels/run.mjs:109-135): per weight word one (scale,bias) pair,
 * dot and xs over that word's 8 activations, everything in JS doubles; q3
 * uses the per-value form of :111-118. Returns the unrounded double. */
static double gemv_row_js(uint32_t bits, int affine, uint32_t K, const uint32_t* row, const uint16_t* s_row,
                          const uint16_t* b_row, const float* x) {
  double acc = 0;
  if (bits == 8) {
    /* the 8-bit kernels' factored form, one (scale, bias) pair per group of 64
     * (src/compiler/shaders/int8_affine_matvec.wgsl:52-69) */
    for (uint32_t g = 0; g < K / 64; g++) {
      double s = zo_f16_to_f32(s_row[g]), b = zo_f16_to_f32(b_row[g]), dot = 0, xs = 0;
      for (uint32_t i = g * 64; i < (g + 1) * 64; i++) {
        dot += (double)x[i] * (double)zo_unpack8(row, i);
        xs += (double)x[i];
      }
      acc += s * dot + b * xs;
    }
    return acc;
  }
  if (bits == 3) {
    for (uint32_t i = 0; i < K; i++) {
      uint32_t g = i >> 6;
      double s = zo_f16_to_f32(s_row[g]), b = zo_f16_to_f32(b_row[g]);
      acc += s * (double)x[i] * (double)zo_unpack3(row, i) + b * (double)x[i];
    }
    return acc;
  }
  for (uint32_t w = 0; w < K / 8; w++) {
    uint32_t packed = row[w];
    uint32_t g = affine ? w >> 3 : w >> 2;
    double scale = zo_f16_to_f32(s_row[g]);
    double dot = 0, xs = 0;
    for (uint32_t n = 0; n < 8; n++) {
      int nib = (int)((packed >> (4 * n)) & 15u);
      dot += (double)x[w * 8 + n] * (double)(affine ? nib : nib - 7);
      xs += (double)x[w * 8 + n];
    }
    acc += scale * dot;
    if (affine) acc += (double)zo_f16_to_f32(b_row[g]) * xs;
  }
  return acc;
}

/* One output element from the formula, per element, never factored
 * (tests/kernels/compile-qwen35.mjs:1062-1069, :1123-1136):
 * acc += (s*q + b) * x   or   s*(q-7)*x, in doubles. */
static double gemm_elem_formula_f64(uint32_t bits, int affine, uint32_t K, const uint32_t* row,
                                    const uint16_t* s_row, const uint16_t* b_row, const float* x) {
  uint32_t G = affine ? 64 : 32;
  double acc = 0;
  for (uint32_t i = 0; i < K; i++) {
    uint32_t g = i / G;
    double q = (double)unpack_q(row, i, bits), s = zo_f16_to_f32(s_row[g]);
    acc += affine ? (s * q + (double)zo_f16_to_f32(b_row[g])) * (double)x[i] : s * (q - 7.0) * (double)x[i];
  }
  return acc;
}

/* Same formula with an f32 accumulator and f32 dequantized weight: the
 * "fp32-accumulated reference" the output tolerance is quoted against
 * (f32 accumulation is the family's contract,
 * src/compiler/shaders/int4_matmul.gen.ts:17-22). */
static float gemm_elem_formula_f32(uint32_t bits, int affine, uint32_t K, const uint32_t* row,
                                   const uint16_t* s_row, const uint16_t* b_row, const float* x) {
  uint32_t G = affine ? 64 : 32;
  float acc = 0.f;
  for (uint32_t g = 0; g < K / G; g++) {
    uint16_t s = s_row[g], b = affine ? b_row[g] : 0;
    for (uint32_t i = g * G; i < (g + 1) * G; i++) {
      float w = zo_dequant_f32(unpack_q(row, i, bits), s, b, affine);
      acc = fmaf(w, x[i], acc);
    }
  }
  return acc;
}

/* Dequantized weight rounded to f16 before the multiply, as the matrix-unit
 * kernels stage it (scripts/gemm-sweep-native.mjs:356-363, :388-406). */
static double gemm_elem_f16w(uint32_t bits, int affine, uint32_t K, const uint32_t* row, const uint16_t* s_row,
                             const uint16_t* b_row, const float* x) {
  uint32_t G = affine ? 64 : 32;
  double acc = 0;
  for (uint32_t i = 0; i < K; i++) {
    uint32_t g = i / G;
    uint16_t w16 = zo_dequant_f16(unpack_q(row, i, bits), s_row[g], affine ? b_row[g] : 0, affine);
    acc += (double)zo_f16_to_f32(w16) * (double)x[i];
  }
  return acc;
}

enum { ZO_MODE_JS = 0, ZO_MODE_FORMULA_F64 = 1, ZO_MODE_FORMULA_F32 = 2, ZO_MODE_F16W = 3 };

/* Y[m,n] for m<M, n<N as doubles (unrounded), `mode` selects the flavour
 * above. A is f16 bits [M,K] row-major with row stride lda elements.
 * threads <= 1 runs the faithful single-thread loop order. */
ZO_API void zo_gemm(int mode, uint32_t bits, int affine, uint32_t M, uint32_t N, uint32_t K, const uint16_t* A,
                    uint32_t lda, const uint32_t* weights, const uint16_t* scales, const uint16_t* biases,
                    double* Y, int threads) {
  uint32_t KP = K * bits / 32, SPR = K / (affine ? 64 : 32);
  float* Af = (float*)malloc((size_t)M * K * sizeof(float));
  for (uint32_t m = 0; m < M; m++) zo_f16_to_f32_array(A + (size_t)m * lda, Af + (size_t)m * K, K);
#ifdef _OPENMP
  if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads)
#endif
  for (int64_t n = 0; n < (int64_t)N; n++) {
    const uint32_t* row = weights + (size_t)n * KP;
    const uint16_t* s_row = scales + (size_t)n * SPR;
    const uint16_t* b_row = affine ? biases + (size_t)n * SPR : NULL;
    for (uint32_t m = 0; m < M; m++) {
      const float* x = Af + (size_t)m * K;
      double y;
      switch (mode) {
        case ZO_MODE_JS: y = gemv_row_js(bits, affine, K, row, s_row, b_row, x); break;
        case ZO_MODE_FORMULA_F32: y = gemm_elem_formula_f32(bits, affine, K, row, s_row, b_row, x); break;
        case ZO_MODE_F16W: y = gemm_elem_f16w(bits, affine, K, row, s_row, b_row, x); break;
        default: y = gemm_elem_formula_f64(bits, affine, K, row, s_row, b_row, x); break;
      }
      Y[(size_t)m * N + n] = y;
    }
  }
  free(Af);
}

/* MoE gathered GEMV: for every (token, slot), expert = ids[token*ids_stride+slot];
 * weight/scale bases expert*N*K_PACKED and expert*N*SPR; input at
 * token*in_tok_stride + slot*in_slot_stride, output (as a double, in a
 * caller buffer indexed like the kernel's f16 output) at
 * token*out_tok_stride + slot*out_slot_stride
 * (src/compiler/shaders/int4_matmul.gen.ts:236-253, PODArgs :216-225). */
ZO_API void zo_moe_gemv(int mode, uint32_t bits, uint32_t N, uint32_t K, uint32_t tokens, uint32_t slots,
                        uint32_t in_slot_stride, uint32_t out_slot_stride, uint32_t in_tok_stride,
                        uint32_t out_tok_stride, uint32_t ids_stride, const uint32_t* ids, const uint16_t* in,
                        const uint32_t* weights, const uint16_t* scales, const uint16_t* biases, double* out,
                        int threads) {
  uint32_t KP = K * bits / 32, SPR = K / 64;
  for (uint32_t t = 0; t < tokens; t++)
    for (uint32_t s = 0; s < slots; s++) {
      uint32_t e = ids[(size_t)t * ids_stride + s];
      zo_gemm(mode, bits, 1, 1, N, K, in + (size_t)t * in_tok_stride + (size_t)s * in_slot_stride, K,
              weights + (size_t)e * N * KP, scales + (size_t)e * N * SPR, biases + (size_t)e * N * SPR,
              out + (size_t)t * out_tok_stride + (size_t)s * out_slot_stride, threads);
    }
}

ZO_API int zo_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
