// Streaming GEMV for 4-bit affine group-64 weights on the int8 matrix cores.
//
// Same contract as gemv.hip (y[n] = sum_k x[k] * w[n,k], weights read once),
// built for the case that kernel loses: on this chip turning nibbles into
// exact f16 numbers costs more vector-ALU time than HBM needs to deliver them.
// Here the nibbles never become floats. A packed word is split into its even
// and odd nibbles with two AND and one shift (bytes 0..15 = int8), and
// v_mfma_i32_16x16x64_i8 forms the integer dot products against the
// ACTIVATIONS converted once per workgroup to block fixed point:
//
//   per group of 64 k:  x[k] ~ X[k] * 2^(e-22),  X = rne(x * 2^(22-e)),
//   2^e > max|x| over the group, |X| <= 2^22,  X = d0 + 256*d1 + 65536*d2 (signed bytes)
//
// The three digit planes occupy three A-operand rows, so ONE matrix
// instruction yields sum(d0*q), sum(d1*q), sum(d2*q) exactly (int32); the
// epilogue recombines them in f32 and applies the group scale and bias as the
// reference's factored form does (src/compiler/shaders/int4_matmul.gen.ts:78-84):
//   y += s*(f * 2^(e-22)) + b*sum(x)        f = c0 + 256*c1 + 65536*c2
// The only deviation from exact f16 activations is their rounding to 22 bits
// below the group maximum (|x - X*2^(e-22)| <= 2^(e-23)), below the noise of
// the f32 accumulation the family is specified with (:17-22). A one-hot x is
// represented exactly, so y reproduces the dequantized weight bit for bit.
//
// Work decomposition
//   unit      two spans of 128 consecutive k (2 x 16 words) of EIGHT rows: lane
//             (g = lane/16, c = lane%16) loads words 4g..4g+3 of span c/8 of row
//             c%8, so one 16-byte load per lane fetches whole 128-byte lines
//             and feeds two MFMAs (words 0,1 and words 2,3)
//   A rows    row 4*slot + d holds digit d of the activations of group slot of
//             the unit (slot = 2*span + half), zero outside that group's k. D
//             column c is meaningful for the slots of the span that column
//             loaded; lane group g = slot holds the three digit sums in c[0..2]
//   LDS       only the non-zero A pieces are stored (24 of 64 lanes per MFMA);
//             every other lane reads a shared zero piece through a zero stride,
//             so the inner loop has no predication at all
//   wave      8 output rows x (K / ksplit) k, a tile; a workgroup of 4 waves covers
//             4/ksplit tiles per iteration and reduces the K split through LDS
//   pipeline  the next batch of units (of this tile or the next) is loaded
//             before the current batch is consumed (double-buffered registers)
//   grid      x: tile groups (grid-stride), y: (token, slot) pair for MoE
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

struct I8Params {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  const uint32_t* ids;
  uint32_t N, K, k_packed, spr, ntiles;
  uint32_t ksplit;          // waves sharing one tile (1, 2 or 4)
  uint32_t units_per_wave;  // 256-k units each wave owns
  uint32_t out_f32, moe, M;
  uint32_t slots, in_slot_stride, out_slot_stride, in_tok_stride, out_tok_stride, ids_stride, experts;
};

// source k offset of byte j of a 16-byte operand piece (even nibbles of a word, then odd)
__host__ __device__ constexpr int piece_k(int j) { return (j >> 3) * 8 + ((j >> 2) & 1) + (j & 3) * 2; }

constexpr int BATCH = 4;          // units whose loads travel together (8 KB per wave in flight)
constexpr int WAVES = 4;
constexpr uint32_t ZERO_BYTES = 32;  // LDS bytes [0, 32): zeros every idle lane reads

template <int MT>
__global__ __launch_bounds__(64 * WAVES) void gemv_i8_kernel(const I8Params p) {
  extern __shared__ __align__(16) unsigned char smem[];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t g = lane >> 4, col = lane & 15u, row_in = col & 7u, col_span = col >> 3;
  const uint32_t U = p.K / 256u, G = p.K / 64u;  // units and groups per activation row

  // ---- MoE prologue (int4_matmul.gen.ts:236-253) ---------------------------------
  const _Float16* x = p.in;
  const uint32_t* wbase = p.weights;
  const _Float16* sbase = p.scales;
  const _Float16* bbase = p.biases;
  size_t out_base = 0;
  if (p.moe) {
    const uint32_t token = blockIdx.y / p.slots, slot = blockIdx.y % p.slots;
    const uint32_t expert = p.ids[(size_t)token * p.ids_stride + slot];
    if (p.experts && expert >= p.experts) return;  // uniform per workgroup
    wbase += (size_t)expert * p.N * p.k_packed;
    sbase += (size_t)expert * p.N * p.spr;
    bbase += (size_t)expert * p.N * p.spr;
    x += (size_t)token * p.in_tok_stride + (size_t)slot * p.in_slot_stride;
    out_base = (size_t)token * p.out_tok_stride + (size_t)slot * p.out_slot_stride;
  }

  // LDS map (bytes): [0,32) zeros | digit pieces [MT][U][2][24] x 16 | {2^(e-22), sum x} [MT][G] x 8 | K-split partials
  const uint32_t DIG0 = ZERO_BYTES;
  const uint32_t EX0 = DIG0 + MT * U * 48u * 16u;
  const uint32_t RED0 = EX0 + MT * G * 8u;
  float* red = reinterpret_cast<float*>(smem + RED0);  // [WAVES][MT][8]

  // ---- this wave's slice --------------------------------------------------------------------
  const uint32_t tiles_per_iter = WAVES / p.ksplit;
  const uint32_t ks = wave % p.ksplit, tile_lane = wave / p.ksplit;
  const uint32_t unit0 = ks * p.units_per_wave;
  const uint32_t nbatches = (p.units_per_wave + BATCH - 1) / BATCH;
  const uint32_t iters = (p.ntiles + tiles_per_iter - 1) / tiles_per_iter;

  struct Load {
    u32x4 w[BATCH];
    _Float16 s[BATCH], b[BATCH];
  };
  // lane-constant parts of the global addresses: row is added per tile, unit offsets are immediates
  const size_t w_lane = (size_t)((unit0 * 2u + col_span) * 16u + g * 4u);  // words
  const size_t s_lane = (size_t)((unit0 * 2u + col_span) * 2u + (g & 1u)); // groups
  auto issue = [&](Load& ld, uint32_t iter, uint32_t batch) {
    uint32_t n = (iter * tiles_per_iter + tile_lane) * 8u + row_in;
    n = n < p.N ? n : p.N - 1;  // clamped rows are never stored
    const uint32_t* wp = wbase + (size_t)n * p.k_packed + w_lane + (size_t)batch * (BATCH * 32u);
    const size_t so = (size_t)n * p.spr + s_lane + (size_t)batch * (BATCH * 4u);
    const uint32_t left = p.units_per_wave - batch * BATCH;
#pragma unroll
    for (int u = 0; u < BATCH; u++) {
      if ((uint32_t)u < left) {
        ld.w[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + u * 32));
        ld.s[u] = sbase[so + u * 4];
        ld.b[u] = bbase[so + u * 4];
      }
    }
  };

  // the first loads go out before the activations are staged
  Load lda, ldb;
  uint32_t iter = blockIdx.x, batch = 0;
  bool have = iter < iters;
  if (have) issue(lda, iter, 0);

  // ---- stage the activations as int8 digit planes ------------------------------------
  // One thread per 16-k operand piece; the 4 threads of a group are neighbouring
  // lanes and agree on the group maximum and sum with quad permutes.
  // Z = X + 0x808080 is read off the mantissa of x*2^(22-e) + 1.5*2^23; its three
  // bytes XOR 0x80 are signed digits with d0 + 256*d1 + 65536*d2 = X exactly.
  if (tid < ZERO_BYTES / 4) reinterpret_cast<uint32_t*>(smem)[tid] = 0u;
  const uint32_t pieces_per_tok = p.K / 16u;
  for (uint32_t pc = tid; pc < MT * pieces_per_tok; pc += blockDim.x) {
    const uint32_t t = pc / pieces_per_tok, pi = pc % pieces_per_tok;
    h2 xv[8];
    if (t < p.M) {
      const u32x4* src = reinterpret_cast<const u32x4*>(x + (size_t)t * p.K + (size_t)pi * 16u);
      const u32x4 a = src[0], b = src[1];
      xv[0] = as_h2(a.x); xv[1] = as_h2(a.y); xv[2] = as_h2(a.z); xv[3] = as_h2(a.w);
      xv[4] = as_h2(b.x); xv[5] = as_h2(b.y); xv[6] = as_h2(b.z); xv[7] = as_h2(b.w);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) xv[i] = as_h2(0u);
    }
    h2 mx = as_h2(as_u32(xv[0]) & 0x7FFF7FFFu);
    float sum = 0.f;
    const h2 ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (i) mx = __builtin_elementwise_max(mx, as_h2(as_u32(xv[i]) & 0x7FFF7FFFu));
      sum = __builtin_amdgcn_fdot2(xv[i], ones, sum, false);
    }
    float amax = __builtin_fmaxf((float)mx.x, (float)mx.y);
    amax = __builtin_fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0xB1, 0xF, 0xF, true)));
    sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, true));
    amax = __builtin_fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x4E, 0xF, 0xF, true)));
    sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0x4E, 0xF, 0xF, true));
    // 2^e > amax; a NaN or Inf anywhere in the group poisons its scale so the outputs turn NaN
    int e = 0;
    (void)__builtin_frexpf(amax, &e);
    const bool finite = amax < __builtin_inff() && sum == sum;
    const float up = finite ? __builtin_ldexpf(1.f, 22 - e) : 0.f;
    if ((pi & 3u) == 0) {
      f2 ex = {finite ? __builtin_ldexpf(1.f, e - 22) : __builtin_nanf(""), sum};
      *reinterpret_cast<f2*>(smem + EX0 + (t * G + (pi >> 2)) * 8u) = ex;
    }
    uint32_t z[16];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float lo = __builtin_fmaf((float)xv[i].x, up, 12582912.f);
      const float hi = __builtin_fmaf((float)xv[i].y, up, 12582912.f);
      z[2 * i] = __builtin_bit_cast(uint32_t, lo) + (0x00808080u - 0x4B400000u);
      z[2 * i + 1] = __builtin_bit_cast(uint32_t, hi) + (0x00808080u - 0x4B400000u);
    }
    // byte planes: word wq of a plane holds the values k = piece_k(4*wq .. 4*wq+3)
    uint32_t pl[3][4];
#pragma unroll
    for (int wq = 0; wq < 4; wq++) {
      const uint32_t za = z[piece_k(4 * wq)], zb = z[piece_k(4 * wq + 1)], zc = z[piece_k(4 * wq + 2)], zd = z[piece_k(4 * wq + 3)];
      const uint32_t ab01 = __builtin_amdgcn_perm(zb, za, 0x05010400u);  // [a0, b0, a1, b1]
      const uint32_t cd01 = __builtin_amdgcn_perm(zd, zc, 0x05010400u);  // [c0, d0, c1, d1]
      const uint32_t ab2 = __builtin_amdgcn_perm(zb, za, 0x0C0C0602u);   // [a2, b2, 0, 0]
      const uint32_t cd2 = __builtin_amdgcn_perm(zd, zc, 0x0C0C0602u);   // [c2, d2, 0, 0]
      pl[0][wq] = __builtin_amdgcn_perm(cd01, ab01, 0x05040100u) ^ 0x80808080u;  // [a0, b0, c0, d0]
      pl[1][wq] = __builtin_amdgcn_perm(cd01, ab01, 0x07060302u) ^ 0x80808080u;  // [a1, b1, c1, d1]
      pl[2][wq] = __builtin_amdgcn_perm(cd2, ab2, 0x05040100u) ^ 0x80808080u;    // [a2, b2, c2, d2]
    }
    // piece (span, gg, ii) -> unit span/2, MFMA ii, compact row gg*6 + (span&1)*3 + d
    const uint32_t span = pi >> 3, gg = (pi >> 1) & 3u, ii = pi & 1u;
    const uint32_t idx = ((t * U + (span >> 1)) * 2u + ii) * 24u + gg * 6u + (span & 1u) * 3u;
#pragma unroll
    for (int d = 0; d < 3; d++)
      *reinterpret_cast<v4i*>(smem + DIG0 + (idx + d) * 16u) = (v4i){(int)pl[d][0], (int)pl[d][1], (int)pl[d][2], (int)pl[d][3]};
  }
  __syncthreads();

  // ---- per-lane LDS addressing: live lanes walk their pieces, idle lanes sit on the zeros ----
  // A operand: row r = lane % 16 -> slot r/4 = 2*span + half, digit r%4; the lane's k slice g is in half g/2
  const uint32_t a_slot = col >> 2, a_dig = col & 3u;
  const bool a_live = a_dig < 3u && (a_slot & 1u) == (g >> 1);
  const uint32_t a_unit = a_live ? 48u * 16u : 0u;  // byte stride per unit
  const uint32_t a_half = a_live ? 24u * 16u : 0u;  // byte stride between the two MFMAs of a unit
  const uint32_t a_tok = a_live ? U * 48u * 16u : 0u;
  const uint32_t a_base = a_live ? DIG0 + (unit0 * 48u + g * 6u + (a_slot >> 1) * 3u + a_dig) * 16u : 0u;
  // D: lane group g = slot; meaningful when the slot's span is the one column `col` loaded
  const bool c_live = (g >> 1) == col_span;
  const uint32_t e_unit = c_live ? 32u : 0u;
  const uint32_t e_tok = c_live ? G * 8u : 0u;
  const uint32_t e_base = c_live ? EX0 + (unit0 * 4u + g) * 8u : 16u;

  float acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = 0.f;
  const v4i vzero = {0, 0, 0, 0};

  // one pipeline stage: prefetch the next batch (of this tile or the next), consume `cur`
  auto stage = [&](const Load& cur, Load& nxt) {
    uint32_t niter = iter, nbatch = batch + 1;
    if (nbatch == nbatches) { nbatch = 0; niter += gridDim.x; }
    const bool nhave = niter < iters;
    if (nhave) issue(nxt, niter, nbatch);
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t left = p.units_per_wave - batch * BATCH;
    const uint32_t a_off = a_base + batch * BATCH * a_unit;
    const uint32_t e_off = e_base + batch * BATCH * e_unit;
    // Three phases over the whole batch, so that the LDS reads, the matrix
    // instructions and the f32 epilogues of different units overlap instead of
    // forming one dependent chain per unit.
    v4i a0[BATCH][MT], a1[BATCH][MT];
    f2 ex[BATCH][MT];
#pragma unroll
    for (int u = 0; u < BATCH; u++)
#pragma unroll
      for (int t = 0; t < MT; t++) {
        const uint32_t ao = a_off + u * a_unit + t * a_tok;
        a0[u][t] = *reinterpret_cast<const v4i*>(smem + ao);
        a1[u][t] = *reinterpret_cast<const v4i*>(smem + ao + a_half);
        ex[u][t] = *reinterpret_cast<const f2*>(smem + e_off + u * e_unit + t * e_tok);  // {2^(e-22), sum x}; zeros on idle lanes
      }
    v4i c[BATCH][MT];
#pragma unroll
    for (int u = 0; u < BATCH; u++) {
      const uint32_t w[4] = {cur.w[u].x, cur.w[u].y, cur.w[u].z, cur.w[u].w};
      v4i b0, b1;
      b0.x = (int)(w[0] & 0x0F0F0F0Fu); b0.y = (int)((w[0] >> 4) & 0x0F0F0F0Fu);
      b0.z = (int)(w[1] & 0x0F0F0F0Fu); b0.w = (int)((w[1] >> 4) & 0x0F0F0F0Fu);
      b1.x = (int)(w[2] & 0x0F0F0F0Fu); b1.y = (int)((w[2] >> 4) & 0x0F0F0F0Fu);
      b1.z = (int)(w[3] & 0x0F0F0F0Fu); b1.w = (int)((w[3] >> 4) & 0x0F0F0F0Fu);
#pragma unroll
      for (int t = 0; t < MT; t++) {
        c[u][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[u][t], b0, vzero, 0, 0, 0);
        c[u][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[u][t], b1, c[u][t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < BATCH; u++) {
      if ((uint32_t)u >= left) break;  // a short last batch: registers of the missing units hold stale data
      const float s = (float)cur.s[u], b = (float)cur.b[u];
#pragma unroll
      for (int t = 0; t < MT; t++) {
        const float f = __builtin_fmaf(65536.f, (float)c[u][t][2], __builtin_fmaf(256.f, (float)c[u][t][1], (float)c[u][t][0]));
        acc[t] += __builtin_fmaf(s, f * ex[u][t].x, b * ex[u][t].y);
      }
    }

    if (batch == nbatches - 1) {
      // tile finished: sum the four lane groups and the two column halves, then the K split
      const uint32_t tile = iter * tiles_per_iter + tile_lane;
      const bool store_ok = lane < 8 && tile < p.ntiles && tile * 8u + lane < p.N;
#pragma unroll
      for (int t = 0; t < MT; t++) {
        float v = acc[t];
        acc[t] = 0.f;
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        v += __shfl_xor(v, 8);
        if (p.ksplit > 1) {
          if (lane < 8) red[(wave * MT + t) * 8 + lane] = v;
        } else if (store_ok && (uint32_t)t < p.M) {
          const size_t o = p.moe ? out_base + tile * 8u + lane : (size_t)t * p.N + tile * 8u + lane;
          if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = v;
          else reinterpret_cast<_Float16*>(p.out)[o] = (_Float16)v;
        }
      }
      if (p.ksplit > 1) {
        __syncthreads();
        if (ks == 0 && store_ok) {
#pragma unroll
          for (int t = 0; t < MT; t++) {
            float y = 0.f;
            for (uint32_t k2 = 0; k2 < p.ksplit; k2++) y += red[((wave + k2) * MT + t) * 8 + lane];
            if ((uint32_t)t < p.M) {
              const size_t o = p.moe ? out_base + tile * 8u + lane : (size_t)t * p.N + tile * 8u + lane;
              if (p.out_f32) reinterpret_cast<float*>(p.out)[o] = y;
              else reinterpret_cast<_Float16*>(p.out)[o] = (_Float16)y;
            }
          }
        }
        __syncthreads();
      }
    }
    iter = niter; batch = nbatch; have = nhave;
  };

  while (have) {
    stage(lda, ldb);
    if (!have) break;
    stage(ldb, lda);
  }
}

// K split: waves per tile. Every wave needs a whole number of 256-k units.
uint32_t pick_ksplit(uint32_t units, uint32_t N, uint32_t pairs, int cus, int want) {
  if (want == 1 || want == 2 || want == 4) return units % (uint32_t)want == 0 ? (uint32_t)want : 0;
  // split K when there are too few 8-row tiles to give every CU several waves
  const uint64_t tiles = (uint64_t)((N + 7) / 8) * pairs;
  uint32_t ks = 1;
  while (ks < 4 && units % (ks * 2) == 0 && (tiles * ks < (uint64_t)cus * 12 || units / ks > 8)) ks *= 2;
  return ks;
}

size_t lds_bytes(uint32_t mt, uint32_t K) {
  return ZERO_BYTES + (size_t)mt * (K / 256) * 48 * 16 + (size_t)mt * (K / 64) * 8 + (size_t)WAVES * mt * 8 * 4;
}

}  // namespace

// 4-bit affine, K a multiple of 256 (whole units), up to 4 activation rows.
bool gemv_i8_supports(const MatmulArgs& a) {
  if (a.bits != 4 || !a.affine || a.K % 256 != 0) return false;
  const uint32_t M = a.slots ? 1 : a.M;
  if (M < 1 || M > 4) return false;
  return lds_bytes(M > 2 ? 4 : M, a.K) <= 150 * 1024;
}

hipError_t launch_gemv_i8(const MatmulArgs& a, const Tune& t, hipStream_t s) {
  I8Params p{};
  p.out = a.out; p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases; p.ids = a.ids;
  p.N = a.N; p.K = a.K; p.k_packed = a.k_packed; p.spr = a.spr;
  p.out_f32 = a.out_f32; p.moe = a.slots > 0; p.M = a.slots ? 1 : a.M;
  p.slots = a.slots; p.in_slot_stride = a.in_slot_stride; p.out_slot_stride = a.out_slot_stride;
  p.in_tok_stride = a.in_tok_stride; p.out_tok_stride = a.out_tok_stride; p.ids_stride = a.ids_stride;
  p.experts = a.experts;
  p.ntiles = (a.N + 7) / 8;
  const uint32_t units = a.K / 256;
  const uint32_t pairs = p.moe ? a.slots * a.tokens : 1;
  p.ksplit = pick_ksplit(units, a.N, pairs, t.num_cus, t.i8_ksplit);
  if (!p.ksplit) return hipErrorInvalidValue;
  p.units_per_wave = units / p.ksplit;
  const int mt = p.M > 2 ? 4 : (int)p.M;
  const size_t smem = lds_bytes(mt, a.K);
  // workgroups: as many as fit the target residency, then evened out so that
  // every workgroup runs the same number of iterations (no half-empty last round)
  const uint32_t iters = (p.ntiles + (WAVES / p.ksplit) - 1) / (WAVES / p.ksplit);
  uint32_t gx = (uint32_t)t.num_cus * (t.i8_wg_per_cu ? t.i8_wg_per_cu : 3) / pairs;
  if (gx < 1) gx = 1;
  if (gx > iters) gx = iters;
  const uint32_t rounds = (iters + gx - 1) / gx;
  gx = (iters + rounds - 1) / rounds;
  const dim3 grid(gx, pairs, 1);
  const void* k = mt == 1 ? (const void*)gemv_i8_kernel<1> : mt == 2 ? (const void*)gemv_i8_kernel<2> : (const void*)gemv_i8_kernel<4>;
  if (smem > 64 * 1024) (void)hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  switch (mt) {
    case 1: hipLaunchKernelGGL((gemv_i8_kernel<1>), grid, dim3(64 * WAVES), smem, s, p); break;
    case 2: hipLaunchKernelGGL((gemv_i8_kernel<2>), grid, dim3(64 * WAVES), smem, s, p); break;
    default: hipLaunchKernelGGL((gemv_i8_kernel<4>), grid, dim3(64 * WAVES), smem, s, p); break;
  }
  return hipGetLastError();
}

}  // namespace ztvm
