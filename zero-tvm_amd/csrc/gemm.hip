// Prefill GEMM for group-quantized weights on the CDNA4 matrix cores:
//   Y[m,n] = sum_k A[m,k] * w[n,k],  A f16 [M,K], w = s*q + b (or s*(q-7)), f32 accumulate.
//
// Replaces the reference's runtime-M, tiled and matrix-unit GEMM generators
// (src/compiler/shaders/int4_matmul.gen.ts: int4MatmulBatchedDynWGSL :580-695,
// int4MatmulTiledMWGSL :805-910, int4MatmulTiledStWGSL :930-1028,
// int4MatmulSgE1WGSL :1171-1299, int4MatmulSgE5WGSL :1329-1456) with one wave64
// MFMA design that keeps the GEMV's arithmetic:
//
//   y = sum_g  s[n,g] * ( sum_{k in g} x[m,k]*q[n,k] )  +  sum_g b[n,g] * xs[m,g]
//
// The weight tile is staged in LDS as the EXACT f16 integers q (or q-7), the
// matrix cores form the inner sums (f16 x f16 products are exact in f32), and
// the group scale is applied in f32 when a group's partial sum is folded into
// the running total. Staging finished f16 weights s*q+b instead, as the
// reference's matrix-unit kernels do (:1175-1180), rounds every weight to 11
// bits and was measured at 3.4e-2 against the formula by the reference itself
// (:954-958); this form keeps the GEMM within f32-accumulation noise of the
// per-token GEMV path. The bias term is a second, tiny GEMM over the groups:
// xs[m,g] = sum_{k in g} x[m,k] is produced once by a pre-pass as an f16
// (hi, lo) pair and multiplied by the f16 biases on the matrix cores too.
//
// Tiling
//   workgroup  WM x WN waves, each wave a 64 x 64 output tile (2 x 2 blocks of
//              v_mfma_f32_32x32x16_f16); A operand = activations, B operand =
//              weights, so lanes of D run along n and stores are contiguous
//   K step     64 = one affine group (two symmetric groups), double-buffered LDS
//   LDS rows   64 f16 = eight 16-byte chunks, chunk index XOR (row & 7): the
//              lanes served together by a 128-bit read hit distinct banks
//   grid       one workgroup per tile, ids remapped so that the tiles sharing
//              a weight panel run on the same XCD (same L2)
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

constexpr int KS = 64;     // k per step
constexpr int CHUNKS = 8;  // 16-byte chunks per LDS row

struct GemmParams {
  _Float16* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  const _Float16* xs16;  // [M][2*G]: hi halves then lo halves of the group sums
  uint32_t M, N, K, k_packed, spr;
  uint32_t mtiles, ntiles, nsteps, bias_steps;
  uint32_t xcd_swizzle;
};

// One packed word -> eight exact f16 integers in natural k order. A byte holds
// values (2j, 2j+1); replicating the low byte pair into both halves of a word
// puts the even nibble at mantissa bit 0 of the low half (offset 1024) and the
// odd nibble at mantissa bit 4 of the high half (offset 64).
template <bool AFFINE>
__device__ __forceinline__ h8 unpack_word_natural(uint32_t w, uint32_t c_mixed) {
  const h2 off = AFFINE ? (h2){(_Float16)1024.f, (_Float16)64.f} : (h2){(_Float16)1031.f, (_Float16)71.f};
  const uint32_t t01 = __builtin_amdgcn_perm(0u, w, 0x01000100u);  // bytes [b0,b1,b0,b1]
  const uint32_t t23 = __builtin_amdgcn_perm(0u, w, 0x03020302u);  // bytes [b2,b3,b2,b3]
  const h2 p0 = as_h2(and_or(t01, 0x00F0000Fu, c_mixed)) - off;       // v0, v1
  const h2 p1 = as_h2(and_or(t01 >> 8, 0x00F0000Fu, c_mixed)) - off;  // v2, v3
  const h2 p2 = as_h2(and_or(t23, 0x00F0000Fu, c_mixed)) - off;       // v4, v5
  const h2 p3 = as_h2(and_or(t23 >> 8, 0x00F0000Fu, c_mixed)) - off;  // v6, v7
  return (h8){p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// Group sums of the activations: xs16[m][g] = f16(xs), xs16[m][G+g] = f16(xs - hi).
__global__ __launch_bounds__(256) void xsum_kernel(const _Float16* __restrict__ in, _Float16* __restrict__ xs16, uint32_t M,
                                                  uint32_t K, uint32_t G) {
  const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= M * G) return;
  const uint32_t m = idx / G, g = idx % G;
  const h8* src = reinterpret_cast<const h8*>(in + (size_t)m * K + (size_t)g * 64);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const h8 v = src[j];
#pragma unroll
    for (int i = 0; i < 8; i++) s += (float)v[i];
  }
  const _Float16 hi = (_Float16)s;
  const _Float16 lo = (_Float16)(s - (float)hi);
  xs16[(size_t)m * 2 * G + g] = hi;
  xs16[(size_t)m * 2 * G + G + g] = lo;
}

template <int WM, int WN, bool AFFINE>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(const GemmParams p) {
  constexpr int THREADS = 64 * WM * WN;
  constexpr int TM = 64 * WM, TN = 64 * WN;
  constexpr int A_LOADS = TM * CHUNKS / THREADS;  // 16-byte loads per thread per step
  constexpr int W_WORDS = TN * 8 / THREADS;       // packed words per thread per step
  static_assert(A_LOADS >= 1 && (W_WORDS == 2 || W_WORDS == 4 || W_WORDS == 8), "tile/thread mismatch");
  constexpr int W_TPR = 8 / W_WORDS;              // threads per weight row
  constexpr int SCALES = AFFINE ? 1 : 2;          // groups per step
  constexpr int SC_LOADS = (TN * SCALES + THREADS - 1) / THREADS;

  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int STAGE_CHUNKS = (TM + TN) * CHUNKS;
  h8* lds = reinterpret_cast<h8*>(smem);                                         // [2][STAGE_CHUNKS]
  float* lds_s = reinterpret_cast<float*>(smem + 2 * STAGE_CHUNKS * 16);         // [2][TN][SCALES]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t wm = wave / WN, wn = wave % WN;

  // workgroup id -> tile: ids sharing an XCD (id % 8) take consecutive tiles,
  // and consecutive tiles walk m fastest, i.e. share a weight panel
  uint32_t id = blockIdx.x;
  const uint32_t total = p.mtiles * p.ntiles;
  if (p.xcd_swizzle && total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const uint32_t mt = id % p.mtiles, nt = id / p.mtiles;
  const uint32_t m0 = mt * TM, n0 = nt * TN;

  uint32_t c_mixed;  // OR constant: 64 in the high half, 1024 in the low half
  asm volatile("v_mov_b32 %0, 0x54006400" : "=v"(c_mixed));

  u32x4 areg[A_LOADS];
  uint32_t wreg[W_WORDS];
  _Float16 sreg[SC_LOADS];
  const uint32_t total_steps = p.nsteps + p.bias_steps;
  const uint32_t G = p.spr;

  const uint32_t w_row = tid / W_TPR, w_part = tid % W_TPR;  // this thread's weight row and word group
  uint32_t w_n = n0 + w_row;
  w_n = w_n < p.N ? w_n : p.N - 1;  // clamped rows are never stored

  // step < nsteps: activations + packed weights of k = 64*step ..
  // step >= nsteps (affine only): group sums + biases, 64 columns of [hi | lo] per step
  auto load_step = [&](uint32_t step) {
    if (step < p.nsteps) {
      const uint32_t k0 = step * KS;
#pragma unroll
      for (int i = 0; i < A_LOADS; i++) {
        const uint32_t c = tid + i * THREADS, row = c / CHUNKS, ch = c % CHUNKS;
        const uint32_t m = m0 + row;
        u32x4 v = {0, 0, 0, 0};
        if (m < p.M) v = *reinterpret_cast<const u32x4*>(p.in + (size_t)m * p.K + k0 + ch * 8);
        areg[i] = v;
      }
      const uint32_t* wp = p.weights + (size_t)w_n * p.k_packed + (k0 >> 3) + w_part * W_WORDS;
      if (W_WORDS == 2) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(wp);
        wreg[0] = v.x; wreg[1] = v.y;
      } else {
#pragma unroll
        for (int q4 = 0; q4 < W_WORDS / 4; q4++) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(wp + 4 * q4);
          wreg[4 * q4 + 0] = v.x; wreg[4 * q4 + 1] = v.y; wreg[4 * q4 + 2] = v.z; wreg[4 * q4 + 3] = v.w;
        }
      }
#pragma unroll
      for (int i = 0; i < SC_LOADS; i++) {
        const uint32_t idx = tid + i * THREADS;
        if (idx < TN * SCALES) {
          uint32_t n = n0 + idx / SCALES;
          n = n < p.N ? n : p.N - 1;
          sreg[i] = p.scales[(size_t)n * p.spr + step * SCALES + idx % SCALES];
        }
      }
    } else {
      const uint32_t c0 = (step - p.nsteps) * KS;  // column of the [hi | lo] matrix
#pragma unroll
      for (int i = 0; i < A_LOADS; i++) {
        const uint32_t c = tid + i * THREADS, row = c / CHUNKS, ch = c % CHUNKS;
        const uint32_t m = m0 + row, col = c0 + ch * 8;
        u32x4 v = {0, 0, 0, 0};
        if (m < p.M && col < 2 * G) {
          const _Float16* src = p.xs16 + (size_t)m * 2 * G + col;
          if (G % 4 == 0) {
            v = *reinterpret_cast<const u32x4*>(src);
          } else {  // narrow K: rows of the [hi | lo] matrix are not 16-byte multiples
            h8 t = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (col + e < 2 * G) t[e] = src[e];
            v = __builtin_bit_cast(u32x4, t);
          }
        }
        areg[i] = v;
      }
      // biases: column c of the B matrix is b[n][c mod G]; W_WORDS chunks of 8 columns per thread
#pragma unroll
      for (int j = 0; j < W_WORDS; j++) wreg[j] = 0;  // unused in this phase
    }
  };

  auto store_step = [&](uint32_t step, uint32_t buf) {
    h8* a_lds = lds + buf * STAGE_CHUNKS;
    h8* w_lds = a_lds + TM * CHUNKS;
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      const uint32_t c = tid + i * THREADS, row = c / CHUNKS, ch = c % CHUNKS;
      a_lds[row * CHUNKS + (ch ^ (row & 7u))] = __builtin_bit_cast(h8, areg[i]);
    }
    if (step < p.nsteps) {
#pragma unroll
      for (int j = 0; j < W_WORDS; j++) {
        const uint32_t ch = w_part * W_WORDS + j;
        w_lds[w_row * CHUNKS + (ch ^ (w_row & 7u))] = unpack_word_natural<AFFINE>(wreg[j], c_mixed);
      }
#pragma unroll
      for (int i = 0; i < SC_LOADS; i++) {
        const uint32_t idx = tid + i * THREADS;
        if (idx < TN * SCALES) lds_s[buf * TN * SCALES + idx] = (float)sreg[i];
      }
    } else {
      const uint32_t c0 = (step - p.nsteps) * KS;
#pragma unroll
      for (int j = 0; j < W_WORDS; j++) {
        const uint32_t ch = w_part * W_WORDS + j, col = c0 + ch * 8;
        h8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (col < 2 * G) {
          const _Float16* brow = p.biases + (size_t)w_n * G;
          if (G % 8 == 0) {
            v = *reinterpret_cast<const h8*>(brow + (col % G));
          } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (col + e < 2 * G) v[e] = brow[(col + e) % G];
          }
        }
        w_lds[w_row * CHUNKS + (ch ^ (w_row & 7u))] = v;
      }
    }
  };

  f16v tot[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) tot[i][j][e] = 0.f;

  load_step(0);
  store_step(0, 0);
  __syncthreads();

  const uint32_t frow = lane & 31u, fk = lane >> 5;  // operand row inside a 32-block, which 8 of the 16 k
  const f16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  for (uint32_t step = 0; step < total_steps; step++) {
    const uint32_t buf = step & 1u;
    if (step + 1 < total_steps) load_step(step + 1);

    const h8* a_lds = lds + buf * STAGE_CHUNKS;
    const h8* w_lds = a_lds + TM * CHUNKS;
    const bool main_phase = step < p.nsteps;

    // PH phases of KS/PH k each; each phase ends with one scale-and-fold
    constexpr int PH = AFFINE ? 1 : 2;
#pragma unroll
    for (int ph = 0; ph < PH; ph++) {
      f16v part[2][2];
#pragma unroll
      for (int ks = 0; ks < KS / 16 / PH; ks++) {
        const uint32_t ch = (ph * (KS / 16 / PH) + ks) * 2 + fk;
        h8 af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
          const uint32_t row = wm * 64 + i * 32 + frow;
          af[i] = a_lds[row * CHUNKS + (ch ^ (row & 7u))];
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const uint32_t row = wn * 64 + j * 32 + frow;
          bf[j] = w_lds[row * CHUNKS + (ch ^ (row & 7u))];
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            part[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], ks == 0 ? zero : part[i][j], 0, 0, 0);
      }
      // fold: the lane's column n is fixed per block column j, so one scale per j
      float sc[2];
#pragma unroll
      for (int j = 0; j < 2; j++) sc[j] = main_phase ? lds_s[(buf * TN + wn * 64 + j * 32 + frow) * SCALES + ph] : 1.f;
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
          for (int e = 0; e < 16; e++) tot[i][j][e] = __builtin_fmaf(sc[j], part[i][j][e], tot[i][j][e]);
    }

    if (step + 1 < total_steps) store_step(step + 1, buf ^ 1u);
    __syncthreads();
  }

  // D layout of a 32x32 block: lane -> column n = lane % 32, register e -> row 8*(e/4) + 4*(lane/32) + e%4
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t n = n0 + wn * 64 + j * 32 + (lane & 31u);
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const uint32_t m = m0 + wm * 64 + i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
        if (m < p.M && n < p.N) p.out[(size_t)m * p.N + n] = (_Float16)tot[i][j][e];
      }
    }
}

template <int WM, int WN>
hipError_t launch_tile(GemmParams p, bool affine, hipStream_t s) {
  constexpr int TM = 64 * WM, TN = 64 * WN, THREADS = 64 * WM * WN;
  p.mtiles = (p.M + TM - 1) / TM;
  p.ntiles = (p.N + TN - 1) / TN;
  const dim3 grid(p.mtiles * p.ntiles);
  const size_t smem = 2 * (size_t)(TM + TN) * CHUNKS * 16 + 2 * (size_t)TN * 2 * sizeof(float);
  if (affine) {
    auto k = gemm_kernel<WM, WN, true>;
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(THREADS), smem, s, p);
  } else {
    auto k = gemm_kernel<WM, WN, false>;
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(THREADS), smem, s, p);
  }
  return hipGetLastError();
}

}  // namespace

// 4-bit, f16 output, dense, K a multiple of 64.
bool gemm_supports(const MatmulArgs& a) { return a.slots == 0 && a.bits == 4 && !a.out_f32 && a.K % KS == 0; }

size_t gemm_scratch_bytes(const MatmulArgs& a) { return a.affine ? (size_t)a.M * 2 * a.spr * sizeof(_Float16) : 0; }

hipError_t launch_gemm(const MatmulArgs& a, const Tune& t, void* scratch, hipStream_t s) {
  GemmParams p{};
  p.out = reinterpret_cast<_Float16*>(a.out);
  p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases;
  p.xs16 = reinterpret_cast<const _Float16*>(scratch);
  p.M = a.M; p.N = a.N; p.K = a.K; p.k_packed = a.k_packed; p.spr = a.spr;
  p.nsteps = a.K / KS;
  p.bias_steps = a.affine ? (2 * a.spr + KS - 1) / KS : 0;
  p.xcd_swizzle = t.gemm_xcd_swizzle;
  if (a.affine) {
    const uint32_t n = a.M * a.spr;
    hipLaunchKernelGGL(xsum_kernel, dim3((n + 255) / 256), dim3(256), 0, s, a.in, reinterpret_cast<_Float16*>(scratch), a.M, a.K, a.spr);
  }
  int tile = t.gemm_tile;
  if (!tile) tile = a.M > 256 ? 3 : (a.M > 64 ? 2 : 1);  // measured: 256x128 wins from M=512 up
  switch (tile) {
    case 3: return launch_tile<4, 2>(p, a.affine, s);  // 256 x 128, 8 waves
    case 2: return launch_tile<2, 2>(p, a.affine, s);  // 128 x 128, 4 waves
    case 4: return launch_tile<2, 4>(p, a.affine, s);  // 128 x 256, 8 waves
    default: return launch_tile<1, 2>(p, a.affine, s);  // 64 x 128, 2 waves
  }
}

}  // namespace ztvm
