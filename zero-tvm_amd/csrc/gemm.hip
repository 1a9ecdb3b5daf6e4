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
// 8-bit affine rows (the reference's int8_affine_batched pipeline, compiler.ts:429-430) and 3-bit
// affine rows (the q3 bitstream, int4_matmul.gen.ts:409-448) run through the same kernel: only the
// staging of the weight tile differs (two packed words, or a 24-bit window, per 16-byte chunk).
//
// Tiling
//   workgroup  WM x WN waves, each wave a 64 x 64 output tile (2 x 2 blocks of
//              v_mfma_f32_32x32x16_f16); A operand = activations, B operand =
//              weights, so lanes of D run along n and stores are contiguous
//   K step     64 = one affine group (two symmetric groups), three LDS stages
//   LDS rows   64 f16 = eight 16-byte chunks, chunk index XOR bits 1..3 of the
//              row: the 16 lanes served together by a 128-bit read cover all
//              64 banks (measured 560 B/ns per CU, same as a linear read)
//   pipeline   step s multiplies stage s%3; the activations of step s+2 go
//              global -> LDS without passing registers, the packed weights of
//              step s+2 are unpacked from registers into the same stage, the
//              fragments of step s+1 are read while those of step s retire,
//              and the previous run's partial sums are folded between MFMAs;
//              one barrier per step. Every matrix instruction is followed by
//              its share of that other work (about seven vector instructions
//              fit in the 32 cycles one of them occupies the matrix core)
//   scales     fetched six steps at a time, global -> LDS like the activations,
//              into a two-batch ring, as stored (f16)
//   grid       one workgroup per tile, ids remapped so that the tiles sharing
//              a weight panel run on the same XCD (same L2)
#include "internal.h"
#include "quant.h"
#include <utility>

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
  const _Float16* xs16;  // [M][xs_stride]: hi halves, lo halves of the group sums, zero padding
  float* partial;        // k split: [split tile][part][TM * TN] f32 totals, in the accumulators' own layout
  uint32_t* counters;    // k split: arrivals per split tile; zero between launches
  uint32_t M, N, K, k_packed, spr;
  uint32_t mtiles, ntiles, nsteps, bias_steps, xs_stride;
  uint32_t xcd_swizzle;
  uint32_t full_tiles, parts, steps_per_part;  // tiles [0, full_tiles) run whole; the others are dealt to `parts` workgroups
};

// LDS swizzle: a 128-bit read serves 16 lanes per cycle = two 128-byte rows of banks, and rows of
// equal parity share a bank half, so the chunk index is XOR-ed with bits 1..3 of the row.
__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row >> 1) & 7u; }

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

// Two words of four bytes each -> eight exact f16 integers in natural k order: 0x6400 | byte is 1024 + byte, the
// low halves of the two masked views are (v0, v1), the high halves (v2, v3).
__device__ __forceinline__ h8 unpack_bytes_natural(uint32_t w0, uint32_t w1, uint32_t c_1024) {
  const h2 off = {(_Float16)1024.f, (_Float16)1024.f};
  h2 q[4];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const uint32_t w = i ? w1 : w0;
    const uint32_t even = and_or(w, 0x00FF00FFu, c_1024);       // v0 | v2
    const uint32_t odd = and_or(w >> 8, 0x00FF00FFu, c_1024);   // v1 | v3
    q[2 * i + 0] = as_h2(__builtin_amdgcn_perm(odd, even, 0x05040100u)) - off;  // v0, v1
    q[2 * i + 1] = as_h2(__builtin_amdgcn_perm(odd, even, 0x07060302u)) - off;  // v2, v3
  }
  return (h8){q[0].x, q[0].y, q[1].x, q[1].y, q[2].x, q[2].y, q[3].x, q[3].y};
}

// A window of eight 3-bit values (value i at bits [3i, 3i+3); bits from 24 up may hold anything) -> eight exact f16
// integers in natural k order: the shared unpack returns the pairs (v0,v4) (v1,v5) (v2,v6) (v3,v7).
__device__ __forceinline__ h8 unpack_q3_natural(uint32_t win, const UnpackConsts& uc) {
  h2 q[4];
  unpack3_views(win << 4, win >> 2, q, uc);
  return (h8){q[0].x, q[1].x, q[2].x, q[3].x, q[0].y, q[1].y, q[2].y, q[3].y};
}

// Group sums of the activations, one row of xs_stride f16 per activation row:
// xs16[m][g] = f16(xs), xs16[m][G+g] = f16(xs - hi), zero from 2G up to the stride.
// One thread per 16-byte chunk, eight consecutive lanes = one 64-k group, summed across lanes.
__global__ __launch_bounds__(256) void xsum_kernel(const _Float16* __restrict__ in, _Float16* __restrict__ xs16, uint32_t M,
                                                  uint32_t K, uint32_t G, uint32_t xs_stride) {
  const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
  const uint32_t cpr = K / 8, total = M * cpr;  // chunks per row; K % 64 == 0, so groups never straddle a wave
  const uint32_t pad = xs_stride - 2 * G;
  if (idx < M * pad) xs16[(size_t)(idx / pad) * xs_stride + 2 * G + idx % pad] = (_Float16)0.f;
  if (idx >= total) return;
  const uint32_t m = idx / cpr, c = idx % cpr;
  const h8 v = *reinterpret_cast<const h8*>(in + (size_t)m * K + (size_t)c * 8);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) s += (float)v[i];
  s += __shfl_xor(s, 1);
  s += __shfl_xor(s, 2);
  s += __shfl_xor(s, 4);
  if ((c & 7u) == 0) {
    const uint32_t g = c >> 3;
    const _Float16 hi = (_Float16)s;
    xs16[(size_t)m * xs_stride + g] = hi;
    xs16[(size_t)m * xs_stride + G + g] = (_Float16)(s - (float)hi);
  }
}

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

constexpr int NSTAGE = 3;
// The value, made opaque to the compiler: what is computed from it inside the loop stays there
// instead of being hoisted into a register that lives through the loop (the 256 x 128 tile runs
// at the register limit, and a reload from scratch in the loop waits for every fetch in flight).
__device__ __forceinline__ uint32_t opaque(uint32_t x) {
  asm volatile("" : "+v"(x));
  return x;
}
constexpr int SCB = 6;  // steps per batch of scales: two turns of the three LDS stages, so the hot loop has no branch

// 16 bytes per lane from global memory (uniform base + 32-bit lane offset) straight into LDS slot
// lds + 16 * lane. Written as assembly: the compiler's wait-count pass treats the builtin as an
// access to both vector memory and LDS, and while one is pending it turns every later LDS wait
// into a full drain. The loads are counted by vmcnt like any other; the kernel waits for them
// itself (vmcnt(0) before the barrier that ends a step). M0 carries the LDS address; nothing
// else in these kernels uses M0.
__device__ __forceinline__ void dma16(const void* base_uniform, uint32_t off, uint32_t lds_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base_uniform), "s"(lds_uniform)
               : "memory", "m0");
}
// The same with 4 bytes per lane: LDS slot lds + 4 * lane.
__device__ __forceinline__ void dma4(const void* base_uniform, uint32_t off, uint32_t lds_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base_uniform), "s"(lds_uniform) : "memory", "m0");
}

// Work that shares a step with the 16 matrix instructions, by half-slot hs = 2 * pair + (0 after
// the first MFMA of the pair, 1 after the second). The thread's packed words are unpacked in the
// first eight half-slots, evenly spaced; the 32 fold FMAs of a run are spread over the run's
// half-slots that have no unpack (over all of them when every one has).
template <int W_CH>
constexpr bool has_unpack(int hs) { return hs < 8 && hs % (8 / W_CH) == 0; }
template <int W_CH, int RUNH>
constexpr int fold_upto(int hs) {  // FMAs of the run done before half-slot hs
  const int r0 = hs / RUNH * RUNH;
  int total = 0;
  for (int k = r0; k < r0 + RUNH; k++) total += has_unpack<W_CH>(k) ? 0 : 1;
  const bool flat = total == 0;
  if (flat) total = RUNH;
  int before = 0;
  for (int k = r0; k < hs; k++) before += flat ? 1 : (has_unpack<W_CH>(k) ? 0 : 1);
  return 32 * before / total;
}

// The 16 MFMAs of a step as 8 pairs (block row i, k slice ks) x 2 block columns. A run of pairs
// accumulates one group into one partial set (set = i); affine: 64-k groups, runs of 4 pairs;
// symmetric: 32-k groups, runs of 2 pairs.
template <bool AFFINE>
struct Seq {
  static constexpr int RUN = AFFINE ? 4 : 2;
  static constexpr int I(int p) { return AFFINE ? p / 4 : (p / 2) % 2; }
  static constexpr int KSL(int p) { return AFFINE ? p % 4 : (p / 4) * 2 + p % 2; }
  static constexpr int GRP(int p) { return AFFINE ? 0 : p / 4; }
};

template <int WM, int WN, bool AFFINE, int BITS, bool SPLIT>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(const GemmParams p) {
  static_assert(BITS == 4 || ((BITS == 8 || BITS == 3) && AFFINE), "4-bit affine or symmetric, 8-bit and 3-bit affine");
  using S = Seq<AFFINE>;
  constexpr int WAVES = WM * WN, THREADS = 64 * WAVES;
  constexpr int TM = 64 * WM, TN = 64 * WN;
  constexpr int A_LOADS = TM * CHUNKS / THREADS;  // 16-byte direct-to-LDS loads per lane per step
  constexpr int W_CH = TN * 8 / THREADS;          // 8-k chunks (16 bytes of f16 in LDS) per thread per step
  // words fetched per thread and step: one (4-bit) or two (8-bit) per chunk; 3-bit chunks are 3 bytes of the row's
  // bitstream, so a thread's 3 * W_CH bytes are fetched as the dwords that cover them
  constexpr int W_WORDS = BITS == 3 ? (W_CH == 2 ? 2 : 3 * W_CH / 4) : W_CH * BITS / 4;
  static_assert(A_LOADS >= 1 && (W_CH == 2 || W_CH == 4 || W_CH == 8), "tile/thread mismatch");
  constexpr int W_TPR = 8 / W_CH;                 // threads per weight row
  constexpr int SCALES = AFFINE ? 1 : 2;          // groups per step
  constexpr uint32_t ROW_BYTES = CHUNKS * 16;
  constexpr uint32_t STAGE_BYTES = (TM + TN) * ROW_BYTES;
  constexpr uint32_t W_BASE = TM * ROW_BYTES;          // weight rows follow the activation rows of a stage
  constexpr uint32_t SC_BASE = NSTAGE * STAGE_BYTES;   // f16 [2 batches][SC_PAIRS][TN][2]
  constexpr int SC_PAIRS = SCB * SCALES / 2;           // 4-byte pairs per column per batch
  constexpr uint32_t SC_BATCH = SC_PAIRS * TN * 4;
  static_assert(TN % 64 == 0 && TN <= THREADS, "whole waves load the scales");

  extern __shared__ __align__(16) unsigned char smem[];

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)smem;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / WN, wn = wave % WN;

  // workgroup id -> tile: ids sharing an XCD (id % 8) take consecutive tiles,
  // and consecutive tiles walk m fastest, i.e. share a weight panel
  // Tiles past full_tiles (the last, partly filled round of workgroups, or every tile when there are few) are
  // split along k: `parts` workgroups take consecutive step ranges of one tile and the last of them to arrive adds
  // the parts' f32 totals in part order, so a tile's result does not depend on who arrives when.
  // (the split tiles run as a launch of their own, SPLIT, after the whole ones)
  uint32_t id = blockIdx.x, kpart = 0;
  if (SPLIT) {
    id = p.full_tiles + blockIdx.x / p.parts;
    kpart = blockIdx.x % p.parts;
  } else if (p.xcd_swizzle && p.full_tiles % 8 == 0) {
    id = (id % 8) * (p.full_tiles / 8) + id / 8;
  }
  const uint32_t mt = id % p.mtiles, nt = id / p.mtiles;
  const uint32_t m0 = mt * TM, n0 = nt * TN;
  const uint32_t k0 = SPLIT ? kpart * p.steps_per_part : 0;                                            // first step
  const uint32_t nsteps = SPLIT ? (p.nsteps - k0 < p.steps_per_part ? p.nsteps - k0 : p.steps_per_part) : p.nsteps;

  UnpackConsts uc3;  // 3-bit: the two OR constants of the shared unpack
  if (BITS == 3) {
    asm volatile("v_mov_b32 %0, 0x64005400" : "=v"(uc3.c3_a));
    asm volatile("v_mov_b32 %0, 0x58004800" : "=v"(uc3.c3_b));
  }
  uint32_t c_mixed;  // OR constant: 4-bit: 64 in the high half, 1024 in the low half; 8-bit: 1024 in both
  if (BITS == 4) asm volatile("v_mov_b32 %0, 0x54006400" : "=v"(c_mixed));
  else asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(c_mixed));

  // ---- activations: global -> LDS without passing registers. One instruction fills 64
  // consecutive 16-byte LDS slots (8 rows), slot = lane; the lane fetches the chunk that the
  // swizzle places there. Rows past M repeat row M-1: they are computed and never stored.
  // Instruction i of a wave fills the eight tile rows of group i * WAVES + wave. A group reaching
  // past row M is moved back to end at row M - 1 (with M < 8: to row 0, and the lanes clamp), so
  // that one lane offset serves every group and the group's base stays uniform. Its tile rows
  // then repeat rows of the group before; the stores at the end use the same mapping.
  static_assert(WAVES % 2 == 0, "the swizzle of a lane's row must not depend on the instruction");
  const uint32_t lrow = lane >> 3;
  const uint32_t a_ch = (lane & 7u) ^ swz(wave * 8 + lrow);
  const uint32_t lrow_c = lrow < p.M ? lrow : p.M - 1;
  const uint32_t a_lane = (lrow_c * p.K + a_ch * 8) * 2u;
  const uint32_t xs_lane = (lrow_c * p.xs_stride + a_ch * 8) * 2u;
  uint32_t a_row0[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) {
    const uint32_t row0 = m0 + (i * WAVES + wave) * 8, last = p.M >= 8 ? p.M - 8 : 0;
    a_row0[i] = row0 < last ? row0 : last;
  }
  const _Float16* a_base[A_LOADS];  // uniform; move one k step per fill
#pragma unroll
  for (int i = 0; i < A_LOADS; i++) a_base[i] = p.in + (size_t)a_row0[i] * p.K + (size_t)k0 * KS;
  auto lds_slot = [&](uint32_t stage, int i) __attribute__((always_inline)) { return lds0 + stage * STAGE_BYTES + (i * WAVES + wave) * 1024u; };

  // ---- weights: registers, unpack, LDS
  const uint32_t w_row = tid / W_TPR, w_part = tid % W_TPR;
  uint32_t w_n = n0 + w_row;
  w_n = w_n < p.N ? w_n : p.N - 1;  // clamped rows are never stored
  // one descriptor + 32-bit lane offset + uniform step offset: no address arithmetic in the loop
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(p.weights), 0, p.N * p.k_packed * 4u, 0x00020000);
  const uint32_t w_byte = w_n * p.k_packed * 4u + w_part * (W_CH * BITS);  // W_CH chunks of BITS bytes each
  const uint32_t w_off = w_byte & ~3u;
  // (w_byte & 3) is nonzero only for 3-bit rows with two chunks (six bytes) per thread: 2 for odd w_part
  uint32_t w_adv = k0 * (KS * BITS / 8);  // uniform, bytes
  uint32_t w_dst[W_CH];
#pragma unroll
  for (int j = 0; j < W_CH; j++) w_dst[j] = W_BASE + w_row * ROW_BYTES + (((w_part * W_CH + j) ^ swz(w_row)) << 4);

  struct WRegs {
    uint32_t w[W_WORDS];
  };
  auto load_w = [&](WRegs& r) __attribute__((always_inline)) {
    if (W_WORDS == 2) {
      const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(wres, w_off, w_adv, 0);
      r.w[0] = v.x; r.w[1] = v.y;
    } else if (BITS == 3) {
#pragma unroll
      for (int q3 = 0; q3 < W_WORDS / 3; q3++) {
        const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(wres, w_off + 12 * q3, w_adv, 0);
        r.w[3 * q3 + 0] = v.x; r.w[3 * q3 + 1] = v.y; r.w[3 * q3 + 2] = v.z;
      }
    } else {
#pragma unroll
      for (int q4 = 0; q4 < W_WORDS / 4; q4++) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(wres, w_off + 16 * q4, w_adv, 0);
        r.w[4 * q4 + 0] = v.x; r.w[4 * q4 + 1] = v.y; r.w[4 * q4 + 2] = v.z; r.w[4 * q4 + 3] = v.w;
      }
    }
    w_adv += KS * BITS / 8;  // bytes of a row per step
  };
  auto store_w_words = [&](const WRegs& r, uint32_t stage, int j0, int j1) __attribute__((always_inline)) {
#pragma unroll
    for (int j = j0; j < j1; j++) {  // chunk j of the thread: one 4-bit word or two 8-bit words
      h8 v;
      if constexpr (BITS == 4) {
        v = unpack_word_natural<AFFINE>(r.w[j], c_mixed);
      } else if constexpr (BITS == 8) {
        v = unpack_bytes_natural(r.w[2 * j], r.w[2 * j + 1], c_mixed);
      } else {
        // chunk j of the thread is the 24-bit window at bit 24 * j of its bytes: four windows per three dwords
        const int g = j / 4 * 3, jj = j % 4;
        uint32_t d0 = r.w[g], d1 = r.w[g + 1], d2 = W_CH == 2 ? 0u : r.w[W_CH == 2 ? g : g + 2];
        if (W_CH == 2) {  // the thread's six bytes start at bit 0 (even w_part = even lane) or 16 of its two dwords
          const uint32_t w_sh = (opaque(lane) & 1u) << 4;  // recomputed here: the kernel is at the register limit
          d0 = __builtin_amdgcn_alignbit(d1, d0, w_sh);
          d1 = d1 >> w_sh;
        }
        const uint32_t win = jj == 0 ? d0 : jj == 1 ? __builtin_amdgcn_alignbit(d1, d0, 24) : jj == 2 ? __builtin_amdgcn_alignbit(d2, d1, 16) : d2 >> 8;
        v = unpack_q3_natural(win, uc3);
      }
      *reinterpret_cast<h8*>(smem + stage * STAGE_BYTES + w_dst[j]) = v;
    }
  };

  // ---- scales: the first TN / 64 waves fetch SCB steps of their 64 columns at a time, one pair
  // of f16 (4 bytes) per lane and instruction, into batch slot (batch & 1) of the ring, laid out
  // [pair][column]. Pairs past a row's end repeat the row's last pair and are never used.
  const bool sc_loader = wave < TN / 64;
  auto load_sc = [&](uint32_t batch) __attribute__((always_inline)) {
    uint32_t sc_n = n0 + wave * 64 + opaque(lane);
    sc_n = sc_n < p.N ? sc_n : p.N - 1;
    const uint32_t sc_off = sc_n * p.spr * 2u;  // spr is even (checked on the host): rows start on 4 bytes
#pragma unroll
    for (int k = 0; k < SC_PAIRS; k++) {
      uint32_t e = k0 * SCALES + batch * (SCB * SCALES) + 2 * k;  // k0 is even: pairs stay aligned
      e = e < p.spr - 2 ? e : p.spr - 2;
      dma4(p.scales, sc_off + e * 2u, lds0 + SC_BASE + (batch & 1u) * SC_BATCH + k * (TN * 4) + wave * 256u);
    }
  };

  // ---- operand fragments: lane -> row frow of a 32-row block, k slice fk of the 16
  const uint32_t frow = lane & 31u, fk = lane >> 5;
  uint32_t a_rd[KS / 16], b_rd[KS / 16];
#pragma unroll
  for (int ks = 0; ks < KS / 16; ks++) {
    const uint32_t x = frow * ROW_BYTES + (((ks * 2 + fk) ^ swz(frow)) << 4);
    a_rd[ks] = x + wm * 64 * ROW_BYTES;
    b_rd[ks] = x + W_BASE + wn * 64 * ROW_BYTES;
  }
  // With a stage known at compile time the stage and block offsets fold into the instruction; the steps outside
  // the hot loop pass a runtime stage and add it to the same address registers (opaque, so that the compiler does
  // not rebuild the addresses from parts it would have to carry through the hot loop).
  auto read_a = [&](uint32_t stage, int i, int ks) __attribute__((always_inline)) {
    if (__builtin_constant_p(stage)) return *reinterpret_cast<const h8*>(smem + stage * STAGE_BYTES + a_rd[ks] + i * 32 * ROW_BYTES);
    return *reinterpret_cast<const h8*>(smem + (opaque(a_rd[ks]) + stage * STAGE_BYTES) + i * 32 * ROW_BYTES);
  };
  auto read_b = [&](uint32_t stage, int j, int ks) __attribute__((always_inline)) {
    if (__builtin_constant_p(stage)) return *reinterpret_cast<const h8*>(smem + stage * STAGE_BYTES + b_rd[ks] + j * 32 * ROW_BYTES);
    return *reinterpret_cast<const h8*>(smem + (opaque(b_rd[ks]) + stage * STAGE_BYTES) + j * 32 * ROW_BYTES);
  };

  f16v tot[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) tot[i][j][e] = 0.f;
  const f16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  f16v part_sum[2][2];  // k split: the sum of the parts, built in part order at the end

  // ---- the pipeline's first fetches go out before anything else: the activations of steps 0 and 1 into stages 0
  // and 1, the packed words of steps 0, 1 and 2 into registers, scale batch 0 into the ring. They land while the
  // bias term below is computed (through stage 2, which the pipeline does not touch before its first step).
  WRegs wcur, wnext, w_first;
  if (sc_loader) load_sc(0);
  auto load_a = [&](uint32_t stage) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < A_LOADS; i++) {
      dma16(a_base[i], a_lane, lds_slot(stage, i));
      a_base[i] += KS;
    }
  };
  load_a(0);
  load_w(w_first);
  if (nsteps > 1) {
    load_a(1);
    load_w(wnext);
  }
  if (nsteps > 2) load_w(wcur);

  // ---- bias term (affine): tot = [xs_hi | xs_lo] x biases on the matrix cores, 64 columns per step, through
  // stage 2 (two or three short steps).
  if (AFFINE && (!SPLIT || kpart == 0)) {
    const uint32_t G = p.spr;
    const _Float16* brow = p.biases + (size_t)w_n * G;
    for (uint32_t bs = 0; bs < p.bias_steps; bs++) {
#pragma unroll
      for (int i = 0; i < A_LOADS; i++) dma16(p.xs16 + (size_t)a_row0[i] * p.xs_stride + bs * KS, xs_lane, lds_slot(2, i));
#pragma unroll
      for (int j = 0; j < W_CH; j++) {
        const uint32_t col = bs * KS + (w_part * W_CH + j) * 8;  // column c meets b[n][c mod G]; zero past 2G
        h8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (col < 2 * G) {
          if (G % 8 == 0) {
            v = *reinterpret_cast<const h8*>(brow + (col % G));
          } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (col + e < 2 * G) v[e] = brow[(col + e) % G];
          }
        }
        *reinterpret_cast<h8*>(smem + 2 * STAGE_BYTES + w_dst[j]) = v;
      }
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < KS / 16; ks++) {
        h8 af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; i++) af[i] = read_a(2, i, ks);
#pragma unroll
        for (int j = 0; j < 2; j++) bf[j] = read_b(2, j, ks);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++) tot[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], tot[i][j], 0, 0, 0);
      }
      __syncthreads();
    }
  }

  // ---- main loop, software pipelined over three LDS stages. Step s multiplies stage s%3 while
  //   * the activations of step s+2 stream into stage (s+2)%3 (issued at the top of step s),
  //   * the packed weights of step s+2 (in registers since step s-1) are unpacked into it,
  //   * the packed weights of step s+3 are fetched into registers,
  //   * the operand fragments of step s+1 are read from stage (s+1)%3 as those of step s retire,
  //   * the partial sums of the previous run are folded into the totals between the MFMAs.
  h8 Bf[2][KS / 16], Aq[4];
  f16v part[2][2];
  float sc[SCALES][2], scp[2];  // scales of this step; of the last group of the previous step

  // stages 0 and 1 complete, weights of step 2 in registers, scale batch 0 in the ring
  __builtin_amdgcn_s_waitcnt(0x0070);
  store_w_words(w_first, 0, 0, W_CH);
  if (nsteps > 1) store_w_words(wnext, 1, 0, W_CH);
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
  static_for<4>([&](auto pc) {
    constexpr int pp = decltype(pc)::value;
    Aq[pp] = read_a(0, S::I(pp), S::KSL(pp));
  });
#pragma unroll
  for (int ks = 0; ks < KS / 16; ks++)
#pragma unroll
    for (int j = 0; j < 2; j++) Bf[j][ks] = read_b(0, j, ks);
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) part[i][j] = zero;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    scp[j] = 0.f;
#pragma unroll
    for (int g = 0; g < SCALES; g++) sc[g][j] = 0.f;
  }

  // pos: place of the step in its batch of scales, batch: that batch, fetch_sc: fetch the next one
  auto step = [&](auto hot_c, uint32_t cur, uint32_t nxt, uint32_t fill, bool fetch_a, bool fetch_w, uint32_t pos, uint32_t batch,
                  bool fetch_sc) __attribute__((always_inline)) {
    constexpr bool HOT = decltype(hot_c)::value;
    constexpr int RUNH = 2 * S::RUN;
    if (HOT || fetch_w) load_w(wnext);
    // the next batch of scales is fetched in the first step of a batch (its ring slot was last
    // read a step ago) and first read six steps on
    if (fetch_sc && sc_loader) load_sc(batch + 1);
    {
      const uint32_t e = pos * SCALES;  // element of the batch: pair e / 2, half e % 2
      const uint32_t at = (opaque(lane) & 31u) * 4 + (SC_BASE + wn * 256 + (batch & 1u) * SC_BATCH + (e >> 1) * (TN * 4) + (e & 1u) * 2);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        scp[j] = sc[SCALES - 1][j];
#pragma unroll
        for (int g = 0; g < SCALES; g++) sc[g][j] = (float)*reinterpret_cast<const _Float16*>(smem + at + j * 32 * 4 + g * 2);
      }
    }
    static_for<8>([&](auto pc) {
      constexpr int pp = decltype(pc)::value;
      constexpr int i = S::I(pp), ks = S::KSL(pp);
      constexpr bool first = pp % S::RUN == 0;
      // the run that ended before this one is folded into the totals: tot += scale * part
      constexpr int prev = (pp - pp % S::RUN + 8 - S::RUN) % 8;  // first pair of the previous run
      constexpr int fi = S::I(prev), fg = S::GRP(prev);
      constexpr bool from_last_step = pp < S::RUN;
      auto fold = [&](auto hs_c) __attribute__((always_inline)) {
        constexpr int hs = decltype(hs_c)::value;
        constexpr int q0 = fold_upto<W_CH, RUNH>(hs), q1 = (hs + 1) % RUNH == 0 ? 32 : fold_upto<W_CH, RUNH>(hs + 1);
#pragma unroll
        for (int q = q0; q < q1; q++) {
          const int j = q / 16, e = q % 16;
          const float sv = from_last_step ? scp[j] : sc[fg][j];
          tot[fi][j][e] = __builtin_fmaf(sv, part[fi][j][e], tot[fi][j][e]);
        }
      };
      auto unpack = [&](auto hs_c) __attribute__((always_inline)) {
        constexpr int hs = decltype(hs_c)::value;
        if constexpr (has_unpack<W_CH>(hs)) {
          constexpr int j = hs / (8 / W_CH);
          if (HOT || fetch_a) store_w_words(wcur, fill, j, j + 1);
        }
      };
      using hs0 = std::integral_constant<int, 2 * pp>;
      using hs1 = std::integral_constant<int, 2 * pp + 1>;
      part[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Aq[pp % 4], Bf[0][ks], first ? zero : part[i][0], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // after block row 1 the weight fragments of this k slice are done: the next step's replace them
      if (i == 1) Bf[0][ks] = read_b(nxt, 0, ks);
      fold(hs0{});
      unpack(hs0{});
      __builtin_amdgcn_sched_barrier(0);
      part[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Aq[pp % 4], Bf[1][ks], first ? zero : part[i][1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // the activation fragment slot just used takes the pair four places on
      if (pp + 4 < 8) Aq[pp % 4] = read_a(cur, S::I(pp + 4), S::KSL(pp + 4));
      else Aq[pp % 4] = read_a(nxt, S::I(pp - 4), S::KSL(pp - 4));
      if (i == 1) Bf[1][ks] = read_b(nxt, 1, ks);
      fold(hs1{});
      unpack(hs1{});
      if (HOT || fetch_a) {
        constexpr int i0 = pp * A_LOADS / 4, i1 = (pp + 1) * A_LOADS / 4;  // spread over the first four pairs
#pragma unroll
        for (int ia = i0; ia < i1 && ia < A_LOADS; ia++) {
          dma16(a_base[ia], a_lane, lds_slot(fill, ia));
          a_base[ia] += KS;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    wcur = wnext;
    // everything this wave fetched or wrote has landed; the empty statements keep the compiler
    // from moving LDS accesses across the barrier
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  using hot_t = std::integral_constant<bool, true>;
  using cold_t = std::integral_constant<bool, false>;
  uint32_t s = 0, batch = 0;
  // hot: one batch of scales per turn; every step's s+3 is still a main step
  for (; s + SCB + 3 <= nsteps; s += SCB, batch++) {
    step(hot_t{}, 0, 1, 2, true, true, 0, batch, true);
    step(hot_t{}, 1, 2, 0, true, true, 1, batch, false);
    step(hot_t{}, 2, 0, 1, true, true, 2, batch, false);
    step(hot_t{}, 0, 1, 2, true, true, 3, batch, false);
    step(hot_t{}, 1, 2, 0, true, true, 4, batch, false);
    step(hot_t{}, 2, 0, 1, true, true, 5, batch, false);
  }
  for (uint32_t pos = 0; s < nsteps; s++) {
    step(cold_t{}, s % 3, (s + 1) % 3, (s + 2) % 3, s + 2 < nsteps, s + 3 < nsteps, pos, batch, pos == 0 && s + SCB < nsteps);
    if (++pos == SCB) pos = 0, batch++;
  }
  // the last run of the last step is still unfolded
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int e = 0; e < 16; e++) tot[1][j][e] = __builtin_fmaf(sc[SCALES - 1][j], part[1][j][e], tot[1][j][e]);

  // ---- k split: every part leaves its totals in memory (the accumulators' own layout: register r of lane l of wave
  // w at ((w * 64 + r) * 64 + l), so every store and load is a full 256-byte run), then counts itself in; the part
  // that finds all the others there adds the totals in part order (its own from registers, at its place in the
  // order) and stores the tile. Nobody waits for anybody. The counter is left at zero for the next launch.
  if constexpr (SPLIT) {
    // The totals and the counter travel with GPU-scope accesses (written through to memory, read past the caches
    // of this XCD), so no cache is flushed or invalidated under the workgroups that are still multiplying.
    const uint32_t st = id - p.full_tiles;
    uint32_t* mine = reinterpret_cast<uint32_t*>(p.partial) + ((size_t)st * p.parts + kpart) * (size_t)(TM * TN) + (size_t)wave * (64 * 64) + lane;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          const float v = tot[i][j][e];
          __hip_atomic_store(mine + ((i * 2 + j) * 16 + e) * 64, __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    __builtin_amdgcn_s_waitcnt(0x0070);  // every store of this wave has been acknowledged
    __syncthreads();                     // ... and of this workgroup: only then is the arrival counted
    volatile uint32_t* arrived = reinterpret_cast<volatile uint32_t*>(smem + SC_BASE);  // the scale ring is done with
    if (tid == 0) *arrived = __hip_atomic_fetch_add(p.counters + st, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*arrived != p.parts - 1) return;
    if (tid == 0) __hip_atomic_store(p.counters + st, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (uint32_t q = 0; q < p.parts; q++) {
      if (q == kpart) {  // uniform: its own totals come from the registers, at their place in the order
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) part_sum[i][j][e] = q == 0 ? tot[i][j][e] : part_sum[i][j][e] + tot[i][j][e];
      } else {
        const uint32_t* theirs = reinterpret_cast<const uint32_t*>(p.partial) + ((size_t)st * p.parts + q) * (size_t)(TM * TN) + (size_t)wave * (64 * 64) + lane;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
              const float v = __builtin_bit_cast(float, __hip_atomic_load(theirs + ((i * 2 + j) * 16 + e) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
              part_sum[i][j][e] = q == 0 ? v : part_sum[i][j][e] + v;
            }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) tot[i][j] = part_sum[i][j];
  }

  // D layout of a 32x32 block: lane -> column n = lane % 32, register e -> row 8*(e/4) + 4*(lane/32) + e%4.
  // Tile rows come in the groups of eight the activations were fetched in; a group moved back writes the values the
  // group before it writes, to the same places.
  const uint32_t ln = opaque(lane);
  const uint32_t last = p.M >= 8 ? p.M - 8 : 0;
  if (p.N % 8 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15u) == 0) {
    // The tile leaves as full rows: through LDS (the stages are done with), 16 bytes per lane. Stored from the
    // accumulator layout a lane writes 2 bytes and an instruction 64 bytes of each of two rows.
    constexpr uint32_t PITCH = TN * 2 + 16;  // the two rows an instruction writes fall into different banks
    static_assert((size_t)TM * PITCH <= NSTAGE * (size_t)STAGE_BYTES, "the output tile fits the stages");
    __builtin_amdgcn_s_waitcnt(0x0070);
    __syncthreads();  // every wave has read its last fragments
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          const uint32_t row = wm * 64 + i * 32 + 8 * (e / 4) + 4 * (ln >> 5) + (e % 4);
          *reinterpret_cast<_Float16*>(smem + row * PITCH + (wn * 64 + j * 32 + (ln & 31u)) * 2) = (_Float16)tot[i][j][e];
        }
    __syncthreads();
    for (uint32_t q = tid; q < TM * TN / 8; q += THREADS) {
      const uint32_t row = q / (TN / 8), c8 = q % (TN / 8);
      const uint32_t row0 = m0 + (row & ~7u), m = (row0 < last ? row0 : last) + (row & 7u), n = n0 + c8 * 8;
      if (row0 < p.M && m < p.M && n < p.N)
        *reinterpret_cast<u32x4*>(p.out + (size_t)m * p.N + n) = *reinterpret_cast<const u32x4*>(smem + row * PITCH + c8 * 16);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t n = n0 + wn * 64 + j * 32 + (ln & 31u);
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const uint32_t row0 = m0 + wm * 64 + i * 32 + 8 * (e / 4);
        const uint32_t m = (row0 < last ? row0 : last) + 4 * (ln >> 5) + (e % 4);
        if (row0 < p.M && m < p.M && n < p.N) p.out[(size_t)m * p.N + n] = (_Float16)tot[i][j][e];
      }
    }
}

template <int WM, int WN, bool AFFINE, int BITS>
hipError_t launch_kernel(const GemmParams& p, hipStream_t s) {
  constexpr int TM = 64 * WM, TN = 64 * WN, THREADS = 64 * WM * WN;
  // stages + scale ring
  const size_t smem = NSTAGE * (size_t)(TM + TN) * CHUNKS * 16 + 2 * (size_t)TN * SCB * (AFFINE ? 1 : 2) * sizeof(_Float16);
  // the whole tiles, then (a launch of their own, so that the common kernel carries nothing of the exchange) the split ones
  if (p.full_tiles) {
    auto k = gemm_kernel<WM, WN, AFFINE, BITS, false>;
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, dim3(p.full_tiles), dim3(THREADS), smem, s, p);
  }
  const uint32_t rest = p.mtiles * p.ntiles - p.full_tiles;
  if (rest) {
    auto k = gemm_kernel<WM, WN, AFFINE, BITS, true>;
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, dim3(rest * p.parts), dim3(THREADS), smem, s, p);
  }
  return hipGetLastError();
}

template <int WM, int WN>
hipError_t launch_tile(const GemmParams& p, bool affine, uint32_t bits, hipStream_t s) {
  if (bits == 8) return launch_kernel<WM, WN, true, 8>(p, s);
  if (bits == 3) return launch_kernel<WM, WN, true, 3>(p, s);
  if (affine) return launch_kernel<WM, WN, true, 4>(p, s);
  return launch_kernel<WM, WN, false, 4>(p, s);
}

// tile shape by number: rows x columns
void tile_dims(int tile, uint32_t* tm, uint32_t* tn) {
  *tm = tile == 3 ? 256 : (tile == 2 || tile == 4 ? 128 : 64);
  *tn = tile == 4 ? 256 : 128;
}
int tile_of(const MatmulArgs& a, const Tune& t) {
  if (t.gemm_tile >= 1 && t.gemm_tile <= 4) return t.gemm_tile;
  return a.M > 256 ? 3 : (a.M > 64 ? 2 : 1);  // measured: 256x128 wins from M=512 up
}

uint32_t xs_stride_of(const MatmulArgs& a) { return (2 * a.spr + KS - 1) / KS * KS; }
size_t xs_bytes_of(const MatmulArgs& a) { return a.affine ? ((size_t)a.M * xs_stride_of(a) * sizeof(_Float16) + 255) / 256 * 256 : 0; }

}  // namespace

// The k split of the tile GEMM. A grid of whole tiles leaves CUs idle where the tiles are few (N = 4096, M = 512:
// 64 tiles on 256 CUs) or where the last round of workgroups is mostly empty (M = 2048, N = 14336: 896 tiles =
// three and a half rounds). Those tiles (all of them, or the ones past the last full round) are dealt to `parts`
// workgroups each, along k, when that fills the round: parts = CUs / tiles, at most eight, never fewer than
// sixteen 64-k steps per part, and only where the f32 totals the parts exchange fit the scratch the caller has.
// A function of the descriptor, the CU count and that limit: a row's bits do not depend on timing.
GemmSplit gemm_split(const MatmulArgs& a, const Tune& t, size_t scratch_limit) {
  uint32_t tm, tn;
  tile_dims(tile_of(a, t), &tm, &tn);
  const uint32_t tiles = ((a.M + tm - 1) / tm) * ((a.N + tn - 1) / tn), cus = (uint32_t)(t.num_cus > 0 ? t.num_cus : 256);
  const uint32_t steps = a.K / KS;
  GemmSplit g{tiles, 1, steps, 0};
  if (t.gemm_split == 1) return g;
  const uint32_t rest = tiles % cus;
  if (rest == 0 || rest * 2 > cus) return g;
  uint32_t parts = cus / rest;
  if (parts > 8) parts = 8;
  while (parts > 1 && steps / parts < 16) parts--;
  if (parts < 2) return g;
  uint32_t per = ((steps + parts - 1) / parts + 1) & ~1u;  // even: the scale pairs of a part stay 4-byte aligned
  parts = (steps + per - 1) / per;
  if (parts < 2 || rest > ZTVM_GEMM_SPLIT_TILES) return g;
  const size_t bytes = (size_t)rest * parts * tm * tn * sizeof(float);
  if (scratch_limit && xs_bytes_of(a) + bytes > scratch_limit) return g;
  g.full_tiles = tiles - rest; g.parts = parts; g.steps_per_part = per; g.partial_bytes = bytes;
  return g;
}

// 4-bit (affine or symmetric), 8-bit or 3-bit affine, f16 output, dense, K a multiple of 64.
// The scales are fetched as 4-byte pairs, so a row of them must start on 4 bytes.
bool gemm_supports(const MatmulArgs& a) {
  return a.slots == 0 && (a.bits == 4 || ((a.bits == 8 || a.bits == 3) && a.affine)) && !a.out_f32 && a.K % KS == 0 && a.spr % 2 == 0;
}

size_t gemm_scratch_bytes(const MatmulArgs& a, const Tune& t, size_t scratch_limit) {
  return xs_bytes_of(a) + gemm_split(a, t, scratch_limit).partial_bytes;
}

// `counters`: ZTVM_GEMM_SPLIT_TILES zeroed words that belong to the caller's context (null: no k split)
hipError_t launch_gemm(const MatmulArgs& a, const Tune& t, void* scratch, uint32_t* counters, size_t scratch_limit, hipStream_t s) {
  GemmParams p{};
  p.out = reinterpret_cast<_Float16*>(a.out);
  p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases;
  p.xs16 = reinterpret_cast<const _Float16*>(scratch);
  p.M = a.M; p.N = a.N; p.K = a.K; p.k_packed = a.k_packed; p.spr = a.spr;
  p.nsteps = a.K / KS;
  p.xs_stride = xs_stride_of(a);
  p.bias_steps = a.affine ? p.xs_stride / KS : 0;
  p.xcd_swizzle = t.gemm_xcd_swizzle;
  Tune tt = t;
  if (!counters) tt.gemm_split = 1;
  const GemmSplit g = gemm_split(a, tt, scratch_limit);
  p.full_tiles = g.full_tiles; p.parts = g.parts; p.steps_per_part = g.steps_per_part;
  p.partial = reinterpret_cast<float*>(reinterpret_cast<char*>(scratch) + xs_bytes_of(a));
  p.counters = counters;
  if (a.affine) {
    const uint32_t pad = p.xs_stride - 2 * a.spr, cpr = a.K / 8;
    const uint32_t n = a.M * (cpr > pad ? cpr : pad);  // one thread per chunk, and enough for the padding columns
    hipLaunchKernelGGL(xsum_kernel, dim3((n + 255) / 256), dim3(256), 0, s, a.in, reinterpret_cast<_Float16*>(scratch), a.M, a.K, a.spr,
                       p.xs_stride);
  }
  const int tile = tile_of(a, t);
  uint32_t tm, tn;
  tile_dims(tile, &tm, &tn);
  p.mtiles = (a.M + tm - 1) / tm;
  p.ntiles = (a.N + tn - 1) / tn;
  switch (tile) {
    case 3: return launch_tile<4, 2>(p, a.affine, a.bits, s);  // 256 x 128, 8 waves
    case 2: return launch_tile<2, 2>(p, a.affine, a.bits, s);  // 128 x 128, 4 waves
    case 4: return launch_tile<2, 4>(p, a.affine, a.bits, s);  // 128 x 256, 8 waves
    default: return launch_tile<1, 2>(p, a.affine, a.bits, s);  // 64 x 128, 2 waves
  }
}

}  // namespace ztvm
