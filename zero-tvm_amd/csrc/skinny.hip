// Weight-streaming matrix-core kernel for 2 <= M rows of activations:
//   Y[m,n] = sum_k A[m,k] * w[n,k],  w = s*q + b (4-bit, 3-bit or 8-bit, group 64) or s*(q-7) (4-bit, group 32).
//
// Replaces the reference's small-batch generators (src/compiler/shaders/int4_matmul.gen.ts:
// int4MatmulBatchedWGSL :430-540, int4MatmulBatchedDynWGSL :580-695, int4MatmulTiledMWGSL
// :805-910) for the dispatches that engine-core.ts issues with M_ROWS between 2 and a few
// hundred (speculative verify, MoE prefill chunks, short prompts; call sites :4280-4293,
// :4386-4390). The per-token GEMV would re-read every weight once per row; the tiled GEMM
// stages unpacked weights in LDS and pays a barrier-bound step. Here the weights never touch
// LDS:
//
//   * a wave owns 32 output columns. Each lane fetches its own packed words of the current
//     64-k step straight into registers (the B operand of v_mfma_f32_32x32x16_f16 wants, per
//     lane, 8 consecutive k of one column = one packed word), unpacks them ONCE into exact f16
//     integers and uses them for every 32-row block of the activation tile;
//   * the activation tile (up to 256 rows x 64 k) streams global -> LDS without passing
//     registers, four stages deep, shared by the four waves of the workgroup;
//   * the arithmetic is the GEMV's: integer partial sums per group on the matrix cores (exact
//     in f32), scaled in f32 when folded into the running total; the affine bias term is a few
//     extra MFMA steps over the group sums of the activations (f16 hi + lo) times the f16
//     biases.
//
// The unpackers produce eight values in slot order [v0,v4,v1,v5,v2,v6,v3,v7]; a pre-pass writes
// a copy of the activations with every 8-element chunk in that order (and the group sums), so
// the 12-instruction natural-order unpack becomes 9 (4-bit) and the 3-bit stream unpacks with
// funnel shifts only. 8-bit words unpack to the pairs (v0,v2), (v1,v3), so for that format the copy
// is in the order [v0,v2,v1,v3,v4,v6,v5,v7] (src/compiler/shaders/int8_affine_batched.wgsl is the
// reference's kernel for it: K_PACKED = K/4, four values per word).
#include "internal.h"
#include "mma.h"
#include "skinny.h"

namespace ztvm {
namespace {

// Pre-pass: slot-ordered copy of the activations and, for affine weights, the group sums
// xs16[m][g] = f16(xs), xs16[m][G+g] = f16(xs - hi), zero from 2G up to the stride.
// One thread per 16-byte chunk, eight consecutive lanes = one 64-k group, summed across lanes.
__global__ __launch_bounds__(256) void prep_kernel(const _Float16* __restrict__ in, _Float16* __restrict__ inp,
                                                   _Float16* __restrict__ xs16, uint32_t M, uint32_t K, uint32_t xs_stride,
                                                   uint32_t want_xs, uint32_t order8) {
  const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
  const uint32_t cpr = K / 8, total = M * cpr, G = K / 64;
  if (want_xs) {
    const uint32_t pad = xs_stride - 2 * G;
    if (idx < M * pad) xs16[(size_t)(idx / pad) * xs_stride + 2 * G + idx % pad] = (_Float16)0.f;
  }
  if (idx >= total) return;
  const uint32_t m = idx / cpr, c = idx % cpr;
  const h8 v = *reinterpret_cast<const h8*>(in + (size_t)m * K + (size_t)c * 8);
  h8 w;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    s += (float)v[i];
    w[i] = order8 ? v[value_in_slot8(i)] : v[value_in_slot(i)];
  }
  *reinterpret_cast<h8*>(inp + (size_t)m * K + (size_t)c * 8) = w;
  if (want_xs) {
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
}

typedef uint32_t u32x3_a4 __attribute__((ext_vector_type(3), aligned(4)));

// Registers of one step's weights of a lane.
struct WRegs {
  u32x4 a;     // 4-bit: words 4h..4h+3 (affine) or 0..3 (symmetric); 8-bit: words 8h..8h+3
  u32x4 b;     // 4-bit symmetric: words 4..7; 8-bit: words 8h+4..8h+7
  u32x3 c;     // 3-bit: words 3h..3h+2
  uint32_t s;  // one f16 scale (affine) or two (symmetric)
};

// step(0); if more(1) { step(1); if more(2) { ... } }, entered only if more(0)
template <int J, int N, class More, class Step>
__device__ __forceinline__ void nested_for(More&& more, Step&& step) {
  if constexpr (J < N) {
    if (more(J)) {
      step(std::integral_constant<int, J>{});
      nested_for<J + 1, N>(more, step);
    }
  }
}

// MB: 32-row blocks of the activation tile. CLAMP: the tile is taller than M, rows past M repeat
// row M-1; otherwise a partial last tile is moved up to end at row M.
//
// Every memory operation here is an ordinary load or store that the compiler tracks, so its
// waits carry exact counts: the packed weights, scales and the activation tile of step s+DEPTH
// are fetched into registers while step s computes (DEPTH steps of latency hidden per wave),
// the activation registers of step s are written to one of two LDS buffers, one barrier per step.
//
// The weight loads are ordinary cached loads: a lane's 16 bytes of step s and the 16 of its lane half partner are
// 32 consecutive bytes of a weight row, so a 128-byte line serves four steps and must stay in the vector cache for
// them (with the streaming hint every step asked the second-level cache again: 2.6 M requests a launch at 32 rows
// against 1.5 M without, 31 us against 27).
constexpr int DEPTH = 4;
template <int MB, int BITS, bool AFFINE, bool CLAMP>
__global__ __launch_bounds__(64 * WAVES) void stream_kernel(const StreamParams p) {
  static_assert(BITS == 4 || ((BITS == 3 || BITS == 8) && AFFINE), "formats");
  static_assert(DEPTH % 2 == 0, "the LDS buffer of a step is its position in the unrolled group, mod 2");
  constexpr int ROWS = MB * 32;
  constexpr uint32_t STAGE_BYTES = ROWS * 128;
  constexpr int RPB = AFFINE ? 1 : 2;  // runs = groups per block and step
  constexpr int NRUN = MB * RPB;
  constexpr int MPR = 4 / RPB;         // MFMAs per run
  constexpr int W_STEP_WORDS = BITS == 4 ? 8 : (BITS == 8 ? 16 : 6);

  extern __shared__ __align__(16) unsigned char smem[];

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t frow = lane & 31u, h = lane >> 5;

  // workgroup id -> (k split, row tile, column group): ids sharing an XCD (id % 8) take
  // consecutive ids, which walk the splits and row tiles of one column group first
  uint32_t id = blockIdx.x;
  const uint32_t per_group = p.mtiles * p.ksplit, total = per_group * p.ngroups;
  if (p.xcd_swizzle && total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const uint32_t ng = id / per_group, rest = id % per_group;
  const uint32_t mt = rest % p.mtiles, split = rest / p.mtiles;
  uint32_t m0 = mt * ROWS;
  if (!CLAMP && m0 + ROWS > p.M) m0 = p.M - ROWS;
  const uint32_t n0 = (ng * WAVES + wave) * 32;
  uint32_t n = n0 + frow;
  n = n < p.N ? n : p.N - 1;  // clamped columns are never stored
  // this workgroup's k steps
  const uint32_t s_begin = split * p.steps_per_split;
  const uint32_t s_end = s_begin + p.steps_per_split < p.nsteps ? s_begin + p.steps_per_split : p.nsteps;
  const uint32_t nsteps = s_end > s_begin ? s_end - s_begin : 0;

  UnpackConsts uc;
  uc.init();

  // ---- activations: per step and 32-row block each thread moves 16 bytes, global -> register
  // -> LDS. Slot (r*4 + wave)*64 + lane of a buffer is row (r*4 + wave)*8 + lane/8, and the
  // lane fetches the chunk that the swizzle places there.
  const _Float16* a_src[MB];
  const _Float16* xs_src[MB];
#pragma unroll
  for (int r = 0; r < MB; r++) {
    const uint32_t row = (r * WAVES + wave) * 8 + (lane >> 3);
    const uint32_t ch = (lane & 7u) ^ swz(row);
    uint32_t m = m0 + row;
    if (CLAMP) m = m < p.M ? m : p.M - 1;
    a_src[r] = p.inp + (size_t)m * p.K + (size_t)s_begin * KS + ch * 8;
    xs_src[r] = p.xs16 + (size_t)m * p.xs_stride + ch * 8;
  }
  struct ARegs {
    u32x4 v[MB];
  };
  // adv: elements to advance by afterwards (0 once the last step of the range has been fetched)
  auto fetch_a = [&](ARegs& a, const _Float16** src, uint32_t adv) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < MB; r++) {
      a.v[r] = *reinterpret_cast<const u32x4*>(src[r]);
      src[r] += adv;
    }
  };
  auto store_a = [&](const ARegs& a, uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < MB; r++) *reinterpret_cast<u32x4*>(smem + buf * STAGE_BYTES + (r * WAVES + wave) * 1024u + lane * 16u) = a.v[r];
  };

  // ---- weights and scales of this lane's column
  const uint32_t* w_src = p.weights + (size_t)n * p.row_words + (size_t)s_begin * W_STEP_WORDS + (BITS == 3 ? h * 3 : (BITS == 8 ? h * 8 : (AFFINE ? h * 4 : 0)));
  const _Float16* sc_src = p.scales + (size_t)n * p.spr + (size_t)s_begin * RPB;
  uint32_t sc_tie = 0;  // always 0, but the compiler must not know
  asm volatile("" : "+v"(sc_tie));
  auto fetch_w = [&](WRegs& r, bool adv) __attribute__((always_inline)) {
    if constexpr (BITS == 3) {
      const u32x3_a4 v = *reinterpret_cast<const u32x3_a4*>(w_src);
      r.c = (u32x3){v.x, v.y, v.z};
    } else {
      r.a = *reinterpret_cast<const u32x4*>(w_src);
      if constexpr (!AFFINE || BITS == 8) r.b = *reinterpret_cast<const u32x4*>(w_src + 4);
    }
    if constexpr (AFFINE) r.s = *reinterpret_cast<const uint16_t*>(sc_src + sc_tie);
    else r.s = *reinterpret_cast<const uint32_t*>(sc_src + sc_tie);
    w_src += adv ? W_STEP_WORDS : 0;
    sc_src += adv ? RPB : 0;
  };
  // MFMA t of a step multiplies k chunk chunk_of(t) of the step: both 8-k halves of an MFMA
  // (lane halves h) must lie in one group
  auto chunk_of = [&](int t) __attribute__((always_inline)) { return AFFINE ? 4 * h + t : 2 * t + h; };
  // B operand t: eight exact integers (q, or q-7) in slot order
  auto unpack_t = [&](const WRegs& r, int t) __attribute__((always_inline)) {
    h2 q[4];
    if constexpr (BITS == 8) {
      unpack8_word(t < 2 ? r.a[2 * t] : r.b[2 * t - 4], q, uc);
      unpack8_word(t < 2 ? r.a[2 * t + 1] : r.b[2 * t - 3], q + 2, uc);
    } else if constexpr (BITS == 4) {
      uint32_t w;
      if constexpr (AFFINE) {
        w = r.a[t];
      } else {
        const uint32_t w0 = t < 2 ? r.a[2 * t] : r.b[2 * t - 4], w1 = t < 2 ? r.a[2 * t + 1] : r.b[2 * t - 3];
        w = h ? w1 : w0;
      }
      unpack4_block(w, q, uc);
      if constexpr (!AFFINE) {
        const h2 k7 = {(_Float16)7.f, (_Float16)7.f};
#pragma unroll
        for (int j = 0; j < 4; j++) q[j] -= k7;
      }
    } else {
      const uint32_t w0 = r.c.x, w1 = r.c.y, w2 = r.c.z;
      if (t == 0) unpack3_views(w0 << 4, w0 >> 2, q, uc);
      if (t == 1) unpack3_views(__builtin_amdgcn_alignbit(w1, w0, 20), __builtin_amdgcn_alignbit(w1, w0, 26), q, uc);
      if (t == 2) unpack3_views(__builtin_amdgcn_alignbit(w2, w1, 12), __builtin_amdgcn_alignbit(w2, w1, 18), q, uc);
      if (t == 3) unpack3_views(w2 >> 4, w2 >> 10, q, uc);
    }
    return (h8){q[0].x, q[0].y, q[1].x, q[1].y, q[2].x, q[2].y, q[3].x, q[3].y};
  };
  auto scale_of = [&](const WRegs& r, int g) __attribute__((always_inline)) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(g ? r.s >> 16 : r.s));
  };

  // ---- activation fragments: lane -> row frow of a 32-row block, chunk chunk_of(t)
  uint32_t a_rd[4];
#pragma unroll
  for (int t = 0; t < 4; t++) a_rd[t] = frow * 128 + ((chunk_of(t) ^ swz(frow)) << 4);
  auto read_a = [&](uint32_t buf, int i, int t) __attribute__((always_inline)) {
    return *reinterpret_cast<const h8*>(smem + buf * STAGE_BYTES + a_rd[t] + i * 4096);
  };

  f16v tot[MB];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) tot[i][e] = 0.f;
  const f16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  // ---- bias term first (affine, first k split only): tot = [xs_hi | xs_lo] x biases, 64 columns
  // per step; the group sums go through LDS buffer 0, the biases straight from memory into the
  // B operand (column c of the [hi | lo] matrix meets b[n][c mod G]; zero past 2G). Natural
  // order on both sides.
  if (AFFINE && split == 0) {
    const uint32_t G = p.spr;
    const _Float16* brow = p.biases + (size_t)n * G;
    for (uint32_t bs = 0; bs < p.bias_steps; bs++) {
      ARegs xa;
      fetch_a(xa, xs_src, KS);
      h8 bf[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const uint32_t col = bs * KS + chunk_of(t) * 8;
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
        bf[t] = v;
      }
      store_a(xa, 0);
      __syncthreads();
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int t = 0; t < 4; t++) tot[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(read_a(0, i, t), bf[t], tot[i], 0, 0, 0);
      __syncthreads();
    }
  }

  // ---- main loop: register rings of DEPTH steps for the weights and the activation tile
  WRegs wq[DEPTH];
  ARegs aq[DEPTH];
  h8 Af[2][4], Bf[4];
  f16v part[2];
  float sc_cur[RPB], sc_prev = 0.f;
  part[0] = zero;
  part[1] = zero;


  // Steps fetched so far. Every step refills its ring slot with step s+DEPTH: past the end of the range the
  // fetch repeats the last step (the pointers stop advancing) and nobody reads the result, so the loop has one
  // shape for every range length and no wait of it ever has to allow for a path with fewer loads in flight.
  uint32_t fetched = 0;
  auto fetch = [&](int j) __attribute__((always_inline)) {
    const bool adv = ++fetched < nsteps;
    fetch_w(wq[j], adv);
    fetch_a(aq[j], a_src, adv ? KS : 0);
  };
  // one step: position j in the ring
  auto step = [&](auto jc) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    constexpr uint32_t buf = j & 1;
    // this step's activations into LDS, its weights into the B operands
    store_a(aq[j], buf);
#pragma unroll
    for (int t = 0; t < 4; t++) Bf[t] = unpack_t(wq[j], t);
#pragma unroll
    for (int g = 0; g < RPB; g++) sc_cur[g] = scale_of(wq[j], g);
    // The scale must be a float before its ring slot is refilled. Left alone the compiler folds the
    // conversion into the FMAs of the NEXT step, keeps the raw halfword alive past the refill, and pays for
    // that with register copies of values still in flight at the top of the loop, where waiting for them
    // drains the ring. The empty statement makes the refill's address (sc_src + sc_tie, sc_tie always 0)
    // depend on the converted value.
#pragma unroll
    for (int g = 0; g < RPB; g++) asm volatile("" : "+v"(sc_cur[g]), "+v"(sc_tie));
    fetch(j);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 4; t++) Af[0][t] = read_a(buf, 0, t);
    static_for<NRUN>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      constexpr int i = r / RPB, sub = r % RPB;
      constexpr int pb = r & 1;  // partial set of this run
      constexpr int ab = i & 1;  // fragment set of this block
      // read ahead the next block's fragments
      if (sub == 0 && i + 1 < MB) {
#pragma unroll
        for (int t = 0; t < 4; t++) Af[ab ^ 1][t] = read_a(buf, i + 1, t);
      }
#pragma unroll
      for (int t = sub * MPR; t < (sub + 1) * MPR; t++)
        part[pb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Af[ab][t], Bf[t], t == sub * MPR ? zero : part[pb], 0, 0, 0);
      // fold the run before this one: tot += scale * part
      {
        constexpr int ri = (r + NRUN - 1) % NRUN;
        const float sc = r == 0 ? sc_prev : sc_cur[ri % RPB];
#pragma unroll
        for (int e = 0; e < 16; e++) tot[ri / RPB][e] = __builtin_fmaf(sc, part[pb ^ 1][e], tot[ri / RPB][e]);
      }
    });
    sc_prev = sc_cur[RPB - 1];
    if (NRUN % 2) part[1] = part[0];  // the next step folds part[1] first
  };
  if (nsteps > 0) {
    static_for<DEPTH>([&](auto jc) { fetch(decltype(jc)::value); });
    // whole turns of the ring, then the rest as nested conditions: a step that is not reached leaves for the
    // end of the kernel, so no step is ever entered from a path that skipped the one before it
    uint32_t s = 0;
    for (; s + DEPTH <= nsteps; s += DEPTH) static_for<DEPTH>(step);
    nested_for<0, DEPTH - 1>([&](int j) { return s + j < nsteps; }, step);
  }
  // the last run is still unfolded
  if (nsteps > 0) {
#pragma unroll
    for (int e = 0; e < 16; e++) tot[MB - 1][e] = __builtin_fmaf(sc_prev, part[1][e], tot[MB - 1][e]);
  }

  // D layout of a 32x32 block: lane -> column frow, register e -> row 8*(e/4) + 4*h + e%4
  const uint32_t nn = n0 + frow;
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const uint32_t m = m0 + i * 32 + 8 * (e / 4) + 4 * h + (e % 4);
      if (m < p.M && nn < p.N) {
        if (p.ksplit > 1) p.partial[((size_t)split * p.M + m) * p.N + nn] = tot[i][e];
        else if (p.out_f32) reinterpret_cast<float*>(p.out)[(size_t)m * p.N + nn] = tot[i][e];
        else reinterpret_cast<_Float16*>(p.out)[(size_t)m * p.N + nn] = (_Float16)tot[i][e];
      }
    }
}

// out = sum over the k splits of the f32 partial results, in split order
__global__ __launch_bounds__(256) void reduce_kernel(const float* __restrict__ partial, void* __restrict__ out, uint32_t count,
                                                     uint32_t ksplit, uint32_t out_f32) {
  const uint32_t i4 = (blockIdx.x * 256u + threadIdx.x) * 4;
  if (i4 >= count) return;
  f4 acc = *reinterpret_cast<const f4*>(partial + i4);
  for (uint32_t k = 1; k < ksplit; k++) acc += *reinterpret_cast<const f4*>(partial + (size_t)k * count + i4);
  if (out_f32) {
    *reinterpret_cast<f4*>(reinterpret_cast<float*>(out) + i4) = acc;
  } else {
    h4 v = {(_Float16)acc.x, (_Float16)acc.y, (_Float16)acc.z, (_Float16)acc.w};
    *reinterpret_cast<h4*>(reinterpret_cast<_Float16*>(out) + i4) = v;
  }
}

template <int MB, int BITS, bool AFFINE>
hipError_t launch_mb(StreamParams p, hipStream_t s) {
  constexpr int ROWS = MB * 32;
  const dim3 grid(p.mtiles * p.ngroups * p.ksplit);
  const size_t smem = 2 * (size_t)ROWS * 128;
  auto go = [&](auto k) { hipLaunchKernelGGL(k, grid, dim3(64 * WAVES), smem, s, p); };
  if (p.M < (uint32_t)ROWS) go(stream_kernel<MB, BITS, AFFINE, true>);
  else go(stream_kernel<MB, BITS, AFFINE, false>);
  return hipGetLastError();
}

template <int BITS, bool AFFINE>
hipError_t launch_fmt(const StreamParams& p, int mb, hipStream_t s) {
  if (mb == 1) return launch_mb<1, BITS, AFFINE>(p, s);
  if (mb == 2) return launch_mb<2, BITS, AFFINE>(p, s);
  return launch_mb<4, BITS, AFFINE>(p, s);
}

int blocks_of(uint32_t M) { return M <= 32 ? 1 : (M <= 64 ? 2 : 4); }

uint32_t xs_stride_of(const MatmulArgs& a) { return a.affine ? (2 * a.spr + KS - 1) / KS * KS : 0; }

// k splits: one round of workgroups over the CUs for a single row tile (measured: 2 beats 3 at 112
// column groups on 256 CUs, 8 wins at 32 groups). A function of N and K only, so that a row's
// result does not depend on how many rows travel with it; bounded so that the f32 partial results
// of a 32-row tile stay smaller than the weights.
uint32_t ksplit_of(const MatmulArgs& a, const Tune& t) {
  if (a.N % 4) return 1;  // the reduction works on groups of four outputs
  if (t.skinny_ksplit > 0) return (uint32_t)t.skinny_ksplit;
  const uint32_t ngroups = (a.N + 32 * WAVES - 1) / (32 * WAVES);
  const uint32_t nsteps = a.K / KS;
  uint32_t want = (uint32_t)t.num_cus / ngroups;
  if (want > a.K / 512u) want = a.K / 512u;
  if (want > 16) want = 16;
  if (want > nsteps / 4) want = nsteps / 4;
  return want < 1 ? 1 : want;
}

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

// Dense, K a multiple of 64, byte offsets within 32 bits.
hipError_t launch_reduce_partials(const float* partial, void* out, uint32_t count, uint32_t ksplit, bool out_f32, hipStream_t s) {
  hipLaunchKernelGGL(reduce_kernel, dim3((count / 4 + 255) / 256), dim3(256), 0, s, partial, out, count, ksplit, (uint32_t)out_f32);
  return hipGetLastError();
}

bool skinny_supports(const MatmulArgs& a) {
  if (a.slots != 0 || a.K % KS != 0 || a.M < 1) return false;
  if (!(a.bits == 4 || ((a.bits == 3 || a.bits == 8) && a.affine))) return false;
  const uint64_t lim = 1ull << 32;
  return (uint64_t)a.M * a.K * 2 < lim && (uint64_t)a.M * (xs_stride_of(a) + 1) * 2 < lim;
}

uint32_t skinny_reg_ksplit(const MatmulArgs& a, const Tune& t) { return ksplit_of(a, t); }

size_t skinny_scratch_bytes(const MatmulArgs& a, const Tune& t) {
  const uint32_t ks = skinny_dma_supports(a, t) ? skinny_dma_ksplit(a, t) : ksplit_of(a, t);
  return align256((size_t)a.M * a.K * sizeof(_Float16)) + align256((size_t)a.M * xs_stride_of(a) * sizeof(_Float16)) +
         (ks > 1 ? align256((size_t)ks * a.M * a.N * sizeof(float)) : 0) + 256;
}

hipError_t launch_skinny(const MatmulArgs& a, const Tune& t, void* scratch, hipStream_t s) {
  StreamParams p{};
  p.out = a.out;
  p.out_f32 = a.out_f32;
  char* base = reinterpret_cast<char*>(scratch);
  _Float16* inp = reinterpret_cast<_Float16*>(base);
  base += align256((size_t)a.M * a.K * sizeof(_Float16));
  _Float16* xs16 = reinterpret_cast<_Float16*>(base);
  base += align256((size_t)a.M * xs_stride_of(a) * sizeof(_Float16));
  p.partial = reinterpret_cast<float*>(base);
  p.inp = inp; p.xs16 = xs16;
  p.scales = a.scales; p.weights = a.weights; p.biases = a.biases;
  p.M = a.M; p.N = a.N; p.K = a.K; p.row_words = a.k_packed; p.spr = a.spr;
  p.nsteps = a.K / KS;
  p.xs_stride = xs_stride_of(a);
  p.bias_steps = a.affine ? p.xs_stride / KS : 0;
  p.xcd_swizzle = t.gemm_xcd_swizzle;
  const bool dma = skinny_dma_supports(a, t);
  const int mb = blocks_of(a.M);
  if (!dma) {
    p.mtiles = (a.M + 32 * mb - 1) / (32 * mb);
    p.ngroups = (a.N + 32 * WAVES - 1) / (32 * WAVES);
    p.ksplit = ksplit_of(a, t);
    p.steps_per_split = (p.nsteps + p.ksplit - 1) / p.ksplit;
  }
  {
    const uint32_t pad = a.affine ? p.xs_stride - 2 * (a.K / 64) : 0, cpr = a.K / 8;
    const uint32_t nthr = a.M * (cpr > pad ? cpr : pad);  // one thread per chunk, and enough for the padding columns
    hipLaunchKernelGGL(prep_kernel, dim3((nthr + 255) / 256), dim3(256), 0, s, a.in, inp, xs16, a.M, a.K, p.xs_stride, (uint32_t)a.affine,
                       (uint32_t)(a.bits == 8));
  }
  hipError_t e;
  if (dma) e = launch_skinny_dma(p, a, t, s);
  else if (a.bits == 3) e = launch_fmt<3, true>(p, mb, s);
  else if (a.bits == 8) e = launch_fmt<8, true>(p, mb, s);
  else if (a.affine) e = launch_fmt<4, true>(p, mb, s);
  else e = launch_fmt<4, false>(p, mb, s);
  if (e != hipSuccess) return e;
  if (p.ksplit > 1) {
    return launch_reduce_partials(p.partial, a.out, a.M * a.N, p.ksplit, a.out_f32 != 0, s);  // N % 4 == 0 whenever ksplit > 1
  }
  return hipSuccess;
}

}  // namespace ztvm
