// Weight-streaming matrix-core kernel for 2 <= M rows, transfer-engine form (4-bit weights, affine group 64 or
// symmetric group 32, K a multiple of 128). Same arithmetic and same operands as stream_kernel in skinny.hip (which
// keeps the 3-bit and 8-bit formats and the K that this form refuses); what differs is how the bytes travel:
//
//   * nothing is fetched into registers. Activations, packed weights and scales all go global -> LDS through the
//     transfer path of the vector memory unit, so a deep pipeline costs LDS, not registers, and the fetches of a wave
//     retire in one queue whose depth the kernel counts by hand (every wave issues the same number per unit);
//   * a weight row is fetched 64 consecutive bytes at a time (two k steps), four lanes per row: every request the
//     vector cache makes is used whole. Fetched one step at a time, a lane pair per row, each request was half used
//     and asked for twice; the scales were asked for once per step, 2 bytes out of 64;
//   * the workgroup is NW column waves (32 output columns each) times KH k parts. Each k part runs its own pipeline
//     over its own share of K; the parts meet at one barrier per unit and add their totals through LDS at the end, in
//     part order. Two waves per SIMD: while one waits at the barrier or for its fragments the other multiplies.
//     (One wave per SIMD, as in stream_kernel, spends its time waiting: 40% of the issue slots at 128 rows.)
//
// Measured at K=4096, N=14336 with per-turn time stamps: the waits for the transfers are empty (76 ticks of a 2400-tick
// turn), so neither a deeper pipeline nor a wave that touches the weights ahead of time into the second-level cache
// changes anything (both tried). A turn is the matrix and vector instructions of its two steps: 16 matrix and about
// 150 vector instructions per wave at 64 rows, two waves per SIMD.
//
// Unit = two k steps = 128 k. LDS of k part p, stage t (D stages):
//     activations  2 x ROWS x 128 B   step j at j*ROWS*128; row r = 8 chunks of 16 B, chunk c at (c ^ swz(r))
//     weights      CW x 64 B          row n = 4 chunks of 16 B, chunk c at (c ^ swzw(n)); chunk 2j+h is the half of
//                                     step j that lane half h multiplies (affine); symmetric rows use both halves
//     scales       NW x 256 B         wave w, lane l: one dword = the unit's two scales of column l%32 (affine), or
//                                     scales 2*(l/32), 2*(l/32)+1 of the unit's four (symmetric)
#include "internal.h"
#include "mma.h"
#include "skinny.h"

namespace ztvm {
namespace {


// Transfers global (base + voff) -> LDS (lds_base + 16*lane, or + 4*lane). Not a memory barrier for the compiler, so
// that it may move the LDS reads of the next run of matrix instructions above a transfer: the order that matters (a
// stage is refilled only after the barrier that follows its last read, and read only after the wait and the barrier
// that follow its transfers) is kept by the wait and barrier statements, which are.
__device__ __forceinline__ void xfer16(const void* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(lds_base) : "m0");
}
__device__ __forceinline__ void xfer4(const void* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(voff), "s"(base), "s"(lds_base) : "m0");
}

// weight rows of 64 bytes: a 128-bit read serves 8 lanes a cycle, rows of equal parity share a bank half
__device__ __forceinline__ uint32_t swzw(uint32_t row) { return (row >> 1) & 3u; }

template <int MB, int NW, int KH, int D, bool AFFINE, bool CLAMP>
__global__ __launch_bounds__(64 * NW * KH) void dma_kernel(const StreamParams p) {
  constexpr int ROWS = MB * 32, CW = NW * 32, T = NW * 64;
  constexpr int AP = ROWS * 8 / T;       // 16-byte pieces of one step's activation tile per thread
  constexpr int RPB = AFFINE ? 1 : 2;    // runs = groups per block and step
  constexpr int NRUN = MB * RPB;
  constexpr int MPR = 4 / RPB;           // MFMAs per run
  constexpr uint32_t A_STEP = ROWS * 128, A_BYTES = 2 * A_STEP, W_BYTES = CW * 64, S_BYTES = NW * 256;
  constexpr uint32_t STAGE = A_BYTES + W_BYTES + S_BYTES, PART = D * STAGE;
  constexpr int L = 2 * AP + 2 + 1;      // transfers per wave and unit
  static_assert(ROWS * 8 % T == 0, "whole pieces per thread");
  static_assert(D >= 2 && (D - 1) * L < 64, "the queue counter holds 63");

  extern __shared__ __align__(16) unsigned char smem[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)smem;

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wc = wave % NW, part = wave / NW;
  const uint32_t tp = wc * 64 + lane;  // thread within its k part
  const uint32_t frow = lane & 31u, h = lane >> 5;

  // workgroup id -> (k split, row tile, column group): ids sharing an XCD (id % 8) take consecutive ids, which walk the
  // splits and row tiles of one column group first
  uint32_t id = blockIdx.x;
  const uint32_t per_group = p.mtiles * p.ksplit, total = per_group * p.ngroups;
  if (p.xcd_swizzle && total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const uint32_t ng = id / per_group, rest = id % per_group;
  const uint32_t mt = rest % p.mtiles, split = rest / p.mtiles;
  uint32_t m0 = mt * ROWS;
  if (!CLAMP && m0 + ROWS > p.M) m0 = p.M - ROWS;
  const uint32_t n0 = ng * CW;

  // ---- units of this workgroup, of this k part. steps_per_split is even; a part may come out empty.
  const uint32_t nunits = p.nsteps / 2, ups = p.steps_per_split / 2;
  const uint32_t u_begin = split * ups, u_stop = u_begin + ups < nunits ? u_begin + ups : nunits;  // u_begin < u_stop
  const uint32_t nsplit = u_stop - u_begin;
  const uint32_t upp = (nsplit + KH - 1) / KH;  // turns of the loop, the same for every part
  // Part p multiplies units u_begin + p, u_begin + p + KH, ...: in one turn the KH parts fetch KH consecutive units,
  // 64*KH consecutive bytes of every weight row.
  const uint32_t my_units = part < nsplit ? (nsplit - part + KH - 1) / KH : 0;
  const uint32_t u_last = u_stop - 1;  // fetches past the part's share repeat the split's last unit; nobody reads them

  // ---- transfers. Piece q = r*T + tp of a step's activation tile is LDS bytes [16q, 16q+16): row q/8, chunk slot q%8.
  uint32_t a_off[AP], xs_off[AP];  // activations; their group sums (the bias term's left operand)
#pragma unroll
  for (int r = 0; r < AP; r++) {
    const uint32_t q = r * T + tp, row = q >> 3;
    const uint32_t ch = (q & 7u) ^ swz(row);
    uint32_t m = m0 + row;
    if (CLAMP) m = m < p.M ? m : p.M - 1;
    a_off[r] = (m * p.K + ch * 8) * 2u;
    xs_off[r] = (m * p.xs_stride + ch * 8) * 2u;
  }
  // Piece q = r*T + tp (r = 0, 1) of a unit's weight tile: row q/4, chunk slot q%4.
  uint32_t w_off[2];
#pragma unroll
  for (int r = 0; r < 2; r++) {
    const uint32_t q = r * T + tp, row = q >> 2;
    const uint32_t ch = (q & 3u) ^ swzw(row);
    uint32_t n = n0 + row;
    n = n < p.N ? n : p.N - 1;  // clamped columns are never stored
    w_off[r] = n * p.row_words * 4u + ch * 16u;
  }
  uint32_t ncol = n0 + wc * 32 + frow;
  ncol = ncol < p.N ? ncol : p.N - 1;
  const uint32_t s_off = (ncol * p.spr + (AFFINE ? 0u : 2u * h)) * 2u;
  const uint32_t lds_part = lds0 + part * PART;
  const bool with_bias = AFFINE && split == 0;
  // bias step of this part that travels as step j of the unit sent e turns past the end (see the bias term below)
  auto bias_step_of = [&](uint32_t e, int j) __attribute__((always_inline)) { return (2 * e + j) * KH + part; };
  // Transfer k (0 .. L-1) of unit i of this part's sequence, into stage t: the activations of step 0, of step 1, the
  // weights, the scales.
  auto issue_one = [&](auto kc, uint32_t i, uint32_t t) __attribute__((always_inline)) {
    constexpr int k = decltype(kc)::value;
    uint32_t u = u_begin + i * KH + part;
    u = u < u_last ? u : u_last;
    const uint32_t st = lds_part + t * STAGE;
    if constexpr (k < 2 * AP) {
      constexpr int j = k / AP, r = k % AP;
      const uint32_t bs = bias_step_of(i - upp, j);  // only meant for i >= upp
      if (with_bias && i >= upp && bs < p.bias_steps)
        xfer16(p.xs16 + bs * KS, xs_off[r], st + j * A_STEP + (r * NW + wc) * 1024u);
      else
        xfer16(reinterpret_cast<const char*>(p.inp) + (size_t)u * 256 + j * 128, a_off[r], st + j * A_STEP + (r * NW + wc) * 1024u);
    } else if constexpr (k < 2 * AP + 2) {
      constexpr int r = k - 2 * AP;
      xfer16(reinterpret_cast<const char*>(p.weights) + (size_t)u * 64, w_off[r], st + A_BYTES + (r * NW + wc) * 1024u);
    } else {
      xfer4(reinterpret_cast<const char*>(p.scales) + (size_t)u * (AFFINE ? 4 : 8), s_off, st + A_BYTES + W_BYTES + wc * 256u);
    }
  };
  // transfers [L*slot/NSLOT, L*(slot+1)/NSLOT): a turn sends its L transfers in NSLOT helpings, between its runs of
  // matrix instructions. Sent all at once after the barrier, every wave of the workgroup stood in the same queue
  // (48 KB go through the vector cache at 64 bytes a clock) and none of them multiplied meanwhile: 0.3 to 0.7 us of a
  // 2.1 us turn at 128 rows.
  constexpr int NSLOT = 2 * NRUN;
  auto issue_slot = [&](auto sc_, uint32_t i, uint32_t t) __attribute__((always_inline)) {
    constexpr int slot = decltype(sc_)::value;
    constexpr int k0 = L * slot / NSLOT, k1 = L * (slot + 1) / NSLOT;
    static_for<k1 - k0>([&](auto kc) { issue_one(ic<k0 + decltype(kc)::value>{}, i, t); });
  };
  auto issue = [&](uint32_t i, uint32_t t) __attribute__((always_inline)) {
    static_for<L>([&](auto kc) { issue_one(kc, i, t); });
  };

  UnpackConsts uc;
  uc.init();
  auto chunk_of = [&](int t) __attribute__((always_inline)) { return AFFINE ? 4 * h + t : 2 * t + h; };

  // ---- LDS read addresses (bytes from the stage's start)
  uint32_t a_rd[4];
#pragma unroll
  for (int t = 0; t < 4; t++) a_rd[t] = frow * 128 + ((chunk_of(t) ^ swz(frow)) << 4);
  const uint32_t wrow = wc * 32 + frow;
  // affine: the lane's 16 bytes of step j are chunk 2j+h; symmetric: both chunks of step j
  uint32_t w_rd[2][2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    w_rd[j][0] = A_BYTES + wrow * 64 + (((AFFINE ? 2 * j + h : 2 * j) ^ swzw(wrow)) << 4);
    w_rd[j][1] = A_BYTES + wrow * 64 + (((2 * j + 1) ^ swzw(wrow)) << 4);
  }
  const uint32_t s_rd = A_BYTES + W_BYTES + wc * 256 + frow * 4;

  f16v tot[MB];
#pragma unroll
  for (int i = 0; i < MB; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) tot[i][e] = 0.f;
  const f16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  // ---- the pipeline's first D-1 units go out before anything else. (All workgroups of the chip start at the same
  // moment on cold caches: the first barrier comes 9000 ticks into a 48000-tick kernel at 128 rows. Sending one unit
  // and the next after the first barrier only puts two such trips one after the other.)
#pragma unroll
  for (int t = 0; t < D - 1; t++) issue(t, t);

  // ---- bias term (affine, first k split): tot += [xs_hi | xs_lo] x biases, 64 columns per step, after the main loop.
  // Bias step (2e + j)*KH + part belongs to this part: its group sums travel as the "activations" of step j of the
  // unit that the pipeline sends e turns past its end (it sends D-1 units past the end anyway, to keep the count of
  // its queue), so they are in LDS when the loop ends; the biases of e = 0, j = 0 wait in registers from here on. Fetched
  // and multiplied before the loop, the term kept every wave waiting for one more trip to memory at the start.
  auto load_biases = [&](uint32_t bs, h8* dst) __attribute__((always_inline)) {
    const uint32_t G = p.spr;
    const _Float16* brow = p.biases + (size_t)ncol * G;
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const uint32_t col = bs * KS + chunk_of(t) * 8;  // column c of [hi | lo] meets b[n][c mod G]; zero past 2G
      h8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (bs < p.bias_steps && col < 2 * G) {
        if (G % 8 == 0) {
          v = *reinterpret_cast<const h8*>(brow + (col % G));
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (col + e < 2 * G) v[e] = brow[(col + e) % G];
        }
      }
      dst[t] = v;
    }
  };
  h8 bf0[4];  // the biases of this part's bias step e = 0, j = 0, in registers from here to the end of the loop
  if (with_bias) load_biases(bias_step_of(0, 0), bf0);

  // ---- main loop
  h8 Af[2][4], Bf[4];
  f16v acc[2];
  float sc_cur[RPB], sc_prev = 0.f;
  acc[0] = zero;
  acc[1] = zero;
  // one k step out of stage t of this part: j = 0, 1
  // (jc: step 0 or 1 of the unit; the turn's transfers for unit i_next go out between the runs)
  auto step = [&](uint32_t st, auto jc, uint32_t i_next, uint32_t t_next) __attribute__((always_inline)) {
    constexpr int j = decltype(jc)::value;
    const unsigned char* base = smem + st;
    const unsigned char* abase = base + j * A_STEP;
    u32x4 wa = *reinterpret_cast<const u32x4*>(base + w_rd[j][0]), wb;
    if (!AFFINE) wb = *reinterpret_cast<const u32x4*>(base + w_rd[j][1]);
    if (AFFINE) {
      sc_cur[0] = (float)*reinterpret_cast<const _Float16*>(base + s_rd + j * 2);
    } else {
      const uint32_t two = *reinterpret_cast<const uint32_t*>(base + s_rd + j * 128);
      sc_cur[0] = (float)__builtin_bit_cast(_Float16, (uint16_t)two);
      sc_cur[RPB - 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(two >> 16));
    }
#pragma unroll
    for (int t = 0; t < 4; t++) Af[0][t] = *reinterpret_cast<const h8*>(abase + a_rd[t]);
#pragma unroll
    for (int t = 0; t < 4; t++) {
      h2 q[4];
      uint32_t w;
      if (AFFINE) {
        w = wa[t];
      } else {
        const uint32_t w0 = t < 2 ? wa[2 * t] : wb[2 * t - 4], w1 = t < 2 ? wa[2 * t + 1] : wb[2 * t - 3];
        w = h ? w1 : w0;
      }
      unpack4_block(w, q, uc);
      if (!AFFINE) {
        const h2 k7 = {(_Float16)7.f, (_Float16)7.f};
#pragma unroll
        for (int e = 0; e < 4; e++) q[e] -= k7;
      }
      Bf[t] = (h8){q[0].x, q[0].y, q[1].x, q[1].y, q[2].x, q[2].y, q[3].x, q[3].y};
    }
    static_for<NRUN>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      constexpr int i = r / RPB, sub = r % RPB;
      constexpr int pb = r & 1;  // partial set of this run
      constexpr int ab = i & 1;  // fragment set of this block
      issue_slot(ic<j * NRUN + r>{}, i_next, t_next);
      if (sub == 0 && i + 1 < MB) {
#pragma unroll
        for (int t = 0; t < 4; t++) Af[ab ^ 1][t] = *reinterpret_cast<const h8*>(abase + a_rd[t] + (i + 1) * 4096);
      }
#pragma unroll
      for (int t = sub * MPR; t < (sub + 1) * MPR; t++)
        acc[pb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Af[ab][t], Bf[t], t == sub * MPR ? zero : acc[pb], 0, 0, 0);
      // fold the run before this one: tot += scale * partial
      {
        constexpr int ri = (r + NRUN - 1) % NRUN;
        const float sc = r == 0 ? sc_prev : sc_cur[ri % RPB];
#pragma unroll
        for (int e = 0; e < 16; e++) tot[ri / RPB][e] = __builtin_fmaf(sc, acc[pb ^ 1][e], tot[ri / RPB][e]);
      }
    });
    sc_prev = sc_cur[RPB - 1];
    if (NRUN % 2) acc[1] = acc[0];  // the next step folds acc[1] first
  };

  // Turn i: wait for unit i of this wave's own transfers (those of the D-2 units after it may still fly), meet the
  // other waves (their pieces of unit i have landed too, and everyone is done reading the stage of unit i-1), send
  // unit i+D-1 into that stage, multiply unit i.
  for (uint32_t i0 = 0; i0 < upp; i0 += D) {
    static_for<D>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      const uint32_t i = i0 + t;
      if (i < upp) {
        wait_vm<(D - 2) * L>();
        wg_barrier();
        if (i < my_units) {
          step(part * PART + t * STAGE, ic<0>{}, i + D - 1, (t + D - 1) % D);
          step(part * PART + t * STAGE, ic<1>{}, i + D - 1, (t + D - 1) % D);
        } else {
          issue(i + D - 1, (t + D - 1) % D);  // a part that has run out of units keeps the count of its queue
        }
      }
    });
  }
  // the last run is still unfolded (sc_prev is 0 for a part without units)
#pragma unroll
  for (int e = 0; e < 16; e++) tot[MB - 1][e] = __builtin_fmaf(sc_prev, acc[1][e], tot[MB - 1][e]);

  wait_vm<0>();  // the units sent past the end have landed (their weights and scales: nobody reads them)
  wg_barrier();
  if (with_bias) {
    for (uint32_t e = 0; e < D - 1; e++) {
      const uint32_t st = part * PART + ((upp + e) % D) * STAGE;
#pragma unroll
      for (int j = 0; j < 2; j++) {
        if (bias_step_of(e, j) < p.bias_steps) {  // uniform per wave
          h8 bf[4];
          if (e == 0 && j == 0) {
#pragma unroll
            for (int t = 0; t < 4; t++) bf[t] = bf0[t];
          } else {
            load_biases(bias_step_of(e, j), bf);  // more than KH bias steps (K above 2048*KH): fetched now
          }
#pragma unroll
          for (int i = 0; i < MB; i++)
#pragma unroll
            for (int t = 0; t < 4; t++)
              tot[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const h8*>(smem + st + j * A_STEP + a_rd[t] + i * 4096), bf[t], tot[i], 0, 0,
                                                              0);
        }
      }
    }
  }

  // ---- the k parts add up through LDS, in part order
  constexpr uint32_t RED_BYTES = (KH - 1) * NW * MB * 4096;
  if (KH > 1) {
    wg_barrier();
    float* red = reinterpret_cast<float*>(smem);
    if (part > 0) {
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) red[(((part - 1) * NW + wc) * MB + i) * 1024 + e * 64 + lane] = tot[i][e];
    }
    wg_barrier();
    if (part == 0) {
      for (uint32_t pp = 1; pp < KH; pp++)
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
          for (int e = 0; e < 16; e++) tot[i][e] += red[(((pp - 1) * NW + wc) * MB + i) * 1024 + e * 64 + lane];
    }
  }

  // ---- f16 results of a whole k range leave as full rows of the workgroup's tile: through LDS (behind the parts'
  // totals, which part 0 may still be reading), 16 bytes per lane, every wave of the workgroup storing. Stored from
  // the accumulator layout a lane writes 2 bytes and an instruction 64 bytes of each of two rows: 3 us of a 29 us
  // kernel at 128 rows.
  // D layout of a 32x32 block: lane -> column frow, register e -> row 8*(e/4) + 4*h + e%4
  if (p.ksplit == 1 && !p.out_f32 && p.N % 8 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15u) == 0) {
    constexpr uint32_t PITCH = CW * 2 + 16;  // the two rows an instruction writes fall into different banks
    static_assert(RED_BYTES + ROWS * PITCH <= KH * PART, "the output tile fits behind the totals");
    unsigned char* ot = smem + RED_BYTES;
    if (part == 0) {
#pragma unroll
      for (int i = 0; i < MB; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          const uint32_t row = i * 32 + 8 * (e / 4) + 4 * h + (e % 4);
          *reinterpret_cast<_Float16*>(ot + row * PITCH + (wc * 32 + frow) * 2) = (_Float16)tot[i][e];
        }
    }
    wg_barrier();
    for (uint32_t q = tid; q < ROWS * CW / 8; q += 64 * NW * KH) {
      const uint32_t row = q / (CW / 8), c8 = q % (CW / 8);
      const uint32_t m = m0 + row, n = n0 + c8 * 8;
      if (m < p.M && n < p.N)
        *reinterpret_cast<u32x4*>(reinterpret_cast<_Float16*>(p.out) + (size_t)m * p.N + n) = *reinterpret_cast<const u32x4*>(ot + row * PITCH + c8 * 16);
    }
    return;
  }
  if (part > 0) return;
  const uint32_t nn = n0 + wc * 32 + frow;
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

// Tile shapes: rows = 32*mb, columns = 32*nw, kh k parts, d stages
struct Shape {
  int mb, nw, kh, d;
};

// By rows unless the knob names one (any shape runs any M; a row's bits depend on the shape, not on M)
Shape shape_of(const MatmulArgs& a, const Tune& t) {
  if (t.skinny_shape == 2) return Shape{2, 4, 2, 3};
  if (t.skinny_shape == 3) return Shape{1, 2, 4, 3};
  return a.M <= 32 ? Shape{1, 2, 4, 3} : Shape{2, 4, 2, 3};
}

template <int MB, int NW, int KH, int D, bool AFFINE>
hipError_t launch_shape(const StreamParams& p, hipStream_t s) {
  constexpr int ROWS = MB * 32;
  constexpr size_t smem = (size_t)KH * D * (2 * ROWS * 128 + NW * 32 * 64 + NW * 256);
  static_assert(smem <= 160 * 1024, "LDS of a CU");
  static_assert(64 * NW * KH <= 1024, "threads of a workgroup");
  auto go = [&](auto k) {
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, dim3(p.mtiles * p.ngroups * p.ksplit), dim3(64 * NW * KH), smem, s, p);
  };
  if (p.M < (uint32_t)ROWS) go(dma_kernel<MB, NW, KH, D, AFFINE, true>);
  else go(dma_kernel<MB, NW, KH, D, AFFINE, false>);
  return hipGetLastError();
}

template <bool AFFINE>
hipError_t launch_affine(const StreamParams& p, const Shape& sh, hipStream_t s) {
  if (sh.mb == 1) return launch_shape<1, 2, 4, 3, AFFINE>(p, s);
  return launch_shape<2, 4, 2, 3, AFFINE>(p, s);
}

}  // namespace

bool skinny_dma_supports(const MatmulArgs& a, const Tune& t) {
  if (t.skinny_dma == 1) return false;  // switched off
  if (a.bits != 4 || a.slots != 0 || a.M < 2 || a.K % 128 != 0) return false;
  if (a.affine && 2 * a.spr > 8 * 64) return false;  // the bias term's steps ride on the units sent past the end: at most 2*KH*(D-1)
  const uint64_t lim = 1ull << 32;
  return (uint64_t)a.N * a.k_packed * 4 < lim && (uint64_t)a.N * a.spr * 2 < lim && (uint64_t)a.M * a.K * 2 < lim &&
         (uint64_t)a.M * (2 * a.spr + 64) * 2 < lim;  // the last: rows of group sums, at most 2*spr + 63 wide
}

// k splits: workgroups enough for one round over the CUs, each split at least two units per k part
uint32_t skinny_dma_ksplit(const MatmulArgs& a, const Tune& t) {
  if (a.N % 4) return 1;  // the reduction works on groups of four outputs
  const Shape sh = shape_of(a, t);
  const uint32_t nunits = a.K / 128;
  uint32_t want;
  if (t.skinny_ksplit > 0) {
    want = (uint32_t)t.skinny_ksplit;
  } else {
    const uint32_t tiles = ((a.N + 32 * sh.nw - 1) / (32 * sh.nw)) * ((a.M + 32 * sh.mb - 1) / (32 * sh.mb));
    want = (uint32_t)t.num_cus / tiles;
    if (want > 16) want = 16;
    if (want > nunits / (2 * sh.kh)) want = nunits / (2 * sh.kh);
  }
  if (want > nunits) want = nunits;
  if (want < 1) want = 1;
  // every split must own at least one unit: with ups = ceil(nunits / want), split want-1 starts at (want-1)*ups
  while (want > 1 && (want - 1) * ((nunits + want - 1) / want) >= nunits) want--;
  return want;
}



hipError_t launch_skinny_dma(StreamParams& p, const MatmulArgs& a, const Tune& t, hipStream_t s) {
  const Shape sh = shape_of(a, t);
  p.mtiles = (a.M + 32 * sh.mb - 1) / (32 * sh.mb);
  p.ngroups = (a.N + 32 * sh.nw - 1) / (32 * sh.nw);
  p.ksplit = skinny_dma_ksplit(a, t);
  const uint32_t nunits = a.K / 128;
  p.steps_per_split = 2 * ((nunits + p.ksplit - 1) / p.ksplit);
  return a.affine ? launch_affine<true>(p, sh, s) : launch_affine<false>(p, sh, s);
}

}  // namespace ztvm
