// Dense decode GEMV, one activation row: y[n] = sum_k x[k] * w[n,k], 4-bit (affine g64 / symmetric g32) and
// 3-bit (affine g64) rows. Same arithmetic as gemv.hip (the generator's factored form
// s*dot(x,q) + b*sum(x), src/compiler/shaders/int4_matmul.gen.ts:78-84, :401-406; exact f16 integers,
// f32 accumulation), built for the launch this dispatch really is: 33 MB of weights, one vector of
// activations, 5 microseconds.
//
// What the measurements behind this layout said (K=4096, N=14336, one launch after another):
//   * the dot products are not the bound once they leave the vector ALU: v_mfma_f32_4x4x4_16b_f16 is sixteen
//     independent 4x4x4 products, one per 4 lanes. Lane j of a block supplies ITS 4 weights as column j of B and
//     ITS 4 activations as row j of A, so D[j][j] (register j of lane j) is the lane's own 4-term dot product:
//     the sixteen dot2 instructions of a 32-value chunk become eight matrix-core instructions and one
//     three-instruction select of the diagonal.
//   * the activations are the critical path of the launch, not the weights: every wave needs all of x before its
//     first dot product, and x comes from memory each launch (the weight stream of the launch before has pushed
//     it out of L2): about 1.2 microseconds after the first wave starts, later if weight loads are queued in
//     front of it. So the workgroup's very first memory instructions fetch x (one 16-byte piece per thread), a
//     barrier keeps every weight load of the CU behind them, and the ring of weight loads a wave keeps in flight
//     is shallow: two passes (2 KB per wave, 32 KB per CU). One pass in flight leaves the memory system idle
//     between a wave's steps; three or more delay the activations of workgroups that start a few hundred
//     nanoseconds later by more than they gain (measured at K=4096, N=14336: 8.5 / 7.7 / 8.9 us for 1 / 2 / 3).
//     Every pass in flight is three memory instructions per wave, 48 per CU, that the CU's address unit takes
//     one after the other before any wave gets to its activations: each pass of depth costs 0.25-0.35 us of
//     start-up (with the arithmetic taken out: 7.23 / 7.47 / 7.71 us for 1 / 2 / 3). Neither is it the
//     first burst that costs: a third and fourth pass requested only after the activations had landed measured
//     like the deeper ring (8.3 / 9.0 us), and so did a deeper ring whose unrolled turn no longer runs past the
//     wave's last row (8.2 us).
//   * the vector ALU is not the bound either: feeding the nibbles to the matrix cores as f16 subnormals (q * 2^-24:
//     one AND per pair, no OR constant, no subtraction; 50 instead of 58 vector instructions per chunk) bought
//     0.1 us, and is not exact: the matrix cores take subnormal operands, but a chain of them is not scale
//     invariant (sums of products near 2^-21 lose bits below about 2^-40: 2^-18 relative per chunk).
//   * x lives in registers: a lane always works on the same chunk index of its row part, so its 64 bytes of
//     activations per pass are loaded from LDS once per kernel, not once per row. A wave holds at most two
//     passes (4096 values) of a row; longer rows are shared by 2, 4 or 8 waves of the workgroup ("k parts")
//     whose partial sums meet in LDS in part order, so a row's result does not depend on timing.
//   * rows are dealt to waves as balanced contiguous ranges fixed at launch (no tile loop, no tail wave), sixteen
//     waves per CU, one workgroup per CU.
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

constexpr int WAVES = 16;
constexpr uint32_t MAX_ROWS_PER_WORKER = 256;  // LDS slots for the partial sums of one row worker

struct StreamGemvParams {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  uint32_t N, k_packed, spr, nchunks, out_f32;
};

constexpr int gcd_of(int a, int b) { return b == 0 ? a : gcd_of(b, a % b); }

// NPW: 2048-value passes per wave and row; KPARTS: waves sharing a row; RING: passes in flight per wave
template <int BITS, bool AFFINE, int NPW, int KPARTS, int RING>
__global__ __launch_bounds__(WAVES * 64) void gemv_stream_kernel(const StreamGemvParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int WPC = BITS == 4 ? 4 : 3;       // words per 32-value chunk
  constexpr int RG = WAVES / KPARTS;           // row workers per workgroup
  constexpr int NPT = NPW * KPARTS;            // passes that cover a row
  constexpr int U = NPW * RING / gcd_of(NPW, RING);  // steps until (pass, ring slot) repeats
  constexpr uint32_t NOWHERE = 0x80000000u;    // a buffer offset past every array: the load returns zeros

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t kpart = wave % KPARTS, rg = wave / KPARTS;

  // ---- 1. x first: one 16-byte piece per thread and turn ----
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(p.in), 0, p.nchunks * 64u, 0x00020000);
  constexpr int NPIECE = NPT * 256, XT = (NPIECE + WAVES * 64 - 1) / (WAVES * 64);
  u32x4 xin[XT];
#pragma unroll
  for (int t = 0; t < XT; t++) {
    const uint32_t pc = t * WAVES * 64 + tid;  // piece = chunk * 4 + quarter
    xin[t] = __builtin_amdgcn_raw_buffer_load_b128(xres, pc < p.nchunks * 4u ? pc * 16u : NOWHERE, 0, 0);
  }
  __builtin_amdgcn_s_barrier();  // no weight load of this CU is issued before the last x load (without it: 8.1-8.4 us against 7.6-7.7)

  // ---- 2. this wave's rows and its ring of loads ----
  // row workers: (row group, workgroup), neighbours in the numbering sit on different CUs
  const uint32_t workers = gridDim.x * RG, wk = rg * gridDim.x + blockIdx.x;
  const uint32_t base = p.N / workers, rem = p.N % workers;
  const uint32_t r0 = wk * base + (wk < rem ? wk : rem), R = base + (wk < rem ? 1u : 0u);

  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(p.weights), 0, p.N * p.k_packed * 4u, 0x00020000);
  const __amdgpu_buffer_rsrc_t sres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(p.scales), 0, p.N * p.spr * 2u, 0x00020000);
  const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(AFFINE ? p.biases : p.scales), 0, p.N * p.spr * 2u, 0x00020000);
  const uint32_t row_wbytes = p.k_packed * 4u, row_sbytes = p.spr * 2u;
  // the lane's place inside a pass never changes; chunks past the end of the row are sent nowhere
  uint32_t voff[NPW], soff[NPW];
#pragma unroll
  for (int ps = 0; ps < NPW; ps++) {
    const uint32_t c = (kpart * NPW + ps) * 64u + lane;
    const bool in_k = c < p.nchunks;
    voff[ps] = in_k ? c * (WPC * 4u) : NOWHERE;
    soff[ps] = in_k ? (AFFINE ? (c >> 1) : c) * 2u : NOWHERE;
  }

  struct Frag {
    uint32_t w[4];
    _Float16 s, b;
  };
  // A step is one pass of one row: step t = row * NPW + pass, in ring slot t % RING. The ring is shallow on
  // purpose (see the head of the file); U steps later both the pass and the slot of a step repeat, so the
  // loop body below is U steps with every register index known at compile time.
  Frag ring[RING];
  auto issue = [&](int slot, int ps, uint32_t rr) __attribute__((always_inline)) {
    const bool ok = rr < R;  // past the wave's last row: fetch nothing
    const uint32_t row = r0 + rr;
    const uint32_t vo = ok ? voff[ps] : NOWHERE, so = ok ? soff[ps] : NOWHERE;
    if (BITS == 4) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(wres, vo, row * row_wbytes, 2);  // 2: non-temporal
      ring[slot].w[0] = v.x; ring[slot].w[1] = v.y; ring[slot].w[2] = v.z; ring[slot].w[3] = v.w;
    } else {
      const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(wres, vo, row * row_wbytes, 2);
      ring[slot].w[0] = v.x; ring[slot].w[1] = v.y; ring[slot].w[2] = v.z; ring[slot].w[3] = 0;
    }
    ring[slot].s = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(sres, so, row * row_sbytes, 0));
    if (AFFINE) ring[slot].b = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(bres, so, row * row_sbytes, 0));
  };
#pragma unroll
  for (int t = 0; t < RING; t++) issue(t, t % NPW, (uint32_t)(t / NPW));

  // ---- 3. x into LDS in the unpackers' slot order [v0,v4 | v1,v5 | v2,v6 | v3,v7], piece sums beside it ----
  u32x4* xs_pieces = reinterpret_cast<u32x4*>(smem);
  float* psum = reinterpret_cast<float*>(smem + (size_t)NPIECE * 16u);
  float* part = psum + NPIECE;  // [KPARTS][RG][MAX_ROWS_PER_WORKER] when KPARTS > 1
#pragma unroll
  for (int t = 0; t < XT; t++) {
    const uint32_t pc = t * WAVES * 64 + tid;
    if (pc < (uint32_t)NPIECE) {
      const h2 a = as_h2(xin[t].x), b = as_h2(xin[t].y), c = as_h2(xin[t].z), d = as_h2(xin[t].w);
      u32x4 o;
      o.x = as_u32((h2){a.x, c.x}); o.y = as_u32((h2){a.y, c.y}); o.z = as_u32((h2){b.x, d.x}); o.w = as_u32((h2){b.y, d.y});
      const uint32_t ch = pc >> 2, q = pc & 3u, at = (ch >> 6) * 256u + q * 64u + (ch & 63u);
      xs_pieces[at] = o;
      psum[at] = (((float)a.x + (float)a.y) + ((float)b.x + (float)b.y)) + (((float)c.x + (float)c.y) + ((float)d.x + (float)d.y));
    }
  }
  __syncthreads();
  h2 xv[NPW][16];
  float xs[NPW];
#pragma unroll
  for (int ps = 0; ps < NPW; ps++) {
    const uint32_t pass = kpart * NPW + ps;
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const u32x4 v = xs_pieces[pass * 256u + q * 64u + lane];
      xv[ps][4 * q + 0] = as_h2(v.x); xv[ps][4 * q + 1] = as_h2(v.y); xv[ps][4 * q + 2] = as_h2(v.z); xv[ps][4 * q + 3] = as_h2(v.w);
      s += psum[pass * 256u + q * 64u + lane];
    }
    xs[ps] = s;
  }

  // OR constants in vector registers, so that (w & mask) | c is one v_and_or_b32 (written in plain C: the
  // compiler then knows the wait states a matrix-core instruction needs after the instruction that wrote its operand)
  uint32_t c1024, c64;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(c1024));
  asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(c64));
  const h2 k1024 = {(_Float16)1024.f, (_Float16)1024.f}, k64 = {(_Float16)64.f, (_Float16)64.f};
  UnpackConsts kc;
  if (BITS == 3) kc.init();
  const bool odd = (lane & 1u) != 0, upper = (lane & 2u) != 0;

  // ---- 4. steps: consume a slot, refill it with the step RING later. Steps past the wave's last row run on
  // the zeros their loads returned and store nothing: no branch sits between a load and its use ----
  float acc = 0.f;
  for (uint32_t rbase = 0; rbase < R; rbase += U / NPW) {
#pragma unroll
    for (int i = 0; i < U; i++) {
      const int ps = i % NPW, slot = i % RING;
      const uint32_t rr = rbase + i / NPW;
      const Frag f = ring[slot];
      issue(slot, (i + RING) % NPW, rbase + (i + RING) / NPW);
      h2 q[16];
      if (BITS == 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const uint32_t w = f.w[j], w8 = w >> 8;
          q[4 * j + 0] = as_h2((w & 0x000F000Fu) | c1024) - k1024;   // v0, v4
          q[4 * j + 1] = as_h2((w & 0x00F000F0u) | c64) - k64;       // v1, v5
          q[4 * j + 2] = as_h2((w8 & 0x000F000Fu) | c1024) - k1024;  // v2, v6
          q[4 * j + 3] = as_h2((w8 & 0x00F000F0u) | c64) - k64;      // v3, v7
        }
      } else {
        unpack3_chunk(f.w[0], f.w[1], f.w[2], q, kc);
      }
      f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 16; j += 2) {
        const h4 qa = {q[j].x, q[j].y, q[j + 1].x, q[j + 1].y};
        const h4 xa = {xv[ps][j].x, xv[ps][j].y, xv[ps][j + 1].x, xv[ps][j + 1].y};
        d = __builtin_amdgcn_mfma_f32_4x4x4f16(xa, qa, d, 0, 0, 0);
      }
      const float lo = odd ? d[1] : d[0], hi = odd ? d[3] : d[2];
      const float dot = upper ? hi : lo;  // the block's diagonal: this lane's own products
      const float sc = (float)f.s;
      acc += AFFINE ? __builtin_fmaf(sc, dot, (float)f.b * xs[ps]) : sc * __builtin_fmaf(-7.f, xs[ps], dot);
      if (ps == NPW - 1) {
        const float total = group_sum_to_last_lane<64>(acc);
        acc = 0.f;
        if (lane == 63 && rr < R) {
          if (KPARTS == 1) {
            if (p.out_f32) reinterpret_cast<float*>(p.out)[r0 + rr] = total;
            else reinterpret_cast<_Float16*>(p.out)[r0 + rr] = (_Float16)total;
          } else {
            part[(kpart * RG + rg) * MAX_ROWS_PER_WORKER + rr] = total;
          }
        }
        // the wave's last row leaves the unrolled turn here (an exit, not a join: the waits of the steps before it
        // stay as they are), so a ring deeper than a row does not run steps on rows that do not exist
        if (U > NPW && rr + 1 >= R) goto rows_done;
      }
    }
  }
rows_done:

  // ---- 5. k parts meet: part 0's wave adds the parts in part order, one row per lane ----
  if (KPARTS > 1) {
    __syncthreads();
    if (kpart == 0) {
      for (uint32_t rr = lane; rr < R; rr += 64) {
        float total = 0.f;
#pragma unroll
        for (int kp = 0; kp < KPARTS; kp++) total += part[(kp * RG + rg) * MAX_ROWS_PER_WORKER + rr];
        if (p.out_f32) reinterpret_cast<float*>(p.out)[r0 + rr] = total;
        else reinterpret_cast<_Float16*>(p.out)[r0 + rr] = (_Float16)total;
      }
    }
  }
}

template <int BITS, bool AFFINE, int NPW, int KPARTS>
hipError_t launch_shape(const StreamGemvParams& p, uint32_t grid, int ring, hipStream_t s) {
  constexpr size_t smem = (size_t)NPW * KPARTS * 256 * 20 + (KPARTS > 1 ? (size_t)WAVES * MAX_ROWS_PER_WORKER * 4 : 0);
  auto go = [&](auto k) {
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, dim3(grid), dim3(WAVES * 64), smem, s, p);
  };
  if (ring == 3) go(gemv_stream_kernel<BITS, AFFINE, NPW, KPARTS, 3>);
  else if (ring == 1) go(gemv_stream_kernel<BITS, AFFINE, NPW, KPARTS, 1>);
  else go(gemv_stream_kernel<BITS, AFFINE, NPW, KPARTS, 2>);
  return hipGetLastError();
}

// passes per row -> waves per row: a wave takes at most two passes of a row (64 bytes of activations per lane
// and pass stay in registers; more passes per wave measured slower than more waves per row)
constexpr uint32_t kparts_of(uint32_t passes) { return passes <= 2 ? 1u : (passes <= 4 ? 2u : (passes <= 8 ? 4u : 8u)); }

template <int BITS, bool AFFINE>
hipError_t launch_fmt(const StreamGemvParams& p, uint32_t passes, uint32_t grid, int ring, hipStream_t s) {
  if (passes == 1) return launch_shape<BITS, AFFINE, 1, 1>(p, grid, ring, s);
  switch (kparts_of(passes)) {
    case 1: return launch_shape<BITS, AFFINE, 2, 1>(p, grid, ring, s);
    case 2: return launch_shape<BITS, AFFINE, 2, 2>(p, grid, ring, s);
    case 4: return launch_shape<BITS, AFFINE, 2, 4>(p, grid, ring, s);
    default: return launch_shape<BITS, AFFINE, 2, 8>(p, grid, ring, s);
  }
}

uint32_t passes_of(const MatmulArgs& a) { return (a.K / 32u + 63u) / 64u; }

}  // namespace

// One dense activation row, 4-bit or 3-bit rows of at most sixteen passes, and few enough rows per row worker
// for the LDS slots of a split row.
bool gemv_stream_supports(const MatmulArgs& a, const Tune& t) {
  if (a.slots != 0 || a.up_weights || a.qkv || a.delta) return false;
  if (!(a.bits == 4 || (a.bits == 3 && a.affine))) return false;
  if (a.K == 0 || a.K % 32u) return false;
  // buffer resources carry 32-bit byte counts, and the out-of-range offset that stands for "no row" (2 GiB) must lie
  // past every array for its loads to return zeros
  const uint64_t lim = 1ull << 31;
  if ((uint64_t)a.N * a.k_packed * 4 >= lim || (uint64_t)a.N * a.spr * 2 >= lim) return false;
  const uint32_t passes = passes_of(a);
  if (passes > 16) return false;
  const uint32_t kparts = kparts_of(passes);
  const uint32_t workers = (uint32_t)t.num_cus * (WAVES / kparts);
  return kparts == 1 || (a.N + workers - 1) / workers <= MAX_ROWS_PER_WORKER;
}

hipError_t launch_gemv_stream(const MatmulArgs& a, const Tune& t, hipStream_t s) {
  if (!gemv_stream_supports(a, t)) return hipErrorInvalidValue;
  StreamGemvParams p{};
  p.out = a.out; p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases;
  p.N = a.N; p.k_packed = a.k_packed; p.spr = a.spr; p.nchunks = a.K / 32u; p.out_f32 = a.out_f32;
  const uint32_t passes = passes_of(a);
  // one workgroup per CU; fewer when there are not enough rows to give every row worker one
  const uint32_t rg = WAVES / kparts_of(passes);
  uint32_t grid = (uint32_t)t.num_cus;
  const uint32_t needed = (a.N + rg - 1) / rg;
  if (grid > needed) grid = needed;
  // passes in flight per wave: two, also where a wave streams dozens of rows (K=2048 N=248320: 55-61 us against
  // 57-63 with three; K=4096 N=128256: 52.6 against 57.4)
  const int ring = t.gemv_ring ? t.gemv_ring : 2;
  if (a.bits == 3) return launch_fmt<3, true>(p, passes, grid, ring, s);
  return a.affine ? launch_fmt<4, true>(p, passes, grid, ring, s) : launch_fmt<4, false>(p, passes, grid, ring, s);
}

}  // namespace ztvm
