// Streaming GEMV for a handful of activation rows (1 <= M <= 16):
//   Y[m,n] = sum_k A[m,k] * w[n,k],  w = s*q + b (4-, 3- or 8-bit, group 64) or s*(q-7) (4-bit, group 32).
//
// Replaces the reference's fixed small-batch kernels for the dispatches that carry a few rows at
// once (src/compiler/shaders/int4_matmul.gen.ts: int4MatmulBatchedWGSL :430-540, entry
// int4_matmul_batched_m4, and int4MatmulBatchedDynWGSL :580-695 at M_ROWS of a speculative
// verify step; call sites src/zero-tvm/engine-core.ts:4280-4293). Those unpack a word once and
// reuse it for four rows; here the reuse happens on the matrix cores while the memory side stays
// the GEMV's: every weight is read once, in runs of 512 bytes and more per row.
//
//   * the unit of work of a lane is one scale group of one weight row (64 k affine, 32 k
//     symmetric): its packed words, one scale, one bias.
//   * v_mfma_f32_4x4x4_16b_f16 is sixteen independent 4x4x4 products. Block b = lane / 4 works on
//     one group; inside a block lane j supplies, as the B column, four exact f16 integers of ITS
//     weight row (row 4*tile + j) and, as the A row, four activations of row m = 4*set + j. After
//     the instructions of a group, register i of lane (b, j) holds
//     dot(x[4*set + i, group], q[row j, group]): the lane that loaded a weight row owns that row's
//     sums for four activation rows, so its scale and bias apply as per-lane scalars exactly as
//     in the GEMV:  acc += s*dot + b*sum(x)  (affine),  s*(dot - 7*sum(x))  (symmetric).
//   * a wave pass covers 4 rows x 16 groups; the sixteen blocks are summed across lanes once per
//     row tile. Activation rows beyond four are further A operands against the same B registers.
//   * activations are staged once per workgroup in LDS, in the unpackers' slot order, laid out
//     per pass so that every read of the loop is the lane's own 16 bytes at a compile-time
//     offset; the per-group sums sit beside them. Only the M real rows are staged: row i of a
//     4x4x4 product depends on row i of A alone, so whatever the unused rows of a set hold stays
//     in sums that are never stored.
//   * K ranges too long for LDS are dealt to several workgroups (grid y); the f32 partial results
//     are summed in range order by the same reduction the 32-row kernel uses. The split depends on
//     K only, and a row's arithmetic does not depend on how many rows travel with it.
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

constexpr int PASS = 16;                            // groups per wave pass = blocks of the 4x4x4 instruction
constexpr uint32_t LDS_ROW_BUDGET = 72 * 1024 / 8;  // bytes of LDS a staged activation row may take (8 rows: 72 KB)

struct RowsParams {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  float* partial;  // [ksplit][M][N] when ksplit > 1
  uint32_t M, N, K, k_packed, spr, nunits, ups, ksplit, ntiles, out_f32;  // units = scale groups; ups = units per split
};


template <int WORDS>
struct RowFrag {
  uint32_t w[WORDS];
  _Float16 s, b;
};

template <int CTRL>
__device__ __forceinline__ float row_shr_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int BITS, bool AFFINE, int MG>
__global__ __launch_bounds__(1024) void rows_kernel(const RowsParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int GC = AFFINE ? 2 : 1;                        // 32-k chunks per unit
  constexpr int WPC = BITS == 8 ? 8 : (BITS == 4 ? 4 : 3);  // words per chunk
  constexpr int CW = BITS == 8 ? 8 : 4;                     // registers a chunk's words take
  constexpr int PIECES = 4 * GC;                            // 16-byte pieces of x per unit and row
  constexpr uint32_t SET_BYTES = PIECES * 1024u;            // one set of four rows, one pass: PIECES x 64 lanes x 16 B
  constexpr uint32_t PASS_BYTES = MG * SET_BYTES;
  constexpr uint32_t SUM_PASS_BYTES = MG * PASS * 16u;      // per pass: [set][block] x four floats

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = tid >> 6, waves = blockDim.x >> 6;
  const uint32_t j = lane & 3u, b = lane >> 2;

  // this workgroup's units of every row
  const uint32_t u_begin = blockIdx.y * p.ups;
  const uint32_t u_count = p.nunits - u_begin < p.ups ? p.nunits - u_begin : p.ups;
  const uint32_t npasses = (u_count + PASS - 1) / PASS;
  unsigned char* const xsum_base = smem + (size_t)npasses * PASS_BYTES;

  UnpackConsts kc;
  kc.init();

  // Loads of one (tile, pass), as buffer loads: the address is a uniform descriptor plus one 32-bit
  // byte offset per lane, and an offset past the end of the array returns zeros without touching
  // memory. Rows past N are past the end by themselves (so are whole tiles past the last one: the
  // pipeline below fetches ahead without asking whether anything is left); units past the end of
  // this workgroup's k range are sent there. No lane diverges and nothing is fetched twice.
  constexpr uint32_t NOWHERE = 0x80000000u;  // every array is shorter than this (checked on the host)
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(p.weights), 0, p.N * p.k_packed * 4u, 0x00020000);
  const __amdgpu_buffer_rsrc_t sres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(p.scales), 0, p.N * p.spr * 2u, 0x00020000);
  const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(AFFINE ? p.biases : p.scales), 0, p.N * p.spr * 2u, 0x00020000);
  auto issue = [&](RowFrag<GC * CW>& f, uint32_t tile, uint32_t pass) {
    const uint32_t row = tile * 4 + j;
    const uint32_t ul = pass * PASS + b;
    const uint32_t u = u_begin + ul;
    const uint32_t woff = ul < u_count ? (row * p.k_packed + u * (GC * WPC)) * 4u : NOWHERE;
    const uint32_t soff = ul < u_count ? (row * p.spr + u) * 2u : NOWHERE;
#pragma unroll
    for (int c = 0; c < GC; c++) {
      if (BITS == 8) {
        const u32x4 v0 = __builtin_amdgcn_raw_buffer_load_b128(wres, woff + c * 32, 0, 2);  // 2: non-temporal
        const u32x4 v1 = __builtin_amdgcn_raw_buffer_load_b128(wres, woff + c * 32 + 16, 0, 2);
        f.w[c * CW + 0] = v0.x; f.w[c * CW + 1] = v0.y; f.w[c * CW + 2] = v0.z; f.w[c * CW + 3] = v0.w;
        f.w[c * CW + 4 % CW] = v1.x; f.w[c * CW + 5 % CW] = v1.y; f.w[c * CW + 6 % CW] = v1.z; f.w[c * CW + 7 % CW] = v1.w;
      } else if (BITS == 4) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(wres, woff + c * 16, 0, 2);
        f.w[c * CW + 0] = v.x; f.w[c * CW + 1] = v.y; f.w[c * CW + 2] = v.z; f.w[c * CW + 3] = v.w;
      } else {
        const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(wres, woff + c * 12, 0, 2);
        f.w[c * CW + 0] = v.x; f.w[c * CW + 1] = v.y; f.w[c * CW + 2] = v.z; f.w[c * CW + 3] = 0;
      }
    }
    f.s = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(sres, soff, 0, 0));
    if (AFFINE) f.b = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(bres, soff, 0, 0));
  };

  const uint32_t wave_stride = gridDim.x * waves;
  // Two register sets: while one (tile, pass) is consumed the next is in flight; the first goes out
  // before x is staged, so the weight stream starts while the workgroup waits for its activations.
  // (Deeper rings measured slower: a wave often owns a single row tile of four passes.)
  auto advance = [&](uint32_t& t, uint32_t& ps) __attribute__((always_inline)) {
    if (++ps == npasses) { ps = 0; t += wave_stride; }
  };
  uint32_t tile = blockIdx.x * waves + wave, pass = 0;
  bool have = tile < p.ntiles;
  RowFrag<GC * CW> fa, fb;
  issue(fa, tile, 0);

  // ---- stage x: one (row, 32-k chunk) per thread and turn; the two chunks of an affine group sit in
  // neighbouring lanes, which add their sums. Piece k of (row m, unit ul) goes to
  //   pass(ul/16) . set(m/4) . piece k . lane (ul%16)*4 + m%4,   its sum to   pass . set . block ul%16 . m%4
  {
    const uint32_t cpad = npasses * PASS * GC;  // chunks per row, padding included; even for GC = 2
    const uint32_t total = p.M * cpad, turns = (total + blockDim.x - 1) / blockDim.x;
    for (uint32_t t = 0; t < turns; t++) {      // every thread runs every turn: lanes exchange sums
      const uint32_t idx = t * blockDim.x + tid;
      const bool mine = idx < total;
      const uint32_t m = mine ? idx / cpad : 0, cl = mine ? idx - m * cpad : 0;
      const uint32_t ul = cl / GC, half = cl % GC;
      const bool real = mine && ul < u_count;  // the padding of the last pass is staged as zeros
      const h8* src = reinterpret_cast<const h8*>(p.in + (size_t)m * p.K + (size_t)(u_begin + (real ? ul : 0)) * (32u * GC) + half * 32u);
      h8 v[4];
#pragma unroll
      for (int k = 0; k < 4; k++) v[k] = src[k];
      unsigned char* dst = smem + (ul / PASS) * PASS_BYTES + (m >> 2) * SET_BYTES + half * 4096u + ((ul % PASS) * 4 + (m & 3u)) * 16u;
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        h8 o;
#pragma unroll
        for (int sl = 0; sl < 8; sl++) o[sl] = real ? v[k][BITS == 8 ? value_in_slot8(sl) : value_in_slot(sl)] : (_Float16)0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) s += (float)v[k][i];
        if (mine) *reinterpret_cast<h8*>(dst + k * 1024u) = o;
      }
      if (GC == 2) s += __shfl_xor(s, 1);
      if (mine && half == 0)
        *reinterpret_cast<float*>(xsum_base + (ul / PASS) * SUM_PASS_BYTES + (m >> 2) * (PASS * 16u) + (ul % PASS) * 16u + (m & 3u) * 4u) = real ? s : 0.f;
    }
  }
  __syncthreads();

  float acc[MG * 4];
#pragma unroll
  for (int r = 0; r < MG * 4; r++) acc[r] = 0.f;

  auto stage = [&](const RowFrag<GC * CW>& cur, RowFrag<GC * CW>& nxt) {
    // always issued, past the last tile as well (that fetches nothing): loads under a branch would
    // make every wait below drain the loads just issued as well
    uint32_t ntile = tile, npass = pass;
    advance(ntile, npass);
    issue(nxt, ntile, npass);
    __builtin_amdgcn_sched_barrier(0);  // keep the loads here: the scheduler would sink the small ones to their use

    // the lane's own 16 bytes of every piece, and its block's sums, at compile-time offsets from these two
    const unsigned char* xp = smem + pass * PASS_BYTES + lane * 16u;
    const unsigned char* sp = xsum_base + pass * SUM_PASS_BYTES + b * 16u;
    const float s = (float)cur.s;
    const float bias = AFFINE ? (float)cur.b : 0.f;
    constexpr int CHAINS = MG == 1 ? 2 : 1;  // a single set would make a group's instructions one dependent chain
    f4 d[MG], e[MG];
#pragma unroll
    for (int mg = 0; mg < MG; mg++) d[mg] = e[mg] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < GC; c++) {
      h2 q[16];
      if constexpr (BITS == 8) unpack8_chunk(cur.w + c * CW, q, kc);
      else if constexpr (BITS == 4) unpack4_chunk(cur.w[c * CW], cur.w[c * CW + 1], cur.w[c * CW + 2], cur.w[c * CW + 3], q, kc);
      else unpack3_chunk(cur.w[c * CW], cur.w[c * CW + 1], cur.w[c * CW + 2], q, kc);
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const h4 qlo = {q[4 * w].x, q[4 * w].y, q[4 * w + 1].x, q[4 * w + 1].y};
        const h4 qhi = {q[4 * w + 2].x, q[4 * w + 2].y, q[4 * w + 3].x, q[4 * w + 3].y};
#pragma unroll
        for (int mg = 0; mg < MG; mg++) {
          const h8 xv = *reinterpret_cast<const h8*>(xp + mg * SET_BYTES + (c * 4 + w) * 1024u);
          const h4 xlo = {xv[0], xv[1], xv[2], xv[3]}, xhi = {xv[4], xv[5], xv[6], xv[7]};
          d[mg] = __builtin_amdgcn_mfma_f32_4x4x4f16(xlo, qlo, d[mg], 0, 0, 0);
          if (CHAINS == 2) e[mg] = __builtin_amdgcn_mfma_f32_4x4x4f16(xhi, qhi, e[mg], 0, 0, 0);
          else d[mg] = __builtin_amdgcn_mfma_f32_4x4x4f16(xhi, qhi, d[mg], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int mg = 0; mg < MG; mg++) {
      const f4 xs = *reinterpret_cast<const f4*>(sp + mg * (PASS * 16u));
      if (CHAINS == 2) d[mg] += e[mg];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        if (AFFINE) acc[mg * 4 + i] = __builtin_fmaf(bias, xs[i], __builtin_fmaf(s, d[mg][i], acc[mg * 4 + i]));
        else acc[mg * 4 + i] = __builtin_fmaf(s, __builtin_fmaf(-7.f, xs[i], d[mg][i]), acc[mg * 4 + i]);
      }
    }

    if (pass == npasses - 1) {
      // the sixteen blocks of a row sit in lanes j, j+4, .., j+60: two row shifts leave the sum of a
      // 16-lane row's four blocks in its lanes 12..15, two exchanges add the four rows
      float v[MG * 4];
#pragma unroll
      for (int r = 0; r < MG * 4; r++) {
        v[r] = row_shr_add<0x118>(row_shr_add<0x114>(acc[r]));
        acc[r] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < MG * 4; r++) v[r] += __shfl_xor(v[r], 16);
#pragma unroll
      for (int r = 0; r < MG * 4; r++) v[r] += __shfl_xor(v[r], 32);
      const uint32_t n = tile * 4 + j;
      if (b == 15 && n < p.N) {
#pragma unroll
        for (int r = 0; r < MG * 4; r++) {
          if ((uint32_t)r < p.M) {
            if (p.ksplit > 1) p.partial[((size_t)blockIdx.y * p.M + r) * p.N + n] = v[r];
            else if (p.out_f32) reinterpret_cast<float*>(p.out)[(size_t)r * p.N + n] = v[r];
            else reinterpret_cast<_Float16*>(p.out)[(size_t)r * p.N + n] = (_Float16)v[r];
          }
        }
      }
    }
    tile = ntile; pass = npass;
    have = tile < p.ntiles;
  };

  // straight-line stages with an exit between them: a join inside the loop would merge paths with
  // different numbers of loads in flight and tighten every wait after it
  while (have) {
    stage(fa, fb);
    if (!have) break;
    stage(fb, fa);
  }
}

// bytes of LDS per staged unit and row: the pieces and one float
uint32_t unit_bytes(bool affine) { return affine ? 132u : 68u; }
uint32_t unit_k(bool affine) { return affine ? 64u : 32u; }

uint32_t units_per_split(uint32_t nunits, bool affine) {
  const uint32_t most = LDS_ROW_BUDGET / unit_bytes(affine) / PASS * PASS;
  const uint32_t ksplit = (nunits + most - 1) / most;
  return ((nunits + ksplit - 1) / ksplit + PASS - 1) / PASS * PASS;
}

template <int BITS, bool AFFINE>
hipError_t launch_sets(const RowsParams& p, int mg, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  auto go = [&](auto k) {
    if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(threads), smem, s, p);
  };
  if (mg == 1) go(rows_kernel<BITS, AFFINE, 1>);
  else if (mg == 2) go(rows_kernel<BITS, AFFINE, 2>);
  else if (mg == 3) go(rows_kernel<BITS, AFFINE, 3>);
  else go(rows_kernel<BITS, AFFINE, 4>);
  return hipGetLastError();
}

}  // namespace

uint32_t rows_ksplit(const MatmulArgs& a) {
  const uint32_t nunits = a.K / unit_k(a.affine), ups = units_per_split(nunits, a.affine);
  return (nunits + ups - 1) / ups;
}

// Dense, up to 16 rows, whole scale groups, every array within 2 GiB (32-bit byte offsets); a split
// k range needs groups of four outputs for its reduction.
bool rows_supports(const MatmulArgs& a) {
  if (a.slots != 0 || a.M < 1 || a.M > 16 || a.K == 0 || a.K % unit_k(a.affine) != 0) return false;
  if (!(a.bits == 4 || ((a.bits == 3 || a.bits == 8) && a.affine))) return false;
  if ((uint64_t)a.N * a.k_packed * 4u >= (1ull << 31)) return false;
  return rows_ksplit(a) == 1 || a.N % 4 == 0;
}

size_t rows_scratch_bytes(const MatmulArgs& a) {
  const uint32_t ks = rows_ksplit(a);
  return ks > 1 ? (size_t)ks * a.M * a.N * sizeof(float) : 0;
}

hipError_t launch_rows(const MatmulArgs& a, const Tune& t, void* scratch, hipStream_t s) {
  RowsParams p{};
  p.out = a.out; p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases;
  p.partial = reinterpret_cast<float*>(scratch);
  p.M = a.M; p.N = a.N; p.K = a.K; p.k_packed = a.k_packed; p.spr = a.spr;
  p.nunits = a.K / unit_k(a.affine);
  p.ups = units_per_split(p.nunits, a.affine);
  p.ksplit = (p.nunits + p.ups - 1) / p.ups;
  p.ntiles = (a.N + 3) / 4;
  p.out_f32 = a.out_f32;
  const int mg = (int)(a.M + 3) / 4;
  const size_t smem = (size_t)mg * 4 * p.ups * unit_bytes(a.affine);  // ups is a whole number of passes

  // workgroups: as many as LDS holds per CU (at most three); one large workgroup where the staged
  // activations are big, so that they are staged once per CU
  uint32_t per_cu = (uint32_t)(160 * 1024 / (smem + 1024));
  per_cu = per_cu < 1 ? 1 : (per_cu > 3 ? 3 : per_cu);
  uint32_t waves = 8;
  if (smem > 40 * 1024) { per_cu = 1; waves = 16; }
  if (t.rows_wg_per_cu > 0) per_cu = (uint32_t)t.rows_wg_per_cu;
  if (t.rows_waves > 0) waves = (uint32_t)t.rows_waves;
  if (waves > 16) waves = 16;
  uint32_t gx = (uint32_t)t.num_cus * per_cu / p.ksplit;
  const uint32_t wg_tiles = (p.ntiles + waves - 1) / waves;
  if (gx < 1) gx = 1;
  if (gx > wg_tiles) gx = wg_tiles;
  const dim3 grid(gx, p.ksplit, 1);
  const uint32_t threads = waves * 64;

  hipError_t e;
  if (a.bits == 3) e = launch_sets<3, true>(p, mg, grid, threads, smem, s);
  else if (a.bits == 8) e = launch_sets<8, true>(p, mg, grid, threads, smem, s);
  else if (a.affine) e = launch_sets<4, true>(p, mg, grid, threads, smem, s);
  else e = launch_sets<4, false>(p, mg, grid, threads, smem, s);
  if (e != hipSuccess) return e;
  if (p.ksplit > 1) return launch_reduce_partials(p.partial, a.out, a.M * a.N, p.ksplit, a.out_f32 != 0, s);
  return hipSuccess;
}

}  // namespace ztvm
