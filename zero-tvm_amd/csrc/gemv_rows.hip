// Streaming GEMV for a handful of activation rows (1 <= M <= 16):
//   Y[m,n] = sum_k A[m,k] * w[n,k],  w = s*q + b (4-, 3- or 8-bit, group 64) or s*(q-7) (4-bit, group 32).
//
// Replaces the reference's fixed small-batch kernels for the dispatches that carry a few rows at
// once (src/compiler/shaders/int4_matmul.gen.ts: int4MatmulBatchedWGSL :430-540, entry
// int4_matmul_batched_m4, and int4MatmulBatchedDynWGSL :580-695 at M_ROWS of a speculative
// verify step; call sites src/zero-tvm/engine-core.ts:4280-4293). Those unpack a word once and
// reuse it for four rows; here the reuse happens on the matrix cores while the memory side stays
// the GEMV's: every weight is read once, in 256-byte runs per row.
//
//   * v_mfma_f32_4x4x4_16b_f16 is sixteen independent 4x4x4 products. Block b = lane / 4 works on
//     one 32-k chunk; inside a block lane j supplies, as the B column, four exact f16 integers of
//     ITS weight row (row 4*tile + j) and, as the A row, four activations of row m = 4*group + j.
//     After the eight instructions of a chunk, register i of lane (b, j) holds
//     dot(x[4*group + i, chunk], q[row j, chunk]): the lane that loaded a weight row owns that
//     row's sums for four activation rows, so its scale and bias apply as per-lane scalars
//     exactly as in the GEMV:  acc += s*dot + b*sum(x)  (affine),  s*(dot - 7*sum(x))  (symmetric).
//   * a wave pass covers 4 rows x 16 chunks; the sixteen blocks are summed across lanes once per
//     row tile. Activation rows beyond four are further A operands against the same B registers.
//   * activations are staged once per workgroup in LDS, in the unpackers' slot order, with the
//     per-chunk sums; rows past M and chunks past K are staged as zeros, so no lane diverges.
//   * K ranges too long for LDS are dealt to several workgroups (grid y); the f32 partial results
//     are summed in range order by the same reduction the 32-row kernel uses. The split depends on
//     K only, and a row's arithmetic does not depend on how many rows travel with it.
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

constexpr int PASS = 16;              // chunks per wave pass = blocks of the 4x4x4 instruction
constexpr int UNROLL = 2;             // passes per pipeline stage: two loads per lane go out together
constexpr int STEP = PASS * UNROLL;   // chunks per stage; staged k ranges are padded to whole stages
constexpr uint32_t LDS_ROW_BUDGET = 72 * 1024 / 8;  // bytes of LDS a staged activation row may take (8 rows: 72 KB)

struct RowsParams {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  float* partial;  // [ksplit][M][N] when ksplit > 1
  uint32_t M, N, K, k_packed, spr, nchunks, cps, ksplit, ntiles, out_f32;
};

typedef uint32_t words3 __attribute__((ext_vector_type(3), aligned(4)));

template <int WORDS>
struct RowFrag {
  uint32_t w[UNROLL][WORDS];
  _Float16 s[UNROLL], b[UNROLL];
};

template <int CTRL>
__device__ __forceinline__ float row_shr_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int BITS, bool AFFINE, int MG>
__global__ __launch_bounds__(1024) void rows_kernel(const RowsParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int M4 = MG * 4;
  constexpr int WPC = BITS == 8 ? 8 : (BITS == 4 ? 4 : 3);  // words per chunk
  constexpr int FW = BITS == 8 ? 8 : 4;

  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = tid >> 6, waves = blockDim.x >> 6;
  const uint32_t j = lane & 3u, b = lane >> 2;

  // this workgroup's chunks of every row
  const uint32_t c_begin = blockIdx.y * p.cps;
  const uint32_t c_count = p.nchunks - c_begin < p.cps ? p.nchunks - c_begin : p.cps;
  const uint32_t npasses = (c_count + STEP - 1) / STEP;  // pipeline stages per row tile
  const uint32_t cpad = npasses * STEP;

  // LDS: 16-byte pieces of x at ((group*4 + piece)*cpad + chunk)*4 + row%4, so the 64 lanes of a
  // read touch 64 consecutive pieces; then float sums at [chunk][row]
  h8* x_pieces = reinterpret_cast<h8*>(smem);
  float* xsum = reinterpret_cast<float*>(smem + (size_t)M4 * cpad * 64u);

  UnpackConsts kc;
  kc.init();

  auto issue = [&](RowFrag<FW>& f, uint32_t tile, uint32_t pass) {
    uint32_t row = tile * 4 + j;
    row = row < p.N ? row : p.N - 1;  // a clamped row is never stored
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      uint32_t cl = pass * STEP + u * PASS + b;
      cl = cl < c_count ? cl : c_count - 1;  // a clamped chunk meets staged zeros
      const uint32_t c = c_begin + cl;
      const uint32_t g = AFFINE ? (c >> 1) : c;
      const uint32_t* wp = p.weights + (size_t)row * p.k_packed + (size_t)c * WPC;
      if (BITS == 8) {
        const u32x4 v0 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp));
        const u32x4 v1 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp) + 1);
        f.w[u][0] = v0.x; f.w[u][1] = v0.y; f.w[u][2] = v0.z; f.w[u][3] = v0.w;
        f.w[u][4 % FW] = v1.x; f.w[u][5 % FW] = v1.y; f.w[u][6 % FW] = v1.z; f.w[u][7 % FW] = v1.w;
      } else if (BITS == 4) {
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp));
        f.w[u][0] = v.x; f.w[u][1] = v.y; f.w[u][2] = v.z; f.w[u][3] = v.w;
      } else {
        const words3 v = __builtin_nontemporal_load(reinterpret_cast<const words3*>(wp));
        f.w[u][0] = v.x; f.w[u][1] = v.y; f.w[u][2] = v.z; f.w[u][3] = 0;
      }
      f.s[u] = p.scales[(size_t)row * p.spr + g];
      if (AFFINE) f.b[u] = p.biases[(size_t)row * p.spr + g];
    }
  };

  const uint32_t wave_stride = gridDim.x * waves;
  uint32_t tile = blockIdx.x * waves + wave, pass = 0;
  bool have = tile < p.ntiles;
  RowFrag<FW> fa, fb;
  issue(fa, have ? tile : p.ntiles - 1, 0);  // the weight stream starts while x is staged

  // ---- stage x: one (row, chunk) per thread and turn, two turns in flight. Only the M real rows are
  // staged: row i of a 4x4x4 product depends on row i of A alone, so what the unused rows of a
  // group hold (anything) stays in sums that are never stored.
  {
    const uint32_t pairs = p.M * cpad;
    auto place = [&](uint32_t idx, const h8 (&v)[4], bool real) __attribute__((always_inline)) {
      const uint32_t m = idx / cpad, cl = idx - m * cpad;
      float s = 0.f;
#pragma unroll
      for (int piece = 0; piece < 4; piece++) {
        h8 o;
#pragma unroll
        for (int sl = 0; sl < 8; sl++) o[sl] = real ? v[piece][BITS == 8 ? value_in_slot8(sl) : value_in_slot(sl)] : (_Float16)0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) s += (float)v[piece][i];
        x_pieces[(((m >> 2) * 4 + piece) * cpad + cl) * 4 + (m & 3u)] = o;
      }
      xsum[cl * M4 + m] = real ? s : 0.f;
    };
    auto fetch = [&](uint32_t idx, h8 (&v)[4]) __attribute__((always_inline)) {
      // chunks past the end of the range (padding of the last pass) read the row's last real chunk and are staged as zeros
      const uint32_t m = idx / cpad, cl = idx - m * cpad;
      const uint32_t cc = cl < c_count ? cl : c_count - 1;
      const h8* src = reinterpret_cast<const h8*>(p.in + (size_t)m * p.K + (size_t)(c_begin + cc) * 32u);
#pragma unroll
      for (int piece = 0; piece < 4; piece++) v[piece] = src[piece];
      return cl < c_count;
    };
    for (uint32_t idx = tid; idx < pairs; idx += 2 * blockDim.x) {
      h8 v0[4], v1[4];
      const uint32_t idx1 = idx + blockDim.x;
      const bool two = idx1 < pairs;
      const bool r0 = fetch(idx, v0);
      const bool r1 = fetch(two ? idx1 : idx, v1);
      place(idx, v0, r0);
      if (two) place(idx1, v1, r1);
    }
  }
  __syncthreads();

  float acc[M4];
#pragma unroll
  for (int r = 0; r < M4; r++) acc[r] = 0.f;

  // the x pieces and chunk sums of one group of four activation rows for this lane's chunk
  struct XGroup {
    h8 v[4];
    f4 sum;
  };
  auto read_x = [&](XGroup& g, uint32_t cl, int mg) __attribute__((always_inline)) {
#pragma unroll
    for (int w = 0; w < 4; w++) g.v[w] = x_pieces[((mg * 4 + w) * cpad + cl) * 4 + j];
    g.sum = *reinterpret_cast<const f4*>(xsum + cl * M4 + mg * 4);
  };

  auto stage = [&](const RowFrag<FW>& cur, RowFrag<FW>& nxt) {
    uint32_t ntile = tile, npass = pass + 1;
    if (npass == npasses) { npass = 0; ntile += wave_stride; }
    const bool nhave = ntile < p.ntiles;
    // always issued (past the end: the last tile again, never consumed): loads under a branch would
    // make every wait below drain the loads just issued as well
    issue(nxt, nhave ? ntile : p.ntiles - 1, npass);
    XGroup xa, xb;
    read_x(xa, pass * STEP + b, 0);
    __builtin_amdgcn_sched_barrier(0);  // loads and LDS reads first; the unpack below covers their latency

#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const uint32_t cl = pass * STEP + u * PASS + b;
      h2 q[16];
      if constexpr (BITS == 8) unpack8_chunk(cur.w[u], q, kc);
      else if constexpr (BITS == 4) unpack4_chunk(cur.w[u][0], cur.w[u][1], cur.w[u][2], cur.w[u][3], q, kc);
      else unpack3_chunk(cur.w[u][0], cur.w[u][1], cur.w[u][2], q, kc);
      const float s = (float)cur.s[u];
      const float bias = AFFINE ? (float)cur.b[u] : 0.f;
      auto group = [&](const XGroup& x, int mg) __attribute__((always_inline)) {
        f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < 4; w++) {
          const h8 xv = x.v[w];
          const h4 xlo = {xv[0], xv[1], xv[2], xv[3]}, xhi = {xv[4], xv[5], xv[6], xv[7]};
          const h4 qlo = {q[4 * w].x, q[4 * w].y, q[4 * w + 1].x, q[4 * w + 1].y};
          const h4 qhi = {q[4 * w + 2].x, q[4 * w + 2].y, q[4 * w + 3].x, q[4 * w + 3].y};
          d0 = __builtin_amdgcn_mfma_f32_4x4x4f16(xlo, qlo, d0, 0, 0, 0);
          d1 = __builtin_amdgcn_mfma_f32_4x4x4f16(xhi, qhi, d1, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float dot = d0[i] + d1[i];
          acc[mg * 4 + i] += AFFINE ? __builtin_fmaf(s, dot, bias * x.sum[i]) : s * __builtin_fmaf(-7.f, x.sum[i], dot);
        }
      };
      // groups alternate between two register sets: the next pieces (the next group's, or the next
      // chunk's first group) are read while this group multiplies
#pragma unroll
      for (int mg = 0; mg < MG; mg++) {
        XGroup& now = (u * MG + mg) % 2 ? xb : xa;
        XGroup& then = (u * MG + mg) % 2 ? xa : xb;
        if (mg + 1 < MG) read_x(then, cl, mg + 1);
        else if (u + 1 < UNROLL) read_x(then, cl + PASS, 0);
        group(now, mg);
      }
    }

    if (pass == npasses - 1) {
      // the sixteen blocks of a row sit in lanes j, j+4, .., j+60: two row shifts leave the sum of a
      // 16-lane row's four blocks in its lanes 12..15, two exchanges add the four rows
      float v[M4];
#pragma unroll
      for (int r = 0; r < M4; r++) {
        v[r] = row_shr_add<0x118>(row_shr_add<0x114>(acc[r]));
        acc[r] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < M4; r++) v[r] += __shfl_xor(v[r], 16);
#pragma unroll
      for (int r = 0; r < M4; r++) v[r] += __shfl_xor(v[r], 32);
      const uint32_t n = tile * 4 + j;
      if (b == 15 && n < p.N) {
#pragma unroll
        for (int r = 0; r < M4; r++) {
          if ((uint32_t)r < p.M) {
            if (p.ksplit > 1) p.partial[((size_t)blockIdx.y * p.M + r) * p.N + n] = v[r];
            else if (p.out_f32) reinterpret_cast<float*>(p.out)[(size_t)r * p.N + n] = v[r];
            else reinterpret_cast<_Float16*>(p.out)[(size_t)r * p.N + n] = (_Float16)v[r];
          }
        }
      }
    }
    tile = ntile; pass = npass; have = nhave;
  };

  while (have) {
    stage(fa, fb);
    if (!have) break;
    stage(fb, fa);
  }
}

uint32_t chunks_per_split(uint32_t nchunks) {
  const uint32_t most = LDS_ROW_BUDGET / 68u / STEP * STEP;  // 68 bytes of LDS per staged chunk and row
  const uint32_t ksplit = (nchunks + most - 1) / most;
  return ((nchunks + ksplit - 1) / ksplit + STEP - 1) / STEP * STEP;
}

template <int BITS, bool AFFINE>
hipError_t launch_groups(const RowsParams& p, int mg, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
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
  const uint32_t nchunks = a.K / 32, cps = chunks_per_split(nchunks);
  return (nchunks + cps - 1) / cps;
}

// Dense, up to 16 rows, whole 32-k chunks; a split k range needs groups of four outputs for its reduction.
bool rows_supports(const MatmulArgs& a) {
  if (a.slots != 0 || a.M < 1 || a.M > 16 || a.K % 32 != 0 || a.K == 0) return false;
  if (!(a.bits == 4 || ((a.bits == 3 || a.bits == 8) && a.affine))) return false;
  if (a.affine && a.K % 64 != 0) return false;
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
  p.nchunks = a.K / 32;
  p.cps = chunks_per_split(p.nchunks);
  p.ksplit = (p.nchunks + p.cps - 1) / p.cps;
  p.ntiles = (a.N + 3) / 4;
  p.out_f32 = a.out_f32;
  const int mg = (int)(a.M + 3) / 4;
  const size_t smem = (size_t)mg * 4 * p.cps * 68;  // cps is a whole number of stages

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
  if (a.bits == 3) e = launch_groups<3, true>(p, mg, grid, threads, smem, s);
  else if (a.bits == 8) e = launch_groups<8, true>(p, mg, grid, threads, smem, s);
  else if (a.affine) e = launch_groups<4, true>(p, mg, grid, threads, smem, s);
  else e = launch_groups<4, false>(p, mg, grid, threads, smem, s);
  if (e != hipSuccess) return e;
  if (p.ksplit > 1) return launch_reduce_partials(p.partial, a.out, a.M * a.N, p.ksplit, a.out_f32 != 0, s);
  return hipSuccess;
}

}  // namespace ztvm
