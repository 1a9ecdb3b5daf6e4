// Streaming GEMV for group-quantized weights, one activation row per dispatch
// unit: y[n] = sum_k x[k] * w[n,k].  HBM-bound: the weight matrix is read
// exactly once with 128-bit (4-bit) or 96-bit (3-bit) per-lane loads, unpacked
// in registers and reduced with f32 dot2 accumulation.
//
// Replaces the whole M=1 family of the reference generator
// (src/compiler/shaders/int4_matmul.gen.ts:170-571: scalar, _sg, _tiled,
// _tiled8, _vec4, _vec4h, _affine, _q3, _moe, _f32 variants) with one wave64
// design; the arithmetic kept is the generator's factored form
//   affine:    y = sum_chunks  s*dot(x,q) + b*sum(x)      (:78-84, :401-406)
//   symmetric: y = sum_chunks  s*(dot(x,q) - 7*sum(x))    (:17-19)
//
// Work decomposition
//   chunk     32 consecutive k (16 B of 4-bit weights, 12 B of 3-bit, 32 B of 8-bit): one lane-load
//   lane      owns chunk (pass*LPR + lane%LPR) of row-slot lane/LPR
//   wave      ROWS*(64/LPR) rows per step, all passes over K, then a DPP reduce
//   workgroup 4 waves; stages x once in LDS (slot-permuted, conflict-free
//             16-byte pieces) plus per-chunk sum(x), then strides over row tiles
//   grid      x: persistent workgroups over row tiles, y: (token,slot) pair for MoE
#include "internal.h"
#include "quant.h"

namespace ztvm {
namespace {

constexpr int MAX_WG_THREADS = 1024;  // 8-wave workgroups use the 512-thread build of the kernel, larger ones the 1024-thread build

struct GemvParams {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  const uint32_t* ids;
  // prologue form: `in` is the residual; x = RMSNorm(residual + delta) * gamma is formed while x is staged
  const _Float16* delta;
  const _Float16* gamma;
  float rms_eps;
  const _Float16* scales2;   // gated form: the up projection's scales / weights / biases (same shape as the gate's)
  const uint32_t* weights2;
  const _Float16* biases2;
  // QKV form: rows are RoPE pairs; the epilogue rotates and scatters into q_out / the paged KV cache
  _Float16* q_out;
  _Float16* kv_pages;
  _Float16* k_slot;  // both set: K and V rows go here, [kv_heads*head_dim] each, instead of into kv_pages
  _Float16* v_slot;
  const int32_t* position_map;
  uint32_t half_dim, head_dim, q_pairs, kv_pairs, q_dim, kv_dim;
  uint32_t page_size, kv_page_stride, head_page_stride, v_page_offset, pos_off, pages_off;
  uint64_t kv_capacity;  // f16 elements in kv_pages; a position whose slot lies past it is not written (0 = unchecked)
  float rope_theta;
  uint32_t N, k_packed, spr, nchunks, npasses, ntiles;
  uint32_t out_f32, moe;
  uint32_t slots, in_slot_stride, out_slot_stride, in_tok_stride, out_tok_stride, ids_stride, experts;
};


// LDS layout of x for chunk c: piece j (8 halves, 16 bytes) sits at 16-byte
// slot (c/64)*256 + j*64 + c%64, so the 64 lanes of one ds_read_b128 touch 64
// consecutive slots.
__device__ __forceinline__ uint32_t x_slot(uint32_t c, uint32_t j) { return (c >> 6) * 256u + j * 64u + (c & 63u); }

// One (tile, pass) worth of global loads for ROWS rows of a wave.
template <int ROWS, int WORDS>
struct Frag {
  uint32_t w[ROWS][WORDS];
  _Float16 s[ROWS], b[ROWS];
};

// GATED: every row is computed twice, against the gate matrix and against the up matrix, and the
// store is SiLU(gate) * up with both sums still in f32 (the reference's fused FFN kernel,
// src/compiler/shaders/fused_ffn.wgsl:52-140: one pass over x, one rounding at the store).
//
// QKV (a GATED launch whose second matrix is the first one shifted by half a head): "row" p is a
// rotary pair of the fused Q|K|V projection, rows row_lo(p) and row_lo(p) + half_dim of the same
// head. The pair is rotated in registers and written straight to q_out (Q) or into the paged KV
// cache (K rotated, V as is): QKV matmul + RoPE + KV append in one dispatch
// (src/compiler/shaders/qkv_fused.wgsl:41-193).
struct QkvPair {
  uint32_t group, head, dim_lo, row_lo;
};
__device__ __forceinline__ QkvPair qkv_pair(const GemvParams& p, uint32_t pair) {
  QkvPair r{0u, 0u, 0u, 0u};
  uint32_t in_group = pair, row_base = 0;
  if (in_group >= p.q_pairs) {
    r.group = 1; in_group -= p.q_pairs; row_base = p.q_dim;
    if (in_group >= p.kv_pairs) { r.group = 2; in_group -= p.kv_pairs; row_base = p.q_dim + p.kv_dim; }
  }
  r.head = in_group / p.half_dim;
  r.dim_lo = in_group - r.head * p.half_dim;
  r.row_lo = row_base + r.head * p.head_dim + r.dim_lo;
  return r;
}

//
// PROLOGUE (a GATED launch): the FFN-entry add + RMSNorm is folded into the staging of x
// (src/compiler/shaders/fused_ffn_prologue.wgsl:62-97): val = f16(residual + delta), the sum of
// val^2 in f32 over the whole row, x = f16(f32(val) * (1 / sqrt(mean + eps)) * f32(gamma)).
// Every workgroup recomputes the norm of the whole row; the add_norm dispatch and the round trip
// of the normed vector through memory disappear.
template <int BITS, bool AFFINE, int LPR, int ROWS, int MAXT, bool GATED = false, bool QKV = false, bool PROLOGUE = false>
__global__ __launch_bounds__(MAXT) void gemv_kernel(const GemvParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int SUB = 64 / LPR;          // row slots per wave load
  constexpr int RPW = ROWS * SUB;        // rows per wave step
  constexpr int WPC = BITS == 8 ? 8 : (BITS == 4 ? 4 : 3);  // words per chunk
  constexpr int FW = BITS == 8 ? 8 : 4;                     // words a fragment row holds
  constexpr int FR = GATED ? 2 * ROWS : ROWS;  // fragment rows: gate rows, then the same rows of the up matrix

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = tid >> 6;
  const uint32_t waves = blockDim.x >> 6;
  const uint32_t lk = lane % LPR;
  const uint32_t sub = lane / LPR;

  // MoE prologue (int4_matmul.gen.ts:236-253): blockIdx.y is the (token, slot) pair.
  const _Float16* x = p.in;
  const uint32_t* wbase = p.weights;
  const _Float16* sbase = p.scales;
  const _Float16* bbase = p.biases;
  const uint32_t* wbase2 = p.weights2;
  const _Float16* sbase2 = p.scales2;
  const _Float16* bbase2 = p.biases2;
  size_t out_base = 0;
  if (p.moe) {
    const uint32_t token = blockIdx.y / p.slots, slot = blockIdx.y % p.slots;
    const uint32_t expert = p.ids[(size_t)token * p.ids_stride + slot];
    if (p.experts && expert >= p.experts) return;  // uniform per workgroup
    wbase += (size_t)expert * p.N * p.k_packed;
    sbase += (size_t)expert * p.N * p.spr;
    bbase += (size_t)expert * p.N * p.spr;
    if (GATED) {
      wbase2 += (size_t)expert * p.N * p.k_packed;
      sbase2 += (size_t)expert * p.N * p.spr;
      bbase2 += (size_t)expert * p.N * p.spr;
    }
    x += (size_t)token * p.in_tok_stride + (size_t)slot * p.in_slot_stride;
    out_base = (size_t)token * p.out_tok_stride + (size_t)slot * p.out_slot_stride;
  }

  UnpackConsts kc;
  kc.init();

  // QKV: the token's position, fetched now (a uniform load) so that neither the rotary table nor the
  // scatter at the end of a row waits for it
  int position = 0;
  if (QKV) position = p.position_map[p.pos_off];

  // Loads of one (tile, pass), as buffer loads: a uniform descriptor (this expert's matrix) plus one
  // 32-bit byte offset per lane, and an offset past the end of the array returns zeros without
  // touching memory. Rows past N are past the end by themselves (so are whole tiles past the last
  // one: the pipeline fetches ahead without asking whether anything is left); chunks past K are
  // sent there. No lane diverges, nothing is fetched twice and no load sits under a branch.
  constexpr uint32_t NOWHERE = 0x80000000u;  // every matrix is shorter than this (checked by the entry points)
  const uint32_t wbytes = QKV ? 0x7FFFFFFFu : p.N * p.k_packed * 4u, sbytes = QKV ? 0x7FFFFFFFu : p.N * p.spr * 2u;
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(wbase), 0, wbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t sres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(sbase), 0, sbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t bres = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(AFFINE ? bbase : sbase), 0, sbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wres2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(GATED ? wbase2 : wbase), 0, wbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t sres2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(GATED ? sbase2 : sbase), 0, sbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t bres2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16*>(GATED && AFFINE ? bbase2 : sbase), 0, sbytes, 0x00020000);
  auto issue = [&](Frag<FR, FW>& f, uint32_t tile, uint32_t pass) {
    const uint32_t c = pass * LPR + lk;
    const bool in_k = c < p.nchunks;
    const uint32_t g = AFFINE ? (c >> 1) : c;
#pragma unroll
    for (int r = 0; r < FR; r++) {
      const bool up = GATED && r >= ROWS;
      uint32_t rr = tile * RPW + (r % ROWS) * SUB + sub;
      bool ok = in_k;
      if (QKV) {  // pairs map to rows of the fused matrix, whose length the pair count does not give
        ok = ok && rr < p.N;
        rr = qkv_pair(p, rr < p.N ? rr : p.N - 1).row_lo;
      }
      const uint32_t woff = ok ? (rr * p.k_packed + c * WPC) * 4u : NOWHERE;
      const uint32_t soff = ok ? (rr * p.spr + g) * 2u : NOWHERE;
      const __amdgpu_buffer_rsrc_t wr = up ? wres2 : wres;
      if (BITS == 8) {
        const u32x4 v0 = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, 0, 2);  // 2: non-temporal
        const u32x4 v1 = __builtin_amdgcn_raw_buffer_load_b128(wr, woff + 16, 0, 2);
        f.w[r][0] = v0.x; f.w[r][1] = v0.y; f.w[r][2] = v0.z; f.w[r][3] = v0.w;
        f.w[r][4 % FW] = v1.x; f.w[r][5 % FW] = v1.y; f.w[r][6 % FW] = v1.z; f.w[r][7 % FW] = v1.w;
      } else if (BITS == 4) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(wr, woff, 0, 2);
        f.w[r][0] = v.x; f.w[r][1] = v.y; f.w[r][2] = v.z; f.w[r][3] = v.w;
      } else {
        const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(wr, woff, 0, 2);
        f.w[r][0] = v.x; f.w[r][1] = v.y; f.w[r][2] = v.z; f.w[r][3] = 0;
      }
      f.s[r] = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(up ? sres2 : sres, soff, 0, 0));
      if (AFFINE) f.b[r] = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(up ? bres2 : bres, soff, 0, 0));
    }
  };

  // The wave's first loads go out before anything else, so the weight stream
  // starts while x is still being staged.
  const uint32_t wave_stride = gridDim.x * waves;
  uint32_t tile = blockIdx.x * waves + wave, pass = 0;
  bool have = tile < p.ntiles;
  Frag<FR, FW> fa, fb;
  issue(fa, tile, 0);

  // ---- stage x: each thread converts whole chunks -------------------------
  h8* xs_pieces = reinterpret_cast<h8*>(smem);
  const uint32_t padded_chunks = (p.nchunks + 63u) & ~63u;
  float* xsum = reinterpret_cast<float*>(smem + (size_t)padded_chunks * 64u);
  if constexpr (!PROLOGUE) {
    for (uint32_t c = tid; c < p.nchunks; c += blockDim.x) {
      float s = 0.f;
      const h8* src = reinterpret_cast<const h8*>(x + (size_t)c * 32u);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const h8 v = src[j];
        h8 o;
#pragma unroll
        for (int sl = 0; sl < 8; sl++) o[sl] = v[BITS == 8 ? value_in_slot8(sl) : value_in_slot(sl)];
        xs_pieces[x_slot(c, j)] = o;
#pragma unroll
        for (int i = 0; i < 8; i++) s += (float)v[i];
      }
      xsum[c] = s;
    }
  } else {
    // pass 1: val = f16(residual + delta) into LDS (slot order already), sum of squares per thread
    float ss = 0.f;
    for (uint32_t c = tid; c < p.nchunks; c += blockDim.x) {
      const h8* res = reinterpret_cast<const h8*>(x + (size_t)c * 32u);
      const h8* del = reinterpret_cast<const h8*>(p.delta + (size_t)c * 32u);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const h8 v = res[j] + del[j];  // f16 addition, as add_norm does
        h8 o;
#pragma unroll
        for (int sl = 0; sl < 8; sl++) o[sl] = v[value_in_slot(sl)];
        xs_pieces[x_slot(c, j)] = o;
#pragma unroll
        for (int i = 0; i < 8; i++) ss = __builtin_fmaf((float)v[i], (float)v[i], ss);
      }
    }
    // the row's sum of squares: lanes by DPP, waves through LDS, every thread adds the wave sums in wave order
    float* wave_ss = reinterpret_cast<float*>(smem + (size_t)padded_chunks * 68u);
    ss = group_sum_to_last_lane<64>(ss);
    if (lane == 63) wave_ss[wave] = ss;
    __syncthreads();
    float total = 0.f;
    for (uint32_t w = 0; w < waves; w++) total += wave_ss[w];
    const float rms_inv = 1.0f / sqrtf(total / (float)(p.nchunks * 32u) + p.rms_eps);
    // pass 2: each thread normalises the pieces it wrote (no barrier needed for those), rounding to f16 as the
    // store of the normed vector did, and sums the rounded values
    for (uint32_t c = tid; c < p.nchunks; c += blockDim.x) {
      const h8* gam = reinterpret_cast<const h8*>(p.gamma + (size_t)c * 32u);
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const h8 g = gam[j];
        h8 o = xs_pieces[x_slot(c, j)];
#pragma unroll
        for (int sl = 0; sl < 8; sl++) {
          o[sl] = narrow_f32((float)o[sl] * rms_inv * (float)g[value_in_slot(sl)]);
          s += (float)o[sl];
        }
        xs_pieces[x_slot(c, j)] = o;
      }
      xsum[c] = s;
    }
  }
  // QKV: the rotation of every pair index, once per workgroup, by the threads at the far end of the
  // workgroup (the staging above keeps the first ones busy); cos and sin are long instruction
  // sequences that would otherwise run once per pair with one lane active
  float2* rope = reinterpret_cast<float2*>(smem + (size_t)padded_chunks * 68u);
  if (QKV) {
    const uint32_t rt = blockDim.x - 1u - tid;
    if (rt < p.half_dim) {
      const float freq = (float)position / powf(p.rope_theta, (float)(rt * 2u) / (float)p.head_dim);
      // the hardware sine and cosine take revolutions and are accurate to about 1e-6 on [0, 1): turning the
      // angle into a fraction of a revolution costs it about |freq| * 2^-24, below what forming the f32
      // angle itself already carries (position * 2^-23), and replaces two long range reductions that
      // every wave of the workgroup would wait for at the barrier
      const float turns = freq * 0.15915494309189535f;
      const float frac = turns - floorf(turns);
      rope[rt] = float2{__builtin_amdgcn_cosf(frac), __builtin_amdgcn_sinf(frac)};
    }
  }
  __syncthreads();

  float acc[FR];
#pragma unroll
  for (int r = 0; r < FR; r++) acc[r] = 0.f;

  // One pipeline stage: prefetch the next (tile, pass) into `nxt`, then consume `cur`.
  auto stage = [&](const Frag<FR, FW>& cur, Frag<FR, FW>& nxt) {
    uint32_t ntile = tile, npass = pass + 1;
    if (npass == p.npasses) { npass = 0; ntile += wave_stride; }
    const bool nhave = ntile < p.ntiles;
    issue(nxt, ntile, npass);  // past the last tile this fetches nothing
    // keep the loads above where they are: the scheduler would otherwise sink
    // the small scale/bias loads down to their first use
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t c = pass * LPR + lk;
    const bool live = c < p.nchunks;
    const uint32_t cc = live ? c : p.nchunks - 1;
    h2 xv[16];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const h8 v = xs_pieces[x_slot(cc, j)];
      xv[4 * j + 0] = (h2){v[0], v[1]};
      xv[4 * j + 1] = (h2){v[2], v[3]};
      xv[4 * j + 2] = (h2){v[4], v[5]};
      xv[4 * j + 3] = (h2){v[6], v[7]};
    }
    const float xs = xsum[cc];
#pragma unroll
    for (int r = 0; r < FR; r++) {
      h2 q[16];
      if constexpr (BITS == 8) unpack8_chunk(cur.w[r], q, kc);
      else if constexpr (BITS == 4) unpack4_chunk(cur.w[r][0], cur.w[r][1], cur.w[r][2], cur.w[r][3], q, kc);
      else unpack3_chunk(cur.w[r][0], cur.w[r][1], cur.w[r][2], q, kc);
      float d0 = 0.f, d1 = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        d0 = __builtin_amdgcn_fdot2(q[i], xv[i], d0, false);
        d1 = __builtin_amdgcn_fdot2(q[i + 1], xv[i + 1], d1, false);
      }
      const float dot = d0 + d1;
      const float s = (float)cur.s[r];
      const float term = AFFINE ? __builtin_fmaf(s, dot, (float)cur.b[r] * xs) : s * __builtin_fmaf(-7.f, xs, dot);
      acc[r] += live ? term : 0.f;
    }

    if (pass == p.npasses - 1) {
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        float total = group_sum_to_last_lane<LPR>(acc[r]);
        acc[r] = 0.f;
        float second = 0.f;
        if (GATED) {
          second = group_sum_to_last_lane<LPR>(acc[r + ROWS]);
          acc[r + ROWS] = 0.f;
          if (!QKV) total = second * (total * (1.0f / (1.0f + expf(-total))));
        }
        const uint32_t rr = tile * RPW + r * SUB + sub;
        if (QKV) {
          if (lk == LPR - 1 && rr < p.N) {
            const QkvPair q = qkv_pair(p, rr);
            const uint32_t page_no = (uint32_t)position / p.page_size, slot = (uint32_t)position - page_no * p.page_size;
            const size_t cache = (size_t)page_no * p.kv_page_stride + (size_t)q.head * p.head_page_stride +
                                 (size_t)slot * p.head_dim + p.pages_off + q.dim_lo;
            float lo = total, hi = second;  // V: no rotation
            if (q.group != 2) {
              const float c = rope[q.dim_lo].x, sn = rope[q.dim_lo].y;
              lo = c * total + sn * (-second);
              hi = c * second + sn * total;
            }
            const size_t at = cache + (q.group == 2 ? p.v_page_offset : 0u);
            const size_t in_row = (size_t)q.head * p.head_dim + q.dim_lo;
            _Float16* dst = q.group == 0 ? p.q_out + in_row : p.kv_pages + at;
            if (p.k_slot && q.group != 0) dst = (q.group == 1 ? p.k_slot : p.v_slot) + in_row;
            if (q.group == 0 || p.k_slot || position >= 0 && (!p.kv_capacity || at + p.half_dim < p.kv_capacity)) {
              dst[0] = (_Float16)lo;
              dst[p.half_dim] = (_Float16)hi;
            }
          }
          continue;
        }
        if (lk == LPR - 1 && rr < p.N) {
          if (p.out_f32) reinterpret_cast<float*>(p.out)[out_base + rr] = total;
          else reinterpret_cast<_Float16*>(p.out)[out_base + rr] = (_Float16)total;
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

// Launch with `smem` bytes of dynamic LDS; above 64 KB the kernel's limit has to be raised first.
template <class Kernel>
void go(Kernel k, dim3 grid, uint32_t threads, size_t smem, hipStream_t s, const GemvParams& p) {
  if (smem > 64 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, dim3(threads), smem, s, p);
}

template <int BITS, bool AFFINE, int LPR, int ROWS>
hipError_t launch_one(const GemvParams& p, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  if (threads > 512) go(gemv_kernel<BITS, AFFINE, LPR, ROWS, 1024>, grid, threads, smem, s, p);
  else go(gemv_kernel<BITS, AFFINE, LPR, ROWS, 512>, grid, threads, smem, s, p);
  return hipGetLastError();
}

template <int BITS, bool AFFINE>
hipError_t launch_qkv(const GemvParams& p, int lpr, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  if (lpr == 64) go(gemv_kernel<BITS, AFFINE, 64, 1, 512, true, true>, grid, threads, smem, s, p);
  else if (lpr == 32) go(gemv_kernel<BITS, AFFINE, 32, 1, 512, true, true>, grid, threads, smem, s, p);
  else go(gemv_kernel<BITS, AFFINE, 16, 1, 512, true, true>, grid, threads, smem, s, p);
  return hipGetLastError();
}

template <int BITS, bool AFFINE>
hipError_t launch_prologue(const GemvParams& p, int lpr, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  if (lpr == 64) go(gemv_kernel<BITS, AFFINE, 64, 1, 512, true, false, true>, grid, threads, smem, s, p);
  else if (lpr == 32) go(gemv_kernel<BITS, AFFINE, 32, 1, 512, true, false, true>, grid, threads, smem, s, p);
  else go(gemv_kernel<BITS, AFFINE, 16, 1, 512, true, false, true>, grid, threads, smem, s, p);
  return hipGetLastError();
}

template <int BITS, bool AFFINE>
hipError_t launch_gated(const GemvParams& p, int lpr, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  if (lpr == 64) go(gemv_kernel<BITS, AFFINE, 64, 1, 512, true>, grid, threads, smem, s, p);
  else if (lpr == 32) go(gemv_kernel<BITS, AFFINE, 32, 1, 512, true>, grid, threads, smem, s, p);
  else go(gemv_kernel<BITS, AFFINE, 16, 1, 512, true>, grid, threads, smem, s, p);
  return hipGetLastError();
}

template <int BITS, bool AFFINE>
hipError_t launch_fmt(const GemvParams& p, int lpr, int rows, dim3 grid, uint32_t threads, size_t smem, hipStream_t s) {
  if (lpr == 64) {
    if (rows == 4) return launch_one<BITS, AFFINE, 64, 4>(p, grid, threads, smem, s);
    if (rows == 2) return launch_one<BITS, AFFINE, 64, 2>(p, grid, threads, smem, s);
    return launch_one<BITS, AFFINE, 64, 1>(p, grid, threads, smem, s);
  }
  if (lpr == 32) return launch_one<BITS, AFFINE, 32, 2>(p, grid, threads, smem, s);
  return launch_one<BITS, AFFINE, 16, 2>(p, grid, threads, smem, s);
}

size_t gemv_lds_bytes(uint32_t K, uint32_t head_dim, bool prologue) {
  const uint32_t padded_chunks = (K / 32u + 63u) & ~63u;
  return (size_t)padded_chunks * 68u + (size_t)(head_dim / 2) * 8u + (prologue ? 64u : 0u);
}

}  // namespace

// The activation row is staged whole in LDS (160 KB per CU).
bool gemv_supports(const MatmulArgs& a) { return gemv_lds_bytes(a.K, a.qkv ? a.qkv->head_dim : 0, a.delta != nullptr) <= 160u * 1024u; }

hipError_t launch_gemv(const MatmulArgs& a, const Tune& t, hipStream_t s) {
  GemvParams p{};
  p.out = a.out; p.in = a.in; p.scales = a.scales; p.weights = a.weights; p.biases = a.biases; p.ids = a.ids;
  p.N = a.N; p.k_packed = a.k_packed; p.spr = a.spr;
  p.nchunks = a.K / 32;
  p.out_f32 = a.out_f32;
  p.moe = a.slots > 0;
  p.slots = a.slots; p.in_slot_stride = a.in_slot_stride; p.out_slot_stride = a.out_slot_stride;
  p.in_tok_stride = a.in_tok_stride; p.out_tok_stride = a.out_tok_stride; p.ids_stride = a.ids_stride;
  p.experts = a.experts;
  const bool gated = a.up_weights != nullptr;
  p.delta = a.delta; p.gamma = a.gamma; p.rms_eps = a.rms_eps;
  p.weights2 = a.up_weights; p.scales2 = a.up_scales; p.biases2 = a.up_biases;
  if (a.qkv) {
    const QkvArgs& q = *a.qkv;
    p.q_out = q.q_out; p.kv_pages = q.kv_pages; p.k_slot = q.k_slot; p.v_slot = q.v_slot; p.position_map = q.position_map;
    p.half_dim = q.head_dim / 2; p.head_dim = q.head_dim;
    p.q_pairs = q.heads * p.half_dim; p.kv_pairs = q.kv_heads * p.half_dim;
    p.q_dim = q.heads * q.head_dim; p.kv_dim = q.kv_heads * q.head_dim;
    // the scratch form has no pages; its cache address is computed and unused
    p.page_size = q.page_size ? q.page_size : 1; p.kv_page_stride = q.kv_page_stride; p.head_page_stride = q.head_page_stride;
    p.v_page_offset = q.v_page_offset; p.pos_off = q.position_map_elem_offset; p.pages_off = q.pages_elem_offset;
    p.rope_theta = q.rope_theta; p.kv_capacity = q.kv_capacity;
  }

  // lanes per row: narrow rows share a wave between several rows
  const int lpr = p.nchunks > 32 ? 64 : (p.nchunks > 16 ? 32 : 16);
  p.npasses = (p.nchunks + lpr - 1) / lpr;
  const uint32_t pairs = p.moe ? a.slots * a.tokens : 1;

  // Launch shape (measured on MI355X): one row per wave step and 8-wave
  // workgroups, 3 per CU, stream best for wide rows; narrow rows (several rows
  // per wave load) use 2 steps in flight.
  const int cus = t.num_cus;
  int rows = lpr == 64 ? (t.gemv_rows == 2 || t.gemv_rows == 4 ? t.gemv_rows : 1) : 2;
  if (gated) rows = 1;  // two matrices per row already give two loads in flight
  // long rows (K >= 8192): the staged activations are 16+ KB per workgroup, so one 16-wave
  // workgroup per CU stages them once instead of three times (measured 9.4 vs 10.2 us at K=14336)
  const bool long_rows = lpr == 64 && p.nchunks >= 256 && !p.moe && !gated;
  uint32_t waves = t.gemv_waves ? t.gemv_waves : (long_rows ? 16 : 8);
  if (waves * 64 > (uint32_t)MAX_WG_THREADS) waves = MAX_WG_THREADS / 64;
  if (gated && waves > 8) waves = 8;  // the gated kernels are built for 512 threads
  uint32_t gx = (uint32_t)cus * (t.gemv_wg_per_cu ? t.gemv_wg_per_cu : (long_rows ? 1 : 3));
  const uint32_t rpw = rows * (64 / lpr);
  p.ntiles = (a.N + rpw - 1) / rpw;

  if (!gemv_supports(a)) return hipErrorInvalidValue;  // rejected by the entry points
  const size_t smem = gemv_lds_bytes(a.K, a.qkv ? a.qkv->head_dim : 0, a.delta != nullptr);

  const uint32_t wg_tiles = (p.ntiles + waves - 1) / waves;
  gx = gx / pairs;
  if (gx < 1) gx = 1;
  if (gx > wg_tiles) gx = wg_tiles;
  // every workgroup the same number of tiles where a grid of up to twice the size allows it: 512 rows of an expert
  // over six 8-wave workgroups are 11 tiles for some waves and 10 for others, over eight they are 8 for all
  // (16 tokens x 8 experts, 2048 -> 512: 16.8 -> 15.4 us; 512 -> 2048: 15.5 -> 14.8 us)
  // Not down to one tile per wave: a wave with a single tile has nothing in flight behind it (4 tokens, 512 -> 2048:
  // 7.1 us on 32 workgroups of one tile per wave, 6.3 on 24 of one or two).
  // Dense dispatches keep their grid of three workgroups per CU: a larger one no longer fits the CUs at once
  // (8-bit, 4096 -> 14336: 13.4 us on 768 workgroups, 14.6 on 896).
  if (!t.gemv_wg_per_cu && pairs > 1)
    for (uint32_t d = gx; d <= 2 * gx && 2 * d <= wg_tiles; d++)
      if (wg_tiles % d == 0) { gx = d; break; }
  const dim3 grid(gx, pairs, 1);
  const uint32_t threads = waves * 64;

  // dense M>1 handled by the caller looping rows; here one activation row
  if (a.qkv) {
    if (a.bits == 4) return a.affine ? launch_qkv<4, true>(p, lpr, grid, threads, smem, s) : launch_qkv<4, false>(p, lpr, grid, threads, smem, s);
    return hipErrorInvalidValue;  // rejected by the entry point
  }
  if (gated && a.delta) {
    if (a.bits == 8 || p.moe) return hipErrorInvalidValue;  // rejected by the entry point
    if (a.bits == 4) return a.affine ? launch_prologue<4, true>(p, lpr, grid, threads, smem, s) : launch_prologue<4, false>(p, lpr, grid, threads, smem, s);
    return launch_prologue<3, true>(p, lpr, grid, threads, smem, s);
  }
  if (gated) {
    if (a.bits == 8) return hipErrorInvalidValue;  // rejected by the entry point
    if (a.bits == 4) return a.affine ? launch_gated<4, true>(p, lpr, grid, threads, smem, s) : launch_gated<4, false>(p, lpr, grid, threads, smem, s);
    return launch_gated<3, true>(p, lpr, grid, threads, smem, s);
  }
  if (a.bits == 4) {
    if (a.affine) return launch_fmt<4, true>(p, lpr, rows, grid, threads, smem, s);
    return launch_fmt<4, false>(p, lpr, rows, grid, threads, smem, s);
  }
  if (a.bits == 8) return launch_fmt<8, true>(p, lpr, rows, grid, threads, smem, s);
  return launch_fmt<3, true>(p, lpr, rows, grid, threads, smem, s);
}

}  // namespace ztvm
