/*
 * libztvm_hip — C ABI of the MI355X (gfx950) int4/int3 group-quantized
 * dequant-matmul path: M=1 decode GEMV, small-M GEMV, prefill GEMM and the
 * MoE gathered GEMV, plus the small dispatches either side of them in a MoE
 * block and the load-time repack of MLX checkpoints into the bound buffers.
 *
 * The boundary it replaces is the WebGPU dispatch surface of the reference
 * engine (paths relative to the reference's root):
 *   uniformBuf()  src/zero-tvm/engine-core.ts:53-65     PODArgs uniform
 *   bg()          src/zero-tvm/engine-core.ts:76-92     bind group, binding i = array index i
 *   dispatch()    src/zero-tvm/engine-core.ts:2151-2179 one compute pass
 * and the binding contract of the kernel generator
 *   src/compiler/shaders/int4_matmul.gen.ts:24-30, :211-226
 *   (0 out / 1 in / 2 scales / 3 weights / 4 PODArgs / 5 biases / 6 ids).
 *
 * Conventions: every entry point is extern "C", takes plain pointers and
 * sizes, returns 0 on success or a negative ZTVM_E_* code, never throws and
 * never falls back to a CPU path. Device memory is named by its 64-bit device
 * address. All work is enqueued on the context's single HIP stream in call
 * order (the reference's queue order); only ztvm_download, ztvm_sync and
 * ztvm_event_elapsed_ms block. The caller owns every buffer.
 */
#ifndef ZTVM_H
#define ZTVM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZTVM_ABI_VERSION 2

/* ztvm_matmul_desc.experts: the caller vouches for every id in ids[] */
#define ZTVM_EXPERTS_UNCHECKED 0xFFFFFFFFu

/* Bytes of device memory ztvm_matmul_static may use as scratch (held per GPU until the process ends). */
#define ZTVM_STATIC_SCRATCH_BYTES (16u << 20)


#if defined(__GNUC__)
#define ZTVM_API __attribute__((visibility("default")))
#else
#define ZTVM_API
#endif

enum {
  ZTVM_OK = 0,
  ZTVM_E_INVALID = -1,     /* descriptor or argument rejected before any GPU work */
  ZTVM_E_HIP = -2,         /* a HIP runtime call failed; see ztvm_last_error */
  ZTVM_E_UNSUPPORTED = -3, /* an explicitly requested kernel cannot run this descriptor */
  ZTVM_E_NODEVICE = -4     /* no gfx950 device visible */
};

/* Kernel families. AUTO picks by M; naming a family that cannot run the
 * descriptor is an error, never a silent substitution (the rule of
 * pickChunkGemm, src/zero-tvm/engine-core.ts:220-245). */
enum {
  ZTVM_KERNEL_AUTO = 0,
  ZTVM_KERNEL_GEMV = 1,   /* one pass per activation row; replaces int4_matmul[_sg|_tiled|_vec4|_vec4h][_affine][_q3][_moe] */
  ZTVM_KERNEL_SKINNY = 2, /* weights streamed once through registers, default for 17 <= M <= 128 (4-bit rows with K a multiple of 128: from 13), and above 128 rows where the tile GEMM's grid of ceil(M/256) x N/128 workgroups is estimated slower; replaces int4_matmul_batched_m4 / _batched_dyn[_affine] */
  ZTVM_KERNEL_GEMM = 3,   /* MFMA tile GEMM, default for M > 128 (4-bit, 3-bit and 8-bit rows, f16 output); replaces int4_matmul_tiled_st / _sg_e1 / _sg_e5 [_affine] and int8_affine_batched at prefill M */
  ZTVM_KERNEL_ROWS = 4    /* one pass over the weights for up to 16 rows, default for 2 <= M <= 16 (4-bit rows with K a multiple of 128: to 12); replaces int4_matmul_batched_m4 and _batched_dyn[_affine] at a speculative-verify M_ROWS */
};

typedef struct ztvm_ctx ztvm_ctx;
typedef struct ztvm_cmdbuf ztvm_cmdbuf;
typedef struct ztvm_event ztvm_event;

/* One quantized matmul dispatch: the PODArgs uniform
 * (src/compiler/shaders/int4_matmul.gen.ts:216-225, :645-650) plus the bind
 * group entries, with the variant options of Int4MatmulOpts (:32-134) that
 * change arithmetic (bits, affine, outF32, moe). Options that only chose a
 * WGSL tiling (rowsPerWG, subgroups, vec4, vec4Half, the grid) have no
 * counterpart: N, M, tokens and slots define the work.
 *
 *   Y[m,n] = sum_k A[m,k] * w[n,k],  f32 accumulation, f16 (or f32) store
 *   affine=1: w = q*s + b, group 64     affine=0: w = (q-7)*s, group 32
 *   bits=4: k_packed = K/8, value k at (W[n,k>>3] >> 4*(k&7)) & 15
 *   bits=3: k_packed = 3K/32, row is an LSB-first bitstream, value k at bits [3k,3k+3)
 *
 * Dense (slots == 0): A is [M,K] f16 row-major, Y is [M,N]; rows >= M are
 * neither read nor written. MoE (slots > 0, M must be 1): for every
 * (token < tokens, slot < slots) expert = ids[token*ids_stride + slot],
 * weights/scales/biases are [experts][N][...] stacks, the input row starts at
 * element token*in_tok_stride + slot*in_slot_stride of `in` and the output
 * row at token*out_tok_stride + slot*out_slot_stride of `out`
 * (:236-253). `experts` is the height of the bound stacks (WebGPU bounds-checks
 * storage accesses against the bound sizes; here the kernel checks the id): a
 * pair whose expert id is >= experts is skipped, so a bad id cannot fault the
 * GPU. A MoE descriptor with experts == 0 is rejected; a caller that has
 * validated its ids itself passes ZTVM_EXPERTS_UNCHECKED. */
typedef struct ztvm_matmul_desc {
  uint32_t bits;           /* 4 | 3 */
  uint32_t affine;         /* 0 | 1 */
  uint32_t out_f32;        /* 0: f16 output, 1: f32 output (LM head) */
  uint32_t kernel;         /* ZTVM_KERNEL_* */
  uint32_t M;              /* PODArgs.M_ROWS (1 for GEMV dispatches) */
  uint32_t N;              /* PODArgs.packGridDimX */
  uint32_t k_packed;       /* PODArgs.K_PACKED, u32 words per weight row */
  uint32_t scales_per_row; /* PODArgs.SCALES_PER_ROW = K/group */
  uint32_t slots;          /* 0 = dense; else grid z of the MoE dispatch */
  uint32_t tokens;         /* grid y of the MoE dispatch (ignored when dense) */
  uint32_t in_slot_stride; /* PODArgs.IN_SLOT_STRIDE, f16 elements */
  uint32_t out_slot_stride;
  uint32_t in_tok_stride;
  uint32_t out_tok_stride;
  uint32_t ids_stride;
  uint32_t experts;        /* MoE: stack height for the id guard (or ZTVM_EXPERTS_UNCHECKED); ignored when dense */
  uint64_t out;            /* binding 0 (device address incl. region offset) */
  uint64_t in;             /* binding 1 */
  uint64_t scales;         /* binding 2 */
  uint64_t weights;        /* binding 3 */
  uint64_t biases;         /* binding 5, affine only */
  uint64_t ids;            /* binding 6, MoE only */
} ztvm_matmul_desc;

/* ---- context ----------------------------------------------------------- */

/* Replaces requestAdapter/requestDevice (src/lib/index.ts:210-377): binds a
 * gfx950 device and creates the stream every later call is ordered on. */
ZTVM_API int ztvm_create(int device, ztvm_ctx** out);
ZTVM_API void ztvm_destroy(ztvm_ctx* ctx);

/* Text of the last failure on this context (or of the last context-less
 * failure when ctx is NULL). Replaces pushErrorScope/uncapturederror
 * (tests/kernels/gpu.mjs:59-62). Never NULL. */
ZTVM_API const char* ztvm_last_error(ztvm_ctx* ctx);

ZTVM_API int ztvm_abi_version(void);

/* Device facts the host layer reports: name, compute units, bytes of HBM. */
ZTVM_API int ztvm_device_info(ztvm_ctx* ctx, char* name, size_t name_len, uint32_t* compute_units, uint64_t* hbm_bytes);

/* ---- buffers (device.createBuffer / queue.writeBuffer / mapAsync) ------- */

/* createBuffer (src/zero-tvm/engine-core.ts:36-41). Address is 256-byte aligned. */
ZTVM_API int ztvm_alloc(ztvm_ctx* ctx, size_t bytes, uint64_t* dptr);
ZTVM_API int ztvm_free(ztvm_ctx* ctx, uint64_t dptr);
/* queue.writeBuffer (src/zero-tvm/engine-core.ts:61-63): the source may be reused on return. */
ZTVM_API int ztvm_upload(ztvm_ctx* ctx, uint64_t dst, size_t dst_off, const void* src, size_t bytes);
/* copyBufferToBuffer + mapAsync (tests/kernels/gpu.mjs:95-121): blocks until earlier work finished. */
ZTVM_API int ztvm_download(ztvm_ctx* ctx, void* dst, uint64_t src, size_t src_off, size_t bytes);
/* Fill with a repeated byte, ordered on the stream (a kernel, so it may be recorded). */
ZTVM_API int ztvm_fill(ztvm_ctx* ctx, uint64_t dst, size_t dst_off, int byte, size_t bytes);
/* copyBufferToBuffer (tests/kernels/gpu.mjs:107-110): device-to-device, ordered on the stream (a kernel,
 * so it may be recorded). Both addresses and the size must be multiples of 16 bytes. */
ZTVM_API int ztvm_copy(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes);
/* Measurement aid with no counterpart in the reference: a kernel that reads `bytes` bytes from src with 16-byte
 * loads and does nothing else (sink: 4 bytes of device memory it practically never writes), ordered on the
 * stream and recordable. Its time is the empirical ceiling a bandwidth-bound dispatch of that size is held
 * against, measured in the same run and the same way as the dispatch (scripts/kernel-ab-ours.mjs:75-99 times
 * its kernels against the device's streaming rate the same way). */
ZTVM_API int ztvm_read_probe(ztvm_ctx* ctx, uint64_t src, size_t bytes, uint64_t sink);
ZTVM_API int ztvm_sync(ztvm_ctx* ctx);

/* ---- dispatch ----------------------------------------------------------- */

/* Pure CPU check of a descriptor against the generator's own legality rules
 * (src/compiler/shaders/int4_matmul.gen.ts:172-197) and the layout contract;
 * needs no GPU. `why` receives the reason on failure. */
ZTVM_API int ztvm_matmul_validate(const ztvm_matmul_desc* desc, char* why, size_t why_len);

/* Which family AUTO resolves to for this descriptor (ZTVM_KERNEL_*), or a
 * negative error. Pure CPU. Replaces resolveMatmul / pickChunkGemm
 * (src/zero-tvm/variants.ts:239-388, src/zero-tvm/engine-core.ts:220-245). */
ZTVM_API int ztvm_matmul_resolve(const ztvm_matmul_desc* desc);

/* bg() + dispatch() of one matmul (src/zero-tvm/engine-core.ts:76-92,
 * :2151-2179; call sites :2290, :2312, :2343-2347, :2517-2524, :2543-2549,
 * :4280-4293, :4386-4390). Validates, then enqueues. */
ZTVM_API int ztvm_matmul(ztvm_ctx* ctx, const ztvm_matmul_desc* desc);

/* Library-owned scratch. The rows, skinny and tile-GEMM families keep activation group sums,
 * reordered activations and split-k partial sums in a buffer the context owns (4 MiB at first). A
 * dispatch that needs more grows it, outside a recording only (inside one the call returns
 * ZTVM_E_UNSUPPORTED and asks for one eager dispatch of that shape first). Growing never frees a
 * buffer that a live command buffer may reference: it is kept until the last such command buffer
 * is destroyed, so a command buffer recorded earlier stays valid to submit after any later
 * dispatch. Destroying the context ends the life of its command buffers. */

/* ztvm_matmul for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same
 * descriptor, same kernels and bit-identical results (one exception below), but the scratch of the rows, skinny and
 * tile-GEMM families is a fixed array of ZTVM_STATIC_SCRATCH_BYTES that lives in the library's
 * device image (one copy per GPU, held until the process ends), so this call never calls hipMalloc
 * or hipFree, whatever the shape. A dispatch that needs more scratch than that is refused with
 * ZTVM_E_UNSUPPORTED and a message that says how much (ztvm_matmul takes any size); where AUTO would
 * give a dispatch of more than 128 rows to the skinny family and its reordered copy of the
 * activations (M x K f16) outgrows the array, the tile GEMM runs it instead (results then agree
 * with ztvm_matmul's to the last f16 bit or two, not bit for bit); likewise the tile GEMM runs
 * without its split along k where the f32 totals the parts exchange would outgrow the array. Nothing in the
 * array has to start at zero: every kernel writes what it later reads. All calls on one GPU share
 * the array, from every context and thread: two ztvm_matmul_static dispatches that overlap on one
 * GPU (different contexts or streams) race on it; dispatches on one context are ordered and safe. */
ZTVM_API int ztvm_matmul_static(ztvm_ctx* ctx, const ztvm_matmul_desc* desc);

/* Gate + up + SiLU in one pass over the activations: out[n] = up[n] * silu(gate[n]) with
 * gate = W_gate x (the descriptor's weights / scales / biases) and up = W_up x (the three
 * extra buffers, same shape and format), both sums kept in f32 until the one store.
 * Replaces fused_ffn_kernel (src/compiler/shaders/fused_ffn.wgsl:52-140; dispatch site
 * src/zero-tvm/engine-core.ts:2503, :2522) whose single [2*FFN, K] weight buffer is
 * up_* = gate_* + FFN rows; with slots > 0 it runs per (token, slot) pair on expert stacks
 * and so also replaces the gate, up and silu_mul dispatches of the MoE block
 * (engine-core.ts:2344-2346) by one, without the f16 rounding of gate and up in between.
 * GEMV family only (kernel AUTO or GEMV); dense M > 1 runs one pass per row. */
ZTVM_API int ztvm_ffn_gated(ztvm_ctx* ctx, const ztvm_matmul_desc* desc, uint64_t up_weights, uint64_t up_scales,
                            uint64_t up_biases);

/* fused_ffn_prologue / fused_ffn_tiled_sg_prologue (src/compiler/shaders/fused_ffn_prologue.wgsl:1-165):
 * ztvm_ffn_gated with the FFN-entry add + RMSNorm folded in. desc->in is the running residual
 * [K] f16, delta the o-proj output to be added, gamma the norm gain:
 *   val = f16(residual + delta);  x = f16(f32(val) * (1 / sqrt(mean(val^2) + rms_eps)) * f32(gamma))
 * with the sum of squares in f32, and x feeds the gate / up dot products exactly as the stored
 * normed vector did. One dense row (M = 1, the decode step), 4-bit symmetric (the reference's),
 * 4-bit affine or 3-bit. Like the reference's kernel it does not write the residual sum anywhere. */
ZTVM_API int ztvm_ffn_gated_prologue(ztvm_ctx* ctx, const ztvm_matmul_desc* desc, uint64_t up_weights, uint64_t up_scales,
                                     uint64_t up_biases, uint64_t delta, uint64_t gamma, float rms_eps);

/* QKV matmul + RoPE + KV append in one dispatch, decode path (one token). Replaces
 * qkv_fused / _sg / _sg_vec4 / _tiled_sg / _tiled2sg (src/compiler/shaders/qkv_fused.wgsl:23-193;
 * dispatch site src/zero-tvm/engine-core.ts:2320): bindings 0 q_out, 1 kv_pages, 2 hidden,
 * 3 scales, 4 weights, 5 position_map, PODArgs {position_map_elem_offset, pages_elem_offset},
 * and the model constants the reference injects as a shader prelude
 * (src/compiler/shader-prelude.ts:43-52). The fused projection is [Q | K | V] rows, Q =
 * heads*head_dim, K = V = kv_heads*head_dim; for every rotary pair (dim, dim + head_dim/2) of a
 * head the two rows are multiplied in one pass, Q and K are rotated by
 * freq = position / theta^(2*dim/head_dim) (cos and sin in f32), Q goes to q_out, K and V into
 * the page the position falls in: element page*kv_page_stride + head*head_page_stride +
 * slot*head_dim + dim (+ v_page_offset for V) + pages_elem_offset. The position is read on
 * the device from position_map[position_map_elem_offset]. A position whose slot would lie at
 * or past kv_capacity (f16 elements; 0 = unchecked) or below zero writes Q only, so a bad
 * position cannot fault the GPU. 4-bit rows, symmetric (the reference's) or affine. */
typedef struct ztvm_qkv_fused_desc {
  uint32_t bits, affine;
  uint32_t k_packed, scales_per_row;
  uint32_t heads, kv_heads, head_dim;
  uint32_t page_size, kv_page_stride, head_page_stride, v_page_offset; /* f16 elements */
  uint32_t position_map_elem_offset, pages_elem_offset;
  float rope_theta;
  uint64_t kv_capacity;
  uint64_t q_out, kv_pages, hidden, scales, weights, position_map, biases;
} ztvm_qkv_fused_desc;
ZTVM_API int ztvm_qkv_fused(ztvm_ctx* ctx, const ztvm_qkv_fused_desc* desc);

/* The int8-KV-mode variant (src/compiler/shaders/qkv_fused_scratch.wgsl:14-150; engine-core.ts:849):
 * the same math, but K (rotated) and V go to two f16 scratch rows k_slot / v_slot of
 * kv_heads*head_dim elements each (row-major head, dim) instead of the paged cache; a
 * ztvm_kv_quantize_int8 dispatch then writes the int8 cache. The descriptor's kv_pages, page
 * layout and kv_capacity fields are not read. */
ZTVM_API int ztvm_qkv_fused_scratch(ztvm_ctx* ctx, const ztvm_qkv_fused_desc* desc, uint64_t k_slot, uint64_t v_slot);

/* kv_quantize_int8 (src/compiler/shaders/kv_quantize_int8.wgsl:47-164): per (token, kv head, side)
 * one scale = max|x| / 127 (at least 1e-8) over the head's head_dim values, stored as f16, and
 * q = clamp(round-half-even(x / scale), -127, 127) packed four to a u32 word. k_slot / v_slot are
 * [tokens][kv_heads*head_dim] f16. Words: page . head . slot . side(K, V) . dim/4, i.e.
 *   page_no*kv_heads*page_size*2*(head_dim/4) + head*page_size*2*(head_dim/4) + slot*2*(head_dim/4) + side*(head_dim/4) + dim/4 + pages_word_offset
 * scales: page_no*kv_heads*page_size*2 + head*page_size*2 + slot*2 + side + scales_elem_offset,
 * with (page_no, slot) from position_map[position_map_elem_offset + token]. tokens = grid y of the
 * reference (1 on the decode path). A negative position, or an index at or past a capacity
 * (0 = unchecked), writes nothing, so a bad position cannot fault the GPU. */
typedef struct ztvm_kv_quantize_desc {
  uint32_t kv_heads, head_dim, page_size, tokens;
  uint32_t position_map_elem_offset, pages_word_offset, scales_elem_offset, reserved;
  uint64_t pages_capacity_words, scales_capacity;
  uint64_t k_slot, v_slot, pages_i8, scales, position_map;
} ztvm_kv_quantize_desc;
ZTVM_API int ztvm_kv_quantize_int8(ztvm_ctx* ctx, const ztvm_kv_quantize_desc* desc);

/* Dequantize a weight stack to [N,K] f16 (out_f32=0) or f32 (out_f32=1):
 * w = fl32(q*s + b) (or (q-7)*s), f16 = RNE of that. Uses bits, affine, N,
 * k_packed, scales_per_row, weights, scales, biases and out of `desc`.
 * Replaces the CPU dequantAffineSplit of src/zero-tvm/mlx-weights.ts:598-667
 * and is the bit-exact parity target. */
ZTVM_API int ztvm_dequant(ztvm_ctx* ctx, const ztvm_matmul_desc* desc);

/* ---- the dispatches either side of the matmuls in an FFN / MoE block --------
 * Each replaces one WGSL pipeline of the reference; arguments are its bindings
 * in binding order followed by its PODArgs fields, and the token count where
 * the reference takes it from the dispatch grid. All may be recorded. */

/* silu_mul (src/compiler/shaders/silu_mul.wgsl:17-44; dispatch sites
 * src/zero-tvm/engine-core.ts:2346, :2358, :2518): gate_up is [rows][2*ffn]
 * f16 (gate half, then up half), out[t*ffn+i] = f16(up * gate/(1+exp(-gate)))
 * computed in f32. rows = PODArgs.seq_len; rows == 0 dispatches nothing. */
ZTVM_API int ztvm_silu_mul(ztvm_ctx* ctx, uint64_t out, uint64_t gate_up, uint32_t rows, uint32_t ffn);

/* moe_combine (src/compiler/shaders/moe_combine.wgsl:22-44; engine-core.ts:2348):
 * out[t*N+i] = f16(sum_s score[t*SLOTS+s] * slots[(t*SLOTS+s)*N+i]), f32
 * accumulation in slot order. tokens = grid y. */
ZTVM_API int ztvm_moe_combine(ztvm_ctx* ctx, uint64_t out, uint64_t slots, uint64_t score, uint32_t tokens, uint32_t N,
                              uint32_t SLOTS);

/* moe_router_logits / _q4 / _f16 (src/compiler/shaders/moe_router_logits.wgsl:30-140,
 * moe_router_logits_f16.wgsl:20-57; engine-core.ts:2331): logits[t*rows+e] f32 =
 * sum over groups of 64 of s*sum(x*q) + b*sum(x); bits 8 (4 values per word) or
 * 4 (8 per word), both MLX-affine group 64; bits 16: w is [rows][D] f16 and
 * scales/biases are ignored (pass 0). x is [tokens][D] f16. */
ZTVM_API int ztvm_moe_router_logits(ztvm_ctx* ctx, uint64_t logits, uint64_t x, uint64_t w, uint64_t scales, uint64_t biases,
                                    uint32_t bits, uint32_t D, uint32_t rows, uint32_t tokens);

/* moe_router_topk (src/compiler/shaders/moe_router_topk.wgsl:50-136;
 * engine-core.ts:2332): per token softmax over the E routed logits, then the K
 * largest in descending order, ties to the lower index; scores renormalised
 * over the survivors when norm_topk; has_shared appends slot K = (index E,
 * sigmoid(logit E)). Strides are E+has_shared logits and K+has_shared slots per
 * token; nothing past a token's slots is written. E <= 512, K <= min(E, 64). */
ZTVM_API int ztvm_moe_router_topk(ztvm_ctx* ctx, uint64_t out_idx, uint64_t out_score, uint64_t logits, uint32_t E, uint32_t K,
                                  uint32_t norm_topk, uint32_t has_shared, uint32_t tokens);

/* moe_slot_translate (src/compiler/shaders/moe_slot_translate.wgsl:22-36):
 * ids_out[i] = slot_map[ids_in[i]], a miss (0xffffffff) becomes slot 0; an id
 * >= map_len is treated as a miss, so a bad id cannot fault the GPU. */
ZTVM_API int ztvm_moe_slot_translate(ztvm_ctx* ctx, uint64_t ids_out, uint64_t ids_in, uint64_t slot_map, uint32_t n,
                                     uint32_t map_len);

/* ---- load-time repack of MLX safetensors records (buildBuffer) -------------
 * The records are uploaded as they sit in the file (ztvm_upload); these calls
 * build the bound buffers from them in device memory. `overflow` is the device
 * address of a u32 counter (or 0): values that do not fit f16 are clamped and
 * counted there, and the host treats a nonzero count as a hard error like the
 * reference does (src/zero-tvm/mlx-weights.ts:533-542). */
enum {
  ZTVM_CONVERT_RAW = 0,      /* Convert 'raw' (mlx-weights.ts:210) */
  ZTVM_CONVERT_BF16_F16 = 1, /* 'bf16->f16', bf16ToF16 (mlx-weights.ts:100-127) */
  ZTVM_CONVERT_BF16_F32 = 2  /* 'bf16->f32', bf16ToF32 (mlx-weights.ts:130-135) */
};

/* One part of a concatenation plan: convert src_bytes of a record and store the
 * result at dst, the part's place in the destination buffer
 * (src/zero-tvm/mlx-weights.ts:490-531). bf16->f32 writes 2*src_bytes. */
ZTVM_API int ztvm_repack_part(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t src_bytes, int convert, uint64_t overflow);

/* PlanOp permuteRows (src/zero-tvm/mlx-weights.ts:558-576): destination row j
 * takes source row src_rows[j]. src_rows is a HOST array of src_len entries; a
 * wrong length, bytes not divisible by rows or an index >= rows is ZTVM_E_INVALID
 * (the reference throws). dst and src must not overlap. */
ZTVM_API int ztvm_repack_permute_rows(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes, uint32_t rows,
                                      const uint32_t* src_rows, uint32_t src_len);

/* PlanOp dequantAffineSplit (src/zero-tvm/mlx-weights.ts:598-667): MLX-affine
 * 4-bit group-64 [heads*(nope+v), k] -> f16 heads blocks of [k][nope] (K
 * transposed) followed by heads blocks of [v][k]; value = fl16(fl32(q*s+b)). */
ZTVM_API int ztvm_repack_dequant_split(ztvm_ctx* ctx, uint64_t dst, uint64_t weights, uint64_t scales, uint64_t biases,
                                       uint32_t k, uint32_t heads, uint32_t nope, uint32_t v, uint64_t overflow);

/* ---- command buffers (createCommandEncoder / finish / queue.submit) ------ */

/* Between begin and end, ztvm_matmul / ztvm_dequant / ztvm_fill / ztvm_copy and
 * the block dispatches above are recorded instead of run (src/zero-tvm/engine-core.ts:2565-2570 records a
 * whole token into one encoder). Uploads, downloads and syncs are rejected
 * while recording. */
ZTVM_API int ztvm_record_begin(ztvm_ctx* ctx);
ZTVM_API int ztvm_record_end(ztvm_ctx* ctx, ztvm_cmdbuf** out);
ZTVM_API int ztvm_submit(ztvm_ctx* ctx, ztvm_cmdbuf* cb);
ZTVM_API void ztvm_cmdbuf_destroy(ztvm_cmdbuf* cb);

/* ---- timing (timestamp-query, src/zero-tvm/engine-core.ts:94-102) -------- */

ZTVM_API int ztvm_event_create(ztvm_ctx* ctx, ztvm_event** out);
ZTVM_API void ztvm_event_destroy(ztvm_event* ev);
ZTVM_API int ztvm_event_record(ztvm_ctx* ctx, ztvm_event* ev);
/* Blocks until `stop` completed; milliseconds between the two records. */
ZTVM_API int ztvm_event_elapsed_ms(ztvm_ctx* ctx, ztvm_event* start, ztvm_event* stop, float* ms);

/* ---- launch tuning -------------------------------------------------------- */

/* Named integer knobs for measurement sweeps (e.g. "gemv.wg_per_cu"). Unknown
 * names are ZTVM_E_INVALID. Defaults are the measured best. Three of them decide the f32 summation
 * order over k and so the last f16 bit or two of a result: "skinny.ksplit" and "skinny.shape" (0 =
 * chosen from M, N and K: the same row may then be summed differently in dispatches of different M)
 * and "gemm.split" (0 = the tile GEMM deals the tiles of a last round of workgroups that fills at
 * most half the CUs to several workgroups along k, which add their f32 totals in a fixed order; 1 =
 * never). Pin them for rows that must not depend on the batch they travel in. */
ZTVM_API int ztvm_set_option(ztvm_ctx* ctx, const char* name, int value);
ZTVM_API int ztvm_get_option(ztvm_ctx* ctx, const char* name, int* value);

#ifdef __cplusplus
}
#endif
#endif /* ZTVM_H */
