// Internal interfaces between the C ABI (ztvm_api.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ztvm {

// The fused QKV form (QKV matmul + RoPE + KV append): where the rotated pairs go.
struct QkvArgs {
  _Float16* q_out;
  _Float16* kv_pages;
  _Float16* k_slot = nullptr;  // both set: K and V go to two [kv_heads*head_dim] rows instead of the paged cache
  _Float16* v_slot = nullptr;
  const int32_t* position_map;
  uint32_t heads, kv_heads, head_dim;
  uint32_t page_size, kv_page_stride, head_page_stride, v_page_offset;  // f16 elements
  uint32_t position_map_elem_offset, pages_elem_offset;
  uint64_t kv_capacity;
  float rope_theta;
};

// Resolved launch arguments for every kernel family (device pointers typed).
struct MatmulArgs {
  void* out;
  const _Float16* in;
  const _Float16* scales;
  const uint32_t* weights;
  const _Float16* biases;
  const uint32_t* ids;
  // gated FFN form (null = plain matmul): the up projection, same shape and format as `weights`
  const uint32_t* up_weights = nullptr;
  const _Float16* up_scales = nullptr;
  const _Float16* up_biases = nullptr;
  // prologue form of the gated FFN (null = none): `in` is the residual, x = RMSNorm(in + delta) * gamma
  const _Float16* delta = nullptr;
  const _Float16* gamma = nullptr;
  float rms_eps = 0.f;
  const QkvArgs* qkv = nullptr;  // with qkv set, N counts rotary pairs and up_* is the same matrix half a head further
  uint32_t M, N, K, k_packed, spr;
  uint32_t bits, affine, out_f32;
  uint32_t slots, tokens;  // slots == 0: dense
  uint32_t in_slot_stride, out_slot_stride, in_tok_stride, out_tok_stride, ids_stride, experts;
};

// Launch knobs (ztvm_set_option). Zero means "use the built-in default".
struct Tune {
  int num_cus = 256;
  int gemv_wg_per_cu = 0;   // workgroups resident per CU for the streaming GEMV
  int gemv_rows = 0;        // rows per wave step (1, 2 or 4)
  int gemv_waves = 0;       // waves per workgroup (4..8)
  int gemv_ring = 0;        // passes in flight per wave of the streaming kernel (0: two; 1, 3)
  int gemv_stream = 0;      // 0: dense single rows go to the register-resident streaming kernel where it applies; 1: never
  int skinny_dma = 0;        // 1: the transfer-engine form of the skinny kernel is switched off
  int skinny_shape = 0;      // transfer-engine form: 0 = by M; 2 = 64 rows x 128 columns x 2 k parts; 3 = 32 x 64 x 4
  int skinny_ksplit = 0;     // workgroups sharing the k range of one skinny tile (0: chosen from M, N, K)
  int rows_wg_per_cu = 0;    // the row-group GEMV: workgroups per CU and waves per workgroup (0: chosen from the LDS it stages)
  int rows_waves = 0;
  int gemm_tile = 0;        // 0 auto
  int gemm_split = 0;       // the tile GEMM's k split: 0 = where it fills a round of workgroups, 1 = never
  int gemm_xcd_swizzle = 1;
};

hipError_t launch_gemv(const MatmulArgs& a, const Tune& t, hipStream_t s);
bool gemv_supports(const MatmulArgs& a);  // the activation row fits the LDS staging
// the dense single-row streaming kernel (gemv_stream.hip)
bool gemv_stream_supports(const MatmulArgs& a, const Tune& t);
hipError_t launch_gemv_stream(const MatmulArgs& a, const Tune& t, hipStream_t s);
hipError_t launch_skinny(const MatmulArgs& a, const Tune& t, void* scratch, hipStream_t s);
size_t skinny_scratch_bytes(const MatmulArgs& a, const Tune& t);
// The tile GEMM's k split for a descriptor: tiles [0, full_tiles) run whole, each of the others is dealt to `parts`
// workgroups of steps_per_part 64-k steps, which exchange partial_bytes of f32 totals through the scratch buffer.
struct GemmSplit {
  uint32_t full_tiles, parts, steps_per_part;
  size_t partial_bytes;
};
constexpr uint32_t ZTVM_GEMM_SPLIT_TILES = 256;  // arrival counters a context owns: at most this many split tiles
GemmSplit gemm_split(const MatmulArgs& a, const Tune& t, size_t scratch_limit);
// scratch_limit: the bytes the caller can give (0: as many as it takes); a split that does not fit is not made
hipError_t launch_gemm(const MatmulArgs& a, const Tune& t, void* scratch, uint32_t* counters, size_t scratch_limit, hipStream_t s);
size_t gemm_scratch_bytes(const MatmulArgs& a, const Tune& t, size_t scratch_limit);
hipError_t launch_dequant(const MatmulArgs& a, hipStream_t s);
hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t s);
hipError_t launch_read_probe(const void* src, size_t bytes, void* sink, hipStream_t s);
hipError_t launch_fill(void* dst, int byte, size_t bytes, hipStream_t s);

// the dispatches around the matmuls of an FFN / MoE block (block_ops.hip)
hipError_t launch_silu_mul(void* out, const void* gate_up, uint32_t rows, uint32_t ffn, hipStream_t s);
hipError_t launch_moe_combine(void* out, const void* slots, const void* score, uint32_t tokens, uint32_t N, uint32_t S, hipStream_t s);
hipError_t launch_router_logits(void* logits, const void* x, const void* w, const void* scales, const void* biases, uint32_t bits,
                                uint32_t D, uint32_t rows, uint32_t tokens, hipStream_t s);
hipError_t launch_router_topk(void* out_idx, void* out_score, const void* logits, uint32_t E, uint32_t K, uint32_t norm_topk,
                              uint32_t has_shared, uint32_t tokens, hipStream_t s);
uint32_t router_topk_max_experts();
hipError_t launch_kv_quantize_int8(void* pages_i8, void* scales, const void* k_slot, const void* v_slot, const int32_t* position_map,
                                   uint32_t kv_heads, uint32_t head_dim, uint32_t page_size, uint32_t tokens, uint32_t pos_off,
                                   uint32_t pages_word_off, uint32_t scales_off, uint64_t pages_capacity_words, uint64_t scales_capacity,
                                   hipStream_t s);
hipError_t launch_slot_translate(void* ids_out, const void* ids_in, const void* slot_map, uint32_t n, uint32_t map_len, hipStream_t s);

// load-time repacking of checkpoint records (repack.hip); convert: 0 raw, 1 bf16->f16, 2 bf16->f32
hipError_t launch_repack_convert(void* dst, const void* src, size_t src_bytes, int convert, uint32_t* counter, hipStream_t s);
hipError_t launch_permute_rows(void* dst, const void* src, const uint32_t* map, uint32_t rows, size_t row_bytes, hipStream_t s);
hipError_t launch_dequant_split(void* out, const void* w, const void* scales, const void* biases, uint32_t k, uint32_t heads,
                                uint32_t nope, uint32_t v, uint32_t* counter, hipStream_t s);

bool skinny_supports(const MatmulArgs& a);
// the row-group GEMV (gemv_rows.hip), 1 <= M <= 16
bool rows_supports(const MatmulArgs& a);
size_t rows_scratch_bytes(const MatmulArgs& a);
hipError_t launch_rows(const MatmulArgs& a, const Tune& t, void* scratch, hipStream_t s);
// out[i] = sum over the k splits of partial[k][i], in split order; count a multiple of four (skinny.hip)
hipError_t launch_reduce_partials(const float* partial, void* out, uint32_t count, uint32_t ksplit, bool out_f32, hipStream_t s);
bool gemm_supports(const MatmulArgs& a);

}  // namespace ztvm
