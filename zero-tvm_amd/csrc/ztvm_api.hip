// C ABI of libztvm_hip: context, buffers, descriptor validation, dispatch,
// command buffers (HIP graphs) and events. See include/ztvm.h for the contract
// and the reference interfaces each entry point replaces.
#include "../../include/ztvm.h"
#include "internal.h"
#include "skinny.h"
#include "scratch_pool.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>

using namespace ztvm;

namespace {
// hipMalloc / hipFree on the context's device
struct DeviceAlloc {
  int device = 0;
  void* allocate(size_t bytes) const {
    void* p = nullptr;
    if (hipSetDevice(device) != hipSuccess || hipMalloc(&p, bytes) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    return p;
  }
  void release(void* p) const {
    (void)hipSetDevice(device);
    (void)hipFree(p);  // waits for the device: nothing in flight still reads the buffer
  }
};
using DevicePool = ScratchPool<DeviceAlloc>;

// Scratch of ztvm_matmul_static: device memory that exists from the moment the library's code object
// is loaded, so the entry point never allocates. Every GPU the library runs on holds its own copy at
// its own address; host code must only ever use the per-device address that hipGetSymbolAddress
// returned (the array's name is not a device address on the host side).
static __device__ __align__(256) __attribute__((used)) unsigned char static_scratch[ZTVM_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
std::mutex g_static_mu;
void* g_static_ptr[kMaxDevices] = {};

// Address of `device`'s copy of the array, looked up once per device with that device current.
hipError_t static_scratch_of(int device, void** out) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[device]) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return e;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_static_ptr[device] = p;
  }
  *out = g_static_ptr[device];
  return hipSuccess;
}
}  // namespace

struct ztvm_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool recording = false;
  Tune tune;
  // Library-owned device memory of the rows / skinny / tile-GEMM families (activation group sums,
  // reordered activations, split-k partial sums). Shared with the command buffers recorded on this
  // context, which keep its addresses alive (scratch_pool.h).
  std::shared_ptr<DevicePool> scratch;
  void* static_scratch = nullptr;  // this device's copy of the file-scope array above
  uint32_t* gemm_counters = nullptr;  // arrival counters of the tile GEMM's k split: zero between launches
  std::string err;
  hipDeviceProp_t prop;
};
struct ztvm_cmdbuf {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::shared_ptr<DevicePool> scratch;  // pinned while this command buffer lives
};
struct ztvm_event {
  hipEvent_t ev = nullptr;
};

namespace {

thread_local std::string g_err = "";

int fail(ztvm_ctx* ctx, int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (ctx) ctx->err = buf;
  g_err = buf;
  return code;
}

#define HIP_TRY(ctx, expr)                                                                          \
  do {                                                                                              \
    hipError_t e_ = (expr);                                                                         \
    if (e_ != hipSuccess) return fail(ctx, ZTVM_E_HIP, "%s: %s", #expr, hipGetErrorString(e_));     \
  } while (0)

void why_set(char* why, size_t n, const char* fmt, ...) {
  if (!why || !n) return;
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(why, n, fmt, ap);
  va_end(ap);
}

// The legality rules of the generator (int4_matmul.gen.ts:172-197) that are
// about arithmetic, plus the layout contract of the bindings.
int validate(const ztvm_matmul_desc* d, char* why, size_t n, bool need_in_out) {
  if (!d) { why_set(why, n, "null descriptor"); return ZTVM_E_INVALID; }
  if (d->bits != 4 && d->bits != 3 && d->bits != 8) { why_set(why, n, "bits must be 4, 3 or 8 (got %u)", d->bits); return ZTVM_E_INVALID; }
  if (d->affine > 1 || d->out_f32 > 1) { why_set(why, n, "affine/out_f32 must be 0 or 1"); return ZTVM_E_INVALID; }
  if (d->bits == 3 && !d->affine) { why_set(why, n, "q3 requires affine (3-bit ships only in the MLX-affine layout)"); return ZTVM_E_INVALID; }
  if (d->bits == 8 && !d->affine) { why_set(why, n, "8-bit requires affine (8-bit ships only in the MLX-affine layout)"); return ZTVM_E_INVALID; }
  if (d->slots && !d->affine) { why_set(why, n, "moe requires affine (the MoE weights are MLX affine-quantised)"); return ZTVM_E_INVALID; }
  if (d->kernel > ZTVM_KERNEL_ROWS) { why_set(why, n, "unknown kernel family %u", d->kernel); return ZTVM_E_INVALID; }
  if (!d->N) { why_set(why, n, "N must be > 0"); return ZTVM_E_INVALID; }
  if (!d->k_packed) { why_set(why, n, "K_PACKED must be > 0"); return ZTVM_E_INVALID; }
  const uint64_t kbits = (uint64_t)d->k_packed * 32u;
  if (kbits % d->bits) { why_set(why, n, "K_PACKED=%u words do not hold a whole number of %u-bit values", d->k_packed, d->bits); return ZTVM_E_INVALID; }
  const uint64_t K = kbits / d->bits;
  const uint32_t G = d->affine ? 64u : 32u;
  if (K % G) { why_set(why, n, "K=%llu is not a multiple of the group size %u", (unsigned long long)K, G); return ZTVM_E_INVALID; }
  if (K > (1u << 24)) { why_set(why, n, "K=%llu too large", (unsigned long long)K); return ZTVM_E_INVALID; }
  if ((uint64_t)d->scales_per_row != K / G) {
    why_set(why, n, "SCALES_PER_ROW=%u but K/group = %llu (K=%llu, group %u)", d->scales_per_row, (unsigned long long)(K / G), (unsigned long long)K, G);
    return ZTVM_E_INVALID;
  }
  // the streaming kernels address a matrix with 32-bit byte offsets from its base
  if ((uint64_t)d->N * d->k_packed * 4u >= (1ull << 31)) { why_set(why, n, "one weight matrix must stay under 2 GiB (N=%u rows of %u words)", d->N, d->k_packed); return ZTVM_E_INVALID; }
  if (need_in_out) {
    if (d->slots) {
      if (d->M != 1) { why_set(why, n, "moe dispatches one activation row per (token,slot): M must be 1 (got %u)", d->M); return ZTVM_E_INVALID; }
      if (!d->tokens) { why_set(why, n, "moe needs tokens > 0"); return ZTVM_E_INVALID; }
      if (d->ids_stride < d->slots) { why_set(why, n, "IDS_STRIDE=%u < slots=%u", d->ids_stride, d->slots); return ZTVM_E_INVALID; }
      if (!d->ids) { why_set(why, n, "null buffer at binding 6 (ids)"); return ZTVM_E_INVALID; }
      if (d->ids & 3u) { why_set(why, n, "ids must be 4-byte aligned"); return ZTVM_E_INVALID; }
      if ((d->in_slot_stride | d->in_tok_stride) & 7u) { why_set(why, n, "moe input strides must be multiples of 8 elements"); return ZTVM_E_INVALID; }
      if (d->out_slot_stride < d->N && d->slots > 1) { why_set(why, n, "OUT_SLOT_STRIDE=%u < N=%u would overlap slot outputs", d->out_slot_stride, d->N); return ZTVM_E_INVALID; }
      if (!d->experts) { why_set(why, n, "moe needs experts > 0 (the height of the bound stacks, which arms the expert-id guard), or ZTVM_EXPERTS_UNCHECKED"); return ZTVM_E_INVALID; }
    } else {
      if (!d->M) { why_set(why, n, "M must be > 0"); return ZTVM_E_INVALID; }
    }
    if (!d->in) { why_set(why, n, "null buffer at binding 1 (input)"); return ZTVM_E_INVALID; }
    if (d->in & 15u) { why_set(why, n, "input must be 16-byte aligned"); return ZTVM_E_INVALID; }
  }
  if (!d->out) { why_set(why, n, "null buffer at binding 0 (output)"); return ZTVM_E_INVALID; }
  if (!d->scales) { why_set(why, n, "null buffer at binding 2 (scales)"); return ZTVM_E_INVALID; }
  if (!d->weights) { why_set(why, n, "null buffer at binding 3 (weights)"); return ZTVM_E_INVALID; }
  if (d->affine && !d->biases) { why_set(why, n, "affine matmul has no bias buffer at binding 5"); return ZTVM_E_INVALID; }
  if (d->weights & 15u) { why_set(why, n, "weights must be 16-byte aligned"); return ZTVM_E_INVALID; }
  if ((d->scales & 15u) || (d->affine && (d->biases & 15u))) { why_set(why, n, "scales/biases must be 16-byte aligned"); return ZTVM_E_INVALID; }
  if (d->out & (d->out_f32 ? 3u : 1u)) { why_set(why, n, "output misaligned for its element type"); return ZTVM_E_INVALID; }
  return ZTVM_OK;
}

MatmulArgs to_args(const ztvm_matmul_desc* d) {
  MatmulArgs a{};
  a.out = reinterpret_cast<void*>(d->out);
  a.in = reinterpret_cast<const _Float16*>(d->in);
  a.scales = reinterpret_cast<const _Float16*>(d->scales);
  a.weights = reinterpret_cast<const uint32_t*>(d->weights);
  a.biases = reinterpret_cast<const _Float16*>(d->biases);
  a.ids = reinterpret_cast<const uint32_t*>(d->ids);
  a.M = d->M; a.N = d->N; a.k_packed = d->k_packed; a.spr = d->scales_per_row;
  a.K = (uint32_t)((uint64_t)d->k_packed * 32u / d->bits);
  a.bits = d->bits; a.affine = d->affine; a.out_f32 = d->out_f32;
  a.slots = d->slots; a.tokens = d->tokens;
  a.in_slot_stride = d->in_slot_stride; a.out_slot_stride = d->out_slot_stride;
  a.in_tok_stride = d->in_tok_stride; a.out_tok_stride = d->out_tok_stride;
  a.ids_stride = d->ids_stride; a.experts = d->experts;
  return a;
}

// Which family runs a descriptor. Thresholds are measured crossovers on
// MI355X: the GEMV re-reads the weights once per activation row, the skinny
// kernel streams them once per tile of up to 128 rows, the tile GEMM needs
// enough tiles to fill the CUs.
int resolve_family(const MatmulArgs& a, uint32_t want, char* why, size_t n);

int resolve(const MatmulArgs& a, uint32_t want, char* why, size_t n) {
  const int fam = resolve_family(a, want, why, n);
  if (fam == ZTVM_KERNEL_GEMV && !gemv_supports(a)) {
    why_set(why, n, "kernel: the GEMV family stages the activation row in LDS and K=%u does not fit (this dispatch has no other family: moe=%d, M=%u)", a.K, (int)(a.slots > 0), a.M);
    return ZTVM_E_UNSUPPORTED;
  }
  return fam;
}

// Above 128 rows two families can run 4-bit rows: the tile GEMM (256 x 128 tiles from 257 rows, 128 x 128 below; no
// k split) and the transfer-engine skinny kernel (64 x 128 tiles, k split when the tiles are few). Per flop the tile
// GEMM is the better kernel, but it leaves CUs idle where ceil(M/256) x N/128 tiles are few or just past a multiple
// of the CU count (N = 4096, M = 512: 64 workgroups). The choice is made on an estimate of both, in nanoseconds,
// fitted to measurements on MI355X at K = 2048..14336, N = 4096..14336, M = 129..2048: every family runs
// ceil(workgroups / CUs) rounds; a 64-k step costs a tile-GEMM workgroup 0.98 us (0.8 us on the smaller tile) and
// a skinny workgroup 0.375 us; around the steps a GEMM launch spends 10 us, a skinny launch 2 us and 4 us per
// round, and 4 us more for the reduction of a k split. The estimate reproduces the measured winner at every
// measured point (K=4096 N=14336: skinny up to 256 rows, 53 against 62 us; K=14336 N=4096: skinny up to 1024
// rows, 92 against 213 us at 512; K=4096 N=4096: skinny up to 1024 rows, 32 against 66 us at 512). The CU count
// is the constant of the GPU this library is written for, so that the choice is a function of the descriptor.
constexpr uint64_t MODEL_CUS = 256;
uint64_t est_gemm_ns(const MatmulArgs& a) {
  const bool big = a.M > 256;
  const uint64_t step_ns = big ? 980 : 800;
  // with the k split of the tiles past the last full round (gemm_split): the full rounds, then one round of
  // `parts` workgroups per tile and the exchange of their f32 totals (12 us)
  Tune t{};
  t.num_cus = (int)MODEL_CUS;
  const GemmSplit g = gemm_split(a, t, 0);
  const uint64_t rounds = g.full_tiles / MODEL_CUS + (g.parts == 1 && g.full_tiles % MODEL_CUS ? 1 : 0);
  uint64_t ns = rounds * (a.K / 64) * step_ns + 10000;
  if (g.parts > 1) ns += g.steps_per_part * step_ns + 12000;
  return ns;
}
// The register-path skinny kernel (3-bit and 8-bit rows, K off a multiple of 128): 128-row tiles, about 1 us per
// 64-k step, a k split that depends on N and K only and whose f32 partial results are written and read back once
// (4 TB/s), a pre-pass that copies the activations (3 TB/s). Fitted like the others (8-bit and 3-bit, the same four
// shapes, M = 192..1024; K=14336 N=4096 M=256: 95 against 205 us, M=512: 170 against 219; K=4096 N=4096 M=256:
// 47 against 64).
uint64_t est_skinny_reg_ns(const MatmulArgs& a) {
  Tune t{};
  t.num_cus = (int)MODEL_CUS;
  const uint64_t ks = skinny_reg_ksplit(a, t);
  const uint64_t tiles = ((a.M + 127) / 128) * (uint64_t)((a.N + 127) / 128);
  const uint64_t rounds = (tiles * ks + MODEL_CUS - 1) / MODEL_CUS;
  const uint64_t steps = (a.K / 64 + ks - 1) / ks;
  const uint64_t partial_bytes = ks > 1 ? 2ull * a.M * a.N * 4 * ks : 0;
  const uint64_t prep_bytes = 2ull * a.M * a.K * 2;
  return rounds * (steps * 1000 + 4000) + 2000 + partial_bytes / 4000 + prep_bytes / 3000;
}
uint64_t est_skinny_ns(const MatmulArgs& a) {
  if (!skinny_dma_supports(a, Tune{})) return est_skinny_reg_ns(a);
  Tune t{};
  t.num_cus = (int)MODEL_CUS;
  const uint64_t ks = skinny_dma_ksplit(a, t);
  const uint64_t tiles = ((a.M + 63) / 64) * (uint64_t)((a.N + 127) / 128);
  const uint64_t rounds = (tiles * ks + MODEL_CUS - 1) / MODEL_CUS;
  const uint64_t steps = (a.K / 64 + ks - 1) / ks;
  return rounds * (steps * 375 + 4000) + 2000 + (ks > 1 ? 4000 : 0);
}

int resolve_family(const MatmulArgs& a, uint32_t want, char* why, size_t n) {
  const bool moe = a.slots > 0;
  const bool sk = !moe && skinny_supports(a);
  const bool ge = !moe && gemm_supports(a);
  const bool ro = !moe && rows_supports(a);
  if (want == ZTVM_KERNEL_GEMV) return ZTVM_KERNEL_GEMV;
  if (want == ZTVM_KERNEL_SKINNY) {
    if (!sk) { why_set(why, n, "kernel: asked for 'skinny', which cannot run this dispatch (moe=%d, M=%u)", (int)moe, a.M); return ZTVM_E_UNSUPPORTED; }
    return ZTVM_KERNEL_SKINNY;
  }
  if (want == ZTVM_KERNEL_GEMM) {
    if (!ge) { why_set(why, n, "kernel: asked for 'gemm', which cannot run this dispatch (moe=%d, bits=%u, out_f32=%u, K=%u)", (int)moe, a.bits, a.out_f32, a.K); return ZTVM_E_UNSUPPORTED; }
    return ZTVM_KERNEL_GEMM;
  }
  if (want == ZTVM_KERNEL_ROWS) {
    if (!ro) { why_set(why, n, "kernel: asked for 'rows', which cannot run this dispatch (moe=%d, M=%u, K=%u, N=%u)", (int)moe, a.M, a.K, a.N); return ZTVM_E_UNSUPPORTED; }
    return ZTVM_KERNEL_ROWS;
  }
  if (moe || a.M == 1) return ZTVM_KERNEL_GEMV;
  // 4-bit rows that the transfer-engine skinny kernel takes: it passes the row-group GEMV at 13 rows (16.3 against
  // 16.9 us at M = 12, 16.8 against 19.5 at M = 16; K = 4096, N = 14336)
  if (ro && !(a.M > 12 && sk && skinny_dma_supports(a, Tune{}))) return ZTVM_KERNEL_ROWS;
  if (ge && a.M > 128) {
    if (sk && est_skinny_ns(a) < est_gemm_ns(a)) return ZTVM_KERNEL_SKINNY;
    return ZTVM_KERNEL_GEMM;
  }
  if (sk) return ZTVM_KERNEL_SKINNY;
  if (ge) return ZTVM_KERNEL_GEMM;
  return ZTVM_KERNEL_GEMV;
}

// The context's scratch buffer, grown to `need` bytes if it is smaller. Growing allocates, which a
// recording cannot hold; outside a recording the old buffer is retired, not freed, while any
// command buffer that may carry its address is alive.
int scratch_for(ztvm_ctx* ctx, size_t need, void** out) {
  DevicePool& pool = *ctx->scratch;
  if (need > pool.bytes()) {
    if (ctx->recording)
      return fail(ctx, ZTVM_E_UNSUPPORTED, "this dispatch needs %zu bytes of scratch (have %zu) and a recording cannot allocate; dispatch it once outside a recording first", need, pool.bytes());
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return fail(ctx, ZTVM_E_HIP, "hipStreamSynchronize: %s", hipGetErrorString(e));
    if (!pool.reserve(need)) return fail(ctx, ZTVM_E_HIP, "no device memory for %zu bytes of scratch", need);
  }
  *out = pool.data();
  return ZTVM_OK;
}

struct Option {
  const char* name;
  int Tune::*field;
};
const Option kOptions[] = {
    {"num_cus", &Tune::num_cus},
    {"gemv.wg_per_cu", &Tune::gemv_wg_per_cu},
    {"gemv.rows", &Tune::gemv_rows},
    {"gemv.waves", &Tune::gemv_waves},
    {"gemv.stream", &Tune::gemv_stream},
    {"gemv.ring", &Tune::gemv_ring},
    {"skinny.ksplit", &Tune::skinny_ksplit},
    {"skinny.dma", &Tune::skinny_dma},
    {"skinny.shape", &Tune::skinny_shape},
    {"rows.wg_per_cu", &Tune::rows_wg_per_cu},
    {"rows.waves", &Tune::rows_waves},
    {"gemm.tile", &Tune::gemm_tile},
    {"gemm.split", &Tune::gemm_split},
    {"gemm.xcd_swizzle", &Tune::gemm_xcd_swizzle},
};

}  // namespace

extern "C" {

int ztvm_abi_version(void) { return ZTVM_ABI_VERSION; }

const char* ztvm_last_error(ztvm_ctx* ctx) { return ctx ? ctx->err.c_str() : g_err.c_str(); }

int ztvm_create(int device, ztvm_ctx** out) {
  if (!out) return fail(nullptr, ZTVM_E_INVALID, "ztvm_create: null out pointer");
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return fail(nullptr, ZTVM_E_NODEVICE, "no HIP device visible");
  if (device < 0 || device >= count) return fail(nullptr, ZTVM_E_INVALID, "device %d out of range (%d visible)", device, count);
  // every exit below that is not the last one gives back what the context holds by then
  struct Guard {
    ztvm_ctx* c;
    ~Guard() { if (c) ztvm_destroy(c); }
  } g{new ztvm_ctx()};
  ztvm_ctx* c = g.c;
  c->device = device;
  HIP_TRY(nullptr, hipSetDevice(device));
  HIP_TRY(nullptr, hipGetDeviceProperties(&c->prop, device));
  if (!strstr(c->prop.gcnArchName, "gfx950"))
    return fail(nullptr, ZTVM_E_NODEVICE, "device %d is %s; this library holds gfx950 code only", device, c->prop.gcnArchName);
  HIP_TRY(nullptr, hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
  c->tune.num_cus = c->prop.multiProcessorCount > 0 ? c->prop.multiProcessorCount : 256;
  {
    hipError_t e = static_scratch_of(device, &c->static_scratch);
    if (e != hipSuccess) return fail(nullptr, ZTVM_E_HIP, "ztvm_create: address of the static scratch array: %s", hipGetErrorString(e));
  }
  c->scratch = std::make_shared<DevicePool>(DeviceAlloc{device});
  if (!c->scratch->reserve(4u << 20)) return fail(nullptr, ZTVM_E_HIP, "ztvm_create: no device memory for the scratch buffer");
  HIP_TRY(nullptr, hipMalloc(reinterpret_cast<void**>(&c->gemm_counters), ZTVM_GEMM_SPLIT_TILES * sizeof(uint32_t)));
  HIP_TRY(nullptr, hipMemset(c->gemm_counters, 0, ZTVM_GEMM_SPLIT_TILES * sizeof(uint32_t)));
  HIP_TRY(nullptr, hipDeviceSynchronize());  // the fill runs on the null stream, which the context's stream does not wait for
  g.c = nullptr;
  *out = c;
  return ZTVM_OK;
}

void ztvm_destroy(ztvm_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
  }
  if (ctx->gemm_counters) (void)hipFree(ctx->gemm_counters);
  if (ctx->scratch) ctx->scratch->release_all();  // command buffers of this context are dead with it
  delete ctx;
}

int ztvm_device_info(ztvm_ctx* ctx, char* name, size_t name_len, uint32_t* cus, uint64_t* hbm) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (name && name_len) snprintf(name, name_len, "%s (%s)", ctx->prop.name, ctx->prop.gcnArchName);
  if (cus) *cus = (uint32_t)ctx->prop.multiProcessorCount;
  if (hbm) *hbm = (uint64_t)ctx->prop.totalGlobalMem;
  return ZTVM_OK;
}

int ztvm_alloc(ztvm_ctx* ctx, size_t bytes, uint64_t* dptr) {
  if (!ctx || !dptr) return fail(ctx, ZTVM_E_INVALID, "ztvm_alloc: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_alloc while recording a command buffer");
  void* p = nullptr;
  HIP_TRY(ctx, hipSetDevice(ctx->device));
  HIP_TRY(ctx, hipMalloc(&p, bytes < 4 ? 4 : bytes));
  *dptr = reinterpret_cast<uint64_t>(p);
  return ZTVM_OK;
}

int ztvm_free(ztvm_ctx* ctx, uint64_t dptr) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_free while recording a command buffer");
  if (!dptr) return ZTVM_OK;
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  HIP_TRY(ctx, hipFree(reinterpret_cast<void*>(dptr)));
  return ZTVM_OK;
}

int ztvm_upload(ztvm_ctx* ctx, uint64_t dst, size_t off, const void* src, size_t bytes) {
  if (!ctx || !dst || (!src && bytes)) return fail(ctx, ZTVM_E_INVALID, "ztvm_upload: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_upload while recording a command buffer");
  if (!bytes) return ZTVM_OK;
  HIP_TRY(ctx, hipMemcpyAsync(reinterpret_cast<char*>(dst) + off, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // the source may be reused on return
  return ZTVM_OK;
}

int ztvm_download(ztvm_ctx* ctx, void* dst, uint64_t src, size_t off, size_t bytes) {
  if (!ctx || !src || (!dst && bytes)) return fail(ctx, ZTVM_E_INVALID, "ztvm_download: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_download while recording a command buffer");
  if (!bytes) return ZTVM_OK;
  HIP_TRY(ctx, hipMemcpyAsync(dst, reinterpret_cast<const char*>(src) + off, bytes, hipMemcpyDeviceToHost, ctx->stream));
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return ZTVM_OK;
}

int ztvm_fill(ztvm_ctx* ctx, uint64_t dst, size_t off, int byte, size_t bytes) {
  if (!ctx || !dst) return fail(ctx, ZTVM_E_INVALID, "ztvm_fill: null argument");
  if (!bytes) return ZTVM_OK;
  HIP_TRY(ctx, launch_fill(reinterpret_cast<char*>(dst) + off, byte, bytes, ctx->stream));
  return ZTVM_OK;
}

int ztvm_copy(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes) {
  if (!ctx || !dst || !src) return fail(ctx, ZTVM_E_INVALID, "ztvm_copy: null argument");
  if ((dst | src | bytes) & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_copy: addresses and size must be multiples of 16 bytes");
  if (!bytes) return ZTVM_OK;
  HIP_TRY(ctx, launch_copy(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), bytes, ctx->stream));
  return ZTVM_OK;
}

int ztvm_read_probe(ztvm_ctx* ctx, uint64_t src, size_t bytes, uint64_t sink) {
  if (!ctx || !src || !sink) return fail(ctx, ZTVM_E_INVALID, "ztvm_read_probe: null argument");
  if ((src & 15u) || (bytes & 15u) || (sink & 3u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_read_probe: src and size must be multiples of 16 bytes, sink of 4");
  if (!bytes) return ZTVM_OK;
  HIP_TRY(ctx, launch_read_probe(reinterpret_cast<const void*>(src), bytes, reinterpret_cast<void*>(sink), ctx->stream));
  return ZTVM_OK;
}

int ztvm_sync(ztvm_ctx* ctx) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_sync while recording a command buffer");
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
  return ZTVM_OK;
}

int ztvm_matmul_validate(const ztvm_matmul_desc* desc, char* why, size_t why_len) {
  if (why && why_len) why[0] = 0;
  int rc = validate(desc, why, why_len, true);
  if (rc) return rc;
  const MatmulArgs a = to_args(desc);
  rc = resolve(a, desc->kernel, why, why_len);
  return rc < 0 ? rc : ZTVM_OK;
}

int ztvm_matmul_resolve(const ztvm_matmul_desc* desc) {
  char why[256];
  int rc = validate(desc, why, sizeof why, true);
  if (rc) return fail(nullptr, rc, "%s", why);
  const MatmulArgs a = to_args(desc);
  rc = resolve(a, desc->kernel, why, sizeof why);
  if (rc < 0) return fail(nullptr, rc, "%s", why);
  return rc;
}

// use_static: the scratch is this device's copy of the file-scope array, nothing is allocated
static int matmul_impl(ztvm_ctx* ctx, const ztvm_matmul_desc* desc, bool use_static) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  char why[256];
  int rc = validate(desc, why, sizeof why, true);
  if (rc) return fail(ctx, rc, "ztvm_matmul: %s", why);
  MatmulArgs a = to_args(desc);
  int fam = resolve(a, desc->kernel, why, sizeof why);
  if (fam < 0) return fail(ctx, fam, "ztvm_matmul: %s", why);
  // the skinny family works on a reordered copy of the activations in scratch; where the choice was the library's
  // and that copy outgrows the fixed buffer, the tile GEMM (group sums only) takes the dispatch
  if (use_static && desc->kernel == ZTVM_KERNEL_AUTO && fam == ZTVM_KERNEL_SKINNY && a.M > 128 && gemm_supports(a) &&
      skinny_scratch_bytes(a, ctx->tune) > (size_t)ZTVM_STATIC_SCRATCH_BYTES)
    fam = ZTVM_KERNEL_GEMM;
  switch (fam) {
    case ZTVM_KERNEL_ROWS:
    case ZTVM_KERNEL_SKINNY:
    case ZTVM_KERNEL_GEMM: {
      // the tile GEMM's k split takes what the fixed buffer leaves after the group sums, or is not made
      const size_t limit = use_static ? (size_t)ZTVM_STATIC_SCRATCH_BYTES : 0;
      const size_t need = fam == ZTVM_KERNEL_GEMM ? gemm_scratch_bytes(a, ctx->tune, limit) : (fam == ZTVM_KERNEL_ROWS ? rows_scratch_bytes(a) : skinny_scratch_bytes(a, ctx->tune));
      void* scratch = nullptr;
      if (use_static) {
        if (need > (size_t)ZTVM_STATIC_SCRATCH_BYTES)
          return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_matmul_static: this dispatch needs %zu bytes of scratch, the static buffer holds %zu (M=%u N=%u K=%u); use ztvm_matmul",
                      need, (size_t)ZTVM_STATIC_SCRATCH_BYTES, a.M, a.N, a.K);
        scratch = ctx->static_scratch;
      } else {
        rc = scratch_for(ctx, need, &scratch);
        if (rc) return rc;
      }
      if (fam == ZTVM_KERNEL_GEMM) HIP_TRY(ctx, launch_gemm(a, ctx->tune, scratch, ctx->gemm_counters, limit, ctx->stream));
      else if (fam == ZTVM_KERNEL_ROWS) HIP_TRY(ctx, launch_rows(a, ctx->tune, scratch, ctx->stream));
      else HIP_TRY(ctx, launch_skinny(a, ctx->tune, scratch, ctx->stream));
      break;
    }
    default: {
      // one streaming pass over the weights per activation row
      const uint32_t M = a.slots ? 1 : a.M;
      const size_t out_elt = a.out_f32 ? 4 : 2;
      for (uint32_t m = 0; m < M; m++) {
        MatmulArgs r = a;
        r.in = a.in + (size_t)m * a.K;
        r.out = reinterpret_cast<char*>(a.out) + (size_t)m * a.N * out_elt;
        r.M = 1;
        if (ctx->tune.gemv_stream == 0 && gemv_stream_supports(r, ctx->tune)) HIP_TRY(ctx, launch_gemv_stream(r, ctx->tune, ctx->stream));
        else HIP_TRY(ctx, launch_gemv(r, ctx->tune, ctx->stream));
      }
    }
  }
  return ZTVM_OK;
}

int ztvm_matmul(ztvm_ctx* ctx, const ztvm_matmul_desc* desc) { return matmul_impl(ctx, desc, false); }

int ztvm_matmul_static(ztvm_ctx* ctx, const ztvm_matmul_desc* desc) { return matmul_impl(ctx, desc, true); }

int ztvm_ffn_gated(ztvm_ctx* ctx, const ztvm_matmul_desc* desc, uint64_t up_weights, uint64_t up_scales, uint64_t up_biases) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  char why[256];
  int rc = validate(desc, why, sizeof why, true);
  if (rc) return fail(ctx, rc, "ztvm_ffn_gated: %s", why);
  if (desc->kernel != ZTVM_KERNEL_AUTO && desc->kernel != ZTVM_KERNEL_GEMV)
    return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated: kernel: only the GEMV family has the gated form");
  if (desc->bits == 8) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated: no 8-bit form");
  if (!up_weights || !up_scales || (desc->affine && !up_biases)) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated: null up-projection buffer");
  if ((up_weights | up_scales | up_biases) & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated: up-projection buffers must be 16-byte aligned");
  MatmulArgs a = to_args(desc);
  a.up_weights = reinterpret_cast<const uint32_t*>(up_weights);
  a.up_scales = reinterpret_cast<const _Float16*>(up_scales);
  a.up_biases = reinterpret_cast<const _Float16*>(up_biases);
  if (!gemv_supports(a)) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated: K=%u does not fit the LDS staging of the activation row", a.K);
  const uint32_t M = a.slots ? 1 : a.M;
  const size_t out_elt = a.out_f32 ? 4 : 2;
  for (uint32_t m = 0; m < M; m++) {  // one pass over both matrices per activation row
    MatmulArgs r = a;
    r.in = a.in + (size_t)m * a.K;
    r.out = reinterpret_cast<char*>(a.out) + (size_t)m * a.N * out_elt;
    r.M = 1;
    HIP_TRY(ctx, launch_gemv(r, ctx->tune, ctx->stream));
  }
  return ZTVM_OK;
}

int ztvm_ffn_gated_prologue(ztvm_ctx* ctx, const ztvm_matmul_desc* desc, uint64_t up_weights, uint64_t up_scales, uint64_t up_biases,
                            uint64_t delta, uint64_t gamma, float rms_eps) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  char why[256];
  int rc = validate(desc, why, sizeof why, true);
  if (rc) return fail(ctx, rc, "ztvm_ffn_gated_prologue: %s", why);
  if (desc->kernel != ZTVM_KERNEL_AUTO && desc->kernel != ZTVM_KERNEL_GEMV)
    return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated_prologue: kernel: only the GEMV family has the gated form");
  if (desc->bits == 8) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated_prologue: no 8-bit form");
  if (desc->slots || desc->M != 1) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated_prologue: one dense activation row (the decode step) only");
  if (!up_weights || !up_scales || (desc->affine && !up_biases)) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated_prologue: null up-projection buffer");
  if ((up_weights | up_scales | up_biases) & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated_prologue: up-projection buffers must be 16-byte aligned");
  if (!delta || !gamma || ((delta | gamma) & 15u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated_prologue: delta and gamma must be given, 16-byte aligned");
  if (!(rms_eps >= 0.f)) return fail(ctx, ZTVM_E_INVALID, "ztvm_ffn_gated_prologue: rms_eps must be >= 0");
  MatmulArgs a = to_args(desc);
  a.up_weights = reinterpret_cast<const uint32_t*>(up_weights);
  a.up_scales = reinterpret_cast<const _Float16*>(up_scales);
  a.up_biases = reinterpret_cast<const _Float16*>(up_biases);
  a.delta = reinterpret_cast<const _Float16*>(delta);
  a.gamma = reinterpret_cast<const _Float16*>(gamma);
  a.rms_eps = rms_eps;
  if (!gemv_supports(a)) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_ffn_gated_prologue: K=%u does not fit the LDS staging of the activation row", a.K);
  HIP_TRY(ctx, launch_gemv(a, ctx->tune, ctx->stream));
  return ZTVM_OK;
}

// k_slot / v_slot non-zero: the int8-KV-mode variant, K and V go to two [kv_heads*head_dim] scratch rows
static int qkv_fused_common(ztvm_ctx* ctx, const ztvm_qkv_fused_desc* d, uint64_t k_slot, uint64_t v_slot) {
  const bool scratch = k_slot || v_slot;
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!d) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: null descriptor");
  if (d->bits != 4) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_qkv_fused: 4-bit rows only (got %u)", d->bits);
  if (d->affine > 1) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: affine must be 0 or 1");
  if (!d->heads || !d->kv_heads || !d->head_dim || (d->head_dim & 1u))
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: heads, kv_heads and an even head_dim are required");
  if (d->head_dim > 512u) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_qkv_fused: head_dim %u > 512", d->head_dim);
  if (!d->k_packed) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: K_PACKED must be > 0");
  const uint64_t K = (uint64_t)d->k_packed * 8u;
  const uint32_t G = d->affine ? 64u : 32u;
  if (K % G || d->scales_per_row != K / G || K > (1u << 24))
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: SCALES_PER_ROW=%u does not match K=%llu at group %u", d->scales_per_row, (unsigned long long)K, G);
  if ((uint64_t)(d->heads + 2u * d->kv_heads) * d->head_dim * d->k_packed * 4u >= (1ull << 31))
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: the fused weight matrix must stay under 2 GiB");
  if (scratch) {
    if (!k_slot || !v_slot || ((k_slot | v_slot) & 1u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused_scratch: k_slot and v_slot must both be given, 2-byte aligned");
  } else if (!d->page_size || !d->kv_page_stride || !d->head_page_stride) {
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: page_size, kv_page_stride and head_page_stride must be > 0");
  } else if ((uint64_t)d->page_size * d->head_dim > d->head_page_stride || (uint64_t)d->kv_heads * d->head_page_stride > d->v_page_offset ||
      (uint64_t)d->v_page_offset + (uint64_t)d->kv_heads * d->head_page_stride > d->kv_page_stride)
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: page layout overlaps (page_size*head_dim <= head_page_stride, kv_heads*head_page_stride <= v_page_offset, v_page_offset + kv_heads*head_page_stride <= kv_page_stride)");
  if (!(d->rope_theta > 0.f)) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: rope_theta must be > 0");
  if (!d->q_out || (!scratch && !d->kv_pages) || !d->hidden || !d->scales || !d->weights || !d->position_map)
    return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: null buffer");
  if (d->affine && !d->biases) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: affine rows have no bias buffer");
  if ((d->hidden | d->weights | d->scales | (d->affine ? d->biases : 0)) & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: hidden, weights, scales and biases must be 16-byte aligned");
  if (((d->q_out | d->kv_pages) & 1u) || (d->position_map & 3u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused: misaligned buffer");
  const uint32_t half = d->head_dim / 2;
  const uint64_t half_w = (uint64_t)half * d->k_packed * 4u, half_s = (uint64_t)half * d->scales_per_row * 2u;
  if ((half_w | half_s) & 15u)
    return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_qkv_fused: half a head of rows (%u) must be a multiple of 16 bytes of weights and of scales", half);
  QkvArgs q{};
  q.q_out = reinterpret_cast<_Float16*>(d->q_out);
  q.kv_pages = reinterpret_cast<_Float16*>(d->kv_pages);
  q.k_slot = reinterpret_cast<_Float16*>(k_slot);
  q.v_slot = reinterpret_cast<_Float16*>(v_slot);
  q.position_map = reinterpret_cast<const int32_t*>(d->position_map);
  q.heads = d->heads; q.kv_heads = d->kv_heads; q.head_dim = d->head_dim;
  q.page_size = d->page_size; q.kv_page_stride = d->kv_page_stride; q.head_page_stride = d->head_page_stride;
  q.v_page_offset = d->v_page_offset; q.position_map_elem_offset = d->position_map_elem_offset;
  q.pages_elem_offset = d->pages_elem_offset; q.kv_capacity = d->kv_capacity; q.rope_theta = d->rope_theta;
  MatmulArgs a{};
  a.in = reinterpret_cast<const _Float16*>(d->hidden);
  a.scales = reinterpret_cast<const _Float16*>(d->scales);
  a.weights = reinterpret_cast<const uint32_t*>(d->weights);
  a.biases = reinterpret_cast<const _Float16*>(d->biases);
  a.out = q.q_out;
  a.M = 1; a.N = (d->heads + 2u * d->kv_heads) * half;  // rotary pairs
  a.K = (uint32_t)K; a.k_packed = d->k_packed; a.spr = d->scales_per_row;
  a.bits = 4; a.affine = d->affine;
  // the pair's second row lives half a head further in the same matrix
  a.up_weights = a.weights + (size_t)half * d->k_packed;
  a.up_scales = a.scales + (size_t)half * d->scales_per_row;
  a.up_biases = d->affine ? a.biases + (size_t)half * d->scales_per_row : nullptr;
  a.qkv = &q;
  if (!gemv_supports(a)) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_qkv_fused: K=%llu does not fit the LDS staging of the activation row", (unsigned long long)K);
  HIP_TRY(ctx, launch_gemv(a, ctx->tune, ctx->stream));
  return ZTVM_OK;
}

int ztvm_qkv_fused(ztvm_ctx* ctx, const ztvm_qkv_fused_desc* d) { return qkv_fused_common(ctx, d, 0, 0); }

int ztvm_qkv_fused_scratch(ztvm_ctx* ctx, const ztvm_qkv_fused_desc* d, uint64_t k_slot, uint64_t v_slot) {
  if (!k_slot || !v_slot) return fail(ctx, ZTVM_E_INVALID, "ztvm_qkv_fused_scratch: null k_slot / v_slot");
  return qkv_fused_common(ctx, d, k_slot, v_slot);
}

int ztvm_kv_quantize_int8(ztvm_ctx* ctx, const ztvm_kv_quantize_desc* d) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!d) return fail(ctx, ZTVM_E_INVALID, "ztvm_kv_quantize_int8: null descriptor");
  if (!d->kv_heads || !d->head_dim || (d->head_dim & 3u) || !d->page_size)
    return fail(ctx, ZTVM_E_INVALID, "ztvm_kv_quantize_int8: kv_heads, page_size and a head_dim that is a multiple of 4 are required");
  if (d->head_dim > 1024u) return fail(ctx, ZTVM_E_UNSUPPORTED, "ztvm_kv_quantize_int8: head_dim %u > 1024", d->head_dim);
  if (!d->k_slot || !d->v_slot || !d->pages_i8 || !d->scales || !d->position_map) return fail(ctx, ZTVM_E_INVALID, "ztvm_kv_quantize_int8: null buffer");
  if (((d->k_slot | d->v_slot) & 7u) || (d->pages_i8 & 3u) || (d->scales & 1u) || (d->position_map & 3u))
    return fail(ctx, ZTVM_E_INVALID, "ztvm_kv_quantize_int8: misaligned buffer (slots 8, pages 4, scales 2, positions 4 bytes)");
  if (((uint64_t)d->kv_heads * d->head_dim) & 3u) return fail(ctx, ZTVM_E_INVALID, "ztvm_kv_quantize_int8: kv_heads*head_dim must be a multiple of 4");
  if (!d->tokens) return ZTVM_OK;
  HIP_TRY(ctx, launch_kv_quantize_int8(reinterpret_cast<void*>(d->pages_i8), reinterpret_cast<void*>(d->scales), reinterpret_cast<const void*>(d->k_slot),
                                       reinterpret_cast<const void*>(d->v_slot), reinterpret_cast<const int32_t*>(d->position_map), d->kv_heads,
                                       d->head_dim, d->page_size, d->tokens, d->position_map_elem_offset, d->pages_word_offset,
                                       d->scales_elem_offset, d->pages_capacity_words, d->scales_capacity, ctx->stream));
  return ZTVM_OK;
}

int ztvm_dequant(ztvm_ctx* ctx, const ztvm_matmul_desc* desc) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  char why[256];
  int rc = validate(desc, why, sizeof why, false);
  if (rc) return fail(ctx, rc, "ztvm_dequant: %s", why);
  if (desc->out & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_dequant: output must be 16-byte aligned");
  const MatmulArgs a = to_args(desc);
  HIP_TRY(ctx, launch_dequant(a, ctx->stream));
  return ZTVM_OK;
}

// ---- the dispatches either side of the matmuls in an FFN / MoE block ------------------

int ztvm_silu_mul(ztvm_ctx* ctx, uint64_t out, uint64_t gate_up, uint32_t rows, uint32_t ffn) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!out || !gate_up) return fail(ctx, ZTVM_E_INVALID, "ztvm_silu_mul: null buffer");
  if ((out | gate_up) & 1u) return fail(ctx, ZTVM_E_INVALID, "ztvm_silu_mul: buffers must be 2-byte aligned");
  if (!ffn) return fail(ctx, ZTVM_E_INVALID, "ztvm_silu_mul: ffn must be > 0");
  if (!rows) return ZTVM_OK;  // a zero-row chunk dispatches nothing
  HIP_TRY(ctx, launch_silu_mul(reinterpret_cast<void*>(out), reinterpret_cast<const void*>(gate_up), rows, ffn, ctx->stream));
  return ZTVM_OK;
}

int ztvm_moe_combine(ztvm_ctx* ctx, uint64_t out, uint64_t slots, uint64_t score, uint32_t tokens, uint32_t N, uint32_t SLOTS) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!out || !slots || !score) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_combine: null buffer");
  if (((out | slots) & 1u) || (score & 3u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_combine: misaligned buffer");
  if (!N || !SLOTS) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_combine: N and SLOTS must be > 0");
  if (tokens > 65535u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_combine: at most 65535 tokens per dispatch (got %u)", tokens);
  if (!tokens) return ZTVM_OK;
  HIP_TRY(ctx, launch_moe_combine(reinterpret_cast<void*>(out), reinterpret_cast<const void*>(slots),
                                  reinterpret_cast<const void*>(score), tokens, N, SLOTS, ctx->stream));
  return ZTVM_OK;
}

int ztvm_moe_router_logits(ztvm_ctx* ctx, uint64_t logits, uint64_t x, uint64_t w, uint64_t scales, uint64_t biases, uint32_t bits,
                           uint32_t D, uint32_t rows, uint32_t tokens) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (bits != 8 && bits != 4 && bits != 16) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: bits must be 8, 4 or 16 (got %u)", bits);
  if (!logits || !x || !w) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: null buffer");
  if (bits != 16 && (!scales || !biases)) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: a quantized router needs scales and biases");
  if ((x | w) & 15u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: x and w must be 16-byte aligned");
  if ((logits & 3u) || ((scales | biases) & 1u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: misaligned buffer");
  if (!D || !rows) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: D and rows must be > 0");
  if (bits == 16 ? D % 8u : D % 64u)
    return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: D=%u is not a multiple of %u", D, bits == 16 ? 8u : 64u);
  if (tokens > 65535u * 8u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_logits: too many tokens (%u)", tokens);
  if (!tokens) return ZTVM_OK;
  HIP_TRY(ctx, launch_router_logits(reinterpret_cast<void*>(logits), reinterpret_cast<const void*>(x), reinterpret_cast<const void*>(w),
                                    reinterpret_cast<const void*>(scales), reinterpret_cast<const void*>(biases), bits, D, rows,
                                    tokens, ctx->stream));
  return ZTVM_OK;
}

int ztvm_moe_router_topk(ztvm_ctx* ctx, uint64_t out_idx, uint64_t out_score, uint64_t logits, uint32_t E, uint32_t K,
                         uint32_t norm_topk, uint32_t has_shared, uint32_t tokens) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!out_idx || !out_score || !logits) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_topk: null buffer");
  if ((out_idx | out_score | logits) & 3u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_topk: buffers must be 4-byte aligned");
  if (!E || E > router_topk_max_experts())
    return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_topk: E must be 1..%u (got %u)", router_topk_max_experts(), E);
  if (!K || K > E || K > 64u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_topk: K must be 1..min(E, 64) (got K=%u, E=%u)", K, E);
  if (norm_topk > 1 || has_shared > 1) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_router_topk: normTopk/hasShared must be 0 or 1");
  if (!tokens) return ZTVM_OK;
  HIP_TRY(ctx, launch_router_topk(reinterpret_cast<void*>(out_idx), reinterpret_cast<void*>(out_score),
                                  reinterpret_cast<const void*>(logits), E, K, norm_topk, has_shared, tokens, ctx->stream));
  return ZTVM_OK;
}

int ztvm_moe_slot_translate(ztvm_ctx* ctx, uint64_t ids_out, uint64_t ids_in, uint64_t slot_map, uint32_t n, uint32_t map_len) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!ids_out || !ids_in || !slot_map) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_slot_translate: null buffer");
  if ((ids_out | ids_in | slot_map) & 3u) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_slot_translate: buffers must be 4-byte aligned");
  if (ids_out == ids_in) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_slot_translate: ids_in and ids_out must be separate buffers (the staging copy carries expert ids)");
  if (!map_len) return fail(ctx, ZTVM_E_INVALID, "ztvm_moe_slot_translate: empty slot map");
  if (!n) return ZTVM_OK;
  HIP_TRY(ctx, launch_slot_translate(reinterpret_cast<void*>(ids_out), reinterpret_cast<const void*>(ids_in),
                                     reinterpret_cast<const void*>(slot_map), n, map_len, ctx->stream));
  return ZTVM_OK;
}

// ---- load-time repack ---------------------------------------------------------------------

int ztvm_repack_part(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t src_bytes, int convert, uint64_t overflow) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (convert < ZTVM_CONVERT_RAW || convert > ZTVM_CONVERT_BF16_F32) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: unknown convert %d", convert);
  if (!dst || (!src && src_bytes)) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: null buffer");
  if (convert != ZTVM_CONVERT_RAW) {
    if (src_bytes & 1u) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: %zu bytes is not a whole number of bf16 values", src_bytes);
    if (src & 1u) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: bf16 source must be 2-byte aligned");
    if (dst & (convert == ZTVM_CONVERT_BF16_F32 ? 3u : 1u)) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: destination misaligned for its element type");
  }
  if (overflow & 3u) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_part: overflow counter must be 4-byte aligned");
  if (!src_bytes) return ZTVM_OK;
  HIP_TRY(ctx, launch_repack_convert(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src), src_bytes, convert,
                                     reinterpret_cast<uint32_t*>(overflow), ctx->stream));
  return ZTVM_OK;
}

int ztvm_repack_permute_rows(ztvm_ctx* ctx, uint64_t dst, uint64_t src, size_t bytes, uint32_t rows, const uint32_t* src_rows,
                             uint32_t src_len) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!dst || !src || !src_rows) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_permute_rows: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_permute_rows while recording a command buffer");
  if (src_len != rows) return fail(ctx, ZTVM_E_INVALID, "permuteRows has %u source indices for %u rows", src_len, rows);
  if (!rows || bytes % rows) return fail(ctx, ZTVM_E_INVALID, "%zu B does not divide into %u rows", bytes, rows);
  for (uint32_t j = 0; j < rows; j++)
    if (src_rows[j] >= rows) return fail(ctx, ZTVM_E_INVALID, "permuteRows src[%u] = %u is out of range", j, src_rows[j]);
  if ((dst < src + bytes) && (src < dst + bytes)) return fail(ctx, ZTVM_E_INVALID, "ztvm_repack_permute_rows: dst and src overlap");
  const size_t need = (size_t)rows * 4u;
  void* map = nullptr;
  int rc = scratch_for(ctx, need, &map);
  if (rc) return rc;
  HIP_TRY(ctx, hipMemcpyAsync(map, src_rows, need, hipMemcpyHostToDevice, ctx->stream));
  HIP_TRY(ctx, launch_permute_rows(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src),
                                   reinterpret_cast<const uint32_t*>(map), rows, bytes / rows, ctx->stream));
  HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // the map may be reused on return, and the scratch by the next dispatch
  return ZTVM_OK;
}

int ztvm_repack_dequant_split(ztvm_ctx* ctx, uint64_t dst, uint64_t weights, uint64_t scales, uint64_t biases, uint32_t k,
                              uint32_t heads, uint32_t nope, uint32_t v, uint64_t overflow) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (!dst || !weights || !scales || !biases) return fail(ctx, ZTVM_E_INVALID, "dequantAffineSplit needs exactly [weight, scales, biases]");
  if (!k || k % 64u) return fail(ctx, ZTVM_E_INVALID, "dequantAffineSplit: k=%u is not a multiple of the group size 64", k);
  if (!heads || !(nope + v)) return fail(ctx, ZTVM_E_INVALID, "dequantAffineSplit: empty shape");
  if ((uint64_t)heads * (nope + v) * (k / 8u) >= (1ull << 40)) return fail(ctx, ZTVM_E_INVALID, "dequantAffineSplit: shape too large");
  if ((dst & 15u) || (weights & 3u) || ((scales | biases) & 1u) || (overflow & 3u))
    return fail(ctx, ZTVM_E_INVALID, "dequantAffineSplit: misaligned buffer (dst 16, weights 4, scales/biases 2, counter 4 bytes)");
  HIP_TRY(ctx, launch_dequant_split(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(weights),
                                    reinterpret_cast<const void*>(scales), reinterpret_cast<const void*>(biases), k, heads, nope, v,
                                    reinterpret_cast<uint32_t*>(overflow), ctx->stream));
  return ZTVM_OK;
}

int ztvm_record_begin(ztvm_ctx* ctx) {
  if (!ctx) return fail(nullptr, ZTVM_E_INVALID, "null context");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "already recording");
  HIP_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
  ctx->recording = true;
  return ZTVM_OK;
}

int ztvm_record_end(ztvm_ctx* ctx, ztvm_cmdbuf** out) {
  if (!ctx || !out) return fail(ctx, ZTVM_E_INVALID, "ztvm_record_end: null argument");
  if (!ctx->recording) return fail(ctx, ZTVM_E_INVALID, "not recording");
  ctx->recording = false;
  ztvm_cmdbuf* cb = new ztvm_cmdbuf();
  hipError_t e = hipStreamEndCapture(ctx->stream, &cb->graph);
  if (e == hipSuccess) e = hipGraphInstantiate(&cb->exec, cb->graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    if (cb->graph) (void)hipGraphDestroy(cb->graph);
    delete cb;
    return fail(ctx, ZTVM_E_HIP, "command buffer finish: %s", hipGetErrorString(e));
  }
  cb->scratch = ctx->scratch;
  cb->scratch->pin();
  *out = cb;
  return ZTVM_OK;
}

int ztvm_submit(ztvm_ctx* ctx, ztvm_cmdbuf* cb) {
  if (!ctx || !cb || !cb->exec) return fail(ctx, ZTVM_E_INVALID, "ztvm_submit: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_submit while recording");
  HIP_TRY(ctx, hipGraphLaunch(cb->exec, ctx->stream));
  return ZTVM_OK;
}

void ztvm_cmdbuf_destroy(ztvm_cmdbuf* cb) {
  if (!cb) return;
  if (cb->exec) (void)hipGraphExecDestroy(cb->exec);
  if (cb->graph) (void)hipGraphDestroy(cb->graph);
  if (cb->scratch) cb->scratch->unpin();
  delete cb;
}

int ztvm_event_create(ztvm_ctx* ctx, ztvm_event** out) {
  if (!ctx || !out) return fail(ctx, ZTVM_E_INVALID, "ztvm_event_create: null argument");
  ztvm_event* e = new ztvm_event();
  hipError_t r = hipEventCreate(&e->ev);
  if (r != hipSuccess) {
    delete e;
    return fail(ctx, ZTVM_E_HIP, "hipEventCreate: %s", hipGetErrorString(r));
  }
  *out = e;
  return ZTVM_OK;
}

void ztvm_event_destroy(ztvm_event* ev) {
  if (!ev) return;
  if (ev->ev) (void)hipEventDestroy(ev->ev);
  delete ev;
}

int ztvm_event_record(ztvm_ctx* ctx, ztvm_event* ev) {
  if (!ctx || !ev) return fail(ctx, ZTVM_E_INVALID, "ztvm_event_record: null argument");
  if (ctx->recording) return fail(ctx, ZTVM_E_INVALID, "ztvm_event_record while recording");
  HIP_TRY(ctx, hipEventRecord(ev->ev, ctx->stream));
  return ZTVM_OK;
}

int ztvm_event_elapsed_ms(ztvm_ctx* ctx, ztvm_event* start, ztvm_event* stop, float* ms) {
  if (!ctx || !start || !stop || !ms) return fail(ctx, ZTVM_E_INVALID, "ztvm_event_elapsed_ms: null argument");
  HIP_TRY(ctx, hipEventSynchronize(stop->ev));
  HIP_TRY(ctx, hipEventElapsedTime(ms, start->ev, stop->ev));
  return ZTVM_OK;
}

int ztvm_set_option(ztvm_ctx* ctx, const char* name, int value) {
  if (!ctx || !name) return fail(ctx, ZTVM_E_INVALID, "ztvm_set_option: null argument");
  for (const Option& o : kOptions)
    if (!strcmp(o.name, name)) {
      if (!strcmp(name, "gemv.rows") && value != 0 && value != 1 && value != 2 && value != 4)
        return fail(ctx, ZTVM_E_INVALID, "gemv.rows must be 0 (default), 1, 2 or 4 (got %d)", value);
      if (!strcmp(name, "gemv.ring") && (value < 0 || value > 3))
        return fail(ctx, ZTVM_E_INVALID, "gemv.ring must be 0 (default), 1, 2 or 3 (got %d)", value);
      if (!strcmp(name, "num_cus") && (value < 1 || value > 4096))
        return fail(ctx, ZTVM_E_INVALID, "num_cus must be 1..4096 (got %d)", value);
      if (value < 0) return fail(ctx, ZTVM_E_INVALID, "option '%s' must be >= 0 (got %d)", name, value);
      ctx->tune.*(o.field) = value;
      return ZTVM_OK;
    }
  return fail(ctx, ZTVM_E_INVALID, "unknown option '%s'", name);
}

int ztvm_get_option(ztvm_ctx* ctx, const char* name, int* value) {
  if (!ctx || !name || !value) return fail(ctx, ZTVM_E_INVALID, "ztvm_get_option: null argument");
  for (const Option& o : kOptions)
    if (!strcmp(o.name, name)) {
      *value = ctx->tune.*(o.field);
      return ZTVM_OK;
    }
  return fail(ctx, ZTVM_E_INVALID, "unknown option '%s'", name);
}

}  // extern "C"
