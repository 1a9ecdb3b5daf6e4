// N-API addon: the thin JavaScript binding of the C ABI in include/ztvm.h.
// One exported function per C entry point; device addresses travel as BigInt,
// descriptors as plain objects whose keys are the ztvm_matmul_desc field names.
// Every failure becomes a JS exception carrying ztvm_last_error().
#include <node_api.h>

#include <cstdint>
#include <cstring>
#include <string>

#include "../../include/ztvm.h"

namespace {

#define NAPI_OK(env, call)                                                    \
  do {                                                                        \
    if ((call) != napi_ok) {                                                  \
      napi_throw_error(env, nullptr, "ztvm addon: N-API call failed: " #call); \
      return nullptr;                                                         \
    }                                                                         \
  } while (0)

napi_value throw_ztvm(napi_env env, ztvm_ctx* ctx, int code, const char* what) {
  std::string msg = std::string(what) + ": " + ztvm_last_error(ctx) + " (code " + std::to_string(code) + ")";
  napi_throw_error(env, code == ZTVM_E_INVALID ? "ZTVM_E_INVALID" : code == ZTVM_E_UNSUPPORTED ? "ZTVM_E_UNSUPPORTED"
                            : code == ZTVM_E_NODEVICE ? "ZTVM_E_NODEVICE" : "ZTVM_E_HIP", msg.c_str());
  return nullptr;
}

bool get_args(napi_env env, napi_callback_info info, size_t want, napi_value* argv) {
  size_t argc = want;
  if (napi_get_cb_info(env, info, &argc, argv, nullptr, nullptr) != napi_ok || argc < want) {
    napi_throw_type_error(env, nullptr, "ztvm addon: too few arguments");
    return false;
  }
  return true;
}

bool get_ptr(napi_env env, napi_value v, void** out) {
  if (napi_get_value_external(env, v, out) != napi_ok || !*out) {
    napi_throw_type_error(env, nullptr, "ztvm addon: expected a handle");
    return false;
  }
  return true;
}

bool get_u64(napi_env env, napi_value v, uint64_t* out) {
  napi_valuetype t;
  napi_typeof(env, v, &t);
  if (t == napi_bigint) {
    bool lossless = false;
    return napi_get_value_bigint_uint64(env, v, out, &lossless) == napi_ok;
  }
  if (t == napi_number) {
    double d = 0;
    napi_get_value_double(env, v, &d);
    *out = (uint64_t)d;
    return true;
  }
  if (t == napi_undefined || t == napi_null) {
    *out = 0;
    return true;
  }
  napi_throw_type_error(env, nullptr, "ztvm addon: expected a BigInt device address or a number");
  return false;
}

bool get_bytes(napi_env env, napi_value v, void** data, size_t* len) {
  bool is = false;
  if (napi_is_typedarray(env, v, &is) == napi_ok && is) {
    napi_typedarray_type tt;
    size_t n = 0, off = 0;
    napi_value ab;
    if (napi_get_typedarray_info(env, v, &tt, &n, data, &ab, &off) != napi_ok) return false;
    static const size_t esz[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
    *len = n * esz[tt];
    return true;
  }
  if (napi_is_arraybuffer(env, v, &is) == napi_ok && is) return napi_get_arraybuffer_info(env, v, data, len) == napi_ok;
  if (napi_is_buffer(env, v, &is) == napi_ok && is) return napi_get_buffer_info(env, v, data, len) == napi_ok;
  napi_throw_type_error(env, nullptr, "ztvm addon: expected a TypedArray, ArrayBuffer or Buffer");
  return false;
}

bool get_desc(napi_env env, napi_value obj, ztvm_matmul_desc* d) {
  memset(d, 0, sizeof *d);
  struct F32 { const char* name; uint32_t ztvm_matmul_desc::*field; };
  static const F32 u32s[] = {
      {"bits", &ztvm_matmul_desc::bits}, {"affine", &ztvm_matmul_desc::affine}, {"out_f32", &ztvm_matmul_desc::out_f32},
      {"kernel", &ztvm_matmul_desc::kernel}, {"M", &ztvm_matmul_desc::M}, {"N", &ztvm_matmul_desc::N},
      {"k_packed", &ztvm_matmul_desc::k_packed}, {"scales_per_row", &ztvm_matmul_desc::scales_per_row},
      {"slots", &ztvm_matmul_desc::slots}, {"tokens", &ztvm_matmul_desc::tokens},
      {"in_slot_stride", &ztvm_matmul_desc::in_slot_stride}, {"out_slot_stride", &ztvm_matmul_desc::out_slot_stride},
      {"in_tok_stride", &ztvm_matmul_desc::in_tok_stride}, {"out_tok_stride", &ztvm_matmul_desc::out_tok_stride},
      {"ids_stride", &ztvm_matmul_desc::ids_stride}, {"experts", &ztvm_matmul_desc::experts}};
  for (const F32& f : u32s) {
    napi_value v;
    bool has = false;
    napi_has_named_property(env, obj, f.name, &has);
    if (!has) continue;
    napi_get_named_property(env, obj, f.name, &v);
    uint32_t x = 0;
    napi_valuetype t;
    napi_typeof(env, v, &t);
    if (t == napi_boolean) {
      bool b = false;
      napi_get_value_bool(env, v, &b);
      x = b;
    } else if (napi_get_value_uint32(env, v, &x) != napi_ok) {
      napi_throw_type_error(env, nullptr, (std::string("ztvm addon: descriptor field '") + f.name + "' must be a number").c_str());
      return false;
    }
    d->*(f.field) = x;
  }
  struct F64 { const char* name; uint64_t ztvm_matmul_desc::*field; };
  static const F64 u64s[] = {{"out", &ztvm_matmul_desc::out}, {"in", &ztvm_matmul_desc::in}, {"scales", &ztvm_matmul_desc::scales},
                             {"weights", &ztvm_matmul_desc::weights}, {"biases", &ztvm_matmul_desc::biases}, {"ids", &ztvm_matmul_desc::ids}};
  for (const F64& f : u64s) {
    napi_value v;
    bool has = false;
    napi_has_named_property(env, obj, f.name, &has);
    if (!has) continue;
    napi_get_named_property(env, obj, f.name, &v);
    if (!get_u64(env, v, &(d->*(f.field)))) return false;
  }
  return true;
}

napi_value make_u64(napi_env env, uint64_t v) {
  napi_value r;
  napi_create_bigint_uint64(env, v, &r);
  return r;
}

napi_value undefined(napi_env env) {
  napi_value r;
  napi_get_undefined(env, &r);
  return r;
}

// ---- entry points ----------------------------------------------------------------------------

napi_value AbiVersion(napi_env env, napi_callback_info) {
  napi_value r;
  napi_create_int32(env, ztvm_abi_version(), &r);
  return r;
}

napi_value Create(napi_env env, napi_callback_info info) {
  napi_value a[1];
  if (!get_args(env, info, 1, a)) return nullptr;
  int32_t dev = 0;
  napi_get_value_int32(env, a[0], &dev);
  ztvm_ctx* ctx = nullptr;
  int rc = ztvm_create(dev, &ctx);
  if (rc) return throw_ztvm(env, nullptr, rc, "ztvm_create");
  napi_value r;
  NAPI_OK(env, napi_create_external(env, ctx, nullptr, nullptr, &r));
  return r;
}

napi_value Destroy(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* p;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &p)) return nullptr;
  ztvm_destroy((ztvm_ctx*)p);
  return undefined(env);
}

napi_value DeviceInfo(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* p;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &p)) return nullptr;
  char name[256];
  uint32_t cus = 0;
  uint64_t hbm = 0;
  int rc = ztvm_device_info((ztvm_ctx*)p, name, sizeof name, &cus, &hbm);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_device_info");
  napi_value o, v;
  napi_create_object(env, &o);
  napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &v);
  napi_set_named_property(env, o, "name", v);
  napi_create_uint32(env, cus, &v);
  napi_set_named_property(env, o, "computeUnits", v);
  napi_set_named_property(env, o, "hbmBytes", make_u64(env, hbm));
  return o;
}

napi_value Alloc(napi_env env, napi_callback_info info) {
  napi_value a[2];
  void* p;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p)) return nullptr;
  uint64_t n = 0, d = 0;
  if (!get_u64(env, a[1], &n)) return nullptr;
  int rc = ztvm_alloc((ztvm_ctx*)p, (size_t)n, &d);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_alloc");
  return make_u64(env, d);
}

napi_value Free(napi_env env, napi_callback_info info) {
  napi_value a[2];
  void* p;
  uint64_t d = 0;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &d)) return nullptr;
  int rc = ztvm_free((ztvm_ctx*)p, d);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_free");
  return undefined(env);
}

napi_value Upload(napi_env env, napi_callback_info info) {  // (ctx, dst, dstOffset, data)
  napi_value a[4];
  void *p, *data;
  uint64_t d = 0, off = 0;
  size_t len = 0;
  if (!get_args(env, info, 4, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &d) || !get_u64(env, a[2], &off) ||
      !get_bytes(env, a[3], &data, &len))
    return nullptr;
  int rc = ztvm_upload((ztvm_ctx*)p, d, (size_t)off, data, len);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_upload");
  return undefined(env);
}

napi_value Download(napi_env env, napi_callback_info info) {  // (ctx, src, srcOffset, bytes) -> ArrayBuffer
  napi_value a[4];
  void* p;
  uint64_t s = 0, off = 0, n = 0;
  if (!get_args(env, info, 4, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &s) || !get_u64(env, a[2], &off) ||
      !get_u64(env, a[3], &n))
    return nullptr;
  void* data = nullptr;
  napi_value ab;
  NAPI_OK(env, napi_create_arraybuffer(env, (size_t)n, &data, &ab));
  int rc = ztvm_download((ztvm_ctx*)p, data, s, (size_t)off, (size_t)n);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_download");
  return ab;
}

napi_value Fill(napi_env env, napi_callback_info info) {  // (ctx, dst, dstOffset, byte, bytes)
  napi_value a[5];
  void* p;
  uint64_t d = 0, off = 0, n = 0;
  int32_t byte = 0;
  if (!get_args(env, info, 5, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &d) || !get_u64(env, a[2], &off) ||
      !get_u64(env, a[4], &n))
    return nullptr;
  napi_get_value_int32(env, a[3], &byte);
  int rc = ztvm_fill((ztvm_ctx*)p, d, (size_t)off, byte, (size_t)n);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_fill");
  return undefined(env);
}

napi_value Copy(napi_env env, napi_callback_info info) {  // (ctx, dst, src, bytes)
  napi_value a[4];
  void* p;
  uint64_t d = 0, s = 0, n = 0;
  if (!get_args(env, info, 4, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &d) || !get_u64(env, a[2], &s) ||
      !get_u64(env, a[3], &n))
    return nullptr;
  int rc = ztvm_copy((ztvm_ctx*)p, d, s, (size_t)n);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_copy");
  return undefined(env);
}

napi_value Sync(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* p;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &p)) return nullptr;
  int rc = ztvm_sync((ztvm_ctx*)p);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_sync");
  return undefined(env);
}

napi_value Validate(napi_env env, napi_callback_info info) {  // (desc) -> {code, why}
  napi_value a[1];
  ztvm_matmul_desc d;
  if (!get_args(env, info, 1, a) || !get_desc(env, a[0], &d)) return nullptr;
  char why[512] = {0};
  int rc = ztvm_matmul_validate(&d, why, sizeof why);
  napi_value o, v;
  napi_create_object(env, &o);
  napi_create_int32(env, rc, &v);
  napi_set_named_property(env, o, "code", v);
  napi_create_string_utf8(env, why, NAPI_AUTO_LENGTH, &v);
  napi_set_named_property(env, o, "why", v);
  return o;
}

napi_value Resolve(napi_env env, napi_callback_info info) {  // (desc) -> family
  napi_value a[1];
  ztvm_matmul_desc d;
  if (!get_args(env, info, 1, a) || !get_desc(env, a[0], &d)) return nullptr;
  int rc = ztvm_matmul_resolve(&d);
  if (rc < 0) return throw_ztvm(env, nullptr, rc, "ztvm_matmul_resolve");
  napi_value v;
  napi_create_int32(env, rc, &v);
  return v;
}

napi_value Matmul(napi_env env, napi_callback_info info) {  // (ctx, desc)
  napi_value a[2];
  void* p;
  ztvm_matmul_desc d;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !get_desc(env, a[1], &d)) return nullptr;
  int rc = ztvm_matmul((ztvm_ctx*)p, &d);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_matmul");
  return undefined(env);
}

napi_value MatmulStatic(napi_env env, napi_callback_info info) {  // (ctx, desc): ztvm_matmul that allocates nothing
  napi_value a[2];
  void* p;
  ztvm_matmul_desc d;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !get_desc(env, a[1], &d)) return nullptr;
  int rc = ztvm_matmul_static((ztvm_ctx*)p, &d);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_matmul_static");
  return undefined(env);
}

napi_value ReadProbe(napi_env env, napi_callback_info info) {  // (ctx, src, bytes, sink)
  napi_value a[4];
  void* p;
  uint64_t s = 0, n = 0, k = 0;
  if (!get_args(env, info, 4, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &s) || !get_u64(env, a[2], &n) ||
      !get_u64(env, a[3], &k))
    return nullptr;
  int rc = ztvm_read_probe((ztvm_ctx*)p, s, (size_t)n, k);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_read_probe");
  return undefined(env);
}

napi_value Dequant(napi_env env, napi_callback_info info) {  // (ctx, desc)
  napi_value a[2];
  void* p;
  ztvm_matmul_desc d;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !get_desc(env, a[1], &d)) return nullptr;
  int rc = ztvm_dequant((ztvm_ctx*)p, &d);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_dequant");
  return undefined(env);
}

napi_value RecordBegin(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* p;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &p)) return nullptr;
  int rc = ztvm_record_begin((ztvm_ctx*)p);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_record_begin");
  return undefined(env);
}

napi_value RecordEnd(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* p;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &p)) return nullptr;
  ztvm_cmdbuf* cb = nullptr;
  int rc = ztvm_record_end((ztvm_ctx*)p, &cb);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_record_end");
  napi_value r;
  NAPI_OK(env, napi_create_external(env, cb, nullptr, nullptr, &r));
  return r;
}

napi_value Submit(napi_env env, napi_callback_info info) {
  napi_value a[2];
  void *p, *cb;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !get_ptr(env, a[1], &cb)) return nullptr;
  int rc = ztvm_submit((ztvm_ctx*)p, (ztvm_cmdbuf*)cb);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_submit");
  return undefined(env);
}

napi_value CmdbufDestroy(napi_env env, napi_callback_info info) {
  napi_value a[1];
  void* cb;
  if (!get_args(env, info, 1, a) || !get_ptr(env, a[0], &cb)) return nullptr;
  ztvm_cmdbuf_destroy((ztvm_cmdbuf*)cb);
  return undefined(env);
}

napi_value SetOption(napi_env env, napi_callback_info info) {  // (ctx, name, value)
  napi_value a[3];
  void* p;
  if (!get_args(env, info, 3, a) || !get_ptr(env, a[0], &p)) return nullptr;
  char name[128];
  size_t n = 0;
  napi_get_value_string_utf8(env, a[1], name, sizeof name, &n);
  int32_t v = 0;
  napi_get_value_int32(env, a[2], &v);
  int rc = ztvm_set_option((ztvm_ctx*)p, name, v);
  if (rc) return throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_set_option");
  return undefined(env);
}

// (ctx, NA device addresses, NB u32 values): the block dispatches all have this shape
template <size_t NA, size_t NB>
bool get_addr_u32(napi_env env, napi_callback_info info, void** ctx, uint64_t (&addr)[NA], uint32_t (&val)[NB]) {
  napi_value a[1 + NA + NB];
  if (!get_args(env, info, 1 + NA + NB, a) || !get_ptr(env, a[0], ctx)) return false;
  for (size_t i = 0; i < NA; i++)
    if (!get_u64(env, a[1 + i], &addr[i])) return false;
  for (size_t i = 0; i < NB; i++)
    if (napi_get_value_uint32(env, a[1 + NA + i], &val[i]) != napi_ok) {
      napi_throw_type_error(env, nullptr, "ztvm addon: expected a number");
      return false;
    }
  return true;
}

napi_value SiluMul(napi_env env, napi_callback_info info) {  // (ctx, out, gateUp, rows, ffn)
  void* p; uint64_t a[2]; uint32_t v[2];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_silu_mul((ztvm_ctx*)p, a[0], a[1], v[0], v[1]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_silu_mul") : undefined(env);
}

napi_value MoeCombine(napi_env env, napi_callback_info info) {  // (ctx, out, slots, score, tokens, N, SLOTS)
  void* p; uint64_t a[3]; uint32_t v[3];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_moe_combine((ztvm_ctx*)p, a[0], a[1], a[2], v[0], v[1], v[2]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_moe_combine") : undefined(env);
}

napi_value MoeRouterLogits(napi_env env, napi_callback_info info) {  // (ctx, logits, x, w, scales, biases, bits, D, rows, tokens)
  void* p; uint64_t a[5]; uint32_t v[4];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_moe_router_logits((ztvm_ctx*)p, a[0], a[1], a[2], a[3], a[4], v[0], v[1], v[2], v[3]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_moe_router_logits") : undefined(env);
}

napi_value MoeRouterTopk(napi_env env, napi_callback_info info) {  // (ctx, outIdx, outScore, logits, E, K, normTopk, hasShared, tokens)
  void* p; uint64_t a[3]; uint32_t v[5];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_moe_router_topk((ztvm_ctx*)p, a[0], a[1], a[2], v[0], v[1], v[2], v[3], v[4]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_moe_router_topk") : undefined(env);
}

napi_value MoeSlotTranslate(napi_env env, napi_callback_info info) {  // (ctx, idsOut, idsIn, slotMap, n, mapLen)
  void* p; uint64_t a[3]; uint32_t v[2];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_moe_slot_translate((ztvm_ctx*)p, a[0], a[1], a[2], v[0], v[1]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_moe_slot_translate") : undefined(env);
}

napi_value FfnGated(napi_env env, napi_callback_info info) {  // (ctx, desc, upWeights, upScales, upBiases)
  napi_value a[5];
  void* p;
  ztvm_matmul_desc d;
  uint64_t up[3];
  if (!get_args(env, info, 5, a) || !get_ptr(env, a[0], &p) || !get_desc(env, a[1], &d)) return nullptr;
  for (int i = 0; i < 3; i++)
    if (!get_u64(env, a[2 + i], &up[i])) return nullptr;
  int rc = ztvm_ffn_gated((ztvm_ctx*)p, &d, up[0], up[1], up[2]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_ffn_gated") : undefined(env);
}

napi_value FfnGatedPrologue(napi_env env, napi_callback_info info) {  // (ctx, desc, upWeights, upScales, upBiases, delta, gamma, rmsEps)
  napi_value a[8];
  void* p;
  ztvm_matmul_desc d;
  uint64_t v[5];
  double eps = 0;
  if (!get_args(env, info, 8, a) || !get_ptr(env, a[0], &p) || !get_desc(env, a[1], &d)) return nullptr;
  for (int i = 0; i < 5; i++)
    if (!get_u64(env, a[2 + i], &v[i])) return nullptr;
  if (napi_get_value_double(env, a[7], &eps) != napi_ok) {
    napi_throw_type_error(env, nullptr, "ztvm addon: rmsEps must be a number");
    return nullptr;
  }
  int rc = ztvm_ffn_gated_prologue((ztvm_ctx*)p, &d, v[0], v[1], v[2], v[3], v[4], (float)eps);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_ffn_gated_prologue") : undefined(env);
}

napi_value RepackPart(napi_env env, napi_callback_info info) {  // (ctx, dst, src, srcBytes, convert, overflow)
  napi_value a[6];
  void* p;
  uint64_t dst, src, bytes, over;
  int32_t conv = 0;
  if (!get_args(env, info, 6, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &dst) || !get_u64(env, a[2], &src) ||
      !get_u64(env, a[3], &bytes) || napi_get_value_int32(env, a[4], &conv) != napi_ok || !get_u64(env, a[5], &over))
    return nullptr;
  int rc = ztvm_repack_part((ztvm_ctx*)p, dst, src, (size_t)bytes, conv, over);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_repack_part") : undefined(env);
}

napi_value RepackPermuteRows(napi_env env, napi_callback_info info) {  // (ctx, dst, src, bytes, rows, Uint32Array srcRows)
  napi_value a[6];
  void *p, *map;
  uint64_t dst, src, bytes;
  uint32_t rows = 0;
  size_t len = 0;
  if (!get_args(env, info, 6, a) || !get_ptr(env, a[0], &p) || !get_u64(env, a[1], &dst) || !get_u64(env, a[2], &src) ||
      !get_u64(env, a[3], &bytes) || napi_get_value_uint32(env, a[4], &rows) != napi_ok || !get_bytes(env, a[5], &map, &len))
    return nullptr;
  int rc = ztvm_repack_permute_rows((ztvm_ctx*)p, dst, src, (size_t)bytes, rows, (const uint32_t*)map, (uint32_t)(len / 4));
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_repack_permute_rows") : undefined(env);
}

napi_value RepackDequantSplit(napi_env env, napi_callback_info info) {  // (ctx, dst, weights, scales, biases, overflow, k, heads, nope, v)
  void* p; uint64_t a[5]; uint32_t v[4];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  int rc = ztvm_repack_dequant_split((ztvm_ctx*)p, a[0], a[1], a[2], a[3], v[0], v[1], v[2], v[3], a[4]);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_repack_dequant_split") : undefined(env);
}

// a JS object whose keys are the ztvm_qkv_fused_desc field names -> the descriptor
bool read_qkv_desc(napi_env env, napi_value obj, ztvm_qkv_fused_desc& d) {
  napi_value a[2] = {nullptr, obj};
  memset(&d, 0, sizeof d);
  struct F32 { const char* name; uint32_t ztvm_qkv_fused_desc::*field; };
  static const F32 u32s[] = {
      {"bits", &ztvm_qkv_fused_desc::bits}, {"affine", &ztvm_qkv_fused_desc::affine}, {"k_packed", &ztvm_qkv_fused_desc::k_packed},
      {"scales_per_row", &ztvm_qkv_fused_desc::scales_per_row}, {"heads", &ztvm_qkv_fused_desc::heads},
      {"kv_heads", &ztvm_qkv_fused_desc::kv_heads}, {"head_dim", &ztvm_qkv_fused_desc::head_dim},
      {"page_size", &ztvm_qkv_fused_desc::page_size}, {"kv_page_stride", &ztvm_qkv_fused_desc::kv_page_stride},
      {"head_page_stride", &ztvm_qkv_fused_desc::head_page_stride}, {"v_page_offset", &ztvm_qkv_fused_desc::v_page_offset},
      {"position_map_elem_offset", &ztvm_qkv_fused_desc::position_map_elem_offset},
      {"pages_elem_offset", &ztvm_qkv_fused_desc::pages_elem_offset}};
  for (const F32& f : u32s) {
    napi_value v;
    bool has = false;
    napi_has_named_property(env, a[1], f.name, &has);
    if (!has) continue;
    napi_get_named_property(env, a[1], f.name, &v);
    if (napi_get_value_uint32(env, v, &(d.*(f.field))) != napi_ok) {
      napi_throw_type_error(env, nullptr, (std::string("ztvm addon: descriptor field '") + f.name + "' must be a number").c_str());
      return false;
    }
  }
  struct F64 { const char* name; uint64_t ztvm_qkv_fused_desc::*field; };
  static const F64 u64s[] = {{"kv_capacity", &ztvm_qkv_fused_desc::kv_capacity}, {"q_out", &ztvm_qkv_fused_desc::q_out},
                             {"kv_pages", &ztvm_qkv_fused_desc::kv_pages}, {"hidden", &ztvm_qkv_fused_desc::hidden},
                             {"scales", &ztvm_qkv_fused_desc::scales}, {"weights", &ztvm_qkv_fused_desc::weights},
                             {"position_map", &ztvm_qkv_fused_desc::position_map}, {"biases", &ztvm_qkv_fused_desc::biases}};
  for (const F64& f : u64s) {
    napi_value v;
    bool has = false;
    napi_has_named_property(env, a[1], f.name, &has);
    if (!has) continue;
    napi_get_named_property(env, a[1], f.name, &v);
    if (!get_u64(env, v, &(d.*(f.field)))) return false;
  }
  napi_value v;
  bool has = false;
  napi_has_named_property(env, a[1], "rope_theta", &has);
  if (has) {
    double t = 0;
    napi_get_named_property(env, a[1], "rope_theta", &v);
    napi_get_value_double(env, v, &t);
    d.rope_theta = (float)t;
  }
  return true;
}

napi_value QkvFused(napi_env env, napi_callback_info info) {  // (ctx, desc)
  napi_value a[2];
  void* p;
  ztvm_qkv_fused_desc d;
  if (!get_args(env, info, 2, a) || !get_ptr(env, a[0], &p) || !read_qkv_desc(env, a[1], d)) return nullptr;
  int rc = ztvm_qkv_fused((ztvm_ctx*)p, &d);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_qkv_fused") : undefined(env);
}

napi_value QkvFusedScratch(napi_env env, napi_callback_info info) {  // (ctx, desc, kSlot, vSlot)
  napi_value a[4];
  void* p;
  uint64_t ks, vs;
  ztvm_qkv_fused_desc d;
  if (!get_args(env, info, 4, a) || !get_ptr(env, a[0], &p) || !read_qkv_desc(env, a[1], d) || !get_u64(env, a[2], &ks) ||
      !get_u64(env, a[3], &vs))
    return nullptr;
  int rc = ztvm_qkv_fused_scratch((ztvm_ctx*)p, &d, ks, vs);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_qkv_fused_scratch") : undefined(env);
}

// (ctx, pagesI8, scales, kSlot, vSlot, positionMap, pagesCapacityWords, scalesCapacity,
//  kvHeads, headDim, pageSize, tokens, positionMapElemOffset, pagesWordOffset, scalesElemOffset)
napi_value KvQuantizeInt8(napi_env env, napi_callback_info info) {
  void* p; uint64_t a[7]; uint32_t v[7];
  if (!get_addr_u32(env, info, &p, a, v)) return nullptr;
  ztvm_kv_quantize_desc d;
  memset(&d, 0, sizeof d);
  d.pages_i8 = a[0]; d.scales = a[1]; d.k_slot = a[2]; d.v_slot = a[3]; d.position_map = a[4];
  d.pages_capacity_words = a[5]; d.scales_capacity = a[6];
  d.kv_heads = v[0]; d.head_dim = v[1]; d.page_size = v[2]; d.tokens = v[3];
  d.position_map_elem_offset = v[4]; d.pages_word_offset = v[5]; d.scales_elem_offset = v[6];
  int rc = ztvm_kv_quantize_int8((ztvm_ctx*)p, &d);
  return rc ? throw_ztvm(env, (ztvm_ctx*)p, rc, "ztvm_kv_quantize_int8") : undefined(env);
}

napi_value Init(napi_env env, napi_value exports) {
  struct E { const char* name; napi_callback fn; };
  static const E table[] = {
      {"abiVersion", AbiVersion}, {"create", Create}, {"destroy", Destroy}, {"deviceInfo", DeviceInfo}, {"alloc", Alloc},
      {"free", Free}, {"upload", Upload}, {"download", Download}, {"fill", Fill}, {"copy", Copy}, {"sync", Sync},
      {"validate", Validate}, {"resolve", Resolve}, {"matmul", Matmul}, {"matmulStatic", MatmulStatic}, {"readProbe", ReadProbe}, {"dequant", Dequant}, {"recordBegin", RecordBegin},
      {"recordEnd", RecordEnd}, {"submit", Submit}, {"cmdbufDestroy", CmdbufDestroy}, {"setOption", SetOption},
      {"siluMul", SiluMul}, {"moeCombine", MoeCombine}, {"moeRouterLogits", MoeRouterLogits}, {"moeRouterTopk", MoeRouterTopk},
      {"moeSlotTranslate", MoeSlotTranslate}, {"ffnGated", FfnGated}, {"ffnGatedPrologue", FfnGatedPrologue}, {"repackPart", RepackPart},
      {"repackPermuteRows", RepackPermuteRows}, {"repackDequantSplit", RepackDequantSplit}, {"qkvFused", QkvFused},
      {"qkvFusedScratch", QkvFusedScratch}, {"kvQuantizeInt8", KvQuantizeInt8}};
  for (const E& e : table) {
    napi_value fn;
    if (napi_create_function(env, e.name, NAPI_AUTO_LENGTH, e.fn, nullptr, &fn) != napi_ok) return nullptr;
    napi_set_named_property(env, exports, e.name, fn);
  }
  return exports;
}

}  // namespace

NAPI_MODULE(NODE_GYP_MODULE_NAME, Init)
