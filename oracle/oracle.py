"""ctypes wrapper over the CPU oracle (oracle/ztvm_oracle.c).

Test infrastructure only: imported by tests/, the smoke check and the
bench's cpu_baseline leg. Nothing in the product package imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libztvm_oracle.so")

MODE_JS, MODE_FORMULA_F64, MODE_FORMULA_F32, MODE_F16W = 0, 1, 2, 3


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        u16p, u32p, f32p, f64p, u8p = (C.POINTER(t) for t in (C.c_uint16, C.c_uint32, C.c_float, C.c_double, C.c_uint8))
        L.zo_f32_to_f16.restype, L.zo_f32_to_f16.argtypes = C.c_uint16, [C.c_float]
        L.zo_f16_to_f32.restype, L.zo_f16_to_f32.argtypes = C.c_float, [C.c_uint16]
        L.zo_f32_to_f16_array.argtypes = [f32p, u16p, C.c_size_t]
        L.zo_f16_to_f32_array.argtypes = [u16p, f32p, C.c_size_t]
        L.zo_mulberry32.restype, L.zo_mulberry32.argtypes = C.c_double, [u32p]
        L.zo_reference_gemv_case.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_int, u16p, u16p, u16p, u32p]
        for f in (L.zo_unpack4, L.zo_unpack3, L.zo_unpack3_window, L.zo_unpack8):
            f.restype, f.argtypes = C.c_uint32, [u32p, C.c_uint32]
        L.zo_pack3.argtypes = [u8p, C.c_uint32, u32p]
        L.zo_pack4.argtypes = [u8p, C.c_uint32, u32p]
        L.zo_pack8.argtypes = [u8p, C.c_uint32, u32p]
        L.zo_dequant_f32.restype = C.c_float
        L.zo_dequant_f32.argtypes = [C.c_uint32, C.c_uint16, C.c_uint16, C.c_int]
        L.zo_dequant_f16.restype = C.c_uint16
        L.zo_dequant_f16.argtypes = [C.c_uint32, C.c_uint16, C.c_uint16, C.c_int]
        L.zo_dequant_matrix.argtypes = [C.c_uint32, C.c_int, C.c_uint32, C.c_uint32, u32p, u16p, u16p, f32p, u16p]
        L.zo_gemm.argtypes = [C.c_int, C.c_uint32, C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, u16p, C.c_uint32,
                              u32p, u16p, u16p, f64p, C.c_int]
        L.zo_moe_gemv.argtypes = [C.c_int, C.c_uint32] + [C.c_uint32] * 9 + [u32p, u16p, u32p, u16p, u16p, f64p, C.c_int]
        L.zo_max_threads.restype = C.c_int
        L.zo_bf16_to_f16.restype, L.zo_bf16_to_f16.argtypes = C.c_uint64, [u16p, u16p, C.c_size_t]
        L.zo_bf16_to_f32.restype, L.zo_bf16_to_f32.argtypes = None, [u16p, u32p, C.c_size_t]
        L.zo_permute_rows.argtypes = [u8p, u8p, C.c_size_t, C.c_uint32, u32p, C.c_uint32]
        L.zo_deint.restype, L.zo_deint.argtypes = C.c_uint32, [C.c_uint32, C.c_uint32]
        L.zo_dequant_affine_split.restype = C.c_uint64
        L.zo_dequant_affine_split.argtypes = [u32p, u16p, u16p] + [C.c_uint32] * 4 + [u16p]
        L.zo_silu_mul.restype, L.zo_silu_mul.argtypes = None, [u16p, C.c_uint32, C.c_uint32, f64p, u16p]
        L.zo_moe_combine.restype = None
        L.zo_moe_combine.argtypes = [u16p, f32p, C.c_uint32, C.c_uint32, C.c_uint32, f64p, u16p]
        L.zo_router_logits.restype = None
        L.zo_router_logits.argtypes = [C.c_uint32] * 4 + [u16p, C.c_void_p, u16p, u16p, f64p]
        L.zo_router_topk.restype = None
        L.zo_router_topk.argtypes = [f32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_int, u32p, f64p]
        L.zo_slot_translate.restype, L.zo_slot_translate.argtypes = None, [u32p, u32p, C.c_uint32, u32p]
        L.zo_qkv_fused.restype = None
        L.zo_qkv_fused.argtypes = [C.c_uint32] * 10 + [C.c_double, C.c_int32, u16p, u32p, u16p, u16p, u16p, u16p]
        L.zo_add_rmsnorm.restype, L.zo_add_rmsnorm.argtypes = None, [u16p, u16p, u16p, C.c_uint32, C.c_float, u16p]
        L.zo_kv_quantize_int8.restype = None
        L.zo_kv_quantize_int8.argtypes = [C.c_uint32] * 4 + [C.POINTER(C.c_int32), C.c_uint32, C.c_uint32, u16p, u16p, u32p, u16p]
        _lib = L
    return _lib


def _p(a, ct):
    return None if a is None else a.ctypes.data_as(C.POINTER(ct))


def _c(a, dt):
    return None if a is None else np.ascontiguousarray(a, dtype=dt)


def f32_to_f16_bits(x):
    x = _c(x, np.float32).ravel()
    out = np.empty(x.size, np.uint16)
    lib().zo_f32_to_f16_array(_p(x, C.c_float), _p(out, C.c_uint16), x.size)
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16).ravel()
    out = np.empty(h.size, np.float32)
    lib().zo_f16_to_f32_array(_p(h, C.c_uint16), _p(out, C.c_float), h.size)
    return out


def mulberry32(seed, n):
    st = C.c_uint32(seed & 0xFFFFFFFF)
    L = lib()
    return np.array([L.zo_mulberry32(C.byref(st)) for _ in range(n)], np.float64)


def reference_gemv_case(N, K, affine, q3, seed=1):
    """The seeded vector of the reference's own GEMV kernel test."""
    KP = K * 3 // 32 if q3 else K // 8
    SPR = K // (64 if affine else 32)
    x = np.empty(K, np.uint16)
    s = np.empty(N * SPR, np.uint16)
    b = np.zeros(N * SPR, np.uint16)
    w = np.empty(N * KP, np.uint32)
    lib().zo_reference_gemv_case(seed, N, K, int(affine), int(q3), _p(x, C.c_uint16), _p(s, C.c_uint16),
                                 _p(b, C.c_uint16), _p(w, C.c_uint32))
    return x, s.reshape(N, SPR), (b.reshape(N, SPR) if affine else None), w.reshape(N, KP)


def unpack(bits, row_words, k, window=False):
    row = _c(row_words, np.uint32)
    f = lib().zo_unpack4 if bits == 4 else lib().zo_unpack8 if bits == 8 else (lib().zo_unpack3_window if window else lib().zo_unpack3)
    return f(_p(row, C.c_uint32), k)


def pack(bits, values):
    v = _c(values, np.uint8).ravel()
    K = v.size
    out = np.zeros(K * bits // 32, np.uint32)
    (lib().zo_pack3 if bits == 3 else lib().zo_pack8 if bits == 8 else lib().zo_pack4)(_p(v, C.c_uint8), K, _p(out, C.c_uint32))
    return out


def dequant_scalar(q, s16, b16, affine, f16=False):
    L = lib()
    return (L.zo_dequant_f16 if f16 else L.zo_dequant_f32)(int(q), int(s16), int(b16), int(affine))


def dequant_matrix(bits, affine, N, K, weights, scales, biases, want="f32"):
    w, s, b = _c(weights, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    o32 = np.empty((N, K), np.float32) if want in ("f32", "both") else None
    o16 = np.empty((N, K), np.uint16) if want in ("f16", "both") else None
    lib().zo_dequant_matrix(bits, int(affine), N, K, _p(w, C.c_uint32), _p(s, C.c_uint16), _p(b, C.c_uint16),
                            _p(o32, C.c_float), _p(o16, C.c_uint16))
    return (o32, o16) if want == "both" else (o32 if o32 is not None else o16)


def gemm(mode, bits, affine, M, N, K, A, weights, scales, biases, lda=None, threads=1):
    """Y[M,N] float64, unrounded. A is f16 bit patterns."""
    A, w, s, b = _c(A, np.uint16), _c(weights, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    Y = np.empty((M, N), np.float64)
    lib().zo_gemm(mode, bits, int(affine), M, N, K, _p(A, C.c_uint16), lda or K, _p(w, C.c_uint32),
                  _p(s, C.c_uint16), _p(b, C.c_uint16), _p(Y, C.c_double), threads)
    return Y


def moe_gemv(mode, bits, N, K, tokens, slots, strides, ids, x, weights, scales, biases, out_elems, threads=1):
    """strides = (in_slot, out_slot, in_tok, out_tok, ids_stride); returns float64[out_elems] (zeros where unwritten)."""
    ids, x = _c(ids, np.uint32), _c(x, np.uint16)
    w, s, b = _c(weights, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    out = np.zeros(out_elems, np.float64)
    lib().zo_moe_gemv(mode, bits, N, K, tokens, slots, *[int(v) for v in strides], _p(ids, C.c_uint32),
                      _p(x, C.c_uint16), _p(w, C.c_uint32), _p(s, C.c_uint16), _p(b, C.c_uint16),
                      _p(out, C.c_double), threads)
    return out


def max_threads():
    return lib().zo_max_threads()


# ---- loader conversions and the dispatches around the matmuls of a MoE block ----

def bf16_to_f16(src):
    """(f16 bit patterns, overflow count)"""
    src = _c(src, np.uint16).ravel()
    out = np.empty(src.size, np.uint16)
    n = lib().zo_bf16_to_f16(_p(src, C.c_uint16), _p(out, C.c_uint16), src.size)
    return out, int(n)


def bf16_to_f32(src):
    src = _c(src, np.uint16).ravel()
    out = np.empty(src.size, np.uint32)
    lib().zo_bf16_to_f32(_p(src, C.c_uint16), _p(out, C.c_uint32), src.size)
    return out.view(np.float32)


def permute_rows(data, rows, src):
    """bytes in, bytes out; raises ValueError where the reference throws."""
    data = np.ascontiguousarray(data).view(np.uint8).ravel()
    src = _c(src, np.uint32).ravel()
    out = np.empty_like(data)
    if lib().zo_permute_rows(_p(data, C.c_uint8), _p(out, C.c_uint8), data.size, rows, _p(src, C.c_uint32), src.size):
        raise ValueError("permuteRows: bad map, row count or index")
    return out


def deint(j, R):
    return lib().zo_deint(j, R)


def dequant_affine_split(weights, scales, biases, k, heads, nope, v):
    """(f16 bit patterns [heads*k*nope + heads*v*k], overflow count)"""
    w, s, b = _c(weights, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    out = np.empty(heads * (nope + v) * k, np.uint16)
    n = lib().zo_dequant_affine_split(_p(w, C.c_uint32), _p(s, C.c_uint16), _p(b, C.c_uint16), k, heads, nope, v,
                                      _p(out, C.c_uint16))
    return out, int(n)


def silu_mul(gate_up, rows, ffn):
    """(float64 unrounded [rows, ffn], f16 bit patterns of the float32 form)"""
    gu = _c(gate_up, np.uint16)
    o64, o16 = np.empty((rows, ffn), np.float64), np.empty((rows, ffn), np.uint16)
    lib().zo_silu_mul(_p(gu, C.c_uint16), rows, ffn, _p(o64, C.c_double), _p(o16, C.c_uint16))
    return o64, o16


def moe_combine(slots, score, tokens, N, S):
    sl, sc = _c(slots, np.uint16), _c(score, np.float32)
    o64, o16 = np.empty((tokens, N), np.float64), np.empty((tokens, N), np.uint16)
    lib().zo_moe_combine(_p(sl, C.c_uint16), _p(sc, C.c_float), tokens, N, S, _p(o64, C.c_double), _p(o16, C.c_uint16))
    return o64, o16


def router_logits(bits, D, rows, tokens, x, w, scales=None, biases=None):
    x = _c(x, np.uint16)
    w = _c(w, np.uint16 if bits == 16 else np.uint32)
    s, b = _c(scales, np.uint16), _c(biases, np.uint16)
    out = np.empty((tokens, rows), np.float64)
    lib().zo_router_logits(bits, D, rows, tokens, _p(x, C.c_uint16), w.ctypes.data_as(C.c_void_p), _p(s, C.c_uint16),
                           _p(b, C.c_uint16), _p(out, C.c_double))
    return out


def router_topk(logits, tokens, E, K, norm_topk, has_shared):
    """(indices [tokens, K+has_shared] u32, scores float64)"""
    lg = _c(logits, np.float32)
    n = K + (1 if has_shared else 0)
    idx, sc = np.empty((tokens, n), np.uint32), np.empty((tokens, n), np.float64)
    lib().zo_router_topk(_p(lg, C.c_float), tokens, E, K, int(norm_topk), int(has_shared), _p(idx, C.c_uint32),
                         _p(sc, C.c_double))
    return idx, sc


def slot_translate(ids, slot_map):
    ids, m = _c(ids, np.uint32).ravel(), _c(slot_map, np.uint32).ravel()
    out = np.empty_like(ids)
    lib().zo_slot_translate(_p(ids, C.c_uint32), _p(m, C.c_uint32), ids.size, _p(out, C.c_uint32))
    return out


def add_rmsnorm(residual, delta, gamma, eps):
    """f16 bits of RMSNorm(residual + delta) * gamma, the fused-FFN prologue's numerics"""
    r, d, g = _c(residual, np.uint16).ravel(), _c(delta, np.uint16).ravel(), _c(gamma, np.uint16).ravel()
    out = np.empty_like(r)
    lib().zo_add_rmsnorm(_p(r, C.c_uint16), _p(d, C.c_uint16), _p(g, C.c_uint16), r.size, C.c_float(eps), _p(out, C.c_uint16))
    return out


def kv_quantize_int8(kv_heads, head_dim, page_size, positions, pages_word_offset, scales_elem_offset, k_slot, v_slot, pages, scales):
    """(pages u32, scales f16 bits) with every token's int8 rows and scales written in"""
    pos = _c(positions, np.int32).ravel()
    k, v = _c(k_slot, np.uint16).ravel(), _c(v_slot, np.uint16).ravel()
    pg, sc = np.array(pages, np.uint32, copy=True).ravel(), np.array(scales, np.uint16, copy=True).ravel()
    lib().zo_kv_quantize_int8(kv_heads, head_dim, page_size, pos.size, _p(pos, C.c_int32), pages_word_offset, scales_elem_offset,
                              _p(k, C.c_uint16), _p(v, C.c_uint16), _p(pg, C.c_uint32), _p(sc, C.c_uint16))
    return pg, sc


def qkv_fused(affine, K, heads, kv_heads, head_dim, page_size, kv_page_stride, head_page_stride, v_page_offset,
              pages_elem_offset, theta, position, hidden, weights, scales, biases, pages):
    """(q_out f16 bits [heads*head_dim], pages f16 bits with the token's K and V written in)"""
    h, w, s, b = _c(hidden, np.uint16), _c(weights, np.uint32), _c(scales, np.uint16), _c(biases, np.uint16)
    q_out = np.zeros(heads * head_dim, np.uint16)
    pg = np.array(pages, np.uint16, copy=True)
    lib().zo_qkv_fused(int(affine), K, heads, kv_heads, head_dim, page_size, kv_page_stride, head_page_stride, v_page_offset,
                       pages_elem_offset, float(theta), int(position), _p(h, C.c_uint16), _p(w, C.c_uint32),
                       _p(s, C.c_uint16), _p(b, C.c_uint16), _p(q_out, C.c_uint16), _p(pg, C.c_uint16))
    return q_out, pg
