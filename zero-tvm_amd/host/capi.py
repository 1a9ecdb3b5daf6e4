"""ctypes binding of libztvm_hip.so (the C ABI declared in include/ztvm.h).

There is no fallback: if the shared library is missing or a call fails, an
exception is raised. Device memory is named by integer device addresses.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, "lib", "libztvm_hip.so")

KERNEL_AUTO, KERNEL_GEMV, KERNEL_SKINNY, KERNEL_GEMM, KERNEL_ROWS = 0, 1, 2, 3, 4
KERNEL_NAMES = {0: "auto", 1: "gemv", 2: "skinny", 3: "gemm", 4: "rows"}
E_INVALID, E_HIP, E_UNSUPPORTED, E_NODEVICE = -1, -2, -3, -4

EXPORTS = [
    "ztvm_abi_version", "ztvm_last_error", "ztvm_create", "ztvm_destroy", "ztvm_device_info",
    "ztvm_alloc", "ztvm_free", "ztvm_upload", "ztvm_download", "ztvm_fill", "ztvm_copy", "ztvm_read_probe", "ztvm_sync",
    "ztvm_matmul_validate", "ztvm_matmul_resolve", "ztvm_matmul", "ztvm_matmul_static", "ztvm_ffn_gated", "ztvm_ffn_gated_prologue", "ztvm_qkv_fused", "ztvm_qkv_fused_scratch",
    "ztvm_kv_quantize_int8", "ztvm_dequant",
    "ztvm_record_begin", "ztvm_record_end", "ztvm_submit", "ztvm_cmdbuf_destroy",
    "ztvm_event_create", "ztvm_event_destroy", "ztvm_event_record", "ztvm_event_elapsed_ms",
    "ztvm_set_option", "ztvm_get_option",
    "ztvm_silu_mul", "ztvm_moe_combine", "ztvm_moe_router_logits", "ztvm_moe_router_topk", "ztvm_moe_slot_translate",
    "ztvm_repack_part", "ztvm_repack_permute_rows", "ztvm_repack_dequant_split",
]
CONVERT_RAW, CONVERT_BF16_F16, CONVERT_BF16_F32 = 0, 1, 2
EXPERTS_UNCHECKED = 0xFFFFFFFF  # ztvm_matmul_desc.experts: the caller vouches for every id


class ZtvmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("ztvm error %d: %s" % (code, msg))
        self.code = code
        self.reason = msg


class MatmulDesc(C.Structure):
    """Mirror of ztvm_matmul_desc."""
    _fields_ = [(n, C.c_uint32) for n in (
        "bits", "affine", "out_f32", "kernel", "M", "N", "k_packed", "scales_per_row", "slots", "tokens",
        "in_slot_stride", "out_slot_stride", "in_tok_stride", "out_tok_stride", "ids_stride", "experts")] + [
        (n, C.c_uint64) for n in ("out", "in_", "scales", "weights", "biases", "ids")]


class QkvFusedDesc(C.Structure):
    """Mirror of ztvm_qkv_fused_desc."""
    _fields_ = [(n, C.c_uint32) for n in (
        "bits", "affine", "k_packed", "scales_per_row", "heads", "kv_heads", "head_dim", "page_size", "kv_page_stride",
        "head_page_stride", "v_page_offset", "position_map_elem_offset", "pages_elem_offset")] + [
        ("rope_theta", C.c_float), ("kv_capacity", C.c_uint64)] + [
        (n, C.c_uint64) for n in ("q_out", "kv_pages", "hidden", "scales", "weights", "position_map", "biases")]


class KvQuantizeDesc(C.Structure):
    """Mirror of ztvm_kv_quantize_desc."""
    _fields_ = [(n, C.c_uint32) for n in (
        "kv_heads", "head_dim", "page_size", "tokens", "position_map_elem_offset", "pages_word_offset", "scales_elem_offset",
        "reserved")] + [(n, C.c_uint64) for n in (
            "pages_capacity_words", "scales_capacity", "k_slot", "v_slot", "pages_i8", "scales", "position_map")]


_lib = None


def load():
    """Load the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ZtvmError(E_NODEVICE, "libztvm_hip.so is not built (%s); run `python zero-tvm_amd/build.py`" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, u64p = C.c_void_p, C.POINTER(C.c_uint64)
    L.ztvm_abi_version.restype = C.c_int
    L.ztvm_last_error.restype, L.ztvm_last_error.argtypes = C.c_char_p, [vp]
    L.ztvm_create.argtypes = [C.c_int, C.POINTER(vp)]
    L.ztvm_destroy.restype, L.ztvm_destroy.argtypes = None, [vp]
    L.ztvm_device_info.argtypes = [vp, C.c_char_p, C.c_size_t, C.POINTER(C.c_uint32), u64p]
    L.ztvm_alloc.argtypes = [vp, C.c_size_t, u64p]
    L.ztvm_free.argtypes = [vp, C.c_uint64]
    L.ztvm_upload.argtypes = [vp, C.c_uint64, C.c_size_t, vp, C.c_size_t]
    L.ztvm_download.argtypes = [vp, vp, C.c_uint64, C.c_size_t, C.c_size_t]
    L.ztvm_fill.argtypes = [vp, C.c_uint64, C.c_size_t, C.c_int, C.c_size_t]
    L.ztvm_copy.argtypes = [vp, C.c_uint64, C.c_uint64, C.c_size_t]
    L.ztvm_read_probe.argtypes = [vp, C.c_uint64, C.c_size_t, C.c_uint64]
    L.ztvm_sync.argtypes = [vp]
    L.ztvm_matmul_validate.argtypes = [C.POINTER(MatmulDesc), C.c_char_p, C.c_size_t]
    L.ztvm_matmul_resolve.argtypes = [C.POINTER(MatmulDesc)]
    L.ztvm_matmul.argtypes = [vp, C.POINTER(MatmulDesc)]
    L.ztvm_matmul_static.argtypes = [vp, C.POINTER(MatmulDesc)]
    L.ztvm_dequant.argtypes = [vp, C.POINTER(MatmulDesc)]
    L.ztvm_record_begin.argtypes = [vp]
    L.ztvm_record_end.argtypes = [vp, C.POINTER(vp)]
    L.ztvm_submit.argtypes = [vp, vp]
    L.ztvm_cmdbuf_destroy.restype, L.ztvm_cmdbuf_destroy.argtypes = None, [vp]
    L.ztvm_event_create.argtypes = [vp, C.POINTER(vp)]
    L.ztvm_event_destroy.restype, L.ztvm_event_destroy.argtypes = None, [vp]
    L.ztvm_event_record.argtypes = [vp, vp]
    L.ztvm_event_elapsed_ms.argtypes = [vp, vp, vp, C.POINTER(C.c_float)]
    L.ztvm_set_option.argtypes = [vp, C.c_char_p, C.c_int]
    L.ztvm_get_option.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int)]
    u32, u64 = C.c_uint32, C.c_uint64
    L.ztvm_ffn_gated.argtypes = [vp, C.POINTER(MatmulDesc), u64, u64, u64]
    L.ztvm_ffn_gated_prologue.argtypes = [vp, C.POINTER(MatmulDesc)] + [C.c_uint64] * 5 + [C.c_float]
    L.ztvm_qkv_fused.argtypes = [vp, C.POINTER(QkvFusedDesc)]
    L.ztvm_qkv_fused_scratch.argtypes = [vp, C.POINTER(QkvFusedDesc), C.c_uint64, C.c_uint64]
    L.ztvm_kv_quantize_int8.argtypes = [vp, C.POINTER(KvQuantizeDesc)]
    L.ztvm_silu_mul.argtypes = [vp, u64, u64, u32, u32]
    L.ztvm_moe_combine.argtypes = [vp, u64, u64, u64, u32, u32, u32]
    L.ztvm_moe_router_logits.argtypes = [vp, u64, u64, u64, u64, u64, u32, u32, u32, u32]
    L.ztvm_moe_router_topk.argtypes = [vp, u64, u64, u64, u32, u32, u32, u32, u32]
    L.ztvm_moe_slot_translate.argtypes = [vp, u64, u64, u64, u32, u32]
    L.ztvm_repack_part.argtypes = [vp, u64, u64, C.c_size_t, C.c_int, u64]
    L.ztvm_repack_permute_rows.argtypes = [vp, u64, u64, C.c_size_t, u32, C.POINTER(u32), u32]
    L.ztvm_repack_dequant_split.argtypes = [vp, u64, u64, u64, u64, u32, u32, u32, u32, u64]
    _lib = L
    return L


def validate(desc):
    """Pure-CPU descriptor check. Returns (code, reason)."""
    buf = C.create_string_buffer(512)
    rc = load().ztvm_matmul_validate(C.byref(desc), buf, len(buf))
    return rc, buf.value.decode()


def resolve(desc):
    """Family AUTO picks for this descriptor; raises on an illegal descriptor."""
    L = load()
    rc = L.ztvm_matmul_resolve(C.byref(desc))
    if rc < 0:
        raise ZtvmError(rc, L.ztvm_last_error(None).decode())
    return rc


class Context:
    """One device + one in-order stream (the reference's GPUDevice + queue)."""

    def __init__(self, device=0):
        self._L = load()
        h = C.c_void_p()
        rc = self._L.ztvm_create(device, C.byref(h))
        if rc:
            raise ZtvmError(rc, self._L.ztvm_last_error(None).decode())
        self._h = h

    def _chk(self, rc):
        if rc:
            raise ZtvmError(rc, self._L.ztvm_last_error(self._h).decode())

    def close(self):
        if getattr(self, "_h", None):
            self._L.ztvm_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def device_info(self):
        name = C.create_string_buffer(256)
        cus, hbm = C.c_uint32(), C.c_uint64()
        self._chk(self._L.ztvm_device_info(self._h, name, len(name), C.byref(cus), C.byref(hbm)))
        return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value}

    def alloc(self, nbytes):
        p = C.c_uint64()
        self._chk(self._L.ztvm_alloc(self._h, nbytes, C.byref(p)))
        return p.value

    def free(self, dptr):
        self._chk(self._L.ztvm_free(self._h, dptr))

    def upload(self, dptr, array, offset=0):
        import numpy as np
        a = np.ascontiguousarray(array)
        self._chk(self._L.ztvm_upload(self._h, dptr, offset, a.ctypes.data_as(C.c_void_p), a.nbytes))

    def download(self, dptr, nbytes, dtype, offset=0):
        import numpy as np
        out = np.empty(nbytes // np.dtype(dtype).itemsize, dtype)
        self._chk(self._L.ztvm_download(self._h, out.ctypes.data_as(C.c_void_p), dptr, offset, out.nbytes))
        return out

    def fill(self, dptr, byte, nbytes, offset=0):
        self._chk(self._L.ztvm_fill(self._h, dptr, offset, byte, nbytes))

    def copy(self, dst, src, nbytes):
        self._chk(self._L.ztvm_copy(self._h, dst, src, nbytes))

    def read_probe(self, src, nbytes, sink):
        """A kernel that only reads nbytes from src: the streaming rate of the memory system, timed like a dispatch."""
        self._chk(self._L.ztvm_read_probe(self._h, src, nbytes, sink))

    def sync(self):
        self._chk(self._L.ztvm_sync(self._h))

    def matmul(self, desc):
        self._chk(self._L.ztvm_matmul(self._h, C.byref(desc)))

    def matmul_static(self, desc):
        """ztvm_matmul on the library's fixed scratch array: never allocates device memory."""
        self._chk(self._L.ztvm_matmul_static(self._h, C.byref(desc)))

    def ffn_gated(self, desc, up_weights, up_scales, up_biases=0):
        self._chk(self._L.ztvm_ffn_gated(self._h, C.byref(desc), up_weights, up_scales, up_biases))

    def ffn_gated_prologue(self, desc, up_weights, up_scales, up_biases, delta, gamma, rms_eps):
        self._chk(self._L.ztvm_ffn_gated_prologue(self._h, C.byref(desc), up_weights, up_scales, up_biases, delta, gamma,
                                                  C.c_float(rms_eps)))

    def qkv_fused(self, desc):
        self._chk(self._L.ztvm_qkv_fused(self._h, C.byref(desc)))

    def qkv_fused_scratch(self, desc, k_slot, v_slot):
        self._chk(self._L.ztvm_qkv_fused_scratch(self._h, C.byref(desc), k_slot, v_slot))

    def kv_quantize_int8(self, desc):
        self._chk(self._L.ztvm_kv_quantize_int8(self._h, C.byref(desc)))

    def dequant(self, desc):
        self._chk(self._L.ztvm_dequant(self._h, C.byref(desc)))

    def record_begin(self):
        self._chk(self._L.ztvm_record_begin(self._h))

    def record_end(self):
        cb = C.c_void_p()
        self._chk(self._L.ztvm_record_end(self._h, C.byref(cb)))
        return cb

    def submit(self, cb):
        self._chk(self._L.ztvm_submit(self._h, cb))

    def cmdbuf_destroy(self, cb):
        self._L.ztvm_cmdbuf_destroy(cb)

    def event(self):
        e = C.c_void_p()
        self._chk(self._L.ztvm_event_create(self._h, C.byref(e)))
        return e

    def event_record(self, e):
        self._chk(self._L.ztvm_event_record(self._h, e))

    def event_destroy(self, e):
        self._L.ztvm_event_destroy(e)

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._chk(self._L.ztvm_event_elapsed_ms(self._h, start, stop, C.byref(ms)))
        return ms.value

    def set_option(self, name, value):
        self._chk(self._L.ztvm_set_option(self._h, name.encode(), int(value)))

    def get_option(self, name):
        v = C.c_int()
        self._chk(self._L.ztvm_get_option(self._h, name.encode(), C.byref(v)))
        return v.value

    # -- the dispatches around the matmuls of an FFN / MoE block --------------------------------
    def silu_mul(self, out, gate_up, rows, ffn):
        self._chk(self._L.ztvm_silu_mul(self._h, out, gate_up, rows, ffn))

    def moe_combine(self, out, slots, score, tokens, N, SLOTS):
        self._chk(self._L.ztvm_moe_combine(self._h, out, slots, score, tokens, N, SLOTS))

    def moe_router_logits(self, logits, x, w, scales, biases, bits, D, rows, tokens=1):
        self._chk(self._L.ztvm_moe_router_logits(self._h, logits, x, w, scales or 0, biases or 0, bits, D, rows, tokens))

    def moe_router_topk(self, out_idx, out_score, logits, E, K, norm_topk, has_shared, tokens=1):
        self._chk(self._L.ztvm_moe_router_topk(self._h, out_idx, out_score, logits, E, K, int(norm_topk), int(has_shared),
                                               tokens))

    def moe_slot_translate(self, ids_out, ids_in, slot_map, n, map_len):
        self._chk(self._L.ztvm_moe_slot_translate(self._h, ids_out, ids_in, slot_map, n, map_len))

    # -- load-time repack ---------------------------------------------------------------------------
    def repack_part(self, dst, src, src_bytes, convert, overflow=0):
        self._chk(self._L.ztvm_repack_part(self._h, dst, src, src_bytes, convert, overflow))

    def repack_permute_rows(self, dst, src, nbytes, rows, src_rows):
        import numpy as np
        m = np.ascontiguousarray(src_rows, dtype=np.uint32)
        self._chk(self._L.ztvm_repack_permute_rows(self._h, dst, src, nbytes, rows,
                                                   m.ctypes.data_as(C.POINTER(C.c_uint32)), m.size))

    def repack_dequant_split(self, dst, weights, scales, biases, k, heads, nope, v, overflow=0):
        self._chk(self._L.ztvm_repack_dequant_split(self._h, dst, weights, scales, biases, k, heads, nope, v, overflow))
