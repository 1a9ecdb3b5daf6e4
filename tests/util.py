"""Shared helpers of the GPU parity tests: buffers, descriptors, error metrics."""
import numpy as np


class Dev:
    """Uploads numpy arrays through the C ABI and frees them on exit."""

    def __init__(self, ctx):
        self.ctx = ctx
        self.ptrs = []

    def put(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.ctx.alloc(max(arr.nbytes, 16))
        self.ptrs.append(p)
        self.ctx.upload(p, arr)
        return p

    def empty(self, nbytes, fill=None):
        p = self.ctx.alloc(max(nbytes, 16))
        self.ptrs.append(p)
        if fill is not None:
            self.ctx.fill(p, fill, nbytes)
        return p

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.ctx.sync()
        for p in self.ptrs:
            self.ctx.free(p)


def rel_err(got, ref, eps):
    """max |got-ref| / (|ref| + eps): the reference tests' metric
    (eps 1e-3 in tests/kernels/run.mjs:153, 1e-2 in tests/kernels/compile-qwen35.mjs:129-133)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert np.all(np.isfinite(got)), "non-finite output"  # NaN must fail, never pass a max()
    return float(np.max(np.abs(got - ref) / (np.abs(ref) + eps)))


def f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


def mutations(w, s, b):
    """The wrong kernels of the reference's mutation gate (scripts/mutation-gate.mjs; its figures at
    BENCH.md:1694-1701: unshifted scale index 2.51e+0, dropped bias 1.95e-1), expressed as wrong INPUTS to a
    correct reference: name -> (weights, scales, biases). A parity gate that passes any of them sees nothing."""
    w, s, b = np.asarray(w), np.asarray(s), np.asarray(b)
    swapped = ((w & np.uint32(0x0F0F0F0F)) << np.uint32(4)) | ((w >> np.uint32(4)) & np.uint32(0x0F0F0F0F))
    return {
        "scale group shifted by one": (w, np.roll(s, 1, axis=-1), b),
        "bias dropped": (w, s, np.zeros_like(b)),
        "nibble order swapped": (swapped.astype(np.uint32), s, b),
    }
