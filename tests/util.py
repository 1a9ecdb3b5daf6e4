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
