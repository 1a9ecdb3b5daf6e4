"""ztvm_matmul_static, the entry point that allocates nothing: same kernels as ztvm_matmul with the scratch of
the rows / skinny / tile-GEMM families in a fixed array of the library's device image. Called through the C ABI
and compared bit for bit with ztvm_matmul, two calls in a row per family, the second on a smaller input (the
array keeps the first call's contents), and on sizes past the array it must refuse with a clear message."""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu

# family, (M, N, K) of the first call, (M, N, K) of the second (smaller) call
CASES = [
    ("gemm", (300, 264, 1024), (130, 136, 512)),       # activation group sums [M][2K/64] f16
    ("skinny", (96, 1024, 2048), (20, 200, 256)),      # reordered activations, group sums, split-k partial sums
    ("rows", (8, 512, 14336), (3, 64, 14336)),         # a k range dealt to two workgroups: f32 partial sums
    ("auto", (512, 14336, 4096), (128, 14336, 4096)),  # configs[2]: tile GEMM, then the streaming kernel
]


def both(ctx, capi, synth, family, M, N, K):
    kernel = {"gemm": capi.KERNEL_GEMM, "skinny": capi.KERNEL_SKINNY, "rows": capi.KERNEL_ROWS, "auto": capi.KERNEL_AUTO}[family]
    A, w, s = synth.activations(M, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    with Dev(ctx) as d:
        out_a, out_s = d.empty(M * N * 2, fill=0), d.empty(M * N * 2, fill=0)
        common = dict(bits=4, affine=1, kernel=kernel, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64, in_=d.put(A),
                      scales=d.put(s), weights=d.put(w), biases=d.put(b))
        ctx.matmul(capi.MatmulDesc(out=out_a, **common))
        ctx.matmul_static(capi.MatmulDesc(out=out_s, **common))
        ya = ctx.download(out_a, M * N * 2, np.uint16).reshape(M, N)
        ys = ctx.download(out_s, M * N * 2, np.uint16).reshape(M, N)
    return A, w, s, b, ya, ys


@pytest.mark.parametrize("family,first,second", CASES)
def test_static_scratch_equals_matmul(ctx, capi, synth, oracle, family, first, second):
    for (M, N, K) in (first, second):
        print("ztvm_matmul_static", family, M, N, K, flush=True)
        A, w, s, b, ya, ys = both(ctx, capi, synth, family, M, N, K)
        assert np.array_equal(ya, ys), (family, M, N, K)
        rows = np.unique(np.array([0, M // 2, M - 1]))
        ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, len(rows), N, K, A[rows], w, s, b, threads=8)
        assert rel_err(ys[rows].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2


def test_static_scratch_refuses_what_does_not_fit(ctx, capi, synth):
    """The skinny family's f32 partial sums at M=128, N=14336 with the k range dealt to four workgroups are
    29 MB: past the 16 MiB array. The call must say so and launch nothing."""
    M, N, K = 128, 14336, 4096
    with Dev(ctx) as d:
        out = d.empty(M * N * 2, fill=0x5A)
        desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_SKINNY, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64,
                               out=out, in_=d.put(synth.activations(M, K)), scales=d.put(synth.scales(N, K)),
                               weights=d.put(synth.packed_weights(N, K)), biases=d.put(synth.biases(N, K, synth.scales(N, K))))
        ctx.set_option("skinny.ksplit", 4)
        try:
            with pytest.raises(capi.ZtvmError) as e:
                ctx.matmul_static(desc)
        finally:
            ctx.set_option("skinny.ksplit", 0)
        assert e.value.code == capi.E_UNSUPPORTED and "static buffer holds" in str(e.value)
        assert (ctx.download(out, M * N * 2, np.uint8) == 0x5A).all()


def test_static_entry_leaves_the_scratch_pool_alone(capi, synth):
    """What the entry point is for: on a fresh context (4 MiB pool) a dispatch that needs 8 MiB of scratch runs through
    ztvm_matmul_static, and afterwards the pool is still 4 MiB: the same dispatch through ztvm_matmul inside a
    recording (which cannot allocate) is refused with the pool's size in the message."""
    M, N, K = 512, 1024, 4096   # tile GEMM with its k split: 16 tiles x 4 parts x 128 KiB of f32 totals
    with capi.Context(0) as fresh:
        with Dev(fresh) as d:
            out = d.empty(M * N * 2, fill=0)
            s = synth.scales(N, K)
            desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64,
                                   out=out, in_=d.put(synth.activations(M, K)), scales=d.put(s), weights=d.put(synth.packed_weights(N, K)),
                                   biases=d.put(synth.biases(N, K, s)))
            fresh.matmul_static(desc)
            fresh.sync()
            assert fresh.download(out, M * N * 2, np.uint16).any()
            fresh.record_begin()
            try:
                fresh.fill(out, 0, 256)   # the recording holds one dispatch whatever happens next
                with pytest.raises(capi.ZtvmError) as e:
                    fresh.matmul(desc)
            finally:
                fresh.cmdbuf_destroy(fresh.record_end())
            assert e.value.code == capi.E_UNSUPPORTED and "have 4194304" in str(e.value), str(e.value)
