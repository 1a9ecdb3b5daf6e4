"""GPU parity of the tile GEMM's k split: tiles that would leave CUs idle (few tiles, or the ones past the last full
round of workgroups) are dealt to several workgroups along k, which exchange f32 totals through scratch memory; the
last part to arrive adds them in part order. Checked through the C ABI: against the formula, against the same
dispatch with the split switched off (`gemm.split = 1`), launch after launch bit for bit (no result may depend on
which part arrives last), rows past M untouched, one-hot activations bit-exact, recorded replays, and the
no-allocation entry point (same plan where the exchange fits its fixed buffer, no split where it does not).
Reference dispatch of the same chunk matmuls: src/zero-tvm/engine-core.ts:4280-4293 (foldGridX :247-259)."""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def make(synth, bits, affine, M, N, K):
    A = synth.activations(M, K)
    w = synth.packed_weights(N, K, bits=bits)
    s = synth.scales(N, K, affine=affine)
    b = synth.biases(N, K, s) if affine else None
    return A, w, s, b


def describe(capi, d, bits, affine, M, N, K, A, w, s, b, out):
    return capi.MatmulDesc(bits=bits, affine=int(affine), kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K * bits // 32,
                           scales_per_row=K // (64 if affine else 32), out=out, in_=d.put(A), scales=d.put(s),
                           weights=d.put(w), biases=d.put(b) if affine else 0)


# M, N, K, bits, affine: tiles (256 x 128 above 256 rows, 128 x 128 below) and the parts they are dealt to on 256 CUs
CASES = [
    (512, 1024, 4096, 4, True),    # 16 tiles, four parts of 16 steps
    (300, 2000, 2048, 4, True),    # 32 tiles (ragged last column tile and row tile), two parts
    (512, 1024, 4096, 4, False),   # symmetric group-32 rows
    (512, 1024, 4096, 8, True),
    (512, 1024, 4096, 3, True),
    (200, 1100, 2048, 4, True),    # 128 x 128 tiles: 18 tiles, two parts
    (2048, 4224, 8192, 4, True),   # 264 tiles: one full round whole, the last eight tiles in eight parts
    (520, 640, 4480, 4, True),     # 70 steps: parts of unequal length (18, 18, 18 and 16 steps)
]


@pytest.mark.parametrize("M,N,K,bits,affine", CASES)
def test_split_against_formula_and_unsplit(ctx, capi, synth, oracle, M, N, K, bits, affine):
    A, w, s, b = make(synth, bits, affine, M, N, K)
    CAP = M + 8
    Acap = np.concatenate([A, np.zeros((8, K), A.dtype)])
    with Dev(ctx) as d:
        out = d.empty(CAP * N * 2, fill=0x5A)
        desc = describe(capi, d, bits, affine, M, N, K, Acap, w, s, b, out)
        runs = []
        for _ in range(4):   # launch after launch: the arrival order of the parts differs, the bits must not
            ctx.matmul(desc)
            runs.append(ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N))
        ctx.set_option("gemm.split", 1)
        try:
            ctx.fill(out, 0x5A, CAP * N * 2)
            ctx.matmul(desc)
            whole = ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N)
        finally:
            ctx.set_option("gemm.split", 0)
    got = runs[0]
    for r in runs[1:]:
        assert np.array_equal(r, got), "a split result depends on the launch"
    assert (got[M:] == 0x5A5A).all() and (whole[M:] == 0x5A5A).all(), "rows past M were written"
    rows = np.unique(np.concatenate([np.arange(0, M, 61), [M - 1, 255 % M, 256 % M]]))
    mode = oracle.MODE_FORMULA_F64
    ref = oracle.gemm(mode, bits, affine, len(rows), N, K, np.ascontiguousarray(A[rows]), w, s, b, threads=8)
    y = got[rows].view(np.float16).astype(np.float64)
    assert rel_err(y, ref, 1e-2) < 1e-2
    # the parts' f32 totals are added in another order than one workgroup's running sum: the last f16 bit or two
    yw = whole[:M].view(np.float16).astype(np.float64)
    assert rel_err(got[:M].view(np.float16).astype(np.float64), yw, 1e-2) < (6e-3 if bits == 8 else 2e-3)
    assert not np.array_equal(got[:M], whole[:M]) or K <= 64 * 16, "the split did not take place"


def test_split_one_hot_is_bit_exact(ctx, capi, synth, oracle):
    """Rows of the identity: every part but one holds zeros, so the sum of the parts is the dequantized weight
    f16(fl32(q*s+b)), bit for bit, whichever part a column's k falls in."""
    N, K = 1024, 4096
    _, w, s, b = make(synth, 4, True, 1, N, K)
    ks = (np.arange(512, dtype=np.int64) * 67 + 3) % K   # spread over all four parts
    A = np.zeros((512, K), np.float16)
    A[np.arange(512), ks] = 1.0
    with Dev(ctx) as d:
        out = d.empty(512 * N * 2, fill=0)
        ctx.matmul(describe(capi, d, 4, True, 512, N, K, A.view(np.uint16), w, s, b, out))
        got = ctx.download(out, 512 * N * 2, np.uint16).reshape(512, N)
    w16 = oracle.dequant_matrix(4, True, N, K, w, s, b, want="f16")
    assert np.array_equal(got, w16[:, ks].T)


def test_split_recorded_replays(ctx, capi, synth):
    """A command buffer that holds a split dispatch: every replay equals the eager result (the arrival counters are
    back at zero after each launch), with eager launches of another split shape in between."""
    M, N, K = 512, 1024, 4096
    A, w, s, b = make(synth, 4, True, M, N, K)
    A2, w2, s2, b2 = make(synth, 4, True, 300, 2000, 2048)
    with Dev(ctx) as d:
        out, out2 = d.empty(M * N * 2, fill=0), d.empty(300 * 2000 * 2, fill=0)
        desc = describe(capi, d, 4, True, M, N, K, A, w, s, b, out)
        other = describe(capi, d, 4, True, 300, 2000, 2048, A2, w2, s2, b2, out2)
        ctx.matmul(desc)
        eager = ctx.download(out, M * N * 2, np.uint16)
        ctx.matmul(other)
        eager2 = ctx.download(out2, 300 * 2000 * 2, np.uint16)
        ctx.record_begin()
        ctx.matmul(desc)
        cb = ctx.record_end()
        try:
            for _ in range(3):
                ctx.fill(out, 0, M * N * 2)
                ctx.submit(cb)
                assert np.array_equal(ctx.download(out, M * N * 2, np.uint16), eager)
                ctx.fill(out2, 0, 300 * 2000 * 2)
                ctx.matmul(other)
                assert np.array_equal(ctx.download(out2, 300 * 2000 * 2, np.uint16), eager2)
        finally:
            ctx.cmdbuf_destroy(cb)


def test_static_entry_splits_only_what_fits(ctx, capi, synth, oracle):
    """ztvm_matmul_static: the exchange of (512, 1024, 4096) is 8 MiB and fits the 16 MiB array: same plan, same bits
    as ztvm_matmul. That of (512, 4096, 4096) is 32 MiB: the dispatch runs unsplit from the array (the bits of
    `gemm.split = 1`), and nothing is refused."""
    for (M, N, K), same_plan in (((512, 1024, 4096), True), ((512, 4096, 4096), False)):
        A, w, s, b = make(synth, 4, True, M, N, K)
        with Dev(ctx) as d:
            out_a, out_s, out_w = (d.empty(M * N * 2, fill=0) for _ in range(3))
            common = dict(bits=4, affine=1, kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64,
                          in_=d.put(A), scales=d.put(s), weights=d.put(w), biases=d.put(b))
            ctx.matmul(capi.MatmulDesc(out=out_a, **common))
            ctx.matmul_static(capi.MatmulDesc(out=out_s, **common))
            ctx.set_option("gemm.split", 1)
            try:
                ctx.matmul(capi.MatmulDesc(out=out_w, **common))
            finally:
                ctx.set_option("gemm.split", 0)
            ya, ys, yw = (ctx.download(o, M * N * 2, np.uint16).reshape(M, N) for o in (out_a, out_s, out_w))
        assert np.array_equal(ys, ya if same_plan else yw), (M, N, K)
        rows = np.array([0, M // 2, M - 1])
        ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, len(rows), N, K, A[rows], w, s, b, threads=8)
        assert rel_err(ys[rows].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
