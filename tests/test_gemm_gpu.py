"""GPU parity of the MFMA prefill GEMM (and of every family on M>1 dense dispatches).

Shapes and invariants follow the reference's GEMM tests
(tests/kernels/compile-qwen35.mjs:963-1152: M=6/CAP=8 N=64, M=31/CAP=64 N=256,
M=47/CAP=64 N=200, K=2560; scripts/gemm-sweep-native.mjs:374: 13x96x128):
  * from-the-formula reference, |y-ref|/(|ref|+1e-2) < 1e-2, for EVERY family: the
    MFMA GEMM multiplies exact integer weights and scales in f32, so it holds the
    same bar as the GEMV instead of the looser one the reference grants its
    f16-staged matrix-unit kernels (scripts/gemm-bench.mjs:516-521)
  * rows past M stay untouched, and M-invariance is bit-exact.
"""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def run(ctx, capi, affine, M, CAP, N, K, A, w, s, b, kernel, prefill=0):
    with Dev(ctx) as d:
        out = d.empty(CAP * N * 2, fill=prefill)
        desc = capi.MatmulDesc(bits=4, affine=int(affine), kernel=kernel, M=M, N=N, k_packed=K // 8,
                               scales_per_row=K // (64 if affine else 32), out=out, in_=d.put(A), scales=d.put(s),
                               weights=d.put(w), biases=d.put(b) if affine else 0)
        ctx.matmul(desc)
        return ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N)


def make(synth, affine, CAP, N, K, regime="A"):
    A = synth.activations(CAP, K)
    w = synth.packed_weights(N, K)
    s = synth.scales(N, K, affine=affine)
    b = synth.biases(N, K, s, regime) if affine else None
    return A, w, s, b


CASES = [(6, 8, 64, 2560, False), (31, 64, 256, 2560, True), (47, 64, 200, 2560, False), (47, 64, 200, 2560, True),
         (13, 64, 96, 128, True), (13, 64, 96, 128, False), (130, 256, 136, 512, True), (300, 320, 264, 1024, True),
         (200, 200, 72, 64, False), (270, 272, 72, 192, False)]  # one and three k steps: no hot loop, short pipelines


@pytest.mark.parametrize("M,CAP,N,K,affine", CASES)
@pytest.mark.parametrize("family", ["gemm", "gemv", "auto"])
def test_ragged_gemm(ctx, capi, synth, oracle, M, CAP, N, K, affine, family):
    kernel = {"gemm": capi.KERNEL_GEMM, "gemv": capi.KERNEL_GEMV, "auto": capi.KERNEL_AUTO}[family]
    A, w, s, b = make(synth, affine, CAP, N, K)
    got = run(ctx, capi, affine, M, CAP, N, K, A, w, s, b, kernel)
    gotcap = run(ctx, capi, affine, CAP, CAP, N, K, A, w, s, b, kernel)
    y = got[:M].view(np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, affine, M, N, K, A, w, s, b, threads=8)
    assert rel_err(y, ref, 1e-2) < 1e-2
    assert rel_err(y, ref, 1e-3) < 2e-2
    assert not got[M:].any(), "rows past M were written"

    def family_of(m):
        return capi.resolve(capi.MatmulDesc(bits=4, affine=int(affine), kernel=kernel, M=m, N=N, k_packed=K // 8,
                                            scales_per_row=K // (64 if affine else 32), out=4096, in_=4096, scales=4096,
                                            weights=4096, biases=4096 if affine else 0))
    # the skinny family has two tile shapes (up to 32 rows, above) that deal K to their waves differently
    same_order = family_of(M) == family_of(CAP) and not (family_of(M) == capi.KERNEL_SKINNY and (M <= 32) != (CAP <= 32))
    if same_order:
        assert np.array_equal(got[:M], gotcap[:M]), "M-variance"
    else:
        # AUTO changes family with M (2, 17 and 129 rows): a row's result is bit-stable inside a family and tile shape;
        # across them it agrees to the last f16 bit or two (different f32 summation order)
        assert rel_err(y, gotcap[:M].view(np.float16).astype(np.float64), 1e-2) < 2e-3


def test_gemm_one_hot_pins_staged_weights(ctx, capi, synth, oracle):
    """A = rows of the identity: Y[m,n] is the dequantized weight f16(fl32(q*s+b)) of W[n,k_m], bit for bit."""
    N, K = 160, 256
    for affine in (True, False):
        _, w, s, b = make(synth, affine, 1, N, K)
        ks = np.array([0, 1, 3, 4, 7, 8, 15, 31, 32, 33, 63, 64, 65, 127, 128, 191, 200, 255] * 4, np.int64)[:64]
        A = np.zeros((64, K), np.float16)
        A[np.arange(64), ks] = 1.0
        got = run(ctx, capi, affine, 64, 64, N, K, A.view(np.uint16), w, s, b, capi.KERNEL_GEMM)
        w16 = oracle.dequant_matrix(4, affine, N, K, w, s, b, want="f16")
        assert np.array_equal(got, w16[:, ks].T)


def test_seeded_random_shapes(ctx, capi, synth, oracle):
    """Thirty seeded shapes through the tile family: every tile height (M up to 600 crosses the 64-, 128- and 256-row
    tiles and their partial last tiles), ragged N, K from two scale pairs up, both formats; rows past M stay untouched."""
    rng = np.random.default_rng(20240611)
    for case in range(30):
        affine = bool(case % 2)
        M = int(rng.choice([1, 7, 8, 9, 63, 65, 129, 255, 257, 300, 511, 600]) if case < 12 else rng.integers(1, 601))
        N = int(rng.integers(1, 420))
        K = 128 * int(rng.choice([1, 2, 3, 5, 8, 11, 16]))
        CAP = M + int(rng.integers(0, 9))
        A, w, s, b = make(synth, affine, CAP, N, K)
        got = run(ctx, capi, affine, M, CAP, N, K, A, w, s, b, capi.KERNEL_GEMM, prefill=0x5A)
        ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, affine, M, N, K, A, w, s, b, threads=8)
        err = rel_err(got[:M].view(np.float16).astype(np.float64), ref, 1e-2)
        assert err < 1e-2, (case, affine, M, N, K, err)
        assert (got[M:] == 0x5A5A).all(), (case, "rows past M were written")


def run3(ctx, capi, M, CAP, N, K, A, w, s, b, kernel, prefill=0):
    with Dev(ctx) as d:
        out = d.empty(CAP * N * 2, fill=prefill)
        desc = capi.MatmulDesc(bits=3, affine=1, kernel=kernel, M=M, N=N, k_packed=3 * K // 32, scales_per_row=K // 64, out=out,
                               in_=d.put(A), scales=d.put(s), weights=d.put(w), biases=d.put(b))
        ctx.matmul(desc)
        return ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N)


@pytest.mark.parametrize("M,CAP,N,K", [(6, 8, 64, 2560), (47, 64, 200, 1024), (130, 256, 136, 512), (300, 320, 264, 1024),
                                       (257, 260, 136, 256), (511, 512, 392, 640)])
def test_three_bit_tile_gemm(ctx, capi, synth, oracle, M, CAP, N, K):
    """The 3-bit form (24-bit windows of the row bitstream, fetched as the dwords that cover a thread's bytes) against
    the formula at every tile height, with rows past M untouched and no dependence on the rows that follow."""
    A = synth.activations(CAP, K)
    w = synth.packed_weights(N, K, bits=3)
    s = synth.scales(N, K)
    b = synth.biases(N, K, s, "A")
    got = run3(ctx, capi, M, CAP, N, K, A, w, s, b, capi.KERNEL_GEMM, prefill=0x5A)
    full = run3(ctx, capi, CAP, CAP, N, K, A, w, s, b, capi.KERNEL_GEMM)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 3, True, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got[:M].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert (got[M:] == 0x5A5A).all(), "rows past M were written"
    assert np.array_equal(got[:M], full[:M]), "M-variance"


def test_three_bit_one_hot_is_the_dequantized_weight(ctx, capi, synth, oracle):
    """Rows of the identity through the 3-bit tile GEMM return f16(fl32(q*s + b)) bit for bit, at k positions on
    both sides of every word boundary of the bitstream."""
    N, K = 160, 256
    w = synth.packed_weights(N, K, bits=3)
    s = synth.scales(N, K)
    b = synth.biases(N, K, s, "A")
    ks = np.array([0, 1, 7, 8, 9, 10, 11, 15, 20, 21, 22, 31, 32, 33, 42, 43, 63, 64, 65, 85, 86, 127, 128, 191, 200, 255] * 3,
                  np.int64)[:64]
    A = np.zeros((64, K), np.float16)
    A[np.arange(64), ks] = 1.0
    got = run3(ctx, capi, 64, 64, N, K, A.view(np.uint16), w, s, b, capi.KERNEL_GEMM)
    w16 = oracle.dequant_matrix(3, True, N, K, w, s, b, want="f16")
    assert np.array_equal(got, w16[:, ks].T)


def test_odd_scale_count_leaves_the_tile_family(ctx, capi, synth, oracle):
    """The tile GEMM fetches scales as 4-byte pairs, so rows of an odd number of scales (K = 192: three groups of
    64) are not its to take: asked for by name it is refused, and the default routing serves them elsewhere."""
    M, N, K = 140, 136, 192
    A, w, s, b = make(synth, True, M, N, K)
    desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K // 8, scales_per_row=3,
                           out=4096, in_=4096, scales=4096, weights=4096, biases=4096)
    rc, why = capi.validate(desc)
    assert rc == capi.E_UNSUPPORTED, why
    desc.kernel = capi.KERNEL_AUTO
    assert capi.resolve(desc) != capi.KERNEL_GEMM
    got = run(ctx, capi, True, M, M, N, K, A, w, s, b, capi.KERNEL_AUTO)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2


@pytest.mark.parametrize("rows", [257, 264, 511])
def test_rows_past_the_last_full_group(ctx, capi, synth, oracle, rows):
    """256 x 128 tiles whose last tile holds 1, 8 or 255 rows: the fetch groups that reach past M are moved back
    over valid rows and must neither disturb the rows they repeat nor write past M."""
    N, K = 136, 256
    A, w, s, b = make(synth, True, 512, N, K)
    got = run(ctx, capi, True, rows, 512, N, K, A, w, s, b, capi.KERNEL_GEMM, prefill=0x5A)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, rows, N, K, A, w, s, b, threads=8)
    assert rel_err(got[:rows].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert (got[rows:] == 0x5A5A).all(), "rows past M were written"
    full = run(ctx, capi, True, 512, 512, N, K, A, w, s, b, capi.KERNEL_GEMM)
    assert np.array_equal(got[:rows], full[:rows]), "a row depends on how many rows follow it"


@pytest.mark.parametrize("M", [128, 512, 2048])
def test_config3_shape(ctx, capi, synth, oracle, M):
    """configs[2]: K=4096, N=14336; checked on a row sample against the formula and the f16-weight reference."""
    K, N = 4096, 14336
    A, w, s, b = make(synth, True, M, N, K)
    got = run(ctx, capi, True, M, M, N, K, A, w, s, b, capi.KERNEL_GEMM)
    # one row of every 256-row tile (at a different place in each), and the first and last row of the matrix: M=2048 is
    # 8 tile rows in 3.5 rounds of workgroups, the last half round split along k
    rows = np.unique(np.concatenate([[0, 1, M - 1], [min(t + (37 * (t // 256 + 1)) % 256, M - 1) for t in range(0, M, 256)]]))
    y = got[rows].view(np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, len(rows), N, K, A[rows], w, s, b, threads=8)
    e = rel_err(y, ref, 1e-2)
    print("M=%d: rel err vs formula %.2e" % (M, e))
    assert e < 1e-2
    # every row agrees with the GEMV family's answer for the same row (two independent kernels)
    gv = run(ctx, capi, True, len(rows), len(rows), N, K, A[rows], w, s, b, capi.KERNEL_GEMV)
    assert rel_err(y, gv.view(np.float16).astype(np.float64), 1e-2) < 1e-2


def test_recorded_gemm_survives_scratch_growth(ctx, capi, synth, oracle):
    """A command buffer keeps the scratch address of its GEMM (activation group sums). A later eager
    dispatch that needs more scratch than the context owns must not free what the command buffer
    references: record, grow, replay, and the replay still equals the eager result and the oracle."""
    M, N, K = 160, 136, 512
    A, w, s, b = make(synth, True, M, N, K)
    eager = run(ctx, capi, True, M, M, N, K, A, w, s, b, capi.KERNEL_GEMM)
    with Dev(ctx) as d:
        out = d.empty(M * N * 2, fill=0)
        desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64,
                               out=out, in_=d.put(A), scales=d.put(s), weights=d.put(w), biases=d.put(b))
        ctx.record_begin()
        ctx.matmul(desc)
        cb = ctx.record_end()
        try:
            ctx.submit(cb)
            first = ctx.download(out, M * N * 2, np.uint16).reshape(M, N)
            assert np.array_equal(first, eager)
            # a skinny dispatch whose f32 partial sums outgrow any scratch this session has allocated so far
            Mb, Nb, Kb = 128, 40960, 256
            big = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_SKINNY, M=Mb, N=Nb, k_packed=Kb // 8, scales_per_row=Kb // 64,
                                  out=d.empty(Mb * Nb * 2), in_=d.put(synth.activations(Mb, Kb)), scales=d.put(synth.scales(Nb, Kb)),
                                  weights=d.put(synth.packed_weights(Nb, Kb)), biases=d.put(synth.biases(Nb, Kb, synth.scales(Nb, Kb))))
            ctx.set_option("skinny.ksplit", 4)   # 4 x 128 x 40960 f32 partial sums = 80 MiB
            try:
                ctx.matmul(big)
                ctx.sync()
            finally:
                ctx.set_option("skinny.ksplit", 0)
            for _ in range(2):
                ctx.fill(out, 0, M * N * 2)
                ctx.submit(cb)
                again = ctx.download(out, M * N * 2, np.uint16).reshape(M, N)
                assert np.array_equal(again, eager), "replay after the scratch grew differs from the eager result"
        finally:
            ctx.cmdbuf_destroy(cb)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, M, N, K, A, w, s, b, threads=8)
    assert rel_err(eager.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
