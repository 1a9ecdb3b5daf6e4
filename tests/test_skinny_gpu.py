"""GPU parity of the weight-streaming matrix-core kernel (family 'skinny', 17 <= M <= 128 rows by
default, any M when asked for).

The cases mirror the reference's small-batch checks (tests/kernels/compile-qwen35.mjs:963-1152:
M=6 N=64, M=31 N=256, M=47 N=200 at K=2560; scripts/gemm-sweep-native.mjs:374: 13x96x128) and add
the formats the reference ships for the same dispatch: symmetric group-32, the 3-bit stream and the
8-bit affine layout (src/compiler/shaders/int8_affine_batched.wgsl).
Bars: |y-ref|/(|ref|+1e-2) < 1e-2 against the from-the-formula f64 oracle (the kernel multiplies
exact integer weights and scales in f32, so it holds the GEMV's bar), rows past M untouched,
results independent of M and of the tile height, one-hot rows bit-exact.
"""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def run(ctx, capi, bits, affine, M, CAP, N, K, A, w, s, b, kernel, out_f32=0, prefill=0):
    esz = 4 if out_f32 else 2
    with Dev(ctx) as d:
        out = d.empty(CAP * N * esz, fill=prefill)
        desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=out_f32, kernel=kernel, M=M, N=N, k_packed=K * bits // 32,
                               scales_per_row=K // (64 if affine else 32), out=out, in_=d.put(A), scales=d.put(s),
                               weights=d.put(w), biases=d.put(b) if affine else 0)
        ctx.matmul(desc)
        return ctx.download(out, CAP * N * esz, np.uint32 if out_f32 else np.uint16).reshape(CAP, N)


def make(synth, bits, affine, CAP, N, K, regime="A"):
    A = synth.activations(CAP, K)
    w = synth.packed_weights(N, K, bits=bits)
    s = synth.scales(N, K, affine=affine)
    b = synth.biases(N, K, s, regime) if affine else None
    return A, w, s, b


FORMATS = [(4, True), (4, False), (3, True), (8, True)]
CASES = [(2, 8, 64, 2560), (6, 8, 64, 2560), (31, 64, 256, 2560), (33, 64, 256, 2560), (47, 64, 200, 2560), (13, 64, 96, 128),
         (64, 64, 136, 64), (65, 128, 136, 192), (100, 128, 264, 1024), (128, 128, 128, 512), (130, 256, 136, 512),
         (300, 320, 264, 1024)]


@pytest.mark.parametrize("M,CAP,N,K", CASES)
@pytest.mark.parametrize("bits,affine", FORMATS)
def test_ragged_skinny(ctx, capi, synth, oracle, M, CAP, N, K, bits, affine):
    A, w, s, b = make(synth, bits, affine, CAP, N, K)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, A, w, s, b, threads=8)

    def check(got):
        y = got[:M].view(np.float16).astype(np.float64)
        assert rel_err(y, ref, 1e-2) < 1e-2
        assert rel_err(y, ref, 1e-3) < 2e-2
        assert not got[M:].any(), "rows past M were written"

    check(run(ctx, capi, bits, affine, M, CAP, N, K, A, w, s, b, capi.KERNEL_SKINNY))  # the tile shape and k split chosen for M
    # one tile shape and one k split whatever M is: a row's bits must not depend on the rows that travel with it
    ctx.set_option("skinny.ksplit", 1)
    ctx.set_option("skinny.shape", 2)
    try:
        got = run(ctx, capi, bits, affine, M, CAP, N, K, A, w, s, b, capi.KERNEL_SKINNY)
        gotcap = run(ctx, capi, bits, affine, CAP, CAP, N, K, A, w, s, b, capi.KERNEL_SKINNY)
    finally:
        ctx.set_option("skinny.ksplit", 0)
        ctx.set_option("skinny.shape", 0)
    check(got)
    assert np.array_equal(got[:M], gotcap[:M]), "M-variance"


@pytest.mark.parametrize("ksplit", [0, 2, 3, 8])
@pytest.mark.parametrize("bits,affine", FORMATS)
def test_k_split(ctx, capi, synth, oracle, bits, affine, ksplit):
    """K dealt to several workgroups, partial results summed in f32 in split order; 0 = the library's choice."""
    M, N, K = 8, 264, 2048
    A, w, s, b = make(synth, bits, affine, M, N, K)
    ctx.set_option("skinny.ksplit", ksplit)
    try:
        got = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b, capi.KERNEL_SKINNY)
        got32 = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b, capi.KERNEL_SKINNY, out_f32=1)
    finally:
        ctx.set_option("skinny.ksplit", 0)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    # f32 accumulation noise; byte-valued weights make the per-group integer sums 16 times larger than nibbles do,
    # and the products that cancel in the total are rounded at that size
    assert rel_err(got32.view(np.float32).astype(np.float64), ref, 1.0) < (4e-5 if bits == 8 else 1e-5)


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("M,N,K,shape", [(24, 136, 14336, 0), (100, 136, 14336, 0), (40, 132, 1024, 0), (40, 130, 1024, 0),
                                         (70, 264, 4096, 3), (20, 264, 4096, 2), (9, 72, 16384, 0), (9, 72, 18432, 0)])
def test_transfer_kernel_corners(ctx, capi, synth, oracle, M, N, K, shape, affine):
    """The 4-bit transfer-engine kernel away from the bench shape: long rows (K = 14336: seven bias steps, so some
    ride on the second unit sent past the end and their biases are fetched after the loop; 16384 is the longest it
    takes, 18432 goes to the register-path kernel), N that is no multiple of 8 (results leave in the accumulator
    layout) or of 4 (no split over workgroups), either tile shape at any M, and an output that starts 2 bytes off a
    16-byte boundary."""
    A, w, s, b = make(synth, 4, affine, M, N, K)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, affine, M, N, K, A, w, s, b, threads=8)
    X, W, S = ctx.alloc(A.nbytes), ctx.alloc(w.nbytes), ctx.alloc(s.nbytes)
    B = ctx.alloc(b.nbytes) if affine else 0
    out = ctx.alloc(M * N * 2 + 16)
    ctx.set_option("skinny.shape", shape)
    try:
        got = run(ctx, capi, 4, affine, M, M, N, K, A, w, s, b, capi.KERNEL_SKINNY)
        got32 = run(ctx, capi, 4, affine, M, M, N, K, A, w, s, b, capi.KERNEL_SKINNY, out_f32=1)
        # the same dispatch into an output 2 bytes past a 16-byte boundary
        ctx.upload(X, A); ctx.upload(W, w); ctx.upload(S, s)
        if affine:
            ctx.upload(B, b)
        ctx.fill(out, 0, M * N * 2 + 16)
        ctx.matmul(capi.MatmulDesc(bits=4, affine=int(affine), kernel=capi.KERNEL_SKINNY, M=M, N=N, k_packed=K // 8,
                                   scales_per_row=K // (64 if affine else 32), out=out + 2, in_=X, scales=S, weights=W, biases=B))
        raw = ctx.download(out, M * N * 2 + 16, np.uint16)
    finally:
        ctx.set_option("skinny.shape", 0)
        for a in (X, W, S, out) + ((B,) if affine else ()):
            ctx.free(a)
    y = got.view(np.float16).astype(np.float64)
    assert rel_err(y, ref, 1e-2) < 1e-2
    assert rel_err(got32.view(np.float32).astype(np.float64), ref, 1.0) < 2e-5
    assert raw[0] == 0 and not raw[1 + M * N:].any(), "bytes around the output were written"
    assert np.array_equal(raw[1:1 + M * N].reshape(M, N), got), "the output's alignment changed the result"


def test_one_hot_pins_streamed_weights(ctx, capi, synth, oracle):
    """A = rows of the identity: Y[m,n] is the dequantized weight f16(fl32(q*s+b)) of W[n,k_m], bit for bit."""
    N, K = 160, 256
    ks = np.array([0, 1, 3, 4, 7, 8, 15, 31, 32, 33, 63, 64, 65, 127, 128, 191, 200, 255] * 4, np.int64)[:64]
    A = np.zeros((64, K), np.float16)
    A[np.arange(64), ks] = 1.0
    for bits, affine in FORMATS:
        _, w, s, b = make(synth, bits, affine, 1, N, K)
        got = run(ctx, capi, bits, affine, 64, 64, N, K, A.view(np.uint16), w, s, b, capi.KERNEL_SKINNY)
        w16 = oracle.dequant_matrix(bits, affine, N, K, w, s, b, want="f16")
        assert np.array_equal(got, w16[:, ks].T), (bits, affine)


@pytest.mark.parametrize("bits,affine", FORMATS)
def test_families_agree(ctx, capi, synth, bits, affine):
    """The per-token GEMV and the streaming kernel follow the same arithmetic: same f16 results up to
    one rounding step on a few outputs (different f32 summation order inside a group)."""
    M, N, K = 16, 256, 1024
    A, w, s, b = make(synth, bits, affine, M, N, K)
    g = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b, capi.KERNEL_GEMV).view(np.float16).astype(np.float64)
    k = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b, capi.KERNEL_SKINNY).view(np.float16).astype(np.float64)
    assert rel_err(k, g, 1e-2) < 2e-3


def test_config5_int3_m8(ctx, capi, synth, oracle):
    """configs[4]: 3-bit weights, M=8, K=4096, N=14336, against the formula."""
    M, K, N = 8, 4096, 14336
    A, w, s, b = make(synth, 3, True, M, N, K)
    got = run(ctx, capi, 3, True, M, M, N, K, A, w, s, b, capi.KERNEL_AUTO)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 3, True, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2


@pytest.mark.parametrize("M,N,K,affine,bits", [(512, 4096, 14336, True, 4), (1000, 4096, 4096, True, 4), (200, 4096, 4096, False, 4),
                                               (640, 6144, 4096, True, 4), (512, 4096, 14336, True, 8), (250, 4096, 4096, True, 3)])
def test_many_row_tiles(ctx, capi, synth, oracle, M, N, K, affine, bits):
    """This family above 128 rows, on shapes with few column tiles: several rounds of workgroups, a last row tile that
    is partly empty, with and without a k split, in the transfer-engine kernel (4-bit) and the register-path kernel
    (8-bit, 3-bit). A sample of rows against the formula, the rows past M untouched, and agreement with the tile GEMM
    (which splits k over workgroups on these shapes)."""
    A, w, s, b = make(synth, bits, affine, M, N, K)
    CAP = M + 8
    Acap = np.concatenate([A, np.zeros((8, K), A.dtype)])
    got = run(ctx, capi, bits, affine, M, CAP, N, K, Acap, w, s, b, capi.KERNEL_SKINNY, prefill=0x5A)
    assert (got[M:] == 0x5A5A).all(), "rows past M were written"
    rows = np.unique(np.concatenate([np.arange(0, M, 37), [M - 1, M - 2, 63, 64, 127, 128]]))
    rows = rows[rows < M]
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, len(rows), N, K, np.ascontiguousarray(A[rows]), w, s, b, threads=8)
    y = got[rows].view(np.float16).astype(np.float64)
    assert rel_err(y, ref, 1e-2) < 1e-2
    # the same rows through the tile GEMM agree to the last bits of f16 (byte-valued weights over a long K give
    # outputs near 100 whose f32 sums differ more between two summation orders than near-zero outputs forgive)
    gemm = run(ctx, capi, bits, affine, M, CAP, N, K, Acap, w, s, b, capi.KERNEL_GEMM)
    assert rel_err(y, gemm[rows].view(np.float16).astype(np.float64), 1e-2) < (6e-3 if bits == 8 else 2e-3)


def test_default_split_follows_the_row_count(ctx, capi, synth, oracle):
    """With the default knobs the transfer-engine kernel deals k to as many workgroups as fill one round of the CUs,
    and the number of row tiles enters that count: at K=4096, N=4096 a row travels with 40 rows in eight k parts and
    with 100 rows in four. Same row, another f32 summation order: the last f16 bit or two, held to a stated
    tolerance here (pin `skinny.ksplit` for bit-stable rows across M; test_ragged_skinny does)."""
    M, CAP, N, K = 40, 100, 4096, 4096
    A, w, s, b = make(synth, 4, True, CAP, N, K)
    small = run(ctx, capi, 4, True, M, M, N, K, A[:M], w, s, b, capi.KERNEL_SKINNY).view(np.float16).astype(np.float64)
    big = run(ctx, capi, 4, True, CAP, CAP, N, K, A, w, s, b, capi.KERNEL_SKINNY).view(np.float16).astype(np.float64)
    assert rel_err(small, big[:M], 1e-2) < 2e-3
    rows = np.array([0, 17, M - 1])
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, len(rows), N, K, np.ascontiguousarray(A[rows]), w, s, b, threads=8)
    assert rel_err(small[rows], ref, 1e-2) < 1e-2 and rel_err(big[rows], ref, 1e-2) < 1e-2


def test_auto_picks_skinny(capi):
    for M, want in ((1, capi.KERNEL_GEMV), (17, capi.KERNEL_SKINNY), (128, capi.KERNEL_SKINNY)):
        desc = capi.MatmulDesc(bits=4, affine=1, M=M, N=256, k_packed=64, scales_per_row=8, out=4096, in_=4096, scales=4096,
                               weights=4096, biases=4096)
        assert capi.resolve(desc) == want, M
    # above 128 rows: the tile GEMM where its tiles (or their k parts) fill the CUs, this family where they do not
    for M, N, K, want in ((512, 14336, 4096, capi.KERNEL_GEMM), (512, 4096, 4096, capi.KERNEL_SKINNY), (512, 4096, 14336, capi.KERNEL_GEMM),
                          (2048, 4096, 14336, capi.KERNEL_GEMM)):
        desc = capi.MatmulDesc(bits=4, affine=1, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64, out=4096, in_=4096, scales=4096,
                               weights=4096, biases=4096)
        assert capi.resolve(desc) == want, (M, N, K)
    desc = capi.MatmulDesc(bits=3, affine=1, M=300, N=14336, k_packed=384, scales_per_row=64, out=4096, in_=4096, scales=4096,
                           weights=4096, biases=4096)
    assert capi.resolve(desc) == capi.KERNEL_GEMM  # 3-bit rows: the same ladder
    for M, want in ((20, capi.KERNEL_SKINNY), (300, capi.KERNEL_GEMM)):  # 8-bit rows: the same ladder as 4-bit
        desc = capi.MatmulDesc(bits=8, affine=1, M=M, N=14336, k_packed=1024, scales_per_row=64, out=4096, in_=4096, scales=4096,
                               weights=4096, biases=4096)
        assert capi.resolve(desc) == want, M
