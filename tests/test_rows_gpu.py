"""GPU parity of the row-group GEMV (family 'rows', 1 <= M <= 16; the default for 2 <= M <= 16).

Cases follow the reference's small-batch checks (tests/kernels/compile-qwen35.mjs:963-1152: M=6 N=64 at K=2560;
the fixed-M=4 bench primitive of src/compiler/shaders/int4_matmul.gen.ts:465-516) in every format the reference
ships for the dispatch, plus ragged N, K that is not a whole pass, K long enough to be dealt to several
workgroups, and configs[4] (3-bit, M=8, K=4096, N=14336).
Bars: |y-ref|/(|ref|+1e-2) < 1e-2 against the from-the-formula f64 oracle, rows past M untouched, a row's result
independent of how many rows travel with it (bit for bit, across the 4-, 8-, 12- and 16-row builds), one-hot rows
bit-exact.
"""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def run(ctx, capi, bits, affine, M, CAP, N, K, A, w, s, b, kernel=None, out_f32=0):
    esz = 4 if out_f32 else 2
    with Dev(ctx) as d:
        out = d.empty(CAP * N * esz, fill=0)
        desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=out_f32, kernel=capi.KERNEL_ROWS if kernel is None else kernel,
                               M=M, N=N, k_packed=K * bits // 32, scales_per_row=K // (64 if affine else 32), out=out,
                               in_=d.put(A), scales=d.put(s), weights=d.put(w), biases=d.put(b) if affine else 0)
        ctx.matmul(desc)
        return ctx.download(out, CAP * N * esz, np.uint32 if out_f32 else np.uint16).reshape(CAP, N)


def make(synth, bits, affine, CAP, N, K, regime="A"):
    A = synth.activations(CAP, K)
    w = synth.packed_weights(N, K, bits=bits)
    s = synth.scales(N, K, affine=affine)
    b = synth.biases(N, K, s, regime) if affine else None
    return A, w, s, b


FORMATS = [(4, True), (4, False), (3, True), (8, True)]
# M, CAP, N, K
CASES = [(1, 4, 64, 2560), (2, 8, 64, 2560), (4, 4, 256, 1024), (6, 8, 64, 2560), (8, 16, 200, 2560), (9, 16, 33, 192),
         (13, 16, 96, 128), (16, 16, 136, 64), (3, 16, 7, 4096), (5, 8, 1000, 512)]


@pytest.mark.parametrize("M,CAP,N,K", CASES)
@pytest.mark.parametrize("bits,affine", FORMATS)
def test_ragged_rows(ctx, capi, synth, oracle, M, CAP, N, K, bits, affine):
    A, w, s, b = make(synth, bits, affine, CAP, N, K)
    got = run(ctx, capi, bits, affine, M, CAP, N, K, A, w, s, b)
    gotcap = run(ctx, capi, bits, affine, CAP, CAP, N, K, A, w, s, b)
    y = got[:M].view(np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, A, w, s, b, threads=8)
    assert rel_err(y, ref, 1e-2) < 1e-2
    assert rel_err(y, ref, 1e-3) < 2e-2
    assert not got[M:].any(), "rows past M were written"
    assert np.array_equal(got[:M], gotcap[:M]), "M-variance"


@pytest.mark.parametrize("bits,affine", FORMATS)
def test_long_k_is_dealt_to_several_workgroups(ctx, capi, synth, oracle, bits, affine):
    """K = 14336 does not fit the staged-activation budget: four k ranges, partial sums added in range order."""
    M, N, K = 5, 264, 14336
    A, w, s, b = make(synth, bits, affine, 16, N, K)
    got = run(ctx, capi, bits, affine, M, 16, N, K, A, w, s, b)
    got16 = run(ctx, capi, bits, affine, 16, 16, N, K, A, w, s, b)
    got32 = run(ctx, capi, bits, affine, M, 16, N, K, A, w, s, b, out_f32=1)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got[:M].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert rel_err(got32[:M].view(np.float32).astype(np.float64), ref, 1.0) < (1e-4 if bits == 8 else 2e-5)
    assert not got[M:].any() and not got32[M:].any()
    assert np.array_equal(got[:M], got16[:M]), "M-variance"


def test_split_needs_groups_of_four_outputs(ctx, capi):
    desc = capi.MatmulDesc(bits=4, affine=1, M=4, N=250, k_packed=14336 // 8, scales_per_row=14336 // 64, out=4096, in_=4096,
                           scales=4096, weights=4096, biases=4096, kernel=capi.KERNEL_ROWS)
    rc, why = capi.validate(desc)
    assert rc == capi.E_UNSUPPORTED and "rows" in why
    with pytest.raises(capi.ZtvmError, match="rows"):
        capi.resolve(desc)
    desc.kernel = capi.KERNEL_AUTO
    assert capi.validate(desc)[0] == 0
    assert capi.resolve(desc) == capi.KERNEL_SKINNY


def test_one_hot_pins_streamed_weights(ctx, capi, synth, oracle):
    """A = rows of the identity: Y[m,n] is the dequantized weight f16(fl32(q*s+b)) of W[n,k_m], bit for bit."""
    N, K = 160, 256
    ks = np.array([0, 1, 3, 4, 7, 8, 15, 31, 32, 33, 63, 64, 65, 127, 128, 255], np.int64)
    A = np.zeros((16, K), np.float16)
    A[np.arange(16), ks] = 1.0
    for bits, affine in FORMATS:
        _, w, s, b = make(synth, bits, affine, 1, N, K)
        got = run(ctx, capi, bits, affine, 16, 16, N, K, A.view(np.uint16), w, s, b)
        w16 = oracle.dequant_matrix(bits, affine, N, K, w, s, b, want="f16")
        assert np.array_equal(got, w16[:, ks].T), (bits, affine)


@pytest.mark.parametrize("bits,affine", FORMATS)
def test_families_agree(ctx, capi, synth, bits, affine):
    """The per-row GEMV and the row-group kernel follow the same factored arithmetic: the same f16 results up to one
    rounding step on a few outputs (the order of the f32 sums inside a chunk differs)."""
    M, N, K = 7, 256, 1024
    A, w, s, b = make(synth, bits, affine, M, N, K)
    g = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b, kernel=capi.KERNEL_GEMV).view(np.float16).astype(np.float64)
    r = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b).view(np.float16).astype(np.float64)
    assert rel_err(r, g, 1e-2) < 2e-3


@pytest.mark.parametrize("M", [1, 8])
def test_config5_int3(ctx, capi, synth, oracle, M):
    """configs[4]: 3-bit weights, K=4096, N=14336, against the formula; M=8 takes this family by default."""
    K, N = 4096, 14336
    A, w, s, b = make(synth, 3, True, M, N, K)
    got = run(ctx, capi, 3, True, M, M, N, K, A, w, s, b, kernel=capi.KERNEL_ROWS if M == 1 else capi.KERNEL_AUTO)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 3, True, M, N, K, A, w, s, b, threads=8)
    assert rel_err(got.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2


def test_auto_routing(capi):
    for M, want in ((1, capi.KERNEL_GEMV), (2, capi.KERNEL_ROWS), (12, capi.KERNEL_ROWS), (13, capi.KERNEL_SKINNY),
                    (128, capi.KERNEL_SKINNY)):
        desc = capi.MatmulDesc(bits=4, affine=1, M=M, N=256, k_packed=64, scales_per_row=8, out=4096, in_=4096, scales=4096,
                               weights=4096, biases=4096)
        assert capi.resolve(desc) == want, M
    desc = capi.MatmulDesc(bits=4, affine=1, M=17, N=256, k_packed=64, scales_per_row=8, out=4096, in_=4096, scales=4096,
                           weights=4096, biases=4096, kernel=capi.KERNEL_ROWS)
    with pytest.raises(capi.ZtvmError, match="rows"):
        capi.resolve(desc)


def test_seeded_random_shapes(ctx, capi, synth, oracle):
    """Forty seeded shapes across the formats: ragged N, K from one scale group to several k ranges, every M."""
    rng = np.random.default_rng(20240607)
    for case in range(40):
        bits, affine = FORMATS[case % len(FORMATS)]
        group = 64 if affine else 32
        M = int(rng.integers(1, 17))
        N = int(rng.integers(1, 300))
        K = group * int(rng.choice([1, 2, 3, 5, 8, 17, 40, 64, 65, 100, 130]))
        if K > 4096 and N % 4:
            N += 4 - N % 4          # a split k range needs groups of four outputs
        A, w, s, b = make(synth, bits, affine, M, N, K)
        got = run(ctx, capi, bits, affine, M, M, N, K, A, w, s, b)
        ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, A, w, s, b, threads=8)
        err = rel_err(got.view(np.float16).astype(np.float64), ref, 1e-2)
        assert err < 1e-2, (case, bits, affine, M, N, K, err)
