"""GPU parity of the streaming GEMV against the CPU oracle, through the C ABI.

Shapes follow the reference's kernel tests (tests/kernels/run.mjs:1080-1215:
N=8, K in {512, 768, 1024, 1408}, symmetric / affine / q3, f16 / f32 out) on
the reference's own seeded vectors, then the benchmark configurations.
Bars: |y-ref|/(|ref|+1e-2) < 1e-2 against the fp32-accumulated oracle (the
contract), and the reference test's own |y-ref|/(|ref|+1e-3) < 2e-2.
"""
import numpy as np
import pytest

from .util import Dev, f16, rel_err

pytestmark = pytest.mark.gpu


def run_dense(ctx, capi, bits, affine, M, N, K, x, w, s, b, out_f32=False, kernel=0, prefill=0x5A):
    with Dev(ctx) as d:
        esz = 4 if out_f32 else 2
        out = d.empty(M * N * esz + 64, fill=prefill)
        desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=int(out_f32), kernel=kernel, M=M, N=N,
                               k_packed=K * bits // 32, scales_per_row=K // (64 if affine else 32),
                               out=out, in_=d.put(x), scales=d.put(s), weights=d.put(w),
                               biases=d.put(b) if affine else 0)
        ctx.matmul(desc)
        raw = ctx.download(out, M * N * esz + 64, np.uint8)
    assert np.all(raw[M * N * esz:] == prefill), "wrote past the output"
    y = raw[:M * N * esz].view(np.float32 if out_f32 else np.float16).astype(np.float64)
    return y.reshape(M, N)


def check(y, oracle, bits, affine, M, N, K, x, w, s, b, out_f32=False):
    ref32 = oracle.gemm(oracle.MODE_FORMULA_F32, bits, affine, M, N, K, x, w, s, b, threads=8)
    ref64 = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, M, N, K, x, w, s, b, threads=8)
    if not out_f32:  # the reference rounds its expectation to f16 too (run.mjs:134)
        ref32r = ref32.astype(np.float16).astype(np.float64)
    else:
        ref32r = ref32
    e_contract = rel_err(y, ref32r, 1e-2)
    e_ref_test = rel_err(y, ref64, 1e-3)
    assert e_contract < 1e-2, e_contract
    assert e_ref_test < 2e-2, e_ref_test
    return e_contract, e_ref_test


@pytest.mark.parametrize("K", [512, 768, 1024, 1408])
@pytest.mark.parametrize("fmt", ["sym", "affine", "q3"])
@pytest.mark.parametrize("out_f32", [False, True])
def test_reference_seeded_vectors(ctx, capi, oracle, K, fmt, out_f32):
    """The reference's makeInt4MatmulTest inputs (rng(1), N=8), regenerated bit for bit."""
    if fmt == "q3" and K % 64:
        pytest.skip("q3 needs K % 64 == 0")
    affine, q3 = fmt != "sym", fmt == "q3"
    bits = 3 if q3 else 4
    if K % (64 if affine else 32):
        pytest.skip("K not a multiple of the group")
    x, s, b, w = oracle.reference_gemv_case(8, K, affine, q3)
    y = run_dense(ctx, capi, bits, affine, 1, 8, K, x, w, s, b, out_f32=out_f32)
    # against the reference test's own factored f64 arithmetic as well
    js = oracle.gemm(oracle.MODE_JS, bits, affine, 1, 8, K, x, w, s, b)
    assert rel_err(y, js, 1e-3) < 2e-2
    check(y, oracle, bits, affine, 1, 8, K, x, w, s, b, out_f32)


CONFIG_SHAPES = [
    ("cfg1", 2048, 8192), ("cfg2a", 4096, 14336), ("cfg2b", 14336, 4096), ("cfg2c", 4096, 6144),
]


@pytest.mark.parametrize("name,K,N", CONFIG_SHAPES)
@pytest.mark.parametrize("regime", ["A", "B"])
def test_int4_affine_configs(ctx, capi, synth, oracle, name, K, N, regime):
    x = synth.activations(1, K)
    w = synth.packed_weights(N, K)
    s = synth.scales(N, K)
    b = synth.biases(N, K, s, regime)
    y = run_dense(ctx, capi, 4, True, 1, N, K, x, w, s, b)
    e = check(y, oracle, 4, True, 1, N, K, x, w, s, b)
    print(name, regime, "rel err (contract, ref-test metric):", e)


@pytest.mark.parametrize("N", [1, 3, 5, 17, 250])
def test_ragged_rows(ctx, capi, synth, oracle, N):
    K = 4096
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    y = run_dense(ctx, capi, 4, True, 1, N, K, x, w, s, b)
    check(y, oracle, 4, True, 1, N, K, x, w, s, b)


def test_one_hot_pins_dequant(ctx, capi, synth, oracle):
    """x = e_k makes y[n] the dequantized weight itself: f16(fl32(q*s+b)) bit for bit."""
    K, N = 4096, 64
    w, s = synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    w16 = oracle.dequant_matrix(4, True, N, K, w, s, b, want="f16")
    for k in (0, 7, 8, 31, 32, 63, 64, 2047, 2048, 4095):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        y = run_dense(ctx, capi, 4, True, 1, N, K, x.view(np.uint16), w, s, b)
        assert np.array_equal(y[0].astype(np.float16).view(np.uint16), w16[:, k]), k


def test_int3_config5_m1(ctx, capi, synth, oracle):
    K, N = 4096, 14336
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K, bits=3), synth.scales(N, K)
    b = synth.biases(N, K, s)
    y = run_dense(ctx, capi, 3, True, 1, N, K, x, w, s, b)
    print("int3 rel err:", check(y, oracle, 3, True, 1, N, K, x, w, s, b))


def test_seeded_random_shapes(ctx, capi, synth, oracle):
    """Forty seeded GEMV shapes across the formats: ragged N, K from one scale group up, dense and f32 output."""
    rng = np.random.default_rng(977)
    formats = [(4, True), (4, False), (3, True), (8, True)]
    for case in range(40):
        bits, affine = formats[case % 4]
        group = 64 if affine else 32
        N = int(rng.integers(1, 400))
        K = group * int(rng.choice([1, 2, 3, 7, 8, 16, 31, 64, 100, 224]))
        out_f32 = int(case % 5 == 0)
        x = synth.activations(1, K)
        w = synth.packed_weights(N, K, bits=bits)
        s = synth.scales(N, K, affine=affine)
        b = synth.biases(N, K, s, "A") if affine else None
        esz = 4 if out_f32 else 2
        with Dev(ctx) as d:
            out = d.empty(N * esz + 16, fill=0)
            desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=out_f32, M=1, N=N, k_packed=K * bits // 32,
                                   scales_per_row=K // group, out=out, in_=d.put(x), scales=d.put(s), weights=d.put(w),
                                   biases=d.put(b) if affine else 0)
            ctx.matmul(desc)
            raw = ctx.download(out, N * esz + 16, np.uint8)
        y = raw[:N * esz].view(np.float32 if out_f32 else np.float16).astype(np.float64)
        ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, 1, N, K, x, w, s, b, threads=8)[0]
        err = rel_err(y, ref, 1e-2)
        assert err < 1e-2, (case, bits, affine, N, K, err)
        assert not raw[N * esz:].any(), "wrote past N"


@pytest.mark.parametrize("regime", ["A", "B"])
def test_gate_sees_a_wrong_kernel(ctx, capi, synth, oracle, regime):
    """configs[0] through the GPU against references computed from deliberately wrong inputs (the mutations of
    scripts/mutation-gate.mjs): the GPU result passes the gate against the right reference and FAILS it against a
    reference with a shifted scale group, a dropped bias or a swapped nibble order — the 1e-2 bar with its 1e-2
    floor in the denominator is tight enough to tell them apart."""
    from .util import mutations
    K, N = 2048, 8192
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s, regime)
    y = run_dense(ctx, capi, 4, True, 1, N, K, x, w, s, b)
    check(y, oracle, 4, True, 1, N, K, x, w, s, b)
    for name, (mw, ms, mb) in mutations(w, s, b).items():
        wrong = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, mw, ms, mb, threads=8)
        assert rel_err(y, wrong, 1e-2) > 10 * 1e-2, name
        assert np.median(np.abs(y - wrong) / (np.abs(wrong) + 1e-2)) > 1e-2, name


def test_long_rows_k32768(ctx, capi, synth, oracle):
    """K = 32768: 68 KB of staged activations, past the 64 KB a launch gets without asking for more."""
    K, N = 32768, 96
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    y = run_dense(ctx, capi, 4, True, 1, N, K, x, w, s, b, kernel=capi.KERNEL_GEMV)
    check(y, oracle, 4, True, 1, N, K, x, w, s, b)
