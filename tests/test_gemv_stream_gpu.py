"""The dense single-row streaming GEMV (csrc/gemv_stream.hip) against the oracle and against itself.

A row's arithmetic is fixed by its length alone: which wave computes it (the row partition follows the number of
CUs the launch is sized for) and how many loads a wave keeps in flight (the ring) change nothing, so outputs must
be bit-identical across those knobs. Rows longer than two 2048-value passes are shared by 2, 4 or 8 waves whose
partial sums meet in LDS in a fixed order; every such split is covered, with ragged tails in K and N."""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu

# (bits, affine, K, N): 1 pass, 2 passes, 2 / 4 / 8 k parts, ragged K inside a pass and across parts, tiny and ragged N
SHAPES = [(4, True, 2048, 300), (4, True, 4096, 1000), (4, True, 6144, 515), (4, True, 8192, 257), (4, True, 14336, 4096),
          (4, True, 11008, 130), (4, True, 28672, 96), (4, True, 32768, 33), (4, True, 4160, 77), (4, True, 64, 5),
          (4, False, 4096, 513), (4, False, 12320, 64), (4, False, 32, 3), (3, True, 4096, 700), (3, True, 14336, 129),
          (3, True, 192, 9)]


def run(ctx, capi, bits, affine, K, N, x, w, s, b, out_f32=False):
    with Dev(ctx) as d:
        esz = 4 if out_f32 else 2
        out = d.empty(N * esz + 64, fill=0x5A)
        desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=int(out_f32), kernel=capi.KERNEL_GEMV, M=1, N=N,
                               k_packed=K * bits // 32, scales_per_row=K // (64 if affine else 32), out=out, in_=d.put(x),
                               scales=d.put(s), weights=d.put(w), biases=d.put(b) if affine else 0)
        ctx.matmul(desc)
        raw = ctx.download(out, N * esz + 64, np.uint8)
    assert (raw[N * esz:] == 0x5A).all(), "wrote past the output"
    return raw[:N * esz].view(np.float32 if out_f32 else np.float16)


def make(synth, bits, affine, K, N):
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K, bits=bits), synth.scales(N, K, affine=affine)
    return x, w, s, (synth.biases(N, K, s) if affine else None)


@pytest.fixture
def knobs(ctx):
    saved = {k: ctx.get_option(k) for k in ("gemv.stream", "gemv.ring", "num_cus")}
    yield ctx
    for k, v in saved.items():
        ctx.set_option(k, v)


@pytest.mark.parametrize("bits,affine,K,N", SHAPES)
def test_stream_matches_oracle_and_is_knob_invariant(knobs, capi, synth, oracle, bits, affine, K, N):
    ctx = knobs
    x, w, s, b = make(synth, bits, affine, K, N)
    ctx.set_option("gemv.stream", 0)
    y = run(ctx, capi, bits, affine, K, N, x, w, s, b)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, bits, affine, 1, N, K, x, w, s, b, threads=8)[0]
    assert rel_err(y.astype(np.float64), ref, 1e-2) < 1e-2
    assert rel_err(y.astype(np.float64), ref, 1e-3) < 2e-2
    for ring in (1, 3):
        ctx.set_option("gemv.ring", ring)
        assert np.array_equal(run(ctx, capi, bits, affine, K, N, x, w, s, b).view(np.uint16), y.view(np.uint16)), ring
    ctx.set_option("gemv.ring", 0)
    for cus in (16, 100):     # another partition of the rows over waves: same sums (few enough rows per wave at 16)
        ctx.set_option("num_cus", cus)
        assert np.array_equal(run(ctx, capi, bits, affine, K, N, x, w, s, b).view(np.uint16), y.view(np.uint16)), cus
    ctx.set_option("num_cus", 256)
    # the tile-loop kernel it replaced for these dispatches: an independent implementation of the same rows
    ctx.set_option("gemv.stream", 1)
    old = run(ctx, capi, bits, affine, K, N, x, w, s, b)
    assert rel_err(y.astype(np.float64), old.astype(np.float64), 1e-2) < 4e-3


@pytest.mark.parametrize("bits,affine,K", [(4, True, 14336), (4, False, 8192), (3, True, 6144), (4, True, 32768)])
def test_one_hot_through_every_k_part(knobs, capi, synth, oracle, bits, affine, K):
    """x = e_k returns the dequantized weights bit for bit, for k in every pass of every k part and at both ends."""
    knobs.set_option("gemv.stream", 0)
    N = 48
    _, w, s, b = make(synth, bits, affine, K, N)
    w16 = oracle.dequant_matrix(bits, affine, N, K, w, s, b, want="f16")
    ks = sorted(set([0, 31, 32, 2047, 2048, K // 2 - 1, K // 2, K - 2049, K - 33, K - 1] + list(range(1000, K, 4096))))
    for k in ks:
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        y = run(knobs, capi, bits, affine, K, N, x.view(np.uint16), w, s, b)
        assert np.array_equal(y.view(np.uint16), w16[:, k]), k


def test_f32_output_and_lm_head_rows(knobs, capi, synth, oracle):
    """f32 stores (the LM head's form) and a row count that gives every wave dozens of rows (the deeper ring)."""
    knobs.set_option("gemv.stream", 0)
    K, N = 2048, 140000
    x, w, s, b = make(synth, 4, True, K, N)
    y = run(knobs, capi, 4, True, K, N, x, w, s, b, out_f32=True)
    rows = np.r_[0:64, N // 2:N // 2 + 64, N - 64:N]
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, 1, len(rows), K, x, w[rows], s[rows], b[rows], threads=8)[0]
    assert rel_err(y[rows].astype(np.float64), ref, 1e-3) < 1e-4   # f32 stores: no f16 rounding of the output
    y16 = run(knobs, capi, 4, True, K, N, x, w, s, b)
    assert np.array_equal(y16, y.astype(np.float16))
