"""What the arithmetic itself fixes, checked on every kernel family without the oracle: closed forms and symmetries of
    y[m,n] = sum_g ( s[n,g] * sum_{k in g} x[m,k] q[n,k]  +  b[n,g] * sum_{k in g} x[m,k] )
(src/compiler/shaders/int4_matmul.gen.ts:78-84, :401-406). Each one fails for a plausible mistake that a tolerance
against a reference could forgive: a dropped bias term, a scale taken from the neighbouring group, a row written to
the wrong place, a lane's partial sum left out.

  * x = 0                      -> y = 0, bit for bit
  * s = 0                      -> y[m,n] = sum_g b[n,g] * sum(x[m, group g]): the weights do not matter
  * q = c for every value      -> y[m,n] = sum_g (c s[n,g] + b[n,g]) * sum(x[m, group g])
  * weight rows permuted       -> output columns permuted, bit for bit (a row's arithmetic does not depend on where the row sits)
  * activation rows permuted   -> output rows permuted, bit for bit (inside one family and tile shape)
"""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu

K, N = 1024, 520          # 16 affine groups; N off every tile width (4, 32, 64, 128)
FAMILIES = [("gemv", 1), ("rows", 6), ("skinny", 20), ("skinny", 40), ("skinny", 150), ("gemm", 150), ("gemm", 300)]


def run(ctx, capi, family, M, x, w, s, b, bits=4):
    kernel = {"gemv": capi.KERNEL_GEMV, "rows": capi.KERNEL_ROWS, "skinny": capi.KERNEL_SKINNY, "gemm": capi.KERNEL_GEMM}[family]
    with Dev(ctx) as d:
        out = d.empty(M * N * 2, fill=0x5A)
        ctx.matmul(capi.MatmulDesc(bits=bits, affine=1, kernel=kernel, M=M, N=N, k_packed=K * bits // 32, scales_per_row=K // 64,
                                   out=out, in_=d.put(x), scales=d.put(s), weights=d.put(w), biases=d.put(b)))
        return ctx.download(out, M * N * 2, np.uint16).reshape(M, N)


def operands(synth, M, bits=4):
    x = synth.activations(M, K, salt=31)
    w = synth.packed_weights(N, K, bits=bits, salt=31)
    s = synth.scales(N, K, salt=31)
    b = synth.biases(N, K, s, "A", salt=31)
    return x, w, s, b


def group_sums(x):
    return x.view(np.float16).astype(np.float64).reshape(x.shape[0], K // 64, 64).sum(axis=2)   # [M, G]


@pytest.mark.parametrize("family,M", FAMILIES)
def test_zero_activations_give_zero(ctx, capi, synth, family, M):
    _, w, s, b = operands(synth, M)
    y = run(ctx, capi, family, M, np.zeros((M, K), np.uint16), w, s, b)
    assert not (y & 0x7FFF).any()   # +0 or -0


@pytest.mark.parametrize("family,M", FAMILIES)
def test_zero_scales_leave_the_bias_term(ctx, capi, synth, family, M):
    x, w, s, b = operands(synth, M)
    y = run(ctx, capi, family, M, x, w, np.zeros_like(s), b).view(np.float16).astype(np.float64)
    want = group_sums(x) @ b.view(np.float16).astype(np.float64).T          # [M, N]
    assert rel_err(y, want, 1e-2) < 2e-3


@pytest.mark.parametrize("family,M", FAMILIES)
@pytest.mark.parametrize("c", [0, 1, 9, 15])
def test_constant_nibbles_closed_form(ctx, capi, synth, family, M, c):
    x, _, s, b = operands(synth, M)
    w = np.full((N, K // 8), c * 0x11111111, np.uint32)
    y = run(ctx, capi, family, M, x, w, s, b).view(np.float16).astype(np.float64)
    coeff = c * s.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)   # [N, G]
    want = group_sums(x) @ coeff.T
    assert rel_err(y, want, 1e-2) < 2e-3


@pytest.mark.parametrize("family,M", FAMILIES)
def test_weight_rows_permuted_permute_the_columns(ctx, capi, synth, family, M):
    x, w, s, b = operands(synth, M)
    perm = np.random.default_rng(5).permutation(N)
    y = run(ctx, capi, family, M, x, w, s, b)
    yp = run(ctx, capi, family, M, x, w[perm], s[perm], b[perm])
    assert np.array_equal(yp, y[:, perm])


@pytest.mark.parametrize("family,M", [f for f in FAMILIES if f[1] > 1])
def test_activation_rows_permuted_permute_the_rows(ctx, capi, synth, family, M):
    x, w, s, b = operands(synth, M)
    perm = np.random.default_rng(6).permutation(M)
    y = run(ctx, capi, family, M, x, w, s, b)
    yp = run(ctx, capi, family, M, np.ascontiguousarray(x[perm]), w, s, b)
    assert np.array_equal(yp, y[perm])


@pytest.mark.parametrize("family,M", [("gemv", 1), ("rows", 6), ("skinny", 40), ("gemm", 150)])
def test_three_bit_constant_values_closed_form(ctx, capi, synth, family, M):
    """3-bit rows: every value 5 is the bitstream of 101 repeated, whatever the word boundaries do to it."""
    x, _, s, b = operands(synth, M, bits=3)
    bits = np.tile(np.array([1, 0, 1], np.uint8), K)                       # value k at bits [3k, 3k+3), LSB first
    row = np.packbits(bits, bitorder="little").view(np.uint32)
    w = np.tile(row, (N, 1))
    y = run(ctx, capi, family, M, x, w, s, b, bits=3).view(np.float16).astype(np.float64)
    coeff = 5 * s.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)
    want = group_sums(x) @ coeff.T
    assert rel_err(y, want, 1e-2) < 2e-3
