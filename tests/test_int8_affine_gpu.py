"""GPU parity of the 8-bit MLX-affine twins of the matmul family (w = s*q + b, group 64, an unsigned byte per
value, four per word, K_PACKED = K/4) through the same descriptor with bits = 8.

Shapes and bars of the reference's own test (tests/kernels/int8-affine.mjs:84-148): matvec K=1024 N=256, batched
M=31 of CAP=64 rows; references written from the FORMULA (per-element w = s*q + b in float64), never from the
kernel's factored form; max |y-ref|/(|ref|+1e-2) < 1e-2; rows past M untouched; results independent of M.
"""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def make8(synth, N, K, M, experts=None, regime="A"):
    w = synth.packed_weights(N, K, bits=8, experts=experts)
    s = synth.scales(N, K, experts=experts, lo=0.01, hi=0.06)
    b = synth.biases(N, K, s, regime, experts=experts)
    return synth.activations(M, K), w, s, b


def desc8(capi, M, N, K, out, x, w, s, b, **kw):
    return capi.MatmulDesc(bits=8, affine=1, M=M, N=N, k_packed=K // 4, scales_per_row=K // 64, out=out, in_=x, weights=w,
                           scales=s, biases=b, **kw)


@pytest.mark.parametrize("N,K", [(256, 1024), (100, 64), (33, 4096), (14336, 4096), (7, 192), (64, 14336)])
def test_matvec(ctx, capi, synth, oracle, N, K):
    x, w, s, b = make8(synth, N, K, 1)
    with Dev(ctx) as d:
        out = d.empty(N * 2 + 32, fill=0)
        ctx.matmul(desc8(capi, 1, N, K, out, d.put(x), d.put(w), d.put(s), d.put(b)))
        got = ctx.download(out, N * 2 + 32, np.uint16)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 8, True, 1, N, K, x, w, s, b, threads=8)[0]
    assert rel_err(got[:N].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert not got[N:].any()


def test_batched_ragged_and_m_invariant(ctx, capi, synth, oracle):
    K, N, M, CAP = 1024, 256, 31, 64
    x, w, s, b = make8(synth, N, K, CAP)
    with Dev(ctx) as d:
        X, W, S, B = d.put(x), d.put(w), d.put(s), d.put(b)
        outs = []
        for m in (M, CAP):
            out = d.empty(CAP * N * 2, fill=0)
            ctx.matmul(desc8(capi, m, N, K, out, X, W, S, B))
            outs.append(ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N))
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 8, True, M, N, K, x, w, s, b, threads=8)
    assert rel_err(outs[0][:M].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert not outs[0][M:].any(), "rows past M were written"
    assert np.array_equal(outs[0][:M], outs[1][:M]), "M-variance"


@pytest.mark.parametrize("M,CAP,N,K", [(6, 8, 64, 2560), (47, 64, 200, 1024), (130, 256, 136, 512), (300, 320, 264, 1024),
                                       (257, 260, 136, 256), (511, 512, 392, 640)])
def test_tile_gemm_family(ctx, capi, synth, oracle, M, CAP, N, K):
    """The 8-bit form of the tile GEMM (bytes staged as exact f16 integers, two words per 16-byte chunk) against the
    formula, at every tile height, with partial last tiles, ragged N, and rows past M untouched; a row does not
    depend on how many rows follow it."""
    x, w, s, b = make8(synth, N, K, CAP)
    with Dev(ctx) as d:
        X, W, S, B = d.put(x), d.put(w), d.put(s), d.put(b)
        outs = []
        for m in (M, CAP):
            out = d.empty(CAP * N * 2, fill=0x5A)
            ctx.matmul(desc8(capi, m, N, K, out, X, W, S, B, kernel=capi.KERNEL_GEMM))
            outs.append(ctx.download(out, CAP * N * 2, np.uint16).reshape(CAP, N))
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 8, True, M, N, K, x, w, s, b, threads=8)
    assert rel_err(outs[0][:M].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2
    assert (outs[0][M:] == 0x5A5A).all(), "rows past M were written"
    assert np.array_equal(outs[0][:M], outs[1][:M]), "M-variance"


def test_tile_gemm_one_hot_is_the_dequantized_weight(ctx, capi, synth, oracle):
    """A = rows of the identity through the 8-bit tile GEMM: Y[m, n] = f16(fl32(q*s + b)) of W[n, k_m], bit for bit."""
    N, K = 160, 256
    _, w, s, b = make8(synth, N, K, 1)
    ks = np.array([0, 1, 2, 3, 4, 7, 8, 15, 31, 32, 33, 63, 64, 65, 127, 128, 191, 200, 254, 255] * 4, np.int64)[:64]
    A = np.zeros((64, K), np.float16)
    A[np.arange(64), ks] = 1.0
    with Dev(ctx) as d:
        out = d.empty(64 * N * 2, fill=0)
        ctx.matmul(desc8(capi, 64, N, K, out, d.put(A), d.put(w), d.put(s), d.put(b), kernel=capi.KERNEL_GEMM))
        got = ctx.download(out, 64 * N * 2, np.uint16).reshape(64, N)
    w16 = oracle.dequant_matrix(8, True, N, K, w, s, b, want="f16")
    assert np.array_equal(got, w16[:, ks].T)


def test_dequant_and_one_hot_are_bit_exact(ctx, capi, synth, oracle):
    N, K = 96, 256
    _, w, s, b = make8(synth, N, K, 1, regime="B")
    want16 = oracle.dequant_matrix(8, True, N, K, w, s, b, want="f16")
    want32 = oracle.dequant_matrix(8, True, N, K, w, s, b, want="f32")
    ks = np.array([0, 1, 2, 3, 4, 5, 31, 32, 63, 64, 65, 127, 128, 200, 254, 255])
    A = np.zeros((len(ks), K), np.float16)
    A[np.arange(len(ks)), ks] = 1.0
    with Dev(ctx) as d:
        W, S, B = d.put(w), d.put(s), d.put(b)
        o16, o32 = d.empty(N * K * 2, fill=0), d.empty(N * K * 4, fill=0)
        ctx.dequant(desc8(capi, 1, N, K, o16, 0, W, S, B))
        ctx.dequant(desc8(capi, 1, N, K, o32, 0, W, S, B, out_f32=1))
        assert np.array_equal(ctx.download(o16, N * K * 2, np.uint16).reshape(N, K), want16)
        assert np.array_equal(ctx.download(o32, N * K * 4, np.float32).reshape(N, K), want32)
        out = d.empty(len(ks) * N * 2, fill=0)
        ctx.matmul(desc8(capi, len(ks), N, K, out, d.put(A), W, S, B))
        got = ctx.download(out, len(ks) * N * 2, np.uint16).reshape(len(ks), N)
    assert np.array_equal(got, want16[:, ks].T), "a one-hot row returns the dequantized weight itself"


def test_moe_pairs_equal_dense_rows(ctx, capi, synth, oracle):
    E, N, K, tokens, S = 5, 128, 512, 3, 2
    x, w, s, b = make8(synth, N, K, tokens, experts=E)
    ids = synth.topk_ids(tokens, S, E)
    with Dev(ctx) as d:
        X, W, Sc, B, IDS = d.put(x), d.put(w), d.put(s), d.put(b), d.put(ids)
        out = d.empty(tokens * S * N * 2, fill=0)
        ctx.matmul(desc8(capi, 1, N, K, out, X, W, Sc, B, slots=S, tokens=tokens, in_slot_stride=0, in_tok_stride=K,
                         out_slot_stride=N, out_tok_stride=S * N, ids=IDS, ids_stride=S, experts=E))
        got = ctx.download(out, tokens * S * N * 2, np.uint16).reshape(tokens, S, N)
        for t in range(tokens):
            for sl in range(S):
                e = int(ids[t, sl])
                one = d.empty(N * 2, fill=0)
                ctx.matmul(desc8(capi, 1, N, K, one, X + t * K * 2, W + e * N * (K // 4) * 4, Sc + e * N * (K // 64) * 2,
                                 B + e * N * (K // 64) * 2))
                assert np.array_equal(got[t, sl], ctx.download(one, N * 2, np.uint16)), (t, sl)
    ref = oracle.gemm(oracle.MODE_FORMULA_F64, 8, True, 1, N, K, x[0:1], w[ids[0, 0]], s[ids[0, 0]], b[ids[0, 0]])[0]
    assert rel_err(got[0, 0].view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2


def test_rules_and_routing(capi):
    ok = capi.MatmulDesc(bits=8, affine=1, M=1, N=64, k_packed=256, scales_per_row=16, out=4096, in_=4096, scales=4096,
                         weights=4096, biases=4096)
    assert capi.validate(ok)[0] == 0 and capi.resolve(ok) == capi.KERNEL_GEMV
    ok.M = 100
    assert capi.resolve(ok) == capi.KERNEL_SKINNY        # the weight-streaming kernel up to 128 rows
    ok.M = 300
    assert capi.resolve(ok) == capi.KERNEL_SKINNY        # one column tile: the tile GEMM would run on three CUs
    big = capi.MatmulDesc(bits=8, affine=1, M=300, N=14336, k_packed=1024, scales_per_row=64, out=4096, in_=4096, scales=4096,
                          weights=4096, biases=4096)
    assert capi.resolve(big) == capi.KERNEL_GEMM         # the tile GEMM above 128 rows where its tiles fill the CUs
    ok.kernel = capi.KERNEL_GEMM
    assert capi.validate(ok)[0] == 0
    ok.out_f32 = 1
    assert capi.validate(ok)[0] == capi.E_UNSUPPORTED    # f32 output is the streaming kernel's
    ok.out_f32, ok.kernel = 0, capi.KERNEL_AUTO
    sym = capi.MatmulDesc(bits=8, affine=0, M=1, N=64, k_packed=256, scales_per_row=32, out=4096, in_=4096, scales=4096, weights=4096)
    rc, why = capi.validate(sym)
    assert rc == capi.E_INVALID and "8-bit requires affine" in why
    bad = capi.MatmulDesc(bits=8, affine=1, M=1, N=64, k_packed=256, scales_per_row=32, out=4096, in_=4096, scales=4096,
                          weights=4096, biases=4096)
    assert capi.validate(bad)[0] == capi.E_INVALID      # SCALES_PER_ROW of the 4-bit reading of the same words
