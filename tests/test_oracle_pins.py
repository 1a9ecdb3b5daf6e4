"""Pins of the CPU oracle (no GPU): every oracle function is checked against an
independent second formulation (numpy, pure-Python integers, closed forms,
brute force) chosen so that a dropped term, a wrong shift or a transposed
operand fails at least one test."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def fx():
    with open(os.path.join(HERE, "golden", "format_vectors.json")) as fh:
        return json.load(fh)


# ---- f16 ---------------------------------------------------------------------

def test_f16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_roundtrip_and_rne(oracle, fx):
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    assert np.array_equal(oracle.f32_to_f16_bits(f[ok]), bits[ok])
    # ties, subnormals, overflow from the committed fixture (numpy float16 cast = IEEE RNE)
    fin = np.array(fx["f32_in_bits"], np.uint32).view(np.float32)
    assert oracle.f32_to_f16_bits(fin).tolist() == fx["f16_out_bits"]
    # a dense random sweep against numpy's cast, including values between f16 neighbours
    g = np.random.default_rng(7)
    r = (g.standard_normal(400000) * np.exp2(g.integers(-30, 18, 400000))).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.f32_to_f16_bits(r), r.astype(np.float16).view(np.uint16))


# ---- rng -----------------------------------------------------------------------

def test_mulberry32_matches_python_integers(oracle, fx):
    assert oracle.mulberry32(1, 16).tolist() == fx["mulberry32_seed1"]
    assert oracle.mulberry32(35, 8).tolist() == fx["mulberry32_seed35"]


def test_reference_case_generator_order(oracle, fx):
    """input, scales, biases, then weights are drawn from ONE stream in that order (run.mjs:83-103)."""
    K, N = 512, 8
    x, s, b, w = oracle.reference_gemv_case(N, K, True, False)
    r = oracle.mulberry32(1, K + 2 * N * (K // 64) + N * (K // 8))
    with np.errstate(over="ignore"):
        assert np.array_equal(x, (r[:K] * 2 - 1).astype(np.float32).astype(np.float16).view(np.uint16))
        o = K
        assert np.array_equal(s.ravel(), (r[o:o + 64] * 0.05 + 0.01).astype(np.float32).astype(np.float16).view(np.uint16))
        o += 64
        assert np.array_equal(b.ravel(), (r[o:o + 64] * 0.1 - 0.05).astype(np.float32).astype(np.float16).view(np.uint16))
        o += 64
    assert np.array_equal(w.ravel(), np.floor(r[o:] * 0xFFFFFFFF).astype(np.uint32))


# ---- unpack ----------------------------------------------------------------------

def test_unpack4_against_bytewise_fixture(oracle, fx):
    for words, vals in zip(fx["q4_words"], fx["q4_values"]):
        row = np.array(words, np.uint32)
        assert [oracle.unpack(4, row, k) for k in range(len(vals))] == vals


def test_unpack4_all_values_all_positions(oracle):
    for pos in range(8):
        for q in range(16):
            row = np.array([0xFFFFFFFF ^ (15 << (4 * pos)) | (q << (4 * pos)), 0], np.uint32)
            assert oracle.unpack(4, row, pos) == q


def test_unpack3_against_unpackbits_fixture(oracle, fx):
    for words, vals in zip(fx["q3_words"], fx["q3_values"]):
        row = np.array(words + [0], np.uint32)
        got = [oracle.unpack(3, row, k) for k in range(len(vals))]
        assert got == vals
        # the kernel's 24-bit window form must agree for every block (shifts 0,24,16,8)
        assert [oracle.unpack(3, row, k, window=True) for k in range(len(vals))] == vals


def test_unpack3_straddling_values(oracle):
    """Values 10 and 21 of every 32-value chunk cross a word boundary (bits 30-32, 63-65)."""
    for k in (10, 21, 42, 53):
        for q in range(8):
            vals = np.zeros(64, np.uint8)
            vals[k] = q
            words = oracle.pack(3, vals)
            assert oracle.unpack(3, np.append(words, 0).astype(np.uint32), k) == q
            # packer cross-check with numpy bits
            bits = np.zeros(192, np.uint8)
            bits[3 * k:3 * k + 3] = [(q >> i) & 1 for i in range(3)]
            assert np.array_equal(np.packbits(bits, bitorder="little").view("<u4"), words)


def test_pack_unpack_roundtrip(oracle):
    g = np.random.default_rng(3)
    for bits in (3, 4):
        vals = g.integers(0, 1 << bits, 256).astype(np.uint8)
        words = np.append(oracle.pack(bits, vals), 0).astype(np.uint32)
        assert [oracle.unpack(bits, words, k) for k in range(256)] == vals.tolist()


# ---- dequant ------------------------------------------------------------------------

def test_dequant_bruteforce_all_scales(oracle):
    """All 16 q x every finite f16 scale x sampled biases, against numpy float32 arithmetic
    (q*s is exact in f32, the add rounds once) and numpy's f16 cast."""
    s_bits = np.array([h for h in range(65536) if (h >> 10) & 31 != 31], np.uint16)
    N, K = s_bits.size, 64
    q = np.tile(np.arange(16, dtype=np.uint8), 4)
    words = np.tile(oracle.pack(4, q), (N, 1))
    g = np.random.default_rng(11)
    sample_b = np.concatenate([np.array([0, 0x8000, 1, 0x0400, 0x3C00, 0xBC00, 0x7BFF, 0xFBFF], np.uint16),
                               g.integers(0, 0x7C00, 24).astype(np.uint16) | (g.integers(0, 2, 24).astype(np.uint16) << 15)])
    sf = s_bits.view(np.float16).astype(np.float32)[:, None]
    qf = q.astype(np.float32)[None, :]
    for b in sample_b:
        b_bits = np.full((N, 1), b, np.uint16)
        w32, w16 = oracle.dequant_matrix(4, True, N, K, words, s_bits.reshape(N, 1), b_bits, want="both")
        with np.errstate(over="ignore", invalid="ignore"):
            ref32 = qf * sf + b_bits.view(np.float16).astype(np.float32)
            ref16 = ref32.astype(np.float16)
        assert np.array_equal(w32.view(np.uint32), ref32.view(np.uint32))
        assert np.array_equal(w16, ref16.view(np.uint16))
    # symmetric, group 32: (q-7)*s exactly
    w32 = oracle.dequant_matrix(4, False, N, 32, words[:, :4], s_bits.reshape(N, 1), None, want="f32")
    with np.errstate(over="ignore", invalid="ignore"):
        ref = (qf[:, :32] - 7.0) * sf
    assert np.array_equal(w32.view(np.uint32), ref.view(np.uint32))


def test_dequant_3bit_matches_numpy(oracle, synth):
    N, K = 16, 256
    w, s = synth.packed_weights(N, K, bits=3), synth.scales(N, K)
    b = synth.biases(N, K, s)
    bits = np.unpackbits(w.view(np.uint8).reshape(N, -1), axis=1, bitorder="little").reshape(N, K, 3)
    q = (bits[..., 0] + 2 * bits[..., 1] + 4 * bits[..., 2]).astype(np.float32)
    sf = np.repeat(s.view(np.float16).astype(np.float32), 64, axis=1)
    bf = np.repeat(b.view(np.float16).astype(np.float32), 64, axis=1)
    got = oracle.dequant_matrix(3, True, N, K, w, s, b, want="f32")
    assert np.array_equal(got.view(np.uint32), (q * sf + bf).view(np.uint32))


# ---- GEMV / GEMM --------------------------------------------------------------------------

def _numpy_dense(bits, affine, w, s, b, K):
    """Independent dequantization in float64 from numpy bit operations."""
    N = w.shape[0]
    if bits == 4:
        by = w.view(np.uint8).reshape(N, -1)
        q = np.empty((N, K), np.float64)
        q[:, 0::2], q[:, 1::2] = by & 15, by >> 4
    else:
        u = np.unpackbits(w.view(np.uint8).reshape(N, -1), axis=1, bitorder="little").reshape(N, K, 3)
        q = (u[..., 0] + 2 * u[..., 1] + 4 * u[..., 2]).astype(np.float64)
    G = 64 if affine else 32
    sf = np.repeat(s.view(np.float16).astype(np.float64), G, axis=1)
    if affine:
        return q * sf + np.repeat(b.view(np.float16).astype(np.float64), G, axis=1)
    return (q - 7.0) * sf


@pytest.mark.parametrize("bits,affine", [(4, True), (4, False), (3, True)])
def test_gemm_modes_against_float64_matmul(oracle, synth, bits, affine):
    M, N, K = 5, 24, 512
    A = synth.activations(M, K)
    w = synth.packed_weights(N, K, bits=bits)
    s = synth.scales(N, K, affine=affine)
    b = synth.biases(N, K, s) if affine else None
    W = _numpy_dense(bits, affine, w, s, b, K)
    ref = A.view(np.float16).astype(np.float64) @ W.T
    for mode, tol in ((oracle.MODE_FORMULA_F64, 1e-12), (oracle.MODE_JS, 1e-12), (oracle.MODE_FORMULA_F32, 2e-5)):
        got = oracle.gemm(mode, bits, affine, M, N, K, A, w, s, b)
        assert np.max(np.abs(got - ref)) < tol * max(1.0, np.max(np.abs(ref))), mode
    # f16-rounded weights: same matmul on the rounded matrix
    W16 = oracle.dequant_matrix(bits, affine, N, K, w, s, b, want="f16").view(np.float16).astype(np.float64)
    got = oracle.gemm(oracle.MODE_F16W, bits, affine, M, N, K, A, w, s, b)
    assert np.max(np.abs(got - A.view(np.float16).astype(np.float64) @ W16.T)) < 1e-10


@pytest.mark.parametrize("bits", [4, 3])
def test_gemv_one_hot_and_special_cases(oracle, synth, bits):
    N, K = 8, 256
    w = synth.packed_weights(N, K, bits=bits)
    s = synth.scales(N, K)
    b = synth.biases(N, K, s)
    W = oracle.dequant_matrix(bits, True, N, K, w, s, b, want="f32").astype(np.float64)
    for k in (0, 9, 10, 21, 63, 64, 255):  # one-hot x: y[n] == W[n,k]
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1
        for mode in (oracle.MODE_JS, oracle.MODE_FORMULA_F64, oracle.MODE_FORMULA_F32):
            y = oracle.gemm(mode, bits, True, 1, N, K, x.view(np.uint16), w, s, b)
            assert np.allclose(y[0], W[:, k], rtol=1e-7, atol=0), (mode, k)
    x = synth.activations(1, K)
    xf = x.view(np.float16).astype(np.float64)[0]
    xg = xf.reshape(-1, 64).sum(1)
    # zero scale: only the bias term survives
    z = np.zeros_like(s)
    y = oracle.gemm(oracle.MODE_FORMULA_F64, bits, True, 1, N, K, x, w, z, b)
    assert np.allclose(y[0], b.view(np.float16).astype(np.float64) @ xg)
    # constant values c: y = sum_g (s*c + b) * sum(x_g)
    c = 5
    wc = np.tile(oracle.pack(bits, np.full(K, c, np.uint8)), (N, 1))
    y = oracle.gemm(oracle.MODE_JS, bits, True, 1, N, K, x, wc, s, b)
    assert np.allclose(y[0], (s.view(np.float16).astype(np.float64) * c + b.view(np.float16).astype(np.float64)) @ xg)
    # zero x
    y = oracle.gemm(oracle.MODE_JS, bits, True, 1, N, K, np.zeros((1, K), np.uint16), w, s, b)
    assert np.all(y == 0)


def test_moe_equals_dense_on_gathered_slab(oracle, synth):
    E, N, K, T, S = 6, 16, 128, 3, 2
    w = synth.packed_weights(N, K, experts=E)
    s = synth.scales(N, K, experts=E)
    b = synth.biases(N, K, s, experts=E)
    ids = synth.topk_ids(T, S, E)
    x = synth.activations(T * S, K)  # per (token, slot) inputs: in_slot_stride=K, in_tok_stride=S*K
    out = oracle.moe_gemv(oracle.MODE_FORMULA_F64, 4, N, K, T, S, (K, N, S * K, S * N, S), ids, x, w, s, b, T * S * N)
    for t in range(T):
        for sl in range(S):
            e = ids[t, sl]
            y = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, 1, N, K, x[t * S + sl], w[e], s[e], b[e])
            assert np.array_equal(out[(t * S + sl) * N:(t * S + sl + 1) * N], y[0])
    # shared input (IN_SLOT_STRIDE = 0) and duplicate experts give identical rows
    ids2 = np.array([[2, 2]], np.uint32)
    out = oracle.moe_gemv(oracle.MODE_FORMULA_F64, 4, N, K, 1, 2, (0, N, K, 2 * N, 2), ids2, x[:1], w, s, b, 2 * N)
    assert np.array_equal(out[:N], out[N:])


def test_8bit_unpack_and_formula(oracle):
    """8-bit rows: value k is byte k of the little-endian word stream; the formula mode equals a float64 matmul
    on a matrix dequantized by numpy alone; reading the same words as 4-bit is a different matrix."""
    rng = np.random.default_rng(8)
    N, K, M = 12, 256, 3
    w = rng.integers(0, 2 ** 32, (N, K // 4), dtype=np.uint64).astype(np.uint32)
    q = w.view(np.uint8).reshape(N, K)
    for k in (0, 1, 2, 3, 4, 63, 64, 255):
        assert oracle.unpack(8, w[5], k) == int(q[5, k])
    assert np.array_equal(oracle.pack(8, q[3]), w[3])
    s = (rng.random((N, K // 64)) * 0.05 + 0.01).astype(np.float16)
    b = (rng.random((N, K // 64)) * 0.1 - 0.05).astype(np.float16)
    x = (rng.random((M, K)) * 2 - 1).astype(np.float16)
    Wd = q.astype(np.float64) * np.repeat(s.astype(np.float64), 64, 1) + np.repeat(b.astype(np.float64), 64, 1)
    want = x.astype(np.float64) @ Wd.T
    for mode in (oracle.MODE_FORMULA_F64, oracle.MODE_JS):
        got = oracle.gemm(mode, 8, True, M, N, K, x.view(np.uint16), w, s.view(np.uint16), b.view(np.uint16))
        assert np.max(np.abs(got - want)) < 1e-9
    w32 = oracle.dequant_matrix(8, True, N, K, w, s.view(np.uint16), b.view(np.uint16), want="f32")
    assert np.array_equal(w32, (q.astype(np.float32) * np.repeat(s.astype(np.float32), 64, 1)
                                + np.repeat(b.astype(np.float32), 64, 1)).astype(np.float32)) or \
        np.max(np.abs(w32.astype(np.float64) - Wd) / (np.abs(Wd) + 1e-30)) < 2.0 ** -23
