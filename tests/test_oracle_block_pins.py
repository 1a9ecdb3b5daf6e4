"""Pins of the oracle's loader conversions and MoE block ops against numpy / scipy.

Each check is chosen so that a plausible mistake fails it: a flushed subnormal, a NaN turned into
infinity, an inverted permutation, an untransposed K block, the 8-bit reader on 4-bit rows, softmax after
top-k, a tie going to the higher index. None of them re-types the oracle's own formula: the comparisons are
numpy casts, fancy indexing, einsum, scipy's expit / softmax and a stable argsort.
"""
import numpy as np
import pytest
from scipy.special import expit, softmax


def f16_of(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


# ---------------------------------------------------------------- bf16 ---------------------------------------

def test_bf16_to_f16_every_pattern(oracle):
    src = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got, overflow = oracle.bf16_to_f16(src)
    f32 = (src.astype(np.uint32) << 16).view(np.float32)
    with np.errstate(over="ignore"):
        want = f32.astype(np.float16).view(np.uint16)
    finite = np.isfinite(f32)
    with np.errstate(invalid="ignore"):
        fits = finite & (np.abs(f32.astype(np.float64)) < 65520.0)  # below the rounding boundary to infinity
    assert np.array_equal(got[fits], want[fits]), "normal / subnormal / zero values must equal numpy's cast"
    big = finite & ~fits
    assert overflow == int(big.sum()) and overflow > 0
    assert np.array_equal(got[big], ((src[big] & 0x8000) | 0x7BFF).astype(np.uint16)), "overflow clamps to +-65504"
    inf = np.isinf(f32)
    assert np.array_equal(got[inf], want[inf])
    nan = np.isnan(f32)
    assert np.all(np.isnan(got[nan].view(np.float16))) and np.array_equal(got[nan] & 0x8000, src[nan] & 0x8000)
    # f16 subnormals survive (quantization scales land there); bf16 is exact in f16's subnormal band only
    # down to its own precision, so compare values, not just non-zeroness
    band = finite & (np.abs(f32) >= 2.0 ** -24) & (np.abs(f32) < 2.0 ** -14)
    assert band.sum() > 1000 and np.all(got[band] & 0x7FFF)


def test_bf16_reference_value_list(oracle):
    """The value list of the reference's own conversion check (tests/kernels/mlx-repack.mjs:87-136)."""
    vals = np.array([1, -2, 65280, 1e38, 3e-5, 1e-6, 1e-7, 1e-40, 0, -0.0], np.float32)
    u = vals.view(np.uint32)
    lo, hi = u & 0xFFFF, u >> 16
    hi = hi + ((lo > 0x8000) | ((lo == 0x8000) & (hi & 1 == 1)))
    bf = (hi & 0xFFFF).astype(np.uint16)
    f32 = oracle.bf16_to_f32(bf)
    assert np.array_equal(f32.view(np.uint32), bf.astype(np.uint32) << 16)
    got, overflow = oracle.bf16_to_f16(bf)
    assert overflow == 1
    dec = f16_of(got)
    assert dec[3] == 65504.0
    for i in (0, 1, 2):
        assert dec[i] == float(vals[i])
    for i in (4, 5, 6):  # subnormal band: nearest representable, never zero
        ulp = 2.0 ** -24
        assert dec[i] != 0 and abs(dec[i] - float(f32[i])) <= ulp / 2 + 1e-30
    assert dec[7] == 0 and dec[8] == 0 and got[9] == 0x8000


# ---------------------------------------------------------------- row permutation ----------------------------

def test_permute_rows_and_deinterleave(oracle):
    rng = np.random.default_rng(5)
    R, lora, rows = 64, 512, 512 + 64
    src = np.arange(rows)
    src[lora:] = lora + np.array([oracle.deint(j, R) for j in range(R)])
    assert list(src[lora:lora + 4]) == [lora, lora + 2, lora + 4, lora + 6]
    assert list(src[lora + R // 2:lora + R // 2 + 3]) == [lora + 1, lora + 3, lora + 5]
    for row_bytes in (1024, 64, 6):
        data = rng.integers(0, 256, rows * row_bytes, dtype=np.uint8)
        got = oracle.permute_rows(data, rows, src)
        assert np.array_equal(got.reshape(rows, row_bytes), data.reshape(rows, row_bytes)[src])
        inv = np.argsort(src)
        assert not np.array_equal(got, oracle.permute_rows(data, rows, inv)), "the inverse map is a different matrix"
    with pytest.raises(ValueError):
        oracle.permute_rows(np.zeros(10, np.uint8), 3, [0, 1, 2])      # 10 bytes do not divide into 3 rows
    with pytest.raises(ValueError):
        oracle.permute_rows(np.zeros(12, np.uint8), 3, [0, 1])         # short map
    with pytest.raises(ValueError):
        oracle.permute_rows(np.zeros(12, np.uint8), 3, [0, 1, 3])      # index out of range


# ---------------------------------------------------------------- dequantAffineSplit -------------------------

def test_dequant_affine_split_is_dequant_plus_transposes(oracle, synth):
    heads, nope, v, k = 3, 16, 8, 128
    rows = heads * (nope + v)
    w = synth.packed_weights(rows, k, bits=4)
    s = synth.scales(rows, k, affine=True)
    b = synth.biases(rows, k, s, "A")
    got, overflow = oracle.dequant_affine_split(w, s, b, k, heads, nope, v)
    assert overflow == 0
    full = oracle.dequant_matrix(4, True, rows, k, w, s, b, want="f16").reshape(heads, nope + v, k)
    kt = np.ascontiguousarray(full[:, :nope, :].transpose(0, 2, 1))   # [heads][k][nope]
    vv = np.ascontiguousarray(full[:, nope:, :])                      # [heads][v][k]
    assert np.array_equal(got[:kt.size], kt.ravel())
    assert np.array_equal(got[kt.size:], vv.ravel())
    assert not np.array_equal(got[:kt.size], full[:, :nope, :].ravel()), "an untransposed K block must differ"


def test_dequant_affine_split_counts_overflow(oracle):
    heads, nope, v, k = 1, 2, 2, 64
    w = np.full((4, 8), 0xFFFFFFFF, np.uint32)
    s = np.full((4, 1), np.float16(60000).view(np.uint16), np.uint16)
    s[3] = np.float16(1).view(np.uint16)
    b = np.zeros((4, 1), np.uint16)
    _, overflow = oracle.dequant_affine_split(w, s, b, k, heads, nope, v)
    assert overflow == 3 * 64


# ---------------------------------------------------------------- silu_mul -----------------------------------

def test_silu_mul(oracle):
    rng = np.random.default_rng(38)
    rows, ffn = 3, 320
    gu = (rng.random((rows, 2 * ffn)) * 6 - 3).astype(np.float16)
    gu[0, :4] = [0, -0.0, 30, -30]
    o64, o16 = oracle.silu_mul(gu.view(np.uint16), rows, ffn)
    g, u = gu[:, :ffn].astype(np.float64), gu[:, ffn:].astype(np.float64)
    want = u * g * expit(g)
    assert np.max(np.abs(o64 - want)) < 1e-12
    got16 = f16_of(o16)
    ulp = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(got16 - want) <= 0.5 * ulp + 1e-6 * np.abs(want) + 1e-12)
    # the halves are not interchangeable
    swapped, _ = oracle.silu_mul(np.concatenate([gu[:, ffn:], gu[:, :ffn]], 1).view(np.uint16), rows, ffn)
    assert np.max(np.abs(swapped - want)) > 0.1


# ---------------------------------------------------------------- moe_combine --------------------------------

def test_moe_combine(oracle):
    rng = np.random.default_rng(9)
    tokens, N, S = 5, 96, 9
    slots = (rng.standard_normal((tokens, S, N))).astype(np.float16)
    score = rng.random((tokens, S)).astype(np.float32)
    o64, o16 = oracle.moe_combine(slots.view(np.uint16), score, tokens, N, S)
    want = np.einsum("ts,tsn->tn", score.astype(np.float64), slots.astype(np.float64))
    assert np.max(np.abs(o64 - want)) < 1e-12
    assert np.max(np.abs(f16_of(o16) - want)) <= np.max(np.abs(want)) * 2.0 ** -10
    # one-hot scores pick one slot's row exactly, of the right token
    hot = np.zeros((tokens, S), np.float32)
    hot[np.arange(tokens), [0, 8, 3, 1, 7]] = 1.0
    _, p16 = oracle.moe_combine(slots.view(np.uint16), hot, tokens, N, S)
    assert np.array_equal(p16, slots.view(np.uint16)[np.arange(tokens), [0, 8, 3, 1, 7]])


# ---------------------------------------------------------------- router logits ------------------------------

def unpack_le(words, bits):
    b = np.ascontiguousarray(words, np.uint32).view(np.uint8)
    if bits == 8:
        return b.astype(np.float64)
    return np.stack([b & 15, b >> 4], -1).reshape(-1).astype(np.float64)


@pytest.mark.parametrize("bits", [8, 4, 16])
def test_router_logits(oracle, bits):
    rng = np.random.default_rng(11 + bits)
    D, rows, tokens = 2048, 9, 3
    x = (rng.random((tokens, D)) * 2 - 1).astype(np.float16)
    if bits == 16:
        w16 = (rng.random((rows, D)) * 0.1 - 0.05).astype(np.float16)
        got = oracle.router_logits(16, D, rows, tokens, x.view(np.uint16), w16.view(np.uint16))
        want = x.astype(np.float64) @ w16.astype(np.float64).T
        assert np.max(np.abs(got - want)) < 1e-10
        return
    words = rng.integers(0, 2 ** 32, (rows, D * bits // 32), dtype=np.uint64).astype(np.uint32)
    s = (rng.random((rows, D // 64)) * 0.02 + 0.005).astype(np.float16)
    b = (rng.random((rows, D // 64)) * 0.2 - 0.1).astype(np.float16)
    got = oracle.router_logits(bits, D, rows, tokens, x.view(np.uint16), words, s.view(np.uint16), b.view(np.uint16))
    q = unpack_le(words, bits).reshape(rows, D)
    wfull = q * np.repeat(s.astype(np.float64), 64, 1) + np.repeat(b.astype(np.float64), 64, 1)
    want = x.astype(np.float64) @ wfull.T
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-2)) < 1e-9
    # the other width's reading of the same bytes is a different answer by O(1), not a rounding difference
    q_other = unpack_le(words, 4 if bits == 8 else 8).reshape(rows, -1)
    q_other = np.concatenate([q_other, q_other], 1)[:, :D]
    w_other = q_other * np.repeat(s.astype(np.float64), 64, 1) + np.repeat(b.astype(np.float64), 64, 1)
    assert np.max(np.abs(got - x.astype(np.float64) @ w_other.T)) > 0.1


# ---------------------------------------------------------------- router top-k -------------------------------

@pytest.mark.parametrize("E,K,norm,shared", [(256, 8, True, True), (128, 8, True, False), (128, 8, False, False),
                                             (60, 4, True, True), (8, 8, False, False), (300, 32, True, True)])
def test_router_topk(oracle, E, K, norm, shared):
    rng = np.random.default_rng(7)
    tokens = 4
    rows = E + (1 if shared else 0)
    logits = (rng.random((tokens, rows)) * 8 - 4).astype(np.float32)
    idx, score = oracle.router_topk(logits, tokens, E, K, norm, shared)
    p = softmax(logits[:, :E].astype(np.float64), axis=1)
    order = np.argsort(-p, axis=1, kind="stable")[:, :K]
    assert np.array_equal(idx[:, :K], order)
    top = np.take_along_axis(p, order, 1)
    want = top / top.sum(1, keepdims=True) if norm else top
    assert np.max(np.abs(score[:, :K] - want)) < 1e-12
    if norm:
        assert np.allclose(score[:, :K].sum(1), 1.0, atol=1e-12)
    if shared:
        assert np.all(idx[:, K] == E)
        assert np.max(np.abs(score[:, K] - expit(logits[:, E].astype(np.float64)))) < 1e-12


def test_router_topk_ties_and_order(oracle):
    E, K = 16, 4
    logits = np.zeros((1, E), np.float32)
    logits[0, [3, 9, 12]] = 2.0           # three equal maxima, then equal zeros
    idx, score = oracle.router_topk(logits, 1, E, K, False, False)
    assert list(idx[0]) == [3, 9, 12, 0]  # ties to the lower index, descending score
    assert score[0, 0] == score[0, 1] == score[0, 2] > score[0, 3]
    # softmax BEFORE top-k: unnormalised scores are the full-softmax probabilities
    p = softmax(logits[0].astype(np.float64))
    assert abs(score[0, 0] - p[3]) < 1e-15 and abs(score[0].sum() - 1.0) > 0.1


def test_slot_translate(oracle):
    m = np.array([5, 0xFFFFFFFF, 2, 7, 0xFFFFFFFF, 0], np.uint32)
    ids = np.array([0, 1, 2, 3, 4, 5, 3], np.uint32)
    got = oracle.slot_translate(ids, m)
    t = m[ids]
    assert np.array_equal(got, np.where(t == 0xFFFFFFFF, 0, t))


# ---------------------------------------------------------------- qkv_fused ----------------------------------

@pytest.mark.parametrize("affine", [False, True])
def test_qkv_fused(oracle, synth, affine):
    """Against numpy alone: dequantized matrix @ x, the rotary pair (lo, hi) as the complex number lo + i*hi
    multiplied by exp(i*freq), and the cache viewed as [page][K|V][kv_head][slot][dim]."""
    heads, kv_heads, hd, K, page, pos, theta = 4, 2, 16, 128, 8, 13, 10000.0
    half = hd // 2
    rows = (heads + 2 * kv_heads) * hd
    hps, vpo, kps = page * hd, kv_heads * page * hd, 2 * kv_heads * page * hd
    x = synth.activations(1, K)
    w = synth.packed_weights(rows, K)
    s = synth.scales(rows, K, affine=affine)
    b = synth.biases(rows, K, s, "A") if affine else None
    pages0 = np.full(3 * kps, 0x1234, np.uint16)
    q16, pg = oracle.qkv_fused(affine, K, heads, kv_heads, hd, page, kps, hps, vpo, 0, theta, pos, x, w, s, b, pages0)
    W = oracle.dequant_matrix(4, affine, rows, K, w, s, b).astype(np.float64)
    y = W @ x.view(np.float16).astype(np.float64)[0]
    q, k, v = (y[:heads * hd].reshape(heads, hd), y[heads * hd:(heads + kv_heads) * hd].reshape(kv_heads, hd),
               y[(heads + kv_heads) * hd:].reshape(kv_heads, hd))
    rot = np.exp(1j * pos / theta ** (np.arange(half) * 2 / hd))

    def rope(t):
        z = (t[:, :half] + 1j * t[:, half:]) * rot
        return np.concatenate([z.real, z.imag], 1)

    def close(bits, want):
        got = np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)
        return np.all(np.abs(got - want) <= np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10 * 0.51 + 1e-9)

    assert close(q16.reshape(heads, hd), rope(q))
    cache = pg.reshape(3, 2, kv_heads, page, hd)
    assert close(cache[pos // page, 0, :, pos % page], rope(k))
    assert close(cache[pos // page, 1, :, pos % page], v), "V is appended unrotated"
    untouched = np.ones(cache.shape[:4], bool)
    untouched[pos // page, :, :, pos % page] = False
    assert np.all(cache[untouched] == 0x1234), "only the position's slot is written"
    assert not close(q16.reshape(heads, hd), np.concatenate([rope(q)[:, half:], rope(q)[:, :half]], 1))


# ---------------------------------------------------------------- kv_quantize_int8 ----------------------------

def _kvq_case(kv_heads, head_dim, page_size, tokens, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    k = (rng.uniform(-1, 1, (tokens, kv_heads * head_dim)) * scale).astype(np.float16)
    v = (rng.uniform(-1, 1, (tokens, kv_heads * head_dim)) * scale).astype(np.float16)
    return k, v


def _kvq_numpy(kv_heads, head_dim, page_size, positions, k, v, pages, scales):
    """Independent float32 formulation: vectorised numpy, np.rint, true division."""
    rw = head_dim // 4
    pages = pages.copy().reshape(-1, kv_heads, page_size, 2, rw)
    scales = scales.copy().reshape(-1, kv_heads, page_size, 2)
    for t, pos in enumerate(positions):
        if pos < 0:
            continue
        page, slot = divmod(int(pos), page_size)
        for side, src in enumerate((k, v)):
            x = src[t].astype(np.float32).reshape(kv_heads, head_dim)
            sc = np.maximum(np.abs(x).max(axis=1) / np.float32(127.0), np.float32(1e-8)).astype(np.float32)
            inv = (np.float32(1.0) / sc).astype(np.float32)
            q = np.clip(np.rint((x * inv[:, None]).astype(np.float32)), -127, 127).astype(np.int32)
            b = (q & 0xFF).astype(np.uint32).reshape(kv_heads, rw, 4)
            pages[page, :, slot, side, :] = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16) | (b[..., 3] << 24)
            scales[page, :, slot, side] = sc.astype(np.float16).view(np.uint16)
    return pages.ravel(), scales.ravel()


@pytest.mark.parametrize("kv_heads,head_dim,page_size,tokens", [(8, 128, 16, 1), (2, 256, 16, 3), (3, 96, 8, 2), (1, 4, 4, 1)])
def test_kv_quantize_int8_equals_numpy_and_bounds(oracle, kv_heads, head_dim, page_size, tokens):
    k, v = _kvq_case(kv_heads, head_dim, page_size, tokens, 5 + head_dim)
    k[0, :head_dim] = 0                                     # an all-zero row: scale clamps at 1e-8, which is 0 in f16
    pages_n = 3
    positions = np.array([2 * page_size + 1, 3, -1][:tokens], np.int32)   # page 2 slot 1, page 0 slot 3, a skipped token
    rw = head_dim // 4
    pages0 = np.full(pages_n * kv_heads * page_size * 2 * rw, 0xDEADBEEF, np.uint32)
    scales0 = np.full(pages_n * kv_heads * page_size * 2, 0x7BFF, np.uint16)
    pg, sc = oracle.kv_quantize_int8(kv_heads, head_dim, page_size, positions, 0, 0, k.view(np.uint16), v.view(np.uint16), pages0, scales0)
    want_pg, want_sc = _kvq_numpy(kv_heads, head_dim, page_size, positions, k, v, pages0, scales0)
    assert np.array_equal(pg, want_pg) and np.array_equal(sc, want_sc)
    # the accuracy contract: |q*scale - x| <= scale/2 (+ the f16 rounding of the stored scale), and nothing else written
    pgv = pg.reshape(pages_n, kv_heads, page_size, 2, rw)
    scv = sc.view(np.float16).reshape(pages_n, kv_heads, page_size, 2).astype(np.float64)
    touched = np.zeros(pgv.shape[:4], bool)
    for t, pos in enumerate(positions):
        if pos < 0:
            continue
        page, slot = divmod(int(pos), page_size)
        for side, src in enumerate((k, v)):
            words = pgv[page, :, slot, side, :]
            q = np.stack([(words >> (8 * i)) & 0xFF for i in range(4)], axis=-1).astype(np.int64).reshape(kv_heads, head_dim)
            q = np.where(q > 127, q - 256, q)
            x = src[t].astype(np.float64).reshape(kv_heads, head_dim)
            s = scv[page, :, slot, side][:, None]
            assert np.all(np.abs(q * s - x) <= s / 2 + np.abs(x) * 2.0 ** -10 + 1e-12)
            assert np.all(np.abs(q) <= 127)
            # the reference test's own float64 reference, to its +-1 count (compile-qwen.mjs:720-747)
            s64 = np.maximum(np.abs(x).max(axis=1, keepdims=True) / 127, 1e-8)
            ref = np.clip(np.floor(x / s64 + 0.5), -127, 127)
            assert np.max(np.abs(q - ref)) <= 1
            touched[page, :, slot, side] = True
    assert np.all(pgv[~touched] == 0xDEADBEEF) and np.all(sc.reshape(touched.shape)[~touched] == 0x7BFF)
    assert sc.reshape(touched.shape)[int(positions[0]) // page_size, 0, int(positions[0]) % page_size, 0] == 0   # the zero row's scale


def test_kv_quantize_int8_offsets(oracle):
    kv_heads, head_dim, page_size = 2, 64, 4
    k, v = _kvq_case(kv_heads, head_dim, page_size, 1, 9)
    rw = head_dim // 4
    n_words, n_sc = 2 * kv_heads * page_size * 2 * rw, 2 * kv_heads * page_size * 2
    base_pg, base_sc = oracle.kv_quantize_int8(kv_heads, head_dim, page_size, [5], 0, 0, k.view(np.uint16), v.view(np.uint16),
                                               np.zeros(n_words, np.uint32), np.zeros(n_sc, np.uint16))
    off_pg, off_sc = oracle.kv_quantize_int8(kv_heads, head_dim, page_size, [5], 7, 3, k.view(np.uint16), v.view(np.uint16),
                                             np.zeros(n_words + 7, np.uint32), np.zeros(n_sc + 3, np.uint16))
    assert np.array_equal(off_pg[7:], base_pg) and not off_pg[:7].any()
    assert np.array_equal(off_sc[3:], base_sc) and not off_sc[:3].any()


# ---------------------------------------------------------------- add + RMSNorm -------------------------------

def test_add_rmsnorm_against_numpy_and_closed_forms(oracle):
    rng = np.random.default_rng(31)
    K, eps = 3072, 1e-5
    res = rng.standard_normal(K).astype(np.float16)
    dlt = (rng.standard_normal(K) * 0.3).astype(np.float16)
    gam = (1 + 0.1 * rng.standard_normal(K)).astype(np.float16)
    got = oracle.add_rmsnorm(res.view(np.uint16), dlt.view(np.uint16), gam.view(np.uint16), eps).view(np.float16)
    val = (res.astype(np.float32) + dlt.astype(np.float32)).astype(np.float16).astype(np.float32)
    ss = np.float32(np.sum(val.astype(np.float64) ** 2))           # the exactly rounded sum of the (exact) squares
    inv = np.float32(1.0) / np.sqrt(np.float32(ss / np.float32(K)) + np.float32(eps))
    want = ((val * inv).astype(np.float32) * gam.astype(np.float32)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # any float32 summation order lands within a rounding step of it on all but a handful of elements
    inv32 = np.float32(1.0) / np.sqrt(np.float32(np.sum(val * val, dtype=np.float32) / np.float32(K)) + np.float32(eps))
    other = ((val * inv32).astype(np.float32) * gam.astype(np.float32)).astype(np.float16)
    ulp = np.abs(got.view(np.int16).astype(np.int32) - other.view(np.int16).astype(np.int32))
    assert ulp.max() <= 1 and (ulp > 0).mean() < 0.02
    # float64 truth, to f16 accuracy
    v64 = val.astype(np.float64)
    t64 = v64 / np.sqrt(np.mean(v64 * v64) + eps) * gam.astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64) - t64) / (np.abs(t64) + 1e-3)) < 1e-3
    # a constant row: c / sqrt(c^2 + eps) * gamma; zeros stay zero; gamma = 1 gives unit RMS
    c = np.full(K, 0.75, np.float16)
    z = np.zeros(K, np.float16)
    one = np.ones(K, np.float16)
    got = oracle.add_rmsnorm(c.view(np.uint16), z.view(np.uint16), gam.view(np.uint16), eps).view(np.float16).astype(np.float64)
    assert np.max(np.abs(got - 0.75 / np.sqrt(0.75 ** 2 + eps) * gam.astype(np.float64))) < 1e-3
    assert not oracle.add_rmsnorm(z.view(np.uint16), z.view(np.uint16), gam.view(np.uint16), eps).any()
    unit = oracle.add_rmsnorm(res.view(np.uint16), dlt.view(np.uint16), one.view(np.uint16), 0.0).view(np.float16).astype(np.float64)
    assert abs(np.sqrt(np.mean(unit * unit)) - 1.0) < 1e-3
    # the sum is over residual + delta, not either alone
    assert not np.array_equal(oracle.add_rmsnorm(res.view(np.uint16), z.view(np.uint16), gam.view(np.uint16), eps), got)
