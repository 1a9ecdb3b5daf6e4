"""GPU parity of the int8-KV pair: qkv_fused_scratch (QKV matmul + RoPE, K and V to two scratch rows) and
kv_quantize_int8 (scratch rows -> packed int8 pages + f16 scales), through the C ABI.

Shapes of the reference's tests: tests/kernels/compile-qwen.mjs:687-760 (head_dim 128, 8 kv heads, position 20 of
two pages, bars: scales within 2e-3, counts within +-1 of the float64 reference, |q*scale - x| < 8e-3) and
compile-qwen35.mjs:1609-1685 (head_dim 256: 64 words per row, more than the reference's 32 threads), plus several
tokens in one dispatch, offsets into both arrays, an all-zero row, and positions outside the cache.
The quantizer is integer work: equal to the oracle bit for bit.
"""
import numpy as np
import pytest

from .util import Dev
from .test_qkv_fused_gpu import layout

pytestmark = pytest.mark.gpu


def kvq(ctx, capi, kv_heads, hd, page, positions, k, v, pages0, scales0, pages_off=0, scales_off=0, pos_off=0,
        pages_cap=None, scales_cap=None):
    pmap = np.full(pos_off + len(positions), -9, np.int32)
    pmap[pos_off:] = positions
    with Dev(ctx) as d:
        pg, sc = d.put(pages0), d.put(scales0)
        desc = capi.KvQuantizeDesc(kv_heads=kv_heads, head_dim=hd, page_size=page, tokens=len(positions),
                                   position_map_elem_offset=pos_off, pages_word_offset=pages_off, scales_elem_offset=scales_off,
                                   pages_capacity_words=pages0.size if pages_cap is None else pages_cap,
                                   scales_capacity=scales0.size if scales_cap is None else scales_cap,
                                   k_slot=d.put(k), v_slot=d.put(v), pages_i8=pg, scales=sc, position_map=d.put(pmap))
        ctx.kv_quantize_int8(desc)
        return ctx.download(pg, pages0.nbytes, np.uint32), ctx.download(sc, scales0.nbytes, np.uint16)


def slots(kv_heads, hd, tokens, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    return ((rng.uniform(-1, 1, (tokens, kv_heads * hd)) * scale).astype(np.float16),
            (rng.uniform(-1, 1, (tokens, kv_heads * hd)) * scale).astype(np.float16))


@pytest.mark.parametrize("kv_heads,hd,page,positions,pages_n,pages_off,scales_off,pos_off", [
    (8, 128, 16, [20], 2, 0, 0, 0),                 # the reference test
    (2, 256, 16, [20], 2, 0, 0, 0),                 # the width that broke: 64 words per row
    (4, 96, 16, [0, 17, 31, 5], 2, 0, 0, 3),        # a prefill chunk: four tokens, one dispatch (Phi-3 head)
    (3, 64, 8, [9], 3, 40, 6, 1),                   # offsets into both arrays
    (1, 512, 4, [3, 2], 1, 0, 0, 0),                # two turns per lane
])
def test_kv_quantize_int8(ctx, capi, oracle, kv_heads, hd, page, positions, pages_n, pages_off, scales_off, pos_off):
    k, v = slots(kv_heads, hd, len(positions), 11 + hd)
    k[0, :hd] = 0
    rw = hd // 4
    pages0 = np.full(pages_n * kv_heads * page * 2 * rw + pages_off, 0xDEADBEEF, np.uint32)
    scales0 = np.full(pages_n * kv_heads * page * 2 + scales_off, 0x7BFF, np.uint16)
    got_pg, got_sc = kvq(ctx, capi, kv_heads, hd, page, positions, k, v, pages0, scales0, pages_off, scales_off, pos_off)
    want_pg, want_sc = oracle.kv_quantize_int8(kv_heads, hd, page, positions, pages_off, scales_off, k.view(np.uint16),
                                               v.view(np.uint16), pages0, scales0)
    assert np.array_equal(got_sc, want_sc)
    assert np.array_equal(got_pg, want_pg)
    # the reference test's own bars, on the GPU's output
    pg = got_pg[pages_off:].reshape(pages_n, kv_heads, page, 2, rw)
    sc = got_sc[scales_off:].view(np.float16).reshape(pages_n, kv_heads, page, 2).astype(np.float64)
    for t, pos in enumerate(positions):
        pno, slot = divmod(pos, page)
        for side, src in enumerate((k, v)):
            words = pg[pno, :, slot, side, :]
            q = np.stack([(words >> (8 * i)) & 0xFF for i in range(4)], axis=-1).astype(np.int64).reshape(kv_heads, hd)
            q = np.where(q > 127, q - 256, q)
            x = src[t].astype(np.float64).reshape(kv_heads, hd)
            s64 = np.maximum(np.abs(x).max(axis=1, keepdims=True) / 127, 1e-8)
            assert np.all(np.abs(sc[pno, :, slot, side][:, None] - s64.astype(np.float16).astype(np.float64)) <= np.abs(s64) * 2e-3)
            assert np.max(np.abs(q - np.clip(np.floor(x / s64 + 0.5), -127, 127))) <= 1
            assert np.max(np.abs(q * sc[pno, :, slot, side][:, None] - x)) < 8e-3


def test_positions_outside_the_cache_write_nothing(ctx, capi):
    kv_heads, hd, page = 2, 64, 4
    k, v = slots(kv_heads, hd, 3, 3)
    rw = hd // 4
    pages0 = np.full(2 * kv_heads * page * 2 * rw, 0xDEADBEEF, np.uint32)
    scales0 = np.full(2 * kv_heads * page * 2, 0x7BFF, np.uint16)
    got_pg, got_sc = kvq(ctx, capi, kv_heads, hd, page, [-1, 8, 10 ** 6], k, v, pages0, scales0)
    assert np.array_equal(got_pg, pages0) and np.array_equal(got_sc, scales0)


def test_rejects(ctx, capi):
    ok = dict(kv_heads=2, head_dim=64, page_size=4, tokens=1, k_slot=0x1000, v_slot=0x2000, pages_i8=0x3000, scales=0x4000,
              position_map=0x5000)
    for bad, needle in ((dict(head_dim=66), "multiple of 4"), (dict(kv_heads=0), "kv_heads"), (dict(pages_i8=0), "null"),
                        (dict(k_slot=0x1004), "misaligned"), (dict(head_dim=2048), "head_dim")):
        with pytest.raises(capi.ZtvmError, match=needle):
            ctx.kv_quantize_int8(capi.KvQuantizeDesc(**{**ok, **bad}))
    ctx.kv_quantize_int8(capi.KvQuantizeDesc(**{**ok, "tokens": 0}))     # nothing to do, nothing dereferenced


@pytest.mark.parametrize("heads,kv_heads,hd,K,page,pos,affine", [
    (32, 32, 96, 3072, 16, 20, False),     # the reference's qkv_fused test shape
    (16, 2, 128, 2048, 16, 37, False),     # grouped-query
    (4, 2, 64, 512, 8, 5, True),           # affine rows
])
def test_scratch_rows_equal_the_paged_write(ctx, capi, synth, heads, kv_heads, hd, K, page, pos, affine):
    """qkv_fused_scratch differs from qkv_fused only in WHERE K and V go: the same f16 bits, as [kv_heads][head_dim]
    rows; Q is the same; the paged form itself is checked against the oracle in its own test."""
    rows = (heads + 2 * kv_heads) * hd
    hps, vpo, kps = layout(kv_heads, hd, page)
    pages = pos // page + 1
    x = synth.activations(1, K)
    w = synth.packed_weights(rows, K)
    s = synth.scales(rows, K, affine=affine, lo=0.01, hi=0.06)
    b = synth.biases(rows, K, s, "A") if affine else None
    with Dev(ctx) as d:
        q1, q2 = d.empty(heads * hd * 2, fill=0), d.empty(heads * hd * 2, fill=0)
        kv = d.empty(pages * kps * 2, fill=0)
        ks, vs = d.empty(kv_heads * hd * 2 + 16, fill=0), d.empty(kv_heads * hd * 2 + 16, fill=0)
        common = dict(bits=4, affine=int(affine), k_packed=K // 8, scales_per_row=K // (64 if affine else 32), heads=heads,
                      kv_heads=kv_heads, head_dim=hd, position_map_elem_offset=0, rope_theta=10000.0, hidden=d.put(x),
                      scales=d.put(s), weights=d.put(w), position_map=d.put(np.array([pos], np.int32)),
                      biases=d.put(b) if affine else 0)
        ctx.qkv_fused(capi.QkvFusedDesc(page_size=page, kv_page_stride=kps, head_page_stride=hps, v_page_offset=vpo,
                                        pages_elem_offset=0, kv_capacity=pages * kps, q_out=q1, kv_pages=kv, **common))
        ctx.qkv_fused_scratch(capi.QkvFusedDesc(q_out=q2, **common), ks, vs)
        paged = ctx.download(kv, pages * kps * 2, np.uint16).reshape(pages, 2, kv_heads, page, hd)
        got_k = ctx.download(ks, kv_heads * hd * 2 + 16, np.uint16)
        got_v = ctx.download(vs, kv_heads * hd * 2 + 16, np.uint16)
        assert np.array_equal(ctx.download(q1, heads * hd * 2, np.uint16), ctx.download(q2, heads * hd * 2, np.uint16))
    pno, slot = divmod(pos, page)
    assert np.array_equal(got_k[:kv_heads * hd].reshape(kv_heads, hd), paged[pno, 0, :, slot, :])
    assert np.array_equal(got_v[:kv_heads * hd].reshape(kv_heads, hd), paged[pno, 1, :, slot, :])
    assert paged[pno, 0, :, slot, :].any() and not got_k[kv_heads * hd:].any() and not got_v[kv_heads * hd:].any()


def test_scratch_then_quantize(ctx, capi, oracle, synth):
    """The int8 decode path end to end: scratch rows from the fused kernel, then the quantizer, equal the oracle's
    quantisation of those rows."""
    heads, kv_heads, hd, K, page, pos = 8, 2, 128, 1024, 16, 21
    rows = (heads + 2 * kv_heads) * hd
    x, w = synth.activations(1, K), synth.packed_weights(rows, K)
    s = synth.scales(rows, K, affine=False, lo=0.01, hi=0.06)
    rw = hd // 4
    pages0, scales0 = np.zeros(2 * kv_heads * page * 2 * rw, np.uint32), np.zeros(2 * kv_heads * page * 2, np.uint16)
    with Dev(ctx) as d:
        q, ks, vs = d.empty(heads * hd * 2, fill=0), d.empty(kv_heads * hd * 2, fill=0), d.empty(kv_heads * hd * 2, fill=0)
        pm = d.put(np.array([pos], np.int32))
        pg, sc = d.put(pages0), d.put(scales0)
        ctx.qkv_fused_scratch(capi.QkvFusedDesc(bits=4, affine=0, k_packed=K // 8, scales_per_row=K // 32, heads=heads,
                                                kv_heads=kv_heads, head_dim=hd, rope_theta=10000.0, q_out=q, hidden=d.put(x),
                                                scales=d.put(s), weights=d.put(w), position_map=pm), ks, vs)
        ctx.kv_quantize_int8(capi.KvQuantizeDesc(kv_heads=kv_heads, head_dim=hd, page_size=page, tokens=1,
                                                 pages_capacity_words=pages0.size, scales_capacity=scales0.size, k_slot=ks,
                                                 v_slot=vs, pages_i8=pg, scales=sc, position_map=pm))
        k_bits, v_bits = ctx.download(ks, kv_heads * hd * 2, np.uint16), ctx.download(vs, kv_heads * hd * 2, np.uint16)
        got_pg, got_sc = ctx.download(pg, pages0.nbytes, np.uint32), ctx.download(sc, scales0.nbytes, np.uint16)
    want_pg, want_sc = oracle.kv_quantize_int8(kv_heads, hd, page, [pos], 0, 0, k_bits, v_bits, pages0, scales0)
    assert np.array_equal(got_pg, want_pg) and np.array_equal(got_sc, want_sc) and got_pg.any()
