"""GPU parity of QKV matmul + RoPE + paged KV append in one dispatch, through the C ABI.

The reference's own test shape (tests/kernels/run.mjs:780-862): the full 9216-row Phi-3 projection (d = 3072,
32 heads of 96, 16 slots per page), position 20, two pages, bar |got-want|/(|want|+1e-3) < 2e-2 on Q, rotated K and
unrotated V at the paged-cache position; plus a grouped-query shape, affine rows, a position in a later page with a
non-zero pages offset, an untouched rest of the cache, and positions that fall outside the cache.
"""
import numpy as np
import pytest

from .util import Dev

pytestmark = pytest.mark.gpu


def layout(kv_heads, hd, page):
    hps = page * hd
    return hps, kv_heads * hps, 2 * kv_heads * hps     # head_page_stride, v_page_offset, kv_page_stride


def run(ctx, capi, oracle, synth, heads, kv_heads, hd, K, page, pos, pages, affine, theta=10000.0, pages_off=0, pos_off=0,
        capacity=None):
    rows = (heads + 2 * kv_heads) * hd
    hps, vpo, kps = layout(kv_heads, hd, page)
    x = synth.activations(1, K)
    w = synth.packed_weights(rows, K)
    s = synth.scales(rows, K, affine=affine, lo=0.01, hi=0.06)
    b = synth.biases(rows, K, s, "A") if affine else None
    pages0 = np.full(pages * kps + pages_off, 0x3C00, np.uint16)
    pmap = np.full(pos_off + 1, -7, np.int32)
    pmap[pos_off] = pos
    with Dev(ctx) as d:
        q_out = d.empty(heads * hd * 2 + 16, fill=0)
        kv = d.put(pages0)
        desc = capi.QkvFusedDesc(bits=4, affine=int(affine), k_packed=K // 8, scales_per_row=K // (64 if affine else 32),
                                 heads=heads, kv_heads=kv_heads, head_dim=hd, page_size=page, kv_page_stride=kps,
                                 head_page_stride=hps, v_page_offset=vpo, position_map_elem_offset=pos_off,
                                 pages_elem_offset=pages_off, rope_theta=theta,
                                 kv_capacity=pages0.size if capacity is None else capacity, q_out=q_out, kv_pages=kv,
                                 hidden=d.put(x), scales=d.put(s), weights=d.put(w), position_map=d.put(pmap),
                                 biases=d.put(b) if affine else 0)
        ctx.qkv_fused(desc)
        got_q = ctx.download(q_out, heads * hd * 2 + 16, np.uint16)
        got_p = ctx.download(kv, pages0.nbytes, np.uint16)
    want_q, want_p = (None, None)
    if 0 <= pos < pages * page:
        want_q, want_p = oracle.qkv_fused(affine, K, heads, kv_heads, hd, page, kps, hps, vpo, pages_off, theta, pos, x, w, s,
                                          b, pages0)
    return got_q, got_p, want_q, want_p, pages0


def rel(got_bits, want_bits, angle_slack=0.0):
    """max |got-want| / (|want| + 1e-3), the reference test's metric. `angle_slack` (radians) forgives what an
    angle error of that size does to a rotated pair: the kernel, like the shader, forms position / theta^(2d/hd)
    in f32, so at position p the angle itself carries about p * 2^-23 of rounding, and a pair of norm r moves by
    that times r whatever its components are. Pairs are (x[d], x[d + half]) of rows laid out [..., head_dim]."""
    g = np.asarray(got_bits, np.uint16).view(np.float16).astype(np.float64)
    w = np.asarray(want_bits, np.uint16).view(np.float16).astype(np.float64)
    assert np.all(np.isfinite(g))
    err = np.abs(g - w)
    if angle_slack:
        half = w.shape[-1] // 2
        norm = np.hypot(w[..., :half], w[..., half:])
        err = np.maximum(err - angle_slack * np.concatenate([norm, norm], -1), 0.0)
    return float(np.max(err / (np.abs(w) + 1e-3)))


@pytest.mark.parametrize("heads,kv_heads,hd,K,page,pos,pages,affine,pages_off,pos_off", [
    (32, 32, 96, 3072, 16, 20, 2, False, 0, 0),      # the reference test: Phi-3, position 20 of two pages
    (16, 2, 128, 2048, 16, 37, 3, False, 0, 2),      # grouped-query: unequal Q / K / V groups
    (4, 2, 64, 512, 8, 0, 1, True, 0, 0),            # affine rows, position 0 (no rotation at all)
    (8, 4, 32, 256, 4, 11, 3, True, 64, 1),          # last page, pages offset, narrow rows (16 lanes per row)
    (6, 2, 64, 1024, 16, 4095, 256, False, 0, 0),    # a late position: large rotation angles
])
def test_qkv_fused(ctx, capi, oracle, synth, heads, kv_heads, hd, K, page, pos, pages, affine, pages_off, pos_off):
    got_q, got_p, want_q, want_p, pages0 = run(ctx, capi, oracle, synth, heads, kv_heads, hd, K, page, pos, pages, affine,
                                               pages_off=pages_off, pos_off=pos_off)
    n = heads * hd
    bar = 2e-2
    slack = max(pos, 1) * 2.0 ** -22       # 0 would do at the reference's position 20; matters at 4095
    assert rel(got_q[:n].reshape(heads, hd), want_q.reshape(heads, hd), slack) < bar
    assert not got_q[n:].any(), "wrote past q_out"
    hps, vpo, kps = layout(kv_heads, hd, page)
    view = lambda a: a[pages_off:].reshape(pages, 2, kv_heads, page, hd)[pos // page, :, :, pos % page]   # [K|V][kv_head][hd]
    assert rel(view(got_p)[0], view(want_p)[0], slack) < bar                # K, rotated
    assert rel(view(got_p)[1], view(want_p)[1]) < bar                       # V, as is
    mask = np.zeros(pages0.size, bool)
    mask[pages_off:].reshape(pages, 2, kv_heads, page, hd)[pos // page, :, :, pos % page] = True
    assert np.array_equal(got_p[~mask], pages0[~mask]), "the rest of the cache is untouched"


def test_v_is_not_rotated_and_k_is(ctx, capi, oracle, synth):
    """Same projection at two positions: V rows equal bit for bit, K rows differ."""
    a = run(ctx, capi, oracle, synth, 4, 2, 64, 512, 8, 3, 2, False)
    b = run(ctx, capi, oracle, synth, 4, 2, 64, 512, 8, 5, 2, False)
    hps, vpo, kps = layout(2, 64, 8)
    pa, pb = a[1].reshape(2, 2, 2, 8, 64), b[1].reshape(2, 2, 2, 8, 64)
    assert np.array_equal(pa[0, 1, :, 3], pb[0, 1, :, 5])
    assert not np.array_equal(pa[0, 0, :, 3], pb[0, 0, :, 5])


@pytest.mark.parametrize("pos", [-1, 16, 10 ** 6])
def test_position_outside_the_cache_writes_q_only(ctx, capi, oracle, synth, pos):
    got_q, got_p, _, _, pages0 = run(ctx, capi, oracle, synth, 4, 2, 64, 512, 8, pos, 2, False)
    assert np.array_equal(got_p, pages0), "a bad position must not touch (or fault on) the cache"
    assert got_q[:4 * 64].any()


def test_rejects(ctx, capi):
    with Dev(ctx) as d:
        p = d.empty(1 << 16, fill=0)
        good = dict(bits=4, affine=0, k_packed=64, scales_per_row=16, heads=4, kv_heads=2, head_dim=64, page_size=8,
                    kv_page_stride=2048, head_page_stride=512, v_page_offset=1024, rope_theta=1e4, q_out=p, kv_pages=p, hidden=p,
                    scales=p, weights=p, position_map=p)
        ctx.qkv_fused(capi.QkvFusedDesc(**good))
        for bad in (dict(bits=3), dict(head_dim=63), dict(scales_per_row=8), dict(v_page_offset=512), dict(kv_page_stride=1536),
                    dict(rope_theta=0.0), dict(position_map=0), dict(affine=1, scales_per_row=8), dict(head_page_stride=256)):
            with pytest.raises(capi.ZtvmError):
                ctx.qkv_fused(capi.QkvFusedDesc(**{**good, **bad}))
