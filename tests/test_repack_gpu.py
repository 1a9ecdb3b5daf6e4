"""GPU parity of the load-time repack: the conversion kernels through the C ABI, and whole checkpoints through
the host mirror of the reference's loader, byte for byte.

The reference checks its TypeScript repacker against byte-exact bundles made from real checkpoints
(tests/kernels/mlx-repack.mjs:144-360); those bundles and checkpoints are not in the repository, so the
expected bytes here are built by numpy from synthetic checkpoints of the same record names and layouts
(concatenate the parts, bf16 conversions by the pinned oracle, rows by fancy indexing, kv_b by the pinned
oracle). No tolerance anywhere: either every byte agrees or something is wrong.
"""
import importlib

import numpy as np
import pytest

from . import mlx_synth
from .util import Dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mw(pkg):
    return importlib.import_module("zero-tvm_amd.host.mlx_weights")


@pytest.fixture(scope="module")
def device(pkg, ctx):
    """The host mirror's Device over the session's context."""
    eng = importlib.import_module("zero-tvm_amd.host.engine")
    d = eng.Device.__new__(eng.Device)
    d.ctx, d._recording = ctx, False
    return d


# ---------------------------------------------------------------- conversion kernels -------------------------

@pytest.mark.parametrize("shift", [0, 2, 6])
def test_bf16_to_f16_every_pattern(ctx, capi, oracle, shift):
    """All 65536 bit patterns (twice over), 16-byte aligned and not; the overflow counter accumulates."""
    src = np.tile(np.arange(65536, dtype=np.uint32).astype(np.uint16), 2)
    want, over = oracle.bf16_to_f16(src)
    with Dev(ctx) as d:
        s = d.put(np.concatenate([np.zeros(8, np.uint16), src]))
        out = d.empty(src.nbytes + 64, fill=0xEE)
        counter = d.empty(16, fill=0)
        ctx.repack_part(out + shift, s + 16 + shift, src.nbytes - shift, capi.CONVERT_BF16_F16, counter)
        got = ctx.download(out, src.nbytes + 64, np.uint8)
        n_over = int(ctx.download(counter, 4, np.uint32)[0])
        k = shift // 2
        assert np.array_equal(got[shift:src.nbytes].view(np.uint16), want[k:])
        assert np.all(got[:shift] == 0xEE) and np.all(got[src.nbytes:] == 0xEE)
        _, over_tail = oracle.bf16_to_f16(src[k:])
        assert n_over == over_tail and over > 0
        ctx.repack_part(out, s + 16, 1024, capi.CONVERT_BF16_F16, counter)      # patterns 0..511: none overflows
        assert int(ctx.download(counter, 4, np.uint32)[0]) == over_tail


def test_bf16_to_f32_and_raw(ctx, capi, oracle):
    src = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    with Dev(ctx) as d:
        s = d.put(src)
        out = d.empty(src.nbytes * 2 + 32, fill=0)
        ctx.repack_part(out + 4, s + 2, src.nbytes - 2, capi.CONVERT_BF16_F32, 0)
        got = ctx.download(out, src.nbytes * 2 + 32, np.uint32)
        assert np.array_equal(got[1:65536], src[1:].astype(np.uint32) << 16) and got[0] == 0 and not got[65536:].any()
        raw = np.random.default_rng(1).integers(0, 256, 100003, dtype=np.uint8)
        r = d.put(raw)
        o2 = d.empty(raw.size + 64, fill=0x11)
        for dst_off, src_off, n in ((0, 0, 100000 // 16 * 16), (3, 1, 99991), (16, 5, 77)):
            ctx.fill(o2, 0x11, raw.size + 64)
            ctx.repack_part(o2 + dst_off, r + src_off, n, capi.CONVERT_RAW, 0)
            g = ctx.download(o2, raw.size + 64, np.uint8)
            assert np.array_equal(g[dst_off:dst_off + n], raw[src_off:src_off + n])
            assert np.all(g[:dst_off] == 0x11) and np.all(g[dst_off + n:] == 0x11)
        for bad in (dict(src_bytes=3, convert=capi.CONVERT_BF16_F16), dict(src_bytes=4, convert=7)):
            with pytest.raises(capi.ZtvmError):
                ctx.repack_part(o2, r, bad["src_bytes"], bad["convert"], 0)


@pytest.mark.parametrize("row_bytes", [1024, 64, 6, 3])
def test_permute_rows(ctx, capi, oracle, row_bytes):
    rng = np.random.default_rng(5)
    R, lora = 64, 512
    rows = lora + R
    src_rows = np.arange(rows)
    src_rows[lora:] = lora + np.array([oracle.deint(j, R) for j in range(R)])
    data = rng.integers(0, 256, rows * row_bytes, dtype=np.uint8)
    with Dev(ctx) as d:
        s = d.put(data)
        out = d.empty(data.size + 16, fill=0)
        ctx.repack_permute_rows(out, s, data.size, rows, src_rows)
        got = ctx.download(out, data.size + 16, np.uint8)
        assert np.array_equal(got[:data.size], oracle.permute_rows(data, rows, src_rows)) and not got[data.size:].any()
        for bad_rows, bad_map in ((rows, src_rows[:-1]), (rows - 1, src_rows[:-1]), (rows, np.r_[src_rows[:-1], rows])):
            if bad_rows == rows - 1 and data.size % (rows - 1) == 0:
                continue
            with pytest.raises(capi.ZtvmError):
                ctx.repack_permute_rows(out, s, data.size, bad_rows, bad_map)
        with pytest.raises(capi.ZtvmError):
            ctx.repack_permute_rows(s, s, data.size, rows, src_rows)      # in place would read rows already overwritten


@pytest.mark.parametrize("heads,nope,v,k", [(3, 16, 8, 128), (2, 128, 128, 512), (1, 5, 3, 64), (4, 7, 0, 64), (2, 0, 9, 192)])
def test_dequant_affine_split(ctx, oracle, synth, heads, nope, v, k):
    rows = heads * (nope + v)
    w = synth.packed_weights(rows, k, bits=4)
    s = synth.scales(rows, k, affine=True)
    b = synth.biases(rows, k, s, "B")
    want, over = oracle.dequant_affine_split(w, s, b, k, heads, nope, v)
    assert over == 0
    with Dev(ctx) as d:
        out = d.empty(want.nbytes + 32, fill=0)
        counter = d.empty(16, fill=0)
        ctx.repack_dequant_split(out, d.put(w), d.put(s), d.put(b), k, heads, nope, v, counter)
        got = ctx.download(out, want.nbytes + 32, np.uint16)
        assert np.array_equal(got[:want.size], want), "K^T blocks then V blocks, bit for bit"
        assert not got[want.size:].any() and int(ctx.download(counter, 4, np.uint32)[0]) == 0


def test_dequant_affine_split_counts_overflow(ctx, oracle):
    heads, nope, v, k = 1, 2, 2, 64
    w = np.full((4, 8), 0xFFFFFFFF, np.uint32)
    s = np.full((4, 1), np.float16(60000).view(np.uint16), np.uint16)
    s[3] = np.float16(1).view(np.uint16)
    b = np.zeros((4, 1), np.uint16)
    _, over = oracle.dequant_affine_split(w, s, b, k, heads, nope, v)
    with Dev(ctx) as d:
        counter = d.empty(16, fill=0)
        ctx.repack_dequant_split(d.empty(4 * 64 * 2, fill=0), d.put(w), d.put(s), d.put(b), k, heads, nope, v, counter)
        assert int(ctx.download(counter, 4, np.uint32)[0]) == over == 192


# ---------------------------------------------------------------- whole checkpoints --------------------------

def expected_bytes(oracle, plan, made):
    """What the reference's buildBuffer produces for this plan, by numpy (src/zero-tvm/mlx-weights.ts:490-543)."""
    pieces = []
    for part in plan.parts:
        dtype, _, data = made[part.record]
        raw = np.frombuffer(data, np.uint8)
        if part.convert == "raw" or (part.convert == "bf16->f16" and dtype == "F16") or (part.convert == "bf16->f32" and dtype == "F32"):
            pieces.append(raw)
        elif part.convert == "bf16->f16":
            out, over = oracle.bf16_to_f16(raw.view(np.uint16))
            assert over == 0
            pieces.append(out.view(np.uint8))
        else:
            pieces.append((raw.view(np.uint16).astype(np.uint32) << 16).view(np.uint8))
    op = plan.op
    if op is not None and op.kind == "dequantAffineSplit":
        out, over = oracle.dequant_affine_split(pieces[0].view(np.uint32), pieces[1].view(np.uint16), pieces[2].view(np.uint16),
                                                op.k, op.heads, op.nope, op.v)
        assert over == 0
        return out.view(np.uint8)
    cat = np.concatenate(pieces)
    if op is not None:
        cat = cat.reshape(op.rows, -1)[np.asarray(op.src)].ravel()
    return cat


def family(mw, name):
    if name == "qwen36":     # hybrid linear / full attention, MoE with a shared expert, 8-bit router, bf16 companions
        spec = mw.make_spec(id="qwen36-tiny", d=128, layers=4, heads=2, ffn=64, qkNorm=True, mlxPrefix="language_model.",
                            fullAttnInterval=4, moe=mw.Moe(experts=6, topK=2))
        dims = {"d": 128, "float": "BF16", "experts": 6, "gdn_heads": 6, "conv_rows": 24, "matrices": {
            "in_proj_qkv": (192, 128, 4), "in_proj_z": (128, 128, 4), "in_proj_a": (3, 128, 4), "in_proj_b": (3, 128, 4),
            "out_proj": (128, 128, 4), "q_proj": (256, 128, 4), "k_proj": (64, 128, 4), "v_proj": (64, 128, 4),
            "o_proj": (128, 128, 4), "switch_mlp.down_proj": (128, 64, 4), "shared_expert.down_proj": (128, 64, 4),
            "shared_expert_gate": (1, 128, 8), ".mlp.gate.": (6, 128, 8), "_proj": (64, 128, 4),
            "embed_tokens": (40, 128, 4), "lm_head": (40, 128, 4)}}
    elif name == "dsv2":     # MLA attention with both loader ops, dense layer 0, f16 router, f16 kv_a norm
        spec = mw.make_spec(id="dsv2-tiny", d=128, layers=2, heads=2, ffn=64,
                            mla=mw.Mla(kvLoraRank=64, qkNopeHeadDim=16, qkRopeHeadDim=8, vHeadDim=32),
                            moe=mw.Moe(experts=4, topK=2, normTopkProb=False, sharedExpert=True, routerBits=16,
                                       denseLayers=(0,), denseFfn=192))
        dims = {"d": 128, "float": "BF16", "experts": 4, "kv_lora": 64, "matrices": {
            "kv_a_proj_with_mqa": (72, 128, 4), "kv_b_proj": (96, 64, 4), "q_proj": (48, 128, 4), "o_proj": (128, 64, 4),
            "switch_mlp.down_proj": (128, 64, 4), "shared_expert.down_proj": (128, 64, 4),
            "shared_expert_gate": (1, 128, 16), ".mlp.gate.": (4, 128, 16),
            "layers.0.mlp.down_proj": (128, 192, 4), "layers.0.mlp": (192, 128, 4), "_proj": (64, 128, 4),
            "embed_tokens": (40, 128, 4), "lm_head": (40, 128, 4)}}
    else:                    # dense, tied embeddings, companions already f16 (pass-through, no conversion)
        spec = mw.make_spec(id="llama-tiny", d=128, layers=2, heads=2, ffn=256, tiedEmbeddings=True)
        dims = {"d": 128, "float": "F16", "matrices": {
            "q_proj": (128, 128, 4), "k_proj": (32, 128, 4), "v_proj": (32, 128, 4), "o_proj": (128, 128, 4),
            "down_proj": (128, 256, 4), "_proj": (256, 128, 4), "embed_tokens": (40, 128, 4)}}
    return spec, dims


@pytest.mark.parametrize("name", ["qwen36", "dsv2", "llama"])
def test_checkpoint_repack_is_byte_exact(mw, device, ctx, oracle, tmp_path, name):
    spec, dims = family(mw, name)
    plans = mw.plan_model(spec)
    made = mlx_synth.write_checkpoint(str(tmp_path), [p.record for plan, _ in plans for p in plan.parts], dims, seed=3)
    src = mw.FileSource(str(tmp_path))
    ck = mw.open_mlx_checkpoint(src)
    seen_ops = set()
    for plan, layer in plans:
        buf = mw.build_plan(device, plan, ck["locate"], src)
        try:
            want = expected_bytes(oracle, plan, made)
            assert buf.size == max(want.size, 4), mw.plan_key(plan, layer)
            assert want.size == mw.plan_bytes(plan, lambda r: len(made[r][2]), lambda r: made[r][0])
            got = ctx.download(buf.addr, want.size, np.uint8)
            assert np.array_equal(got, want), mw.plan_key(plan, layer)
        finally:
            buf.destroy()
        if plan.op is not None:
            seen_ops.add(plan.op.kind)
    if name == "dsv2":
        assert seen_ops == {"permuteRows", "dequantAffineSplit"}


def test_assemble_places_buffers_and_aliases_a_tied_head(mw, device, ctx, tmp_path):
    spec, dims = family(mw, "llama")
    plans = mw.plan_model(spec)
    made = mlx_synth.write_checkpoint(str(tmp_path), [p.record for plan, _ in plans for p in plan.parts], dims, seed=4)
    src = mw.FileSource(str(tmp_path))
    ck = mw.open_mlx_checkpoint(src)
    progress = []
    w = mw.assemble_mlx(device, spec, src, ck["locate"], on_buffer=lambda done, total, nbytes: progress.append((done, total)))
    try:
        assert progress[-1] == (len(plans), len(plans))
        assert w["lmHeadWeights"] is w["embdWeights"] and w["lmHeadScales"] is w["embdScales"]
        assert w["initNormGamma"] is w["layers"][0]["normGamma1"]
        qkv = w["layers"][1]["qkvWeights"]
        want = b"".join(made["model.layers.1.self_attn.%s_proj.weight" % n][2] for n in "qkv")
        assert ctx.download(qkv.addr, len(want), np.uint8).tobytes() == want
        assert set(w["layers"][0]) == {"normGamma1", "normGamma2", "qkvWeights", "qkvScales", "qkvBiases", "oProjWeights",
                                       "oProjScales", "oProjBiases", "ffnWeights", "ffnScales", "ffnBiases", "ffnDownWeights",
                                       "ffnDownScales", "ffnDownBiases"}
    finally:
        bufs = {id(b): b for b in list(w.values()) + [b for l in w["layers"] for b in l.values()] if hasattr(b, "destroy")}
        for b in bufs.values():
            b.destroy()


def test_build_buffer_error_behaviour(mw, device, ctx):
    """The loader's hard errors (src/zero-tvm/mlx-weights.ts:516-541): a companion of an unexpected dtype, and a
    bf16 value that does not fit f16."""
    plan = mw.BufferPlan("x_s", (mw.BufferPart("a.scales", "bf16->f16"),))
    big = np.array([0x7E96, 0x3F80] * 8, np.uint16).tobytes()      # 1e38 as bf16
    with pytest.raises(ValueError, match="8 bf16 value.*exceed f16 range"):
        mw.build_buffer(device, plan, lambda r: big)
    with pytest.raises(ValueError, match="is F32, expected BF16"):
        mw.build_buffer(device, plan, lambda r: big, lambda r: "F32")
    buf, over = mw.build_buffer(device, plan, lambda r: big, lambda r: "F16")     # already f16: passes through untouched
    try:
        assert over == 0 and ctx.download(buf.addr, len(big), np.uint8).tobytes() == big
    finally:
        buf.destroy()
    split = mw.BufferPlan("kvb", (mw.BufferPart("w", "raw"), mw.BufferPart("s", "bf16->f16")),
                          mw.DequantAffineSplit(k=64, heads=1, nope=1, v=1))
    with pytest.raises(ValueError, match="exactly \\[weight, scales, biases\\]"):
        mw.build_buffer(device, split, lambda r: b"\0" * 64)
