"""GPU parity of the remaining GEMV variants: symmetric group-32, f32 output, int3,
the MoE gathered GEMV (configs[3]) and the dequantization entry point."""
import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


def test_dequant_entry_bit_exact(ctx, capi, synth, oracle):
    """ztvm_dequant == oracle dequant (f32 and f16 forms), 4-bit affine / symmetric and 3-bit."""
    N, K = 96, 1024
    for bits, affine in ((4, True), (4, False), (3, True)):
        w = synth.packed_weights(N, K, bits=bits)
        s = synth.scales(N, K, affine=affine)
        b = synth.biases(N, K, s, "B") if affine else None
        o32, o16 = oracle.dequant_matrix(bits, affine, N, K, w, s, b, want="both")
        for out_f32, ref in ((1, o32.view(np.uint32)), (0, o16)):
            with Dev(ctx) as d:
                out = d.empty(N * K * (4 if out_f32 else 2))
                desc = capi.MatmulDesc(bits=bits, affine=int(affine), out_f32=out_f32, N=N, k_packed=K * bits // 32,
                                       scales_per_row=K // (64 if affine else 32), out=out, scales=d.put(s),
                                       weights=d.put(w), biases=d.put(b) if affine else 0)
                ctx.dequant(desc)
                got = ctx.download(out, N * K * (4 if out_f32 else 2), np.uint32 if out_f32 else np.uint16)
            assert np.array_equal(got.reshape(N, K), ref), (bits, affine, out_f32)


def test_dequant_extreme_scales_bit_exact(ctx, capi, oracle):
    """Every finite f16 scale with all 16 nibbles and a few biases, GPU vs oracle."""
    s_bits = np.array([h for h in range(65536) if (h >> 10) & 31 != 31], np.uint16)
    N, K = s_bits.size, 64
    q = np.tile(np.arange(16, dtype=np.uint8), 4)
    words = np.tile(oracle.pack(4, q), (N, 1))
    for bval in (0, 0x8000, 1, 0x3C00, 0xB266, 0x7BFF):
        b = np.full((N, 1), bval, np.uint16)
        ref = oracle.dequant_matrix(4, True, N, K, words, s_bits.reshape(N, 1), b, want="f16")
        with Dev(ctx) as d:
            out = d.empty(N * K * 2)
            desc = capi.MatmulDesc(bits=4, affine=1, N=N, k_packed=K // 8, scales_per_row=1, out=out,
                                   scales=d.put(s_bits), weights=d.put(words), biases=d.put(b))
            ctx.dequant(desc)
            got = ctx.download(out, N * K * 2, np.uint16).reshape(N, K)
        nan = (ref & 0x7FFF) > 0x7C00
        assert np.array_equal(got[~nan], ref[~nan])
        assert np.all((got[nan] & 0x7FFF) > 0x7C00)


@pytest.mark.parametrize("K,N", [(2048, 8192), (3072, 4096), (4096, 1000)])
@pytest.mark.parametrize("out_f32", [False, True])
def test_symmetric_g32(ctx, capi, synth, oracle, K, N, out_f32):
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K, affine=False)
    esz = 4 if out_f32 else 2
    with Dev(ctx) as d:
        out = d.empty(N * esz)
        desc = capi.MatmulDesc(bits=4, affine=0, out_f32=int(out_f32), M=1, N=N, k_packed=K // 8, scales_per_row=K // 32,
                               out=out, in_=d.put(x), scales=d.put(s), weights=d.put(w))
        ctx.matmul(desc)
        y = ctx.download(out, N * esz, np.float32 if out_f32 else np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, False, 1, N, K, x, w, s, None, threads=8)[0]
    assert rel_err(y, ref, 1e-2) < 1e-2
    if out_f32:  # LM-head logits keep f32 precision: error far below an f16 ulp of the typical output
        ref64 = oracle.gemm(oracle.MODE_FORMULA_F64, 4, False, 1, N, K, x, w, s, None, threads=8)[0]
        assert rel_err(y, ref64, 1.0) < 1e-5


def moe_case(synth, E, N, K, tokens, slots, bits, shared_input):
    w = synth.packed_weights(N, K, bits=bits, experts=E)
    s = synth.scales(N, K, experts=E)
    b = synth.biases(N, K, s, experts=E)
    ids = synth.topk_ids(tokens, slots, E)
    x = synth.activations(tokens if shared_input else tokens * slots, K)
    return w, s, b, ids, x


@pytest.mark.parametrize("tokens", [1, 16])
@pytest.mark.parametrize("bits", [4, 3])
def test_moe_block_config4(ctx, capi, synth, oracle, tokens, bits):
    """configs[3]: 256 experts, top-8, hidden 2048, expert intermediate 512.
    gate and up share the token's input and write interleaved halves of one
    [token][slot][2*ffn] buffer; down reads per-slot inputs
    (src/zero-tvm/engine-core.ts:1049-1056, :2038-2047)."""
    E, slots, d_model, ffn = 256, 8, 2048, 512
    with Dev(ctx) as d:
        # ---- gate / up: K = d_model, N = ffn, two dispatches into one buffer ----
        wg, sg, bg, ids, x = moe_case(synth, E, ffn, d_model, tokens, slots, bits, True)
        wu = synth.packed_weights(ffn, d_model, bits=bits, experts=E, salt=7)
        gu = d.empty(tokens * slots * 2 * ffn * 2, fill=0)
        d_ids, d_x, d_s, d_b = d.put(ids), d.put(x), d.put(sg), d.put(bg)
        common = dict(bits=bits, affine=1, M=1, N=ffn, k_packed=d_model * bits // 32, scales_per_row=d_model // 64,
                      slots=slots, tokens=tokens, in_slot_stride=0, out_slot_stride=2 * ffn, in_tok_stride=d_model,
                      out_tok_stride=slots * 2 * ffn, ids_stride=slots, experts=E, in_=d_x, scales=d_s, biases=d_b,
                      ids=d_ids)
        ctx.matmul(capi.MatmulDesc(out=gu, weights=d.put(wg), **common))
        ctx.matmul(capi.MatmulDesc(out=gu + ffn * 2, weights=d.put(wu), **common))
        got = ctx.download(gu, tokens * slots * 2 * ffn * 2, np.float16).astype(np.float64)
        strides = (0, 2 * ffn, d_model, slots * 2 * ffn, slots)
        ref = oracle.moe_gemv(oracle.MODE_FORMULA_F32, bits, ffn, d_model, tokens, slots, strides, ids, x, wg, sg, bg,
                              got.size, threads=8)
        refu = oracle.moe_gemv(oracle.MODE_FORMULA_F32, bits, ffn, d_model, tokens, slots, strides, ids, x, wu, sg, bg,
                               got.size + ffn, threads=8)
        g3 = got.reshape(tokens, slots, 2, ffn)
        assert rel_err(g3[:, :, 0], ref.reshape(tokens, slots, 2, ffn)[:, :, 0], 1e-2) < 1e-2
        assert rel_err(g3[:, :, 1], refu[: got.size].reshape(tokens, slots, 2, ffn)[:, :, 0], 1e-2) < 1e-2

        # ---- down: K = ffn, N = d_model, per-slot inputs ----
        wd, sd, bd, _, xd = moe_case(synth, E, d_model, ffn, tokens, slots, bits, False)
        out = d.empty(tokens * slots * d_model * 2, fill=0)
        desc = capi.MatmulDesc(bits=bits, affine=1, M=1, N=d_model, k_packed=ffn * bits // 32, scales_per_row=ffn // 64,
                               slots=slots, tokens=tokens, in_slot_stride=ffn, out_slot_stride=d_model,
                               in_tok_stride=slots * ffn, out_tok_stride=slots * d_model, ids_stride=slots, experts=E,
                               out=out, in_=d.put(xd), scales=d.put(sd), weights=d.put(wd), biases=d.put(bd), ids=d_ids)
        ctx.matmul(desc)
        gotd = ctx.download(out, tokens * slots * d_model * 2, np.float16).astype(np.float64)
        refd = oracle.moe_gemv(oracle.MODE_FORMULA_F32, bits, d_model, ffn, tokens, slots,
                               (ffn, d_model, slots * ffn, slots * d_model, slots), ids, xd, wd, sd, bd, gotd.size, threads=8)
        assert rel_err(gotd, refd, 1e-2) < 1e-2

        # ---- each pair equals the dense GEMV on the gathered expert slab, bit for bit ----
        t, sl = tokens - 1, 3
        e = int(ids[t, sl])
        dense_out = d.empty(d_model * 2)
        dd = capi.MatmulDesc(bits=bits, affine=1, M=1, N=d_model, k_packed=ffn * bits // 32, scales_per_row=ffn // 64,
                             out=dense_out, in_=d.put(xd[t * slots + sl]), scales=d.put(sd[e]), weights=d.put(wd[e]),
                             biases=d.put(bd[e]))
        ctx.matmul(dd)
        dense = ctx.download(dense_out, d_model * 2, np.uint16)
        pair = ctx.download(out, d_model * 2, np.uint16, offset=(t * slots + sl) * d_model * 2)
        assert np.array_equal(dense, pair)


def test_moe_out_of_range_expert_is_skipped(ctx, capi, synth):
    """A bad id must not fault the GPU: its pair is left untouched."""
    E, N, K = 4, 64, 256
    w, s = synth.packed_weights(N, K, experts=E), synth.scales(N, K, experts=E)
    b = synth.biases(N, K, s, experts=E)
    ids = np.array([[1, 9999]], np.uint32)
    with Dev(ctx) as d:
        out = d.empty(2 * N * 2, fill=0x11)
        desc = capi.MatmulDesc(bits=4, affine=1, M=1, N=N, k_packed=K // 8, scales_per_row=K // 64, slots=2, tokens=1,
                               in_slot_stride=0, out_slot_stride=N, in_tok_stride=K, out_tok_stride=2 * N, ids_stride=2,
                               experts=E, out=out, in_=d.put(synth.activations(1, K)), scales=d.put(s), weights=d.put(w),
                               biases=d.put(b), ids=d.put(ids))
        ctx.matmul(desc)
        got = ctx.download(out, 2 * N * 2, np.uint16)
    assert np.all(got[N:] == 0x1111) and not np.all(got[:N] == 0x1111)


def test_command_buffer_replay_matches_eager(ctx, capi, synth):
    """Recorded dispatches replay to the same bytes as eager ones, on every replay."""
    K, N = 4096, 512
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    with Dev(ctx) as d:
        out = d.empty(N * 2)
        desc = capi.MatmulDesc(bits=4, affine=1, M=1, N=N, k_packed=K // 8, scales_per_row=K // 64, out=out,
                               in_=d.put(x), scales=d.put(s), weights=d.put(w), biases=d.put(b))
        ctx.matmul(desc)
        eager = ctx.download(out, N * 2, np.uint16)
        ctx.record_begin()
        ctx.fill(out, 0, N * 2)
        ctx.matmul(desc)
        cb = ctx.record_end()
        for _ in range(4):
            ctx.fill(out, 0x7F, N * 2)
            ctx.sync()
            ctx.submit(cb)
            assert np.array_equal(ctx.download(out, N * 2, np.uint16), eager)
        ctx.cmdbuf_destroy(cb)
        with pytest.raises(capi.ZtvmError):
            ctx.record_begin()
            try:
                ctx.sync()
            finally:
                ctx.cmdbuf_destroy(ctx.record_end())
