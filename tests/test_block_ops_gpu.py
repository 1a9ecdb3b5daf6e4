"""GPU parity of the dispatches either side of the matmuls in a MoE / FFN block, through the C ABI.

Shapes and bars follow the reference's own kernel tests:
  silu_mul            tests/kernels/compile-qwen35.mjs:1583-1605   SEQ=3 rows of the model's ffn, max abs err < 5e-3
  moe_router_logits*  tests/kernels/run.mjs:199-280                9 rows x D=2048, 8 / 4 / 16 bits, rel err < 1e-4 (eps 1e-2)
  moe_router_topk     tests/kernels/run.mjs:284-343, :1205-1207    (256,8,norm,shared) (128,8,norm,-) (128,8,-,-): indices
                                                                   equal, score err < 2e-6, slot K untouched without a shared expert
  moe_combine         src/compiler/shaders/moe_combine.wgsl        f32 accumulation in slot order
plus ragged, multi-token and edge cases the engine dispatches (chunked prefill puts the token in the grid).
"""
import numpy as np
import pytest

from .util import Dev, f16

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------- silu_mul -----------------------------------

@pytest.mark.parametrize("rows,ffn", [(3, 9216), (1, 512), (9, 768), (5, 100), (2, 7), (512, 14336)])
def test_silu_mul(ctx, oracle, rows, ffn):
    rng = np.random.default_rng(38 + rows)
    gu = (rng.random((rows, 2 * ffn)) * 6 - 3).astype(np.float16)
    gu.ravel()[:6] = [0, -0.0, 30, -30, 65504, -65504]
    with Dev(ctx) as d:
        out = d.empty((rows + 1) * ffn * 2, fill=0)
        ctx.silu_mul(out, d.put(gu), rows, ffn)
        got = ctx.download(out, (rows + 1) * ffn * 2, np.uint16).reshape(rows + 1, ffn)
    ref64, ref16 = oracle.silu_mul(gu.view(np.uint16), rows, ffn)
    y = f16(got[:rows])
    with np.errstate(invalid="ignore"):
        ok = np.isfinite(ref64) & (np.abs(ref64) < 65504)
    assert np.max(np.abs(y[ok] - ref64[ok])) < 5e-3 or np.max(np.abs(y[ok] - ref64[ok]) / (np.abs(ref64[ok]) + 1)) < 1e-3
    # against the f32 form of the shader: identical up to one f16 step where the two exp() differ in the last bit
    step = np.abs(got[:rows].astype(np.int32) - ref16.astype(np.int32))
    assert step.max() <= 1 and (step != 0).mean() < 1e-3
    assert not got[rows].any(), "wrote past the last row"


def test_silu_mul_zero_rows_dispatches_nothing(ctx):
    with Dev(ctx) as d:
        out = d.empty(64, fill=0x5A)
        ctx.silu_mul(out, d.empty(256, fill=0), 0, 32)
        assert np.all(ctx.download(out, 64, np.uint8) == 0x5A)


# ---------------------------------------------------------------- moe_combine --------------------------------

@pytest.mark.parametrize("tokens,N,S", [(1, 2048, 9), (1, 2048, 8), (16, 2048, 9), (3, 100, 5), (2, 7, 1), (64, 4096, 3)])
def test_moe_combine(ctx, oracle, tokens, N, S):
    rng = np.random.default_rng(tokens * 100 + S)
    slots = rng.standard_normal((tokens, S, N)).astype(np.float16)
    score = rng.random((tokens, S)).astype(np.float32)
    with Dev(ctx) as d:
        out = d.empty((tokens + 1) * N * 2, fill=0)
        ctx.moe_combine(out, d.put(slots), d.put(score), tokens, N, S)
        got = ctx.download(out, (tokens + 1) * N * 2, np.uint16).reshape(tokens + 1, N)
    ref64, ref16 = oracle.moe_combine(slots.view(np.uint16), score, tokens, N, S)
    assert np.array_equal(got[:tokens], ref16), "f32 accumulation in slot order is bit-exact"
    assert np.max(np.abs(f16(got[:tokens]) - ref64)) <= np.max(np.abs(ref64)) * 2.0 ** -10
    assert not got[tokens].any()


# ---------------------------------------------------------------- router logits ------------------------------

def router_case(bits, D, rows, tokens, seed):
    rng = np.random.default_rng(seed)
    x = (rng.random((tokens, D)) * 2 - 1).astype(np.float16)
    if bits == 16:
        w = (rng.random((rows, D)) * 0.1 - 0.05).astype(np.float16).view(np.uint16)
        return x, w, None, None
    w = rng.integers(0, 2 ** 32, (rows, D * bits // 32), dtype=np.uint64).astype(np.uint32)
    s = (rng.random((rows, D // 64)) * 0.02 + 0.005).astype(np.float16)
    b = (rng.random((rows, D // 64)) * 0.2 - 0.1).astype(np.float16)
    return x, w, s, b


@pytest.mark.parametrize("bits", [8, 4, 16])
@pytest.mark.parametrize("D,rows,tokens", [(2048, 9, 1), (2048, 257, 1), (2048, 128, 5), (4096, 65, 19), (64, 3, 2), (1024, 7, 8)])
def test_router_logits(ctx, oracle, bits, D, rows, tokens):
    x, w, s, b = router_case(bits, D, rows, tokens, 11 + bits)
    with Dev(ctx) as d:
        out = d.empty((tokens * rows + 4) * 4, fill=0xFF)
        ctx.moe_router_logits(out, d.put(x), d.put(w), d.put(s) if s is not None else 0, d.put(b) if b is not None else 0,
                              bits, D, rows, tokens)
        got = ctx.download(out, (tokens * rows + 4) * 4, np.float32)
    ref = oracle.router_logits(bits, D, rows, tokens, x.view(np.uint16), w, None if s is None else s.view(np.uint16),
                               None if b is None else b.view(np.uint16))
    y = got[:tokens * rows].astype(np.float64).reshape(tokens, rows)
    err = np.abs(y - ref)
    if rows == 9:   # the reference test's own shape and bar
        assert np.max(err / (np.abs(ref) + 1e-2)) < 1e-4
    # many more outputs than the reference checks: some logits cancel to ~0.1 out of group terms that sum to
    # ~100, so f32 accumulation (the shader's too) leaves an absolute error of a few 2^-24 of the largest logit
    assert np.all(err <= 1e-4 * (np.abs(ref) + 1e-2) + 2.0 ** -22 * np.max(np.abs(ref)))
    assert np.all(got[tokens * rows:].view(np.uint32) == 0xFFFFFFFF), "wrote past the last logit"


def test_router_logits_rejects_bad_shapes(ctx, capi):
    with Dev(ctx) as d:
        p = d.empty(4096, fill=0)
        for kw in (dict(bits=5, D=2048), dict(bits=8, D=2000), dict(bits=16, D=100)):
            with pytest.raises(capi.ZtvmError):
                ctx.moe_router_logits(p, p, p, p, p, kw["bits"], kw["D"], 4, 1)
        with pytest.raises(capi.ZtvmError):
            ctx.moe_router_logits(p, p, p, 0, 0, 8, 2048, 4, 1)   # quantized router without scales


# ---------------------------------------------------------------- router top-k -------------------------------

POISON_I, POISON_F = 0xDEADBEEF, np.float32(-999)


def run_topk(ctx, logits, tokens, E, K, norm, shared):
    stride = K + (1 if shared else 0)
    with Dev(ctx) as d:
        idx = d.put(np.full(tokens * stride + 1, POISON_I, np.uint32))
        sc = d.put(np.full(tokens * stride + 1, POISON_F, np.float32))
        ctx.moe_router_topk(idx, sc, d.put(logits), E, K, norm, shared, tokens)
        gi = ctx.download(idx, (tokens * stride + 1) * 4, np.uint32)
        gs = ctx.download(sc, (tokens * stride + 1) * 4, np.float32)
    return gi, gs


@pytest.mark.parametrize("E,K,norm,shared", [(256, 8, True, True), (128, 8, True, False), (128, 8, False, False),
                                             (64, 6, False, True), (60, 4, True, True), (8, 8, False, False),
                                             (512, 32, True, True), (300, 64, True, False), (1, 1, True, True)])
@pytest.mark.parametrize("tokens", [1, 7])
def test_router_topk(ctx, oracle, E, K, norm, shared, tokens):
    rng = np.random.default_rng(7 + E + tokens)
    rows = E + (1 if shared else 0)
    logits = (rng.random((tokens, rows)) * 8 - 4).astype(np.float32)
    gi, gs = run_topk(ctx, logits, tokens, E, K, norm, shared)
    ri, rs = oracle.router_topk(logits, tokens, E, K, norm, shared)
    n = ri.size
    assert np.array_equal(gi[:n].reshape(ri.shape), ri)
    assert np.max(np.abs(gs[:n].reshape(rs.shape).astype(np.float64) - rs)) < 2e-6
    assert gi[n] == POISON_I and gs[n] == POISON_F, "the slot past the block must stay untouched"
    if norm:
        stride = K + (1 if shared else 0)
        assert np.allclose(gs[:n].reshape(tokens, stride)[:, :K].sum(1), 1.0, atol=1e-5)


def test_router_topk_ties_go_to_the_lower_index(ctx):
    E, K = 200, 5
    logits = np.zeros((1, E), np.float32)
    logits[0, [150, 3, 67, 130]] = 2.0     # equal maxima held by different lanes and register slots
    gi, gs = run_topk(ctx, logits, 1, E, K, False, False)
    assert list(gi[:K]) == [3, 67, 130, 150, 0]
    assert gs[0] == gs[1] == gs[2] == gs[3] > gs[4]


def test_router_topk_rejects(ctx, capi):
    with Dev(ctx) as d:
        p = d.empty(4096, fill=0)
        for E, K in ((0, 1), (513, 8), (8, 9), (256, 65), (256, 0)):
            with pytest.raises(capi.ZtvmError):
                ctx.moe_router_topk(p, p, p, E, K, 1, 0, 1)


# ---------------------------------------------------------------- slot translate -----------------------------

def test_slot_translate(ctx, oracle, capi):
    m = np.array([5, 0xFFFFFFFF, 2, 7, 0xFFFFFFFF, 0, 9, 1], np.uint32)
    ids = np.array([0, 1, 2, 3, 4, 5, 3, 7, 6], np.uint32)
    with Dev(ctx) as d:
        out = d.put(np.full(ids.size + 1, POISON_I, np.uint32))
        ctx.moe_slot_translate(out, d.put(ids), d.put(m), ids.size, m.size)
        got = ctx.download(out, (ids.size + 1) * 4, np.uint32)
        assert np.array_equal(got[:-1], oracle.slot_translate(ids, m)) and got[-1] == POISON_I
        bad = np.array([2, 1000, 3], np.uint32)     # an id past the map is a miss, not a fault
        ctx.moe_slot_translate(out, d.put(bad), d.put(m), 3, m.size)
        assert list(ctx.download(out, 12, np.uint32)) == [2, 0, 7]
        with pytest.raises(capi.ZtvmError):
            ctx.moe_slot_translate(out, out, d.put(m), 3, m.size)


# ---------------------------------------------------------------- a whole routed FFN block -------------------

def test_moe_block_end_to_end(ctx, capi, synth, oracle):
    """router logits -> top-k -> gate / up (gathered GEMV) -> silu_mul -> down -> combine, the dispatch
    sequence of src/zero-tvm/engine-core.ts:2329-2349, for 3 tokens, against the oracle run stage by stage in
    float64 on the same expert choice."""
    D, F, E, K, tokens = 512, 256, 16, 4, 3
    S = K + 1
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((tokens, D)) * 0.5).astype(np.float16)
    _, rw, rs, _ = router_case(8, D, E + 1, tokens, 5)
    rs = (rs.astype(np.float32) * 0.02).astype(np.float16)       # centred router weights: logits of order 1,
    rb = (-127.5 * rs.astype(np.float32)).astype(np.float16)     # so every top-k probability is far above f32 underflow
    wg, wu = synth.packed_weights((E + 1) * F, D, bits=4), synth.packed_weights((E + 1) * F, D, bits=4, salt=2)
    sg, su = synth.scales((E + 1) * F, D, affine=True), synth.scales((E + 1) * F, D, affine=True, salt=2)
    bg, bu = synth.biases((E + 1) * F, D, sg, "A"), synth.biases((E + 1) * F, D, su, "A", salt=2)
    wd = synth.packed_weights((E + 1) * D, F, bits=4, salt=3)
    sd = synth.scales((E + 1) * D, F, affine=True, salt=3)
    bd = synth.biases((E + 1) * D, F, sd, "A", salt=3)
    with Dev(ctx) as d:
        X = d.put(x)
        logits = d.empty(tokens * (E + 1) * 4, fill=0)
        ids, score = d.empty(tokens * S * 4, fill=0), d.empty(tokens * S * 4, fill=0)
        gate_up = d.empty(tokens * S * 2 * F * 2, fill=0)
        h = d.empty(tokens * S * F * 2, fill=0)
        down = d.empty(tokens * S * D * 2, fill=0)
        y = d.empty(tokens * D * 2, fill=0)
        ctx.moe_router_logits(logits, X, d.put(rw), d.put(rs), d.put(rb), 8, D, E + 1, tokens)
        ctx.moe_router_topk(ids, score, logits, E, K, True, True, tokens)
        common = dict(bits=4, affine=1, M=1, slots=S, tokens=tokens, ids=ids, ids_stride=S, experts=E + 1,
                      kernel=capi.KERNEL_GEMV)
        for W, Sc, B, off in ((wg, sg, bg, 0), (wu, su, bu, F)):
            ctx.matmul(capi.MatmulDesc(N=F, k_packed=D // 8, scales_per_row=D // 64, in_slot_stride=0, in_tok_stride=D,
                                       out_slot_stride=2 * F, out_tok_stride=S * 2 * F, out=gate_up + off * 2, in_=X,
                                       weights=d.put(W), scales=d.put(Sc), biases=d.put(B), **common))
        ctx.silu_mul(h, gate_up, tokens * S, F)
        ctx.matmul(capi.MatmulDesc(N=D, k_packed=F // 8, scales_per_row=F // 64, in_slot_stride=F, in_tok_stride=S * F,
                                   out_slot_stride=D, out_tok_stride=S * D, out=down, in_=h, weights=d.put(wd),
                                   scales=d.put(sd), biases=d.put(bd), **common))
        ctx.moe_combine(y, down, score, tokens, D, S)
        got_ids = ctx.download(ids, tokens * S * 4, np.uint32).reshape(tokens, S)
        got_score = ctx.download(score, tokens * S * 4, np.float32).reshape(tokens, S)
        got = f16(ctx.download(y, tokens * D * 2, np.uint16)).reshape(tokens, D)
    # the oracle, stage by stage
    lg = oracle.router_logits(8, D, E + 1, tokens, x.view(np.uint16), rw, rs.view(np.uint16), rb.view(np.uint16))
    ri, rsc = oracle.router_topk(lg.astype(np.float32), tokens, E, K, True, True)
    assert np.array_equal(got_ids, ri) and np.max(np.abs(got_score - rsc)) < 1e-5
    Wg = oracle.dequant_matrix(4, True, (E + 1) * F, D, wg, sg, bg).astype(np.float64).reshape(E + 1, F, D)
    Wu = oracle.dequant_matrix(4, True, (E + 1) * F, D, wu, su, bu).astype(np.float64).reshape(E + 1, F, D)
    Wd = oracle.dequant_matrix(4, True, (E + 1) * D, F, wd, sd, bd).astype(np.float64).reshape(E + 1, D, F)
    xf = x.astype(np.float64)
    ref = np.zeros((tokens, D))
    for t in range(tokens):
        for s in range(S):
            e = int(ri[t, s])
            g = (Wg[e] @ xf[t]).astype(np.float16).astype(np.float64)
            u = (Wu[e] @ xf[t]).astype(np.float16).astype(np.float64)
            hh = (u * g / (1 + np.exp(-g))).astype(np.float16).astype(np.float64)
            dn = (Wd[e] @ hh).astype(np.float16).astype(np.float64)
            ref[t] += float(rsc[t, s]) * dn
    assert np.max(np.abs(got - ref) / (np.abs(ref) + 1e-2)) < 2e-2


# ---------------------------------------------------------------- gate + up + SiLU in one pass ---------------

def gated_reference(oracle, bits, affine, N, K, x_bits, wg, sg, bg, wu, su, bu):
    """float64: up * silu(gate) on the dequantized matrices, nothing rounded in between
    (src/compiler/shaders/fused_ffn.wgsl:128-139 keeps both sums in f32 until the store)."""
    Wg = oracle.dequant_matrix(bits, affine, N, K, wg, sg, bg).astype(np.float64)
    Wu = oracle.dequant_matrix(bits, affine, N, K, wu, su, bu).astype(np.float64)
    x = np.asarray(x_bits, np.uint16).view(np.float16).astype(np.float64)
    g, u = x @ Wg.T, x @ Wu.T
    return u * g / (1 + np.exp(-g))


@pytest.mark.parametrize("bits,affine", [(4, False), (4, True), (3, True)])
@pytest.mark.parametrize("M,N,K", [(1, 9216, 2560), (1, 100, 512), (3, 130, 1024), (1, 64, 64)])
def test_ffn_gated_dense(ctx, capi, synth, oracle, bits, affine, M, N, K):
    """The reference's fused FFN layout: ONE [2N, K] buffer, gate rows then up rows."""
    x = synth.activations(M, K)
    w = synth.packed_weights(2 * N, K, bits=bits)
    s = synth.scales(2 * N, K, affine=affine)
    b = synth.biases(2 * N, K, s, "A") if affine else None
    kp, spr = K * bits // 32, K // (64 if affine else 32)
    with Dev(ctx) as d:
        out = d.empty((M + 1) * N * 2, fill=0)
        W, S, B = d.put(w), d.put(s), (d.put(b) if affine else 0)
        desc = capi.MatmulDesc(bits=bits, affine=int(affine), M=M, N=N, k_packed=kp, scales_per_row=spr, out=out, in_=d.put(x),
                               weights=W, scales=S, biases=B)
        ctx.ffn_gated(desc, W + N * kp * 4, S + N * spr * 2, B + N * spr * 2 if affine else 0)
        got = ctx.download(out, (M + 1) * N * 2, np.uint16).reshape(M + 1, N)
    ref = gated_reference(oracle, bits, affine, N, K, x, w[:N], s[:N], b[:N] if affine else None, w[N:], s[N:],
                          b[N:] if affine else None)
    assert np.max(np.abs(f16(got[:M]) - ref) / (np.abs(ref) + 1e-2)) < 1e-2
    assert not got[M].any()


def _prologue_run(ctx, capi, bits, affine, N, K, res, dlt, gam, eps, w, s, b, normed):
    kp, spr = K * bits // 32, K // (64 if affine else 32)
    with Dev(ctx) as d:
        out, out2 = d.empty(2 * N * 2, fill=0), d.empty(N * 2, fill=0)
        W, S, B = d.put(w), d.put(s), (d.put(b) if affine else 0)
        common = dict(bits=bits, affine=int(affine), M=1, N=N, k_packed=kp, scales_per_row=spr, weights=W, scales=S, biases=B)
        ups = (W + N * kp * 4, S + N * spr * 2, B + N * spr * 2 if affine else 0)
        ctx.ffn_gated_prologue(capi.MatmulDesc(out=out, in_=d.put(res), **common), *ups, d.put(dlt), d.put(gam), eps)
        ctx.ffn_gated(capi.MatmulDesc(out=out2, in_=d.put(normed), **common), *ups)
        got = ctx.download(out, 2 * N * 2, np.uint16).reshape(2, N)
        return got, ctx.download(out2, N * 2, np.uint16)


def test_ffn_gated_prologue_reference_case(ctx, capi, oracle):
    """The reference's own test of the kernel (tests/kernels/run.mjs:1021-1072): Phi-3 width, eight output rows,
    residual and delta uniform in +-0.75, gamma in 0.75..1.25, scales in 0.01..0.06, float64 sum of squares in the
    reference, bar |got-ref| / (|ref| + 1e-3) < 2e-2."""
    rng = np.random.default_rng(8)
    K, N, eps = 3072, 8, 1e-5
    res = (rng.random(K) * 1.5 - 0.75).astype(np.float16)
    dlt = (rng.random(K) * 1.5 - 0.75).astype(np.float16)
    gam = (rng.random(K) * 0.5 + 0.75).astype(np.float16)
    w = rng.integers(0, 2 ** 32, (2 * N, K // 8), dtype=np.uint64).astype(np.uint32)
    s = (rng.random((2 * N, K // 32)) * 0.05 + 0.01).astype(np.float16).view(np.uint16)
    summed = (res.astype(np.float32) + dlt.astype(np.float32)).astype(np.float16).astype(np.float64)
    normed64 = (summed / np.sqrt(np.mean(summed * summed) + eps) * gam.astype(np.float64)).astype(np.float16)
    got, _ = _prologue_run(ctx, capi, 4, False, N, K, res, dlt, gam, eps, w, s, None, normed64.view(np.uint16))
    ref = gated_reference(oracle, 4, False, N, K, normed64.view(np.uint16).reshape(1, K), w[:N], s[:N], None, w[N:], s[N:], None)[0]
    assert np.max(np.abs(f16(got[0]) - ref) / (np.abs(ref) + 1e-3)) < 2e-2


@pytest.mark.parametrize("bits,affine", [(4, False), (4, True), (3, True)])
@pytest.mark.parametrize("N,K", [(8192, 3072), (100, 512), (64, 64), (130, 14336)])
def test_ffn_gated_prologue(ctx, capi, synth, oracle, bits, affine, N, K):
    """The fused FFN with the add + RMSNorm prologue at the reference kernel's shape (D = 3072, FFN_DIM = 8192) and
    others, against the float64 reference on the oracle's normed vector and against the plain gated form fed that
    vector. The normed vector is f16 and the sum of squares is f32: its summation order (index order in the oracle, a
    tree in the kernel, another tree in the shader) moves 1/sqrt by a few f32 steps, which flips the f16 rounding of a
    handful of the K normed values by one step. An output near zero whose up factor is large sees that as an absolute
    error, so the floor of the relative bar is tied to the output scale: |got-ref| / (|ref| + 0.05*rms(ref)) < 1e-2."""
    rng = np.random.default_rng(N + K)
    res = rng.standard_normal(K).astype(np.float16)
    dlt = (rng.standard_normal(K) * 0.3).astype(np.float16)
    gam = (1 + 0.1 * rng.standard_normal(K)).astype(np.float16)
    eps = 1e-5
    w = synth.packed_weights(2 * N, K, bits=bits)
    s = synth.scales(2 * N, K, affine=affine)
    b = synth.biases(2 * N, K, s, "A") if affine else None
    normed = oracle.add_rmsnorm(res.view(np.uint16), dlt.view(np.uint16), gam.view(np.uint16), eps)
    got, two_step = _prologue_run(ctx, capi, bits, affine, N, K, res, dlt, gam, eps, w, s, b, normed)
    ref = gated_reference(oracle, bits, affine, N, K, normed.reshape(1, K), w[:N], s[:N], b[:N] if affine else None, w[N:], s[N:],
                          b[N:] if affine else None)[0]
    floor = 0.05 * np.sqrt(np.mean(ref * ref))
    assert np.max(np.abs(f16(got[0]) - ref) / (np.abs(ref) + floor)) < 1e-2
    assert not got[1].any()
    assert np.max(np.abs(f16(got[0]) - f16(two_step)) / (np.abs(f16(two_step)) + floor)) < 2e-3
    # and most outputs are the same f16 value as the two-dispatch form gives
    assert np.mean(got[0] == two_step) > 0.9


def test_ffn_gated_prologue_rejects(ctx, capi):
    p = 0x10000
    desc = capi.MatmulDesc(bits=4, affine=0, M=1, N=64, k_packed=64, scales_per_row=16, out=p, in_=p, weights=p, scales=p)
    for kw, args, needle in ((dict(), (p, p, 0, 0, p, 1e-5), "delta and gamma"), (dict(), (p, p, 0, p, p + 2, 1e-5), "aligned"),
                             (dict(M=2), (p, p, 0, p, p, 1e-5), "one dense activation row"),
                             (dict(), (p, p, 0, p, p, -1.0), "rms_eps"),
                             (dict(bits=8, affine=1, k_packed=128, scales_per_row=8, biases=p), (p, p, p, p, p, 1e-5), "8-bit")):
        dsc = capi.MatmulDesc(**{**{f[0]: getattr(desc, f[0]) for f in desc._fields_}, **kw})
        with pytest.raises(capi.ZtvmError, match=needle):
            ctx.ffn_gated_prologue(dsc, *args)


def test_ffn_gated_moe_matches_three_dispatches(ctx, capi, synth, oracle):
    """Per (token, slot) pair on expert stacks: the one-pass form against gate, up and silu_mul dispatched
    separately (which round gate and up to f16 in between) and against the float64 formula."""
    D, F, E, S, tokens = 512, 192, 6, 3, 4
    x = synth.activations(tokens, D)
    wg, wu = synth.packed_weights(E * F, D), synth.packed_weights(E * F, D, salt=2)
    sg, su = synth.scales(E * F, D), synth.scales(E * F, D, salt=2)
    bg, bu = synth.biases(E * F, D, sg, "B"), synth.biases(E * F, D, su, "B", salt=2)
    ids = synth.topk_ids(tokens, S, E)
    ids[1, 2] = 99      # a bad id: that pair is skipped by every dispatch
    with Dev(ctx) as d:
        X, IDS = d.put(x), d.put(ids)
        WG, SG, BG, WU, SU, BU = (d.put(a) for a in (wg, sg, bg, wu, su, bu))
        gate_up = d.empty(tokens * S * 2 * F * 2, fill=0)
        h3, h1 = d.empty(tokens * S * F * 2, fill=0), d.empty(tokens * S * F * 2, fill=0)
        common = dict(bits=4, affine=1, M=1, N=F, k_packed=D // 8, scales_per_row=D // 64, slots=S, tokens=tokens,
                      ids=IDS, ids_stride=S, experts=E, in_=X, in_slot_stride=0, in_tok_stride=D)
        ctx.matmul(capi.MatmulDesc(out=gate_up, out_slot_stride=2 * F, out_tok_stride=S * 2 * F, weights=WG, scales=SG, biases=BG, **common))
        ctx.matmul(capi.MatmulDesc(out=gate_up + F * 2, out_slot_stride=2 * F, out_tok_stride=S * 2 * F, weights=WU, scales=SU, biases=BU, **common))
        ctx.silu_mul(h3, gate_up, tokens * S, F)
        ctx.ffn_gated(capi.MatmulDesc(out=h1, out_slot_stride=F, out_tok_stride=S * F, weights=WG, scales=SG, biases=BG, **common), WU, SU, BU)
        a = f16(ctx.download(h3, tokens * S * F * 2, np.uint16)).reshape(tokens, S, F)
        b = f16(ctx.download(h1, tokens * S * F * 2, np.uint16)).reshape(tokens, S, F)
    assert not b[1, 2].any() and not a[1, 2].any()
    assert np.max(np.abs(a - b) / (np.abs(b) + 1e-2)) < 1e-2
    for t in range(tokens):
        for s in range(S):
            e = int(ids[t, s])
            if e >= E:
                continue
            sl = slice(e * F, (e + 1) * F)
            ref = gated_reference(oracle, 4, True, F, D, x[t:t + 1], wg[sl], sg[sl], bg[sl], wu[sl], su[sl], bu[sl])[0]
            assert np.max(np.abs(b[t, s] - ref) / (np.abs(ref) + 1e-2)) < 1e-2, (t, s)


def test_ffn_gated_rejects(ctx, capi):
    with Dev(ctx) as d:
        p = d.empty(1 << 16, fill=0)
        desc = capi.MatmulDesc(bits=4, affine=1, M=1, N=64, k_packed=8, scales_per_row=1, out=p, in_=p, weights=p, scales=p, biases=p)
        with pytest.raises(capi.ZtvmError):
            ctx.ffn_gated(desc, p, p, 0)                       # affine without up biases
        with pytest.raises(capi.ZtvmError):
            ctx.ffn_gated(desc, 0, p, p)
        desc.kernel = capi.KERNEL_GEMM
        with pytest.raises(capi.ZtvmError):
            ctx.ffn_gated(desc, p, p, p)


# ---------------------------------------------------------------- recorded replay ----------------------------

def test_recorded_block_replays_match_eager(ctx, capi, synth, oracle):
    """The whole routed FFN (five dispatches with the gated form) recorded into one command buffer and replayed
    with new activations each time: every replay equals the eager result bit for bit, including the routing."""
    D, F, E, K, tokens = 512, 256, 12, 3, 2
    S = K + 1
    _, rw, rs, _ = router_case(8, D, E + 1, tokens, 5)
    rs = (rs.astype(np.float32) * 0.02).astype(np.float16)
    rb = (-127.5 * rs.astype(np.float32)).astype(np.float16)
    wg, wu, wd = (synth.packed_weights((E + 1) * F, D), synth.packed_weights((E + 1) * F, D, salt=2),
                  synth.packed_weights((E + 1) * D, F, salt=3))
    sg, su, sd = (synth.scales((E + 1) * F, D), synth.scales((E + 1) * F, D, salt=2), synth.scales((E + 1) * D, F, salt=3))
    bg, bu, bd = synth.biases((E + 1) * F, D, sg), synth.biases((E + 1) * F, D, su, salt=2), synth.biases((E + 1) * D, F, sd, salt=3)
    with Dev(ctx) as d:
        X = d.empty(tokens * D * 2, fill=0)
        logits, ids, score = d.empty(tokens * (E + 1) * 4, fill=0), d.empty(tokens * S * 4, fill=0), d.empty(tokens * S * 4, fill=0)
        h, down, y = d.empty(tokens * S * F * 2, fill=0), d.empty(tokens * S * D * 2, fill=0), d.empty(tokens * D * 2, fill=0)
        RW, RS, RB = d.put(rw), d.put(rs), d.put(rb)
        WG, SG, BG, WU, SU, BU, WD, SD, BD = (d.put(a) for a in (wg, sg, bg, wu, su, bu, wd, sd, bd))
        common = dict(bits=4, affine=1, M=1, slots=S, tokens=tokens, ids=ids, ids_stride=S, experts=E + 1)
        gate = capi.MatmulDesc(N=F, k_packed=D // 8, scales_per_row=D // 64, in_slot_stride=0, in_tok_stride=D, out_slot_stride=F,
                               out_tok_stride=S * F, out=h, in_=X, weights=WG, scales=SG, biases=BG, **common)
        dn = capi.MatmulDesc(N=D, k_packed=F // 8, scales_per_row=F // 64, in_slot_stride=F, in_tok_stride=S * F,
                             out_slot_stride=D, out_tok_stride=S * D, out=down, in_=h, weights=WD, scales=SD, biases=BD, **common)

        def block():
            ctx.moe_router_logits(logits, X, RW, RS, RB, 8, D, E + 1, tokens)
            ctx.moe_router_topk(ids, score, logits, E, K, True, True, tokens)
            ctx.ffn_gated(gate, WU, SU, BU)
            ctx.matmul(dn)
            ctx.moe_combine(y, down, score, tokens, D, S)

        ctx.record_begin()
        block()
        cb = ctx.record_end()
        try:
            seen = set()
            for rep in range(4):
                x = synth.activations(tokens, D, salt=40 + rep)
                ctx.upload(X, x)
                block()
                eager = (ctx.download(y, tokens * D * 2, np.uint16), ctx.download(ids, tokens * S * 4, np.uint32))
                ctx.fill(y, 0, tokens * D * 2)
                ctx.fill(ids, 0xFF, tokens * S * 4)
                ctx.submit(cb)
                replay = (ctx.download(y, tokens * D * 2, np.uint16), ctx.download(ids, tokens * S * 4, np.uint32))
                assert np.array_equal(eager[0], replay[0]) and np.array_equal(eager[1], replay[1]), rep
                assert eager[0].any()
                seen.add(eager[1].tobytes())
            assert len(seen) > 1, "different activations route differently"
        finally:
            ctx.cmdbuf_destroy(cb)
