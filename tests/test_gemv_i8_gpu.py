"""GPU parity of the int8 matrix-core GEMV (opt-in path `gemv.path=2`): the same bars as the default
GEMV on dense 4-bit affine shapes with up to four activation rows, and on the MoE block."""
import numpy as np
import pytest

from .test_gemv_gpu import check, run_dense
from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture()
def i8(ctx):
    ctx.set_option("gemv.path", 2)
    yield ctx
    ctx.set_option("gemv.path", 0)
    ctx.set_option("i8.ksplit", 0)


@pytest.mark.parametrize("K,N", [(2048, 8192), (4096, 14336), (14336, 4096), (4096, 6144), (256, 8), (512, 2048), (768, 100)])
@pytest.mark.parametrize("regime", ["A", "B"])
def test_dense_shapes(i8, capi, synth, oracle, K, N, regime):
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s, regime)
    y = run_dense(i8, capi, 4, True, 1, N, K, x, w, s, b, kernel=capi.KERNEL_GEMV)
    check(y, oracle, 4, True, 1, N, K, x, w, s, b)


@pytest.mark.parametrize("ksplit", [1, 2, 4])
@pytest.mark.parametrize("N", [1, 7, 9, 250])
def test_ragged_rows_and_k_splits(i8, capi, synth, oracle, ksplit, N):
    K = 4096
    i8.set_option("i8.ksplit", ksplit)
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    y = run_dense(i8, capi, 4, True, 1, N, K, x, w, s, b, kernel=capi.KERNEL_GEMV)
    check(y, oracle, 4, True, 1, N, K, x, w, s, b)


@pytest.mark.parametrize("M", [2, 3, 4, 7])
def test_several_rows_and_f32_out(i8, capi, synth, oracle, M):
    K, N = 2048, 520
    x, w, s = synth.activations(M, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    for out_f32 in (False, True):
        y = run_dense(i8, capi, 4, True, M, N, K, x, w, s, b, out_f32=out_f32, kernel=capi.KERNEL_GEMV)
        check(y, oracle, 4, True, M, N, K, x, w, s, b, out_f32)


def test_one_hot_and_wide_dynamic_range(i8, capi, synth, oracle):
    K, N = 4096, 64
    w, s = synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    w16 = oracle.dequant_matrix(4, True, N, K, w, s, b, want="f16")
    for k in (0, 7, 31, 64, 2047, 4095):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1.0
        y = run_dense(i8, capi, 4, True, 1, N, K, x.view(np.uint16), w, s, b, kernel=capi.KERNEL_GEMV)
        assert np.array_equal(y[0].astype(np.float16).view(np.uint16), w16[:, k]), k
    # one large value per group next to tiny ones: the block fixed point must not lose the tiny ones' sum
    x = (synth.activations(1, K).view(np.float16).astype(np.float32) * 1e-3)
    x[0, ::64] = 300.0
    xb = x.astype(np.float16).view(np.uint16)
    y = run_dense(i8, capi, 4, True, 1, N, K, xb, w, s, b, kernel=capi.KERNEL_GEMV)
    check(y, oracle, 4, True, 1, N, K, xb, w, s, b)
    # non-finite activations poison the output instead of producing a finite wrong number
    x[0, 5] = np.inf
    y = run_dense_raw(i8, capi, N, K, x.astype(np.float16).view(np.uint16), w, s, b)
    assert not np.isfinite(y).any()


def run_dense_raw(ctx, capi, N, K, x, w, s, b):
    with Dev(ctx) as d:
        out = d.empty(N * 2)
        desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_GEMV, M=1, N=N, k_packed=K // 8, scales_per_row=K // 64,
                               out=out, in_=d.put(x), scales=d.put(s), weights=d.put(w), biases=d.put(b))
        ctx.matmul(desc)
        return ctx.download(out, N * 2, np.float16).astype(np.float64)


@pytest.mark.parametrize("tokens", [1, 16])
def test_moe_block(i8, capi, synth, oracle, tokens):
    E, slots, d_model, ffn = 256, 8, 2048, 512
    w = synth.packed_weights(ffn, d_model, experts=E)
    s = synth.scales(ffn, d_model, experts=E)
    b = synth.biases(ffn, d_model, s, experts=E)
    ids = synth.topk_ids(tokens, slots, E)
    x = synth.activations(tokens, d_model)
    with Dev(i8) as d:
        gu = d.empty(tokens * slots * 2 * ffn * 2, fill=0)
        desc = capi.MatmulDesc(bits=4, affine=1, M=1, N=ffn, k_packed=d_model // 8, scales_per_row=d_model // 64, slots=slots,
                               tokens=tokens, in_slot_stride=0, out_slot_stride=2 * ffn, in_tok_stride=d_model,
                               out_tok_stride=slots * 2 * ffn, ids_stride=slots, experts=E, out=gu, in_=d.put(x),
                               scales=d.put(s), weights=d.put(w), biases=d.put(b), ids=d.put(ids))
        i8.matmul(desc)
        got = i8.download(gu, tokens * slots * 2 * ffn * 2, np.float16).astype(np.float64).reshape(tokens, slots, 2, ffn)
    ref = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d_model, tokens, slots, (0, 2 * ffn, d_model, slots * 2 * ffn, slots),
                          ids, x, w, s, b, got.size, threads=8).reshape(tokens, slots, 2, ffn)
    assert rel_err(got[:, :, 0], ref[:, :, 0], 1e-2) < 1e-2
    assert not got[:, :, 1].any()
    # down projection: K = 512 (two units), per-slot inputs
    wd = synth.packed_weights(d_model, ffn, experts=E)
    sd = synth.scales(d_model, ffn, experts=E)
    bd = synth.biases(d_model, ffn, sd, experts=E)
    xd = synth.activations(tokens * slots, ffn)
    with Dev(i8) as d:
        out = d.empty(tokens * slots * d_model * 2, fill=0)
        desc = capi.MatmulDesc(bits=4, affine=1, M=1, N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, slots=slots,
                               tokens=tokens, in_slot_stride=ffn, out_slot_stride=d_model, in_tok_stride=slots * ffn,
                               out_tok_stride=slots * d_model, ids_stride=slots, experts=E, out=out, in_=d.put(xd),
                               scales=d.put(sd), weights=d.put(wd), biases=d.put(bd), ids=d.put(ids))
        i8.matmul(desc)
        gotd = i8.download(out, tokens * slots * d_model * 2, np.float16).astype(np.float64)
    refd = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, d_model, ffn, tokens, slots,
                           (ffn, d_model, slots * ffn, slots * d_model, slots), ids, xd, wd, sd, bd, gotd.size, threads=8)
    assert rel_err(gotd, refd, 1e-2) < 1e-2
