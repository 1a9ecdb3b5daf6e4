"""The dispatch surface end to end on the GPU: uniformBuf / bg / dispatch with the reference's
entry-point names, binding order and MoE grid meaning (y = tokens, z = slots)."""
import importlib

import numpy as np
import pytest

from .util import rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng(pkg):
    return importlib.import_module("zero-tvm_amd.host.engine")


@pytest.fixture(scope="module")
def dev(eng):
    d = eng.Device(0)
    yield d
    d.close()


def put(dev, arr, label=""):
    b = dev.create_buffer(arr.nbytes, label)
    dev.write_buffer(b, 0, arr)
    return b


def test_dense_decode_dispatch_and_errors(dev, eng, synth, oracle):
    K, N = 2048, 512
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    out = dev.create_buffer(N * 2)
    pipe = dev.create_pipeline("int4_matmul_tiled_vec4h_affine")
    pod = dev.uniform_buf(eng.dense_pod(K, N))
    bufs = [out, put(dev, x), put(dev, s), put(dev, w), pod, put(dev, b)]
    with pytest.raises(ValueError, match="no bias buffer at binding 5"):
        dev.bg(pipe, bufs[:5])
    with pytest.raises(ValueError, match="null buffer at binding 3"):
        dev.bg(pipe, bufs[:3] + [None] + bufs[4:])
    group = dev.bg(pipe, bufs)
    dev.dispatch(pipe, group, N // 4)  # the WGSL grid is accepted and ignored
    y = dev.read_buffer(out, np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, w, s, b)[0]
    assert rel_err(y, ref, 1e-2) < 1e-2
    other = dev.create_pipeline("int4_matmul_affine")
    with pytest.raises(ValueError, match="bind group was built for"):
        dev.dispatch(other, group, N)


def test_runtime_m_uniform_update_and_recorded_replay(dev, eng, synth, oracle):
    """Chunked prefill writes M_ROWS at byte 12 of the uniform before each chunk
    (src/zero-tvm/engine-core.ts:4251-4254)."""
    K, N, CAP = 1024, 192, 64
    A, w, s = synth.activations(CAP, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    out = dev.create_buffer(CAP * N * 2)
    pod = dev.uniform_buf(eng.dense_pod(K, N, M=0))
    for entry in ("int4_matmul_batched_dyn_affine", "int4_matmul_sg_e5_affine"):
        pipe = dev.create_pipeline(entry)
        group = dev.bg(pipe, [out, put(dev, A), put(dev, s), put(dev, w), pod, put(dev, b)])
        for M in (0, 5, 47):
            dev.ctx.fill(out.addr, 0, CAP * N * 2)
            pod.write_u32(12, M)
            dev.dispatch(pipe, group, (N + 31) // 32, (M + 63) // 64)
            got = dev.read_buffer(out, np.float16).astype(np.float64).reshape(CAP, N)
            assert not got[M:].any()
            if M:
                ref = oracle.gemm(oracle.MODE_FORMULA_F64, 4, True, M, N, K, A, w, s, b, threads=8)
                assert rel_err(got[:M], ref, 1e-2) < 1e-2
    # one encoder, several dispatches, one submit
    dev.begin_encoder()
    dev.dispatch(pipe, group, 6, 1)
    cb = dev.finish_encoder()
    dev.ctx.fill(out.addr, 0, CAP * N * 2)
    dev.submit(cb)
    again = dev.read_buffer(out, np.float16).astype(np.float64).reshape(CAP, N)
    assert np.array_equal(again, got)


def test_moe_block_through_the_dispatch_surface(dev, eng, synth, oracle):
    """recordMoeExperts (src/zero-tvm/engine-core.ts:2342-2349): gate and up bind one [slot][2*ffn]
    buffer, up at byte offset ffn*2; grid (ffn/4, tokens, slots)."""
    E, slots, d_model, ffn, tokens = 16, 4, 512, 256, 3
    wg = synth.packed_weights(ffn, d_model, experts=E)
    wu = synth.packed_weights(ffn, d_model, experts=E, salt=3)
    s = synth.scales(ffn, d_model, experts=E)
    b = synth.biases(ffn, d_model, s, experts=E)
    ids = synth.topk_ids(tokens, slots, E)
    x = synth.activations(tokens, d_model)
    gate_pod, _ = eng.moe_pods(d_model, ffn, slots)
    pipe = dev.create_pipeline("int4_matmul_tiled_vec4h_affine_moe")
    gu = dev.create_buffer(tokens * slots * 2 * ffn * 2)
    dev.ctx.fill(gu.addr, 0, gu.size)
    common = [put(dev, x), put(dev, s)]
    pod, bb, bi = dev.uniform_buf(gate_pod), put(dev, b), put(dev, ids)
    g_gate = dev.bg(pipe, [gu] + common + [put(dev, wg), pod, bb, bi])
    up_region = eng.Region(gu, ffn * 2, gu.size - ffn * 2)
    assert up_region.offset % 256 == 0
    g_up = dev.bg(pipe, [up_region] + common + [put(dev, wu), pod, bb, bi])
    dev.dispatch(pipe, g_gate, ffn // 4, tokens, slots)
    dev.dispatch(pipe, g_up, ffn // 4, tokens, slots)
    got = dev.read_buffer(gu, np.float16).astype(np.float64).reshape(tokens, slots, 2, ffn)
    st = tuple(gate_pod[3:8])
    rg = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d_model, tokens, slots, st, ids, x, wg, s, b, got.size)
    ru = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d_model, tokens, slots, st, ids, x, wu, s, b, got.size)
    assert rel_err(got[:, :, 0], rg.reshape(tokens, slots, 2, ffn)[:, :, 0], 1e-2) < 1e-2
    assert rel_err(got[:, :, 1], ru.reshape(tokens, slots, 2, ffn)[:, :, 0], 1e-2) < 1e-2
    with pytest.raises(ValueError, match="256-byte aligned"):
        dev.bg(pipe, [eng.Region(gu, 64, 128)] + common + [put(dev, wu), pod, bb, bi])
