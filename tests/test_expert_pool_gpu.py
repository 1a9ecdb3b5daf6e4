"""The pooled MoE path on the GPU: a SLOTS-row buffer with ids[] holding slot indices gives the same bytes as
the full expert stack with ids[] holding expert indices, token after token, through evictions — the property
the reference's pool test asserts end to end as "token-identical" (scripts/moe-pool-test.mjs:150-170) — for the
serial path (ids rewritten on the host) and the optimistic path (ids translated on the device through the
resident map, a miss detected afterwards and replayed)."""
import importlib

import numpy as np
import pytest

from .util import Dev, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ep(pkg):
    return importlib.import_module("zero-tvm_amd.host.expert_pool")


@pytest.fixture(scope="module")
def device(pkg, ctx):
    eng = importlib.import_module("zero-tvm_amd.host.engine")
    d = eng.Device.__new__(eng.Device)
    d.ctx, d._recording = ctx, False
    return d


def stacks(synth, E1, d, ffn):
    out = {}
    for proj, N, K, salt in (("gate", ffn, d, 1), ("up", ffn, d, 2), ("down", d, ffn, 3)):
        s = synth.scales(N, K, experts=E1, salt=salt)
        out[proj] = (synth.packed_weights(N, K, experts=E1, salt=salt), s, synth.biases(N, K, s, "B", experts=E1, salt=salt))
    return out


class _B:
    """A bare device address where the host mirror expects a buffer."""

    def __init__(self, addr):
        self.addr = addr


def gate_desc(capi, N, K, S, ids, x, out, w, s, b, experts):
    return capi.MatmulDesc(bits=4, affine=1, M=1, N=N, k_packed=K // 8, scales_per_row=K // 64, slots=S, tokens=1,
                           in_slot_stride=0, in_tok_stride=K, out_slot_stride=N, out_tok_stride=S * N, ids=ids,
                           ids_stride=S, experts=experts, in_=x, out=out, weights=w, scales=s, biases=b)


@pytest.mark.parametrize("optimistic", [False, True])
def test_pooled_equals_full_stack(ctx, capi, synth, oracle, ep, device, optimistic):
    d, ffn, E, K, SLOTS = 256, 128, 24, 4, 8
    E1, S = E + 1, K + 1                       # a shared expert at index E, pinned
    st = stacks(synth, E1, d, ffn)
    source = ep.ArraySlabSource({(0, proj, kind): arr for proj, (w, s, b) in st.items()
                                 for kind, arr in (("w", w), ("s", s), ("b", b))})
    lp = ep.LayerPool(device, 0, d, ffn, E, SLOTS, source, shared_expert_index=E, per_token_slots=S, optimistic=optimistic)
    rng = np.random.default_rng(1)
    replays = 0
    try:
        with Dev(ctx) as dv:
            full = {proj: tuple(dv.put(a) for a in st[proj]) for proj in st}
            ids_e, ids_s = dv.empty(S * 4, fill=0), dv.empty(S * 4, fill=0)
            out_f, out_p = dv.empty(S * ffn * 2, fill=0), dv.empty(S * ffn * 2, fill=0)
            for step in range(40):
                experts = np.r_[rng.choice(E, K, replace=False), E].astype(np.uint32)
                xh = synth.activations(1, d, salt=step)
                x = dv.put(xh)
                ctx.upload(ids_e, experts)
                for proj in ("gate", "up"):
                    w, s, b = full[proj]
                    ctx.matmul(gate_desc(capi, ffn, d, S, ids_e, x, out_f, w, s, b, E1))
                    want = ctx.download(out_f, S * ffn * 2, np.uint16)
                    if step % 8 == 0:
                        # the full-stack result itself against the oracle: "pooled == full" alone would pass a shared error
                        ref = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d, 1, S, (0, ffn, d, S * ffn, S), experts, xh,
                                              *st[proj], S * ffn, threads=4)
                        assert rel_err(want.view(np.float16).astype(np.float64), ref, 1e-2) < 1e-2, (step, proj)
                    bufs = lp.buffers
                    pw, ps, pb = (bufs[proj + "Weights"].addr, bufs[proj + "Scales"].addr, bufs[proj + "Biases"].addr)
                    if optimistic:
                        # one submit: translate on the device, dispatch, then learn whether the map was right
                        lp.translate(_B(ids_s), _B(ids_e), S)
                        ctx.matmul(gate_desc(capi, ffn, d, S, ids_s, x, out_p, pw, ps, pb, SLOTS))
                        if lp.missed(experts):
                            replays += 1
                            lp.resolve(experts)              # uploads the misses, pushes the new map
                            lp.translate(_B(ids_s), _B(ids_e), S)
                            ctx.matmul(gate_desc(capi, ffn, d, S, ids_s, x, out_p, pw, ps, pb, SLOTS))
                        else:
                            lp.resolve(experts)              # pure hits: ages the LRU only
                    else:
                        slots, _ = lp.resolve(experts)
                        ctx.upload(ids_s, slots)
                        ctx.matmul(gate_desc(capi, ffn, d, S, ids_s, x, out_p, pw, ps, pb, SLOTS))
                    got = ctx.download(out_p, S * ffn * 2, np.uint16)
                    assert np.array_equal(got, want), (step, proj)
        assert lp.pool.slot_for(E) == 0, "the shared expert keeps its slot"
        assert 0.0 < lp.pool.hit_rate < 1.0
        assert source.reads % 9 == 0 and source.reads >= 9 * SLOTS   # whole experts only: nine slabs per miss
        if optimistic:
            assert replays > 0
    finally:
        lp.destroy()


def test_pool_below_floor_refuses(ep, device):
    src = ep.ArraySlabSource({(0, p, k): np.zeros((4, n), np.uint8) for (_, p, k, n) in ep.slab_tensors(128, 64)})
    with pytest.raises(ValueError, match="below the pool's minimum 10"):
        ep.LayerPool(device, 0, 128, 64, 3, 9, src, shared_expert_index=3, per_token_slots=9)
    bad = ep.ArraySlabSource({(0, p, k): np.zeros((4, n + 4), np.uint8) for (_, p, k, n) in ep.slab_tensors(128, 64)})
    with pytest.raises(ValueError, match="per expert by the spec"):
        ep.LayerPool(device, 0, 128, 64, 3, 4, bad)
