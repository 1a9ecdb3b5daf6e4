"""Host logic of the MLX checkpoint loader, no GPU: the safetensors header, the per-layer and global plans,
their byte budgets and cache keys. Expectations are written from the reference's layout rules
(src/zero-tvm/mlx-weights.ts:272-472, src/zero-tvm/weight-loader-mlx.ts:93-137) and from the constants its own
test asserts (tests/kernels/mlx-repack.mjs:200-202, :274-280)."""
import importlib
import json
import re
import struct

import pytest

from . import mlx_synth


@pytest.fixture(scope="module")
def mw(pkg):
    return importlib.import_module("zero-tvm_amd.host.mlx_weights")


def qwen36(mw, layers=40):
    return mw.make_spec(id="qwen36-35b-a3b", d=2048, layers=layers, heads=16, ffn=512, qkNorm=True, tiedEmbeddings=False,
                        mlxPrefix="language_model.", fullAttnInterval=4, moe=mw.Moe(experts=256, topK=8))


def dsv2(mw):
    return mw.make_spec(id="deepseek-v2-lite", d=2048, layers=27, heads=16, ffn=1408,
                        mla=mw.Mla(kvLoraRank=512, qkNopeHeadDim=128, qkRopeHeadDim=64, vHeadDim=128),
                        moe=mw.Moe(experts=64, topK=6, normTopkProb=False, sharedExpert=True, routerBits=16,
                                   denseLayers=(0,), denseFfn=10944))


def names(plans):
    return [p.name for p in plans]


def records(plan):
    return [(p.record, p.convert) for p in plan.parts]


def test_safetensors_header_round_trip(mw, tmp_path):
    tensors = {"a.weight": ("U32", (4, 8), b"\x01" * 128), "a.scales": ("BF16", (4, 1), b"\x02" * 8)}
    path = tmp_path / "x.safetensors"
    mlx_synth.write_safetensors(str(path), tensors)
    blob = path.read_bytes()
    n = struct.unpack("<Q", blob[:8])[0]
    h = mw.parse_safetensors_header(blob[:8 + n])
    assert h["dataStart"] == 8 + n and set(h["tensors"]) == {"a.weight", "a.scales"}       # __metadata__ dropped
    t = h["tensors"]["a.scales"]
    assert (t.dtype, t.shape, t.begin, t.end) == ("BF16", (4, 1), 128, 136)
    assert blob[h["dataStart"] + t.begin:h["dataStart"] + t.end] == b"\x02" * 8
    with pytest.raises(ValueError, match="at least 8 bytes"):
        mw.parse_safetensors_header(blob[:4])
    with pytest.raises(ValueError, match="only"):
        mw.parse_safetensors_header(blob[:8 + n - 1])
    with pytest.raises(ValueError, match="4 GB"):
        mw.parse_safetensors_header(struct.pack("<II", 16, 1) + b" " * 16)


def test_layer_kinds(mw):
    s = qwen36(mw)
    assert [i for i, k in enumerate(s.layerKinds) if k == "attn"] == list(range(3, 40, 4))   # 10 of 40
    assert set(s.ffnKinds) == {"moe"}
    d = dsv2(mw)
    assert d.ffnKinds[0] == "dense" and set(d.ffnKinds[1:]) == {"moe"} and set(d.layerKinds) == {"attn"}
    assert (d.mlaQProjRows, d.mlaKvaRows) == (16 * 192, 576)
    with pytest.raises(ValueError, match="denseFfn"):
        mw.make_spec(id="x", layers=2, heads=1, moe=mw.Moe(experts=4, topK=2, denseLayers=(0,)))


def test_plan_layer_qwen36(mw):
    s = qwen36(mw)
    gdn = {p.name: p for p in mw.plan_layer(s, 0)}
    attn = {p.name: p for p in mw.plan_layer(s, 3)}
    p0, p3 = "language_model.model.layers.0", "language_model.model.layers.3"
    assert records(gdn["gdn_proj_w"]) == [(p0 + ".linear_attn.in_proj_%s.weight" % n, "raw") for n in ("qkv", "z", "a", "b")]
    assert records(gdn["gdn_proj_s"]) == [(p0 + ".linear_attn.in_proj_%s.scales" % n, "bf16->f16") for n in ("qkv", "z", "a", "b")]
    assert records(gdn["gdn_a_log"]) == [(p0 + ".linear_attn.A_log", "bf16->f32")]
    assert records(gdn["gdn_dt_bias"]) == [(p0 + ".linear_attn.dt_bias", "bf16->f32")]
    assert records(gdn["gdn_conv"]) == [(p0 + ".linear_attn.conv1d.weight", "bf16->f16")]
    assert "c_attn_w" not in gdn and "gdn_proj_w" not in attn
    assert records(attn["c_attn_b"]) == [(p3 + ".self_attn.%s_proj.biases" % n, "bf16->f16") for n in "qkv"]
    assert records(attn["q_norm"]) == [(p3 + ".self_attn.q_norm.weight", "bf16->f16")]
    # the shared expert is appended to every stack, its gate to the router (8-bit: a full trio)
    assert records(gdn["moe_down_proj_w"]) == [(p0 + ".mlp.switch_mlp.down_proj.weight", "raw"),
                                               (p0 + ".mlp.shared_expert.down_proj.weight", "raw")]
    assert records(gdn["router_s"]) == [(p0 + ".mlp.gate.scales", "bf16->f16"), (p0 + ".mlp.shared_expert_gate.scales", "bf16->f16")]
    assert all(p.op is None for p in gdn.values())
    assert names(mw.plan_layer(s, 0))[:2] == ["norm1", "norm2"]


def test_plan_layer_without_shared_expert_and_dense(mw):
    s = mw.make_spec(id="qwen3-30b-a3b-4bit", layers=2, heads=32, qkNorm=True,
                     moe=mw.Moe(experts=128, topK=8, sharedExpert=False, routerBits=4))
    pl = {p.name: p for p in mw.plan_layer(s, 1)}
    assert records(pl["moe_gate_proj_w"]) == [("model.layers.1.mlp.switch_mlp.gate_proj.weight", "raw")]
    assert records(pl["router_w"]) == [("model.layers.1.mlp.gate.weight", "raw")]
    dense = mw.make_spec(id="llama", layers=1, heads=32, tiedEmbeddings=True)
    pl = {p.name: p for p in mw.plan_layer(dense, 0)}
    assert records(pl["ffn_w"]) == [("model.layers.0.mlp.gate_proj.weight", "raw"), ("model.layers.0.mlp.up_proj.weight", "raw")]
    assert records(pl["ffn_down_s"]) == [("model.layers.0.mlp.down_proj.scales", "bf16->f16")]
    assert "q_norm" not in pl
    assert names(mw.plan_global(dense)) == ["embed_w", "embed_s", "embed_b", "final_norm"]       # tied: no lm_head plans


def test_plan_layer_mla(mw):
    s = dsv2(mw)
    pl = {p.name: p for p in mw.plan_layer(s, 0)}
    assert "c_attn_w" not in pl and "ffn_w" in pl and "router_w" not in pl                 # layer 0 is a dense FFN
    NOPE, R, KVL = 128, 64, 512
    de = lambda j: 2 * j if j < R // 2 else 2 * (j - R // 2) + 1
    q = pl["mla_q_w"].op
    assert q.kind == "permuteRows" and q.rows == 16 * 192 and pl["mla_q_s"].op == q and pl["mla_q_b"].op == q
    for j in range(q.rows):      # the reference test's closed form (tests/kernels/mlx-repack.mjs:206-208)
        i = j % (NOPE + R)
        assert q.src[j] == (j if i < NOPE else j - i + NOPE + de(i - NOPE))
    kva = pl["mla_kva_w"].op
    assert [kva.src[j] for j in range(KVL)] == list(range(KVL))
    assert [kva.src[KVL + j] for j in range(R)] == [KVL + de(j) for j in range(R)]
    assert sorted(kva.src) == list(range(576)), "a permutation"
    kvb = pl["mla_kvb"]
    assert [r for r, _ in records(kvb)] == ["model.layers.0.self_attn.kv_b_proj." + n for n in ("weight", "scales", "biases")]
    assert (kvb.op.kind, kvb.op.k, kvb.op.heads, kvb.op.nope, kvb.op.v) == ("dequantAffineSplit", 512, 16, 128, 128)
    assert records(pl["mla_kva_norm"]) == [("model.layers.0.self_attn.kv_a_layernorm.weight", "bf16->f16")]
    # a MoE layer of the same model: f16 router, one buffer, shared gate appended
    moe = {p.name: p for p in mw.plan_layer(s, 1)}
    assert records(moe["router_w"]) == [("model.layers.1.mlp.gate.weight", "bf16->f16"),
                                        ("model.layers.1.mlp.shared_expert_gate.weight", "bf16->f16")]
    assert "router_s" not in moe


def test_plan_bytes_and_keys(mw):
    s = dsv2(mw)
    pl = {p.name: p for p in mw.plan_layer(s, 0)}
    # 4 MiB per layer against 1.125 MiB of int4 trio: the constant the reference's test asserts
    assert mw.plan_bytes(pl["mla_kvb"], lambda r: 123) == 4194304
    assert re.match(r"^l0\.mla_kvb\.[0-9a-f]{4}$", mw.plan_key(pl["mla_kvb"], 0))
    assert mw.plan_key(pl["norm1"], 0) == "l0.norm1"
    assert mw.plan_key(mw.plan_global(s)[0], None) == "g.embed_w"
    assert mw.plan_key(pl["mla_q_w"], 0) != mw.plan_key(pl["mla_q_s"], 0).replace("_s", "_w"), "the hash covers the parts"
    assert (mw.fnv1a32(""), mw.fnv1a32("a"), mw.fnv1a32("foobar")) == (0x811C9DC5, 0xE40C292C, 0xBF9CF968)   # published FNV-1a vectors
    q = qwen36(mw)
    g = {p.name: p for p in mw.plan_layer(q, 0)}
    size = {"language_model.model.layers.0.linear_attn.A_log": 64}
    assert mw.plan_bytes(g["gdn_a_log"], size.__getitem__) == 128                              # bf16 -> f32 doubles
    assert mw.plan_bytes(g["gdn_a_log"], lambda r: 128, lambda r: "F32") == 128                 # already f32: no doubling
    assert mw.plan_bytes(g["gdn_proj_w"], lambda r: 10) == 40
    keys = [mw.plan_key(p, L) for p, L in mw.plan_model(qwen36(mw, layers=8))]
    assert len(keys) == len(set(keys))
    stage = mw.plan_model(qwen36(mw, layers=8), {"start": 4, "end": 8})
    assert names([p for p, _ in stage])[:4] == ["lm_head_w", "lm_head_s", "lm_head_b", "final_norm"]   # no embedding on the last stage
    assert {L for _, L in stage if L is not None} == {4, 5, 6, 7}
    assert names(mw.plan_global(q))[3:6] == ["lm_head_w", "lm_head_s", "lm_head_b"]
    assert records(mw.plan_global(q)[3]) == [("language_model.lm_head.weight", "raw")]          # one level above model.


def test_slots_cover_every_plan(mw):
    for spec in (qwen36(mw, layers=4), dsv2(mw)):
        for plan, _ in mw.plan_model(spec):
            assert plan.name in mw.SLOTS, plan.name
    assert mw.SLOTS["c_attn_w"] == ("layer", "qkvWeights") and mw.SLOTS["mla_kvb"] == ("mla", "kvbF16")
    assert mw.SLOTS["router_b"] == ("moe", "routerBiases") and mw.SLOTS["gdn_a_log"] == ("gdn", "aLog")


def test_open_checkpoint_locates_by_range(mw, tmp_path):
    spec = mw.make_spec(id="t", layers=1, heads=2, tiedEmbeddings=True)
    recs = [p.record for plan, _ in mw.plan_model(spec) for p in plan.parts]
    dims = {"d": 128, "float": "BF16", "matrices": {"embed_tokens": (32, 128, 4), "down_proj": (128, 256, 4), "_proj": (256, 128, 4)}}
    made = mlx_synth.write_checkpoint(str(tmp_path), recs, dims)
    src = mw.FileSource(str(tmp_path))
    ck = mw.open_mlx_checkpoint(src)
    assert len(ck["shards"]) == 2 and sorted(ck["records"]) == sorted(made)
    for r, (dtype, shape, data) in made.items():
        loc = ck["locate"](r)
        assert (loc.info.dtype, loc.info.shape) == (dtype, shape)
        assert src.range(loc.file, loc.begin, loc.end) == data
    with pytest.raises(KeyError, match="not in checkpoint index"):
        ck["locate"]("model.layers.9.nope")
    total = mw.model_bytes(spec, ck["locate"])
    assert total == sum(len(d) for _, _, d in made.values())            # no f32 targets here: plan bytes == file bytes
    idx = json.load(open(tmp_path / "model.safetensors.index.json"))
    assert set(idx["weight_map"].values()) == set(ck["shards"])


def test_tied_head_must_alias(mw):
    spec = mw.make_spec(id="t", layers=1, heads=1, tiedEmbeddings=True)
    a = object()
    mw.assert_tied_head({"embdWeights": a, "lmHeadWeights": a, "embdScales": a, "lmHeadScales": a, "embdBiases": a,
                         "lmHeadBiases": a}, spec)
    with pytest.raises(ValueError, match="must alias"):
        mw.assert_tied_head({"embdWeights": a, "lmHeadWeights": object()}, spec)
