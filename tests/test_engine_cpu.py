"""Host-layer decisions, restated from the reference's own unit tests (no GPU):
tests/unit/resolve-matmul-affine.test.ts:76-148, tests/unit/chunk-gemm-pick.test.ts:27-120,
tests/unit/chunk-grid-limits.test.ts:37-54, and the generator's naming / legality rules
(src/compiler/shaders/int4_matmul.gen.ts:137-152, :172-197, :701-766)."""
import importlib

import pytest


@pytest.fixture(scope="module")
def eng(pkg):
    return importlib.import_module("zero-tvm_amd.host.engine")


def test_entry_names_of_the_shipped_variants(eng):
    names = [eng.int4_matmul_entry(o) for o in eng.INT4_MATMUL_VARIANTS]
    assert len(names) == 34 and len(set(names)) == 34
    for must in ("int4_matmul", "int4_matmul_sg", "int4_matmul_tiled", "int4_matmul_tiled8", "int4_matmul_f32_tiled",
                 "int4_matmul_batched_m4", "int4_matmul_batched_dyn", "int4_matmul_batched_dyn_affine",
                 "int4_matmul_tiled_vec4", "int4_matmul_f32_sg_vec4h", "int4_matmul_tiled_vec4h_affine",
                 "int4_matmul_f32_tiled_vec4h_affine", "int4_matmul_tiled_affine_moe",
                 "int4_matmul_tiled_vec4h_affine_moe", "int4_matmul_affine_q3", "int4_matmul_tiled_affine_q3",
                 "int4_matmul_tiled_affine_q3_moe"):
        assert must in names, must
    for o in eng.INT4_MATMUL_VARIANTS:
        eng.check_opts(o)  # every shipped variant is legal


@pytest.mark.parametrize("kw,needle", [
    (dict(moe=True), "moe requires affine"),
    (dict(q3=True), "q3 requires affine"),
    (dict(affine=True, m=4, subgroups=True, rowsPerWG=4), "affine is implemented at m=1"),
    (dict(affine=True, q3=True, subgroups=True, vec4Half=True), "no wide-load path"),
    (dict(affine=True, moe=True, subgroups=True, vec4=True), "no full-vec4 path"),
    (dict(rowsPerWG=4), "requires subgroups"),
    (dict(m=4, subgroups=True), "m=4 requires"),
    (dict(vec4=True), "vec4 requires subgroups"),
    (dict(vec4=True, vec4Half=True, subgroups=True), "mutually exclusive"),
    (dict(mDyn=True, subgroups=True), "mDyn requires"),
])
def test_generator_legality_rules(eng, kw, needle):
    with pytest.raises(ValueError, match=needle):
        eng.check_opts(eng.Int4MatmulOpts(**kw))


def test_pipeline_semantics(eng, capi):
    p = eng.create_pipeline("int4_matmul_f32_tiled_vec4h_affine")
    assert p.affine and p.out_f32 and p.bits == 4 and not p.moe and p.kernel == capi.KERNEL_GEMV
    p = eng.create_pipeline("int4_matmul_tiled_affine_q3_moe")
    assert p.affine and p.bits == 3 and p.moe
    assert eng.create_pipeline("int4_matmul_batched_dyn_affine").runtime_m
    assert eng.create_pipeline("int4_matmul_batched_m4").fixed_m == 4
    assert eng.create_pipeline("int4_matmul_sg_e5_affine").kernel == capi.KERNEL_GEMM
    with pytest.raises(ValueError):
        eng.create_pipeline("int4_matmul_nonsense")


ALL = None


def everything(eng):
    return set(eng.ALL_ENTRIES)


def test_affine_resolves_first_and_takes_the_wide_rung(eng):
    # Qwen3.6: d=2048 and qDim=4096 are both %512 -> the vec4h affine rung, f16 and f32 siblings
    for k in (2048, 4096, 512):
        r = eng.resolve_matmul("tiled", everything(eng), vec4=True, k=k, affine=True, vec4_affine=True)
        assert r["pipeline"] == "int4_matmul_tiled_vec4h_affine"
        assert r["pipelineF32"] == "int4_matmul_f32_tiled_vec4h_affine" and r["rowsPerWG"] == 4
    # ?vec4=0 falls back to the narrow affine rung
    r = eng.resolve_matmul("tiled", everything(eng), vec4=False, k=2048, affine=True, vec4_affine=False)
    assert r["pipeline"] == "int4_matmul_tiled_affine" and "affine" in r["label"]
    # K=768 (qwen30b down) misses the %512 gate
    assert eng.resolve_matmul("tiled", everything(eng), True, 768, None, True, True)["label"] == "tiled_affine"


def test_scalar_lever_reaches_scalar_on_affine_and_symmetric(eng):
    r = eng.resolve_matmul("scalar", everything(eng), vec4=True, k=2048, affine=True, vec4_affine=True)
    assert r["label"] == "scalar_affine" and r["pipeline"] == "int4_matmul_affine"
    assert r["pipelineF32"] == "int4_matmul_f32_affine"
    assert eng.resolve_matmul("scalar", everything(eng), vec4=True, k=3072)["label"] == "scalar"


def test_symmetric_ladder(eng):
    A = everything(eng)
    assert eng.resolve_matmul("tiled", A, vec4=True, k=2560)["pipeline"] == "int4_matmul_tiled_vec4h"  # %1024 fails, %512 passes
    assert eng.resolve_matmul("tiled", A, vec4=True, k=4096)["pipeline"] == "int4_matmul_tiled_vec4"
    assert eng.resolve_matmul("tiled", A, vec4=True, k=9216)["pipeline"] == "int4_matmul_tiled_vec4"
    assert eng.resolve_matmul("sg", A, vec4=True, k=2560)["label"] == "sg_vec4h"
    assert eng.resolve_matmul("tiled8", A, vec4=True, k=4096)["rowsPerWG"] == 8
    assert eng.resolve_matmul("tiled", A, vec4=False, k=4096)["label"] == "tiled"
    # subgroups feature off: only the scalar pipelines were compiled
    scalar_only = {"int4_matmul", "int4_matmul_f32", "int4_matmul_affine", "int4_matmul_f32_affine"}
    assert eng.resolve_matmul("tiled", scalar_only, vec4=True, k=4096)["label"] == "scalar"
    assert eng.resolve_matmul("tiled", scalar_only, True, 4096, None, True, True)["label"] == "scalar_affine"
    # a tiled pipeline resolves only when BOTH the f16 and the f32 sibling exist
    no_f32 = A - {"int4_matmul_f32_tiled_affine", "int4_matmul_f32_tiled_vec4h_affine"}
    assert eng.resolve_matmul("tiled", no_f32, True, 2048, None, True, True)["label"] == "sg_vec4h_affine"


FULL = dict(chunk_tiled=False, dims_ok=True, cap_tiles64=True, e5_ready=True, sgmat_ready=True, cap=1024)


def test_pick_chunk_gemm_automatic(eng):
    pick = lambda **kw: eng.pick_chunk_gemm(**{**FULL, **kw})
    assert pick()["used"] == "e5"
    assert pick(e5_ready=False)["used"] == "sgmat"
    assert pick(cap_tiles64=False, cap=96)["used"] == "sgmat"
    p = pick(e5_ready=False, sgmat_ready=False)
    assert p["used"] == "matvec" and p["rejected"] is None
    p = pick(dims_ok=False)
    assert p["used"] == "matvec" and p["rejected"] is None
    assert pick(e5_ready=False, sgmat_ready=False, chunk_tiled=True)["used"] == "tiled"
    assert pick(chunk_tiled=True)["used"] == "e5"


def test_pick_chunk_gemm_explicit(eng):
    pick = lambda **kw: eng.pick_chunk_gemm(**{**FULL, **kw})
    for want in ("e5", "sgmat", "tiled", "matvec"):
        p = pick(want=want)
        assert p["used"] == want and p["rejected"] is None
    p = pick(want="e5", cap_tiles64=False, cap=96)
    assert p["used"] == "sgmat" and "asked for 'e5', can only run 'sgmat'" in p["rejected"]
    assert "cap must be %64 (got 96)" in p["rejected"]
    p = pick(want="e5", e5_ready=False, sgmat_ready=False)
    assert p["used"] == "matvec" and "chromium-experimental-subgroup-matrix" in p["rejected"]
    p = pick(want="sgmat", e5_ready=False, sgmat_ready=False)
    assert p["used"] == "matvec" and "asked for 'sgmat'" in p["rejected"]
    for want in ("e5", "sgmat", "tiled"):
        p = pick(want=want, dims_ok=False)
        assert p["used"] == "matvec" and "dims do not tile" in p["rejected"]
    p = eng.pick_chunk_gemm(want="matvec", chunk_tiled=False, dims_ok=False, cap_tiles64=False, e5_ready=False,
                            sgmat_ready=False, cap=96)
    assert p["used"] == "matvec" and p["rejected"] is None
    p = pick(want="matvec", chunk_tiled=True)
    assert p["used"] == "tiled" and "asked for 'matvec', can only run 'tiled'" in p["rejected"]
    assert "that pipeline was not built" in p["rejected"]


def test_fold_grid_x_and_chunk_cap(eng):
    assert eng.fold_grid_x(68) == {"x": 68, "z": 1}
    assert eng.fold_grid_x(16384) == {"x": 16384, "z": 1}
    assert eng.fold_grid_x(69632) == {"x": 16384, "z": 5}
    for total in (65535, 65536, 69632, 1000000):
        f = eng.fold_grid_x(total)
        assert f["x"] <= 16384 and f["x"] * f["z"] >= total and (f["z"] - 1) * f["x"] < total
    assert eng.resolve_chunk_cap(None, None, True) == 1024
    assert eng.resolve_chunk_cap(None, None, False) == 64
    assert eng.resolve_chunk_cap(None, 256, True) == 256
    assert eng.resolve_chunk_cap(96, 256, True) == 96


def test_pod_builders_match_the_engine(eng):
    gate, down = eng.moe_pods(2048, 512, 8)
    assert gate == [256, 32, 512, 0, 1024, 2048, 8 * 1024, 8]
    assert down == [64, 8, 2048, 512, 2048, 8 * 512, 8 * 2048, 8]
    g3, d3 = eng.moe_pods(2048, 512, 8, bits=3)
    assert g3[0] == 192 and d3[0] == 48
    assert eng.dense_pod(4096, 14336) == [512, 64, 14336]
    assert eng.dense_pod(4096, 14336, affine=False, M=31) == [512, 128, 14336, 31]


def test_moe_descriptor_arms_the_expert_guard(eng, capi):
    """The engine-built MoE descriptor carries the stack height taken from the bound sizes (what WebGPU's
    bounds-checked storage access gave the reference), and bound stacks that disagree are refused."""
    E, d_model, ffn, slots = 6, 256, 128, 3
    gate, _ = eng.moe_pods(d_model, ffn, slots)

    class FakeBuf:
        def __init__(self, size):
            self.addr, self.size = 0x10000, size

    dev = eng.Device.__new__(eng.Device)
    pipe = eng.create_pipeline("int4_matmul_tiled_affine_moe")
    per_w, per_s = ffn * (d_model // 8) * 4, ffn * (d_model // 64) * 2
    bufs = [FakeBuf(slots * 2 * ffn * 2), FakeBuf(d_model * 2), FakeBuf(E * per_s), FakeBuf(E * per_w), dev.uniform_buf(gate),
            FakeBuf(E * per_s), FakeBuf(slots * 4)]
    desc = dev.descriptor(dev.bg(pipe, bufs), ffn // 4, 1, slots)
    assert desc.experts == E and desc.slots == slots and desc.tokens == 1
    assert capi.validate(desc)[0] == 0
    bufs[5] = FakeBuf((E - 2) * per_s)             # a bias stack two experts short: the guard takes the smallest
    assert dev.descriptor(dev.bg(pipe, bufs), ffn // 4, 1, slots).experts == E - 2
    bufs[3] = FakeBuf(per_w - 4)                   # not even one whole expert bound
    with pytest.raises(ValueError, match="no whole expert"):
        dev.descriptor(dev.bg(pipe, bufs), ffn // 4, 1, slots)
