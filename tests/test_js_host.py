"""The JavaScript host layer (N-API addon + index.js): decisions on the CPU, dispatches on the GPU."""
import json
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

from .util import rel_err

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NODE = shutil.which("node")
ADDON = os.path.join(ROOT, "zero-tvm_amd", "js", "ztvm_napi.node")

needs_node = pytest.mark.skipif(NODE is None, reason="no node binary on this machine")


def ensure_addon():
    if not os.path.exists(ADDON):
        sys.path.insert(0, ROOT)
        import importlib
        importlib.import_module("zero-tvm_amd.js.build_addon").build()


@needs_node
def test_js_host_decisions_and_validator():
    ensure_addon()
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "host_cpu.js")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "js host cpu checks ok" in r.stdout, r.stdout + r.stderr


@needs_node
@pytest.mark.gpu
def test_js_dispatch_on_gpu(tmp_path, synth, oracle):
    assert os.path.exists(ADDON), "the N-API addon must be built in-tree before GPU runs"
    K, N = 4096, 1024
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)
    E, slots, tokens, d, ffn = 8, 2, 3, 512, 128
    mw, ms = synth.packed_weights(ffn, d, experts=E), synth.scales(ffn, d, experts=E)
    mb = synth.biases(ffn, d, ms, experts=E)
    ids, mx = synth.topk_ids(tokens, slots, E), synth.activations(tokens, d)
    for name, arr in (("x", x), ("w", w), ("s", s), ("b", b), ("mw", mw), ("ms", ms), ("mb", mb), ("ids", ids), ("mx", mx)):
        arr.tofile(str(tmp_path / (name + ".bin")))
    # the block dispatches: router, silu_mul, combine, gated FFN
    rng = np.random.default_rng(4)
    D, RE, RK, rowsS, F, N2, S, GK, GF = 512, 16, 4, 5, 64, 96, 5, 512, 128
    rx = (rng.random((1, D)) * 2 - 1).astype(np.float16)
    rw = rng.integers(0, 2 ** 32, (RE + 1, D // 4), dtype=np.uint64).astype(np.uint32)
    rs = (rng.random((RE + 1, D // 64)) * 4e-4 + 2e-4).astype(np.float16)
    rb = (-127.5 * rs.astype(np.float32)).astype(np.float16)
    gu = (rng.random((rowsS, 2 * F)) * 6 - 3).astype(np.float16)
    cslots = rng.standard_normal((1, S, N2)).astype(np.float16)
    cscore = rng.random((1, S)).astype(np.float32)
    gx, gw, gs = synth.activations(1, GK, salt=7), synth.packed_weights(2 * GF, GK, salt=7), synth.scales(2 * GF, GK, salt=7)
    gb = synth.biases(2 * GF, GK, gs, salt=7)
    pres = rng.standard_normal(GK).astype(np.float16)
    pdelta = (rng.standard_normal(GK) * 0.3).astype(np.float16)
    pgamma = (1 + 0.1 * rng.standard_normal(GK)).astype(np.float16)
    for name, arr in (("rx", rx), ("rw", rw), ("rs", rs), ("rb", rb), ("gu", gu), ("slots", cslots), ("cscore", cscore),
                      ("gx", gx), ("gw", gw), ("gs", gs), ("gb", gb), ("pres", pres), ("pdelta", pdelta), ("pgamma", pgamma)):
        arr.tofile(str(tmp_path / (name + ".bin")))
    # the fused QKV forms: paged, and scratch rows + int8 quantisation
    QH, QKV, QHD, QK, QPAGE, QPOS = 4, 2, 64, 512, 8, 13
    qrows = (QH + 2 * QKV) * QHD
    qx, qw = synth.activations(1, QK, salt=9), synth.packed_weights(qrows, QK, salt=9)
    qs = synth.scales(qrows, QK, affine=False, lo=0.01, hi=0.06, salt=9)
    for name, arr in (("qx", qx), ("qw", qw), ("qs", qs), ("qpos", np.array([QPOS], np.int32))):
        arr.tofile(str(tmp_path / (name + ".bin")))
    (tmp_path / "meta.json").write_text(json.dumps({"dense": {"K": K, "N": N},
                                                    "qkv": {"heads": QH, "kvHeads": QKV, "headDim": QHD, "d": QK, "pageSize": QPAGE,
                                                            "pages": 2},
                                                    "moe": {"E": E, "slots": slots, "tokens": tokens, "d": d, "ffn": ffn},
                                                    "block": {"D": D, "E": RE, "K": RK, "rowsS": rowsS, "F": F, "N2": N2, "S": S,
                                                              "GK": GK, "GF": GF}}))
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "gemv_gpu.js"), str(tmp_path)], capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0 and "js gpu dispatch ok" in r.stdout, r.stdout + r.stderr
    y = np.fromfile(str(tmp_path / "y_dense.bin"), np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, w, s, b, threads=8)[0]
    assert rel_err(y, ref, 1e-2) < 1e-2
    # the boot-time GEMM probe: the row-group family stops at 16 rows, the others are timed at both sizes; the pick is
    # stored under the device's key and the second resolve replays it without probing again
    tune = json.loads((tmp_path / "tune.json").read_text())
    assert tune["timed"] == ["gemm", "gemv", "skinny"] and sorted(tune["sizes"]) == [64, 256]
    assert tune["first"]["source"] == "probed" and tune["first"]["pick"] in ("gemm", "skinny")
    assert tune["second"] == {"pick": tune["first"]["pick"], "source": "stored"} and tune["probes"] == 1 and tune["adapter"]
    ym = np.fromfile(str(tmp_path / "y_moe.bin"), np.float16).astype(np.float64).reshape(tokens, slots, 2, ffn)
    rm = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d, tokens, slots, (0, 2 * ffn, d, slots * 2 * ffn, slots), ids, mx,
                         mw, ms, mb, ym.size).reshape(tokens, slots, 2, ffn)
    assert rel_err(ym[:, :, 0], rm[:, :, 0], 1e-2) < 1e-2
    assert not ym[:, :, 1].any()  # the up half was not dispatched
    lg = np.fromfile(str(tmp_path / "r_logits.bin"), np.float32).reshape(1, RE + 1)
    ref_lg = oracle.router_logits(8, D, RE + 1, 1, rx.view(np.uint16), rw, rs.view(np.uint16), rb.view(np.uint16))
    assert np.max(np.abs(lg - ref_lg)) < 1e-4
    ri, rsc = oracle.router_topk(lg, 1, RE, RK, True, True)
    assert np.array_equal(np.fromfile(str(tmp_path / "r_idx.bin"), np.uint32).reshape(1, RK + 1), ri)
    assert np.max(np.abs(np.fromfile(str(tmp_path / "r_score.bin"), np.float32).reshape(1, RK + 1) - rsc)) < 2e-6
    h64, _ = oracle.silu_mul(gu.view(np.uint16), rowsS, F)
    assert np.max(np.abs(np.fromfile(str(tmp_path / "h.bin"), np.float16).astype(np.float64).reshape(rowsS, F) - h64)) < 5e-3
    _, c16 = oracle.moe_combine(cslots.view(np.uint16), cscore, 1, N2, S)
    assert np.array_equal(np.fromfile(str(tmp_path / "comb.bin"), np.uint16).reshape(1, N2), c16)
    Wd = oracle.dequant_matrix(4, True, 2 * GF, GK, gw, gs, gb).astype(np.float64)
    xv = gx.view(np.float16).astype(np.float64)[0]
    g, u = Wd[:GF] @ xv, Wd[GF:] @ xv
    assert rel_err(np.fromfile(str(tmp_path / "gated.bin"), np.float16).astype(np.float64), u * g / (1 + np.exp(-g)), 1e-2) < 1e-2
    xn = oracle.add_rmsnorm(pres.view(np.uint16), pdelta.view(np.uint16), pgamma.view(np.uint16), 1e-5).view(np.float16).astype(np.float64)
    gp, upj = Wd[:GF] @ xn, Wd[GF:] @ xn
    refp = upj * gp / (1 + np.exp(-gp))
    gotp = np.fromfile(str(tmp_path / "gated_prologue.bin"), np.float16).astype(np.float64)
    assert np.max(np.abs(gotp - refp) / (np.abs(refp) + 0.05 * np.sqrt(np.mean(refp * refp)))) < 1e-2
    # fused QKV through the JS host: the paged form against the oracle, the scratch rows equal to the paged write,
    # the int8 cache equal to the oracle's quantisation of those rows
    hps, vpo, kps = QPAGE * QHD, QKV * QPAGE * QHD, 2 * QKV * QPAGE * QHD
    want_q, want_p = oracle.qkv_fused(False, QK, QH, QKV, QHD, QPAGE, kps, hps, vpo, 0, 10000.0, QPOS, qx, qw, qs, None,
                                      np.zeros(2 * kps, np.uint16))
    got_q = np.fromfile(str(tmp_path / "q_paged.bin"), np.uint16)
    got_p = np.fromfile(str(tmp_path / "kv_paged.bin"), np.uint16)
    f = lambda a: a.view(np.float16).astype(np.float64)
    assert np.max(np.abs(f(got_q) - f(want_q)) / (np.abs(f(want_q)) + 1e-3)) < 2e-2
    assert np.max(np.abs(f(got_p) - f(want_p)) / (np.abs(f(want_p)) + 1e-3)) < 2e-2
    paged = got_p.reshape(2, 2, QKV, QPAGE, QHD)
    ks, vs = np.fromfile(str(tmp_path / "k_slot.bin"), np.uint16), np.fromfile(str(tmp_path / "v_slot.bin"), np.uint16)
    assert np.array_equal(ks.reshape(QKV, QHD), paged[QPOS // QPAGE, 0, :, QPOS % QPAGE, :])
    assert np.array_equal(vs.reshape(QKV, QHD), paged[QPOS // QPAGE, 1, :, QPOS % QPAGE, :])
    assert np.array_equal(np.fromfile(str(tmp_path / "q_scratch.bin"), np.uint16), got_q)
    rw4 = QHD // 4
    want_pg, want_sc = oracle.kv_quantize_int8(QKV, QHD, QPAGE, [QPOS], 0, 0, ks, vs, np.zeros(2 * QKV * QPAGE * 2 * rw4, np.uint32),
                                               np.zeros(2 * QKV * QPAGE * 2, np.uint16))
    assert np.array_equal(np.fromfile(str(tmp_path / "kv_i8.bin"), np.uint32), want_pg)
    assert np.array_equal(np.fromfile(str(tmp_path / "kv_sc.bin"), np.uint16), want_sc)
