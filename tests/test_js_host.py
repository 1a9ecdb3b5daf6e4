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
    (tmp_path / "meta.json").write_text(json.dumps({"dense": {"K": K, "N": N},
                                                    "moe": {"E": E, "slots": slots, "tokens": tokens, "d": d, "ffn": ffn}}))
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "gemv_gpu.js"), str(tmp_path)], capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0 and "js gpu dispatch ok" in r.stdout, r.stdout + r.stderr
    y = np.fromfile(str(tmp_path / "y_dense.bin"), np.float16).astype(np.float64)
    ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, w, s, b, threads=8)[0]
    assert rel_err(y, ref, 1e-2) < 1e-2
    ym = np.fromfile(str(tmp_path / "y_moe.bin"), np.float16).astype(np.float64).reshape(tokens, slots, 2, ffn)
    rm = oracle.moe_gemv(oracle.MODE_FORMULA_F32, 4, ffn, d, tokens, slots, (0, 2 * ffn, d, slots * 2 * ffn, slots), ids, mx,
                         mw, ms, mb, ym.size).reshape(tokens, slots, 2, ffn)
    assert rel_err(ym[:, :, 0], rm[:, :, 0], 1e-2) < 1e-2
    assert not ym[:, :, 1].any()  # the up half was not dispatched
