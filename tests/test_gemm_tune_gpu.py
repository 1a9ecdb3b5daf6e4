"""The boot-time GEMM probe on the device: the kernel families are timed through the C ABI with the family forced,
the pick is one of the runnable ones, it is persisted under the device's key and replayed without probing."""
import importlib
import json

import numpy as np
import pytest

from .util import Dev

pytestmark = pytest.mark.gpu
gt = importlib.import_module("zero-tvm_amd.host.gemm_tune")


def test_probe_picks_persists_and_replays(ctx, capi, synth, tmp_path):
    N, K, CAP = 1024, 512, 256
    with Dev(ctx) as d:
        w, s = synth.packed_weights(N, K), synth.scales(N, K)
        b = synth.biases(N, K, s, "A")
        desc = capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_AUTO, M=CAP, N=N, k_packed=K // 8, scales_per_row=K // 64,
                               out=d.empty(CAP * N * 2), in_=d.put(np.zeros((CAP, K), np.float16)), scales=d.put(s),
                               weights=d.put(w), biases=d.put(b))
        timings = gt.probe_families(ctx, capi, desc, ["gemm", "skinny", "rows", "gemv"], Ms=(64, 256), warmup=1, rounds=3)
        assert set(timings) == {"gemm", "skinny", "gemv"}  # the row-group family stops at 16 rows: not a candidate
        for name, per_size in timings.items():
            assert set(per_size) == {64, 256} and all(len(v) == 3 and min(v) > 0 for v in per_size.values()), name

        store = gt.FileTuneStore(str(tmp_path / "tune.json"))
        adapter = gt.device_fingerprint(ctx.device_info())
        assert adapter
        probes = []

        def run_probe():
            probes.append(1)
            return gt.probe_families(ctx, capi, desc, ["gemm", "skinny", "gemv"], Ms=(64, 256), warmup=1, rounds=3)
        first = gt.resolve_tuned_gemm("synthetic-1024x512", ["gemm", "skinny", "gemv"], run_probe, store=store, adapter_id=adapter)
        assert first["source"] == "probed" and first["pick"] in ("gemm", "skinny", "gemv") and probes == [1]
        entry = json.loads(store.load(gt.tune_key(adapter, "synthetic-1024x512")))
        assert entry["pick"] == first["pick"] and set(entry["ms"]) == {"gemm", "skinny", "gemv"}
        second = gt.resolve_tuned_gemm("synthetic-1024x512", ["gemm", "skinny", "gemv"], run_probe, store=store, adapter_id=adapter)
        assert second == {"pick": first["pick"], "source": "stored"} and probes == [1]
        # one row per launch loses to both matrix-core families at these sizes on any MI355X
        assert first["pick"] != "gemv"
