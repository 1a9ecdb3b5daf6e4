"""Policy of the boot-time GEMM choice (zero-tvm_amd/host/gemm_tune.py): the behaviours the reference pins in
tests/unit/gemm-tune.test.ts, re-expressed with hand-derived numbers: deterministic, versioned, ties reproduce the
ladder, stale entries re-tune, and a store or a probe that throws never breaks boot."""
import importlib
import json
import time

import pytest

gt = importlib.import_module("zero-tvm_amd.host.gemm_tune")


def saved(**over):
    d = dict(version=gt.TUNE_VERSION, pick="e5", ms={"e5": 1}, candidates=["e5", "sgmat", "matvec"], at=time.time() * 1000)
    d.update(over)
    return json.dumps(d)


class BadStore:
    def load(self, key):
        raise RuntimeError("x")

    def save(self, key, value):
        raise RuntimeError("x")


def test_median():
    assert gt.median([3, 1, 2]) == 2
    assert gt.median([4, 1, 3, 2]) == 2.5


def test_lowest_geometric_mean_across_sizes_wins():
    # e5 wins small and loses big, sgmat is steady: geomean e5 = 16^(1/3) = 2.52, sgmat = 2
    assert gt.pick_from_timings({"e5": [1, 1, 16], "sgmat": [2, 2, 2]}, ["e5", "sgmat", "matvec"]) == "sgmat"


def test_exact_ties_go_to_the_ladder_order():
    m = {"e5": [2, 2], "sgmat": [2, 2], "matvec": [2, 2]}
    assert gt.pick_from_timings(m, ["e5", "sgmat", "matvec"]) == "e5"
    assert gt.pick_from_timings(m, ["sgmat", "matvec"]) == "sgmat"


def test_candidates_without_timings_are_ignored():
    assert gt.pick_from_timings({"matvec": [5]}, ["e5", "sgmat", "matvec"]) == "matvec"
    assert gt.pick_from_timings({}, ["e5", "sgmat", "matvec"]) == "matvec"


def test_key_names_version_device_and_model():
    assert gt.tune_key("apple/m4", "llama32") == "ztvm.gemmTune.v%d.apple/m4.llama32" % gt.TUNE_VERSION


def test_device_fingerprint():
    assert gt.device_fingerprint({"name": "AMD Instinct MI355X", "compute_units": 256, "hbm_bytes": 309220868096}) == \
        "AMD_Instinct_MI355X/256/309220868096"
    assert gt.device_fingerprint({"name": "gfx950"}) == "gfx950/_/_"
    assert gt.device_fingerprint({}) is None
    assert gt.device_fingerprint(None) is None


def test_stored_pick_is_used_when_fresh_versioned_and_covering():
    key, runnable = "k", ["e5", "sgmat", "matvec"]
    assert gt.load_tuned_pick(gt.MemoryTuneStore({key: saved()}), key, runnable) == "e5"


@pytest.mark.parametrize("over", [dict(version=gt.TUNE_VERSION + 1), dict(at=time.time() * 1000 - gt.TUNE_TTL_MS - 1000),
                                  dict(pick="tiled"), dict(candidates=["matvec"]), dict(at="yesterday"), dict(candidates=None)])
def test_stale_or_foreign_entries_mean_retune(over):
    key, runnable = "k", ["e5", "sgmat", "matvec"]
    assert gt.load_tuned_pick(gt.MemoryTuneStore({key: saved(**over)}), key, runnable) is None


def test_missing_corrupt_and_throwing_stores():
    key, runnable = "k", ["e5", "sgmat", "matvec"]
    assert gt.load_tuned_pick(gt.MemoryTuneStore(), key, runnable) is None
    assert gt.load_tuned_pick(None, key, runnable) is None
    assert gt.load_tuned_pick(gt.MemoryTuneStore({key: "not json"}), key, runnable) is None
    assert gt.load_tuned_pick(gt.MemoryTuneStore({key: "[1, 2]"}), key, runnable) is None
    assert gt.load_tuned_pick(BadStore(), key, runnable) is None
    gt.save_tuned_pick(BadStore(), key, "e5", {}, ["e5"])  # must not raise
    assert gt.load_tuned_pick(gt.MemoryTuneStore({key: saved()}), key, []) is None


def test_explicit_wins_without_store_or_probe():
    probed = []
    r = gt.resolve_tuned_gemm("llama32", ["e5", "sgmat", "matvec"], lambda: probed.append(1) or {}, explicit="matvec",
                              store=gt.MemoryTuneStore(), adapter_id="d")
    assert r == {"pick": "matvec", "source": "explicit"} and not probed


def test_single_candidate_defers_to_the_ladder_without_probing():
    probed = []
    assert gt.resolve_tuned_gemm("llama32", ["matvec"], lambda: probed.append(1) or {}) is None
    assert not probed


def test_probe_then_persist_then_replay():
    store = gt.MemoryTuneStore()
    probe = lambda: {"e5": {64: [1, 1.1], 256: [2, 2.2]}, "sgmat": {64: [3, 3], 256: [4, 4]}}
    first = gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], probe, store=store, adapter_id="d")
    assert first == {"pick": "e5", "source": "probed"}
    entry = json.loads(store.load(gt.tune_key("d", "llama32")))
    assert entry["pick"] == "e5" and entry["candidates"] == ["e5", "sgmat"] and entry["ms"]["e5"] == pytest.approx(1.575)
    # a probe that would now pick otherwise is not consulted: the stored pick replays
    second = gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], lambda: {"sgmat": {64: [0.1]}}, store=store, adapter_id="d")
    assert second == {"pick": "e5", "source": "stored"}
    # without a device identity nothing is stored
    anon = gt.MemoryTuneStore()
    assert gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], probe, store=anon)["source"] == "probed" and not anon.data


def test_throwing_or_empty_probe_means_ladder():
    def boom():
        raise RuntimeError("gpu busy")
    assert gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], boom, store=gt.MemoryTuneStore(), adapter_id="d") is None
    assert gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], lambda: {}, store=gt.MemoryTuneStore(), adapter_id="d") is None
    assert gt.resolve_tuned_gemm("llama32", ["e5", "sgmat"], lambda: {"tiled": {64: [1]}}) is None  # not runnable: ignored


def test_kernel_families_as_candidates_keep_their_ladder_order():
    tie = lambda: {"skinny": {64: [2.0]}, "gemm": {64: [2.0]}}
    assert gt.resolve_tuned_gemm("m", ["skinny", "gemm"], tie)["pick"] == "gemm"
    assert gt.resolve_tuned_gemm("m", ["skinny", "gemm"], lambda: {"skinny": {64: [1.9]}, "gemm": {64: [2.0]}})["pick"] == "skinny"


def test_time_closures_interleaves_and_survives_a_failing_candidate():
    calls, t = [], [0.0]

    def clock():
        return t[0]

    def run(name, cost):
        def f(m):
            calls.append((name, m))
            t[0] += cost * m
        return f
    out = gt.time_closures(lambda: None, {"a": run("a", 0.125), "b": run("b", 0.25)}, [4, 8], warmup=1, rounds=2, clock=clock)
    assert out == {"a": {4: [500.0, 500.0], 8: [1000.0, 1000.0]}, "b": {4: [1000.0, 1000.0], 8: [2000.0, 2000.0]}}
    assert calls[:6] == [("a", 4), ("b", 4), ("a", 4), ("b", 4), ("a", 4), ("b", 4)]  # warm-up round, then A,B per round

    def bad(m):
        raise RuntimeError("no such pipeline")
    assert gt.time_closures(lambda: None, {"a": run("a", 0.125), "bad": bad}, [4], warmup=0, rounds=1, clock=clock) == {"a": {4: [500.0]}}


def test_file_store_round_trip(tmp_path):
    store = gt.FileTuneStore(str(tmp_path / "tune.json"))
    assert store.load("k") is None
    store.save("k", "v")
    store.save("k2", "v2")
    assert gt.FileTuneStore(str(tmp_path / "tune.json")).load("k") == "v"
    (tmp_path / "tune.json").write_text("garbage")
    assert store.load("k") is None
