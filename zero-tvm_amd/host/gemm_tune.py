"""Boot-time choice of the prefill ("chunk") GEMM by measurement, remembered per device and model.

Mirrors the policy of the reference's src/zero-tvm/gemm-tune.ts (tuneKey :52-54, deviceFingerprint :61-78,
median :81-85, pickFromTimings :90-105, loadTunedPick :110-129, saveTunedPick :131-145, timeClosures
:162-189, resolveTunedGemm :208-233; wired at engine-core.ts:3875-3938): time every runnable candidate on
the real gate/up weights at a ragged, a middle and a full chunk size, interleaved so that clock drift
cancels, take the median per size and the geometric mean across sizes, lowest wins, exact ties go to the
static ladder order; an explicit request bypasses all of it; anything that goes wrong means "let the
ladder decide" (None), never an error at boot.

Candidates are plain names. The reference's are its WGSL pipelines ('e5', 'sgmat', 'tiled', 'matvec');
this library's are its kernel families ('gemm', 'skinny', 'rows', 'gemv' = ZTVM_KERNEL_*), and
`probe_families` times those through `ztvm_matmul` with the family forced. Without a stored or probed
pick `ztvm_matmul` routes by its built-in row thresholds.
"""
import json
import math
import os
import time

TUNE_VERSION = 1                       # bump when a GEMM kernel changes shape or speed: stored picks go stale
TUNE_TTL_MS = 30 * 24 * 3600 * 1000    # drivers move performance too: re-tune monthly
TUNE_MS = (64, 256, 1024)              # probe sizes (chunk rows): ragged head, middle, full cap
TUNE_WARMUP = 2
TUNE_ROUNDS = 4
REFERENCE_LADDER = ("e5", "sgmat", "tiled", "matvec")
FAMILY_LADDER = ("gemm", "skinny", "rows", "gemv")


def tune_key(adapter_id, spec_id):
    return "ztvm.gemmTune.v%d.%s.%s" % (TUNE_VERSION, adapter_id, spec_id)


def device_fingerprint(info):
    """Identity of the device for the key, from `Context.info()`-like data: name / compute units / memory.
    None when nothing identifies it (the caller then tunes without persisting)."""
    try:
        if not info:
            return None
        name = info.get("name") or info.get("arch")
        if name:
            parts = [str(name), str(info.get("compute_units", "?")), str(info.get("hbm_bytes", "?"))]
            return "".join(c if (c.isalnum() or c in "._/-") else "_" for c in "/".join(parts))
    except Exception:  # a fingerprint must never break boot
        pass
    return None


def median(xs):
    s = sorted(xs)
    m = len(s) >> 1
    return s[m] if len(s) % 2 else (s[m - 1] + s[m]) / 2


def pick_from_timings(medians, ladder):
    """Lowest geometric mean (across sizes) of the per-size medians; strictly-less keeps the earlier ladder
    entry on exact ties; candidates without timings are ignored; nothing timed -> the ladder's last entry."""
    best, best_score = ladder[-1], math.inf
    for name in ladder:
        ms = medians.get(name)
        if not ms:
            continue
        geo = math.exp(sum(math.log(max(m, 1e-9)) for m in ms) / len(ms))
        if geo < best_score:
            best_score, best = geo, name
    return best


def _now_ms():
    return time.time() * 1000.0


def load_tuned_pick(store, key, runnable, now=None):
    """A stored pick counts only if it is current-version, fresh, still runnable, and was measured against a
    candidate set that covers today's runnable ones. Anything else (also corrupt data, a throwing store)
    means re-tune: None."""
    if store is None or not runnable:
        return None
    try:
        raw = store.load(key)
    except Exception:
        return None
    if not raw:
        return None
    try:
        saved = json.loads(raw)
    except Exception:
        return None
    if not isinstance(saved, dict) or saved.get("version") != TUNE_VERSION:
        return None
    at = saved.get("at")
    now = _now_ms() if now is None else now
    if not isinstance(at, (int, float)) or isinstance(at, bool) or now - at > TUNE_TTL_MS:
        return None
    if saved.get("pick") not in runnable:
        return None
    cands = saved.get("candidates")
    if not isinstance(cands, list) or not all(c in cands for c in runnable):
        return None
    return saved["pick"]


def save_tuned_pick(store, key, pick, ms, candidates):
    if store is None:
        return
    try:
        store.save(key, json.dumps({"version": TUNE_VERSION, "pick": pick, "ms": ms, "candidates": list(candidates),
                                    "at": _now_ms()}))
    except Exception:  # persistence must never break boot
        pass


class MemoryTuneStore:
    def __init__(self, init=None):
        self.data = dict(init or {})

    def load(self, key):
        return self.data.get(key)

    def save(self, key, value):
        self.data[key] = value


class FileTuneStore:
    """One JSON file of key -> value (the place of the browser's localStorage)."""

    def __init__(self, path):
        self.path = path

    def _read(self):
        try:
            with open(self.path) as f:
                d = json.load(f)
            return d if isinstance(d, dict) else {}
        except (OSError, ValueError):
            return {}

    def load(self, key):
        return self._read().get(key)

    def save(self, key, value):
        d = self._read()
        d[key] = value
        tmp = self.path + ".tmp"
        with open(tmp, "w") as f:
            json.dump(d, f)
        os.replace(tmp, self.path)


def time_closures(sync, runs, Ms, warmup=TUNE_WARMUP, rounds=TUNE_ROUNDS, clock=time.perf_counter):
    """Time each candidate's `run(m)` (one enqueued GEMM dispatch of m rows) to completion (`sync()` blocks
    until the queue is empty), candidates interleaved within a round. Returns {name: {m: [ms, ...]}}.
    Raises nothing: a failure ends the probe and what was measured so far is returned."""
    names = list(runs)
    out = {}
    try:
        for m in Ms:
            for _ in range(warmup):
                for name in names:
                    runs[name](m)
            sync()
            for _ in range(rounds):
                for name in names:
                    t0 = clock()
                    runs[name](m)
                    sync()
                    out.setdefault(name, {}).setdefault(m, []).append((clock() - t0) * 1e3)
    except Exception:  # timing is advisory; the ladder is the fallback
        pass
    return out


def resolve_tuned_gemm(spec_id, runnable, run_probe, explicit=None, store=None, adapter_id=None, order=None):
    """The boot-time decision: {'pick', 'source': 'explicit' | 'stored' | 'probed'} or None when the static
    ladder should decide (one candidate, a stored miss plus a failed or empty probe)."""
    if explicit:
        return {"pick": explicit, "source": "explicit"}
    runnable = list(runnable)
    if len(runnable) <= 1:
        return None
    key = tune_key(adapter_id, spec_id) if adapter_id else None
    if key:
        stored = load_tuned_pick(store, key, runnable)
        if stored:
            return {"pick": stored, "source": "stored"}
    try:
        timings = run_probe() or {}
    except Exception:
        timings = {}
    medians = {}
    for name in runnable:
        per_size = timings.get(name)
        if not per_size:
            continue
        arr = [median(v) for v in per_size.values() if v]
        arr = [m for m in arr if math.isfinite(m)]
        if arr:
            medians[name] = arr
    if not medians:
        return None
    order = order if order is not None else REFERENCE_LADDER + FAMILY_LADDER
    ladder = [n for n in order if n in runnable]
    pick = pick_from_timings(medians, ladder if ladder else runnable)
    if key:
        save_tuned_pick(store, key, pick, {n: median(a) for n, a in medians.items()}, runnable)
    return {"pick": pick, "source": "probed"}


def probe_families(ctx, capi, desc, families, Ms=TUNE_MS, warmup=TUNE_WARMUP, rounds=TUNE_ROUNDS):
    """Time this library's kernel families on one dense GEMM descriptor (the caller's real gate/up weights and
    an activation buffer of at least max(Ms) rows; the content of the activations does not matter). A family
    that cannot take the shape is left out."""
    kernels = {"gemm": capi.KERNEL_GEMM, "skinny": capi.KERNEL_SKINNY, "rows": capi.KERNEL_ROWS, "gemv": capi.KERNEL_GEMV}
    runs = {}

    def make(kernel):
        def run(m):
            d = capi.MatmulDesc.from_buffer_copy(desc)
            d.kernel, d.M = kernel, m
            ctx.matmul(d)
        return run

    for name in families:
        ok = True
        for m in Ms:
            d = capi.MatmulDesc.from_buffer_copy(desc)
            d.kernel, d.M = kernels[name], m
            if capi.validate(d)[0] != 0:
                ok = False
        if ok:
            runs[name] = make(kernels[name])
    return time_closures(ctx.sync, runs, Ms, warmup, rounds)
