#!/usr/bin/env python3
"""Benchmark of the int4 dequant-matmul path on one MI355X.

Headline (BASELINE.json metric, configs[1]): int4 affine group-64 decode GEMV
at 8B shapes, M=1: (K=4096,N=14336), (K=14336,N=4096), (K=4096,N=6144).
One step = the three GEMVs on one weight set; steps rotate over distinct
weight sets whose total exceeds the 256 MB last-level cache, so every step
streams its weights from HBM. Inputs are resident in HBM before timing.

Timing discipline (the reference's, scripts/kernel-ab-ours.mjs:75-99): outputs are validated against the
oracle before anything is timed; every memory-bound row rotates over more than 256 MB of distinct
operands (`rotation_MB` in the row); the headline is the median of ROUNDS timed replays of the recorded
steps (HIP events around each, each queued behind an untimed replay so that the host's
hand-over of the command buffer is not in the timed region), with min and max beside it; a plain streaming read of the same
byte count is timed the same way in the same run (`extra.hbm_read_probe_*`); clocks are recorded.

Prints ONE JSON line: value = algorithmic weight GB/s over the timed steps,
plus `roofline` (HBM) and `cpu_baseline` (the CPU oracle on the host cores).
"""
import argparse
import importlib
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
# HBM bytes per GEMV launch (mean of the three configs[1] shapes) from two `rocprofv3 --pmc` runs of
# `bench.py --pmc` (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 256 MiB copy);
# summary in profiles/gemv_int4_configs1_hbm_traffic.md
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 27.00e6
ROTATION_FLOOR_BYTES = 300e6   # distinct operand bytes a memory-bound row rotates over: past the 256 MB last-level cache
ROUNDS = 5                     # timed replays of the headline; the median is reported
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16 MFMA, published

GEMV_SHAPES = [("ffn_gate_or_up", 4096, 14336), ("ffn_down", 14336, 4096), ("qkv_fused", 4096, 6144)]


def make_desc(capi, bits, K, N, M, bufs, kernel=0):
    return capi.MatmulDesc(bits=bits, affine=1, out_f32=0, kernel=kernel, M=M, N=N, k_packed=K * bits // 32,
                           scales_per_row=K // 64, out=bufs["out"], in_=bufs["in"], scales=bufs["s"],
                           weights=bufs["w"], biases=bufs["b"])


def upload_set(ctx, synth, K, N, bits, salt, M=1, share_in=None):
    """One weight set with its own output; `share_in` = (device address, host array) of an activation buffer that the
    sets of a rotation share (the reference's bench does: one activation buffer per shape, one output per rotation
    slot, scripts/kernel-ab-ours.mjs:97-105: in a decode loop the activations were written by the dispatch before)."""
    w = synth.packed_weights(N, K, bits=bits, salt=salt)
    s = synth.scales(N, K, salt=salt)
    b = synth.biases(N, K, s, "A", salt=salt)
    x = share_in[1] if share_in else synth.activations(M, K, salt=salt)
    bufs = {}
    for key, arr in (("w", w), ("s", s), ("b", b)) + (() if share_in else (("in", x),)):
        bufs[key] = ctx.alloc(arr.nbytes)
        ctx.upload(bufs[key], arr)
    if share_in:
        bufs["in"] = share_in[0]
    bufs["out"] = ctx.alloc(M * N * 2)
    return bufs, (x, w, s, b)


def _put(ctx, arr):
    addr = ctx.alloc(arr.nbytes)
    ctx.upload(addr, arr)
    return addr


def timed_graph(ctx, launches, reps=1, warm=1, rounds=False):
    """Record `launches` (callables) into one command buffer, replay `warm` times untimed, then time `reps` replays.
    Returns the mean milliseconds per replay, or with rounds=True the sorted list of the replays' times.
    Every timed replay is queued right behind an untimed replay of the same command buffer, with the two events
    around the second: the host needs some 25 us to hand a recorded command buffer to the GPU, and with nothing
    queued ahead the GPU would sit idle for that long inside the timed region (6 % of a replay of 20 steps; the
    kernels are what is measured, as the time stamps of a kernel trace measure them). The replays of a pair run one
    after the other on the stream, and the pair is waited for before the next is submitted.
    Compute-bound rows pass warm > 1: after an idle stretch (the oracle check before a row is one) the clock takes
    tens of milliseconds of load to come back up (the M=512 GEMM: 88 us cold, 76 after a few ms, 72 sustained)."""
    ctx.record_begin()
    for fn in launches:
        fn()
    cb = ctx.record_end()
    for _ in range(warm):
        ctx.submit(cb)
        ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    times = []
    for _ in range(reps):
        ctx.submit(cb)                          # untimed: keeps the GPU busy while the host queues what follows
        ctx.event_record(e0)
        ctx.submit(cb)
        ctx.event_record(e1)
        times.append(ctx.elapsed_ms(e0, e1))   # waits for the pair
    ctx.event_destroy(e0)
    ctx.event_destroy(e1)
    ctx.cmdbuf_destroy(cb)
    return sorted(times) if rounds else sum(times) / reps


def n_sets(bytes_per_set):
    """How many distinct operand sets a row rotates over to stay past the last-level cache."""
    return int(ROTATION_FLOOR_BYTES // bytes_per_set) + 1


def clocks():
    """Clock and power state as rocm-smi reports it, for the record (empty if the tool is not there)."""
    try:
        out = subprocess.run(["rocm-smi", "--showclocks", "--showperflevel", "--showpower", "--json"], capture_output=True,
                             text=True, timeout=20).stdout
        card = next(iter(json.loads(out).values()))
        keep = {}
        for k, v in card.items():
            kl = k.lower()
            if any(t in kl for t in ("sclk", "mclk", "fclk", "performance level", "power")):
                keep[k] = v
        return keep
    except Exception:
        return {}


def error_metrics(y, ref):
    """The three denominators the reference's own checks use, side by side: |ref| + 1e-3
    (tests/kernels/run.mjs:153), max |ref| (scripts/real-weights.mjs:72-73), max(1e-2, |ref|)
    (scripts/gemm-bench.mjs:516), and the contract's |ref| + 1e-2."""
    d = np.abs(np.asarray(y, np.float64) - ref)
    a = np.abs(ref)
    return {"ref_plus_1e-3": float(np.max(d / (a + 1e-3))), "max_abs_ref": float(np.max(d) / np.max(a)),
            "max_1e-2_ref": float(np.max(d / np.maximum(a, 1e-2))), "ref_plus_1e-2": float(np.max(d / (a + 1e-2)))}


def verify(ctx, oracle, capi, desc, host, bits, K, N, M, f16w=False):
    """Validate before timing: a launch that did not run times as ~0 and must never be reported."""
    x, w, s, b = host
    ctx.fill(desc.out, 0xFF, M * N * 2)
    ctx.matmul(desc)
    y = ctx.download(desc.out, M * N * 2, np.float16).astype(np.float64).reshape(M, N)
    rows = min(M, 4)
    # byte-valued weights give outputs near 100: an f32-accumulated reference carries more noise of its own than the
    # 1e-2 bar leaves at outputs near zero, so those rows are checked against the f64 formula
    mode = oracle.MODE_F16W if f16w else (oracle.MODE_FORMULA_F64 if bits == 8 else oracle.MODE_FORMULA_F32)
    ref = oracle.gemm(mode, bits, True, rows, N, K, x[:rows], w, s, b, threads=oracle.max_threads())
    err = float(np.max(np.abs(y[:rows] - ref) / (np.abs(ref) + 1e-2)))
    if not np.all(np.isfinite(y)) or err >= 1e-2:
        raise SystemExit("bench: output check failed (K=%d N=%d M=%d): rel err %.3e" % (K, N, M, err))
    return err


_MOE_STACK = {}


def routed_ffn_five(ctx, capi, synth, tokens, salt=0):
    """The routed FFN of configs[3] with a shared expert (257 stacked experts, 9 slots) as its five dispatches:
    router logits (8-bit) -> softmax top-k -> gate + up + SiLU (one gated GEMV pass per pair) -> down -> combine.
    Returns [(name, launch)]; the expert stack is uploaded once per context."""
    E, slots, d_model, ffn = 256, 8, 2048, 512
    E1, S = E + 1, slots + 1
    if id(ctx) not in _MOE_STACK:
        full_w = {}
        for name, N_, K_ in (("gate", ffn, d_model), ("up", ffn, d_model), ("down", d_model, ffn)):
            w = synth.packed_weights(N_, K_, experts=E1, salt=10 + len(name))
            sc = synth.scales(N_, K_, experts=E1, salt=10 + len(name))
            bi = synth.biases(N_, K_, sc, experts=E1, salt=10 + len(name))
            full_w[name] = tuple(_put(ctx, a) for a in (w, sc, bi))
        rng = np.random.default_rng(17)
        r_w = _put(ctx, rng.integers(0, 2 ** 32, (E1, d_model // 4), dtype=np.uint64).astype(np.uint32))
        r_sh = (rng.random((E1, d_model // 64)) * 2e-4 + 2e-4).astype(np.float16)
        _MOE_STACK[id(ctx)] = (full_w, r_w, _put(ctx, r_sh), _put(ctx, (-127.5 * r_sh.astype(np.float32)).astype(np.float16)))
    full_w, r_w, r_s, r_b = _MOE_STACK[id(ctx)]
    x = _put(ctx, synth.activations(tokens, d_model, salt=600 + salt))
    logits, ids, score = ctx.alloc(tokens * E1 * 4), ctx.alloc(tokens * S * 4), ctx.alloc(tokens * S * 4)
    h, dn, y = ctx.alloc(tokens * S * ffn * 2), ctx.alloc(tokens * S * d_model * 2), ctx.alloc(tokens * d_model * 2)
    common = dict(bits=4, affine=1, M=1, slots=S, tokens=tokens, ids_stride=S, experts=E1, ids=ids)
    dgated = capi.MatmulDesc(N=ffn, k_packed=d_model // 8, scales_per_row=d_model // 64, in_slot_stride=0, in_tok_stride=d_model,
                             in_=x, out_slot_stride=ffn, out_tok_stride=S * ffn, out=h, weights=full_w["gate"][0],
                             scales=full_w["gate"][1], biases=full_w["gate"][2], **common)
    dd = capi.MatmulDesc(N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, in_slot_stride=ffn, out_slot_stride=d_model,
                         in_tok_stride=S * ffn, out_tok_stride=S * d_model, in_=h, out=dn, weights=full_w["down"][0],
                         scales=full_w["down"][1], biases=full_w["down"][2], **common)
    return [("router_logits", lambda: ctx.moe_router_logits(logits, x, r_w, r_s, r_b, 8, d_model, E1, tokens)),
            ("router_topk", lambda: ctx.moe_router_topk(ids, score, logits, E, slots, True, True, tokens)),
            ("gate_up_silu", lambda: ctx.ffn_gated(dgated, full_w["up"][0], full_w["up"][1], full_w["up"][2])),
            ("down", lambda: ctx.matmul(dd)),
            ("combine", lambda: ctx.moe_combine(y, dn, score, tokens, d_model, S))]


def f16_gemm_probe(K, N, Ms, child=False):
    """The empirical ceiling beside the prefill GEMM: a plain f16 [M,K] x [K,N] product through the vendor library
    (torch.matmul -> hipBLASLt) at the same shapes, rotating over three weight matrices (352 MB), six untimed and six
    timed replays like the GEMM rows (the reference's competitor arm at the same shapes, scripts/kernel-ab-ours.mjs:
    134-140). Measurement only: nothing of the product imports torch, and the probe runs in a process of its own
    (torch brings its own copy of the HIP runtime). Empty if torch is not there."""
    if not child:
        try:
            out = subprocess.run([sys.executable, os.path.abspath(__file__), "--f16-probe-child"], capture_output=True, text=True,
                                 timeout=600)
            return json.loads(out.stdout.strip().splitlines()[-1])
        except Exception as e:   # no torch, no GPU for it, a crash of its own: the bench goes on without the rows
            sys.stderr.write("bench: f16 probe skipped (%s)\n" % (e,))
            return {}
    import torch
    rows = {}
    ws = [torch.randn(N, K, device="cuda", dtype=torch.float16) for _ in range(3)]
    for M in Ms:
        a = torch.randn(M, K, device="cuda", dtype=torch.float16)
        reps = 4 if M <= 512 else 2

        def replay():
            for _ in range(reps):
                for w in ws:
                    torch.matmul(a, w.t())

        for _ in range(6):
            replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        times = []
        for _ in range(6):
            e0.record()
            replay()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / (reps * len(ws)))
        ms = sum(times) / len(times)
        tf = 2.0 * M * K * N / ms / 1e9
        rows["f16_gemm_probe_M%d_K%d_N%d" % (M, K, N)] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1),
                                                          "mfma_f16_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                                                          "what": "torch.matmul f16 (vendor GEMM), weights as [N,K] f16",
                                                          "rotation_MB": round(3 * N * K * 2 / 1e6, 1)}
        del a
    del ws
    torch.cuda.empty_cache()
    return rows


def cpu_baseline(oracle, synth, budget_s=12.0):
    """The CPU oracle (a port of the reference's JS kernel-test reference) on this host's cores."""
    threads = oracle.max_threads()
    sets = []
    for _, K, N in GEMV_SHAPES:
        w = synth.packed_weights(N, K, salt=99)
        s = synth.scales(N, K, salt=99)
        sets.append((K, N, synth.activations(1, K, salt=99), w, s, synth.biases(N, K, s, "A", salt=99)))
    nbytes = sum(synth.weight_bytes(N, K) for _, K, N in GEMV_SHAPES)

    def one_pass(th):
        t0 = time.perf_counter()
        for K, N, x, w, s, b in sets:
            oracle.gemm(oracle.MODE_JS, 4, True, 1, N, K, x, w, s, b, threads=th)
        return time.perf_counter() - t0

    one_pass(threads)
    t_multi, t_end = [], time.perf_counter() + budget_s * 0.5
    while time.perf_counter() < t_end or len(t_multi) < 3:
        t_multi.append(one_pass(threads))
    t_single, t_end = [], time.perf_counter() + budget_s * 0.5
    while time.perf_counter() < t_end or len(t_single) < 2:
        t_single.append(one_pass(1))
    med_m, med_s = float(np.median(t_multi)), float(np.median(t_single))
    return {
        "value": round(nbytes / med_m / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "%d passes of the three configs[1] GEMVs (80.2 MB of weights each) on %d OpenMP threads; "
                  "single thread: %.3f GB/s over %d passes" % (len(t_multi), threads, nbytes / med_s / 1e9, len(t_single)),
        "single_thread_value": round(nbytes / med_s / 1e9, 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--sets", type=int, default=8, help="distinct weight sets rotated through (8 x 80 MB > 256 MB cache)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-shape, GEMM, MoE and int3 extras")
    ap.add_argument("--no-f16-probe", action="store_true", help="skip the vendor f16 GEMM rows (they import torch)")
    ap.add_argument("--pmc", nargs="?", const="base", default=None, choices=["base", "down", "moe"],
                    help="counter-collection mode for `rocprofv3 --pmc`: a few eager launches of a 256 MiB copy "
                         "(calibration), then (base) of each configs[1] GEMV, of the M=512 prefill GEMM and of the "
                         "small-batch families (M = 8, 32, 128), or (down) of the down projection of a 512-row "
                         "prefill chunk (K=14336, N=4096) in the family the library picks and in the tile GEMM, or (moe) of the routed "
                         "FFN of configs[3] as five dispatches at 1 and 16 tokens and of the row-group GEMV at M=8 (int4, int3); no timing")
    ap.add_argument("--option", action="append", default=[], help="name=value launch knob (ztvm_set_option)")
    ap.add_argument("--f16-probe-child", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.f16_probe_child:
        print(json.dumps(f16_gemm_probe(4096, 14336, (128, 512, 2048), child=True)))
        return
    if args.gpus != 1:
        raise SystemExit("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
                         "(a second GPU would own a column range of each weight matrix; nothing here uses one)" % args.gpus)

    pkg = importlib.import_module("zero-tvm_amd")
    capi = pkg.capi
    synth = importlib.import_module("zero-tvm_amd.host.synth")
    from oracle import oracle

    ctx = capi.Context(0)
    for opt in args.option:
        k, v = opt.split("=")
        ctx.set_option(k, int(v))
    info = ctx.device_info()

    if args.pmc:
        nbytes = 256 << 20
        src, dst = ctx.alloc(nbytes), ctx.alloc(nbytes)
        ctx.fill(src, 1, nbytes)
        for _ in range(3):
            ctx.copy(dst, src, nbytes)
        if args.pmc == "moe":
            for tokens in (1, 16):
                blocks = [routed_ffn_five(ctx, capi, synth, tokens, salt=r) for r in range(3)]
                for r in range(6):
                    for _, fn in blocks[r % 3]:
                        fn()
            K, N = 4096, 14336
            for bits in (4, 3):
                bdescs = [make_desc(capi, bits, K, N, 8, upload_set(ctx, synth, K, N, bits, salt=r, M=8)[0]) for r in range(2)]
                for r in range(6):
                    ctx.matmul(bdescs[r % 2])
            ctx.sync()
            ctx.close()
            print(json.dumps({"pmc_mode": "moe", "copy_bytes": nbytes}))
            return
        if args.pmc == "down":
            K, N, M = 14336, 4096, 512
            for kern in (capi.KERNEL_AUTO, capi.KERNEL_GEMM):
                ddescs = [make_desc(capi, 4, K, N, M, upload_set(ctx, synth, K, N, 4, salt=r, M=M)[0], kernel=kern) for r in range(2)]
                for r in range(6):
                    ctx.matmul(ddescs[r % 2])
            ctx.sync()
            ctx.close()
            print(json.dumps({"pmc_mode": "down", "copy_bytes": nbytes}))
            return
        for i, (_, K, N) in enumerate(GEMV_SHAPES):
            descs = [make_desc(capi, 4, K, N, 1, upload_set(ctx, synth, K, N, 4, salt=r)[0]) for r in range(4)]
            for r in range(8):
                ctx.matmul(descs[r % 4])
        # the prefill GEMM of configs[2] at M=512, for its own counters
        K, N, M = 4096, 14336, 512
        gdescs = [make_desc(capi, 4, K, N, M, upload_set(ctx, synth, K, N, 4, salt=r, M=M)[0], kernel=capi.KERNEL_GEMM)
                  for r in range(2)]
        for r in range(6):
            ctx.matmul(gdescs[r % 2])
        # the small-batch families at their bench shapes (family chosen by the library), six launches each over two sets
        for bits, M in ((4, 8), (3, 8), (4, 32), (4, 128), (8, 128)):
            bdescs = [make_desc(capi, bits, K, N, M, upload_set(ctx, synth, K, N, bits, salt=r, M=M)[0]) for r in range(2)]
            for r in range(6):
                ctx.matmul(bdescs[r % 2])
        ctx.sync()
        ctx.close()
        print(json.dumps({"pmc_mode": True, "copy_bytes": nbytes}))
        return

    # ---- headline: rotating weight sets, three GEMVs per step ------------------
    # per shape enough distinct sets to rotate past the last-level cache on its own (the small QKV shape needs
    # twenty), so the per-shape rows below are HBM measurements too; step r takes set r % n of every shape
    shape_sets, shape_hosts, shape_bytes = [], [], []
    for i, (_, K, N) in enumerate(GEMV_SHAPES):
        wb = synth.weight_bytes(N, K)
        per_set, first_host = [], None
        x_host = synth.activations(1, K, salt=i)
        x_shared = (_put(ctx, x_host), x_host)   # one activation vector per shape, as in a decode loop
        for r in range(max(args.sets, n_sets(wb))):
            bufs, host = upload_set(ctx, synth, K, N, 4, salt=10 * r + i, share_in=x_shared)
            desc = make_desc(capi, 4, K, N, 1, bufs)
            if r == 0:
                verify(ctx, oracle, capi, desc, host, 4, K, N, 1)
                first_host = host
            per_set.append(desc)
        shape_sets.append(per_set)
        shape_hosts.append(first_host)
        shape_bytes.append(wb)
    step_bytes = sum(shape_bytes)
    rotation_bytes = sum(len(ss) * wb for ss, wb in zip(shape_sets, shape_bytes))
    sets = [[ss[r % len(ss)] for ss in shape_sets] for r in range(max(len(ss) for ss in shape_sets))]  # sets[r][shape]

    def step(i, table=None):
        for desc in (table or sets)[i % len(sets)]:
            ctx.matmul(desc)

    for i in range(args.warmup):
        step(i)
    ctx.sync()
    rounds = timed_graph(ctx, [lambda i=i: step(i) for i in range(args.steps)], reps=ROUNDS, rounds=True)
    ms_total = rounds[len(rounds) // 2]
    ms_per_step = ms_total / args.steps
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    launches = 3 * args.steps
    avg_launch_us = ms_total * 1e3 / launches

    result = {
        "metric": "int4 GEMV GB/s (% of HBM peak) at M=1; prefill GEMM TFLOP/s at M=512",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights (u32-packed), f16 activations, f32 accumulate", "data": "synthetic",
        "config": {"workload": "configs[1]: int4 affine g64 decode GEMV, M=1, (4096->14336)+(14336->4096)+(4096->6144) "
                               "per step, rotating over %.0f MB of distinct weights" % (rotation_bytes / 1e6),
                   "device": info["name"], "compute_units": info["compute_units"], "rotation_MB": round(rotation_bytes / 1e6, 1),
                   "timing": "median of %d replays of %d recorded steps, HIP events around each, each queued behind an untimed replay" % (ROUNDS, args.steps),
                   "activations": "one vector per shape shared by its weight sets, one output per set (scripts/kernel-ab-ours.mjs:97-105)",
                   "ms_per_step_min": round(rounds[0] / args.steps, 6), "ms_per_step_max": round(rounds[-1] / args.steps, 6),
                   "clocks": clocks()},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel": "ztvm::gemv_stream_kernel<4,true,2,*,*>", "bytes_per_launch": step_bytes / 3.0,
                     "avg_launch_us": round(avg_launch_us, 3), "launches": launches},
    }

    if not args.no_extra:
        extra = {}
        sink = ctx.alloc(64)
        # per shape, each alone over its own rotating sets, with a plain streaming read of the same bytes beside it
        # (the packed words of the same sets read by a kernel that does nothing else): the empirical ceiling
        for i, (name, K, N) in enumerate(GEMV_SHAPES):
            ss, wb = shape_sets[i], shape_bytes[i]
            reps = max(2, 160 // len(ss))
            n = reps * len(ss)
            ms = timed_graph(ctx, [lambda d=ss[j % len(ss)]: ctx.matmul(d) for j in range(n)], reps=ROUNDS, rounds=True)[ROUNDS // 2] / n
            pb = N * (K // 8) * 4
            ms_r = timed_graph(ctx, [lambda d=ss[j % len(ss)]: ctx.read_probe(d.weights, pb, sink) for j in range(n)], reps=ROUNDS,
                               rounds=True)[ROUNDS // 2] / n
            extra["gemv_%s_K%d_N%d" % (name, K, N)] = {"us": round(ms * 1e3, 3), "GB/s": round(wb / ms / 1e6, 1),
                                                       "hbm_frac": round(wb / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                       "rotation_MB": round(len(ss) * wb / 1e6, 1)}
            extra["hbm_read_probe_%.0fMB_%s" % (pb / 1e6, name)] = {"us": round(ms_r * 1e3, 3), "GB/s": round(pb / ms_r / 1e6, 1),
                                                                   "hbm_frac": round(pb / ms_r / 1e6 / HBM_PEAK_GBS, 4),
                                                                   "bytes": pb, "rotation_MB": round(len(ss) * pb / 1e6, 1)}
        # bias regime B (MLX-like centred biases, b = -7.5 s (1 +- 0.1): every weight sits near zero and the two terms
        # of s*dot + b*sum(x) cancel): same weights and scales, other biases; validated, then the same step timed.
        # The errors of both regimes under the reference's three denominators are reported side by side.
        errs = {}
        setsB = []
        for r in range(len(sets)):
            rowB = []
            for i, (_, K, N) in enumerate(GEMV_SHAPES):
                d = sets[r][i]
                if r < len(shape_sets[i]):
                    sc_host = synth.scales(N, K, salt=10 * r + i)
                    bB = synth.biases(N, K, sc_host, "B", salt=10 * r + i)
                    dB = capi.MatmulDesc(bits=4, affine=1, M=1, N=N, k_packed=K // 8, scales_per_row=K // 64, out=d.out, in_=d.in_,
                                         scales=d.scales, weights=d.weights, biases=_put(ctx, bB))
                    if r == 0:
                        x0, w0, s0, bA = shape_hosts[i]
                        for regime, dd, bb in (("A", d, bA), ("B", dB, bB)):
                            ctx.matmul(dd)
                            y = ctx.download(dd.out, N * 2, np.float16).astype(np.float64)
                            ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x0, w0, s0, bb, threads=oracle.max_threads())[0]
                            m = error_metrics(y, ref)
                            if m["ref_plus_1e-2"] >= 1e-2:
                                raise SystemExit("bench: regime %s output check failed (K=%d N=%d): %r" % (regime, K, N, m))
                            errs["regime%s_K%d_N%d" % (regime, K, N)] = {k: float("%.3g" % v) for k, v in m.items()}
                    rowB.append(dB)
                else:
                    rowB.append(setsB[r % len(shape_sets[i])][i])
            setsB.append(rowB)
        msB = timed_graph(ctx, [lambda i=i: step(i, setsB) for i in range(args.steps)], reps=ROUNDS, rounds=True)[ROUNDS // 2] / args.steps
        extra["gemv_step_bias_regime_B"] = {"ms_per_step": round(msB, 6), "GB/s": round(step_bytes / msB / 1e6, 1),
                                            "hbm_frac": round(step_bytes / msB / 1e6 / HBM_PEAK_GBS, 4),
                                            "rotation_MB": round(rotation_bytes / 1e6, 1)}
        extra["gemv_max_rel_err_vs_fp32_accumulated_reference"] = errs
        # prefill GEMM (configs[2]): K=4096, N=14336, M in {128, 512, 2048}
        gsets = []
        g_wb = synth.weight_bytes(14336, 4096)
        gx_host = synth.activations(2048, 4096, salt=100)
        gx = (_put(ctx, gx_host), gx_host)   # one activation buffer for every weight set of the rotation
        for r in range(n_sets(g_wb)):
            bufs, host = upload_set(ctx, synth, 4096, 14336, 4, salt=100 + r, M=2048, share_in=gx)
            gsets.append((bufs, host))
        ng = len(gsets)
        for M in (128, 512, 2048):
            descs = [make_desc(capi, 4, 4096, 14336, M, b, kernel=capi.KERNEL_GEMM) for b, _ in gsets]
            verify(ctx, oracle, capi, descs[0], gsets[0][1], 4, 4096, 14336, M)
            reps = 4 if M <= 512 else 1
            ms = timed_graph(ctx, [lambda d=descs[j % ng]: ctx.matmul(d) for j in range(reps * ng)], reps=6, warm=6) / (reps * ng)
            tf = 2.0 * M * 4096 * 14336 / ms / 1e9
            extra["gemm_M%d_K4096_N14336" % M] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1),
                                                  "mfma_f16_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "family": "gemm (forced)",
                                                  "rotation_MB": round((ng * g_wb + M * 4096 * 2) / 1e6, 1)}
            # the same dispatch with the family left to the library
            adescs = [make_desc(capi, 4, 4096, 14336, M, b) for b, _ in gsets]
            fam = capi.KERNEL_NAMES[capi.resolve(adescs[0])]
            if fam != "gemm":
                verify(ctx, oracle, capi, adescs[0], gsets[0][1], 4, 4096, 14336, M)
                ms = timed_graph(ctx, [lambda d=adescs[j % ng]: ctx.matmul(d) for j in range(reps * ng)], reps=6, warm=6) / (reps * ng)
                tf = 2.0 * M * 4096 * 14336 / ms / 1e9
            extra["gemm_M%d_K4096_N14336_auto" % M] = {"us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1),
                                                       "mfma_f16_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "family": fam}
        if not args.no_f16_probe:
            extra.update(f16_gemm_probe(4096, 14336, (128, 512, 2048)))
        # the down projection of the same prefill chunk (K=14336 -> N=4096, M=512): 32 column tiles, where the family
        # choice goes by an estimate of both kernels; the library's choice beside the tile GEMM forced. Weights: the
        # headline's rotating sets of this shape; one activation buffer, one output per set
        Kd, Nd, Md = 14336, 4096, 512
        xa = synth.activations(Md, Kd, salt=77)
        a_dev = _put(ctx, xa)
        dsets = shape_sets[1]
        outs = [ctx.alloc(Md * Nd * 2) for _ in dsets]
        x0, w0, s0, b0 = shape_hosts[1]
        for fam_name, kern in (("auto", capi.KERNEL_AUTO), ("tile_gemm", capi.KERNEL_GEMM)):
            descs = [capi.MatmulDesc(bits=4, affine=1, kernel=kern, M=Md, N=Nd, k_packed=Kd // 8, scales_per_row=Kd // 64, out=o,
                                     in_=a_dev, scales=d.scales, weights=d.weights, biases=d.biases) for d, o in zip(dsets, outs)]
            verify(ctx, oracle, capi, descs[0], (xa, w0, s0, b0), 4, Kd, Nd, Md)
            nd_ = len(descs)
            ms = timed_graph(ctx, [lambda d=descs[j % nd_]: ctx.matmul(d) for j in range(2 * nd_)], reps=6, warm=6) / (2 * nd_)
            tf = 2.0 * Md * Kd * Nd / ms / 1e9
            extra["gemm_M512_K14336_N4096_%s" % fam_name] = {
                "us": round(ms * 1e3, 2), "TFLOP/s": round(tf, 1), "mfma_f16_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                "family": {capi.KERNEL_SKINNY: "skinny", capi.KERNEL_GEMM: "gemm"}.get(capi.resolve(descs[0]), "?"),
                "rotation_MB": round(nd_ * shape_bytes[1] / 1e6, 1)}
        # int3 decode GEMV (configs[4], M=1)
        wb = synth.weight_bytes(14336, 4096, bits=3)
        n3 = n_sets(wb)
        x3_host = synth.activations(1, 4096, salt=200)
        x3 = (_put(ctx, x3_host), x3_host)
        i3 = [upload_set(ctx, synth, 4096, 14336, 3, salt=200 + r, share_in=x3) for r in range(n3)]
        d3 = [make_desc(capi, 3, 4096, 14336, 1, b) for b, _ in i3]
        verify(ctx, oracle, capi, d3[0], i3[0][1], 3, 4096, 14336, 1)
        ms = timed_graph(ctx, [lambda d=d3[j % n3]: ctx.matmul(d) for j in range(16 * n3)], reps=ROUNDS, rounds=True)[ROUNDS // 2] / (16 * n3)
        extra["gemv_int3_K4096_N14336"] = {"us": round(ms * 1e3, 3), "GB/s": round(wb / ms / 1e6, 1),
                                           "hbm_frac": round(wb / ms / 1e6 / HBM_PEAK_GBS, 4), "rotation_MB": round(n3 * wb / 1e6, 1)}
        # 8-bit affine decode GEMV (int8_affine_matvec's shape family): twice the bytes per value, fewer vector
        # instructions per byte
        i8 = []
        for r in range(6):
            w = synth.packed_weights(14336, 4096, bits=8, salt=400 + r)
            sc = synth.scales(14336, 4096, salt=400 + r)
            bi = synth.biases(14336, 4096, sc, "A", salt=400 + r)
            xx = synth.activations(1, 4096, salt=400 + r)
            bufs = {"w": _put(ctx, w), "s": _put(ctx, sc), "b": _put(ctx, bi), "in": _put(ctx, xx), "out": ctx.alloc(14336 * 2)}
            dsc = capi.MatmulDesc(bits=8, affine=1, M=1, N=14336, k_packed=4096 // 4, scales_per_row=64, out=bufs["out"],
                                  in_=bufs["in"], scales=bufs["s"], weights=bufs["w"], biases=bufs["b"])
            if r == 0:
                verify(ctx, oracle, capi, dsc, (xx, w, sc, bi), 8, 4096, 14336, 1)
            i8.append(dsc)
        ms = timed_graph(ctx, [lambda d=i8[j % 6]: ctx.matmul(d) for j in range(120)]) / 120
        wb = synth.weight_bytes(14336, 4096, bits=8)
        extra["gemv_int8_K4096_N14336"] = {"us": round(ms * 1e3, 3), "GB/s": round(wb / ms / 1e6, 1),
                                           "hbm_frac": round(wb / ms / 1e6 / HBM_PEAK_GBS, 4), "rotation_MB": round(6 * wb / 1e6, 1)}
        # QKV matmul + RoPE + KV append in one dispatch at the configs[1] qkv shape (32 heads, 8 KV heads of 128 = 6144 rows)
        qs = []
        hps, vpo, kps = 16 * 128, 8 * 16 * 128, 2 * 8 * 16 * 128
        kvbuf, qout = ctx.alloc(64 * kps * 2), ctx.alloc(4096 * 2)
        ctx.fill(kvbuf, 0, 64 * kps * 2)
        pmap = _put(ctx, np.array([517], np.int32))
        nq = len(shape_sets[2])
        for r in range(nq):
            d0 = shape_sets[2][r]   # the (4096 -> 6144) weight sets of the headline
            qs.append(capi.QkvFusedDesc(bits=4, affine=1, k_packed=512, scales_per_row=64, heads=32, kv_heads=8, head_dim=128,
                                        page_size=16, kv_page_stride=kps, head_page_stride=hps, v_page_offset=vpo,
                                        rope_theta=500000.0, kv_capacity=64 * kps, q_out=qout, kv_pages=kvbuf, hidden=d0.in_,
                                        scales=d0.scales, weights=d0.weights, position_map=pmap, biases=d0.biases))
        ctx.qkv_fused(qs[0])
        if not np.all(np.isfinite(ctx.download(qout, 4096 * 2, np.float16))):
            raise SystemExit("bench: fused QKV check failed")
        ms = timed_graph(ctx, [lambda d=qs[j % nq]: ctx.qkv_fused(d) for j in range(8 * nq)]) / (8 * nq)
        wb = synth.weight_bytes(6144, 4096)
        extra["qkv_fused_rope_kvappend_K4096_N6144"] = {"us": round(ms * 1e3, 3), "GB/s": round(wb / ms / 1e6, 1),
                                                        "hbm_frac": round(wb / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                        "rotation_MB": round(nq * wb / 1e6, 1)}
        # the int8-KV pair at the same shape: QKV + RoPE to scratch rows, then the quantizer into the int8 pages
        kslot, vslot = ctx.alloc(1024 * 2), ctx.alloc(1024 * 2)
        i8pages, i8scales = ctx.alloc(64 * 8 * 16 * 2 * 32 * 4), ctx.alloc(64 * 8 * 16 * 2 * 2)
        kvq = capi.KvQuantizeDesc(kv_heads=8, head_dim=128, page_size=16, tokens=1, pages_capacity_words=64 * 8 * 16 * 2 * 32,
                                  scales_capacity=64 * 8 * 16 * 2, k_slot=kslot, v_slot=vslot, pages_i8=i8pages, scales=i8scales,
                                  position_map=pmap)

        def int8_pair(d):
            ctx.qkv_fused_scratch(d, kslot, vslot)
            ctx.kv_quantize_int8(kvq)

        int8_pair(qs[0])
        got_sc = ctx.download(i8scales, 64 * 8 * 16 * 2 * 2, np.float16).reshape(64, 8, 16, 2)[517 // 16, :, 517 % 16, :]
        krow = np.abs(ctx.download(kslot, 1024 * 2, np.float16).astype(np.float32)).reshape(8, 128).max(axis=1) / np.float32(127)
        if not np.array_equal(got_sc[:, 0], krow.astype(np.float16)):
            raise SystemExit("bench: int8 KV scale check failed")
        ms2 = timed_graph(ctx, [lambda d=qs[j % nq]: int8_pair(d) for j in range(8 * nq)]) / (8 * nq)
        ms1 = timed_graph(ctx, [lambda: ctx.kv_quantize_int8(kvq) for j in range(160)]) / 160
        extra["qkv_scratch_then_kv_quantize_int8_K4096_N6144"] = {"us": round(ms2 * 1e3, 3), "kv_quantize_us": round(ms1 * 1e3, 3)}
        # the four weight-streaming dispatches of one 8B decoder layer with the fused forms: QKV + RoPE + KV append,
        # o_proj, gate + up + SiLU, down (attention itself is not part of this path): 122.7 MB of weights per layer
        lsets = []
        for r in range(6):
            o_b, _ = upload_set(ctx, synth, 4096, 4096, 4, salt=500 + r)
            up_b, _ = upload_set(ctx, synth, 4096, 14336, 4, salt=520 + r)
            hbuf = ctx.alloc(14336 * 2)
            g0, d0 = shape_sets[0][r % len(shape_sets[0])], shape_sets[1][r % len(shape_sets[1])]
            gated = capi.MatmulDesc(bits=4, affine=1, M=1, N=14336, k_packed=512, scales_per_row=64, out=hbuf, in_=g0.in_,
                                    scales=g0.scales, weights=g0.weights, biases=g0.biases)
            down = capi.MatmulDesc(bits=4, affine=1, M=1, N=4096, k_packed=1792, scales_per_row=224, out=d0.out, in_=hbuf,
                                   scales=d0.scales, weights=d0.weights, biases=d0.biases)
            lsets.append((qs[r % nq], make_desc(capi, 4, 4096, 4096, 1, o_b), gated, (up_b["w"], up_b["s"], up_b["b"]), down))

        def layer(L):
            q_, o_, g_, u_, d_ = L
            ctx.qkv_fused(q_)
            ctx.matmul(o_)
            ctx.ffn_gated(g_, *u_)
            ctx.matmul(d_)

        layer(lsets[0])
        ms = timed_graph(ctx, [lambda L=lsets[j % 6]: layer(L) for j in range(60)]) / 60
        lbytes = (synth.weight_bytes(6144, 4096) + synth.weight_bytes(4096, 4096) + 2 * synth.weight_bytes(14336, 4096)
                  + synth.weight_bytes(4096, 14336))
        extra["decode_layer_8b_four_dispatches"] = {"us": round(ms * 1e3, 2), "GB/s": round(lbytes / ms / 1e6, 1),
                                                    "hbm_frac": round(lbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "weight_MB": round(lbytes / 1e6, 1),
                                                    "rotation_MB": round(6 * lbytes / 1e6, 1)}
        # gate + up + SiLU at the 8B layer shape, plain and with the add + RMSNorm prologue folded in
        dl, gm = _put(ctx, (synth.activations(1, 4096, salt=77).view(np.float16) * 0.3).astype(np.float16)), \
            _put(ctx, np.full(4096, 1.0, np.float16))
        ms_g = timed_graph(ctx, [lambda L=lsets[j % 6]: ctx.ffn_gated(L[2], *L[3]) for j in range(60)]) / 60
        ms_p = timed_graph(ctx, [lambda L=lsets[j % 6]: ctx.ffn_gated_prologue(L[2], *L[3], dl, gm, 1e-5) for j in range(60)]) / 60
        gbytes = 2 * synth.weight_bytes(14336, 4096)
        extra["ffn_gated_K4096_N14336"] = {"us": round(ms_g * 1e3, 2), "GB/s": round(gbytes / ms_g / 1e6, 1),
                                           "hbm_frac": round(gbytes / ms_g / 1e6 / HBM_PEAK_GBS, 4),
                                           "with_add_rmsnorm_prologue_us": round(ms_p * 1e3, 2), "rotation_MB": round(6 * gbytes / 1e6, 1)}
        # small batches: the row-group GEMV (M <= 16) and the weight-streaming matrix-core kernel (M <= 128); int4,
        # configs[4]'s int3 M=8, and 8-bit rows (M=512: the 3-bit and 8-bit forms of the tile GEMM)
        other_sets = {}
        for bits, M in ((4, 2), (4, 4), (4, 8), (4, 16), (4, 32), (4, 128), (3, 8), (3, 512), (8, 8), (8, 128), (8, 512)):
            wb = synth.weight_bytes(14336, 4096, bits=bits)
            if bits == 4:
                descs = [make_desc(capi, 4, 4096, 14336, M, b) for b, _ in gsets]
                host0 = gsets[0][1]
            else:
                if (bits, "sets") not in other_sets:   # one rotation per width, built for the largest M it is used at
                    ox_host = synth.activations(512, 4096, salt=300 + bits)
                    ox = (_put(ctx, ox_host), ox_host)
                    other_sets[(bits, "sets")] = [upload_set(ctx, synth, 4096, 14336, bits, salt=300 + 10 * bits + r, M=512, share_in=ox)
                                                  for r in range(n_sets(wb))]
                other = other_sets[(bits, "sets")]
                descs = [make_desc(capi, bits, 4096, 14336, M, b) for b, _ in other]
                host0 = other[0][1]
            nd = len(descs)
            verify(ctx, oracle, capi, descs[0], host0, bits, 4096, 14336, M)
            heavy = M >= 128  # matrix-core rows: sustained clock, as for the GEMM rows above
            ms = timed_graph(ctx, [lambda d=descs[j % nd]: ctx.matmul(d) for j in range(4 * nd)], reps=6 if heavy else 3,
                             warm=6 if heavy else 1) / (4 * nd)
            extra["batch_int%d_M%d_K4096_N14336" % (bits, M)] = {
                "us": round(ms * 1e3, 2), "TFLOP/s": round(2.0 * M * 4096 * 14336 / ms / 1e9, 1),
                "weights_GB/s": round(wb / ms / 1e6, 1), "family": capi.KERNEL_NAMES[capi.resolve(descs[0])],
                "rotation_MB": round(nd * wb / 1e6, 1)}
        # MoE expert block (configs[3]): 256 experts, top-8, hidden 2048, intermediate 512; gate + up + down per token batch
        E, slots, d_model, ffn = 256, 8, 2048, 512
        moe_w = {}
        for name, N_, K_ in (("gate", ffn, d_model), ("up", ffn, d_model), ("down", d_model, ffn)):
            w = synth.packed_weights(N_, K_, experts=E, salt=len(name))
            sc = synth.scales(N_, K_, experts=E, salt=len(name))
            bi = synth.biases(N_, K_, sc, experts=E, salt=len(name))
            moe_w[name] = tuple(_put(ctx, a) for a in (w, sc, bi))
        per_expert = 2 * synth.weight_bytes(ffn, d_model) + synth.weight_bytes(d_model, ffn)
        for tokens in (1, 16):
            # every replay routes to other experts: one token walks a permutation of all 256 experts in 32 replays,
            # sixteen tokens draw fresh ids per replay, so the experts touched across the rotation (the whole 453 MB
            # stack) do not fit the last-level cache and expert_GB/s is an HBM figure
            if tokens == 1:
                perm = np.random.default_rng(23).permutation(E).astype(np.uint32)
                id_sets = [perm[8 * r:8 * r + 8].reshape(1, slots) for r in range(E // slots)]
            else:
                id_sets = [synth.topk_ids(tokens, slots, E, salt=100 * tokens + r) for r in range(6)]
            x = _put(ctx, synth.activations(tokens, d_model, salt=5))
            gu = ctx.alloc(tokens * slots * 2 * ffn * 2)
            out = ctx.alloc(tokens * slots * d_model * 2)
            hf, out_f = ctx.alloc(tokens * slots * ffn * 2), ctx.alloc(tokens * slots * d_model * 2)
            trios, pairs = [], []
            for ids in id_sets:
                d_ids = _put(ctx, ids)
                gcommon = dict(bits=4, affine=1, M=1, N=ffn, k_packed=d_model // 8, scales_per_row=d_model // 64, slots=slots,
                               tokens=tokens, in_slot_stride=0, out_slot_stride=2 * ffn, in_tok_stride=d_model,
                               out_tok_stride=slots * 2 * ffn, ids_stride=slots, experts=E, in_=x, ids=d_ids)
                dg = capi.MatmulDesc(out=gu, weights=moe_w["gate"][0], scales=moe_w["gate"][1], biases=moe_w["gate"][2], **gcommon)
                du = capi.MatmulDesc(out=gu + ffn * 2, weights=moe_w["up"][0], scales=moe_w["up"][1], biases=moe_w["up"][2], **gcommon)
                dd = capi.MatmulDesc(bits=4, affine=1, M=1, N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, slots=slots,
                                     tokens=tokens, in_slot_stride=2 * ffn, out_slot_stride=d_model, in_tok_stride=slots * 2 * ffn,
                                     out_tok_stride=slots * d_model, ids_stride=slots, experts=E, out=out, in_=gu, ids=d_ids,
                                     weights=moe_w["down"][0], scales=moe_w["down"][1], biases=moe_w["down"][2])
                trios.append((dg, du, dd))
                # the same block as two launches: gate + up + SiLU in one pass over the token's activations, then down
                fcommon = dict(gcommon, out_slot_stride=ffn, out_tok_stride=slots * ffn)
                dgu = capi.MatmulDesc(out=hf, weights=moe_w["gate"][0], scales=moe_w["gate"][1], biases=moe_w["gate"][2], **fcommon)
                ddf = capi.MatmulDesc(bits=4, affine=1, M=1, N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, slots=slots,
                                      tokens=tokens, in_slot_stride=ffn, out_slot_stride=d_model, in_tok_stride=slots * ffn,
                                      out_tok_stride=slots * d_model, ids_stride=slots, experts=E, out=out_f, in_=hf, ids=d_ids,
                                      weights=moe_w["down"][0], scales=moe_w["down"][1], biases=moe_w["down"][2])
                pairs.append((dgu, ddf))
            nrep = 2 * len(trios)
            ms = timed_graph(ctx, [lambda d=d_: ctx.matmul(d) for r in range(nrep) for d_ in trios[r % len(trios)]], reps=3) / nrep
            per_replay = [len(set(int(v) for v in ids.reshape(-1))) for ids in id_sets]
            union = len(set(int(v) for ids in id_sets for v in ids.reshape(-1)))
            distinct = float(np.mean(per_replay))
            extra["moe_block_tokens%d" % tokens] = {"us": round(ms * 1e3, 2), "launches": 3, "pairs": tokens * slots, "distinct_experts": round(distinct, 1),
                                                     "expert_GB/s": round(distinct * per_expert / ms / 1e6, 1),
                                                     "hbm_frac": round(distinct * per_expert / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                     "rotation_MB": round(union * per_expert / 1e6, 1)}

            def fused_block(pr):
                ctx.ffn_gated(pr[0], moe_w["up"][0], moe_w["up"][1], moe_w["up"][2])
                ctx.matmul(pr[1])

            # checked against the three-launch form before it is timed: down(silu(gate) * up) of the same experts
            for d_ in trios[0]:
                ctx.matmul(d_)
            fused_block(pairs[0])
            g_u = ctx.download(gu, tokens * slots * 2 * ffn * 2, np.float16).astype(np.float32).reshape(tokens * slots, 2, ffn)
            h_ref = (g_u[:, 1] * (g_u[:, 0] / (1.0 + np.exp(-g_u[:, 0])))).astype(np.float64)
            h_got = ctx.download(hf, tokens * slots * ffn * 2, np.float16).astype(np.float64).reshape(tokens * slots, ffn)
            if not np.all(np.isfinite(h_got)) or float(np.max(np.abs(h_got - h_ref) / (np.abs(h_ref) + 1e-2))) > 1e-2:
                raise SystemExit("bench: two-launch MoE block disagrees with the three-launch form (tokens=%d)" % tokens)
            ms = timed_graph(ctx, [lambda pr=pairs[r % len(pairs)]: fused_block(pr) for r in range(nrep)], reps=3) / nrep
            extra["moe_block_fused_tokens%d" % tokens] = {"us": round(ms * 1e3, 2), "launches": 2, "pairs": tokens * slots,
                                                           "expert_GB/s": round(distinct * per_expert / ms / 1e6, 1),
                                                           "hbm_frac": round(distinct * per_expert / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                           "rotation_MB": round(union * per_expert / 1e6, 1)}
        # the whole routed FFN of configs[3] with a shared expert (257 stacked experts, 9 slots): router logits
        # (8-bit) -> softmax top-k -> gate, up -> silu_mul -> down -> combine, routed on the device
        E1, S = E + 1, slots + 1
        full_w = {}
        for name, N_, K_ in (("gate", ffn, d_model), ("up", ffn, d_model), ("down", d_model, ffn)):
            w = synth.packed_weights(N_, K_, experts=E1, salt=10 + len(name))
            sc = synth.scales(N_, K_, experts=E1, salt=10 + len(name))
            bi = synth.biases(N_, K_, sc, experts=E1, salt=10 + len(name))
            full_w[name] = tuple(_put(ctx, a) for a in (w, sc, bi))
        rng = np.random.default_rng(17)
        r_w = _put(ctx, rng.integers(0, 2 ** 32, (E1, d_model // 4), dtype=np.uint64).astype(np.uint32))
        # router weights centred on zero (w = s*(q - 127.5)) so the logits are O(1) like a trained router's;
        # logits of +-100 would push all but one probability under the f32 range and leave the top-k to ties
        r_sh = (rng.random((E1, d_model // 64)) * 2e-4 + 2e-4).astype(np.float16)
        r_s = _put(ctx, r_sh)
        r_b = _put(ctx, (-127.5 * r_sh.astype(np.float32)).astype(np.float16))
        for tokens in (1, 16):
            # other activations every replay, so the router sends every replay to other experts and the experts
            # touched across the rotation outgrow the last-level cache
            NX = 32 if tokens == 1 else 6
            xbank = [_put(ctx, synth.activations(tokens, d_model, salt=600 + r)) for r in range(NX)]
            logits, ids, score = ctx.alloc(tokens * E1 * 4), ctx.alloc(tokens * S * 4), ctx.alloc(tokens * S * 4)
            gu, hbuf = ctx.alloc(tokens * S * 2 * ffn * 2), ctx.alloc(tokens * S * ffn * 2)
            dn, y = ctx.alloc(tokens * S * d_model * 2), ctx.alloc(tokens * d_model * 2)
            h2buf, dn2, y2 = ctx.alloc(tokens * S * ffn * 2), ctx.alloc(tokens * S * d_model * 2), ctx.alloc(tokens * d_model * 2)
            common = dict(bits=4, affine=1, M=1, slots=S, tokens=tokens, ids_stride=S, experts=E1, ids=ids)
            dd = capi.MatmulDesc(N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, in_slot_stride=ffn,
                                 out_slot_stride=d_model, in_tok_stride=S * ffn, out_tok_stride=S * d_model, in_=hbuf, out=dn,
                                 weights=full_w["down"][0], scales=full_w["down"][1], biases=full_w["down"][2], **common)
            dd2 = capi.MatmulDesc(N=d_model, k_packed=ffn // 8, scales_per_row=ffn // 64, in_slot_stride=ffn,
                                  out_slot_stride=d_model, in_tok_stride=S * ffn, out_tok_stride=S * d_model, in_=h2buf, out=dn2,
                                  weights=full_w["down"][0], scales=full_w["down"][1], biases=full_w["down"][2], **common)

            def block(x):
                gshape = dict(N=ffn, k_packed=d_model // 8, scales_per_row=d_model // 64, in_slot_stride=0, in_tok_stride=d_model, in_=x)
                dg = capi.MatmulDesc(out_slot_stride=2 * ffn, out_tok_stride=S * 2 * ffn, out=gu, weights=full_w["gate"][0],
                                     scales=full_w["gate"][1], biases=full_w["gate"][2], **gshape, **common)
                du = capi.MatmulDesc(out_slot_stride=2 * ffn, out_tok_stride=S * 2 * ffn, out=gu + ffn * 2, weights=full_w["up"][0],
                                     scales=full_w["up"][1], biases=full_w["up"][2], **gshape, **common)
                dgated = capi.MatmulDesc(out_slot_stride=ffn, out_tok_stride=S * ffn, out=h2buf, weights=full_w["gate"][0],
                                         scales=full_w["gate"][1], biases=full_w["gate"][2], **gshape, **common)
                route = [("router_logits", lambda: ctx.moe_router_logits(logits, x, r_w, r_s, r_b, 8, d_model, E1, tokens)),
                         ("router_topk", lambda: ctx.moe_router_topk(ids, score, logits, E, slots, True, True, tokens))]
                seven = route + [("gate", lambda: ctx.matmul(dg)), ("up", lambda: ctx.matmul(du)),
                                 ("silu_mul", lambda: ctx.silu_mul(hbuf, gu, tokens * S, ffn)),
                                 ("down", lambda: ctx.matmul(dd)),
                                 ("combine", lambda: ctx.moe_combine(y, dn, score, tokens, d_model, S))]
                five = route + [("gate_up_silu", lambda: ctx.ffn_gated(dgated, full_w["up"][0], full_w["up"][1], full_w["up"][2])),
                                ("down", lambda: ctx.matmul(dd2)),
                                ("combine", lambda: ctx.moe_combine(y2, dn2, score, tokens, d_model, S))]
                return seven, five

            blocks = [block(x) for x in xbank]
            touched = set()
            for k, (seven, five) in enumerate(blocks):
                for _, fn in seven:
                    fn()
                got_ids = ctx.download(ids, tokens * S * 4, np.uint32).reshape(tokens, S)
                touched.update(int(v) for v in got_ids.reshape(-1))
                if k == 0:
                    # routing checked against the oracle before anything is timed, and the five-dispatch form against the seven
                    lg = ctx.download(logits, tokens * E1 * 4, np.float32).reshape(tokens, E1)
                    ref_ids, _ = oracle.router_topk(lg, tokens, E, slots, True, True)
                    yy = ctx.download(y, tokens * d_model * 2, np.float16)
                    if not np.array_equal(got_ids, ref_ids) or not np.all(np.isfinite(yy)):
                        raise SystemExit("bench: routed FFN check failed (tokens=%d)" % tokens)
                    for _, fn in five:
                        fn()
                    y_f = ctx.download(y2, tokens * d_model * 2, np.float16).astype(np.float64)
                    y_u = yy.astype(np.float64)
                    if (not np.array_equal(ctx.download(ids, tokens * S * 4, np.uint32).reshape(tokens, S), ref_ids)
                            or float(np.max(np.abs(y_f - y_u)) / (np.max(np.abs(y_u)) + 1e-2)) > 1e-2):  # outputs cross zero: scale by the largest
                        raise SystemExit("bench: fused routed FFN disagrees with the seven-dispatch form (tokens=%d)" % tokens)
            rot_mb = round(len(touched) * per_expert / 1e6, 1)
            for which, key in ((0, "moe_ffn_routed_tokens%d"), (1, "moe_ffn_routed_fused_tokens%d")):
                lists = [b_[which] for b_ in blocks]
                nrep = 2 * NX
                ms = timed_graph(ctx, [fn for r in range(nrep) for _, fn in lists[r % NX]], reps=3) / nrep
                row = {"us": round(ms * 1e3, 2), "dispatches": len(lists[0]), "slots": S, "rotation_MB": rot_mb}
                for i_op, (name, _) in enumerate(lists[0]):
                    # a dispatch alone, rotating over the same activations (the ids the router left last are the last set's:
                    # the expert dispatches alone re-read one set of experts, so their solo times are lower bounds)
                    row[name + "_us"] = round(timed_graph(ctx, [lists[r % NX][i_op][1] for r in range(2 * NX)]) / (2 * NX) * 1e3, 2)
                extra[key % tokens] = row
        # elementwise / load-time kernels at their large shapes: HBM-bound, bytes moved per second
        rows_, f_ = 512, 14336
        nsl = n_sets(rows_ * f_ * 6)
        gus, hos = [ctx.alloc(rows_ * 2 * f_ * 2) for _ in range(nsl)], [ctx.alloc(rows_ * f_ * 2) for _ in range(nsl)]
        for g_ in gus:
            ctx.fill(g_, 0x3C, rows_ * 2 * f_ * 2)
        ms = timed_graph(ctx, [lambda j=j: ctx.silu_mul(hos[j % nsl], gus[j % nsl], rows_, f_) for j in range(3 * nsl)], reps=3) / (3 * nsl)
        extra["silu_mul_rows512_ffn14336"] = {"us": round(ms * 1e3, 2), "GB/s": round(rows_ * f_ * 6 / ms / 1e6, 1),
                                              "rotation_MB": round(nsl * rows_ * f_ * 6 / 1e6, 1)}
        nb = 256 << 20
        src_, dst_ = ctx.alloc(nb), ctx.alloc(nb)
        ctx.fill(src_, 0x3C, nb)
        ms = timed_graph(ctx, [lambda: ctx.repack_part(dst_, src_, nb, capi.CONVERT_BF16_F16, 0)] * 6) / 6
        extra["repack_bf16_to_f16_256MiB"] = {"us": round(ms * 1e3, 1), "GB/s": round(2 * nb / ms / 1e6, 1), "rotation_MB": round(2 * nb / 1e6, 1)}
        result["extra"] = extra

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(oracle, synth)

    ctx.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
