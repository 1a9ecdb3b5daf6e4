'use strict'
// Boot-time choice of the prefill ("chunk") GEMM by measurement, remembered per device and model: the policy of
// the reference's src/zero-tvm/gemm-tune.ts (tuneKey :52-54, deviceFingerprint :61-78, median :81-85,
// pickFromTimings :90-105, loadTunedPick :110-129, saveTunedPick :131-145, timeClosures :162-189,
// resolveTunedGemm :208-233). Candidates are plain names: the reference's pipelines ('e5', 'sgmat', 'tiled',
// 'matvec') or this library's kernel families ('gemm', 'skinny', 'rows', 'gemv'), which probeFamilies times
// through Device.dispatch with the family forced. Without a pick ztvm_matmul routes by its own row thresholds.

const TUNE_VERSION = 1 // bump when a GEMM kernel changes shape or speed: stored picks go stale
const TUNE_TTL_MS = 30 * 24 * 3600 * 1000 // drivers move performance too: re-tune monthly
const TUNE_MS = [64, 256, 1024] // probe sizes (chunk rows): ragged head, middle, full cap
const TUNE_WARMUP = 2
const TUNE_ROUNDS = 4
const REFERENCE_LADDER = ['e5', 'sgmat', 'tiled', 'matvec']
const FAMILY_LADDER = ['gemm', 'skinny', 'rows', 'gemv']

function tuneKey(adapterId, specId) { return 'ztvm.gemmTune.v' + TUNE_VERSION + '.' + adapterId + '.' + specId }

// Identity of the device for the key, from Device.info(): name / compute units / memory; null when nothing
// identifies it (the caller then tunes without persisting).
function deviceFingerprint(info) {
  try {
    if (info && info.name) {
      const cu = info.computeUnits === undefined ? '?' : String(info.computeUnits)
      const mem = info.hbmBytes === undefined ? '?' : String(info.hbmBytes)
      return [String(info.name), cu, mem].join('/').replace(/[^\w./-]/g, '_')
    }
  } catch (e) { /* a fingerprint must never break boot */ }
  return null
}

function median(xs) {
  const s = xs.slice().sort((a, b) => a - b)
  const m = s.length >> 1
  return s.length % 2 ? s[m] : (s[m - 1] + s[m]) / 2
}

// Lowest geometric mean (across sizes) of the per-size medians; strictly-less keeps the earlier ladder entry on
// exact ties; candidates without timings are ignored; nothing timed -> the ladder's last entry.
function pickFromTimings(medians, ladder) {
  let best = ladder[ladder.length - 1]
  let bestScore = Infinity
  for (const name of ladder) {
    const ms = medians[name]
    if (!ms || !ms.length) continue
    const geo = Math.exp(ms.reduce((a, m) => a + Math.log(Math.max(m, 1e-9)), 0) / ms.length)
    if (geo < bestScore) { bestScore = geo; best = name }
  }
  return best
}

// A stored pick counts only if it is current-version, fresh, still runnable, and was measured against a
// candidate set covering today's runnable ones; anything else (also corrupt data, a throwing store): re-tune.
function loadTunedPick(store, key, runnable, now) {
  if (!store || !runnable.length) return null
  let raw = null
  try { raw = store.load(key) } catch (e) { return null }
  if (!raw) return null
  let saved
  try { saved = JSON.parse(raw) } catch (e) { return null }
  if (!saved || typeof saved !== 'object' || saved.version !== TUNE_VERSION) return null
  const t = now === undefined ? Date.now() : now
  if (typeof saved.at !== 'number' || t - saved.at > TUNE_TTL_MS) return null
  if (!runnable.includes(saved.pick)) return null
  if (!Array.isArray(saved.candidates) || !runnable.every((c) => saved.candidates.includes(c))) return null
  return saved.pick
}

function saveTunedPick(store, key, pick, ms, candidates) {
  if (!store) return
  try {
    store.save(key, JSON.stringify({ version: TUNE_VERSION, pick, ms, candidates, at: Date.now() }))
  } catch (e) { /* persistence must never break boot */ }
}

function memoryTuneStore(init) {
  const m = new Map(Object.entries(init || {}))
  return { load: (k) => (m.has(k) ? m.get(k) : null), save: (k, v) => { m.set(k, v) } }
}

// One JSON file of key -> value (the place of the browser's localStorage).
function fileTuneStore(file) {
  const fs = require('fs')
  const read = () => {
    try {
      const d = JSON.parse(fs.readFileSync(file, 'utf8'))
      return d && typeof d === 'object' && !Array.isArray(d) ? d : {}
    } catch (e) { return {} }
  }
  return {
    load: (k) => { const d = read(); return k in d ? d[k] : null },
    save: (k, v) => { const d = read(); d[k] = v; fs.writeFileSync(file + '.tmp', JSON.stringify(d)); fs.renameSync(file + '.tmp', file) },
  }
}

// Time each candidate's run(m) (one enqueued GEMM dispatch of m rows) to completion (sync() blocks until the
// queue is empty), candidates interleaved within a round. Returns {name: {m: [ms, ...]}}; throws nothing: a
// failure ends the probe and what was measured so far is returned.
function timeClosures(sync, runs, Ms, opts) {
  const o = Object.assign({ warmup: TUNE_WARMUP, rounds: TUNE_ROUNDS, clock: () => Number(process.hrtime.bigint()) / 1e6 }, opts || {})
  const names = Object.keys(runs)
  const out = {}
  try {
    for (const m of Ms) {
      for (let w = 0; w < o.warmup; w++) for (const name of names) runs[name](m)
      sync()
      for (let r = 0; r < o.rounds; r++) {
        for (const name of names) {
          const t0 = o.clock()
          runs[name](m)
          sync()
          const dt = o.clock() - t0
          if (!out[name]) out[name] = {}
          if (!out[name][m]) out[name][m] = []
          out[name][m].push(dt)
        }
      }
    }
  } catch (e) { /* timing is advisory; the ladder is the fallback */ }
  return out
}

// The boot-time decision: {pick, source: 'explicit' | 'stored' | 'probed'} or null when the static ladder should
// decide (one candidate, a stored miss plus a failed or empty probe).
function resolveTunedGemm(opts) {
  if (opts.explicit) return { pick: opts.explicit, source: 'explicit' }
  const runnable = opts.runnable
  if (runnable.length <= 1) return null
  const store = opts.store || null
  const key = opts.adapterId ? tuneKey(opts.adapterId, opts.specId) : null
  if (key) {
    const stored = loadTunedPick(store, key, runnable)
    if (stored) return { pick: stored, source: 'stored' }
  }
  let timings = {}
  try { timings = opts.runProbe() || {} } catch (e) { timings = {} }
  const medians = {}
  for (const name of runnable) {
    const perSize = timings[name]
    if (!perSize) continue
    const arr = Object.values(perSize).filter((v) => v && v.length).map(median).filter((m) => Number.isFinite(m))
    if (arr.length) medians[name] = arr
  }
  if (!Object.keys(medians).length) return null
  const order = opts.order || REFERENCE_LADDER.concat(FAMILY_LADDER)
  const ladder = order.filter((n) => runnable.includes(n))
  const pick = pickFromTimings(medians, ladder.length ? ladder : runnable)
  const ms = {}
  for (const name of Object.keys(medians)) ms[name] = median(medians[name])
  if (key) saveTunedPick(store, key, pick, ms, runnable)
  return { pick, source: 'probed' }
}

// Time this library's kernel families on one dense GEMM (the caller's real gate/up weights behind `desc`, an
// activation buffer of at least max(Ms) rows). validate/matmul: the addon's descriptor calls; a family that cannot
// take the shape is left out.
function probeFamilies(api, desc, families, Ms, opts) {
  const kernels = { gemm: 3, skinny: 2, rows: 4, gemv: 1 }
  const sizes = Ms || TUNE_MS
  const runs = {}
  for (const name of families) {
    const fits = sizes.every((m) => api.validate(Object.assign({}, desc, { kernel: kernels[name], M: m })).code === 0)
    if (fits) runs[name] = (m) => api.matmul(Object.assign({}, desc, { kernel: kernels[name], M: m }))
  }
  return timeClosures(api.sync, runs, sizes, opts)
}

module.exports = {
  TUNE_VERSION, TUNE_TTL_MS, TUNE_MS, TUNE_WARMUP, TUNE_ROUNDS, REFERENCE_LADDER, FAMILY_LADDER,
  tuneKey, deviceFingerprint, median, pickFromTimings, loadTunedPick, saveTunedPick, memoryTuneStore, fileTuneStore,
  timeClosures, resolveTunedGemm, probeFamilies,
}
