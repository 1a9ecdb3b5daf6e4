'use strict'
// Which prefill GEMM runs the chunk dispatches, decided once at start-up by timing the candidates on the device
// and remembered per (device, model). This replaces the role of src/zero-tvm/gemm-tune.ts in the reference and keeps
// its exported names so callers switch over unchanged; the rules, stated once:
//
//   score      a candidate's score is the geometric mean, over the probe sizes, of the median of its samples at
//              each size; the lowest score wins and an exact tie goes to whichever stands earlier in the ladder
//   memory     a remembered choice is a JSON record {version, pick, ms, candidates, at}; it is honoured only while
//              its version is current, it is younger than TUNE_TTL_MS, its pick can still run, and every candidate
//              that can run today was part of the measurement that produced it
//   priority   an explicit request is never overridden; with fewer than two candidates there is nothing to decide;
//              whatever goes wrong (store, clock, probe) the answer is "no opinion" (null) and the static
//              thresholds of ztvm_matmul decide
//
// Candidates are names: the reference's pipelines ('e5', 'sgmat', 'tiled', 'matvec') or this library's kernel
// families ('gemm', 'skinny', 'rows', 'gemv'), which probeFamilies times with the family forced in the descriptor.

const TUNE_VERSION = 2            // raise when a kernel family changes speed: older records stop counting
const TUNE_TTL_MS = 2592000000    // 30 days
const TUNE_MS = [64, 256, 1024]   // chunk rows probed: a ragged head, a middle, a full chunk
const TUNE_WARMUP = 2
const TUNE_ROUNDS = 4
const REFERENCE_LADDER = ['e5', 'sgmat', 'tiled', 'matvec']
const FAMILY_LADDER = ['gemm', 'skinny', 'rows', 'gemv']
const FAMILY_KERNEL = { gemv: 1, skinny: 2, gemm: 3, rows: 4 } // ZTVM_KERNEL_* of include/ztvm.h

const tuneKey = (adapterId, specId) => ['ztvm.gemmTune', 'v' + TUNE_VERSION, adapterId, specId].join('.')

/** A stable id for the device out of Device.info(); null when the device will not say who it is. */
function deviceFingerprint(info) {
  if (!info || typeof info !== 'object' || !info.name) return null
  const field = (v) => (v === undefined || v === null ? '?' : String(v))
  return [info.name, info.computeUnits, info.hbmBytes].map(field).join('/').replace(/[^\w./-]/g, '_')
}

function median(samples) {
  const sorted = Array.from(samples).sort((p, q) => p - q)
  const upper = sorted[Math.floor(sorted.length / 2)]
  return sorted.length & 1 ? upper : 0.5 * (sorted[sorted.length / 2 - 1] + upper)
}

/** Scores of the candidates that were measured: name -> geometric mean of its per-size medians. */
class Scoreboard {
  constructor() { this.perSize = new Map() }
  /** medians: one number per probe size */
  add(name, medians) {
    const usable = (medians || []).filter((v) => Number.isFinite(v))
    if (usable.length) this.perSize.set(name, usable)
    return this
  }
  get size() { return this.perSize.size }
  score(name) {
    const m = this.perSize.get(name)
    if (!m) return null
    let logSum = 0
    for (const v of m) logSum += Math.log(v > 1e-9 ? v : 1e-9)
    return Math.exp(logSum / m.length)
  }
  /** The measured ladder entry with the lowest score, earlier entries first among equals; the ladder's
   *  last entry when none of them was measured. */
  winner(ladder) {
    const ranked = ladder.map((name, rank) => ({ name, rank, score: this.score(name) })).filter((c) => c.score !== null)
    if (!ranked.length) return ladder[ladder.length - 1]
    ranked.sort((p, q) => p.score - q.score || p.rank - q.rank)
    return ranked[0].name
  }
  summary() {
    const out = {}
    for (const [name, m] of this.perSize) out[name] = median(m)
    return out
  }
}

function pickFromTimings(medians, ladder) {
  const board = new Scoreboard()
  for (const name of Object.keys(medians)) board.add(name, medians[name])
  return board.winner(ladder)
}

/** The remembered choice and the test of whether it still applies. */
class TuneRecord {
  constructor(pick, ms, candidates, at) { Object.assign(this, { version: TUNE_VERSION, pick, ms, candidates, at }) }
  static parse(text) {
    if (typeof text !== 'string' || !text) return null
    let obj
    try { obj = JSON.parse(text) } catch (err) { return null }
    if (obj === null || typeof obj !== 'object') return null
    const rec = new TuneRecord(obj.pick, obj.ms, obj.candidates, obj.at)
    rec.version = obj.version
    return rec
  }
  appliesTo(runnable, now) {
    const fresh = typeof this.at === 'number' && now - this.at <= TUNE_TTL_MS
    const covered = Array.isArray(this.candidates) && runnable.every((name) => this.candidates.indexOf(name) >= 0)
    return this.version === TUNE_VERSION && fresh && covered && runnable.indexOf(this.pick) >= 0
  }
}

function loadTunedPick(store, key, runnable, now) {
  if (!store || !runnable.length) return null
  let text
  try { text = store.load(key) } catch (err) { return null }
  const rec = TuneRecord.parse(text)
  return rec && rec.appliesTo(runnable, now === undefined ? Date.now() : now) ? rec.pick : null
}

function saveTunedPick(store, key, pick, ms, candidates) {
  if (!store) return
  try { store.save(key, JSON.stringify(new TuneRecord(pick, ms, candidates, Date.now()))) } catch (err) { /* the choice still stands for this run */ }
}

/** key -> string stores: in memory, or one JSON file standing where the browser has localStorage. */
function memoryTuneStore(init) {
  const cells = Object.assign(Object.create(null), init || {})
  return { load: (key) => (key in cells ? cells[key] : null), save: (key, value) => { cells[key] = value } }
}

function fileTuneStore(file) {
  const fs = require('fs')
  const slurp = () => {
    let parsed = null
    try { parsed = JSON.parse(fs.readFileSync(file, 'utf8')) } catch (err) { /* absent or unreadable: empty */ }
    return parsed && typeof parsed === 'object' && !Array.isArray(parsed) ? parsed : {}
  }
  return {
    load(key) { const all = slurp(); return Object.prototype.hasOwnProperty.call(all, key) ? all[key] : null },
    save(key, value) {
      const all = slurp()
      all[key] = value
      const tmp = file + '.tmp'
      fs.writeFileSync(tmp, JSON.stringify(all))
      fs.renameSync(tmp, file) // readers see the old file or the new one, never half of one
    },
  }
}

/** Wall-clock samples of runs[name](m), each run to completion (sync() returns when the queue is empty). Within a
 *  round every candidate runs once before any runs twice, so drift of the clocks hits all of them alike. A throw
 *  anywhere ends the probe; the samples taken so far are returned. Result: {name: {m: [ms, ...]}}. */
function timeClosures(sync, runs, Ms, opts) {
  const cfg = opts || {}
  const warmup = cfg.warmup === undefined ? TUNE_WARMUP : cfg.warmup
  const rounds = cfg.rounds === undefined ? TUNE_ROUNDS : cfg.rounds
  const clock = cfg.clock || (() => Number(process.hrtime.bigint()) / 1e6)
  const order = Object.keys(runs)
  const samples = {}
  const note = (name, m, ms) => {
    const bySize = samples[name] || (samples[name] = {})
    ;(bySize[m] || (bySize[m] = [])).push(ms)
  }
  try {
    for (const m of Ms) {
      for (let i = 0; i < warmup; i++) order.forEach((name) => runs[name](m))
      sync()
      for (let round = 0; round < rounds; round++) {
        for (const name of order) {
          const start = clock()
          runs[name](m)
          sync()
          note(name, m, clock() - start)
        }
      }
    }
  } catch (err) { /* a partial probe is still a probe */ }
  return samples
}

/** {pick, source} with source 'explicit' | 'stored' | 'probed', or null for "no opinion". */
function resolveTunedGemm(opts) {
  if (opts.explicit) return { pick: opts.explicit, source: 'explicit' }
  const runnable = opts.runnable
  if (!runnable || runnable.length < 2) return null
  const store = opts.store || null
  const key = opts.adapterId ? tuneKey(opts.adapterId, opts.specId) : null // an anonymous device is tuned but not remembered
  const remembered = key ? loadTunedPick(store, key, runnable) : null
  if (remembered) return { pick: remembered, source: 'stored' }

  let samples = null
  try { samples = opts.runProbe() } catch (err) { samples = null }
  const board = new Scoreboard()
  for (const name of runnable) {
    const bySize = samples && samples[name]
    if (bySize) board.add(name, Object.keys(bySize).map((m) => bySize[m]).filter((s) => s && s.length).map(median))
  }
  if (!board.size) return null
  const preference = (opts.order || REFERENCE_LADDER.concat(FAMILY_LADDER)).filter((name) => runnable.indexOf(name) >= 0)
  const pick = board.winner(preference.length ? preference : runnable)
  if (key) saveTunedPick(store, key, pick, board.summary(), runnable)
  return { pick, source: 'probed' }
}

/** Samples for this library's kernel families on one dense GEMM: `desc` names the caller's real weights and an
 *  activation buffer of at least max(Ms) rows; api = {validate, matmul, sync} of the addon. A family that refuses
 *  the descriptor at any probe size is not a candidate. */
function probeFamilies(api, desc, families, Ms, opts) {
  const sizes = Ms || TUNE_MS
  const forced = (name, m) => Object.assign({}, desc, { kernel: FAMILY_KERNEL[name], M: m })
  const runs = {}
  for (const name of families) {
    if (sizes.every((m) => api.validate(forced(name, m)).code === 0)) runs[name] = (m) => api.matmul(forced(name, m))
  }
  return timeClosures(api.sync, runs, sizes, opts)
}

module.exports = {
  TUNE_VERSION, TUNE_TTL_MS, TUNE_MS, TUNE_WARMUP, TUNE_ROUNDS, REFERENCE_LADDER, FAMILY_LADDER,
  tuneKey, deviceFingerprint, median, pickFromTimings, loadTunedPick, saveTunedPick, memoryTuneStore, fileTuneStore,
  timeClosures, resolveTunedGemm, probeFamilies, Scoreboard, TuneRecord,
}
