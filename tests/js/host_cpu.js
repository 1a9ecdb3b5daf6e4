'use strict'
// Decision logic of the JavaScript host layer, no GPU: the same truth tables the Python mirror is held to
// (reference: tests/unit/resolve-matmul-affine.test.ts, chunk-gemm-pick.test.ts, chunk-grid-limits.test.ts).
const assert = require('assert')
const path = require('path')
const z = require(path.join(__dirname, '..', '..', 'zero-tvm_amd', 'js'))

assert.strictEqual(z.abiVersion(), 2)
const names = z.INT4_MATMUL_VARIANTS.map(z.int4MatmulEntry)
assert.strictEqual(names.length, 34)
assert.strictEqual(new Set(names).size, 34)
for (const o of z.INT4_MATMUL_VARIANTS) z.checkOpts(o)
assert.throws(() => z.checkOpts({ moe: true }), /moe requires affine/)
assert.throws(() => z.checkOpts({ q3: true }), /q3 requires affine/)
assert.throws(() => z.checkOpts({ rowsPerWG: 4 }), /requires subgroups/)
assert.throws(() => z.createPipeline('int4_matmul_nonsense'), /unknown/)
const p = z.createPipeline('int4_matmul_tiled_affine_q3_moe')
assert.ok(p.affine && p.moe && p.bits === 3)
assert.strictEqual(z.createPipeline('int4_matmul_sg_e5_affine').kernel, z.KERNEL.GEMM)

const A = new Set(z.ALL_ENTRIES)
assert.strictEqual(z.resolveMatmul('tiled', A, true, 2048, null, true, true).pipeline, 'int4_matmul_tiled_vec4h_affine')
assert.strictEqual(z.resolveMatmul('tiled', A, false, 2048, null, true, false).pipeline, 'int4_matmul_tiled_affine')
assert.strictEqual(z.resolveMatmul('scalar', A, true, 2048, null, true, true).label, 'scalar_affine')
assert.strictEqual(z.resolveMatmul('tiled', A, true, 2560).pipeline, 'int4_matmul_tiled_vec4h')
assert.strictEqual(z.resolveMatmul('tiled', A, true, 4096).pipelineF32, 'int4_matmul_f32_tiled_vec4')
assert.strictEqual(z.resolveMatmul('scalar', A, true, 3072).label, 'scalar')

const FULL = { chunkTiled: false, dimsOK: true, capTiles64: true, e5Ready: true, sgmatReady: true, cap: 1024 }
assert.strictEqual(z.pickChunkGemm(FULL).used, 'e5')
assert.strictEqual(z.pickChunkGemm(Object.assign({}, FULL, { e5Ready: false })).used, 'sgmat')
let pick = z.pickChunkGemm(Object.assign({}, FULL, { want: 'e5', capTiles64: false, cap: 96 }))
assert.ok(pick.used === 'sgmat' && /cap must be %64 \(got 96\)/.test(pick.rejected))
pick = z.pickChunkGemm(Object.assign({}, FULL, { want: 'matvec', chunkTiled: true }))
assert.ok(pick.used === 'tiled' && /asked for 'matvec', can only run 'tiled'/.test(pick.rejected))
assert.deepStrictEqual(z.foldGridX(69632), { x: 16384, z: 5 })
assert.strictEqual(z.resolveChunkCap({}, { maxChunkCap: 256 }, true), 256)
assert.deepStrictEqual(z.moePods(2048, 512, 8).down, [64, 8, 2048, 512, 2048, 4096, 16384, 8])

// boot-time GEMM choice: the behaviours the reference pins in tests/unit/gemm-tune.test.ts
{
  const saved = (over) => JSON.stringify(Object.assign({ version: z.TUNE_VERSION, pick: 'e5', ms: { e5: 1 },
    candidates: ['e5', 'sgmat', 'matvec'], at: Date.now() }, over || {}))
  const runnable = ['e5', 'sgmat', 'matvec']
  assert.strictEqual(z.median([3, 1, 2]), 2)
  assert.strictEqual(z.median([4, 1, 3, 2]), 2.5)
  assert.strictEqual(z.pickFromTimings({ e5: [1, 1, 16], sgmat: [2, 2, 2] }, runnable), 'sgmat') // geomean 2.52 against 2
  const tie = { e5: [2, 2], sgmat: [2, 2], matvec: [2, 2] }
  assert.strictEqual(z.pickFromTimings(tie, runnable), 'e5')
  assert.strictEqual(z.pickFromTimings(tie, ['sgmat', 'matvec']), 'sgmat')
  assert.strictEqual(z.pickFromTimings({ matvec: [5] }, runnable), 'matvec')
  assert.strictEqual(z.tuneKey('apple/m4', 'llama32'), 'ztvm.gemmTune.v' + z.TUNE_VERSION + '.apple/m4.llama32')
  assert.strictEqual(z.deviceFingerprint({ name: 'AMD Instinct MI355X', computeUnits: 256, hbmBytes: 309220868096n }),
    'AMD_Instinct_MI355X/256/309220868096')
  assert.strictEqual(z.deviceFingerprint({}), null)
  assert.strictEqual(z.loadTunedPick(z.memoryTuneStore({ k: saved() }), 'k', runnable), 'e5')
  for (const over of [{ version: z.TUNE_VERSION + 1 }, { at: Date.now() - z.TUNE_TTL_MS - 1 }, { pick: 'tiled' },
    { candidates: ['matvec'] }, { at: 'yesterday' }]) {
    assert.strictEqual(z.loadTunedPick(z.memoryTuneStore({ k: saved(over) }), 'k', runnable), null)
  }
  assert.strictEqual(z.loadTunedPick(z.memoryTuneStore(), 'k', runnable), null)
  assert.strictEqual(z.loadTunedPick(null, 'k', runnable), null)
  assert.strictEqual(z.loadTunedPick(z.memoryTuneStore({ k: 'not json' }), 'k', runnable), null)
  const bad = { load: () => { throw new Error('x') }, save: () => { throw new Error('x') } }
  assert.strictEqual(z.loadTunedPick(bad, 'k', runnable), null)
  z.saveTunedPick(bad, 'k', 'e5', {}, ['e5']) // must not throw
  let probed = 0
  assert.deepStrictEqual(z.resolveTunedGemm({ specId: 'llama32', runnable, explicit: 'matvec', store: z.memoryTuneStore(),
    adapterId: 'd', runProbe: () => { probed++; return {} } }), { pick: 'matvec', source: 'explicit' })
  assert.strictEqual(z.resolveTunedGemm({ specId: 'llama32', runnable: ['matvec'], runProbe: () => { probed++; return {} } }), null)
  assert.strictEqual(probed, 0)
  const store = z.memoryTuneStore()
  const probe = () => ({ e5: { 64: [1, 1.1], 256: [2, 2.2] }, sgmat: { 64: [3, 3], 256: [4, 4] } })
  assert.deepStrictEqual(z.resolveTunedGemm({ specId: 'llama32', runnable: ['e5', 'sgmat'], store, adapterId: 'd', runProbe: probe }),
    { pick: 'e5', source: 'probed' })
  assert.deepStrictEqual(z.resolveTunedGemm({ specId: 'llama32', runnable: ['e5', 'sgmat'], store, adapterId: 'd',
    runProbe: () => ({ sgmat: { 64: [0.1] } }) }), { pick: 'e5', source: 'stored' })
  assert.strictEqual(z.resolveTunedGemm({ specId: 'llama32', runnable: ['e5', 'sgmat'], store: z.memoryTuneStore(), adapterId: 'd',
    runProbe: () => { throw new Error('gpu busy') } }), null)
  assert.strictEqual(z.resolveTunedGemm({ specId: 'm', runnable: ['skinny', 'gemm'],
    runProbe: () => ({ skinny: { 64: [2] }, gemm: { 64: [2] } }) }).pick, 'gemm')
  let t = 0
  const calls = []
  const run = (name, cost) => (m) => { calls.push(name + m); t += cost * m }
  assert.deepStrictEqual(z.timeClosures(() => {}, { a: run('a', 0.125), b: run('b', 0.25) }, [4, 8], { warmup: 1, rounds: 2, clock: () => t }),
    { a: { 4: [0.5, 0.5], 8: [1, 1] }, b: { 4: [1, 1], 8: [2, 2] } })
  assert.deepStrictEqual(calls.slice(0, 6), ['a4', 'b4', 'a4', 'b4', 'a4', 'b4'])
}

// descriptor validation through the addon, no device needed
const good = { bits: 4, affine: 1, M: 1, N: 64, k_packed: 512, scales_per_row: 64, out: 4096n, in: 8192n, scales: 12288n, weights: 16384n, biases: 20480n }
assert.strictEqual(z.validate(good).code, 0)
assert.ok(/binding 5/.test(z.validate(Object.assign({}, good, { biases: 0n })).why))
assert.ok(/SCALES_PER_ROW/.test(z.validate(Object.assign({}, good, { scales_per_row: 63 })).why))
// above 128 rows: the tile GEMM where its tiles fill the CUs, the skinny family where they would not
assert.strictEqual(z.resolve(Object.assign({}, good, { M: 512, N: 14336 })), z.KERNEL.GEMM)
assert.strictEqual(z.resolve(Object.assign({}, good, { M: 512, N: 4096 })), z.KERNEL.SKINNY)
console.log('js host cpu checks ok')
