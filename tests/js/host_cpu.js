'use strict'
// Decision logic of the JavaScript host layer, no GPU: the same truth tables the Python mirror is held to
// (reference: tests/unit/resolve-matmul-affine.test.ts, chunk-gemm-pick.test.ts, chunk-grid-limits.test.ts).
const assert = require('assert')
const path = require('path')
const z = require(path.join(__dirname, '..', '..', 'zero-tvm_amd', 'js'))

assert.strictEqual(z.abiVersion(), 1)
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

// descriptor validation through the addon, no device needed
const good = { bits: 4, affine: 1, M: 1, N: 64, k_packed: 512, scales_per_row: 64, out: 4096n, in: 8192n, scales: 12288n, weights: 16384n, biases: 20480n }
assert.strictEqual(z.validate(good).code, 0)
assert.ok(/binding 5/.test(z.validate(Object.assign({}, good, { biases: 0n })).why))
assert.ok(/SCALES_PER_ROW/.test(z.validate(Object.assign({}, good, { scales_per_row: 63 })).why))
assert.strictEqual(z.resolve(Object.assign({}, good, { M: 512 })), z.KERNEL.GEMM)
console.log('js host cpu checks ok')
