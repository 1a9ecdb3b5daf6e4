'use strict'
// Runs one dense decode GEMV and one MoE gate dispatch through uniformBuf / bg / dispatch on the GPU.
// Inputs come from <dir>/*.bin (written by the pytest driver); outputs go to <dir>/y_dense.bin, y_moe.bin.
const fs = require('fs')
const path = require('path')
const z = require(path.join(__dirname, '..', '..', 'zero-tvm_amd', 'js'))
const dir = process.argv[2]
const meta = JSON.parse(fs.readFileSync(path.join(dir, 'meta.json'), 'utf8'))
const load = (n) => fs.readFileSync(path.join(dir, n))
const dev = new z.Device(0)
const put = (name) => { const b = load(name); const buf = dev.createBuffer(b.length, name); dev.writeBuffer(buf, 0, b); return buf }

{
  const { K, N } = meta.dense
  const pipe = dev.createPipeline('int4_matmul_tiled_vec4h_affine')
  const out = dev.createBuffer(N * 2, 'out')
  const group = dev.bg(pipe, [out, put('x.bin'), put('s.bin'), put('w.bin'), dev.uniformBuf(z.densePod(K, N)), put('b.bin')])
  dev.dispatch(pipe, group, N / 4)
  fs.writeFileSync(path.join(dir, 'y_dense.bin'), Buffer.from(dev.readBuffer(out)))
  let threw = false
  try { dev.bg(pipe, [out, put('x.bin'), put('s.bin'), put('w.bin'), dev.uniformBuf(z.densePod(K, N))]) } catch (e) { threw = /binding 5/.test(e.message) }
  if (!threw) throw new Error('affine pipeline without bias did not throw')
}
{
  // boot-time GEMM probe on the dense weights: families timed with the family forced, pick stored and replayed
  const { K, N } = meta.dense
  const CAP = 256
  const pipe = dev.createPipeline('int4_matmul_batched_dyn_affine')
  const act = dev.createBuffer(CAP * K * 2, 'chunk'), out = dev.createBuffer(CAP * N * 2, 'chunk_out')
  dev.fill(act, 0)
  const group = dev.bg(pipe, [out, act, put('s.bin'), put('w.bin'), dev.uniformBuf(z.densePod(K, N, 4, true, CAP)), put('b.bin')])
  const desc = dev.descriptor(group)
  // the entry point that allocates nothing gives the same bytes as the ordinary one (M = 24 rows: scratch in use)
  {
    const d24 = Object.assign({}, desc, { M: 24 })
    dev.fill(out, 0)
    dev.matmul(d24)
    const a = Buffer.from(dev.readBuffer(out, 0, 24 * N * 2))
    dev.fill(out, 0)
    dev.matmulStatic(d24)
    const b = Buffer.from(dev.readBuffer(out, 0, 24 * N * 2))
    if (!a.equals(b)) throw new Error('matmulStatic differs from matmul')
    const sink = dev.createBuffer(64, 'sink')
    dev.readProbe(act, CAP * K * 2, sink)
    dev.sync()
  }
  const timings = dev.probeFamilies(desc, ['gemm', 'skinny', 'rows', 'gemv'], [64, 256], { warmup: 1, rounds: 2 })
  const store = z.fileTuneStore(path.join(dir, 'tune_store.json'))
  const adapter = z.deviceFingerprint(dev.info())
  let probes = 0
  const runProbe = () => { probes++; return dev.probeFamilies(desc, ['gemm', 'skinny', 'gemv'], [64, 256], { warmup: 1, rounds: 2 }) }
  const first = z.resolveTunedGemm({ specId: 'js-dense', runnable: ['gemm', 'skinny', 'gemv'], store, adapterId: adapter, runProbe })
  const second = z.resolveTunedGemm({ specId: 'js-dense', runnable: ['gemm', 'skinny', 'gemv'], store, adapterId: adapter, runProbe })
  fs.writeFileSync(path.join(dir, 'tune.json'), JSON.stringify({ timed: Object.keys(timings).sort(), first, second, probes, adapter,
    sizes: Object.keys(timings.gemm || {}).map(Number) }))
}
{
  const { E, slots, tokens, d, ffn } = meta.moe
  const pipe = dev.createPipeline('int4_matmul_tiled_affine_moe')
  const out = dev.createBuffer(tokens * slots * 2 * ffn * 2, 'gu')
  dev.fill(out, 0)
  const pods = z.moePods(d, ffn, slots)
  const group = dev.bg(pipe, [out, put('mx.bin'), put('ms.bin'), put('mw.bin'), dev.uniformBuf(pods.gate), put('mb.bin'), put('ids.bin')])
  dev.beginEncoder()
  dev.dispatch(pipe, group, ffn / 4, tokens, slots)
  const cb = dev.finishEncoder()
  dev.submit(cb)
  fs.writeFileSync(path.join(dir, 'y_moe.bin'), Buffer.from(dev.readBuffer(out)))
  if (E <= 0) throw new Error('meta')
}
{
  // the dispatches around the matmuls: router logits -> top-k, silu_mul, combine, gate + up + SiLU in one pass
  const { D, E, K, rowsS, F, N2, S, GK, GF } = meta.block
  const logits = dev.createBuffer((E + 1) * 4, 'logits'), idx = dev.createBuffer((K + 1) * 4, 'idx'), sc = dev.createBuffer((K + 1) * 4, 'score')
  dev.moeRouterLogits(logits, put('rx.bin'), put('rw.bin'), put('rs.bin'), put('rb.bin'), 8, D, E + 1, 1)
  dev.moeRouterTopk(idx, sc, logits, E, K, true, true, 1)
  fs.writeFileSync(path.join(dir, 'r_logits.bin'), Buffer.from(dev.readBuffer(logits)))
  fs.writeFileSync(path.join(dir, 'r_idx.bin'), Buffer.from(dev.readBuffer(idx)))
  fs.writeFileSync(path.join(dir, 'r_score.bin'), Buffer.from(dev.readBuffer(sc)))
  const h = dev.createBuffer(rowsS * F * 2, 'h')
  dev.siluMul(h, put('gu.bin'), rowsS, F)
  fs.writeFileSync(path.join(dir, 'h.bin'), Buffer.from(dev.readBuffer(h)))
  const y = dev.createBuffer(N2 * 2, 'y')
  dev.moeCombine(y, put('slots.bin'), put('cscore.bin'), 1, N2, S)
  fs.writeFileSync(path.join(dir, 'comb.bin'), Buffer.from(dev.readBuffer(y)))
  // the reference's fused FFN layout: one [2*GF, GK] buffer, gate rows then up rows
  const pipe = dev.createPipeline('int4_matmul_tiled_affine')
  const gw = put('gw.bin'), gs = put('gs.bin'), gb = put('gb.bin'), go = dev.createBuffer(GF * 2, 'gated')
  const group = dev.bg(pipe, [go, put('gx.bin'), gs, gw, dev.uniformBuf(z.densePod(GK, GF)), gb])
  const kp = GK / 8, spr = GK / 64
  dev.ffnGated(pipe, group, { buffer: gw, offset: GF * kp * 4, size: GF * kp * 4 }, { buffer: gs, offset: GF * spr * 2, size: GF * spr * 2 },
    { buffer: gb, offset: GF * spr * 2, size: GF * spr * 2 }, GF / 4)
  fs.writeFileSync(path.join(dir, 'gated.bin'), Buffer.from(dev.readBuffer(go)))
  // the same dispatch with the add + RMSNorm prologue: binding 1 is the residual
  const go2 = dev.createBuffer(GF * 2, 'gated_prologue')
  const group2 = dev.bg(pipe, [go2, put('pres.bin'), gs, gw, dev.uniformBuf(z.densePod(GK, GF)), gb])
  dev.ffnGatedPrologue(pipe, group2, { buffer: gw, offset: GF * kp * 4, size: GF * kp * 4 }, { buffer: gs, offset: GF * spr * 2, size: GF * spr * 2 },
    { buffer: gb, offset: GF * spr * 2, size: GF * spr * 2 }, put('pdelta.bin'), put('pgamma.bin'), 1e-5, GF / 4)
  fs.writeFileSync(path.join(dir, 'gated_prologue.bin'), Buffer.from(dev.readBuffer(go2)))
  let threw = false
  try { dev.moeRouterTopk(idx, sc, logits, E, E + 1, true, true, 1) } catch (e) { threw = /K must be/.test(e.message) }
  if (!threw) throw new Error('top-k with K > E did not throw')
}
{
  // fused QKV: the paged form, then the int8-KV pair (scratch rows + quantizer)
  const { heads, kvHeads, headDim, d, pageSize, pages } = meta.qkv
  const hps = pageSize * headDim, vpo = kvHeads * hps, kps = 2 * kvHeads * hps
  const model = { d, affine: false, heads, kvHeads, headDim, pageSize, kvPageStride: kps, headPageStride: hps, vPageOffset: vpo, ropeTheta: 10000.0 }
  const hidden = put('qx.bin'), scales = put('qs.bin'), weights = put('qw.bin'), pos = put('qpos.bin')
  const q1 = dev.createBuffer(heads * headDim * 2, 'q'), kv = dev.createBuffer(pages * kps * 2, 'kv')
  dev.fill(kv, 0)
  dev.qkvFused([q1, kv, hidden, scales, weights, pos], dev.uniformBuf([0, 0]), model)
  fs.writeFileSync(path.join(dir, 'q_paged.bin'), Buffer.from(dev.readBuffer(q1)))
  fs.writeFileSync(path.join(dir, 'kv_paged.bin'), Buffer.from(dev.readBuffer(kv)))
  const q2 = dev.createBuffer(heads * headDim * 2, 'q2'), ks = dev.createBuffer(kvHeads * headDim * 2, 'k_slot'), vs = dev.createBuffer(kvHeads * headDim * 2, 'v_slot')
  dev.qkvFusedScratch([q2, ks, vs, hidden, scales, weights, pos], dev.uniformBuf([0, (heads + 2 * kvHeads) * headDim / 2]), model)
  fs.writeFileSync(path.join(dir, 'q_scratch.bin'), Buffer.from(dev.readBuffer(q2)))
  fs.writeFileSync(path.join(dir, 'k_slot.bin'), Buffer.from(dev.readBuffer(ks)))
  fs.writeFileSync(path.join(dir, 'v_slot.bin'), Buffer.from(dev.readBuffer(vs)))
  const rowWords = headDim / 4
  const i8 = dev.createBuffer(pages * kvHeads * pageSize * 2 * rowWords * 4, 'kv_i8'), sc = dev.createBuffer(pages * kvHeads * pageSize * 2 * 2, 'kv_scales')
  dev.fill(i8, 0); dev.fill(sc, 0)
  dev.kvQuantizeInt8([ks, vs, i8, sc, pos], dev.uniformBuf([0, 0, 0, kvHeads * 2]), model)
  fs.writeFileSync(path.join(dir, 'kv_i8.bin'), Buffer.from(dev.readBuffer(i8)))
  fs.writeFileSync(path.join(dir, 'kv_sc.bin'), Buffer.from(dev.readBuffer(sc)))
}
dev.close()
console.log('js gpu dispatch ok')
