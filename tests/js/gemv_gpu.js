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
dev.close()
console.log('js gpu dispatch ok')
