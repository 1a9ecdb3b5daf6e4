'use strict'
// JavaScript host layer: the reference engine's kernel-dispatch surface over the HIP library.
//
// Keeps the names, argument orders and error behaviour of (paths relative to the reference's root)
//   uniformBuf / bg / dispatch          src/zero-tvm/engine-core.ts:53-65, :76-92, :2151-2179
//   int4MatmulEntry / INT4_MATMUL_VARIANTS   src/compiler/shaders/int4_matmul.gen.ts:137-152, :701-766
//   resolveMatmul                       src/zero-tvm/variants.ts:239-321
//   pickChunkGemm / resolveChunkCap / foldGridX   src/zero-tvm/engine-core.ts:195-259
// and turns a (pipeline, bind group, grid) triple into one ztvm_matmul descriptor. Plain ES2019 CommonJS
// so it loads on any Node with N-API >= 6; TypeScript callers use index.d.ts.
const path = require('path')
const tune = require('./gemm_tune')

let native = null
function addon() {
  if (native) return native
  try {
    native = require(path.join(__dirname, 'ztvm_napi.node'))
  } catch (e) {
    // no fallback: without the addon there is no matmul path at all
    throw new Error('zero-tvm_amd: the N-API addon is not built (python zero-tvm_amd/js/build_addon.py): ' + e.message)
  }
  return native
}

const KERNEL = { AUTO: 0, GEMV: 1, SKINNY: 2, GEMM: 3, ROWS: 4 }

// ---- variant naming ----------------------------------------------------------------------------

function int4MatmulEntry(opts) {
  const o = Object.assign({ outF32: false, rowsPerWG: 1, subgroups: false, m: 1, vec4: false, vec4Half: false, mDyn: false, affine: false, moe: false, q3: false }, opts || {})
  if (o.mDyn) return o.affine ? 'int4_matmul_batched_dyn_affine' : 'int4_matmul_batched_dyn'
  if (o.m === 4) return 'int4_matmul_batched_m4'
  let name = 'int4_matmul'
  if (o.outF32) name += '_f32'
  if (o.rowsPerWG === 4) name += '_tiled'
  else if (o.rowsPerWG === 8) name += '_tiled8'
  else if (o.subgroups) name += '_sg'
  if (o.vec4) name += '_vec4'
  else if (o.vec4Half) name += '_vec4h'
  if (o.affine) name += '_affine'
  if (o.q3) name += '_q3'
  if (o.moe) name += '_moe'
  return name
}

function checkOpts(opts) {
  const o = Object.assign({ outF32: false, rowsPerWG: 1, subgroups: false, m: 1, vec4: false, vec4Half: false, mDyn: false, affine: false, moe: false, q3: false }, opts || {})
  if (o.moe && !o.affine) throw new Error('moe requires affine (the MoE weights are MLX affine-quantised)')
  if (o.q3 && !o.affine) throw new Error('q3 requires affine (3-bit ships only in the MLX-affine layout)')
  if (o.affine && o.m !== 1) throw new Error('affine is implemented at m=1 (plus the mDyn path); no fixed-M sibling exists')
  if (o.q3 && (o.vec4 || o.vec4Half)) throw new Error('q3 has no wide-load path: its 3-bit bitstream is not word-aligned')
  if (o.moe && o.vec4) throw new Error('moe has no full-vec4 path: that body does not apply the slot/token offsets')
  if (o.rowsPerWG !== 1 && !o.subgroups) throw new Error('rowsPerWG > 1 requires subgroups')
  if (o.m === 4 && (!o.subgroups || o.rowsPerWG !== 4)) throw new Error('m=4 requires subgroups + rowsPerWG=4')
  if (o.vec4 && !o.subgroups) throw new Error('vec4 requires subgroups (32-thread WG keeps K=3072 divisible)')
  if (o.vec4 && o.m !== 1) throw new Error('vec4 not implemented for m=4')
  if (o.vec4Half && (o.vec4 || !o.subgroups || o.m !== 1)) throw new Error('vec4Half requires subgroups + m=1 and is mutually exclusive with vec4')
  if (o.mDyn && (!o.subgroups || o.rowsPerWG !== 4 || o.m !== 1 || o.vec4 || o.vec4Half || o.outF32)) throw new Error('mDyn requires subgroups + rowsPerWG=4 (no vec4/outF32/m=4)')
}

const sg = true
const INT4_MATMUL_VARIANTS = [
  {}, { subgroups: sg }, { subgroups: sg, rowsPerWG: 4 }, { subgroups: sg, rowsPerWG: 8 },
  { outF32: true }, { outF32: true, subgroups: sg }, { outF32: true, subgroups: sg, rowsPerWG: 4 }, { outF32: true, subgroups: sg, rowsPerWG: 8 },
  { subgroups: sg, rowsPerWG: 4, m: 4 }, { subgroups: sg, rowsPerWG: 4, mDyn: true }, { subgroups: sg, rowsPerWG: 4, mDyn: true, affine: true },
  { subgroups: sg, vec4: true }, { subgroups: sg, rowsPerWG: 4, vec4: true }, { outF32: true, subgroups: sg, vec4: true }, { outF32: true, subgroups: sg, rowsPerWG: 4, vec4: true },
  { subgroups: sg, vec4Half: true }, { subgroups: sg, rowsPerWG: 4, vec4Half: true }, { outF32: true, subgroups: sg, vec4Half: true }, { outF32: true, subgroups: sg, rowsPerWG: 4, vec4Half: true },
  { affine: true }, { outF32: true, affine: true }, { subgroups: sg, affine: true }, { subgroups: sg, rowsPerWG: 4, affine: true },
  { outF32: true, subgroups: sg, affine: true }, { outF32: true, subgroups: sg, rowsPerWG: 4, affine: true },
  { subgroups: sg, vec4Half: true, affine: true }, { subgroups: sg, rowsPerWG: 4, vec4Half: true, affine: true },
  { outF32: true, subgroups: sg, vec4Half: true, affine: true }, { outF32: true, subgroups: sg, rowsPerWG: 4, vec4Half: true, affine: true },
  { affine: true, moe: true, subgroups: sg, rowsPerWG: 4 }, { affine: true, moe: true, subgroups: sg, rowsPerWG: 4, vec4Half: true },
  { affine: true, q3: true }, { affine: true, q3: true, subgroups: sg, rowsPerWG: 4 }, { affine: true, q3: true, moe: true, subgroups: sg, rowsPerWG: 4 },
]
const GEMM_ENTRIES = []
for (const n of ['int4_matmul_tiled_m', 'int4_matmul_tiled_st', 'int4_matmul_sgmat', 'int4_matmul_sg_e1', 'int4_matmul_sg_e5']) {
  GEMM_ENTRIES.push(n, n + '_affine')
}
// the 8-bit MLX-affine twins: same bindings and PODArgs, K_PACKED = K/4 (compiler.ts:429-430)
const INT8_ENTRIES = ['int8_affine_matvec', 'int8_affine_batched']
const ALL_ENTRIES = INT4_MATMUL_VARIANTS.map(int4MatmulEntry).concat(GEMM_ENTRIES, INT8_ENTRIES)

/** compile()'s job for one entry point: name -> what it means for the descriptor. */
function createPipeline(entry) {
  if (ALL_ENTRIES.indexOf(entry) < 0) throw new Error("unknown int4 matmul entry point '" + entry + "'")
  if (INT8_ENTRIES.indexOf(entry) >= 0) {
    const batched = /_batched$/.test(entry)
    return Object.freeze({ label: entry, affine: true, bits: 8, outF32: false, moe: false, runtimeM: batched, fixedM: 1,
                           kernel: batched ? KERNEL.AUTO : KERNEL.GEMV })
  }
  const affine = entry.indexOf('_affine') >= 0
  const base = { label: entry, affine, bits: 4, outF32: false, moe: false, runtimeM: false, fixedM: 1, kernel: KERNEL.GEMV }
  if (GEMM_ENTRIES.indexOf(entry) >= 0) return Object.freeze(Object.assign(base, { runtimeM: true, kernel: KERNEL.GEMM }))
  if (entry.indexOf('int4_matmul_batched_dyn') === 0) return Object.freeze(Object.assign(base, { runtimeM: true, kernel: KERNEL.AUTO }))
  if (entry === 'int4_matmul_batched_m4') return Object.freeze(Object.assign(base, { affine: false, fixedM: 4, kernel: KERNEL.AUTO }))
  return Object.freeze(Object.assign(base, { bits: entry.indexOf('_q3') >= 0 ? 3 : 4, outF32: entry.indexOf('_f32') >= 0, moe: /_moe$/.test(entry) }))
}

// ---- resolution ---------------------------------------------------------------------------------

/** `available` is a Set (or array) of compiled entry names; affine resolves first. */
function resolveMatmul(variant, available, vec4, k, vec4Half, affine, vec4Affine) {
  const A = available instanceof Set ? available : new Set(available)
  if (vec4Half === undefined || vec4Half === null) vec4Half = !!vec4
  const f32 = (n) => n.replace('int4_matmul', 'int4_matmul_f32')
  const have = (n) => A.has(n) && A.has(f32(n))
  const pick = (n, rows, label) => ({ pipeline: n, pipelineF32: f32(n), rowsPerWG: rows, label })
  if (affine) {
    const wide = k !== undefined && k !== null && !!vec4Affine && k % 512 === 0
    const ladder = [
      [wide && variant !== 'scalar', 'int4_matmul_tiled_vec4h_affine', 4, 'tiled_vec4h_affine'],
      [wide && variant !== 'scalar', 'int4_matmul_sg_vec4h_affine', 1, 'sg_vec4h_affine'],
      [variant !== 'scalar', 'int4_matmul_tiled_affine', 4, 'tiled_affine'],
      [variant !== 'scalar', 'int4_matmul_sg_affine', 1, 'sg_affine'],
    ]
    for (const [cond, n, rows, label] of ladder) if (cond && have(n)) return pick(n, rows, label)
    return pick('int4_matmul_affine', 1, 'scalar_affine')
  }
  let useHalf = false
  if (k !== undefined && k !== null && k % 1024 !== 0) {
    useHalf = !!vec4Half && k % 512 === 0
    vec4 = false
  }
  const ladder = [
    [useHalf && variant === 'tiled', 'int4_matmul_tiled_vec4h', 4, 'tiled_vec4h'],
    [useHalf && variant === 'sg', 'int4_matmul_sg_vec4h', 1, 'sg_vec4h'],
    [vec4 && variant === 'tiled', 'int4_matmul_tiled_vec4', 4, 'tiled_vec4'],
    [vec4 && variant === 'sg', 'int4_matmul_sg_vec4', 1, 'sg_vec4'],
    [variant === 'tiled8', 'int4_matmul_tiled8', 8, 'tiled8'],
    [variant === 'tiled', 'int4_matmul_tiled', 4, 'tiled'],
    [variant === 'sg', 'int4_matmul_sg', 1, 'sg'],
  ]
  for (const [cond, n, rows, label] of ladder) if (cond && have(n)) return pick(n, rows, label)
  return pick('int4_matmul', 1, 'scalar')
}

function resolveChunkCap(opts, spec, sgmatAvail) {
  if (opts.chunkCap !== undefined && opts.chunkCap !== null) return opts.chunkCap
  const m = spec.maxChunkCap === undefined || spec.maxChunkCap === null ? Infinity : spec.maxChunkCap
  return Math.min(sgmatAvail ? 1024 : 64, m)
}

function pickChunkGemm(caps) {
  const want = caps.want || (caps.e5Ready ? 'e5' : caps.sgmatReady ? 'sgmat' : 'matvec')
  const ladder = [
    ['e5', want === 'e5' && caps.dimsOK && caps.capTiles64 && caps.e5Ready],
    ['sgmat', (want === 'sgmat' || want === 'e5') && caps.dimsOK && caps.sgmatReady],
    ['tiled', (want === 'tiled' || caps.chunkTiled) && caps.dimsOK],
    ['matvec', true],
  ]
  const used = ladder.find((e) => e[1])[0]
  if (caps.want && used !== caps.want) {
    const why = !caps.dimsOK ? 'dims do not tile (cap ' + caps.cap + ', d/qDim/ffn must be %64 and cap %32)'
      : caps.want === 'e5' && !caps.capTiles64 ? 'E5 stages a 64-row tile, so cap must be %64 (got ' + caps.cap + ')'
      : caps.want === 'e5' || caps.want === 'sgmat' ? 'its pipeline was not built — usually a device without chromium-experimental-subgroup-matrix'
      : 'that pipeline was not built'
    return { used, rejected: "chunkGemm: asked for '" + caps.want + "', can only run '" + used + "' — " + why }
  }
  return { used, rejected: null }
}

function foldGridX(total, maxX) {
  const x = Math.min(total, maxX === undefined ? 16384 : maxX)
  return { x, z: Math.ceil(total / x) }
}

// ---- device, buffers, bind groups, dispatch ----------------------------------------------------------

class ZtvmBuffer {
  constructor(device, size, label) {
    this.device = device
    this.size = Math.max(size, 4)
    this.label = label || ''
    this.addr = addon().alloc(device.ctx, this.size)
  }
  destroy() {
    if (this.addr) addon().free(this.device.ctx, this.addr)
    this.addr = 0n
  }
}

class Uniform {
  constructor(words) { this.words = words }
  /** queue.writeBuffer(uniform, byteOffset, u32) — M_ROWS lives at byte 12 (engine-core.ts:4251-4254). */
  writeU32(byteOffset, value) { this.words[byteOffset >> 2] = value >>> 0 }
}

class Device {
  constructor(index) { this.ctx = addon().create(index || 0) }
  close() { if (this.ctx) addon().destroy(this.ctx); this.ctx = null }
  info() { return addon().deviceInfo(this.ctx) }
  createBuffer(size, label) { return new ZtvmBuffer(this, size, label) }
  writeBuffer(buf, offset, data) {
    if (offset + data.byteLength > buf.size) throw new Error("writeBuffer past the end of '" + buf.label + "'")
    addon().upload(this.ctx, buf.addr, offset, data)
  }
  readBuffer(buf, offset, bytes) { return addon().download(this.ctx, buf.addr, offset || 0, bytes === undefined ? buf.size - (offset || 0) : bytes) }
  fill(buf, byte) { addon().fill(this.ctx, buf.addr, 0, byte, buf.size) }
  /** uniformBuf(device, [u32...]): padded to 16 bytes; kept host-side because shapes travel by value. */
  uniformBuf(data) {
    const words = data.map((v) => v >>> 0)
    while (words.length % 4) words.push(0)
    return new Uniform(words)
  }
  createPipeline(entry) { return createPipeline(entry) }
  /** bg(pipeline, [out, in, scales, weights, pod, (biases), (ids)]): binding i = array index i. */
  bg(pipeline, bufs) {
    const addr = (i, b) => {
      if (!b) throw new Error('bg: null buffer at binding ' + i + " of pipeline '" + pipeline.label + "'")
      if (b.buffer) {
        if (b.offset % 256) throw new Error('bg: binding ' + i + ' offset ' + b.offset + ' is not 256-byte aligned')
        return b.buffer.addr + BigInt(b.offset)
      }
      return b.addr
    }
    if (pipeline.affine && bufs.length < 6) throw new Error("affine matmul '" + pipeline.label + "' has no bias buffer at binding 5")
    const need = 5 + (pipeline.affine ? 1 : 0) + (pipeline.moe ? 1 : 0)
    if (bufs.length < need) throw new Error("bg: pipeline '" + pipeline.label + "' needs " + need + ' bindings, got ' + bufs.length)
    if (!(bufs[4] instanceof Uniform)) throw new Error("bg: binding 4 of '" + pipeline.label + "' must be the PODArgs uniform")
    // bytes bound at a binding: WebGPU bounds-checks storage accesses against them, here they arm the expert-id guard
    const size = (b) => (b ? b.size : 0)
    return {
      pipeline, pod: bufs[4], out: addr(0, bufs[0]), in: addr(1, bufs[1]), scales: addr(2, bufs[2]), weights: addr(3, bufs[3]),
      biases: pipeline.affine ? addr(5, bufs[5]) : 0n, ids: pipeline.moe ? addr(6, bufs[6]) : 0n,
      sizes: { scales: size(bufs[2]), weights: size(bufs[3]), biases: pipeline.affine ? size(bufs[5]) : 0 },
    }
  }
  descriptor(group, wgX, wgY, wgZ) {
    const p = group.pipeline, w = group.pod.words
    const d = {
      bits: p.bits, affine: p.affine ? 1 : 0, out_f32: p.outF32 ? 1 : 0, kernel: p.kernel, k_packed: w[0], scales_per_row: w[1], N: w[2], M: 1,
      out: group.out, in: group.in, scales: group.scales, weights: group.weights, biases: group.biases, ids: group.ids,
    }
    if (p.moe) {
      if (w.length < 8) throw new Error("moe pipeline '" + p.label + "' needs the 8-field PODArgs")
      d.in_slot_stride = w[3]; d.out_slot_stride = w[4]; d.in_tok_stride = w[5]; d.out_tok_stride = w[6]; d.ids_stride = w[7]
      d.tokens = wgY === undefined ? 1 : wgY
      d.slots = wgZ === undefined ? 1 : wgZ
      d.experts = stackHeight(group, d)
    } else if (p.runtimeM) d.M = w[3]
    else d.M = p.fixedM
    return d
  }
  /** dispatch(pipeline, bindGroup, wgX, wgY, wgZ): the WGSL grid is ignored except for MoE (y = tokens, z = slots). */
  dispatch(pipeline, group, wgX, wgY, wgZ) {
    if (group.pipeline !== pipeline) throw new Error("dispatch: bind group was built for '" + group.pipeline.label + "', not '" + pipeline.label + "'")
    const d = this.descriptor(group, wgX, wgY, wgZ)
    if (d.M === 0 && !pipeline.moe) return
    addon().matmul(this.ctx, d)
  }
  // ---- the dispatches either side of the matmuls (bindings in binding order, then the PODArgs fields, then tokens) ----
  _a(b) { return b ? (b.buffer ? b.buffer.addr + BigInt(b.offset) : b.addr) : 0n }
  /** silu_mul.wgsl: out [rows, ffn] <- gateUp [rows, 2*ffn] */
  siluMul(out, gateUp, rows, ffn) { addon().siluMul(this.ctx, this._a(out), this._a(gateUp), rows, ffn) }
  /** moe_combine.wgsl */
  moeCombine(out, slots, score, tokens, N, SLOTS) { addon().moeCombine(this.ctx, this._a(out), this._a(slots), this._a(score), tokens, N, SLOTS) }
  /** moe_router_logits / _q4 / _f16 by bits = 8 / 4 / 16 (scales and biases null for 16) */
  moeRouterLogits(logits, x, w, scales, biases, bits, D, rows, tokens) {
    addon().moeRouterLogits(this.ctx, this._a(logits), this._a(x), this._a(w), this._a(scales), this._a(biases), bits, D, rows, tokens === undefined ? 1 : tokens)
  }
  /** moe_router_topk.wgsl */
  moeRouterTopk(outIdx, outScore, logits, E, K, normTopk, hasShared, tokens) {
    addon().moeRouterTopk(this.ctx, this._a(outIdx), this._a(outScore), this._a(logits), E, K, normTopk ? 1 : 0, hasShared ? 1 : 0, tokens === undefined ? 1 : tokens)
  }
  /** moe_slot_translate.wgsl */
  moeSlotTranslate(idsOut, idsIn, slotMap, n, mapLen) { addon().moeSlotTranslate(this.ctx, this._a(idsOut), this._a(idsIn), this._a(slotMap), n, mapLen) }
  /** gate + up + SiLU in one pass: the gate's bind group and grid, plus the up projection's weights / scales / biases */
  ffnGated(pipeline, group, upWeights, upScales, upBiases, wgX, wgY, wgZ) {
    if (group.pipeline !== pipeline) throw new Error("ffnGated: bind group was built for '" + group.pipeline.label + "', not '" + pipeline.label + "'")
    addon().ffnGated(this.ctx, this.descriptor(group, wgX, wgY, wgZ), this._a(upWeights), this._a(upScales), this._a(upBiases))
  }
  /**
   * fused_ffn_prologue.wgsl: ffnGated with the FFN-entry add + RMSNorm folded in; the bind group's input (binding 1)
   * is the residual, `delta` the o-proj output added to it, `gamma` the norm gain, rmsEps the prelude's RMS_EPS
   */
  ffnGatedPrologue(pipeline, group, upWeights, upScales, upBiases, delta, gamma, rmsEps, wgX, wgY, wgZ) {
    if (group.pipeline !== pipeline) throw new Error("ffnGatedPrologue: bind group was built for '" + group.pipeline.label + "', not '" + pipeline.label + "'")
    addon().ffnGatedPrologue(this.ctx, this.descriptor(group, wgX, wgY, wgZ), this._a(upWeights), this._a(upScales), this._a(upBiases),
      this._a(delta), this._a(gamma), rmsEps)
  }
  /**
   * qkv_fused*.wgsl: bindings [q_out, kv_pages, hidden, scales, weights, position_map, (biases)], the PODArgs
   * {position_map_elem_offset, pages_elem_offset} and the model constants of the shader prelude
   * (heads, kvHeads, headDim, pageSize, kvPageStride, headPageStride, vPageOffset, ropeTheta).
   */
  qkvFused(bufs, pod, model) {
    const w = pod.words, a = (b) => this._a(b)
    const K = model.d
    addon().qkvFused(this.ctx, {
      bits: 4, affine: model.affine ? 1 : 0, k_packed: K / 8, scales_per_row: K / (model.affine ? 64 : 32),
      heads: model.heads, kv_heads: model.kvHeads, head_dim: model.headDim, page_size: model.pageSize,
      kv_page_stride: model.kvPageStride, head_page_stride: model.headPageStride, v_page_offset: model.vPageOffset,
      position_map_elem_offset: w[0], pages_elem_offset: w[1], rope_theta: model.ropeTheta,
      kv_capacity: BigInt(Math.floor(bufs[1].size / 2)),
      q_out: a(bufs[0]), kv_pages: a(bufs[1]), hidden: a(bufs[2]), scales: a(bufs[3]), weights: a(bufs[4]),
      position_map: a(bufs[5]), biases: bufs[6] ? a(bufs[6]) : 0n,
    })
  }
  /**
   * qkv_fused_scratch.wgsl (int8-KV mode): bindings [q_out, k_slot, v_slot, hidden, scales, weights, position_map,
   * (biases)], the PODArgs {position_map_elem_offset, packGridDimX} and the model constants of the shader prelude.
   */
  qkvFusedScratch(bufs, pod, model) {
    const a = (b) => this._a(b)
    const K = model.d
    addon().qkvFusedScratch(this.ctx, {
      bits: 4, affine: model.affine ? 1 : 0, k_packed: K / 8, scales_per_row: K / (model.affine ? 64 : 32),
      heads: model.heads, kv_heads: model.kvHeads, head_dim: model.headDim, position_map_elem_offset: pod.words[0],
      rope_theta: model.ropeTheta, q_out: a(bufs[0]), hidden: a(bufs[3]), scales: a(bufs[4]), weights: a(bufs[5]),
      position_map: a(bufs[6]), biases: bufs[7] ? a(bufs[7]) : 0n,
    }, a(bufs[1]), a(bufs[2]))
  }
  /**
   * kv_quantize_int8.wgsl: bindings [k_slot, v_slot, pages_i8, scales, position_map], the PODArgs
   * {position_map_elem_offset, pages_elem_offset (words), scales_elem_offset, packGridDimX}; tokens = grid y.
   */
  kvQuantizeInt8(bufs, pod, model, tokens) {
    const w = pod.words, a = (b) => this._a(b)
    addon().kvQuantizeInt8(this.ctx, a(bufs[2]), a(bufs[3]), a(bufs[0]), a(bufs[1]), a(bufs[4]),
      BigInt(Math.floor(bufs[2].size / 4)), BigInt(Math.floor(bufs[3].size / 2)),
      model.kvHeads, model.headDim, model.pageSize, tokens === undefined ? 1 : tokens, w[0], w[1], w[2])
  }
  beginEncoder() { addon().recordBegin(this.ctx) }
  finishEncoder() { return addon().recordEnd(this.ctx) }
  submit(cmdbuf) { addon().submit(this.ctx, cmdbuf) }
  sync() { addon().sync(this.ctx) }

  // one ztvm_matmul from a ready descriptor (what dispatch() builds from a pipeline and a bind group)
  matmul(desc) { addon().matmul(this.ctx, desc) }
  // the same dispatch with the library's fixed scratch array: no device allocation, whatever the shape (for callers
  // under graph capture or in loops that must not allocate); throws where the dispatch needs more scratch than that
  matmulStatic(desc) { addon().matmulStatic(this.ctx, desc) }
  // a kernel that only reads `bytes` of `buffer` (`sink`: four bytes it practically never writes): the streaming-read time
  // of this device, to put a GEMV's time beside
  readProbe(buffer, bytes, sink) { addon().readProbe(this.ctx, buffer.addr, bytes, sink.addr) }

  // Time this library's kernel families on `desc` (gemm_tune.js: probeFamilies) with this device's queue.
  probeFamilies(desc, families, Ms, opts) {
    return tune.probeFamilies({ validate: (d) => addon().validate(d), matmul: (d) => this.matmul(d), sync: () => this.sync() },
      desc, families, Ms, opts)
  }
}

function densePod(K, N, bits, affine, M) {
  const pod = [K * (bits || 4) / 32, K / (affine === false ? 32 : 64), N]
  if (M !== undefined) pod.push(M)
  return pod
}

/** Experts in the bound stacks, from the bound sizes; the three stacks must each hold that many. */
function stackHeight(group, d) {
  const label = group.pipeline.label
  const perW = d.N * d.k_packed * 4, perS = d.N * d.scales_per_row * 2
  if (!perW || !perS) throw new Error("moe pipeline '" + label + "': empty expert (N=" + d.N + ', K_PACKED=' + d.k_packed + ')')
  const sz = group.sizes || { weights: 0, scales: 0, biases: 0 }
  let experts = Math.min(Math.floor(sz.weights / perW), Math.floor(sz.scales / perS))
  if (group.pipeline.affine) experts = Math.min(experts, Math.floor(sz.biases / perS))
  if (experts < 1) throw new Error("moe pipeline '" + label + "': the bound stacks hold no whole expert (weights " + sz.weights + ' B, scales ' + sz.scales + ' B)')
  return experts
}

function moePods(dModel, ffn, slots, bits) {
  const b = bits || 4
  return {
    gate: [dModel * b / 32, dModel / 64, ffn, 0, 2 * ffn, dModel, slots * 2 * ffn, slots],
    down: [ffn * b / 32, ffn / 64, dModel, ffn, dModel, slots * ffn, slots * dModel, slots],
  }
}

module.exports = {
  KERNEL, Device, Uniform, int4MatmulEntry, checkOpts, INT4_MATMUL_VARIANTS, GEMM_ENTRIES, INT8_ENTRIES, ALL_ENTRIES, createPipeline,
  resolveMatmul, resolveChunkCap, pickChunkGemm, foldGridX, densePod, moePods,
  // boot-time choice of the prefill GEMM by measurement (gemm_tune.js)
  TUNE_VERSION: tune.TUNE_VERSION, TUNE_TTL_MS: tune.TUNE_TTL_MS, TUNE_MS: tune.TUNE_MS, tuneKey: tune.tuneKey,
  deviceFingerprint: tune.deviceFingerprint, median: tune.median, pickFromTimings: tune.pickFromTimings,
  loadTunedPick: tune.loadTunedPick, saveTunedPick: tune.saveTunedPick, memoryTuneStore: tune.memoryTuneStore,
  fileTuneStore: tune.fileTuneStore, timeClosures: tune.timeClosures, resolveTunedGemm: tune.resolveTunedGemm,
  validate: (desc) => addon().validate(desc), resolve: (desc) => addon().resolve(desc), abiVersion: () => addon().abiVersion(),
}
