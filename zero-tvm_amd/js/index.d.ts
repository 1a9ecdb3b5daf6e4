// Typings of the JavaScript host layer (index.js) for TypeScript callers such as the reference engine.
export interface Int4MatmulOpts {
  outF32?: boolean; rowsPerWG?: 1 | 4 | 8; subgroups?: boolean; m?: 1 | 4; vec4?: boolean; vec4Half?: boolean
  mDyn?: boolean; affine?: boolean; moe?: boolean; q3?: boolean
}
export interface Pipeline {
  readonly label: string; readonly affine: boolean; readonly bits: 3 | 4 | 8; readonly outF32: boolean
  readonly moe: boolean; readonly runtimeM: boolean; readonly fixedM: number; readonly kernel: number
}
export interface MatmulDesc {
  bits: number; affine: number; out_f32: number; kernel: number; M: number; N: number; k_packed: number; scales_per_row: number
  slots?: number; tokens?: number; in_slot_stride?: number; out_slot_stride?: number; in_tok_stride?: number
  out_tok_stride?: number; ids_stride?: number; experts?: number
  out: bigint; in: bigint; scales: bigint; weights: bigint; biases?: bigint; ids?: bigint
}
export declare class Uniform { words: number[]; writeU32(byteOffset: number, value: number): void }
export interface ZtvmBuffer { readonly size: number; readonly label: string; readonly addr: bigint; destroy(): void }
export type BindEntry = ZtvmBuffer | { buffer: ZtvmBuffer; offset: number; size: number } | Uniform
export interface BindGroup { pipeline: Pipeline; pod: Uniform }
export declare class Device {
  constructor(index?: number)
  close(): void
  info(): { name: string; computeUnits: number; hbmBytes: bigint }
  createBuffer(size: number, label?: string): ZtvmBuffer
  writeBuffer(buf: ZtvmBuffer, offset: number, data: ArrayBufferView | ArrayBuffer): void
  readBuffer(buf: ZtvmBuffer, offset?: number, bytes?: number): ArrayBuffer
  fill(buf: ZtvmBuffer, byte: number): void
  uniformBuf(data: number[]): Uniform
  createPipeline(entry: string): Pipeline
  bg(pipeline: Pipeline, bufs: BindEntry[]): BindGroup
  descriptor(group: BindGroup, wgX?: number, wgY?: number, wgZ?: number): MatmulDesc
  dispatch(pipeline: Pipeline, group: BindGroup, wgX: number, wgY?: number, wgZ?: number): void
  siluMul(out: BindEntry, gateUp: BindEntry, rows: number, ffn: number): void
  moeCombine(out: BindEntry, slots: BindEntry, score: BindEntry, tokens: number, N: number, SLOTS: number): void
  moeRouterLogits(logits: BindEntry, x: BindEntry, w: BindEntry, scales: BindEntry | null, biases: BindEntry | null,
    bits: 4 | 8 | 16, D: number, rows: number, tokens?: number): void
  moeRouterTopk(outIdx: BindEntry, outScore: BindEntry, logits: BindEntry, E: number, K: number, normTopk: boolean,
    hasShared: boolean, tokens?: number): void
  moeSlotTranslate(idsOut: BindEntry, idsIn: BindEntry, slotMap: BindEntry, n: number, mapLen: number): void
  ffnGated(pipeline: Pipeline, group: BindGroup, upWeights: BindEntry, upScales: BindEntry, upBiases: BindEntry | null,
    wgX?: number, wgY?: number, wgZ?: number): void
  ffnGatedPrologue(pipeline: Pipeline, group: BindGroup, upWeights: BindEntry, upScales: BindEntry, upBiases: BindEntry | null,
    delta: BindEntry, gamma: BindEntry, rmsEps: number, wgX?: number, wgY?: number, wgZ?: number): void
  qkvFused(bufs: BindEntry[], pod: Uniform, model: { d: number; affine?: boolean; heads: number; kvHeads: number; headDim: number
    pageSize: number; kvPageStride: number; headPageStride: number; vPageOffset: number; ropeTheta: number }): void
  qkvFusedScratch(bufs: BindEntry[], pod: Uniform, model: { d: number; affine?: boolean; heads: number; kvHeads: number
    headDim: number; ropeTheta: number }): void
  kvQuantizeInt8(bufs: BindEntry[], pod: Uniform, model: { kvHeads: number; headDim: number; pageSize: number },
    tokens?: number): void
  matmul(desc: MatmulDesc): void
  matmulStatic(desc: MatmulDesc): void
  readProbe(buffer: ZtvmBuffer, bytes: number, sink: ZtvmBuffer): void
  probeFamilies(desc: MatmulDesc, families: KernelFamily[], Ms?: number[],
    opts?: { warmup?: number; rounds?: number }): TuneTimings
  beginEncoder(): void
  finishEncoder(): unknown
  submit(cmdbuf: unknown): void
  sync(): void
}
export declare const KERNEL: { AUTO: 0; GEMV: 1; SKINNY: 2; GEMM: 3; ROWS: 4 }
export declare const INT4_MATMUL_VARIANTS: ReadonlyArray<Int4MatmulOpts>
export declare const GEMM_ENTRIES: ReadonlyArray<string>
export declare const INT8_ENTRIES: ReadonlyArray<string>
export declare const ALL_ENTRIES: ReadonlyArray<string>
export declare function int4MatmulEntry(opts?: Int4MatmulOpts): string
export declare function checkOpts(opts?: Int4MatmulOpts): void
export declare function createPipeline(entry: string): Pipeline
export declare function resolveMatmul(variant: string, available: Set<string> | string[], vec4?: boolean, k?: number,
  vec4Half?: boolean, affine?: boolean, vec4Affine?: boolean): { pipeline: string; pipelineF32: string; rowsPerWG: number; label: string }
export declare function resolveChunkCap(opts: { chunkCap?: number }, spec: { maxChunkCap?: number }, sgmatAvail: boolean): number
export type ChunkGemmName = 'e5' | 'sgmat' | 'tiled' | 'matvec'
export declare function pickChunkGemm(caps: { want?: ChunkGemmName; chunkTiled: boolean; dimsOK: boolean; capTiles64: boolean
  e5Ready: boolean; sgmatReady: boolean; cap: number }): { used: ChunkGemmName; rejected: string | null }
export type KernelFamily = 'gemm' | 'skinny' | 'rows' | 'gemv'
export type TuneTimings = { [candidate: string]: { [m: number]: number[] } }
export interface TuneStore { load(key: string): string | null; save(key: string, value: string): void }
export declare const TUNE_VERSION: number
export declare const TUNE_TTL_MS: number
export declare const TUNE_MS: number[]
export declare function tuneKey(adapterId: string, specId: string): string
export declare function deviceFingerprint(info: { name?: string; computeUnits?: number; hbmBytes?: bigint } | null): string | null
export declare function median(xs: number[]): number
export declare function pickFromTimings(medians: { [candidate: string]: number[] }, ladder: string[]): string
export declare function loadTunedPick(store: TuneStore | null, key: string, runnable: string[], now?: number): string | null
export declare function saveTunedPick(store: TuneStore | null, key: string, pick: string, ms: { [c: string]: number },
  candidates: string[]): void
export declare function memoryTuneStore(init?: { [key: string]: string }): TuneStore
export declare function fileTuneStore(file: string): TuneStore
export declare function timeClosures(sync: () => void, runs: { [candidate: string]: (m: number) => void }, Ms: number[],
  opts?: { warmup?: number; rounds?: number; clock?: () => number }): TuneTimings
export declare function resolveTunedGemm(opts: { specId: string; runnable: string[]; explicit?: string; store?: TuneStore | null
  adapterId?: string | null; order?: string[]; runProbe: () => TuneTimings }): { pick: string; source: 'explicit' | 'stored' | 'probed' } | null
export declare function foldGridX(total: number, maxX?: number): { x: number; z: number }
export declare function densePod(K: number, N: number, bits?: number, affine?: boolean, M?: number): number[]
export declare function moePods(dModel: number, ffn: number, slots: number, bits?: number): { gate: number[]; down: number[] }
export declare function validate(desc: MatmulDesc): { code: number; why: string }
export declare function resolve(desc: MatmulDesc): number
export declare function abiVersion(): number
