"""Host-side mirror of the reference's kernel-dispatch surface for the quantized matmul family.

The reference engine talks to its kernels through three closures and a set of
named pipelines (paths relative to the reference's root):

  uniformBuf(device, [u32...])                 src/zero-tvm/engine-core.ts:53-65
  bg(device, pipeline, [out, in, scales, weights, pod, (biases), (ids)])   :76-92
  dispatch(enc, pipeline, bindGroup, wgX, wgY, wgZ)                        :2151-2179
  pipelines named by int4MatmulEntry()         src/compiler/shaders/int4_matmul.gen.ts:137-152

This module keeps those names, argument orders and error behaviour, and turns a
(pipeline, bind group, grid) triple into one ztvm_matmul descriptor. What a
WGSL variant only tuned (rowsPerWG, subgroups, vec4/vec4h loads, the workgroup
grid) is accepted and ignored: the HIP library sizes its own launches from
N, M, tokens and slots. What changes arithmetic (affine, q3, moe, outF32, the
runtime-M GEMM entries) selects descriptor fields.
"""
import struct
from dataclasses import dataclass

import numpy as np

from . import capi

# ---------------------------------------------------------------------------------------
# Variant naming (int4_matmul.gen.ts:32-152, :172-197, :701-766)
# ---------------------------------------------------------------------------------------


@dataclass(frozen=True)
class Int4MatmulOpts:
    outF32: bool = False
    rowsPerWG: int = 1
    subgroups: bool = False
    m: int = 1
    vec4: bool = False
    vec4Half: bool = False
    mDyn: bool = False
    affine: bool = False
    moe: bool = False
    q3: bool = False


def int4_matmul_entry(o=Int4MatmulOpts()):
    """Entry-point name of a variant (int4_matmul.gen.ts:137-152)."""
    if o.mDyn:
        return "int4_matmul_batched_dyn_affine" if o.affine else "int4_matmul_batched_dyn"
    if o.m == 4:
        return "int4_matmul_batched_m4"
    name = "int4_matmul"
    if o.outF32:
        name += "_f32"
    if o.rowsPerWG == 4:
        name += "_tiled"
    elif o.rowsPerWG == 8:
        name += "_tiled8"
    elif o.subgroups:
        name += "_sg"
    if o.vec4:
        name += "_vec4"
    elif o.vec4Half:
        name += "_vec4h"
    if o.affine:
        name += "_affine"
    if o.q3:
        name += "_q3"
    if o.moe:
        name += "_moe"
    return name


def check_opts(o):
    """The generator's legality rules (int4_matmul.gen.ts:172-197); raises ValueError with its messages."""
    if o.moe and not o.affine:
        raise ValueError("moe requires affine (the MoE weights are MLX affine-quantised)")
    if o.q3 and not o.affine:
        raise ValueError("q3 requires affine (3-bit ships only in the MLX-affine layout)")
    if o.affine and o.m != 1:
        raise ValueError("affine is implemented at m=1 (plus the mDyn path); no fixed-M sibling exists")
    if o.q3 and (o.vec4 or o.vec4Half):
        raise ValueError("q3 has no wide-load path: its 3-bit bitstream is not word-aligned")
    if o.moe and o.vec4:
        raise ValueError("moe has no full-vec4 path: that body does not apply the slot/token offsets")
    if o.rowsPerWG != 1 and not o.subgroups:
        raise ValueError("rowsPerWG > 1 requires subgroups")
    if o.m == 4 and (not o.subgroups or o.rowsPerWG != 4):
        raise ValueError("m=4 requires subgroups + rowsPerWG=4")
    if o.vec4 and not o.subgroups:
        raise ValueError("vec4 requires subgroups (32-thread WG keeps K=3072 divisible)")
    if o.vec4 and o.m != 1:
        raise ValueError("vec4 not implemented for m=4")
    if o.vec4Half and (o.vec4 or not o.subgroups or o.m != 1):
        raise ValueError("vec4Half requires subgroups + m=1 and is mutually exclusive with vec4")
    if o.mDyn and (not o.subgroups or o.rowsPerWG != 4 or o.m != 1 or o.vec4 or o.vec4Half or o.outF32):
        raise ValueError("mDyn requires subgroups + rowsPerWG=4 (no vec4/outF32/m=4)")


_O = Int4MatmulOpts
# The shipped variants, in the reference's order (int4_matmul.gen.ts:701-766).
INT4_MATMUL_VARIANTS = (
    _O(), _O(subgroups=True), _O(subgroups=True, rowsPerWG=4), _O(subgroups=True, rowsPerWG=8),
    _O(outF32=True), _O(outF32=True, subgroups=True), _O(outF32=True, subgroups=True, rowsPerWG=4),
    _O(outF32=True, subgroups=True, rowsPerWG=8),
    _O(subgroups=True, rowsPerWG=4, m=4), _O(subgroups=True, rowsPerWG=4, mDyn=True),
    _O(subgroups=True, rowsPerWG=4, mDyn=True, affine=True),
    _O(subgroups=True, vec4=True), _O(subgroups=True, rowsPerWG=4, vec4=True),
    _O(outF32=True, subgroups=True, vec4=True), _O(outF32=True, subgroups=True, rowsPerWG=4, vec4=True),
    _O(subgroups=True, vec4Half=True), _O(subgroups=True, rowsPerWG=4, vec4Half=True),
    _O(outF32=True, subgroups=True, vec4Half=True), _O(outF32=True, subgroups=True, rowsPerWG=4, vec4Half=True),
    _O(affine=True), _O(outF32=True, affine=True), _O(subgroups=True, affine=True),
    _O(subgroups=True, rowsPerWG=4, affine=True),
    _O(outF32=True, subgroups=True, affine=True), _O(outF32=True, subgroups=True, rowsPerWG=4, affine=True),
    _O(subgroups=True, vec4Half=True, affine=True), _O(subgroups=True, rowsPerWG=4, vec4Half=True, affine=True),
    _O(outF32=True, subgroups=True, vec4Half=True, affine=True),
    _O(outF32=True, subgroups=True, rowsPerWG=4, vec4Half=True, affine=True),
    _O(affine=True, moe=True, subgroups=True, rowsPerWG=4),
    _O(affine=True, moe=True, subgroups=True, rowsPerWG=4, vec4Half=True),
    _O(affine=True, q3=True), _O(affine=True, q3=True, subgroups=True, rowsPerWG=4),
    _O(affine=True, q3=True, moe=True, subgroups=True, rowsPerWG=4),
)

# The tiled / matrix-unit GEMM generators (compiler.ts:354-363; gemm-bench.mjs:412-430), symmetric and affine.
GEMM_ENTRIES = tuple(n + s for n in ("int4_matmul_tiled_m", "int4_matmul_tiled_st", "int4_matmul_sgmat",
                                     "int4_matmul_sg_e1", "int4_matmul_sg_e5") for s in ("", "_affine"))

# The 8-bit MLX-affine twins: same bindings and PODArgs, K_PACKED = K/4 (compiler.ts:429-430;
# src/compiler/shaders/int8_affine_matvec.wgsl, int8_affine_batched.wgsl).
INT8_ENTRIES = ("int8_affine_matvec", "int8_affine_batched")

ALL_ENTRIES = tuple(int4_matmul_entry(o) for o in INT4_MATMUL_VARIANTS) + GEMM_ENTRIES + INT8_ENTRIES


@dataclass(frozen=True)
class Pipeline:
    """What an entry-point name means for the descriptor."""
    label: str
    affine: bool
    bits: int
    out_f32: bool
    moe: bool
    runtime_m: bool   # PODArgs carries M_ROWS (batched_dyn and the GEMM generators)
    fixed_m: int      # 4 for int4_matmul_batched_m4, else 1
    kernel: int       # ZTVM_KERNEL_* family request


def create_pipeline(entry):
    """compile()'s job for one entry point (compiler.ts:341-371): name -> Pipeline. Unknown names raise."""
    if entry not in ALL_ENTRIES:
        raise ValueError("unknown int4 matmul entry point '%s'" % entry)
    if entry in INT8_ENTRIES:
        batched = entry.endswith("_batched")
        return Pipeline(entry, True, 8, False, False, batched, 1, capi.KERNEL_AUTO if batched else capi.KERNEL_GEMV)
    affine = "_affine" in entry
    if entry in GEMM_ENTRIES:
        # the reference's matrix-unit rungs; tiled_m / tiled_st keep f32 weights, which every family here does
        return Pipeline(entry, affine, 4, False, False, True, 1, capi.KERNEL_GEMM)
    if entry.startswith("int4_matmul_batched_dyn"):
        return Pipeline(entry, affine, 4, False, False, True, 1, capi.KERNEL_AUTO)
    if entry == "int4_matmul_batched_m4":
        return Pipeline(entry, False, 4, False, False, False, 4, capi.KERNEL_AUTO)
    return Pipeline(entry, affine, 3 if "_q3" in entry else 4, "_f32" in entry, entry.endswith("_moe"), False, 1,
                    capi.KERNEL_GEMV)


# ---------------------------------------------------------------------------------------
# Variant resolution (src/zero-tvm/variants.ts:239-321) and the prefill ladder (engine-core.ts:195-259)
# ---------------------------------------------------------------------------------------

def resolve_matmul(variant, available, vec4=False, k=None, vec4_half=None, affine=False, vec4_affine=False):
    """Which pipeline pair a matmul instance resolves to. `available` is the set of compiled entry names.
    Affine MUST resolve first: a symmetric kernel reads MLX buffers without error and returns wrong logits."""
    if vec4_half is None:
        vec4_half = vec4
    have = lambda *names: all(n in available for n in names)

    def pick(f16, rows, label):
        f32 = f16.replace("int4_matmul", "int4_matmul_f32", 1)
        return {"pipeline": f16, "pipelineF32": f32, "rowsPerWG": rows, "label": label}

    if affine:
        wide = k is not None and vec4_affine and k % 512 == 0
        ladder = [
            (wide and variant != "scalar", "int4_matmul_tiled_vec4h_affine", 4, "tiled_vec4h_affine"),
            (wide and variant != "scalar", "int4_matmul_sg_vec4h_affine", 1, "sg_vec4h_affine"),
            (variant != "scalar", "int4_matmul_tiled_affine", 4, "tiled_affine"),
            (variant != "scalar", "int4_matmul_sg_affine", 1, "sg_affine"),
        ]
        for cond, name, rows, label in ladder:
            if cond and have(name, name.replace("int4_matmul", "int4_matmul_f32", 1)):
                return pick(name, rows, label)
        return pick("int4_matmul_affine", 1, "scalar_affine")
    use_half = False
    if k is not None and k % 1024 != 0:
        use_half = vec4_half and k % 512 == 0
        vec4 = False
    ladder = [
        (use_half and variant == "tiled", "int4_matmul_tiled_vec4h", 4, "tiled_vec4h"),
        (use_half and variant == "sg", "int4_matmul_sg_vec4h", 1, "sg_vec4h"),
        (vec4 and variant == "tiled", "int4_matmul_tiled_vec4", 4, "tiled_vec4"),
        (vec4 and variant == "sg", "int4_matmul_sg_vec4", 1, "sg_vec4"),
        (variant == "tiled8", "int4_matmul_tiled8", 8, "tiled8"),
        (variant == "tiled", "int4_matmul_tiled", 4, "tiled"),
        (variant == "sg", "int4_matmul_sg", 1, "sg"),
    ]
    for cond, name, rows, label in ladder:
        if cond and have(name, name.replace("int4_matmul", "int4_matmul_f32", 1)):
            return pick(name, rows, label)
    return pick("int4_matmul", 1, "scalar")


def resolve_chunk_cap(opts_chunk_cap, spec_max_chunk_cap, sgmat_avail):
    """engine-core.ts:195-202."""
    if opts_chunk_cap is not None:
        return opts_chunk_cap
    cap = 1024 if sgmat_avail else 64
    return min(cap, spec_max_chunk_cap) if spec_max_chunk_cap is not None else cap


def pick_chunk_gemm(want=None, chunk_tiled=False, dims_ok=True, cap_tiles64=True, e5_ready=True, sgmat_ready=True,
                    cap=1024):
    """The prefill GEMM ladder e5 > sgmat > tiled > matvec (engine-core.ts:220-245). An explicit `want`
    that cannot run is a rejection, never a silent substitution."""
    w = want if want is not None else ("e5" if e5_ready else "sgmat" if sgmat_ready else "matvec")
    ladder = [
        ("e5", w == "e5" and dims_ok and cap_tiles64 and e5_ready),
        ("sgmat", w in ("sgmat", "e5") and dims_ok and sgmat_ready),
        ("tiled", (w == "tiled" or chunk_tiled) and dims_ok),
        ("matvec", True),
    ]
    used = next(name for name, ok in ladder if ok)
    if want and used != want:
        if not dims_ok:
            why = "dims do not tile (cap %d, d/qDim/ffn must be %%64 and cap %%32)" % cap
        elif want == "e5" and not cap_tiles64:
            why = "E5 stages a 64-row tile, so cap must be %%64 (got %d)" % cap
        elif want in ("e5", "sgmat"):
            why = "its pipeline was not built — usually a device without chromium-experimental-subgroup-matrix"
        else:
            why = "that pipeline was not built"
        return {"used": used, "rejected": "chunkGemm: asked for '%s', can only run '%s' — %s" % (want, used, why)}
    return {"used": used, "rejected": None}


def fold_grid_x(total, max_x=16384):
    """engine-core.ts:247-259. Kept for callers that still compute WebGPU grids; HIP grids need no fold."""
    x = min(total, max_x)
    return {"x": x, "z": -(-total // x)}


# ---------------------------------------------------------------------------------------
# Device, buffers, bind groups, dispatch
# ---------------------------------------------------------------------------------------

class Buffer:
    """A device allocation (GPUBuffer)."""

    def __init__(self, device, size, label=""):
        self.device, self.size, self.label = device, max(int(size), 4), label
        self.addr = device.ctx.alloc(self.size)

    def destroy(self):
        if self.addr:
            self.device.ctx.free(self.addr)
            self.addr = 0


@dataclass(frozen=True)
class Region:
    """{buffer, offset, size} bind entry; offsets must be 256-byte aligned (engine-core.ts:71-74)."""
    buffer: Buffer
    offset: int
    size: int


@dataclass
class Uniform:
    """PODArgs uniform: u32 fields padded to 16 bytes (engine-core.ts:53-65). Kept host-side:
    the HIP library takes shapes by value, so a uniform update is a field write."""
    words: list

    def write_u32(self, byte_offset, value):
        """queue.writeBuffer(uniform, byte_offset, u32) — e.g. M_ROWS at byte 12 (engine-core.ts:4251-4254)."""
        self.words[byte_offset // 4] = int(value) & 0xFFFFFFFF

    def bytes(self):
        return struct.pack("<%dI" % len(self.words), *self.words)


@dataclass
class BindGroup:
    pipeline: Pipeline
    out: tuple
    inp: tuple
    scales: tuple
    weights: tuple
    pod: Uniform
    biases: tuple
    ids: tuple


class Device:
    """GPUDevice + queue over one ztvm context."""

    def __init__(self, index=0):
        self.ctx = capi.Context(index)
        self._recording = False

    def close(self):
        self.ctx.close()

    # -- buffers -------------------------------------------------------------------------
    def create_buffer(self, size, label=""):
        return Buffer(self, size, label)

    def write_buffer(self, buf, offset, data):
        arr = np.ascontiguousarray(data)
        if offset + arr.nbytes > buf.size:
            raise ValueError("writeBuffer past the end of '%s'" % buf.label)
        self.ctx.upload(buf.addr, arr, offset)

    def read_buffer(self, buf, dtype, offset=0, nbytes=None):
        return self.ctx.download(buf.addr, buf.size - offset if nbytes is None else nbytes, dtype, offset)

    def uniform_buf(self, data):
        words = [int(v) & 0xFFFFFFFF for v in data]
        while len(words) % 4:
            words.append(0)
        return Uniform(words)

    # -- pipelines and bind groups ----------------------------------------------------------
    create_pipeline = staticmethod(create_pipeline)

    def bg(self, pipeline, bufs):
        """Binding i = list index i: out, in, scales, weights, pod, (biases), (ids)."""
        def addr(i, b):
            if b is None:
                raise ValueError("bg: null buffer at binding %d of pipeline '%s'" % (i, pipeline.label))
            if isinstance(b, Region):
                if b.offset % 256:
                    raise ValueError("bg: binding %d offset %d is not 256-byte aligned" % (i, b.offset))
                return (b.buffer.addr + b.offset, b.size)
            return (b.addr, b.size)

        need = 5 + (1 if pipeline.affine else 0) + (1 if pipeline.moe else 0)
        if pipeline.affine and len(bufs) < 6:
            raise ValueError("affine matmul '%s' has no bias buffer at binding 5" % pipeline.label)
        if len(bufs) < need:
            raise ValueError("bg: pipeline '%s' needs %d bindings, got %d" % (pipeline.label, need, len(bufs)))
        if not isinstance(bufs[4], Uniform):
            raise ValueError("bg: binding 4 of '%s' must be the PODArgs uniform" % pipeline.label)
        a = [addr(i, b) if i != 4 else None for i, b in enumerate(bufs)]
        return BindGroup(pipeline, a[0], a[1], a[2], a[3], bufs[4], a[5] if pipeline.affine else (0, 0),
                         a[6] if pipeline.moe else (0, 0))

    # -- command encoding ----------------------------------------------------------------------
    def begin_encoder(self):
        self.ctx.record_begin()
        self._recording = True

    def finish_encoder(self):
        self._recording = False
        return self.ctx.record_end()

    def submit(self, cmdbuf):
        self.ctx.submit(cmdbuf)

    def descriptor(self, group, wg_x=1, wg_y=1, wg_z=1):
        """PODArgs + pipeline + grid -> ztvm_matmul_desc. The grid only matters for MoE, where
        y = tokens and z = slots (int4_matmul.gen.ts:236-243)."""
        p, w = group.pipeline, group.pod.words
        d = capi.MatmulDesc(bits=p.bits, affine=int(p.affine), out_f32=int(p.out_f32), kernel=p.kernel,
                            k_packed=w[0], scales_per_row=w[1], N=w[2], M=1,
                            out=group.out[0], in_=group.inp[0], scales=group.scales[0], weights=group.weights[0],
                            biases=group.biases[0], ids=group.ids[0])
        if p.moe:
            if len(w) < 8:
                raise ValueError("moe pipeline '%s' needs the 8-field PODArgs" % p.label)
            d.in_slot_stride, d.out_slot_stride, d.in_tok_stride, d.out_tok_stride, d.ids_stride = w[3:8]
            d.tokens, d.slots = wg_y, wg_z
            d.experts = self.stack_height(group, d)
        elif p.runtime_m:
            d.M = w[3]
        else:
            d.M = p.fixed_m
        return d

    @staticmethod
    def stack_height(group, d):
        """Experts in the bound stacks, from the sizes of the bound regions: WebGPU bounds-checks
        every storage access against those sizes, here the kernel's expert-id guard does, so the
        guard is always armed for a dispatch built from a bind group. The three stacks must agree."""
        per_w = d.N * d.k_packed * 4
        per_s = d.N * d.scales_per_row * 2
        if per_w == 0 or per_s == 0:
            raise ValueError("moe pipeline '%s': empty expert (N=%d, K_PACKED=%d)" % (group.pipeline.label, d.N, d.k_packed))
        heights = [group.weights[1] // per_w, group.scales[1] // per_s]
        if group.pipeline.affine:
            heights.append(group.biases[1] // per_s)
        experts = min(heights)
        if experts < 1:
            raise ValueError("moe pipeline '%s': the bound stacks hold no whole expert (weights %d B, scales %d B)"
                             % (group.pipeline.label, group.weights[1], group.scales[1]))
        return experts

    def dispatch(self, pipeline, group, wg_x, wg_y=1, wg_z=1, label=None):
        """One compute pass. M_ROWS == 0 dispatches nothing, like a zero-row chunk."""
        if group.pipeline is not pipeline:
            raise ValueError("dispatch: bind group was built for '%s', not '%s'" % (group.pipeline.label, pipeline.label))
        d = self.descriptor(group, wg_x, wg_y, wg_z)
        if d.M == 0 and not pipeline.moe:
            return
        self.ctx.matmul(d)

    def sync(self):
        self.ctx.sync()


def dense_pod(K, N, bits=4, affine=True, M=None):
    """PODArgs of a dense dispatch: K_PACKED, SCALES_PER_ROW, N (, M_ROWS) (engine-core.ts:787-794, :4030-4038)."""
    pod = [K * bits // 32, K // (64 if affine else 32), N]
    if M is not None:
        pod.append(M)
    return pod


def moe_pods(d_model, ffn, slots, bits=4):
    """The gate/up and down PODArgs of a MoE block (engine-core.ts:1049-1056)."""
    gate = [d_model * bits // 32, d_model // 64, ffn, 0, 2 * ffn, d_model, slots * 2 * ffn, slots]
    down = [ffn * bits // 32, ffn // 64, d_model, ffn, d_model, slots * ffn, slots * d_model, slots]
    return gate, down
