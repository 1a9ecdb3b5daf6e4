"""MLX safetensors checkpoints -> the buffers the kernels bind, built in device memory.

Host-side mirror of the reference's loader (paths relative to the reference's root):

  parseSafetensorsHeader, planLayer, planGlobal, planBytes, buildBuffer     src/zero-tvm/mlx-weights.ts
  openMlxCheckpoint, planModel, planKey, buildPlan, modelBytes, SLOTS,
  assertTiedHead, assembleMlx                                                src/zero-tvm/weight-loader-mlx.ts

Same plan names, record names, byte layouts and error behaviour. What differs is where the bytes are
made: the reference converts and concatenates on the CPU and uploads the result; here each record is
uploaded exactly as it sits in the file and converted / concatenated / permuted / dequantized by HIP
kernels into its place in the destination buffer (ztvm_repack_* of the C ABI), so the host never touches
a weight and a checkpoint crosses PCIe once. There is no CPU fallback: without the library nothing loads.
"""
import json
import re
import struct
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from . import capi

# ---------------------------------------------------------------------------------------------------
# safetensors container (mlx-weights.ts:37-75)
# ---------------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class TensorInfo:
    dtype: str
    shape: tuple
    begin: int  # byte range within the shard's data section
    end: int


def parse_safetensors_header(head):
    """{'tensors': {name: TensorInfo}, 'dataStart': int}. `head` is at least the first 8 + header-length bytes."""
    head = bytes(head)
    if len(head) < 8:
        raise ValueError("safetensors: need at least 8 bytes for the header length")
    lo, hi = struct.unpack_from("<II", head, 0)
    if hi != 0:
        raise ValueError("safetensors: header longer than 4 GB")
    if len(head) < 8 + lo:
        raise ValueError("safetensors: header is %d bytes, only %d supplied" % (lo, len(head) - 8))
    meta = json.loads(head[8:8 + lo].decode("utf-8"))
    tensors = {}
    for name, m in meta.items():
        if name == "__metadata__":
            continue
        tensors[name] = TensorInfo(m["dtype"], tuple(m["shape"]), m["data_offsets"][0], m["data_offsets"][1])
    return {"tensors": tensors, "dataStart": 8 + lo}


# ---------------------------------------------------------------------------------------------------
# model description: the fields of the reference's ModelSpec that the plans read
# (src/compiler/model-spec.ts:555-660)
# ---------------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class Mla:
    kvLoraRank: int
    qkNopeHeadDim: int
    qkRopeHeadDim: int
    vHeadDim: int


@dataclass(frozen=True)
class Moe:
    experts: int
    topK: int
    normTopkProb: bool = True
    sharedExpert: Optional[bool] = None     # None = the reference's default (present)
    routerBits: Optional[int] = None        # None = 8 (moe_router_logits), 4 or 16 otherwise
    denseLayers: tuple = ()
    denseFfn: Optional[int] = None


@dataclass(frozen=True)
class MlxSpec:
    id: str
    layers: int
    heads: int
    d: int = 0
    ffn: int = 0
    qkNorm: bool = False
    tiedEmbeddings: bool = False
    mlxPrefix: str = ""
    fullAttnInterval: int = 0
    mla: Optional[Mla] = None
    moe: Optional[Moe] = None
    layerKinds: tuple = field(default=())
    ffnKinds: tuple = field(default=())

    @property
    def mlaQProjRows(self):
        return self.heads * (self.mla.qkNopeHeadDim + self.mla.qkRopeHeadDim) if self.mla else 0

    @property
    def mlaKvaRows(self):
        return self.mla.kvLoraRank + self.mla.qkRopeHeadDim if self.mla else 0

    @staticmethod
    def bias_for(weight_record):
        """paramNaming.biasFor of the MLX specs (model-spec.ts:503)."""
        return re.sub(r"\.weight$", ".biases", weight_record)


def make_spec(**kw):
    """Derives layerKinds / ffnKinds like makeModelSpec (model-spec.ts:559-575): layer i is linear attention
    ('gdn') iff fullAttnInterval and (i+1) % interval != 0; a MoE model's layers are 'moe' except moe.denseLayers."""
    spec = MlxSpec(**kw)
    iv = spec.fullAttnInterval
    kinds = tuple("gdn" if iv and (i + 1) % iv != 0 else "attn" for i in range(spec.layers))
    dense = set(spec.moe.denseLayers) if spec.moe else set()
    if dense and spec.moe.denseFfn is None:
        raise ValueError("%s: moe.denseLayers needs moe.denseFfn — a dense layer's width is not moe_intermediate_size" % spec.id)
    ffn = tuple("moe" if spec.moe and i not in dense else "dense" for i in range(spec.layers))
    return MlxSpec(**{**kw, "layerKinds": kinds, "ffnKinds": ffn})


# ---------------------------------------------------------------------------------------------------
# plans (mlx-weights.ts:209-444)
# ---------------------------------------------------------------------------------------------------

CONVERTS = ("raw", "bf16->f16", "bf16->f32")


@dataclass(frozen=True)
class BufferPart:
    record: str
    convert: str


@dataclass(frozen=True)
class PermuteRows:
    rows: int
    src: tuple
    kind: str = "permuteRows"


@dataclass(frozen=True)
class DequantAffineSplit:
    k: int
    heads: int
    nope: int
    v: int
    bits: int = 4
    group: int = 64
    kind: str = "dequantAffineSplit"


@dataclass(frozen=True)
class BufferPlan:
    name: str
    parts: tuple
    op: object = None


def _q(base):
    return (BufferPart(base + ".weight", "raw"), BufferPart(base + ".scales", "bf16->f16"),
            BufferPart(base + ".biases", "bf16->f16"))


def _trio(name, bases, op=None):
    """Weights, scales and biases buffers of one logical tensor: each the concatenation of that component
    of every base, in order."""
    cols = [_q(b) for b in bases]
    return [BufferPlan("%s_%s" % (name, c), tuple(t[i] for t in cols), op) for i, c in enumerate("wsb")]


def _one(name, record, convert="bf16->f16"):
    return BufferPlan(name, (BufferPart(record, convert),))


def deint(j, R):
    """Row j of the permuted rotary block takes original row deint(j): the even rows, then the odd ones
    (mlx-weights.ts:303-310). The inverse map is just as plausible a matrix and a different model."""
    return 2 * j if j < R // 2 else 2 * (j - R // 2) + 1


def plan_layer(spec, L, prefix=None):
    """Every buffer one decoder layer needs and the records that build it (mlx-weights.ts:272-393)."""
    p = "%slayers.%d" % (prefix if prefix is not None else (spec.mlxPrefix or "") + "model.", L)
    plans = [_one("norm1", p + ".input_layernorm.weight"), _one("norm2", p + ".post_attention_layernorm.weight")]
    kind = spec.layerKinds[L]
    if kind == "attn" and spec.mla:
        M = spec.mla
        R, nope = M.qkRopeHeadDim, M.qkNopeHeadDim
        q_src = list(range(spec.mlaQProjRows))
        for h in range(spec.heads):
            pe = h * (nope + R) + nope
            for j in range(R):
                q_src[pe + j] = pe + deint(j, R)
        kv_src = list(range(spec.mlaKvaRows))
        for j in range(R):
            kv_src[M.kvLoraRank + j] = M.kvLoraRank + deint(j, R)
        plans += _trio("mla_q", [p + ".self_attn.q_proj"], PermuteRows(spec.mlaQProjRows, tuple(q_src)))
        plans += _trio("mla_kva", [p + ".self_attn.kv_a_proj_with_mqa"], PermuteRows(spec.mlaKvaRows, tuple(kv_src)))
        plans.append(_one("mla_kva_norm", p + ".self_attn.kv_a_layernorm.weight"))
        # one buffer holding [K^T | V], K^T first
        plans.append(BufferPlan("mla_kvb", _q(p + ".self_attn.kv_b_proj"),
                                DequantAffineSplit(k=M.kvLoraRank, heads=spec.heads, nope=nope, v=M.vHeadDim)))
        plans += _trio("o_proj", [p + ".self_attn.o_proj"])
    elif kind == "attn":
        plans += _trio("c_attn", [p + ".self_attn." + n for n in ("q_proj", "k_proj", "v_proj")])
        plans += _trio("o_proj", [p + ".self_attn.o_proj"])
        if spec.qkNorm:
            plans += [_one("q_norm", p + ".self_attn.q_norm.weight"), _one("k_norm", p + ".self_attn.k_norm.weight")]
    else:
        g = p + ".linear_attn"
        plans += _trio("gdn_proj", [g + "." + n for n in ("in_proj_qkv", "in_proj_z", "in_proj_a", "in_proj_b")])
        plans += _trio("gdn_out", [g + ".out_proj"])
        plans += [_one("gdn_conv", g + ".conv1d.weight"), _one("gdn_norm", g + ".norm.weight"),
                  _one("gdn_a_log", g + ".A_log", "bf16->f32"), _one("gdn_dt_bias", g + ".dt_bias", "bf16->f32")]

    if spec.ffnKinds[L] == "moe" and spec.moe:
        shared = True if spec.moe.sharedExpert is None else spec.moe.sharedExpert
        for proj in ("gate_proj", "up_proj", "down_proj"):
            bases = [p + ".mlp.switch_mlp." + proj] + ([p + ".mlp.shared_expert." + proj] if shared else [])
            plans += _trio("moe_" + proj, bases)
        gates = [p + ".mlp.gate"] + ([p + ".mlp.shared_expert_gate"] if shared else [])
        if spec.moe.routerBits == 16:
            # a router the quantizer skipped has no scales or biases to plan for
            plans.append(BufferPlan("router_w", tuple(BufferPart(g + ".weight", "bf16->f16") for g in gates)))
        else:
            plans += _trio("router", gates)
    else:
        plans += _trio("ffn", [p + ".mlp.gate_proj", p + ".mlp.up_proj"])
        plans += _trio("ffn_down", [p + ".mlp.down_proj"])
    return plans


def plan_global(spec, prefix=None, range_=None):
    """Embedding table, untied lm_head and final norm (mlx-weights.ts:413-444). lm_head sits one prefix level
    above the decoder stack; a tied head ships no lm_head records and the loader aliases the embedding."""
    pre = prefix if prefix is not None else (spec.mlxPrefix or "")
    first = (range_["start"] if range_ else 0) == 0
    last = (range_["end"] if range_ else spec.layers) == spec.layers

    def q(name, base):
        return [BufferPlan(name + "_w", (BufferPart(base + ".weight", "raw"),)),
                BufferPlan(name + "_s", (BufferPart(base + ".scales", "bf16->f16"),)),
                BufferPlan(name + "_b", (BufferPart(spec.bias_for(base + ".weight"), "bf16->f16"),))]

    out = []
    if first or (last and spec.tiedEmbeddings):
        out += q("embed", pre + "model.embed_tokens")
    if not spec.tiedEmbeddings and last:
        out += q("lm_head", pre + "lm_head")
    if last:
        out.append(_one("final_norm", pre + "model.norm.weight"))
    return out


def plan_bytes(plan, source_bytes, dtype_of=None):
    """Bytes a plan produces on the GPU (mlx-weights.ts:452-472): op-aware, and bf16->f32 doubles only when
    the source really is two bytes wide."""
    op = plan.op
    if op is not None and op.kind == "dequantAffineSplit":
        return op.heads * (op.nope + op.v) * op.k * 2
    n = 0
    for part in plan.parts:
        b = source_bytes(part.record)
        wide = part.convert == "bf16->f32" and (dtype_of(part.record) if dtype_of else "BF16") != "F32"
        n += b * 2 if wide else b
    return n


# ---------------------------------------------------------------------------------------------------
# buildBuffer, in device memory (mlx-weights.ts:490-543)
# ---------------------------------------------------------------------------------------------------

_CONVERT_CODE = {"raw": capi.CONVERT_RAW, "bf16->f16": capi.CONVERT_BF16_F16, "bf16->f32": capi.CONVERT_BF16_F32}


def _effective_convert(plan, part, dtype):
    """The dtype-aware pass-through rules: 'bf16->f16' means "the kernels read f16", not "the file is bf16"."""
    if part.convert == "raw":
        return "raw"
    if part.convert == "bf16->f16" and dtype == "F16":
        return "raw"
    if part.convert == "bf16->f32" and dtype == "F32":
        return "raw"
    if dtype != "BF16":
        raise ValueError("%s: %s is %s, expected BF16 for %s" % (plan.name, part.record, dtype, part.convert))
    return part.convert


def build_buffer(device, plan, read_record, dtype_of=None):
    """Build one plan's buffer on the device from raw record bytes. Returns (Buffer, overflow count); a nonzero
    count raises, like the reference, because a clamped scale is a wrong weight."""
    ctx = device.ctx
    raws, convs, sizes = [], [], []
    for part in plan.parts:
        raw = np.frombuffer(bytes(read_record(part.record)), np.uint8)
        conv = _effective_convert(plan, part, dtype_of(part.record) if dtype_of else "BF16")
        if conv != "raw" and raw.size % 2:
            raise ValueError("%s: %s has an odd byte count for a bf16 record" % (plan.name, part.record))
        raws.append(raw)
        convs.append(conv)
        sizes.append(raw.size * 2 if conv == "bf16->f32" else raw.size)
    total = sum(sizes)
    op = plan.op
    temps = []

    def temp(n):
        p = ctx.alloc(max(n, 16))
        temps.append(p)
        return p

    try:
        counter = temp(16)
        ctx.fill(counter, 0, 16)
        staging = temp(max([r.size for r in raws] + [16]))
        if op is not None and op.kind == "dequantAffineSplit":
            if len(raws) != 3:
                raise ValueError("%s: dequantAffineSplit needs exactly [weight, scales, biases], got %d parts"
                                 % (plan.name, len(raws)))
            rows, wpr, gpr = op.heads * (op.nope + op.v), op.k * op.bits // 32, op.k // op.group
            for n, got, what in ((rows * wpr * 4, sizes[0], "weight"), (rows * gpr * 2, sizes[1], "scales"),
                                 (rows * gpr * 2, sizes[2], "biases")):
                if n != got:
                    raise ValueError("%s: %s is %d B, expected %d B for [%d, %d] at %d bits"
                                     % (plan.name, what, got, n, rows, op.k, op.bits))
            pieces = []
            for raw, conv, size in zip(raws, convs, sizes):
                piece = temp(size)
                ctx.upload(staging, raw)
                ctx.repack_part(piece, staging, raw.size, _CONVERT_CODE[conv], counter)
                pieces.append(piece)
            out = device.create_buffer(plan_bytes(plan, lambda r: 0), plan.name)
            split_counter = temp(16)
            ctx.fill(split_counter, 0, 16)
            ctx.repack_dequant_split(out.addr, pieces[0], pieces[1], pieces[2], op.k, op.heads, op.nope, op.v, split_counter)
            over = int(ctx.download(split_counter, 4, np.uint32)[0])
            if over:
                out.destroy()
                raise ValueError("%s: %d dequantized value(s) exceed f16 range — these weights cannot be represented "
                                 "at f16 and the model would run wrong" % (plan.name, over))
        else:
            permute = op is not None and op.kind == "permuteRows"
            if permute:
                if len(op.src) != op.rows:
                    raise ValueError("%s: permuteRows has %d source indices for %d rows" % (plan.name, len(op.src), op.rows))
                if total % op.rows:
                    raise ValueError("%s: %d B does not divide into %d rows" % (plan.name, total, op.rows))
                for j, s in enumerate(op.src):
                    if s < 0 or s >= op.rows:
                        raise ValueError("%s: permuteRows src[%d] = %d is out of range" % (plan.name, j, s))
            out = device.create_buffer(total, plan.name)
            dst = temp(total) if permute else out.addr
            off = 0
            for raw, conv, size in zip(raws, convs, sizes):
                if raw.size:
                    ctx.upload(staging, raw)
                    ctx.repack_part(dst + off, staging, raw.size, _CONVERT_CODE[conv], counter)
                off += size
            if permute:
                ctx.repack_permute_rows(out.addr, dst, total, op.rows, op.src)
        overflow = int(ctx.download(counter, 4, np.uint32)[0])
        if overflow:
            out.destroy()
            raise ValueError("%s: %d bf16 value(s) exceed f16 range and were clamped — these weights cannot be "
                             "represented at f16 and the model would run wrong" % (plan.name, overflow))
        return out, overflow
    finally:
        ctx.sync()
        for p in temps:
            ctx.free(p)


# ---------------------------------------------------------------------------------------------------
# checkpoint index, plan keys, whole-model assembly (weight-loader-mlx.ts)
# ---------------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class RecordLoc:
    file: str
    begin: int  # absolute byte range in the shard file
    end: int
    info: TensorInfo


class FileSource:
    """MlxSource over a local directory: range(file, begin, end) and whole(file) (weight-loader-mlx.ts:37-40)."""

    def __init__(self, root):
        self.root = root

    def range(self, file, begin, end):
        import os
        with open(os.path.join(self.root, file), "rb") as f:
            f.seek(begin)
            return f.read(end - begin)

    def whole(self, file):
        import os
        with open(os.path.join(self.root, file), "rb") as f:
            return f.read()


def open_mlx_checkpoint(src):
    """Read model.safetensors.index.json and every shard's header with ranged reads
    (weight-loader-mlx.ts:48-83). Returns {'locate', 'records', 'shards'}."""
    index = json.loads(bytes(src.whole("model.safetensors.index.json")).decode("utf-8"))
    wmap = index["weight_map"]
    shards = sorted(set(wmap.values()))
    headers = {}
    for file in shards:
        lo, hi = struct.unpack("<II", bytes(src.range(file, 0, 8)))
        if hi != 0:
            raise ValueError("%s: safetensors header longer than 4 GB" % file)
        headers[file] = parse_safetensors_header(src.range(file, 0, 8 + lo))

    def locate(record):
        file = wmap.get(record)
        if not file:
            raise KeyError("record not in checkpoint index: %s" % record)
        h = headers[file]
        info = h["tensors"].get(record)
        if info is None:
            raise KeyError("record in index but not in %s's header: %s" % (file, record))
        return RecordLoc(file, h["dataStart"] + info.begin, h["dataStart"] + info.end, info)

    return {"locate": locate, "records": list(wmap.keys()), "shards": shards}


def plan_model(spec, range_=None):
    """Globals first, then every layer of the stage (weight-loader-mlx.ts:93-106)."""
    L0 = range_["start"] if range_ else 0
    L1 = range_["end"] if range_ else spec.layers
    out = [(p, None) for p in plan_global(spec, None, range_)]
    for L in range(L0, L1):
        out += [(p, L) for p in plan_layer(spec, L)]
    return out


def fnv1a32(text):
    """32-bit FNV-1a over the UTF-16 code units of `text` (the reference hashes charCodeAt values)."""
    h = 0x811C9DC5
    for ch in text:
        h = ((h ^ ord(ch)) * 0x01000193) & 0xFFFFFFFF
    return h


def _op_hash(plan):
    op = plan.op
    if op.kind == "permuteRows":
        params = "rows=%d;src=%s" % (op.rows, ",".join(str(s) for s in op.src))
    else:
        params = "bits=%d;group=%d;k=%d;heads=%d;nope=%d;v=%d" % (op.bits, op.group, op.k, op.heads, op.nope, op.v)
    text = "%s;%s;%s" % (op.kind, params, ",".join("%s:%s" % (p.record, p.convert) for p in plan.parts))
    h = fnv1a32(text)
    return "%04x" % (((h >> 16) ^ h) & 0xFFFF)


def plan_key(plan, layer):
    """Stable cache key; op-bearing plans carry a 16-bit FNV-1a hash of the op and its parts so a changed
    preparation invalidates the cached buffer (weight-loader-mlx.ts:117-137)."""
    base = "g.%s" % plan.name if layer is None else "l%d.%s" % (layer, plan.name)
    return "%s.%s" % (base, _op_hash(plan)) if plan.op is not None else base


def build_plan(device, plan, locate, src):
    """Fetch the plan's records by byte range and build its buffer on the device (weight-loader-mlx.ts:146-162)."""
    parts = {}
    for part in plan.parts:
        loc = locate(part.record)
        parts[part.record] = src.range(loc.file, loc.begin, loc.end)
    buf, _ = build_buffer(device, plan, lambda n: parts[n], lambda n: locate(n).info.dtype)
    return buf


def model_bytes(spec, locate):
    src = lambda r: locate(r).end - locate(r).begin
    dt = lambda r: locate(r).info.dtype
    return sum(plan_bytes(p, src, dt) for p, _ in plan_model(spec))


# plan name -> (group, field) of the loaded-weights record (weight-loader-mlx.ts:224-247)
SLOTS = {
    "embed_w": ("root", "embdWeights"), "embed_s": ("root", "embdScales"), "embed_b": ("root", "embdBiases"),
    "lm_head_w": ("root", "lmHeadWeights"), "lm_head_s": ("root", "lmHeadScales"), "lm_head_b": ("root", "lmHeadBiases"),
    "final_norm": ("root", "finalNormGamma"),
    "norm1": ("layer", "normGamma1"), "norm2": ("layer", "normGamma2"),
    "c_attn_w": ("layer", "qkvWeights"), "c_attn_s": ("layer", "qkvScales"), "c_attn_b": ("layer", "qkvBiases"),
    "o_proj_w": ("layer", "oProjWeights"), "o_proj_s": ("layer", "oProjScales"), "o_proj_b": ("layer", "oProjBiases"),
    "q_norm": ("layer", "qNormGamma"), "k_norm": ("layer", "kNormGamma"),
    "mla_q_w": ("mla", "qWeights"), "mla_q_s": ("mla", "qScales"), "mla_q_b": ("mla", "qBiases"),
    "mla_kva_w": ("mla", "kvaWeights"), "mla_kva_s": ("mla", "kvaScales"), "mla_kva_b": ("mla", "kvaBiases"),
    "mla_kva_norm": ("mla", "kvaNormGamma"), "mla_kvb": ("mla", "kvbF16"),
    "gdn_proj_w": ("gdn", "projWeights"), "gdn_proj_s": ("gdn", "projScales"), "gdn_proj_b": ("gdn", "projBiases"),
    "gdn_out_w": ("gdn", "outWeights"), "gdn_out_s": ("gdn", "outScales"), "gdn_out_b": ("gdn", "outBiases"),
    "gdn_conv": ("gdn", "convWeight"), "gdn_norm": ("gdn", "normGamma"),
    "gdn_a_log": ("gdn", "aLog"), "gdn_dt_bias": ("gdn", "dtBias"),
    "moe_gate_proj_w": ("moe", "gateWeights"), "moe_gate_proj_s": ("moe", "gateScales"), "moe_gate_proj_b": ("moe", "gateBiases"),
    "moe_up_proj_w": ("moe", "upWeights"), "moe_up_proj_s": ("moe", "upScales"), "moe_up_proj_b": ("moe", "upBiases"),
    "moe_down_proj_w": ("moe", "downWeights"), "moe_down_proj_s": ("moe", "downScales"), "moe_down_proj_b": ("moe", "downBiases"),
    "router_w": ("moe", "routerWeights"), "router_s": ("moe", "routerScales"), "router_b": ("moe", "routerBiases"),
    "ffn_w": ("layer", "ffnWeights"), "ffn_s": ("layer", "ffnScales"), "ffn_b": ("layer", "ffnBiases"),
    "ffn_down_w": ("layer", "ffnDownWeights"), "ffn_down_s": ("layer", "ffnDownScales"), "ffn_down_b": ("layer", "ffnDownBiases"),
}


def assert_tied_head(weights, spec):
    """A tied lm_head must BE the embedding buffers, not a second load (weight-loader-mlx.ts:289-310)."""
    if not spec.tiedEmbeddings:
        return
    for e, l in (("embdWeights", "lmHeadWeights"), ("embdScales", "lmHeadScales"), ("embdBiases", "lmHeadBiases")):
        if weights.get(e) is not weights.get(l):
            raise ValueError("%s: tied embeddings but %s is not %s — split-stage loaders must alias, not re-load"
                             % (spec.id, l, e))


def assemble_mlx(device, spec, src, locate, range_=None, on_buffer=None):
    """Build every planned buffer on the device and place it in the loaded-weights record by plan name
    (weight-loader-mlx.ts:330-452, without the browser cache and expert-pool hooks)."""
    plans = plan_model(spec, range_)
    root = {"device": device}
    layers = [dict() for _ in range(spec.layers)]
    done = nbytes = 0
    for plan, layer in plans:
        slot = SLOTS.get(plan.name)
        if slot is None:
            raise KeyError("assembleMlx: no LoadedWeights slot for plan '%s'" % plan.name)
        want = plan_bytes(plan, lambda r: locate(r).end - locate(r).begin, lambda r: locate(r).info.dtype)
        buf = build_plan(device, plan, locate, src)
        if buf.size != max(want, 4):
            raise ValueError("assembleMlx: %s built %d B, expected %d B — the plan and the checkpoint disagree; "
                             "refusing to keep a buffer of the wrong size" % (plan_key(plan, layer), buf.size, want))
        group, fld = slot
        if group == "root":
            root[fld] = buf
        elif layer is None:
            raise ValueError("assembleMlx: '%s' is a layer plan with no layer" % plan.name)
        elif group == "layer":
            layers[layer][fld] = buf
        else:
            layers[layer].setdefault(group, {})[fld] = buf
        done += 1
        nbytes += buf.size
        if on_buffer:
            on_buffer(done, len(plans), nbytes)
    root["layers"] = layers
    if spec.tiedEmbeddings:
        root["lmHeadWeights"], root["lmHeadScales"], root["lmHeadBiases"] = (
            root.get("embdWeights"), root.get("embdScales"), root.get("embdBiases"))
    assert_tied_head(root, spec)
    root["initNormGamma"] = layers[range_["start"] if range_ else 0].get("normGamma1")
    return root
