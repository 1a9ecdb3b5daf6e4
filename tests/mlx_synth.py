"""A synthetic MLX-style safetensors checkpoint for the loader tests: every record a model's plans name,
at small dimensions, split over two shards with an index file. Test data only; written with numpy."""
import json
import os
import struct

import numpy as np

ITEM = {"U32": 4, "BF16": 2, "F16": 2, "F32": 4}


def write_safetensors(path, tensors):
    """tensors: {name: (dtype string, shape, bytes)} -> one safetensors file."""
    header, off = {"__metadata__": {"format": "mlx"}}, 0
    for name, (dtype, shape, data) in tensors.items():
        assert len(data) == int(np.prod(shape)) * ITEM[dtype], name
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + len(data)]}
        off += len(data)
    text = json.dumps(header).encode("utf-8")
    text += b" " * ((8 - len(text) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for _, (_, _, data) in tensors.items():
            f.write(data)


def record_shape(record, dims):
    """(dtype, shape) of a record from its name. dims["matrices"] maps a name fragment (first match wins) to
    (rows, K, bits): bits 4 / 8 are MLX-affine [rows, K*bits/32] u32 with [rows, K/64] scales and biases,
    bits 16 is a plain float matrix; expert stacks under switch_mlp get a leading expert axis. Everything
    else is a vector."""
    for frag, (rows, K, bits) in dims["matrices"].items():
        if frag in record:
            lead = (dims["experts"],) if "switch_mlp" in record else ()
            if not record.endswith(".weight"):
                return dims["float"], lead + (rows, K // 64)
            if bits == 16:
                return dims["float"], lead + (rows, K)
            return "U32", lead + (rows, K * bits // 32)
    if record.endswith("A_log") or record.endswith("dt_bias"):
        return dims.get("alog", dims["float"]), (dims["gdn_heads"],)
    if "conv1d" in record:
        return dims["float"], (dims["conv_rows"], 4, 1)
    if "kv_a_layernorm" in record:
        return "F16", (dims["kv_lora"],)
    return dims["float"], (dims["d"],)


def random_bytes(rng, dtype, shape):
    n = int(np.prod(shape))
    if dtype == "U32":
        return rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).tobytes()
    vals = (rng.standard_normal(n) * 0.05).astype(np.float32)
    vals[: min(n, 3)] = [3e-5, -1e-6, 1.5][: min(n, 3)]      # f16-subnormal-band values survive the conversion
    if dtype == "F32":
        return vals.tobytes()
    if dtype == "F16":
        return vals.astype(np.float16).tobytes()
    u = vals.view(np.uint32)
    lo, hi = u & 0xFFFF, u >> 16
    hi = hi + ((lo > 0x8000) | ((lo == 0x8000) & ((hi & 1) == 1)))
    return (hi & 0xFFFF).astype(np.uint16).tobytes()


def write_checkpoint(root, records, dims, seed=1):
    """Two shards + model.safetensors.index.json. Returns {record: (dtype, shape, bytes)}."""
    rng = np.random.default_rng(seed)
    made = {}
    for r in sorted(set(records)):
        dtype, shape = record_shape(r, dims)
        made[r] = (dtype, shape, random_bytes(rng, dtype, shape))
    names = list(made)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    wmap = {}
    for file, rs in shards.items():
        write_safetensors(os.path.join(root, file), {r: made[r] for r in rs})
        wmap.update({r: file for r in rs})
    with open(os.path.join(root, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": wmap}, f)
    return made
