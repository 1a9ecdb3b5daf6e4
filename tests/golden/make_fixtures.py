"""Writes tests/golden/format_vectors.json: small known-answer vectors for the
packed formats and the seeded generator, produced WITHOUT the oracle and
without the reference (pure Python integers + numpy), so the oracle can be
checked against an independent second formulation.

  python tests/golden/make_fixtures.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def mulberry32(seed, n):
    """Closed form of the PRNG in the reference's kernel tests, in Python ints."""
    out, s = [], seed & 0xFFFFFFFF
    for _ in range(n):
        s = (s + 0x6D2B79F5) & 0xFFFFFFFF
        t = ((s ^ (s >> 15)) * (1 | s)) & 0xFFFFFFFF
        t = ((t + (((t ^ (t >> 7)) * (61 | t)) & 0xFFFFFFFF)) & 0xFFFFFFFF) ^ t
        out.append(((t ^ (t >> 14)) & 0xFFFFFFFF) / 4294967296.0)
    return out


def bits_le(words):
    """LSB-first bit array of little-endian u32 words (numpy.unpackbits formulation)."""
    return np.unpackbits(np.asarray(words, "<u4").view(np.uint8), bitorder="little")


def main():
    g = np.random.default_rng(12345)
    fx = {}
    fx["mulberry32_seed1"] = mulberry32(1, 16)
    fx["mulberry32_seed35"] = mulberry32(35, 8)
    # 3-bit rows: K=256 (24 words); values via unpackbits, value k = bits [3k,3k+3)
    rows3 = g.integers(0, 1 << 32, size=(4, 24), dtype=np.uint32)
    vals3 = []
    for r in rows3:
        b = bits_le(r).reshape(-1, 3)
        vals3.append((b[:, 0] + 2 * b[:, 1] + 4 * b[:, 2]).astype(int).tolist())
    fx["q3_words"] = rows3.tolist()
    fx["q3_values"] = vals3
    # 4-bit rows: K=128 (16 words); byte-wise even/odd formulation
    rows4 = g.integers(0, 1 << 32, size=(4, 16), dtype=np.uint32)
    vals4 = []
    for r in rows4:
        by = np.asarray(r, "<u4").view(np.uint8)
        v = np.empty(by.size * 2, int)
        v[0::2] = by & 15        # low nibble of each byte = even k
        v[1::2] = by >> 4        # high nibble = odd k
        vals4.append(v.tolist())
    fx["q4_words"] = rows4.tolist()
    fx["q4_values"] = vals4
    # f16 conversion spot values incl. ties, subnormals, overflow (numpy float16 is IEEE RNE)
    f = np.array([0.0, 1.0, -2.5, 65504.0, 65520.0, 65519.996, 1e-8, 5.9604645e-8, 2.9802322e-8, 2.98023224e-8 * 1.0001,
                  6.1035156e-05, 6.097555e-05, 1.0009765625, 1.00048828125, 1.00146484375, 0.333333, -1e-10, 3.0e38], np.float32)
    fx["f32_in_bits"] = f.view(np.uint32).tolist()
    with np.errstate(over="ignore"):
        fx["f16_out_bits"] = f.astype(np.float16).view(np.uint16).tolist()
    with open(os.path.join(HERE, "format_vectors.json"), "w") as fh:
        json.dump(fx, fh, indent=0)
    print("wrote", os.path.join(HERE, "format_vectors.json"))


if __name__ == "__main__":
    main()
