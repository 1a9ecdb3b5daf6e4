"""Seeded synthetic tensors in the reference's weight-buffer formats.

Layouts (paths relative to the reference's root):
  weights  [N, K*bits/32] u32, row-major; 4-bit nibbles LSB-first, 3-bit rows
           one LSB-first bitstream (src/compiler/shaders/int4_matmul.gen.ts:115-133, :157-167)
  scales   [N, K/G] f16, biases [N, K/G] f16 (affine only); G = 64 affine, 32 symmetric
  x / A    [M, K] f16
MoE stacks put the expert axis first ([E, N, ...], src/zero-tvm/weight-loader.ts:995-1003).

Every tensor has its own seeded stream so CPU and GPU sides can regenerate
any one of them independently.
"""
import numpy as np

SEEDS = {"x": 1, "w": 2, "s": 3, "b": 4, "ids": 5}


def _rng(kind, salt=0):
    return np.random.Generator(np.random.Philox(key=SEEDS[kind] + 1000 * salt))


def activations(M, K, salt=0):
    """f16 bits [M,K], N(0,1)."""
    return _rng("x", salt).standard_normal((M, K), dtype=np.float32).astype(np.float16).view(np.uint16)


def packed_weights(N, K, bits=4, salt=0, experts=None):
    """Uniform random values; for 4 bits whole random words, for 3 bits a packed bitstream."""
    shape = (N,) if experts is None else (experts, N)
    # uniformly random bits are uniformly random 4-bit (or 3-bit) values
    return _rng("w", salt).integers(0, 1 << 32, size=shape + (K * bits // 32,), dtype=np.uint32)


def scales(N, K, affine=True, salt=0, experts=None, lo=0.005, hi=0.02):
    G = 64 if affine else 32
    shape = ((N,) if experts is None else (experts, N)) + (K // G,)
    return _rng("s", salt).uniform(lo, hi, size=shape).astype(np.float32).astype(np.float16).view(np.uint16)


def biases(N, K, scale_bits, regime="A", salt=0, experts=None):
    """Regime A: U(-0.05, 0.05) as in the reference's kernel tests (tests/kernels/run.mjs:85).
    Regime B: MLX-like centred bias -7.5*s*(1+U(-0.1,0.1)), the cancellation stress case."""
    shape = ((N,) if experts is None else (experts, N)) + (K // 64,)
    g = _rng("b", salt)
    if regime == "A":
        b = g.uniform(-0.05, 0.05, size=shape)
    else:
        s = scale_bits.view(np.float16).astype(np.float64).reshape(shape)
        b = -7.5 * s * (1.0 + g.uniform(-0.1, 0.1, size=shape))
    return b.astype(np.float32).astype(np.float16).view(np.uint16)


def topk_ids(tokens, slots, experts, salt=0):
    """Per token `slots` distinct expert ids drawn uniformly (top-k ids are distinct by construction)."""
    g = _rng("ids", salt)
    return np.stack([g.permutation(experts)[:slots] for _ in range(tokens)]).astype(np.uint32)


def weight_bytes(N, K, bits=4, affine=True):
    """Algorithmic bytes of one weight matrix: packed words + f16 scales (+ f16 biases).
    Same accounting as the reference's benches (scripts/kernel-ab-ours.mjs:74, :134-140)."""
    G = 64 if affine else 32
    return N * (K * bits // 32) * 4 + N * (K // G) * 2 * (2 if affine else 1)
