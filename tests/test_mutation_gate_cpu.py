"""The parity gate must see a wrong kernel (reference: scripts/mutation-gate.mjs, BENCH.md:1694-1701).
On configs[0] (K=2048, N=8192, int4 affine g64) the fp32-accumulated reference of a kernel with a
shifted scale group, a dropped bias or a swapped nibble order is compared with the correct one under
the contract's metric max |y-ref| / (|ref| + 1e-2) < 1e-2 and under the reference test's own
(eps 1e-3, bar 2e-2): each mutation has to fail both, in both bias regimes, and the f16 rounding of
the correct result has to pass them."""
import numpy as np
import pytest

from .util import mutations, rel_err

K, N = 2048, 8192


@pytest.mark.parametrize("regime", ["A", "B"])
def test_gate_rejects_every_mutation(synth, oracle, regime):
    x, w, s = synth.activations(1, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s, regime)
    ref = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, w, s, b, threads=8)[0]
    rounded = ref.astype(np.float16).astype(np.float64)   # what a correct kernel stores
    assert rel_err(rounded, ref, 1e-2) < 1e-2 and rel_err(rounded, ref, 1e-3) < 2e-2
    for name, (mw, ms, mb) in mutations(w, s, b).items():
        wrong = oracle.gemm(oracle.MODE_FORMULA_F32, 4, True, 1, N, K, x, mw, ms, mb, threads=8)[0]
        wrong = wrong.astype(np.float16).astype(np.float64)
        e2, e3 = rel_err(wrong, ref, 1e-2), rel_err(wrong, ref, 1e-3)
        print("%-28s regime %s: %.3g (eps 1e-2)  %.3g (eps 1e-3)" % (name, regime, e2, e3))
        assert e2 > 10 * 1e-2, (name, e2)    # an order of magnitude past the bar, not a near miss
        assert e3 > 10 * 2e-2, (name, e3)
        # and not through one lucky element: half of all outputs are off by more than the bar
        assert np.median(np.abs(wrong - ref) / (np.abs(ref) + 1e-2)) > 1e-2, name
