"""MI355X-native int4/int3 group-quantized dequant-matmul path of zero-tvm.

The directory name carries a hyphen, so import it with
``importlib.import_module("zero-tvm_amd")``. Sub-modules:

  host.capi    ctypes binding of the C ABI (lib/libztvm_hip.so)
  host.engine  mirror of the reference's dispatch surface (uniformBuf / bg / dispatch)
  host.synth   seeded synthetic tensors of the benchmark configurations
  host.gemm_tune  boot-time choice of the prefill GEMM by measurement (policy of the reference's gemm-tune.ts)
  build        hipcc build recipe
"""
from .host import capi  # noqa: F401

__all__ = ["capi"]
