"""Build recipe for libztvm_hip.so (hipcc, gfx950 only) and the oracle.

`python zero-tvm_amd/build.py` compiles every HIP source under csrc/ into
object files in parallel and links them into zero-tvm_amd/lib/libztvm_hip.so.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libztvm_hip.so")
SOURCES = ["ztvm_api.hip", "gemv.hip", "gemv_stream.hip", "gemv_rows.hip", "skinny.hip", "skinny_dma.hip", "gemm.hip", "dequant.hip", "block_ops.hip", "repack.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off", "-fno-gpu-rdc",
    # packed-fp32 VALU forms are switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def _compile(src, extra):
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, extra=()):
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(lambda s: _compile(s, list(extra)), SOURCES))
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode:
        raise RuntimeError("link failed:\n" + r.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
