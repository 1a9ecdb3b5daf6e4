"""Contexts come and go without leaving device memory behind: ztvm_create gives back what it holds on every failing
exit, ztvm_destroy frees the stream, the scratch pool and the arrival counters of the tile GEMM's k split. The
reference's counterpart is the lifetime of a GPUDevice and its buffers (src/zero-tvm/engine-core.ts:1135-1190)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def free_bytes():
    # the runtime the library itself is linked to, by the path it was loaded from (a torch in the same process
    # brings a second copy of its own, which is not the one that holds this library's allocations)
    with open("/proc/self/maps") as maps:
        paths = sorted({line.split()[-1] for line in maps if "libamdhip64.so" in line and "torch" not in line})
    assert paths, "the HIP runtime is not mapped"
    hip = C.CDLL(paths[0])
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_device_out_of_range_hands_out_nothing(ctx, capi):
    L = capi.load()
    h = C.c_void_p(0xDEAD)
    assert L.ztvm_create(99, C.byref(h)) == capi.E_INVALID and not h.value
    assert b"out of range" in L.ztvm_last_error(None)


def test_contexts_leave_no_device_memory_behind(ctx, capi, synth):
    """Thirty contexts, each of which grows its scratch pool with one split GEMM before it goes: free device memory
    afterwards is where it was (within the runtime's own slack)."""
    M, N, K = 512, 1024, 4096
    A, w, s = synth.activations(M, K), synth.packed_weights(N, K), synth.scales(N, K)
    b = synth.biases(N, K, s)

    def once():
        with capi.Context(0) as c:
            ptrs = [c.alloc(x.nbytes) for x in (A, w, s, b)] + [c.alloc(M * N * 2)]
            for p, x in zip(ptrs, (A, w, s, b)):
                c.upload(p, x)
            c.matmul(capi.MatmulDesc(bits=4, affine=1, kernel=capi.KERNEL_GEMM, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64,
                                     in_=ptrs[0], weights=ptrs[1], scales=ptrs[2], biases=ptrs[3], out=ptrs[4]))
            y = c.download(ptrs[4], M * N * 2, np.uint16)
            for p in ptrs:
                c.free(p)
            return y

    first = once()
    before = free_bytes()
    for _ in range(30):
        assert np.array_equal(once(), first)
    # a leak would be 30 x (4 MiB of scratch pool + 8 MiB grown for the split) = 360 MiB
    assert before - free_bytes() < (64 << 20), "contexts leak device memory"
