"""The C-ABI library on a machine without a GPU: it loads, exports every symbol
declared in include/ztvm.h, validates descriptors by the generator's legality
rules (src/compiler/shaders/int4_matmul.gen.ts:172-197) and refuses to create a
context instead of falling back to anything."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ztvm.h")).read()
    return sorted(set(re.findall(r"ZTVM_API[^;(]*?\b(ztvm_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(capi):
    lib = capi.load()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.EXPORTS) == names
    assert lib.ztvm_abi_version() == 2


def test_desc_struct_matches_header_layout(capi):
    d = capi.MatmulDesc
    assert ctypes.sizeof(d) == 16 * 4 + 6 * 8
    assert d.out.offset == 64 and d.ids.offset == 64 + 40


def good(capi, **kw):
    base = dict(bits=4, affine=1, out_f32=0, kernel=0, M=1, N=64, k_packed=512, scales_per_row=64,
                out=0x1000, in_=0x2000, scales=0x3000, weights=0x4000, biases=0x5000)
    base.update(kw)
    return capi.MatmulDesc(**base)


def test_validator_accepts_reference_shapes(capi):
    assert capi.validate(good(capi))[0] == 0
    assert capi.validate(good(capi, affine=0, scales_per_row=128, biases=0))[0] == 0
    assert capi.validate(good(capi, bits=3, k_packed=384, scales_per_row=64))[0] == 0
    moe = good(capi, N=512, k_packed=256, scales_per_row=32, slots=8, tokens=16, in_slot_stride=0, out_slot_stride=1024,
               in_tok_stride=2048, out_tok_stride=8 * 1024, ids_stride=8, ids=0x6000, experts=256)
    assert capi.validate(moe)[0] == 0
    assert capi.resolve(moe) == capi.KERNEL_GEMV


@pytest.mark.parametrize("kw,needle", [
    (dict(bits=5), "bits"),
    (dict(bits=3, affine=0, k_packed=384, scales_per_row=128, biases=0), "q3 requires affine"),
    (dict(affine=0, scales_per_row=128, biases=0, slots=8, tokens=1, ids=0x6000, ids_stride=8), "moe requires affine"),
    (dict(k_packed=0), "K_PACKED"),
    (dict(k_packed=4, scales_per_row=1), "group"),          # K=32 is not a multiple of 64
    (dict(scales_per_row=63), "SCALES_PER_ROW"),
    (dict(bits=3, k_packed=385, scales_per_row=64), "3-bit"),
    (dict(N=0), "N"),
    (dict(M=0), "M"),
    (dict(biases=0), "binding 5"),
    (dict(out=0), "binding 0"),
    (dict(in_=0), "binding 1"),
    (dict(scales=0), "binding 2"),
    (dict(weights=0), "binding 3"),
    (dict(weights=0x4004), "aligned"),
    (dict(in_=0x2002), "aligned"),
    (dict(out=0x1001), "misaligned"),
    (dict(slots=8, tokens=2, ids=0, ids_stride=8, out_slot_stride=64), "binding 6"),
    (dict(slots=8, tokens=2, ids=0x6000, ids_stride=4, out_slot_stride=64), "IDS_STRIDE"),
    (dict(slots=8, tokens=2, ids=0x6000, ids_stride=8, M=4, out_slot_stride=64), "M must be 1"),
    (dict(slots=8, tokens=2, ids=0x6000, ids_stride=8, in_slot_stride=4, out_slot_stride=64), "multiples of 8"),
    (dict(slots=8, tokens=2, ids=0x6000, ids_stride=8, out_slot_stride=8), "overlap"),
    (dict(slots=8, tokens=2, ids=0x6000, ids_stride=8, out_slot_stride=64), "experts"),   # the id guard must be armed
    (dict(kernel=9), "kernel"),
    (dict(N=1 << 20), "2 GiB"),                            # 2^20 rows of 512 words = 2 GiB: 32-bit byte offsets end here
])
def test_validator_rejects(capi, kw, needle):
    rc, why = capi.validate(good(capi, **kw))
    assert rc == capi.E_INVALID and needle.lower() in why.lower(), (rc, why)


def test_explicit_kernel_that_cannot_run_is_an_error(capi):
    """Never a silent substitution (pickChunkGemm, src/zero-tvm/engine-core.ts:220-245)."""
    moe = good(capi, N=512, k_packed=256, scales_per_row=32, slots=8, tokens=1, out_slot_stride=512, ids_stride=8,
               ids=0x6000, experts=256, kernel=capi.KERNEL_GEMM)
    rc, why = capi.validate(moe)
    assert rc == capi.E_UNSUPPORTED and "asked for" in why
    with pytest.raises(capi.ZtvmError):
        capi.resolve(moe)


def test_auto_picks_a_family_by_rows(capi):
    """M = 1: per-row GEMV; 2..12: row-group GEMV (to 16 for what the transfer-engine skinny kernel does not take: 3-bit,
    8-bit, K not a multiple of 128); then to 128: weight-streaming matrix-core kernel; above: tile GEMM, or the
    skinny kernel where the tile GEMM's tiles would leave most CUs idle (test_skinny_or_tile_gemm_above_128_rows)."""
    for M, want in ((1, capi.KERNEL_GEMV), (2, capi.KERNEL_ROWS), (12, capi.KERNEL_ROWS), (13, capi.KERNEL_SKINNY),
                    (17, capi.KERNEL_SKINNY), (128, capi.KERNEL_SKINNY)):
        assert capi.resolve(good(capi, M=M)) == want, M
    assert capi.resolve(good(capi, M=16, bits=3, k_packed=384, scales_per_row=64)) == capi.KERNEL_ROWS
    assert capi.resolve(good(capi, M=16, k_packed=24, scales_per_row=3)) == capi.KERNEL_ROWS  # K = 192
    assert capi.resolve(good(capi, M=8, bits=3, k_packed=384, scales_per_row=64)) == capi.KERNEL_ROWS
    assert capi.resolve(good(capi, M=300, N=14336, bits=3, k_packed=384, scales_per_row=64)) == capi.KERNEL_GEMM
    assert capi.resolve(good(capi, M=300, N=14336, bits=3, k_packed=384, scales_per_row=64, out_f32=1)) == capi.KERNEL_SKINNY
    rc, why = capi.validate(good(capi, M=17, kernel=capi.KERNEL_ROWS))
    assert rc == capi.E_UNSUPPORTED and "rows" in why
    # an odd number of scales per row (K = 192) is outside the tile GEMM: the default goes to the streaming kernel
    odd = dict(M=300, k_packed=24, scales_per_row=3)
    assert capi.resolve(good(capi, **odd)) == capi.KERNEL_SKINNY
    assert capi.validate(good(capi, kernel=capi.KERNEL_GEMM, **odd))[0] == capi.E_UNSUPPORTED


def test_skinny_or_tile_gemm_above_128_rows(capi):
    """Above 128 rows the 4-bit family is chosen on an estimate of both kernels' time (rounds of workgroups over 256 CUs
    x steps x time per step; the tile GEMM deals the tiles past its last full round to several workgroups along k).
    The table is the measured winner on MI355X at each point (whole dispatch, us, skinny / gemm):
    K=4096 N=14336: M=256 62 / 65, M=320 77 / 72, M=512 100 / 71, M=2048 393 / 272; K=14336 N=4096: M=512 104 / 94,
    M=1024 172 / 143, M=2048 370 / 254; K=4096 N=6144: M=320 36 / 50, M=512 56 / 49, M=768 78 / 69, M=1024 87 / 71;
    K=2048 N=8192: M=512 37 / 38, M=768 49 / 41, M=1024 63 / 46; K=4096 N=4096: M=256 28 / 34, M=512 34 / 44,
    M=1024 65 / 56, M=2048 115 / 81."""
    S, G = capi.KERNEL_SKINNY, capi.KERNEL_GEMM
    table = [(4096, 14336, ((129, S), (256, S), (320, G), (512, G), (640, G), (1024, G), (2048, G))),
             (14336, 4096, ((512, G), (1024, G), (2048, G))),
             (4096, 6144, ((320, S), (512, G), (768, G), (1024, G), (2048, G))),
             (2048, 8192, ((512, S), (768, G), (1024, G))),
             (4096, 4096, ((129, S), (256, S), (512, S), (1024, G), (2048, G)))]
    for K, N, rows in table:
        for M, want in rows:
            assert capi.resolve(good(capi, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64)) == want, (K, N, M)
    # 3-bit and 8-bit rows and K off a multiple of 128 have the register-path skinny kernel (128-row tiles, about
    # 1 us per step, k-split partials through memory) against the same tile GEMM, which wins at every measured point
    # since it splits k where its tiles are few. Measured, 8-bit / 3-bit, skinny against gemm: K=14336 N=4096: M=256
    # 100 / 87 against 80 / 78, M=512 173 / 155 against 97 / 93, M=1024 327 / 284 against 153 / 143; K=4096 N=4096:
    # M=256 47 / 45 against 35 / 34, M=512 81 / 77 against 45 / 44; K=4096 N=6144: M=256 56 / 52 against 45 / 44,
    # M=512 97 / 91 against 48 / 48; K=4096 N=14336: M=256 91 / 81 against 62 / 62
    for bits, kp in ((8, lambda K: K // 4), (3, lambda K: 3 * K // 32)):
        for K, N, rows in [(14336, 4096, ((256, G), (512, G), (1024, G))), (4096, 4096, ((256, G), (512, G), (1024, G))),
                           (4096, 6144, ((256, G), (512, G))), (4096, 14336, ((192, G), (256, G), (512, G)))]:
            for M, want in rows:
                assert capi.resolve(good(capi, M=M, N=N, bits=bits, k_packed=kp(K), scales_per_row=K // 64)) == want, (bits, K, N, M)
    assert capi.resolve(good(capi, M=512, N=4096, affine=0, biases=0, k_packed=520, scales_per_row=130)) == G  # K = 4160
    # an explicit request is honoured either way
    big = dict(M=512, N=4096, k_packed=512, scales_per_row=64)
    assert capi.resolve(good(capi, kernel=G, **big)) == G and capi.resolve(good(capi, **big)) == S


def test_family_estimate_is_sane_on_random_shapes(capi):
    """Whatever the shape, more than 128 rows resolve to one of the two matrix-core families without an error; a grid
    of full tiles of the tile GEMM that fills whole rounds of the 256 CUs is never given away; a single column tile is, at moderate M and K."""
    import random
    rnd = random.Random(7)
    S, G = capi.KERNEL_SKINNY, capi.KERNEL_GEMM
    for _ in range(400):
        M = rnd.choice([129, 200, 256, 257, 400, 512, 1000, 2048, 5000, 16384])
        K = 128 * rnd.randint(1, 256)
        N = rnd.choice([8, 64, 120, 128, 1000, 4096, 6144, 8192, 14336, 32000, 65536])
        fam = capi.resolve(good(capi, M=M, N=N, k_packed=K // 8, scales_per_row=K // 64))
        assert fam in (S, G), (M, N, K, fam)
        tiles = -(-M // 256) * -(-N // 128)
        if M > 256 and M % 256 == 0 and tiles % 256 == 0:
            assert fam == G, (M, N, K)
        if N <= 128 and 1024 <= K <= 8192 and M <= 2048:   # (long rows: the skinny family's copy of the activations weighs in)
            assert fam == S, (M, N, K)


def test_unchecked_experts_is_an_explicit_choice(capi):
    moe = dict(N=512, k_packed=256, scales_per_row=32, slots=8, tokens=1, out_slot_stride=512, ids_stride=8, ids=0x6000)
    assert capi.validate(good(capi, **moe))[0] == capi.E_INVALID
    assert capi.validate(good(capi, experts=capi.EXPERTS_UNCHECKED, **moe))[0] == 0


def test_rows_too_long_for_the_gemv_staging_are_refused(capi):
    """The GEMV family stages the activation row in LDS (160 KB): a dispatch that has no other family
    (M = 1 explicit GEMV, MoE) and a longer row is an error before any launch, dense rows go elsewhere."""
    K = 1 << 17
    big = dict(k_packed=K // 8, scales_per_row=K // 64, N=64)
    rc, why = capi.validate(good(capi, kernel=capi.KERNEL_GEMV, **big))
    assert rc == capi.E_UNSUPPORTED and "LDS" in why, why
    K = 65536  # 139264 B of staging: fits
    assert capi.validate(good(capi, kernel=capi.KERNEL_GEMV, k_packed=K // 8, scales_per_row=K // 64, N=64))[0] == 0


def test_no_device_is_a_loud_error(capi):
    import subprocess, sys
    code = ("import importlib,sys; sys.path.insert(0,%r); c=importlib.import_module('zero-tvm_amd.host.capi');\n"
            "try:\n  c.Context(0); print('CREATED')\nexcept c.ZtvmError as e:\n  print('ERR', e.code)") % ROOT
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=120).stdout
    assert "ERR -4" in out, out


def test_failed_create_hands_out_nothing(capi):
    """Every failing exit of ztvm_create leaves *out null (so a caller that ignores the code cannot use or leak a
    half-built context) and says why; a null out pointer is refused."""
    import subprocess, sys
    code = ("import ctypes as C, importlib, sys; sys.path.insert(0,%r)\n"
            "c = importlib.import_module('zero-tvm_amd.host.capi'); L = c.load()\n"
            "for i in range(50):\n"
            "  h = C.c_void_p(0xDEAD)\n"
            "  rc = L.ztvm_create(0, C.byref(h)); assert rc == -4 and not h.value, (rc, h.value)\n"
            "  assert b'no HIP device' in L.ztvm_last_error(None)\n"
            "assert L.ztvm_create(0, None) == -1\n"
            "L.ztvm_destroy(None); print('FINE')") % ROOT
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=120)
    assert "FINE" in r.stdout, r.stdout + r.stderr
