"""The scratch buffer's lifetime rules on the CPU: a buffer whose address a live command buffer may
hold is never freed by a later, larger dispatch (zero-tvm_amd/csrc/scratch_pool.h). The C++ driver
uses a counting allocator in place of hipMalloc / hipFree."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_scratch_pool_bookkeeping(tmp_path):
    exe = str(tmp_path / "scratch_pool_test")
    src = os.path.join(ROOT, "tests", "cpp", "scratch_pool_test.cc")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-fsanitize=address,undefined", "-o", exe, src],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and "ALL OK" in run.stdout, run.stdout + run.stderr
    assert "FAIL" not in run.stdout
