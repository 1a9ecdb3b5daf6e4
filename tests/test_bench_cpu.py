"""bench.py on a machine without a GPU: it measures one GPU and says so when asked for more, and without a device it
stops with the library's error instead of timing anything else (there is no CPU path to fall back to)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args, **env):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300,
                          env=dict(os.environ, **env))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0 and "ONE GPU" in r.stderr and not r.stdout.strip()


def test_no_device_is_an_error_not_a_cpu_run():
    r = run("--steps", "1", "--warmup", "0", HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    assert r.returncode != 0 and "no HIP device visible" in r.stderr
    assert not any(line.startswith("{") for line in r.stdout.splitlines()), "a result line without a GPU"
