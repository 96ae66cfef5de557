"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)


def test_flags_of_the_driver_contract_exist():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--workload"):
        assert flag in r.stdout
    for w in ("wkv6", "wkv6_state", "wkv5", "rwkv7", "wkv4", "timex"):
        assert w in r.stdout
