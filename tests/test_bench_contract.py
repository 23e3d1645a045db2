"""Host-only checks of bench.py's command line: the parts of its contract that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run_bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_help_names_the_contract_flags():
    r = run_bench("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--shapes", "--algo"):
        assert flag in r.stdout
