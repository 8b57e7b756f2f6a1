"""The parts of bench.py's command-line contract that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def test_help_lists_the_workloads_and_the_contract_flags():
    r = _run("--help")
    assert r.returncode == 0
    for word in ("--gpus", "--steps", "--warmup", "--workload", "stories110m", "embed", "optimizer", "aux", "host"):
        assert word in r.stdout, word
