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


def test_traffic_figures_come_from_the_tracked_profile_summaries():
    """bench.py holds no HBM-traffic number of its own: every kernel it prices is a row of profiles/traffic.json,
    and that file agrees with the tables of the profile summaries written by the same command."""
    import json
    import re
    sys.path.insert(0, ROOT)
    import bench
    table = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    for key, ops in (("qwen3_sweep", bench.OP_KERNELS), ("embed_config2", bench.EMBED_KERNELS)):
        rows = table[key]["kernels"]
        md = open(os.path.join(ROOT, table[key]["source"])).read()
        for op, kernels in ops.items():
            assert bench.traffic_bytes(key, kernels) > 0, op
            for k, _ in kernels:
                m = re.search(r"\| `%s` \| \d+ \| ([\d.]+) \| ([\d.]+) \| ([\d.]+) \|" % re.escape(k), md)
                assert m, (key, k)
                assert abs(float(m.group(3)) - rows[k]["traffic_mb"]) <= 0.011, (key, k)
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert not re.search(r"TRAFFIC_BYTES\s*=", src)
