"""The tool that turns rocprofv3 CSV output into profiles/*.md and profiles/traffic.json, on synthetic CSV files."""
import csv
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from ane_amd import profile_summary as P


def _counter_csv(path, name, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
        for i, (kernel, value) in enumerate(rows):
            w.writerow([i + 1, kernel, name, value])


def test_kernel_names_are_shortened():
    assert P.short("void (anonymous namespace)::swiglu_bwd_kernel<1>(float*, float*, unsigned long)") == "swiglu_bwd_kernel<1>"
    assert P.short("void (anonymous namespace)::axpby_kernel<1, 1>(float*, float const*)") == P.COPY_KERNEL
    assert P.skipped("__amd_rocclr_fillBufferAligned") and P.skipped("fill_normal_kernel") and not P.skipped("gather_kernel<true>")


def test_counter_runs_become_a_table_and_a_json_entry(tmp_path, monkeypatch):
    """Both counters are scaled by what they read for the copy of known size (its largest dispatch); a kernel's figure
    is the median over its dispatches; the markdown table and the JSON entry hold the same numbers."""
    monkeypatch.setattr(P, "PROFILES", str(tmp_path))
    monkeypatch.setattr(P, "TRAFFIC_JSON", str(tmp_path / "traffic.json"))
    copy = "void (anonymous namespace)::axpby_kernel<1, 1>(float*, float const*, float const*, float, unsigned long)"
    k = "void (anonymous namespace)::toy_kernel<4>(float*, float const*)"
    # FETCH_SIZE under-reports by two, WRITE_SIZE is exact; the copy also runs once on a smaller tensor
    _counter_csv(str(tmp_path / "f" / "x_counter_collection.csv"), "FETCH_SIZE",
                 [(copy, 500.0), (copy, 100.0), (k, 250.0), (k, 260.0), (k, 1000.0), ("__amd_rocclr_fillBufferAligned", 7.0)])
    _counter_csv(str(tmp_path / "w" / "x_counter_collection.csv"), "WRITE_SIZE",
                 [(copy, 1000.0), (copy, 200.0), (k, 125.0), (k, 125.0), (k, 125.0)])
    P.write_pmc(str(tmp_path / "f"), str(tmp_path / "w"), "toy.md", "toy", "cmd-f", "cmd-w", 1000.0, "1x1")
    table = json.load(open(tmp_path / "traffic.json"))["toy"]
    assert table["fetch_scale"] == 2.0 and table["write_scale"] == 1.0 and table["source"] == "profiles/toy.md"
    row = table["kernels"]["toy_kernel<4>"]
    assert row["dispatches"] == 3
    assert abs(row["fetch_mb"] - 260.0 * 2 * 1024 / 1e6) < 0.006 and abs(row["write_mb"] - 125.0 * 1024 / 1e6) < 0.006
    assert abs(table["kernels"][P.COPY_KERNEL]["traffic_mb"] - 2 * 1000.0 * 1024 / 1e6) < 0.011
    assert "__amd_rocclr_fillBufferAligned" not in table["kernels"]
    md = open(tmp_path / "toy.md").read()
    assert "cmd-f" in md and "cmd-w" in md and "| `toy_kernel<4>` | 3 | %.2f | %.2f | %.2f |" % (
        row["fetch_mb"], row["write_mb"], row["fetch_mb"] + row["write_mb"]) in md
    # a second key joins the same file
    P.write_pmc(str(tmp_path / "f"), str(tmp_path / "w"), "toy2.md", "toy2", "a", "b", 1000.0, "1x1")
    assert set(json.load(open(tmp_path / "traffic.json"))) == {"toy", "toy2"}


def test_kernel_stats_become_a_table(tmp_path, monkeypatch):
    monkeypatch.setattr(P, "PROFILES", str(tmp_path))
    os.makedirs(tmp_path / "run")
    with open(tmp_path / "run" / "sweep_kernel_stats.csv", "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(["Name", "Calls", "TotalDurationNs", "AverageNs", "Percentage", "MinNs", "MaxNs", "StdDev"])
        w.writerow(["void (anonymous namespace)::toy_kernel<4>(float*)", 10, 414000, 41400.0, 60.0, 40000, 46000, 1.0])
        w.writerow(["fill_normal_kernel(float*, unsigned long)", 3, 3000, 1000.0, 1.0, 900, 1100, 1.0])
    P.write_stats(str(tmp_path / "run"), "stats.md", "the command", "a title", "a note")
    md = open(tmp_path / "stats.md").read()
    assert "the command" in md and "a title" in md and "a note" in md
    assert "| `toy_kernel<4>` | 10 | 41.4 | 40.0 | 46.0 | 60.00 |" in md and "fill_normal_kernel(" not in md
