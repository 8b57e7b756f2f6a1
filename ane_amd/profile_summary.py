#!/usr/bin/env python3
"""Turns rocprofv3 CSV output into the short summaries kept under ``profiles/``.

Two kinds of summary, each written by one command so that the text a reader sees and the numbers ``bench.py`` loads
cannot drift apart:

``stats``   a ``--kernel-trace --stats`` run  ->  ``profiles/<name>.md`` (calls, average / min / max duration per kernel)
``pmc``     two ``--pmc`` runs (``FETCH_SIZE``, then ``WRITE_SIZE``)  ->  ``profiles/<name>.md`` and the entry ``<key>`` of
            ``profiles/traffic.json`` (HBM-side megabytes per dispatch of every kernel).  Both counters are scaled by
            what they read for the largest dispatch of ``axpby_kernel<1, 1>``, a plain ``y = alpha*a`` copy whose size
            is given with ``--known-kib``.

Usage (from the repo root, after the rocprofv3 runs have written their CSV files):

    python3 -m ane_amd.profile_summary stats DIR OUT.md --cmd "rocprofv3 ..." [--title T] [--note N]
    python3 -m ane_amd.profile_summary pmc FETCH_DIR WRITE_DIR OUT.md --key KEY --cmd-fetch "..." --cmd-write "..."
                                       [--known-kib K] [--shape TEXT]
"""
import argparse
import collections
import csv
import glob
import json
import os
import re
import shlex
import statistics
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROFILES = os.path.join(ROOT, "profiles")
TRAFFIC_JSON = os.path.join(PROFILES, "traffic.json")
COPY_KERNEL = "axpby_kernel<1, 1>"
PRELUDE = "Command (run from the repo root on the MI355X box, after `cd /tmp && export TMPDIR=/tmp`):"


def made_by():
    """The line of a summary that says which command wrote it from the CSV files."""
    if len(sys.argv) > 1 and sys.argv[1] in ("stats", "pmc"):
        return "Written from the CSV files of that run by `python3 -m ane_amd.profile_summary %s`." % " ".join(
            shlex.quote(a) for a in sys.argv[1:])
    return "Written from the CSV files of that run by `ane_amd/profile_summary.py`."


def short(name):
    """A kernel's demangled name without namespace, return type and argument list."""
    name = name.replace("(anonymous namespace)::", "").replace("void ", "")
    name = re.sub(r"rocprim::ROCPRIM_\d+_NS::", "rocprim::", name)
    name = re.sub(r"\(.*", "", name)
    return name if len(name) <= 96 else name[:93] + "..."


def skipped(name):
    return name.startswith("__amd") or name.startswith("fill_")


def find_csv(directory, suffix):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not hits:
        raise SystemExit("no *%s under %s" % (suffix, directory))
    return hits[0]


def write_stats(directory, out_md, cmd, title, note):
    rows = list(csv.DictReader(open(find_csv(directory, "kernel_stats.csv"))))
    lines = ["# rocprofv3 kernel-trace summary: " + title, "", PRELUDE, "", "    " + cmd, "", made_by(), ""]
    if note:
        lines += [note, ""]
    lines += ["| kernel | calls | avg us | min us | max us | % of GPU time |", "|---|---:|---:|---:|---:|---:|"]
    for r in rows:
        n = short(r["Name"])
        if skipped(n):
            continue
        lines.append("| `%s` | %s | %.1f | %.1f | %.1f | %.2f |" % (n, r["Calls"], float(r["AverageNs"]) / 1e3,
                                                                  float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3,
                                                                  float(r["Percentage"])))
    lines += ["", "`__amd_rocclr_fillBufferAligned` and `fill_*` kernels (buffer zeroing and synthetic-input generation "
                  "before the timed region) are omitted."]
    open(os.path.join(PROFILES, out_md), "w").write("\n".join(lines) + "\n")


def load_counter(path):
    per_kernel = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        per_kernel[short(r["Kernel_Name"])].append(float(r["Counter_Value"]))
    return per_kernel


def write_pmc(fetch_dir, write_dir, out_md, key, cmd_fetch, cmd_write, known_kib, shape):
    f = load_counter(find_csv(fetch_dir, "counter_collection.csv"))
    w = load_counter(find_csv(write_dir, "counter_collection.csv"))
    if COPY_KERNEL not in f or COPY_KERNEL not in w:
        raise SystemExit("the runs hold no dispatch of %s to scale the counters by" % COPY_KERNEL)
    ff = known_kib / max(f[COPY_KERNEL])
    wf = known_kib / max(w[COPY_KERNEL])          # the largest dispatch is the copy of known size
    lines = ["# rocprofv3 PMC: HBM-side traffic per dispatch (FETCH_SIZE, WRITE_SIZE)", "",
             "Two runs, one counter each (run from the repo root on the MI355X box, after `cd /tmp && export TMPDIR=/tmp`):",
             "", "    " + cmd_fetch, "    " + cmd_write, "", made_by(), "",
             "Calibration: `%s` (y = alpha*a over %s fp32) reads and writes exactly %.0f KiB;" % (COPY_KERNEL, shape, known_kib),
             "the counters report %.1f / %.1f KiB for it, so FETCH_SIZE is scaled by %.4f and WRITE_SIZE by %.4f." % (
                 max(f[COPY_KERNEL]), max(w[COPY_KERNEL]), ff, wf),
             "The same figures are entry `%s` of `profiles/traffic.json`, which `bench.py` loads." % key, "",
             "| kernel | dispatches | fetch MB (scaled) | write MB (scaled) | traffic MB |", "|---|---:|---:|---:|---:|"]
    kernels = {}
    for n in f:
        if skipped(n):
            continue
        pick = max if n == COPY_KERNEL else statistics.median      # the copy kernel also runs on smaller tensors
        fm = pick(f[n]) * ff * 1024 / 1e6
        wm = pick(w.get(n, [0.0])) * wf * 1024 / 1e6
        kernels[n] = {"fetch_mb": round(fm, 2), "write_mb": round(wm, 2), "traffic_mb": round(fm + wm, 2),
                      "dispatches": len(f[n])}
        lines.append("| `%s` | %d | %.2f | %.2f | %.2f |" % (n, len(f[n]), fm, wm, fm + wm))
    open(os.path.join(PROFILES, out_md), "w").write("\n".join(lines) + "\n")
    table = {}
    if os.path.exists(TRAFFIC_JSON):
        table = json.load(open(TRAFFIC_JSON))
    table[key] = {"source": "profiles/" + out_md, "fetch_scale": round(ff, 4), "write_scale": round(wf, 4),
                  "kernels": kernels}
    json.dump(table, open(TRAFFIC_JSON, "w"), indent=1, sort_keys=True)
    open(TRAFFIC_JSON, "a").write("\n")


def load_traffic():
    """``profiles/traffic.json`` as a dict (empty when the file is absent)."""
    try:
        return json.load(open(TRAFFIC_JSON))
    except OSError:
        return {}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="kind", required=True)
    s = sub.add_parser("stats")
    s.add_argument("directory"); s.add_argument("out_md")
    s.add_argument("--cmd", required=True); s.add_argument("--title", default="Qwen3-0.6B fused-op sweep (bench.py default workload)")
    s.add_argument("--note", default="")
    p = sub.add_parser("pmc")
    p.add_argument("fetch_dir"); p.add_argument("write_dir"); p.add_argument("out_md")
    p.add_argument("--key", required=True); p.add_argument("--cmd-fetch", required=True); p.add_argument("--cmd-write", required=True)
    p.add_argument("--known-kib", type=float, default=16 * 3072 * 256 * 4 / 1024.0)
    p.add_argument("--shape", default="16x3072x256")
    a = ap.parse_args()
    if a.kind == "stats":
        write_stats(a.directory, a.out_md, a.cmd, a.title, a.note)
    else:
        write_pmc(a.fetch_dir, a.write_dir, a.out_md, a.key, a.cmd_fetch, a.cmd_write, a.known_kib, a.shape)


if __name__ == "__main__":
    main()
