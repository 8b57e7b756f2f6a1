"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the headers
declare, the ctypes table matches the header, and entry points fail cleanly without a GPU."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HDR = os.path.join(ROOT, "include", "mi355_bridge.h")


def declared_symbols():
    text = open(HDR).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import ane_amd.bridge as br
    syms = declared_symbols()
    assert len(syms) >= 45
    for s in syms:
        assert hasattr(br.lib, s), "libmi355_ops.so lacks " + s
    assert sorted(br.SIGNATURES) == syms, "ctypes table and header disagree"
    # nothing but the C-ABI is exported
    out = subprocess.run(["nm", "-D", "--defined-only", br.LIB_PATH], capture_output=True, text=True).stdout
    exported = [l.split()[-1] for l in out.splitlines() if " T " in l]
    extra = [e for e in exported if not e.startswith("mi355_") and not e.startswith("_")]
    assert not extra, extra


def test_cpu_ops_header_compiles_as_c99(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#define VOCAB 32000\n#include "mi355_cpu_ops.h"\nint main(void){return 0;}\n')
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-Wno-unused-function", "-fsyntax-only", "-I",
                        os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_entry_points_fail_cleanly_without_a_gpu():
    """On a host with no gfx950 device every call returns an error and touches nothing."""
    import ane_amd.bridge as br
    if br.lib.mi355_init() == 0:
        return      # a GPU is present: the error path is covered by the GPU tests
    assert "no" in br.last_error().lower() or "gfx950" in br.last_error()
    y = np.full(8, 3.0, np.float32)
    assert br.lib.mi355_rmsnorm_fwd_dev(y.ctypes.data, y.ctypes.data, y.ctypes.data, 2, 4, 1, 1e-5) == -1
    assert br.lib.mi355_sync() == -1
    assert br.lib.mi355_buf_alloc(64) is None
    br.lib.mi355_rmsnorm(y.ctypes.data, y.ctypes.data, y.ctypes.data, 2, 4)
    assert np.all(y == 3.0)
    br.lib.mi355_shutdown()


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_product_does_not_touch_the_oracle():
    """No file of the shipped package or the public headers refers to the CPU oracle."""
    bad = []
    for base in ("ane_amd", "include"):
        for dp, _, fns in os.walk(os.path.join(ROOT, base)):
            if "build" in dp.split(os.sep) or "__pycache__" in dp:
                continue
            for fn in fns:
                if fn.endswith((".py", ".h", ".hip", ".c", ".cpp")):
                    t = open(os.path.join(dp, fn), errors="ignore").read()
                    if re.search(r"\boracle\b|liboracle|orc_", t):
                        bad.append(os.path.join(dp, fn))
    assert not bad, bad
