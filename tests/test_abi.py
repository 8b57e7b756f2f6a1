"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the headers
declare, the ctypes table matches the header, and entry points fail cleanly without a GPU."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

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


@pytest.mark.parametrize("loop", ["dynamic_loop", "static_loop"])
def test_reference_call_sites_compile_against_the_cpu_ops_header(tmp_path, loop):
    """tests/callsites/*.c hold every CPU-op call of the reference's loops with the loops' own argument lists
    (both adam_update forms, the VocabMap functions); they must compile as C99 with -Wall -Werror against
    include/mi355_cpu_ops.h and link against the library."""
    import ane_amd.bridge as br
    src = os.path.join(ROOT, "tests", "callsites", loop + ".c")
    exe = str(tmp_path / loop)
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-Wno-unused-function", "-I",
                        os.path.join(ROOT, "include"), src, "-L", os.path.dirname(br.LIB_PATH), "-lmi355_ops", "-lm",
                        "-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    # the same unit as C++ and as Objective-C-free C11 with pedantic warnings
    r = subprocess.run(["g++", "-x", "c++", "-std=c++17", "-Wall", "-Werror", "-Wno-unused-function", "-fsyntax-only",
                        "-I", os.path.join(ROOT, "include"), src], capture_output=True, text=True)
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


def test_every_rmsnorm_shape_has_a_kernel():
    """The tile picker may only choose tiles that are instantiated: every channel count from 1 to 4200, at column
    counts on both sides of its thresholds (including 128 x 256 columns, where 16-lane strips of 512 threads win),
    for all three entry points, aligned or not, and under every tuning knob."""
    import ane_amd.bridge as br
    tile = (ctypes.c_int * 5)()
    shapes = [(256, 1), (256, 16), (256, 32), (256, 128), (256, 300), (64, 2), (37, 2), (20, 3), (4, 1), (1024, 64)]
    seen = set()
    try:
        for lpr, thr in [(0, 0)] + [(l, t) for l in (4, 8, 16) for t in (256, 512, 1024)]:
            br.lib.mi355_tune_set(b"rms_lpr", lpr); br.lib.mi355_tune_set(b"rms_threads", thr)
            for C in list(range(1, 1100)) + list(range(1100, 4200, 37)) + [5000, 8192, 16384]:
                if (lpr or thr) and C % 7:
                    continue
                for S, batch in shapes:
                    for op in (0, 1, 2):
                        for aligned in (1, 0):
                            assert br.lib.mi355_rmsnorm_tile(op, C, S, batch, aligned, tile) == 0, \
                                (op, C, S, batch, aligned, lpr, thr, list(tile), br.last_error())
                            seen.add(tuple(tile))
    finally:
        br.lib.mi355_tune_set(b"rms_lpr", 0); br.lib.mi355_tune_set(b"rms_threads", 0)
    assert (4, 16, 512, 8, 0) in seen or (4, 16, 512, 16, 0) in seen  # the tile that used to be missing
    assert br.lib.mi355_rmsnorm_tile(0, 1024, 256, 16, 1, tile) == 0 and tuple(tile) == (4, 16, 1024, 4, 4)   # Qwen3: 4 x 256 rows
    assert br.lib.mi355_rmsnorm_tile(1, 768, 256, 1, 1, tile) == 0 and tile[4] == 8                           # Stories110M
    assert br.lib.mi355_rmsnorm_tile(0, 1024, 256, 64, 1, tile) == 0 and tile[4] == 0                         # enough columns
    assert br.lib.mi355_rmsnorm_tile(3, 8, 8, 1, 1, None) == -1


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


# ---- checkpoint header and index: host-only code, no GPU needed ----
CK_GQA = dict(layers=3, vocab=101, dim=64, hidden=160, heads=4, kv_heads=2, head_dim=24, q_dim=96, kv_dim=48, seq=32)
CK_MHA = dict(layers=2, vocab=77, dim=48, hidden=128, heads=4, kv_heads=4, head_dim=12, q_dim=48, kv_dim=48, seq=16)


def _locate(br, hdr, layer, tensor, part):
    off, cnt = ctypes.c_uint64(), ctypes.c_uint64()
    assert br.lib.mi355_ckpt_locate(ctypes.byref(hdr), layer, tensor, part, ctypes.byref(off), ctypes.byref(cnt)) == 0
    return off.value, cnt.value


def test_checkpoint_header_and_index_match_the_reference_layout(tmp_path):
    import ane_amd.bridge as br
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import helpers as H
    assert ctypes.sizeof(br.CkptHdr) == 96 == len(H.ckpt_header_bytes(CK_GQA, 4))
    for cfg, version in ((CK_GQA, 4), (CK_MHA, 2)):
        path = str(tmp_path / ("ck%d.bin" % version))
        tensors = H.ckpt_write_like_reference(path, cfg, version)
        hdr = br.CkptHdr()
        assert br.lib.mi355_ckpt_read_header(path.encode(), ctypes.byref(hdr)) == 0
        assert (hdr.magic, hdr.version, hdr.step, hdr.total_steps, hdr.adam_t) == (H.CKPT_MAGIC, version, 7, 100, 9)
        assert (hdr.n_layers, hdr.vocab_size, hdr.dim, hdr.hidden_dim, hdr.n_heads, hdr.seq_len) == \
            (cfg["layers"], cfg["vocab"], cfg["dim"], cfg["hidden"], cfg["heads"], cfg["seq"])
        assert abs(hdr.lr - 3e-4) < 1e-9 and hdr.loss == 2.5 and (hdr.cum_compile, hdr.cum_train, hdr.cum_wall) == (1.5, 2.5, 3.5)
        assert (hdr.cum_steps, hdr.cum_batches) == (11, 12)
        assert br.lib.mi355_ckpt_file_bytes(ctypes.byref(hdr)) == os.path.getsize(path)
        raw = open(path, "rb").read()
        for (L, t, part), a in tensors.items():                              # every tensor sits where locate says
            off, cnt = _locate(br, hdr, L, t, part)
            assert cnt == a.size and raw[off:off + 4 * cnt] == a.tobytes(), (L, t, part)
        for (L, t), off in H.ckpt_weight_offsets_like_dashboard(cfg).items():   # and where the dashboard seeks
            assert _locate(br, hdr, L, t, 0)[0] == off
        # create: same header bytes, same file size
        out = str(tmp_path / ("new%d.bin" % version))
        assert br.lib.mi355_ckpt_create(out.encode(), ctypes.byref(hdr)) == 0
        assert os.path.getsize(out) == os.path.getsize(path) and open(out, "rb").read(96) == raw[:96]


def test_checkpoint_rejects_foreign_files(tmp_path):
    import ane_amd.bridge as br
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import helpers as H
    hdr = br.CkptHdr()
    assert br.lib.mi355_ckpt_read_header(str(tmp_path / "missing.bin").encode(), ctypes.byref(hdr)) == -1
    short = tmp_path / "short.bin"; short.write_bytes(b"\0" * 40)
    assert br.lib.mi355_ckpt_read_header(str(short).encode(), ctypes.byref(hdr)) == -1
    good = bytearray(H.ckpt_header_bytes(CK_GQA, 4))
    for pos, val in ((0, b"\x01\x02\x03\x04"), (4, (3).to_bytes(4, "little"))):     # magic, version 3
        bad = bytearray(good); bad[pos:pos + 4] = val
        p = tmp_path / ("bad%d.bin" % pos); p.write_bytes(bytes(bad))
        assert br.lib.mi355_ckpt_read_header(str(p).encode(), ctypes.byref(hdr)) == -1
    assert "ckpt" in br.last_error()
    assert br.lib.mi355_ckpt_file_bytes(ctypes.byref(br.CkptHdr())) == 0
    hdr = br.CkptHdr.from_buffer_copy(bytes(good))
    off, cnt = ctypes.c_uint64(), ctypes.c_uint64()
    assert br.lib.mi355_ckpt_locate(ctypes.byref(hdr), 3, 0, 0, ctypes.byref(off), ctypes.byref(cnt)) == -1   # layer 3 of 3
    assert br.lib.mi355_ckpt_locate(ctypes.byref(hdr), 0, 11, 0, ctypes.byref(off), ctypes.byref(cnt)) == -1
    assert br.lib.mi355_ckpt_locate(ctypes.byref(hdr), 0, 0, 3, ctypes.byref(off), ctypes.byref(cnt)) == -1
