"""Writes tests/golden/kat_small.npz: inputs built with the input recipes of the reference's own
tests (training/test_rmsnorm_bwd.m:26-33, training/test_classifier.m:25-27,132-134 — srand48 seeds 42
and 999, regenerated with the POSIX drand48 LCG) at reduced shapes, and expected outputs from the
float64 closed forms in tests/helpers.py.  Nothing from the reference tree is imported or executed.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers as H  # noqa: E402


def main():
    out = {}
    # --- recipe of test_rmsnorm_bwd.m: x, dy interleaved per element, then w; seed 42 ---
    C, S = 48, 20
    g = H.Drand48(42)
    x = np.empty(C * S, np.float32); dy = np.empty(C * S, np.float32)
    for i in range(C * S):
        x[i] = np.float32(g.next() * 2 - 1) * np.float32(0.5)
        dy[i] = np.float32(g.next() * 2 - 1) * np.float32(0.1)
    w = np.array([np.float32(g.next() * 0.5 + 0.75) for _ in range(C)], np.float32)
    x = x.reshape(C, S); dy = dy.reshape(C, S)
    out["rms_x"], out["rms_dy"], out["rms_w"] = x, dy, w
    out["rms_y"] = H.np_rmsnorm(x, w)
    dx0, dw = H.np_rmsnorm_bwd(dy, x, w, variant=0)
    dx1, _ = H.np_rmsnorm_bwd(dy, x, w, variant=1)
    out["rms_dx_v0"], out["rms_dx_v1"], out["rms_dw"] = dx0, dx1, dw

    # --- recipe of test_classifier.m T3: logits = 10u-5, seed 999; targets (7t+13)%V as in training/train.m:50-51 ---
    V, S2 = 37, 12
    g = H.Drand48(999)
    logits = np.array([np.float32(g.next() * 10 - 5) for _ in range(V * S2)], np.float32).reshape(V, S2)
    tgt = np.array([(7 * t + 13) % V for t in range(S2)], np.int32)
    out["ce_logits"], out["ce_targets"] = logits, tgt
    loss, dl = H.np_cross_entropy(logits, tgt)
    out["ce_loss"], out["ce_dlogits"] = np.float64(loss), dl

    # --- SwiGLU / RoPE / QK-norm on the test_classifier.m T1 recipe (x = 2u-1, seed 42) ---
    g = H.Drand48(42)
    n = 4 * 16 * 8
    a = np.array([np.float32(g.next() * 2 - 1) for _ in range(3 * n)], np.float32) * np.float32(3.0)
    h1, h3, d = a[:n], a[n:2 * n], a[2 * n:]
    out["sw_h1"], out["sw_h3"], out["sw_d"] = h1, h3, d
    out["sw_out"] = H.np_swiglu_fwd(h1, h3)
    out["sw_dh1"], out["sw_dh3"] = H.np_swiglu_bwd(d, h1, h3)
    hd, nh, S3 = 16, 4, 8
    q = h1.reshape(nh * hd, S3)
    out["rope_x"] = q
    for theta in (10000.0, 1e6):
        tag = "1e4" if theta == 10000.0 else "1e6"
        out["rope_fwd_" + tag] = H.np_rope(q, hd, theta, +1)
        out["rope_bwd_" + tag] = H.np_rope(q, hd, theta, -1)
    wq = (np.float32(0.75) + np.float32(0.5) * np.array([np.float32(g.next()) for _ in range(hd)], np.float32))
    out["qk_w"] = wq
    out["qk_fwd"] = H.np_qknorm_rope_fwd(q, wq, hd, 1e6)
    gq = h3.reshape(nh * hd, S3)
    out["qk_dy"] = gq
    out["qk_dx_v0"], out["qk_dw"] = H.np_qknorm_rope_bwd(gq, q, wq, hd, 1e6, variant=0)

    # --- INT8 ties: values chosen so x/scale lands exactly on k+0.5 ---
    x8 = np.array([127.0, -127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 0.25, 63.49, 0.0], np.float32)
    out["i8_x"] = x8                      # max|x| = 127 -> scale exactly 1
    out["i8_rne"] = np.array([127, -127, 0, 2, 2, 0, -2, -2, 126, -126, 0, 63, 0], np.int8)
    out["i8_away"] = np.array([127, -127, 1, 2, 3, -1, -2, -3, 127, -127, 0, 63, 0], np.int8)

    np.savez(os.path.join(HERE, "kat_small.npz"), **out)
    print("wrote", os.path.join(HERE, "kat_small.npz"), sorted(out))


if __name__ == "__main__":
    main()
