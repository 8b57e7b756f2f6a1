"""Parity of the HIP path with the CPU oracle, called through the C-ABI (ctypes) on a real MI355X.

Bars: bit-exact for id/byte work (gather, scatter-add, INT8, the residual family); for fp32 ops
max_i |gpu_i - ref_i| / max(|ref_i|, f * rms(ref)) <= 1e-5 with f = 1e-3 (helpers.err_std), f = 0 for outputs formed
without a subtraction (helpers.err_elem), and f = 1 only where the formula cancels (helpers.rel_err: dx, dw, the
rotation behind a norm, GEMM results)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu

TOL = H.TOL_F32
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "kat_small.npz"))


def dev(br, a):
    return br.DevArray.from_numpy(a)


def say(msg):
    print("[case] " + msg, flush=True)


def rms_cluster_blocks(br, op, Cc, S, B):
    """Workgroups that a norm entry point launches as clusters for this shape under the current knobs (op 0 = forward,
    1 = backward, 2 = backward + residual); 0 when it runs the single-workgroup tile."""
    t = (C.c_int * 5)()
    br.check(br.lib.mi355_rmsnorm_tile(op, Cc, S, B, 1, t))
    return t[4] * B * ((S + 63) // 64)


def ce_one_launch_blocks(br, V, S):
    """Workgroups of the one-launch softmax-CE for a shape that takes it (one per compute unit at most)."""
    cus = br.device_info()[2]
    strips = S // 64
    return min(cus // strips, 64) * strips


# ---------------------------------------------------------------------------------------------
# RMSNorm
# ---------------------------------------------------------------------------------------------
RMS_SHAPES = [
    (1, 768, 256),      # BASELINE.json config 0
    (16, 1024, 256),    # Qwen3-0.6B layer shape
    (3, 48, 20),        # golden-sized, S % 4 == 0 but narrow
    (2, 100, 37),       # S % 4 != 0 -> scalar columns
    (2, 5000, 64),      # C too large for the register tile -> streaming variant
    (5, 128, 256),      # head-sized C
    (1, 1, 4),          # degenerate
]


@pytest.mark.parametrize("B,Cc,S", RMS_SHAPES)
def test_rmsnorm_fwd_bwd(br, B, Cc, S):
    say("rmsnorm B=%d C=%d S=%d" % (B, Cc, S))
    x = H.normal(0, (B, Cc, S)); w = H.normal(1, Cc, 1.0, 0.02); dy = H.normal(2, (B, Cc, S))
    dw0 = H.normal(3, Cc)
    xd, wd, dyd = dev(br, x), dev(br, w), dev(br, dy)
    yd = br.DevArray(x.shape); dxd = br.DevArray(x.shape)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5))
    assert H.err_elem(yd.numpy(), O.rmsnorm(x, w)) <= TOL
    assert H.err_elem(yd.numpy(), H.np_rmsnorm(x, w)) <= TOL
    for variant in (0, 1):
        dwd = dev(br, dw0)
        dxd.upload(np.full(x.shape, 7.0, np.float32))          # dx is assigned, not accumulated
        br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5, variant))
        rdx, rdw = O.rmsnorm_bwd(dy, x, w, variant=variant, dw=dw0)
        assert H.rel_err(dxd.numpy(), rdx) <= TOL
        assert H.rel_err(dwd.numpy(), rdw) <= TOL
        if Cc >= 16:        # with a handful of channels dy - x*dot cancels almost exactly: fp32 itself is off by > 1e-5
            t64dx, t64dw = H.np_rmsnorm_bwd(dy, x, w, variant=variant)
            assert H.rel_err(dxd.numpy(), t64dx) <= TOL
            assert H.rel_err(dwd.numpy(), dw0 + t64dw) <= TOL


def test_rmsnorm_columns_of_zeros_tiny_and_huge_values(br):
    """Columns the reference loop handles without a special case: all zeros (the scale is rsqrt(eps)), values whose
    squares underflow, and values whose squares overflow fp32 (the mean is inf, the scale 0, the output 0)."""
    B, Cc, S = 2, 256, 64
    x = H.normal(4, (B, Cc, S)); w = H.normal(5, Cc, 1.0, 0.02); dy = H.normal(6, (B, Cc, S))
    x[0, :, 0] = 0.0
    x[0, :, 1] *= np.float32(1e-25)
    x[1, :, 2] *= np.float32(1e19)
    x[1, :, 3] = 0.0; x[1, 7, 3] = 3.0          # one non-zero channel
    xd, wd, dyd = dev(br, x), dev(br, w), dev(br, dy)
    yd = br.DevArray(x.shape); dxd = br.DevArray(x.shape); dwd = br.DevArray(Cc)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5))
    y, ry = yd.numpy(), O.rmsnorm(x, w)
    assert np.isfinite(ry).all() and np.isfinite(y).all()
    assert np.array_equal(y[0, :, 0], np.zeros(Cc, np.float32)) and np.array_equal(y[1, :, 2], ry[1, :, 2])
    # column by column: the columns differ by 40 orders of magnitude, so one tensor-wide scale would hide the small ones
    for b in range(B):
        for t in range(4):
            assert H.err_elem(y[b, :, t], ry[b, :, t]) <= TOL, (b, t)
    assert H.err_elem(y[:, :, 4:], ry[:, :, 4:]) <= TOL
    br.check(br.lib.mi355_buf_zero(dwd.handle))
    br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5, 0))
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, variant=0)
    dx = dxd.numpy()
    fin = np.isfinite(rdx)
    assert np.array_equal(np.isfinite(dx), fin)                 # the overflowing column is inf/nan in both, or in neither
    for b in range(B):
        for t in range(S):
            if fin[b, :, t].all():
                assert H.rel_err(dx[b, :, t], rdx[b, :, t]) <= TOL, (b, t)
    if np.isfinite(rdw).all():
        assert H.rel_err(dwd.numpy(), rdw) <= TOL


@pytest.mark.parametrize("B,Cc,S", [(16, 1024, 256), (32, 1024, 256), (1, 768, 256), (2, 100, 37), (2, 2500, 64), (3, 48, 20)])
def test_rmsnorm_bwd_with_residual_equals_the_separate_passes(br, B, Cc, S):
    """dx = rmsnorm_bwd + res and dx_scaled = alpha*dx in one launch (training/training_dynamic/train.m:586-595):
    bit for bit what rmsnorm_bwd, the add and the scale give as three launches, and the oracle's composition."""
    x = H.normal(10, (B, Cc, S)); w = H.normal(11, Cc, 1.0, 0.02); dy = H.normal(12, (B, Cc, S))
    res = H.normal(13, (B, Cc, S)); dw0 = H.normal(14, Cc)
    alpha = np.float32(1 / np.sqrt(2 * 28))
    xd, wd, dyd, rd = dev(br, x), dev(br, w), dev(br, dy), dev(br, res)
    n = x.size
    # the same tile for both (at 32 x 256 columns and up the plain op would take a 16-row tile that the fused one,
    # with three operands in registers, cannot: then the column sums are rounded differently)
    br.tune("rms_lpr", 4); br.tune("rms_threads", 512)
    try:
        _bwd_residual_cases(br, B, Cc, S, x, w, dy, res, dw0, alpha, xd, wd, dyd, rd, n)
    finally:
        br.tune("rms_lpr", 0); br.tune("rms_threads", 0)
    # default tiles: within tolerance of the oracle whatever the tile
    b_dx = br.DevArray(x.shape); b_dw = dev(br, dw0)
    br.check(br.lib.mi355_rmsnorm_bwd_residual_dev(b_dx.ptr, None, b_dw.ptr, dyd.ptr, xd.ptr, wd.ptr, rd.ptr, 0.0, Cc, S, B,
                                                   1e-5, 0))
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, variant=0, dw=dw0)
    assert H.rel_err(b_dx.numpy(), O.axpby(rdx, res, 0.0, 2)) <= TOL and H.rel_err(b_dw.numpy(), rdw) <= TOL


def _bwd_residual_cases(br, B, Cc, S, x, w, dy, res, dw0, alpha, xd, wd, dyd, rd, n):
    for variant in (0, 1):
        # three launches
        a_dx = br.DevArray(x.shape); a_sc = br.DevArray(x.shape); a_dw = dev(br, dw0)
        br.check(br.lib.mi355_rmsnorm_bwd_dev(a_dx.ptr, a_dw.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5, variant))
        br.check(br.lib.mi355_axpby_dev(a_dx.ptr, a_dx.ptr, rd.ptr, 0.0, n, 2))
        br.check(br.lib.mi355_axpby_dev(a_sc.ptr, a_dx.ptr, None, alpha, n, 1))
        # one launch
        b_dx = br.DevArray(x.shape); b_sc = br.DevArray(x.shape); b_dw = dev(br, dw0)
        br.check(br.lib.mi355_rmsnorm_bwd_residual_dev(b_dx.ptr, b_sc.ptr, b_dw.ptr, dyd.ptr, xd.ptr, wd.ptr, rd.ptr, alpha,
                                                       Cc, S, B, 1e-5, variant))
        assert b_dx.numpy().tobytes() == a_dx.numpy().tobytes()
        assert b_sc.numpy().tobytes() == a_sc.numpy().tobytes()
        assert b_dw.numpy().tobytes() == a_dw.numpy().tobytes()
        rdx, rdw = O.rmsnorm_bwd(dy, x, w, variant=variant, dw=dw0)
        want = O.axpby(rdx, res, 0.0, 2)
        assert H.rel_err(b_dx.numpy(), want) <= TOL
        assert H.rel_err(b_sc.numpy(), O.axpby(want, None, alpha, 1)) <= TOL
        assert H.rel_err(b_dw.numpy(), rdw) <= TOL
        # in place over the residual, without the scaled copy (train.m:714-721)
        c_dx = dev(br, res); c_dw = dev(br, dw0)
        br.check(br.lib.mi355_rmsnorm_bwd_residual_dev(c_dx.ptr, None, c_dw.ptr, dyd.ptr, xd.ptr, wd.ptr, c_dx.ptr, 0.0,
                                                       Cc, S, B, 1e-5, variant))
        assert c_dx.numpy().tobytes() == a_dx.numpy().tobytes()
    assert br.lib.mi355_rmsnorm_bwd_residual_dev(b_dx.ptr, b_dx.ptr, b_dw.ptr, dyd.ptr, xd.ptr, wd.ptr, rd.ptr, alpha, Cc, S, B,
                                                 1e-5, 0) == -1


def test_rmsnorm_golden_reference_recipe(br):
    x, dy, w = GOLD["rms_x"], GOLD["rms_dy"], GOLD["rms_w"]
    Cc, S = x.shape
    xd, wd, dyd = dev(br, x), dev(br, w), dev(br, dy)
    yd = br.DevArray(x.shape); dxd = br.DevArray(x.shape); dwd = br.DevArray(Cc)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, Cc, S, 1, 1e-5))
    br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, 1, 1e-5, 0))
    assert H.err_elem(yd.numpy(), GOLD["rms_y"]) <= TOL
    assert H.rel_err(dxd.numpy(), GOLD["rms_dx_v0"]) <= TOL
    assert H.rel_err(dwd.numpy(), GOLD["rms_dw"]) <= TOL
    # the full-size recipe of training/test_rmsnorm_bwd.m:26-33 (DIM 768, SEQ 256, srand48(42))
    xr, dyr, wr = O.recipe_drand48(0, 42, 768 * 256, 768)
    xr = xr.reshape(768, 256); dyr = dyr.reshape(768, 256)
    xd, wd, dyd = dev(br, xr), dev(br, wr), dev(br, dyr)
    dxd = br.DevArray(xr.shape); dwd = br.DevArray(768)
    br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, 768, 256, 1, 1e-5, 0))
    rdx, rdw = O.rmsnorm_bwd(dyr, xr, wr)
    assert H.rel_err(dxd.numpy(), rdx) <= TOL and H.rel_err(dwd.numpy(), rdw) <= TOL


def test_rmsnorm_unaligned_pointers_and_every_tile(br):
    """A tensor that starts 4 bytes into an allocation takes the scalar-column kernel; every
    register-tile configuration gives the same answer."""
    B, Cc, S = 2, 96, 64
    x = H.normal(4, (B, Cc, S)); w = H.normal(5, Cc, 1.0, 0.02); dy = H.normal(6, (B, Cc, S))
    big = br.DevArray(x.size + 1); bigy = br.DevArray(x.size + 1)
    br.lib.mi355_buf_write(big.handle, 4, x.ctypes.data, x.nbytes)
    wd = dev(br, w)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(bigy.ptr + 4, big.ptr + 4, wd.ptr, Cc, S, B, 1e-5))
    out = np.empty_like(x)
    br.lib.mi355_buf_read(bigy.handle, 4, out.ctypes.data, out.nbytes)
    ref = O.rmsnorm(x, w)
    assert H.err_elem(out, ref) <= TOL
    xd, dyd = dev(br, x), dev(br, dy)
    rdx, rdw = O.rmsnorm_bwd(dy, x, w)
    try:
        for lpr in (4, 8, 16):
            for thr in (256, 1024):
                say("rmsnorm tile lpr=%d threads=%d" % (lpr, thr))
                br.tune("rms_lpr", lpr); br.tune("rms_threads", thr)
                yd = br.DevArray(x.shape); dxd = br.DevArray(x.shape); dwd = br.DevArray(Cc)
                br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5))
                br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5, 0))
                assert H.err_elem(yd.numpy(), ref) <= TOL
                assert H.rel_err(dxd.numpy(), rdx) <= TOL and H.rel_err(dwd.numpy(), rdw) <= TOL
    finally:
        br.tune("rms_lpr", 0); br.tune("rms_threads", 0)


@pytest.mark.parametrize("B,Cc,S", [(16, 1024, 256), (3, 2049, 12), (9, 600, 1024), (1, 768, 256), (2, 515, 100)])
def test_rmsnorm_clustered_every_split_and_the_expired_wait(br, B, Cc, S):
    """The channel axis split over 2, 4 or 8 cooperating workgroups (and the library's own choice): all four norm
    entry points against the oracle; then the same calls with the bounded wait set to expire at once, so that every
    workgroup recomputes its partners' sums itself — same bits, and every kernel still exits."""
    say("rmsnorm clustered B=%d C=%d S=%d" % (B, Cc, S))
    x = H.normal(130, (B, Cc, S)); w = H.normal(131, Cc, 1.0, 0.02); dy = H.normal(132, (B, Cc, S))
    res = H.normal(133, (B, Cc, S)); dw0 = H.normal(134, Cc)
    alpha = np.float32(1 / np.sqrt(2 * 28))
    xd, wd, dyd, rd = dev(br, x), dev(br, w), dev(br, dy), dev(br, res)
    ry = O.rmsnorm(x, w)
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, dw=dw0)
    r2 = O.axpby(x, res, alpha, 0)
    r2n = O.rmsnorm(r2, w)

    def run_all():
        y = br.DevArray(x.shape); dx = br.DevArray(x.shape); dwd = dev(br, dw0)
        dx3 = br.DevArray(x.shape); dxs = br.DevArray(x.shape); dw3 = dev(br, dw0)
        y2 = br.DevArray(x.shape); y2n = br.DevArray(x.shape)
        br.check(br.lib.mi355_rmsnorm_fwd_dev(y.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5))
        br.check(br.lib.mi355_rmsnorm_bwd_dev(dx.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5, 0))
        br.check(br.lib.mi355_rmsnorm_bwd_residual_dev(dx3.ptr, dxs.ptr, dw3.ptr, dyd.ptr, xd.ptr, wd.ptr, rd.ptr, alpha,
                                                       Cc, S, B, 1e-5, 0))
        br.check(br.lib.mi355_residual_rmsnorm_fwd_dev(y2.ptr, y2n.ptr, xd.ptr, rd.ptr, alpha, wd.ptr, Cc, S, B, 1e-5))
        return [a.numpy() for a in (y, dx, dwd, dx3, dxs, dw3, y2, y2n)]

    try:
        for split in (0, 2, 4, 8):
            br.tune("rms_cluster", split); br.tune("rms_cluster_spin", 0)
            blocks = (2 * rms_cluster_blocks(br, 0, Cc, S, B) + rms_cluster_blocks(br, 1, Cc, S, B) +
                      rms_cluster_blocks(br, 2, Cc, S, B))               # of the four launches of run_all
            if split == 0 and (B, Cc, S) in ((16, 1024, 256), (1, 768, 256)):
                assert blocks > 0                                        # the shapes the library clusters by itself
            expired = br.exchange_fallbacks()[0]
            got = run_all()
            y, dx, dwv, dx3, dxs, dw3, y2, y2n = got
            assert H.err_elem(y, ry) <= TOL, split
            assert H.rel_err(dx, rdx) <= TOL and H.rel_err(dwv, rdw) <= TOL, split
            want3 = O.axpby(rdx, res, 0.0, 2)
            assert H.rel_err(dx3, want3) <= TOL and H.rel_err(dxs, O.axpby(want3, None, alpha, 1)) <= TOL, split
            assert H.rel_err(dw3, rdw) <= TOL, split
            assert np.array_equal(y2, r2) and H.err_elem(y2n, r2n) <= TOL, split
            again = run_all()                                            # run-to-run deterministic
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, again)), split
            # these two runs took every column sum from the partners: no workgroup's wait expired
            assert br.exchange_fallbacks()[0] == expired, split
            br.tune("rms_cluster_spin", -1)                              # the wait expires before it starts: a partner's
            alone = run_all()                                            # value is taken only if it is already there
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, alone)), split
            br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 1)
            expired = br.exchange_fallbacks()[0]
            refused = run_all()                                          # every workgroup computes its partners' sums itself
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, refused)), split
            assert br.exchange_fallbacks()[0] - expired == blocks, split
            br.tune("xch_take_nothing", 0)
    finally:
        br.tune("rms_cluster", 0); br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)
    br.tune("rms_cluster", -1)                                           # never clustered: the single-workgroup tiles
    try:
        y = run_all()[0]
        assert H.err_elem(y, ry) <= TOL
    finally:
        br.tune("rms_cluster", 0)


@pytest.mark.parametrize("B,Cc,S", [(16, 1024, 256), (1, 768, 256), (2, 100, 37), (3, 48, 20), (2, 300, 64)])
def test_residual_rmsnorm_fused_equals_two_calls(br, B, Cc, S):
    say("residual_rmsnorm B=%d C=%d S=%d" % (B, Cc, S))
    a = H.normal(7, (B, Cc, S)); b = H.normal(8, (B, Cc, S)); w = H.normal(9, Cc, 1.0, 0.02)
    alpha = np.float32(1 / np.sqrt(2 * 28))                     # training/training_dynamic/train.m:188
    ad, bd, wd = dev(br, a), dev(br, b), dev(br, w)
    y = br.DevArray(a.shape); yn = br.DevArray(a.shape)
    br.check(br.lib.mi355_residual_rmsnorm_fwd_dev(y.ptr, yn.ptr, ad.ptr, bd.ptr, alpha, wd.ptr, Cc, S, B, 1e-5))
    ry = O.axpby(a, b, alpha, 0)
    assert np.array_equal(y.numpy(), ry)                        # the residual is exact fp32 arithmetic
    assert H.err_elem(yn.numpy(), O.rmsnorm(ry, w)) <= TOL
    y2 = br.DevArray(a.shape); yn2 = br.DevArray(a.shape)
    br.check(br.lib.mi355_axpby_dev(y2.ptr, ad.ptr, bd.ptr, alpha, a.size, 0))
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yn2.ptr, y2.ptr, wd.ptr, Cc, S, B, 1e-5))
    assert H.rel_err(yn.numpy(), yn2.numpy()) <= 2e-6           # same math, different summation tree
    # in place on a (x_cur updated to x2)
    br.check(br.lib.mi355_residual_rmsnorm_fwd_dev(ad.ptr, yn2.ptr, ad.ptr, bd.ptr, alpha, wd.ptr, Cc, S, B, 1e-5))
    # (in place the library keeps to the single-workgroup tile, whose column sums are rounded in another order)
    assert np.array_equal(ad.numpy(), ry) and H.rel_err(yn2.numpy(), yn.numpy()) <= 2e-6
    assert br.lib.mi355_residual_rmsnorm_fwd_dev(y.ptr, y.ptr, ad.ptr, bd.ptr, alpha, wd.ptr, Cc, S, B, 1e-5) == -1


# ---------------------------------------------------------------------------------------------
# SwiGLU
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [2048 * 256, 3072 * 256 * 16, 1003, 3, 4 * 256 * 8 + 1])
def test_swiglu_fwd_bwd(br, n):
    say("swiglu n=%d" % n)
    h1 = H.normal(10, n); h3 = H.normal(11, n); d = H.normal(12, n)
    special = np.array([0.0, 30.0, -30.0, 88.0, -88.0, 1e-8, -100.0, 100.0], np.float32)
    h1[:min(8, n)] = special[:min(8, n)]             # saturating and tiny gate inputs
    h1d, h3d, dd = dev(br, h1), dev(br, h3), dev(br, d)
    od = br.DevArray(n); d1 = br.DevArray(n); d3 = br.DevArray(n)
    br.check(br.lib.mi355_swiglu_fwd_dev(od.ptr, h1d.ptr, h3d.ptr, n))
    br.check(br.lib.mi355_swiglu_bwd_dev(d1.ptr, d3.ptr, dd.ptr, h1d.ptr, h3d.ptr, n))
    assert H.err_elem(od.numpy(), O.swiglu_fwd(h1, h3)) <= TOL
    r1, r3 = O.swiglu_bwd(d, h1, h3)
    t1, t3 = H.np_swiglu_bwd(d, h1, h3)
    # against float64 the floor is 1e-3 of the tensor's scale: where sigmoid(-88) is a subnormal fp32 number the
    # fp32 formula itself (oracle and GPU alike) is 1e-4 away from the exact value
    assert H.err_elem(d3.numpy(), r3) <= TOL and H.err_std(d3.numpy(), t3) <= TOL
    assert H.err_std(od.numpy(), H.np_swiglu_fwd(h1, h3)) <= TOL
    # dh1 carries the factor 1 + h1*(1 - sig), which passes through zero at h1 = -1.2785: element-wise relative
    # error away from that zero, the tensor's scale as the yardstick next to it (the subtraction cancels there)
    h64 = h1.astype(np.float64); sg = 1.0 / (1.0 + np.exp(-h64))
    away = np.abs(1.0 + h64 * (1.0 - sg)) > 0.05
    assert H.err_elem(d1.numpy()[away], r1[away]) <= TOL and H.err_std(d1.numpy()[away], t1[away]) <= TOL
    assert H.rel_err(d1.numpy(), r1) <= TOL and H.rel_err(d1.numpy(), t1) <= TOL
    assert np.all(np.isfinite(od.numpy())) and np.all(np.isfinite(d1.numpy()))


def test_swiglu_golden(br):
    h1, h3, d = GOLD["sw_h1"], GOLD["sw_h3"], GOLD["sw_d"]
    n = h1.size
    h1d, h3d, dd = dev(br, h1), dev(br, h3), dev(br, d)
    od = br.DevArray(n); d1 = br.DevArray(n); d3 = br.DevArray(n)
    br.check(br.lib.mi355_swiglu_fwd_dev(od.ptr, h1d.ptr, h3d.ptr, n))
    br.check(br.lib.mi355_swiglu_bwd_dev(d1.ptr, d3.ptr, dd.ptr, h1d.ptr, h3d.ptr, n))
    assert H.err_elem(od.numpy(), GOLD["sw_out"]) <= TOL
    assert H.rel_err(d1.numpy(), GOLD["sw_dh1"]) <= TOL and H.err_elem(d3.numpy(), GOLD["sw_dh3"]) <= TOL


# ---------------------------------------------------------------------------------------------
# residual family: bit-exact
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [768 * 256, 1024 * 256 * 16, 1001, 2])
def test_axpby_bit_exact(br, n):
    a = H.normal(20, n); b = H.normal(21, n)
    ad, bd = dev(br, a), dev(br, b)
    yd = br.DevArray(n)
    for alpha in (np.float32(24 ** 0.25), np.float32(1 / np.sqrt(2 * 28))):
        br.check(br.lib.mi355_axpby_dev(yd.ptr, ad.ptr, bd.ptr, alpha, n, 0))
        assert np.array_equal(yd.numpy(), O.axpby(a, b, alpha, 0))
        br.check(br.lib.mi355_axpby_dev(yd.ptr, ad.ptr, None, alpha, n, 1))
        assert np.array_equal(yd.numpy(), O.axpby(a, None, alpha, 1))
    br.check(br.lib.mi355_axpby_dev(yd.ptr, ad.ptr, bd.ptr, 0.0, n, 2))
    assert np.array_equal(yd.numpy(), O.axpby(a, b, 0.0, 2))
    # in place on a (the dx2 += dy pattern of training/training_dynamic/train.m:590)
    br.check(br.lib.mi355_axpby_dev(ad.ptr, ad.ptr, bd.ptr, 0.0, n, 2))
    assert np.array_equal(ad.numpy(), a + b)


# ---------------------------------------------------------------------------------------------
# RoPE
# ---------------------------------------------------------------------------------------------
ROPE_CASES = [
    (1, 12, 12, 64, 256, 10000.0),    # Stories110M, BASELINE.json config 1
    (16, 16, 8, 128, 256, 1e6),       # Qwen3-0.6B, GQA 16/8
    (2, 3, 1, 8, 10, 10000.0),        # S % 4 != 0
    (1, 4, 0, 16, 8, 1e6),            # Q only
]


@pytest.mark.parametrize("B,h,kvh,hd,S,theta", ROPE_CASES)
def test_rope_fwd_bwd(br, B, h, kvh, hd, S, theta):
    say("rope B=%d heads=%d/%d hd=%d S=%d theta=%g" % (B, h, kvh, hd, S, theta))
    q = H.normal(30, (B, h * hd, S)); k = H.normal(31, (B, max(kvh, 1) * hd, S))
    cd, sd = br.rope_tables_dev(S, hd, theta)
    # the host table builder equals the oracle's table bit for bit (same libm, same expression)
    ch = np.empty((hd // 2, S), np.float32); sh = np.empty((hd // 2, S), np.float32)
    br.check(br.lib.mi355_rope_tables(ch.ctypes.data, sh.ctypes.data, S, hd, theta))
    oc, os_ = O.rope_tables(S, hd, theta)
    assert np.array_equal(ch, oc) and np.array_equal(sh, os_)
    for direction in (+1, -1):
        qd, kd = dev(br, q), dev(br, k)
        qo = br.DevArray(q.shape); ko = br.DevArray(k.shape)
        br.check(br.lib.mi355_rope_dev(qo.ptr, ko.ptr if kvh else None, qd.ptr, kd.ptr if kvh else None, h, kvh, hd, S,
                                       B, cd, sd, direction))
        rq = O.rope(q, hd, theta, direction)
        assert H.err_elem(qo.numpy(), rq) <= TOL
        assert np.array_equal(qo.numpy(), rq)          # same table, same operation order: bit-identical
        if kvh:
            assert np.array_equal(ko.numpy(), O.rope(k, hd, theta, direction))
        # in place, as rope_backward_inplace is used (training/training_dynamic/train.m:659-660)
        br.check(br.lib.mi355_rope_dev(qd.ptr, kd.ptr if kvh else None, qd.ptr, kd.ptr if kvh else None, h, kvh, hd, S,
                                       B, cd, sd, direction))
        assert np.array_equal(qd.numpy(), rq)
        # sanity against float64 angles: the reference's float32 angle p*(1/powf(..)) is itself off by up to
        # ~|angle| * 2^-23 (angles reach 255 rad), which is what separates the two here
        assert H.rel_err(qo.numpy(), H.np_rope(q, hd, theta, direction)) <= 2e-4


def test_rope_golden(br):
    x = GOLD["rope_x"]; hd = 16; S = x.shape[1]
    for theta, tag in ((10000.0, "1e4"), (1e6, "1e6")):
        cd, sd = br.rope_tables_dev(S, hd, theta)
        xd = dev(br, x); od = br.DevArray(x.shape)
        br.check(br.lib.mi355_rope_dev(od.ptr, None, xd.ptr, None, 4, 0, hd, S, 1, cd, sd, +1))
        assert H.err_elem(od.numpy(), GOLD["rope_fwd_" + tag]) <= TOL
        br.check(br.lib.mi355_rope_dev(od.ptr, None, xd.ptr, None, 4, 0, hd, S, 1, cd, sd, -1))
        assert H.err_elem(od.numpy(), GOLD["rope_bwd_" + tag]) <= TOL


def test_rope_table_cache_grows_and_keeps_its_tables(br):
    """Many distinct (S, hd, theta) in one process: the cache grows, earlier pointers stay valid and are handed out again."""
    say("rope table cache: 200 distinct tables")
    first = br.rope_tables_dev(12, 8, 10000.0)
    ptrs = {first}
    for i in range(200):
        ptrs.add(br.rope_tables_dev(4 + i, 8, 12345.0))
    assert len(ptrs) == 201
    assert br.rope_tables_dev(12, 8, 10000.0) == first
    x = H.normal(33, (1, 8, 12)); xd = dev(br, x); od = br.DevArray(x.shape)
    br.check(br.lib.mi355_rope_dev(od.ptr, None, xd.ptr, None, 1, 0, 8, 12, 1, first[0], first[1], +1))
    assert np.array_equal(od.numpy(), O.rope(x, 8, 10000.0, +1))
    # one table beyond the byte limit (2 GiB) is refused with a message, and the cache goes on working
    assert br.lib.mi355_rope_tables_dev(C.byref(C.c_void_p()), C.byref(C.c_void_p()), 1 << 20, 512, 10000.0) != 0
    assert "table cache full" in br.last_error()
    assert br.rope_tables_dev(12, 8, 10000.0) == first


# ---------------------------------------------------------------------------------------------
# fused QK-RMSNorm + RoPE
# ---------------------------------------------------------------------------------------------
QK_CASES = [
    (16, 16, 8, 128, 256, 1e6),     # Qwen3-0.6B
    (2, 12, 12, 64, 256, 10000.0),
    (2, 3, 2, 16, 24, 1e6),         # narrow strips
    (1, 2, 1, 8, 10, 1e6),          # S % 4 != 0 -> unfused composition
    (1, 1, 1, 2048, 16, 1e6),       # head_dim beyond the widest register tile -> unfused composition
]


@pytest.mark.parametrize("B,h,kvh,hd,S,theta", QK_CASES)
def test_qknorm_rope_fwd_bwd(br, B, h, kvh, hd, S, theta):
    say("qknorm_rope B=%d heads=%d/%d hd=%d S=%d" % (B, h, kvh, hd, S))
    q = H.normal(40, (B, h * hd, S)); k = H.normal(41, (B, kvh * hd, S))
    wq = H.normal(42, hd, 1.0, 0.02); wk = H.normal(43, hd, 1.0, 0.02)
    gq = H.normal(44, q.shape); gk = H.normal(45, k.shape)
    dwq0 = H.normal(46, hd); dwk0 = H.normal(47, hd)
    cd, sd = br.rope_tables_dev(S, hd, theta)
    qd, kd, wqd, wkd, gqd, gkd = (dev(br, a) for a in (q, k, wq, wk, gq, gk))
    qo = br.DevArray(q.shape); ko = br.DevArray(k.shape)
    br.check(br.lib.mi355_qknorm_rope_fwd_dev(qo.ptr, ko.ptr, qd.ptr, kd.ptr, wqd.ptr, wkd.ptr, h, kvh, hd, S, B, cd, sd,
                                              1e-5))
    assert H.rel_err(qo.numpy(), O.qknorm_rope_fwd(q, wq, hd, theta)) <= TOL
    assert H.rel_err(ko.numpy(), O.qknorm_rope_fwd(k, wk, hd, theta)) <= TOL
    for variant in (0, 1):
        dq = br.DevArray(q.shape); dk = br.DevArray(k.shape)
        dwq = dev(br, dwq0); dwk = dev(br, dwk0)
        br.check(br.lib.mi355_qknorm_rope_bwd_dev(dq.ptr, dk.ptr, dwq.ptr, dwk.ptr, gqd.ptr, gkd.ptr, qd.ptr, kd.ptr,
                                                  wqd.ptr, wkd.ptr, h, kvh, hd, S, B, cd, sd, 1e-5, variant))
        rdq, rdwq = O.qknorm_rope_bwd(gq, q, wq, hd, theta, variant=variant, dw=dwq0)
        rdk, rdwk = O.qknorm_rope_bwd(gk, k, wk, hd, theta, variant=variant, dw=dwk0)
        assert H.rel_err(dq.numpy(), rdq) <= TOL and H.rel_err(dk.numpy(), rdk) <= TOL
        assert H.rel_err(dwq.numpy(), rdwq) <= TOL and H.rel_err(dwk.numpy(), rdwk) <= TOL


def test_qknorm_rope_golden(br):
    x, w, dy = GOLD["rope_x"], GOLD["qk_w"], GOLD["qk_dy"]
    S = x.shape[1]
    cd, sd = br.rope_tables_dev(S, 16, 1e6)
    xd, wd, gd = dev(br, x), dev(br, w), dev(br, dy)
    od = br.DevArray(x.shape); dxd = br.DevArray(x.shape); dwd = br.DevArray(16)
    br.check(br.lib.mi355_qknorm_rope_fwd_dev(od.ptr, None, xd.ptr, None, wd.ptr, None, 4, 0, 16, S, 1, cd, sd, 1e-5))
    assert H.rel_err(od.numpy(), GOLD["qk_fwd"]) <= TOL
    br.check(br.lib.mi355_qknorm_rope_bwd_dev(dxd.ptr, None, dwd.ptr, None, gd.ptr, None, xd.ptr, None, wd.ptr, None, 4,
                                              0, 16, S, 1, cd, sd, 1e-5, 0))
    assert H.rel_err(dxd.numpy(), GOLD["qk_dx_v0"]) <= TOL and H.rel_err(dwd.numpy(), GOLD["qk_dw"]) <= TOL


def test_deferred_weight_gradients_equal_immediate(br):
    """mi355_dw_defer(1): reductions queue up and run at mi355_dw_flush(); same bits as the immediate mode,
    including two ops that add into the same dw (they must keep their order) and more jobs than one launch holds."""
    B, Cc, S, hd, heads, kvh = 2, 256, 64, 32, 4, 2
    cd, sd = br.rope_tables_dev(S, hd, 1e6)
    w = dev(br, H.normal(1, Cc, 1.0, 0.02)); wq = dev(br, H.normal(2, hd, 1.0, 0.02)); wk = dev(br, H.normal(3, hd, 1.0, 0.02))
    xs = [dev(br, H.normal(10 + i, (B, Cc, S))) for i in range(20)]
    dys = [dev(br, H.normal(40 + i, (B, Cc, S))) for i in range(20)]
    q = dev(br, H.normal(70, (B, heads * hd, S))); k = dev(br, H.normal(71, (B, kvh * hd, S)))
    gq = dev(br, H.normal(72, (B, heads * hd, S))); gk = dev(br, H.normal(73, (B, kvh * hd, S)))

    def run(defer):
        br.check(br.lib.mi355_dw_defer(1 if defer else 0))
        dws = [dev(br, H.normal(90 + i, Cc)) for i in range(19)]
        dwq = dev(br, H.normal(120, hd)); dwk = dev(br, H.normal(121, hd))
        dx = br.DevArray((B, Cc, S)); dq = br.DevArray((B, heads * hd, S)); dk = br.DevArray((B, kvh * hd, S))
        for i in range(20):
            tgt = dws[min(i, 18)]                       # ops 18 and 19 accumulate into the same dw
            br.check(br.lib.mi355_rmsnorm_bwd_dev(dx.ptr, tgt.ptr, dys[i].ptr, xs[i].ptr, w.ptr, Cc, S, B, 1e-5, 0))
            br.check(br.lib.mi355_qknorm_rope_bwd_dev(dq.ptr, dk.ptr, dwq.ptr, dwk.ptr, gq.ptr, gk.ptr, q.ptr, k.ptr,
                                                      wq.ptr, wk.ptr, heads, kvh, hd, S, B, cd, sd, 1e-5, 0))
        br.check(br.lib.mi355_dw_flush())
        out = [d.numpy().tobytes() for d in dws] + [dwq.numpy().tobytes(), dwk.numpy().tobytes()]
        br.check(br.lib.mi355_dw_defer(0))
        return out

    try:
        assert run(False) == run(True)
    finally:
        br.lib.mi355_dw_defer(0)


# ---------------------------------------------------------------------------------------------
# embedding
# ---------------------------------------------------------------------------------------------
def _embed_case(seed, V, D, B, S, oob=0):
    E = H.normal(seed, (V, D), 0, 0.02)
    ids = H.zipf_ids(seed + 1, B * S, V).reshape(B, S)
    rng = np.random.default_rng(seed + 2)
    for _ in range(oob):
        ids[rng.integers(B), rng.integers(S)] = V + int(rng.integers(0, 3)) if rng.random() < 0.5 else -1
    return E, ids


@pytest.mark.parametrize("V,D,B,S,oob", [
    (32000, 768, 64, 256, 0),     # BASELINE.json config 2
    (500, 50, 3, 37, 4),          # ragged D and S, out-of-range ids
    (70, 4, 1, 1, 0),
    (1000, 1024, 2, 256, 2),
    (1000, 32, 2048, 8, 3),       # many short sequences: a block of 64 positions spans eight of them
    (1000, 20, 700, 6, 2),        # ... with S not a multiple of 4
    (50, 3, 1, 257, 5),
])
def test_embed_gather_bit_exact(br, V, D, B, S, oob):
    say("gather V=%d D=%d B=%d S=%d" % (V, D, B, S))
    E, ids = _embed_case(50, V, D, B, S, oob)
    pre = H.normal(53, (B, D, S))
    Ed, idd, xd = dev(br, E), dev(br, ids), dev(br, pre)
    br.check(br.lib.mi355_embed_gather_dev(xd.ptr, Ed.ptr, idd.ptr, V, D, S, B))
    ref, skipped = O.embed_lookup(E, ids, out=pre)
    got = xd.numpy()
    assert got.tobytes() == ref.tobytes()
    assert skipped == int(((ids < 0) | (ids >= V)).sum())


@pytest.mark.parametrize("V,D,B,S,oob", [
    (32000, 768, 64, 256, 0),     # BASELINE.json config 2: Zipf(1.1), heavy duplicates
    (500, 50, 3, 37, 4),
    (64, 768, 8, 256, 0),         # tiny vocabulary: every segment is long
    (70, 4, 1, 1, 0),
    (40, 130, 2, 100, 1),
    (3000, 24, 160, 256, 3),      # 40960 positions: the library-sort planner
    (900, 16, 128, 256, 0),       # 32768 positions
    (5000, 8, 64, 256, 2),        # 16384 positions: the most the in-LDS planner takes
    (5000, 8, 1, 16385, 2),       # one more: library sort
    (300000, 8, 4, 100, 1),       # vocabulary of 2^18 and more: library sort whatever the length
    (262143, 8, 4, 100, 3),       # the largest vocabulary of the in-LDS planner (out-of-range ids share the top key)
    (300, 4, 64, 256, 0),         # ~55 positions per token: 300 long segments, more than are ordered by length
    (9, 36, 1, 255, 0),           # a partial last chunk of the planner
    (1000, 32, 2048, 8, 3),       # many short sequences: a block of 64 positions spans eight of them
    (1000, 20, 700, 6, 2),        # ... with S not a multiple of 4
    (50, 3, 1, 257, 5),
    (20, 12001, 1, 130, 2),       # wide rows: more column chunks than compute units
    (7, 8192, 1, 600, 0),
    (524287, 6, 3, 3000, 2),      # the largest vocabulary of the column form; a partial second block of positions
    (2000, 770, 5, 4096, 0),      # 20480 positions, 257 workgroups of three columns, the last with two
    (40, 515, 1, 8192, 0),        # exactly one block; one column left over for the last workgroup
    (32000, 1024, 64, 256, 2),    # the width of Qwen3-0.6B: four columns per workgroup, 256 workgroups
    (700, 1000, 3, 1000, 0),      # four columns, 250 workgroups, three runs of ~4 per token and block
    (90, 1022, 2, 2052, 1),       # four columns, the last workgroup with two
    (100, 7, 2, 256, 0),          # 512 positions: the most the single-launch column kernel takes
    (100, 7, 4, 129, 1),          # 516: one more (S not a multiple of 4: row form)
    (3000, 770, 1, 511, 3),       # single launch, S odd, 257 workgroups, the last with two columns
    (2, 1, 1, 512, 0),            # single launch: two runs of ~256, one column
])
def test_embed_scatter_add_bit_exact_and_deterministic(br, V, D, B, S, oob):
    say("scatter_add V=%d D=%d B=%d S=%d" % (V, D, B, S))
    _, ids = _embed_case(60, V, D, B, S, oob)
    dx = H.normal(63, (B, D, S))
    dE0 = H.normal(64, (V, D), 0, 0.5)
    idd, dxd = dev(br, ids), dev(br, dx)
    ref = O.embed_backward(dE0, dx, ids)
    # the form chosen for the shape, then the two forms by name: a token-major copy of dx summed row by row (-1),
    # columns of dE owned by workgroups (1; shapes it does not take fall back to the other)
    for form in (0, -1, 1):
        br.tune("scatter_cols", form)
        try:
            outs = []
            for _ in range(2):
                dEd = dev(br, dE0)
                br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
                outs.append(dEd.numpy())
        finally:
            br.tune("scatter_cols", 0)
        assert outs[0].tobytes() == outs[1].tobytes(), form            # run-to-run deterministic
        assert outs[0].tobytes() == ref.tobytes(), form                # the ordered fp32 sum of the reference loop


def test_embed_scatter_add_form_follows_how_the_ids_repeat(br):
    """Left to itself the library takes the column form, whose cost goes by the distinct (token, block) pairs, learns
    from each call's report how the ids repeated, and moves an input that hardly repeats to the row form (and back).
    Same bytes whichever form runs."""
    V, D, B, S = 32000, 768, 64, 256
    say("scatter_add form choice V=%d D=%d B=%d S=%d" % (V, D, B, S))
    zipf = H.zipf_ids(3, B * S, V).astype(np.int32).reshape(B, S)
    flat = np.random.default_rng(4).integers(0, V, (B, S)).astype(np.int32)
    dx = H.normal(65, (B, D, S)); dE0 = H.normal(66, (V, D), 0, 0.5)
    dxd = dev(br, dx)
    form = lambda: br.lib.mi355_embed_scatter_add_form(V, D, S, B, 1)

    def call(ids):
        dEd = dev(br, dE0)
        br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, dev(br, ids).ptr, V, D, S, B))
        br.sync()                                  # the report of this call is in host memory now
        return dEd.numpy().tobytes()

    try:
        br.tune("scatter_cols", 1)
        ref_zipf = call(zipf)                      # a column-form report of this shape: a known starting point
        br.tune("scatter_cols", 0)
        assert ref_zipf == O.embed_backward(dE0, dx, zipf).tobytes()
        assert form() == 1
        ref_flat = O.embed_backward(dE0, dx, flat).tobytes()
        assert call(flat) == ref_flat              # (ran in the column form)
        assert form() == -1                        # ~12800 distinct ids in 16384 positions: the row form next
        assert call(flat) == ref_flat and form() == -1      # ... and it stays there
        assert call(zipf) == ref_zipf              # (ran in the row form)
        assert form() == 1                         # ids that repeat: back to the columns
        assert call(zipf) == ref_zipf and form() == 1
        br.tune("scatter_cols", -1)
        assert form() == -1 and call(zipf) == ref_zipf
        br.tune("scatter_cols", 0)
        assert form() == 1                         # a forced call of the other form leaves a report too
        assert br.lib.mi355_embed_scatter_add_form(0, D, S, B, 1) == 0
        assert br.lib.mi355_embed_scatter_add_form(V, D, 255, B, 1) == -1      # S not a multiple of 4: rows only
        assert br.lib.mi355_embed_scatter_add_form(V, D, S, 100, 1) == -1      # 25600 positions: rows only
    finally:
        br.tune("scatter_cols", 0)


def test_embed_scatter_add_tree_order_is_deterministic_and_close(br):
    """The opt-in fixed-tree order: same bytes on every run, within 1e-5 of the reference order, and only long
    segments are affected."""
    V, D, B, S = 32000, 768, 64, 256
    _, ids = _embed_case(60, V, D, B, S, 0)
    dx = H.normal(63, (B, D, S)); dE0 = H.normal(64, (V, D), 0, 0.5)
    idd, dxd = dev(br, ids), dev(br, dx)
    ref = O.embed_backward(dE0, dx, ids)
    br.tune("scatter_tree", 1)                  # (selects the token-major form: the tree is an order of its long segments)
    try:
        outs = []
        for _ in range(2):
            dEd = dev(br, dE0)
            br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
            outs.append(dEd.numpy())
    finally:
        br.tune("scatter_tree", 0)
    assert outs[0].tobytes() == outs[1].tobytes()
    # a reordered fp32 sum of n terms differs by ~sqrt(n) ulps of its partial sums: judge each row against its own
    # scale, and against the exact sum, where the tree is no worse than the reference's chain
    row_rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2, axis=1))
    assert np.max(np.max(np.abs(outs[0].astype(np.float64) - ref), axis=1) / row_rms) <= TOL
    exact = H.np_embed_backward(dE0, dx, ids)
    assert np.max(np.abs(outs[0] - exact)) <= 1.5 * np.max(np.abs(ref - exact)) + 1e-7
    counts = np.bincount(ids.ravel(), minlength=V)
    short = counts <= 96           # segments of up to 96 rows are summed by one wave, in the reference order
    assert np.array_equal(outs[0][short], ref[short])                 # rows of short segments keep the reference order
    assert not np.array_equal(outs[0][~short], ref[~short])           # the long ones are rounded differently


@pytest.mark.parametrize("V,D,B,S", [(32000, 768, 8, 256), (500, 96, 3, 40), (1000, 64, 80, 256), (300, 7, 2, 256)])
@pytest.mark.parametrize("off_dx,off_dE", [(1, 0), (0, 1), (3, 2)])
def test_embed_scatter_add_unaligned_pointers(br, V, D, B, S, off_dx, off_dE):
    """dx and dE at addresses that are multiples of 4 bytes only (the reference takes any float pointer): every form,
    same bytes as the reference loop."""
    say("scatter_add unaligned V=%d D=%d B=%d S=%d +%d/+%d floats" % (V, D, B, S, off_dx, off_dE))
    _, ids = _embed_case(160, V, D, B, S, 1)
    dx = H.normal(163, (B, D, S)); dE0 = H.normal(164, (V, D), 0, 0.5)
    ref = O.embed_backward(dE0, dx, ids)
    idd = dev(br, ids)
    dxd = dev(br, np.concatenate([np.zeros(off_dx, np.float32), dx.ravel()]))
    for form in (0, -1, 1):
        br.tune("scatter_cols", form)
        try:
            dEd = dev(br, np.concatenate([np.full(off_dE, 7.0, np.float32), dE0.ravel(), np.full(4, 9.0, np.float32)]))
            br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr + 4 * off_dE, dxd.ptr + 4 * off_dx, idd.ptr, V, D, S, B))
        finally:
            br.tune("scatter_cols", 0)
        out = dEd.numpy()
        assert out[off_dE:off_dE + V * D].tobytes() == ref.tobytes(), form
        assert (out[:off_dE] == 7.0).all() and (out[off_dE + V * D:] == 9.0).all(), form      # nothing written outside


def test_embed_scatter_add_no_valid_id(br):
    """Every id out of range: nothing is added (ids outside [0,V) are skipped, as the oracle's loop does)."""
    V, D, B, S = 100, 20, 2, 50
    ids = np.where(np.arange(B * S).reshape(B, S) % 2 == 0, -1, V).astype(np.int32)
    dx = H.normal(66, (B, D, S))
    dE0 = H.normal(67, (V, D))
    idd, dxd, dEd = dev(br, ids), dev(br, dx), dev(br, dE0)
    br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
    assert dEd.numpy().tobytes() == dE0.tobytes()


@pytest.mark.parametrize("form", [-1, 1])
@pytest.mark.parametrize("B", [4, 80])
def test_embed_scatter_add_single_hot_token(br, form, B):
    """One token at every position: one chain of B*256 dependent adds per column; with 80 sequences it runs through
    three blocks of positions of the column form, carried from block to block on the chip."""
    V, D, S = 10, 192, 256
    ids = np.full((B, S), 7, np.int32)
    dx = H.normal(65, (B, D, S)) * np.float32(100)
    dE0 = np.zeros((V, D), np.float32)
    idd, dxd, dEd = dev(br, ids), dev(br, dx), dev(br, dE0)
    br.tune("scatter_cols", form)
    try:
        br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
    finally:
        br.tune("scatter_cols", 0)
    assert dEd.numpy().tobytes() == O.embed_backward(dE0, dx, ids).tobytes()


def test_embed_scatter_add_column_form_runs_that_change_length(br):
    """Tokens whose runs are long in one block of positions and short or absent in the next, in every order: the
    sums carried on the chip from block to block and the ones re-read from dE must agree with the reference loop."""
    V, D, S, B = 600, 9, 256, 128                      # 32768 positions: four blocks of 8192
    rng = np.random.default_rng(77)
    N = B * S
    ids = rng.integers(300, V, N).astype(np.int32)     # background: tokens that occur a few times per block
    blk = np.arange(N) // 8192
    for tok, pattern in enumerate([(40, 0, 40, 40), (0, 40, 3, 40), (40, 3, 0, 1), (1, 40, 40, 0), (16, 15, 16, 15),
                                   (2000, 2000, 1, 2000), (3, 2, 1, 0)]):
        for b, n in enumerate(pattern):
            pos = rng.choice(np.flatnonzero(blk == b), n, replace=False)
            ids[pos] = tok
    # tokens 256 apart share an entry of the table that carries sums between blocks
    ids[rng.choice(N, 3000, replace=False)] = 256
    ids[rng.choice(N, 3000, replace=False)] = 0
    ids = ids.reshape(B, S)
    dx = H.normal(68, (B, D, S)); dE0 = H.normal(69, (V, D))
    idd, dxd, dEd = dev(br, ids), dev(br, dx), dev(br, dE0)
    br.tune("scatter_cols", 1)
    try:
        br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
    finally:
        br.tune("scatter_cols", 0)
    assert dEd.numpy().tobytes() == O.embed_backward(dE0, dx, ids).tobytes()


@pytest.mark.parametrize("n", [1024 * 4096, 13, 4099, 3, 1024 * 1024 * 5 + 2, 9 * 1024 * 1024 + 4])
@pytest.mark.parametrize("rounding", [0, 1])
def test_int8_quantize_dynamic_equals_scale_then_quant(br, n, rounding):
    """The reference's quantizer (maximum, then rounding) in one call: up to 8.4 M floats one launch whose workgroups
    keep the tensor in registers and hand one another their maxima; the same bytes as the two separate steps and the
    oracle, also when every wait is made to expire or every maximum is refused, and the counter says which it was."""
    x = H.normal(72, n) * np.float32(3.0)
    if n > 8: x[5] = np.float32(-11.0)
    if n > 4096: x[n - 2] = np.float32(12.5)            # the maximum among the last elements (n % 4 != 0: in the tail)
    xd = dev(br, x)
    s1 = br.DevArray(1); q1 = br.DevArray(n, np.int8)
    br.check(br.lib.mi355_int8_scale_dev(s1.ptr, xd.ptr, n))
    br.check(br.lib.mi355_int8_quant_dev(q1.ptr, xd.ptr, s1.ptr, n, rounding))
    s2 = br.DevArray(1); q2 = br.DevArray(n, np.int8)
    one_launch = 4 <= n <= 8 * 1024 * 1024
    # workgroups that wait for one another: those of the one launch; below four elements the scale kernel's one
    blocks = min(-(-(n // 4) // 1024), br.device_info()[2]) if one_launch else (1 if n < 4 else 0)
    try:
        for spin, refuse in ((0, 0), (-1, 0), (0, 1)):
            br.tune("rms_cluster_spin", spin); br.tune("xch_take_nothing", refuse)
            s2.upload(np.zeros(1, np.float32)); q2.upload(np.zeros(n, np.int8))
            expired = br.exchange_fallbacks()[0]
            br.check(br.lib.mi355_int8_quantize_dynamic_dev(q2.ptr, s2.ptr, xd.ptr, n, rounding))
            assert s2.numpy().tobytes() == s1.numpy().tobytes() and q2.numpy().tobytes() == q1.numpy().tobytes(), (spin, refuse)
            if spin == 0:       # handed over in the normal run; every workgroup on its own when it refuses the others' maxima
                assert br.exchange_fallbacks()[0] - expired == blocks * refuse, (refuse, blocks)
        br.tune("rms_cluster", -1)                       # the cooperating forms switched off: two launches
        br.check(br.lib.mi355_int8_quantize_dynamic_dev(q2.ptr, s2.ptr, xd.ptr, n, rounding))
        assert s2.numpy().tobytes() == s1.numpy().tobytes() and q2.numpy().tobytes() == q1.numpy().tobytes()
    finally:
        br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0); br.tune("rms_cluster", 0)
    sc = O.int8_scale(x)
    assert np.float32(sc) == s2.numpy()[0] and np.array_equal(q2.numpy(), O.int8_quant(x, sc, rounding))
    z = dev(br, np.zeros(64, np.float32))               # all zeros: scale 1
    br.check(br.lib.mi355_int8_quantize_dynamic_dev(q2.ptr, s2.ptr, z.ptr, min(n, 64), rounding))
    assert s2.numpy()[0] == 1.0 and not q2.numpy()[:min(n, 64)].any()


@pytest.mark.parametrize("n", [1024 * 4096, 4099, 5, 3 * 1024 * 1024 + 1])
def test_int8_scale_single_launch_and_its_expired_wait(br, n):
    """The scale comes from one launch whose workgroups hand their maxima to workgroup 0; with the bounded wait set
    to expire at once workgroup 0 takes the maximum itself.  Same bits either way, also on an unaligned tensor."""
    x = H.normal(140, n + 1) * np.float32(2.5)
    x[n // 2] = np.float32(-123.25)
    xd = dev(br, x); sd = br.DevArray(1)
    try:
        for spin, refuse in ((0, 0), (-1, 0), (0, 1)):
            br.tune("rms_cluster_spin", spin); br.tune("xch_take_nothing", refuse)
            for off in (0, 1):                       # off = 1: the address is not 16-byte aligned (scalar path)
                sd.upload(np.zeros(1, np.float32))
                expired = br.exchange_fallbacks()[0]
                for _ in range(3):
                    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, xd.ptr + 4 * off, n))
                assert sd.numpy()[0] == np.float32(O.int8_scale(x[off:off + n])), (spin, refuse, off)
                # handed over in the normal run (no wait expired); workgroup 0 alone when it refuses the others' maxima
                if spin == 0:
                    assert br.exchange_fallbacks()[0] - expired == 3 * refuse, (refuse, off)
    finally:
        br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)
    z = dev(br, np.zeros(4096, np.float32))
    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, z.ptr, 4096))
    assert sd.numpy()[0] == 1.0


def test_cooperating_kernels_are_switched_off_after_repeated_expiries(br):
    """A device on which the cooperating workgroups keep missing one another: forced here from the host with a wait of
    one clock tick.  mi355_sync looks at the expired-wait counters; when they have grown at three syncs in a row the
    library takes the non-cooperating forms by itself (same results), and setting the knobs back switches them on."""
    B, Cc, S, V = 16, 1024, 256, 32000
    x = H.normal(150, (B, Cc, S)); w = H.normal(151, Cc, 1.0, 0.02)
    logits = H.normal(152, (V, S), 0, 2.0); tgt = np.random.default_rng(153).integers(0, V, S).astype(np.int32)
    x8 = H.normal(154, 1024 * 4096)
    xd, wd, ld, td, x8d = dev(br, x), dev(br, w), dev(br, logits), dev(br, tgt), dev(br, x8)
    ry = O.rmsnorm(x, w); rl, rd = O.cross_entropy(logits, tgt); rs = np.float32(O.int8_scale(x8))
    plan = (C.c_int * 5)()

    def run():
        y = br.DevArray(x.shape); dl = br.DevArray(logits.shape); lossd = br.DevArray(1); sd = br.DevArray(1)
        br.check(br.lib.mi355_rmsnorm_fwd_dev(y.ptr, xd.ptr, wd.ptr, Cc, S, B, 1e-5))
        br.check(br.lib.mi355_softmax_ce_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
        br.check(br.lib.mi355_int8_scale_dev(sd.ptr, x8d.ptr, x8.size))
        br.sync()
        assert H.err_elem(y.numpy(), ry) <= TOL and H.err_std(dl.numpy(), rd) <= TOL and sd.numpy()[0] == rs
        assert abs(float(lossd.numpy()[0]) - rl) <= TOL * abs(rl)

    try:
        br.tune("rms_cluster_spin", 1)                # 10 ns: a value that is not there at the first look is given up
        for i in range(4):                            # the first sync after a knob change only takes the counters' level
            br.check(br.lib.mi355_rmsnorm_tile(0, Cc, S, B, 1, plan))
            assert plan[4] > 0, i                     # still clustered
            run()
        br.check(br.lib.mi355_rmsnorm_tile(0, Cc, S, B, 1, plan))
        assert plan[4] == 0                           # switched off by the library
        before = br.exchange_fallbacks()
        run()                                         # single-workgroup tiles, three-launch cross-entropy, two-launch scale
        assert br.exchange_fallbacks() == before
    finally:
        br.tune("rms_cluster_spin", 0); br.tune("rms_cluster", 0); br.tune("ce_resident", 0)
    br.check(br.lib.mi355_rmsnorm_tile(0, Cc, S, B, 1, plan))
    assert plan[4] > 0
    before = br.exchange_fallbacks()
    for i in range(4):                                # the normal configuration: nothing expires, nothing is switched off
        run()
    assert br.exchange_fallbacks() == before
    br.check(br.lib.mi355_rmsnorm_tile(0, Cc, S, B, 1, plan))
    assert plan[4] > 0


@pytest.mark.parametrize("n", [1024 * 4096, 2048 * 256 * 16, 13, 1, 4099])
def test_minmax_exact(br, n):
    say("minmax n=%d" % n)
    x = H.normal(71, n) * np.float32(2.0)
    if n > 100:
        x[n // 3] = np.float32(-77.0); x[n // 2] = np.float32(55.5); x[7] = np.nan
    xd = dev(br, x); od = br.DevArray(3)
    br.check(br.lib.mi355_minmax_dev(od.ptr, xd.ptr, n))
    assert od.numpy().tobytes() == O.minmax(x).tobytes()
    if n > 4:       # an address that is not 16-byte aligned takes the scalar path
        off = dev(br, np.concatenate([np.array([1e9], np.float32), x]))
        br.check(br.lib.mi355_minmax_dev(od.ptr, off.ptr + 4, n))
        assert od.numpy().tobytes() == O.minmax(x).tobytes()


# ---------------------------------------------------------------------------------------------
# softmax + cross-entropy
# ---------------------------------------------------------------------------------------------
def _ce_check(br, logits, tgt, grad_scale=1.0, inplace=False):
    V, S = logits.shape
    ld, td = dev(br, logits), dev(br, tgt)
    dd = ld if inplace else br.DevArray(logits.shape)
    lossd = br.DevArray(1)
    br.check(br.lib.mi355_softmax_ce_dev(dd.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, grad_scale))
    loss = float(lossd.numpy()[0]); dl = dd.numpy()
    rl, rd = O.cross_entropy(logits, tgt, grad_scale)
    assert abs(loss - rl) <= TOL * abs(rl) + 1e-12
    assert H.err_std(dl, rd) <= TOL
    tl, td64 = H.np_cross_entropy(logits, tgt, grad_scale)
    assert abs(loss - tl) <= TOL * abs(tl) + 1e-12
    assert H.err_std(dl, td64) <= TOL
    return loss, dl


@pytest.mark.parametrize("V,S", [(32000, 256), (37, 12), (1000, 5), (151936, 256), (300, 1024)])
def test_softmax_ce(br, V, S):
    say("softmax_ce V=%d S=%d" % (V, S))
    logits = H.normal(70, (V, S), 0, 2.0)
    tgt = np.random.default_rng(71).integers(0, V, S).astype(np.int32)
    loss, dl = _ce_check(br, logits, tgt)
    assert np.max(np.abs(dl.astype(np.float64).sum(axis=0))) < 1e-6     # sum_v (p - onehot)/S = 0


def test_softmax_ce_golden_policy_scale_inplace(br):
    logits, tgt = GOLD["ce_logits"], GOLD["ce_targets"]
    loss, dl = _ce_check(br, logits, tgt)
    assert abs(loss - float(GOLD["ce_loss"])) <= TOL * float(GOLD["ce_loss"])
    assert H.err_std(dl, GOLD["ce_dlogits"]) <= TOL
    V, S = 4099, 64
    big = H.normal(72, (V, S), 0, 2.0)
    t2 = np.random.default_rng(73).integers(0, V, S).astype(np.int32)
    t2[3] = V; t2[10] = -1; t2[63] = 70000                              # out-of-range targets are skipped
    _ce_check(br, big, t2)
    _ce_check(br, big, t2, grad_scale=256.0)                            # loss scaling of train.m:497 fused
    _ce_check(br, big, t2, inplace=True)
    # extreme logits: one dominant entry per column, and a constant column
    ext = H.normal(74, (V, S), 0, 30.0); ext[:, 5] = 3.25
    _ce_check(br, ext, t2)
    # the recipe of training/test_classifier.m:132-134 at its own size
    x, _, _ = O.recipe_drand48(2, 999, 32000 * 256, 0)
    _ce_check(br, x.reshape(32000, 256), (np.arange(256, dtype=np.int32) * 7 + 13) % 256 + 1)


def test_softmax_ce_deterministic(br):
    V, S = 32000, 256
    logits = H.normal(75, (V, S), 0, 2.0)
    tgt = np.random.default_rng(76).integers(0, V, S).astype(np.int32)
    ld, td = dev(br, logits), dev(br, tgt)
    res = []
    for _ in range(2):
        dd = br.DevArray(logits.shape); lossd = br.DevArray(1)
        br.check(br.lib.mi355_softmax_ce_dev(dd.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
        res.append((lossd.numpy().tobytes(), dd.numpy().tobytes()))
    assert res[0] == res[1]


@pytest.mark.parametrize("V,S", [(4099, 64), (32000, 256), (151936, 256), (700, 128), (40, 64), (9000, 1024), (5000, 192),
                                 (70000, 64)])
def test_softmax_ce_one_launch_and_its_expired_wait(br, V, S):
    """The form that keeps the logits on the chip between the passes (one workgroup per compute unit, partials
    exchanged inside the launch), forced for every shape it accepts: against the oracle; run to run and with the
    bounded wait set to expire at once (partners' partials recomputed from memory) the same bits; and close to the
    three-launch form, which sums in another order."""
    say("softmax_ce one launch V=%d S=%d" % (V, S))
    logits = H.normal(77, (V, S), 0, 2.0)
    tgt = np.random.default_rng(78).integers(0, V, S).astype(np.int32)
    tgt[1] = V; tgt[S - 2] = -1                                         # out-of-range targets are skipped
    ld, td = dev(br, logits), dev(br, tgt)

    def run(scale):
        dd = br.DevArray(logits.shape); lossd = br.DevArray(1)
        br.check(br.lib.mi355_softmax_ce_dev(dd.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, scale))
        return lossd.numpy().copy(), dd.numpy()

    try:
        br.tune("ce_resident", 1); br.tune("rms_cluster_spin", 0)
        for scale in (1.0, 256.0):
            loss, dl = run(scale)
            rl, rd = O.cross_entropy(logits, tgt, scale)
            assert abs(float(loss[0]) - rl) <= TOL * abs(rl) + 1e-12
            assert H.err_std(dl, rd) <= TOL
        expired = br.exchange_fallbacks()[1]
        loss, dl = run(1.0)
        loss2, dl2 = run(1.0)
        assert loss.tobytes() == loss2.tobytes() and dl.tobytes() == dl2.tobytes()
        assert br.exchange_fallbacks()[1] == expired                     # every partial was handed over: no wait expired
        br.tune("rms_cluster_spin", -1)                                  # the wait expires before it starts
        loss3, dl3 = run(1.0)
        assert loss.tobytes() == loss3.tobytes() and dl.tobytes() == dl3.tobytes()
        br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 1)   # no partner's value is taken at all: every
        expired = br.exchange_fallbacks()[1]                             # workgroup recomputes its whole strip, workgroup 0
        loss5, dl5 = run(1.0)                                            # the other strips' loss terms
        assert loss.tobytes() == loss5.tobytes() and dl.tobytes() == dl5.tobytes()
        assert br.exchange_fallbacks()[1] - expired == ce_one_launch_blocks(br, V, S)
        br.tune("xch_take_nothing", 0)
        br.tune("ce_resident", -1)                                       # the three-launch form
        loss4, dl4 = run(1.0)
        assert abs(float(loss4[0]) - float(loss[0])) <= 2e-6 * abs(float(loss[0]))
        assert H.err_std(dl4, dl) <= 2e-6
    finally:
        br.tune("ce_resident", 0); br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)


# ---------------------------------------------------------------------------------------------
# INT8: bit-exact
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1024 * 4096, 13, 4099])
def test_int8_bit_exact(br, n):
    say("int8 n=%d" % n)
    x = H.normal(80, n) * 3
    if n > 100:                       # plant exact ties for scale = max|x|/127 = 1/8... use a power-of-two max
        x = np.clip(x, -15.0, 15.0); x[0] = 15.875        # scale = 15.875/127 = 0.125
        x[1:9] = [0.0625, 0.1875, 0.3125, -0.0625, -0.1875, -0.3125, 15.8125, -15.8125]   # k + 0.5 after /0.125
    xd = dev(br, x)
    sd = br.DevArray(1)
    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, xd.ptr, n))
    scale = sd.numpy()[0]
    assert scale == np.float32(O.int8_scale(x))
    for mode in (0, 1):
        qd = br.DevArray(n, np.int8)
        br.check(br.lib.mi355_int8_quant_dev(qd.ptr, xd.ptr, sd.ptr, n, mode))
        q = qd.numpy()
        assert np.array_equal(q, O.int8_quant(x, scale, mode))
        yd = br.DevArray(n)
        br.check(br.lib.mi355_int8_dequant_dev(yd.ptr, qd.ptr, sd.ptr, n))
        assert np.array_equal(yd.numpy(), O.int8_dequant(q, scale))
        assert np.max(np.abs(yd.numpy().astype(np.float64) - x)) <= scale / 2 * (1 + 1e-6)
    if n > 100:
        assert not np.array_equal(O.int8_quant(x, scale, 0)[:9], O.int8_quant(x, scale, 1)[:9])   # ties differ


def test_int8_golden_and_zero_tensor(br):
    x = GOLD["i8_x"]
    xd = dev(br, x); sd = br.DevArray(1)
    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, xd.ptr, x.size))
    assert sd.numpy()[0] == 1.0
    for mode, key in ((0, "i8_rne"), (1, "i8_away")):
        qd = br.DevArray(x.size, np.int8)
        br.check(br.lib.mi355_int8_quant_dev(qd.ptr, xd.ptr, sd.ptr, x.size, mode))
        assert np.array_equal(qd.numpy(), GOLD[key])
    zd = dev(br, np.zeros(100, np.float32))
    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, zd.ptr, 100))
    assert sd.numpy()[0] == 1.0


# ---------------------------------------------------------------------------------------------
# next rows: optimizer tail and GQA helpers
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1024 * 3072, 1024, 100003, 5])
def test_optimizer_tail(br, n):
    """Scale + global norm + clip + AdamW as two sweeps (training/training_dynamic/train.m:748-877)."""
    say("optimizer tail n=%d" % n)
    w = H.normal(50, n, 0, 0.05); g = H.normal(51, n) * 40; m = H.normal(52, n, 0, 0.01)
    v = np.abs(H.normal(53, n, 0, 0.01))
    gsc = np.float32(1.0 / 256.0); clip = np.float32(1e-3)
    t, lr, b1, b2, eps, wd = 7, 3e-4, 0.9, 0.95, 1e-8, 0.1
    wd_, gd, md, vd = dev(br, w), dev(br, g), dev(br, m), dev(br, v)
    ss = dev(br, np.zeros(1, np.float32)); cs = br.DevArray(1)
    br.check(br.lib.mi355_sumsq_accum_dev(ss.ptr, gd.ptr, n, gsc))
    br.check(br.lib.mi355_sumsq_accum_dev(ss.ptr, gd.ptr, n, gsc))           # accumulates over tensors
    t64 = 2 * float(np.sum((g * gsc).astype(np.float64) ** 2))
    assert abs(ss.numpy()[0] - t64) <= TOL * t64
    # the oracle sums millions of float32 terms in eight running lanes (vDSP_dotpr's order is unpublished); its own
    # distance from the float64 sum is ~1e-4 at this length, so it can only be held to that
    r_ss = O.sumsq_scaled(g, gsc)
    assert abs(ss.numpy()[0] - 2 * r_ss) <= 5e-4 * 2 * r_ss
    br.check(br.lib.mi355_clip_scale_dev(cs.ptr, ss.ptr, clip))
    r_cs = O.clip_scale(float(ss.numpy()[0]), clip)
    assert cs.numpy()[0] == np.float32(r_cs) and r_cs < 1.0
    br.check(br.lib.mi355_adam_update_dev(wd_.ptr, gd.ptr, md.ptr, vd.ptr, n, t, lr, b1, b2, eps, wd, gsc, cs.ptr, 1))
    g2 = (g * gsc) * np.float32(r_cs)                                         # the two scale passes of the reference
    rw, rm, rv = O.adam_update(w, g2, m, v, t, lr, b1, b2, eps, wd)
    assert H.rel_err(md.numpy(), rm) <= TOL and H.rel_err(vd.numpy(), rv) <= TOL
    assert H.rel_err(wd_.numpy(), rw) <= TOL
    assert H.rel_err(wd_.numpy() - w, rw - w) <= 1e-4                         # the update itself, not just w
    assert not gd.numpy().any()                                               # zero_grad
    # no clip, no zeroing, NULL scale pointer
    wd_, gd, md, vd = dev(br, w), dev(br, g), dev(br, m), dev(br, v)
    br.check(br.lib.mi355_adam_update_dev(wd_.ptr, gd.ptr, md.ptr, vd.ptr, n, 1, lr, b1, b2, eps, 0.0, 1.0, None, 0))
    rw, rm, rv = O.adam_update(w, g, m, v, 1, lr, b1, b2, eps, 0.0)
    assert H.rel_err(wd_.numpy(), rw) <= TOL and H.rel_err(md.numpy(), rm) <= TOL and H.rel_err(vd.numpy(), rv) <= TOL
    assert np.array_equal(gd.numpy(), g)
    br.check(br.lib.mi355_clip_scale_dev(cs.ptr, ss.ptr, np.float32(1e9)))
    assert cs.numpy()[0] == 1.0


def test_optimizer_tail_multi_tensor_equals_per_tensor(br):
    import ctypes as C
    sizes = [4096, 1024 * 1024 + 4, 12, 300000] + [2048] * 17                  # more tensors than one launch holds
    ws = [H.normal(60 + i, n, 0, 0.05) for i, n in enumerate(sizes)]
    gs = [H.normal(90 + i, n) for i, n in enumerate(sizes)]
    ms = [H.normal(120 + i, n, 0, 0.01) for i, n in enumerate(sizes)]
    vs = [np.abs(H.normal(150 + i, n, 0, 0.01)) for i, n in enumerate(sizes)]
    wds = [0.1 if i % 2 else 0.0 for i in range(len(sizes))]
    hp = dict(t=4, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8)
    D = lambda arrs: [dev(br, a) for a in arrs]
    w1, g1, m1, v1 = D(ws), D(gs), D(ms), D(vs)
    w2, g2, m2, v2 = D(ws), D(gs), D(ms), D(vs)
    ss1 = dev(br, np.zeros(1, np.float32)); ss2 = dev(br, np.zeros(1, np.float32))
    k = len(sizes)
    parr = lambda ds: (C.c_void_p * k)(*[d.ptr for d in ds])
    narr = (C.c_size_t * k)(*sizes); wdarr = (C.c_float * k)(*wds)
    for i in range(k):
        br.check(br.lib.mi355_sumsq_accum_dev(ss1.ptr, g1[i].ptr, sizes[i], 0.5))
        br.check(br.lib.mi355_adam_update_dev(w1[i].ptr, g1[i].ptr, m1[i].ptr, v1[i].ptr, sizes[i], hp["t"], hp["lr"],
                                              hp["b1"], hp["b2"], hp["eps"], wds[i], 0.5, None, 1))
    br.check(br.lib.mi355_sumsq_accum_multi_dev(ss2.ptr, parr(g2), narr, k, 0.5))
    br.check(br.lib.mi355_adam_update_multi_dev(parr(w2), parr(g2), parr(m2), parr(v2), narr, wdarr, k, hp["t"], hp["lr"],
                                                hp["b1"], hp["b2"], hp["eps"], 0.5, None, 1))
    assert abs(ss1.numpy()[0] - ss2.numpy()[0]) <= 2e-6 * ss1.numpy()[0]
    for i in range(k):
        assert np.array_equal(w1[i].numpy(), w2[i].numpy()) and np.array_equal(m1[i].numpy(), m2[i].numpy())
        assert np.array_equal(v1[i].numpy(), v2[i].numpy()) and not g2[i].numpy().any()
        rw, rm, rv = O.adam_update(ws[i], gs[i] * np.float32(0.5), ms[i], vs[i], wd=wds[i], **hp)
        assert H.rel_err(w2[i].numpy(), rw) <= TOL


@pytest.mark.parametrize("V,D,ntok", [(32000, 768, 20000), (300, 6, 500), (1000, 1024, 64)])
def test_vocab_compaction_bit_exact(br, V, D, ntok):
    data = H.zipf_ids(45, ntok, V).astype(np.uint16)
    _, c2f = O.vocab_map_build(data, V)
    CV = c2f.size
    E = H.normal(46, (V, D), 0, 0.02); g = H.normal(47, (CV, D)); G0 = H.normal(48, (V, D))
    Ed, md, gd, Gd = dev(br, E), dev(br, c2f), dev(br, g), dev(br, G0)
    ce = br.DevArray((CV, D))
    br.check(br.lib.mi355_vocab_compact_embed_dev(ce.ptr, Ed.ptr, md.ptr, CV, V, D))
    assert ce.numpy().tobytes() == O.vocab_compact_embed(E, c2f).tobytes()
    br.check(br.lib.mi355_vocab_scatter_grads_dev(Gd.ptr, gd.ptr, md.ptr, CV, V, D))
    assert Gd.numpy().tobytes() == O.vocab_scatter_grads(G0, g, c2f).tobytes()
    new = (ce.numpy() * np.float32(0.5)).astype(np.float32)
    nd = dev(br, new)
    br.check(br.lib.mi355_vocab_update_full_dev(Ed.ptr, nd.ptr, md.ptr, CV, V, D))
    assert Ed.numpy().tobytes() == O.vocab_update_full(E, new, c2f).tobytes()


@pytest.mark.parametrize("V,ntok", [(32000, 200000), (300, 500), (1000, 64), (5, 1000), (151936, 16384), (1031, 1)])
def test_vocab_map_build_and_remap_exact(br, V, ntok):
    """The map of training/training_dynamic/cpu_ops.h:102-126 built on the device, and the id remap of train.m:403."""
    data = H.zipf_ids(49, ntok, min(V, 65536)).astype(np.uint16)
    f2c, c2f = O.vocab_map_build(data, V)
    dd = br.DevArray.from_numpy(data)
    f2cd = br.DevArray(V, np.int32); c2fd = br.DevArray(V, np.int32); cvd = br.DevArray(1, np.int32)
    br.check(br.lib.mi355_vocab_map_build_dev(f2cd.ptr, c2fd.ptr, cvd.ptr, dd.ptr, ntok, V))
    cv = int(cvd.numpy()[0])
    assert cv == c2f.size
    assert np.array_equal(f2cd.numpy(), f2c) and np.array_equal(c2fd.numpy()[:cv], c2f)
    ids = np.concatenate([data.astype(np.int32), np.array([-1, V, V + 7, 0, V - 1], np.int32)])
    want = np.where((ids >= 0) & (ids < V), f2c[np.clip(ids, 0, V - 1)], -1).astype(np.int32)
    idd = br.DevArray.from_numpy(ids); od = br.DevArray(ids.size, np.int32)
    br.check(br.lib.mi355_vocab_remap_dev(od.ptr, idd.ptr, f2cd.ptr, ids.size, V))
    assert np.array_equal(od.numpy(), want)
    assert (od.numpy()[:ntok] >= 0).all()                      # every token of the data has a compact id


@pytest.mark.parametrize("B,kvh,ratio,hd,S", [(16, 8, 2, 128, 256), (2, 3, 4, 6, 5), (1, 1, 1, 4, 4)])
def test_gqa_tile_reduce(br, B, kvh, ratio, hd, S):
    k = H.normal(54, (B, kvh * hd, S)); g = H.normal(55, (B, kvh * ratio * hd, S))
    kd, gd = dev(br, k), dev(br, g)
    td = br.DevArray(g.shape); rd = br.DevArray(k.shape)
    br.check(br.lib.mi355_gqa_tile_dev(td.ptr, kd.ptr, kvh, ratio, hd, S, B))
    br.check(br.lib.mi355_gqa_reduce_dev(rd.ptr, gd.ptr, kvh, ratio, hd, S, B))
    for b in range(B):
        assert np.array_equal(td.numpy()[b], O.gqa_tile(k[b], kvh, ratio, hd))
        assert np.array_equal(rd.numpy()[b], O.gqa_reduce(g[b], kvh, ratio, hd))   # same add order: bit-exact


# ---------------------------------------------------------------------------------------------
# fp16 staging converts and the attention-gradient finish
# ---------------------------------------------------------------------------------------------
def test_cvt_f16_all_bit_patterns(br):
    allh = np.arange(65536, dtype=np.uint16)
    hd_ = dev(br, allh)
    fd = br.DevArray(allh.shape)
    br.check(br.lib.mi355_cvt_f16_f32_dev(fd.ptr, allh.size, hd_.ptr, allh.size, 1, allh.size))
    got, ref = fd.numpy(), O.cvt_f16_f32(allh)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    # and back: every non-NaN half is reproduced
    bd = br.DevArray(allh.shape, np.uint16)
    br.check(br.lib.mi355_cvt_f32_f16_dev(bd.ptr, allh.size, fd.ptr, allh.size, 1, allh.size))
    assert np.array_equal(bd.numpy()[~nan], allh[~nan])
    assert np.isnan(bd.numpy()[nan].view(np.float16)).all()


def test_cvt_f32_f16_rounding_boundaries(br):
    v = H.f16_boundary_values()
    rnd = np.random.default_rng(6).integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    v = np.concatenate([v, rnd[~np.isnan(rnd)]])
    v = v[:v.size // 8 * 8]
    vd = dev(br, v)
    od = br.DevArray(v.shape, np.uint16)
    br.check(br.lib.mi355_cvt_f32_f16_dev(od.ptr, v.size, vd.ptr, v.size, 1, v.size))
    assert np.array_equal(od.numpy(), O.cvt_f32_f16(v))


@pytest.mark.parametrize("rows,cols,dst_ld,src_ld", [(1024, 256, 256 + 3072, 256), (7, 13, 19, 13), (5, 16, 16, 24),
                                                     (3, 8, 12, 8)])
def test_cvt_rectangles(br, rows, cols, dst_ld, src_ld):
    """The packers write runs of `cols` elements at a row pitch (io_write_dyn: [ic, seq+oc] surfaces)."""
    src = H.normal(120, (rows, src_ld), 0, 30.0)
    dst0 = np.random.default_rng(121).integers(0, 65536, (rows, dst_ld)).astype(np.uint16)
    sd, dd = dev(br, src), dev(br, dst0)
    br.check(br.lib.mi355_cvt_f32_f16_dev(dd.ptr, dst_ld, sd.ptr, src_ld, rows, cols))
    want = dst0.copy()
    want[:, :cols] = O.cvt_f32_f16(src[:, :cols])
    assert np.array_equal(dd.numpy(), want)                       # converted rectangle, everything else untouched
    back0 = H.normal(122, (rows, src_ld))
    bd = dev(br, back0)
    br.check(br.lib.mi355_cvt_f16_f32_dev(bd.ptr, src_ld, dd.ptr, dst_ld, rows, cols))
    wantb = back0.copy()
    wantb[:, :cols] = O.cvt_f16_f32(want[:, :cols])
    assert np.array_equal(bd.numpy().view(np.uint32), wantb.view(np.uint32))


def _finish_reference(dq16, dk16, dv16, heads, kvh, hd, theta, in_f16, rotate=True):
    """train.m:646-660 with the oracle's pieces: read (convert), reduce dK and dV, copy dQ, un-rotate dQ and dK."""
    cv = O.cvt_f16_f32 if in_f16 else (lambda a: a)
    ratio = heads // kvh
    B = dq16.shape[0]
    dq = np.stack([cv(dq16[b]) for b in range(B)])
    dk = np.stack([O.gqa_reduce(cv(dk16[b]), kvh, ratio, hd) for b in range(B)])
    dv = np.stack([O.gqa_reduce(cv(dv16[b]), kvh, ratio, hd) for b in range(B)])
    if rotate:
        dq, dk = O.rope(dq, hd, theta, -1), O.rope(dk, hd, theta, -1)
    return dq, dk, dv


@pytest.mark.parametrize("B,heads,kvh,hd,S,in_f16", [(16, 16, 8, 128, 256, 1), (2, 12, 12, 64, 256, 1),
                                                      (2, 6, 2, 8, 24, 1), (1, 4, 2, 6, 5, 1), (1, 2, 1, 4, 7, 0),
                                                      (3, 8, 2, 16, 32, 0)])
def test_attn_grads_finish_equals_separate_steps(br, B, heads, kvh, hd, S, in_f16):
    theta = 1e6
    full = (B, heads * hd, S)
    src = [H.normal(130 + i, full) for i in range(3)]
    ins = [O.cvt_f32_f16(a) for a in src] if in_f16 else src
    ind = [dev(br, a) for a in ins]
    dq, dk, dv = br.DevArray(full), br.DevArray((B, kvh * hd, S)), br.DevArray((B, kvh * hd, S))
    cosd, sind = br.rope_tables_dev(S, hd, theta)
    br.check(br.lib.mi355_attn_grads_finish_dev(dq.ptr, dk.ptr, dv.ptr, ind[0].ptr, ind[1].ptr, ind[2].ptr, in_f16,
                                                0, 0, 0, heads, kvh, hd, S, B, cosd, sind))
    rq, rk, rv = _finish_reference(*ins, heads, kvh, hd, theta, in_f16)
    for got, ref in ((dq, rq), (dk, rk), (dv, rv)):
        assert np.array_equal(got.numpy().view(np.uint32), ref.view(np.uint32))
    # equals the library's own separate calls too
    if not in_f16:
        k2, q2 = br.DevArray((B, kvh * hd, S)), br.DevArray(full)
        br.check(br.lib.mi355_gqa_reduce_dev(k2.ptr, ind[1].ptr, kvh, heads // kvh, hd, S, B))
        br.check(br.lib.mi355_rope_dev(q2.ptr, k2.ptr, ind[0].ptr, k2.ptr, heads, kvh, hd, S, B, cosd, sind, -1))
        assert np.array_equal(q2.numpy(), dq.numpy()) and np.array_equal(k2.numpy(), dk.numpy())


def test_attn_grads_finish_surface_offsets_in_place_and_no_rotation(br):
    """dQ and dK as channel ranges of one [2*Q_DIM, S] fp16 surface per sequence (the layout the reference reads at
    train.m:647-648); fp32 in place; NULL tables leave the rotation out."""
    B, heads, kvh, hd, S, theta = 3, 4, 2, 8, 16, 1e4
    qd = heads * hd
    surf = O.cvt_f32_f16(H.normal(140, (B, 2 * qd, S)))
    dv16 = O.cvt_f32_f16(H.normal(141, (B, qd, S)))
    sd, vd = dev(br, surf), dev(br, dv16)
    dq, dk, dv = br.DevArray((B, qd, S)), br.DevArray((B, kvh * hd, S)), br.DevArray((B, kvh * hd, S))
    cosd, sind = br.rope_tables_dev(S, hd, theta)
    br.check(br.lib.mi355_attn_grads_finish_dev(dq.ptr, dk.ptr, dv.ptr, sd.ptr, sd.ptr + qd * S * 2, vd.ptr, 1,
                                                2 * qd * S, 2 * qd * S, 0, heads, kvh, hd, S, B, cosd, sind))
    rq, rk, rv = _finish_reference(surf[:, :qd], surf[:, qd:], dv16, heads, kvh, hd, theta, 1)
    assert np.array_equal(dq.numpy(), rq) and np.array_equal(dk.numpy(), rk) and np.array_equal(dv.numpy(), rv)

    src = [H.normal(142 + i, (B, qd, S)) for i in range(3)]
    qd_, kd_, vd_ = (dev(br, a) for a in src)
    br.check(br.lib.mi355_attn_grads_finish_dev(qd_.ptr, dk.ptr, dv.ptr, qd_.ptr, kd_.ptr, vd_.ptr, 0, 0, 0, 0, heads,
                                                kvh, hd, S, B, None, None))
    rq, rk, rv = _finish_reference(*src, heads, kvh, hd, theta, 0, rotate=False)
    assert np.array_equal(qd_.numpy(), rq) and np.array_equal(dk.numpy(), rk) and np.array_equal(dv.numpy(), rv)


def test_staging_bad_arguments(br):
    a = br.DevArray(64); h = br.DevArray(64, np.uint16)
    assert br.lib.mi355_cvt_f32_f16_dev(h.ptr, 4, a.ptr, 8, 2, 8) == -1            # pitch below the run length
    assert br.lib.mi355_cvt_f16_f32_dev(None, 8, h.ptr, 8, 1, 8) == -1
    assert br.lib.mi355_attn_grads_finish_dev(a.ptr, a.ptr, a.ptr, a.ptr, a.ptr, a.ptr, 0, 0, 0, 0, 3, 2, 4, 4, 1,
                                              None, None) == -1                    # heads not a multiple of kv_heads
    assert br.lib.mi355_attn_grads_finish_dev(a.ptr, a.ptr, a.ptr, a.ptr, a.ptr, a.ptr, 0, 0, 0, 0, 2, 2, 4, 4, 1,
                                              a.ptr, None) == -1                   # one table only
    assert "attn_grads_finish" in br.last_error()


# ---------------------------------------------------------------------------------------------
# cblas_sgemm call sites (classifier, weight gradients)
# ---------------------------------------------------------------------------------------------
def test_sgemm_classifier_products(br):
    """The three classifier products of train.m:490-508 at a compact-vocabulary shape."""
    CV, D, S = 4096, 1024, 256
    cembed = H.normal(160, (CV, D), 0, 0.02); x = H.normal(161, (D, S)); dlog = H.normal(162, (CV, S), 0, 1e-3)
    g0 = H.normal(163, (CV, D), 0, 1e-3)
    ed, xd, dd, gd = dev(br, cembed), dev(br, x), dev(br, dlog), dev(br, g0)
    logits, dy = br.DevArray((CV, S)), br.DevArray((D, S))
    br.check(br.lib.mi355_sgemm_dev(111, 111, CV, S, D, 1.0, ed.ptr, D, xd.ptr, S, 0.0, logits.ptr, S))
    br.check(br.lib.mi355_sgemm_dev(112, 111, D, S, CV, 1.0, ed.ptr, D, dd.ptr, S, 0.0, dy.ptr, S))
    br.check(br.lib.mi355_sgemm_dev(111, 112, CV, D, S, 1.0, dd.ptr, S, xd.ptr, S, 1.0, gd.ptr, D))
    assert H.rel_err(logits.numpy(), O.sgemm(0, 0, 1.0, cembed, x)) <= TOL
    assert H.rel_err(dy.numpy(), O.sgemm(1, 0, 1.0, cembed, dlog)) <= TOL
    assert H.rel_err(gd.numpy(), O.sgemm(0, 1, 1.0, dlog, x, 1.0, g0)) <= TOL


def test_classifier_head_chain_stays_on_device(br):
    """train.m:485-515 with every stage on the device: final RMSNorm, logits product, softmax-CE with the loss
    scale folded in, the two backward products, RMSNorm backward.  Each stage is checked against the oracle fed
    with the device result of the stage before it."""
    CV, D, S, loss_scale = 4099, 768, 256, 256.0
    x_cur = H.normal(180, (D, S)); w = H.normal(181, D, 1.0, 0.02); cembed = H.normal(182, (CV, D), 0, 0.02)
    tgt = np.random.default_rng(183).integers(0, CV, S).astype(np.int32)
    gce0 = H.normal(184, (CV, D), 0, 1e-3); grms0 = H.normal(185, D, 0, 1e-3)
    xd, wd, ed, td, gced, grmsd = (dev(br, a) for a in (x_cur, w, cembed, tgt, gce0, grms0))
    xf, logits, dlog, lossd = br.DevArray((D, S)), br.DevArray((CV, S)), br.DevArray((CV, S)), br.DevArray(1)
    dy, dx = br.DevArray((D, S)), br.DevArray((D, S))
    L = br.lib
    br.check(L.mi355_rmsnorm_fwd_dev(xf.ptr, xd.ptr, wd.ptr, D, S, 1, 1e-5))
    br.check(L.mi355_sgemm_dev(111, 111, CV, S, D, 1.0, ed.ptr, D, xf.ptr, S, 0.0, logits.ptr, S))
    br.check(L.mi355_softmax_ce_dev(dlog.ptr, lossd.ptr, logits.ptr, td.ptr, CV, S, loss_scale))
    br.check(L.mi355_sgemm_dev(112, 111, D, S, CV, 1.0, ed.ptr, D, dlog.ptr, S, 0.0, dy.ptr, S))
    br.check(L.mi355_sgemm_dev(111, 112, CV, D, S, 1.0, dlog.ptr, S, xf.ptr, S, 1.0, gced.ptr, D))
    br.check(L.mi355_rmsnorm_bwd_dev(dx.ptr, grmsd.ptr, dy.ptr, xd.ptr, wd.ptr, D, S, 1, 1e-5, 0))
    g_xf, g_logits, g_dlog, g_dy = xf.numpy(), logits.numpy(), dlog.numpy(), dy.numpy()
    assert H.rel_err(g_xf, O.rmsnorm(x_cur, w)) <= TOL
    assert H.rel_err(g_logits, O.sgemm(0, 0, 1.0, cembed, g_xf)) <= TOL
    r_loss, r_dlog = O.cross_entropy(g_logits, tgt, grad_scale=loss_scale)
    assert abs(float(lossd.numpy()[0]) - r_loss) <= TOL * abs(r_loss) and H.rel_err(g_dlog, r_dlog) <= TOL
    assert H.rel_err(g_dy, O.sgemm(1, 0, 1.0, cembed, g_dlog)) <= TOL
    assert H.rel_err(gced.numpy(), O.sgemm(0, 1, 1.0, g_dlog, g_xf, 1.0, gce0)) <= TOL
    r_dx, r_grms = O.rmsnorm_bwd(g_dy, x_cur, w, dw=grms0)
    assert H.rel_err(dx.numpy(), r_dx) <= TOL and H.rel_err(grmsd.numpy(), r_grms) <= TOL
    # end to end against the all-oracle chain: error compounds over six stages, so a looser bound
    o_xf = O.rmsnorm(x_cur, w); o_loss, o_dlog = O.cross_entropy(O.sgemm(0, 0, 1.0, cembed, o_xf), tgt, grad_scale=loss_scale)
    o_dx, _ = O.rmsnorm_bwd(O.sgemm(1, 0, 1.0, cembed, o_dlog), x_cur, w, dw=grms0)
    assert H.rel_err(dx.numpy(), o_dx) <= 1e-4 and abs(float(lossd.numpy()[0]) - o_loss) <= 1e-5 * abs(o_loss)


def test_sgemm_reference_test_recipes(br):
    """The inputs of the reference's own classifier tests at their own size (VOCAB 32000, DIM 768, SEQ 256):
    forward training/test_classifier.m:60-69 (srand48(123)), backward :205-214 (srand48(456)).  The reference
    compares against an fp16 accelerator at 0.05-1.0 absolute; here the product is checked at 1e-5."""
    V, D, S = 32000, 768, 256
    x, _, emb = O.recipe_drand48(3, 123, D * S, V * D)
    x = x.reshape(D, S); emb = emb.reshape(V, D)
    xd, ed = dev(br, x), dev(br, emb)
    logits = br.DevArray((V, S))
    br.check(br.lib.mi355_sgemm_dev(111, 111, V, S, D, 1.0, ed.ptr, D, xd.ptr, S, 0.0, logits.ptr, S))
    assert H.rel_err(logits.numpy(), O.sgemm(0, 0, 1.0, emb, x)) <= TOL
    dlog, _, emb2 = O.recipe_drand48(4, 456, V * S, V * D)
    dlog = dlog.reshape(V, S); emb2 = emb2.reshape(V, D)
    dd, e2d = dev(br, dlog), dev(br, emb2)
    dx = br.DevArray((D, S))
    br.check(br.lib.mi355_sgemm_dev(112, 111, D, S, V, 1.0, e2d.ptr, D, dd.ptr, S, 0.0, dx.ptr, S))
    assert H.rel_err(dx.numpy(), O.sgemm(1, 0, 1.0, emb2, dlog)) <= TOL


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_sgemm_pitched_operands(br, ta, tb):
    M, N, K, pad = 45, 70, 33, 5
    A = H.normal(170, ((K, M + pad) if ta else (M, K + pad))); B = H.normal(171, ((N, K + pad) if tb else (K, N + pad)))
    C0 = H.normal(172, (M, N + pad))
    ad, bd, cd = dev(br, A), dev(br, B), dev(br, C0)
    br.check(br.lib.mi355_sgemm_dev(ta, tb, M, N, K, 0.5, ad.ptr, A.shape[1], bd.ptr, B.shape[1], 2.0, cd.ptr, N + pad))
    Ao = A[:, :M] if ta else A[:, :K]; Bo = B[:, :K] if tb else B[:, :N]
    want = C0.copy()
    want[:, :N] = O.sgemm(ta, tb, 0.5, Ao, Bo, 2.0, C0[:, :N])
    got = cd.numpy()
    assert H.rel_err(got[:, :N], want[:, :N]) <= TOL
    assert np.array_equal(got[:, N:], C0[:, N:])                          # padding columns untouched


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_sgemm_long_inner_dimension_is_split_deterministically(br, ta, tb):
    """Small output, long K (the dy = cembed^T . dlogits shape): the K-sliced path, including a ragged last slice."""
    M, N, K = 96, 64, 9001
    A = H.normal(190, (K, M) if ta else (M, K)); B = H.normal(191, (N, K) if tb else (K, N)); C0 = H.normal(192, (M, N))
    ad, bd = dev(br, A), dev(br, B)
    outs = []
    for knob in (0, 7, 1):                                           # automatic, forced 7 slices, unsplit
        br.tune("gemm_splitk", knob)
        for beta in (0.0, -0.5):
            cd = dev(br, C0)
            br.check(br.lib.mi355_sgemm_dev(ta, tb, M, N, K, 0.75, ad.ptr, A.shape[1], bd.ptr, B.shape[1], beta, cd.ptr, N))
            got = cd.numpy()
            assert H.rel_err(got, O.sgemm(ta, tb, 0.75, A, B, beta, C0)) <= TOL, (knob, beta)
            cd2 = dev(br, C0)
            br.check(br.lib.mi355_sgemm_dev(ta, tb, M, N, K, 0.75, ad.ptr, A.shape[1], bd.ptr, B.shape[1], beta, cd2.ptr, N))
            assert cd2.numpy().tobytes() == got.tobytes()            # same bits on a second run
    br.tune("gemm_splitk", 0)


def test_sgemm_bad_arguments(br):
    a = br.DevArray(64)
    assert br.lib.mi355_sgemm_dev(0, 0, 4, 4, 4, 1.0, a.ptr, 3, a.ptr, 4, 0.0, a.ptr, 4) == -1
    assert br.lib.mi355_sgemm_dev(2, 0, 4, 4, 4, 1.0, a.ptr, 4, a.ptr, 4, 0.0, a.ptr, 4) == -1
    assert br.lib.mi355_sgemm_dev(0, 0, 0, 4, 4, 1.0, a.ptr, 4, a.ptr, 4, 0.0, a.ptr, 4) == -1
    assert "sgemm" in br.last_error()


# ---------------------------------------------------------------------------------------------
# checkpoints: file <-> device memory
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("version", [4, 2])
def test_checkpoint_load_store_round_trip(br, tmp_path, version):
    import ctypes
    cfg = dict(layers=2, vocab=300, dim=64, hidden=160, heads=4, kv_heads=2 if version == 4 else 4,
               head_dim=24 if version == 4 else 16, q_dim=96 if version == 4 else 64, kv_dim=48 if version == 4 else 64,
               seq=32)
    src = str(tmp_path / "src.bin"); dst = str(tmp_path / "dst.bin")
    tensors = H.ckpt_write_like_reference(src, cfg, version, seed=3)
    hdr = br.CkptHdr()
    br.check(br.lib.mi355_ckpt_read_header(src.encode(), ctypes.byref(hdr)))
    br.check(br.lib.mi355_ckpt_create(dst.encode(), ctypes.byref(hdr)))
    # every tensor: file -> device (compare with what the writer put there) -> new file, in reverse order
    for (L, t, part), a in reversed(list(tensors.items())):
        off, cnt = ctypes.c_uint64(), ctypes.c_uint64()
        br.check(br.lib.mi355_ckpt_locate(ctypes.byref(hdr), L, t, part, ctypes.byref(off), ctypes.byref(cnt)))
        d = br.DevArray(cnt.value)
        br.check(br.lib.mi355_ckpt_load_dev(src.encode(), off.value, d.ptr, cnt.value))
        assert d.numpy().tobytes() == a.tobytes(), (L, t, part)
        br.check(br.lib.mi355_ckpt_store_dev(dst.encode(), off.value, d.ptr, cnt.value))
    assert open(dst, "rb").read() == open(src, "rb").read()                  # byte-identical checkpoint
    d = br.DevArray(16)
    assert br.lib.mi355_ckpt_load_dev(src.encode(), os.path.getsize(src) - 8, d.ptr, 16) == -1   # runs off the end
    assert br.lib.mi355_ckpt_store_dev(str(tmp_path / "absent.bin").encode(), 96, d.ptr, 16) == -1


# ---------------------------------------------------------------------------------------------
# host-pointer drop-ins (reference signatures) and error behaviour
# ---------------------------------------------------------------------------------------------
def _p(a):
    return a.ctypes.data


def test_host_dropins_match_oracle(br):
    Cc, S = 768, 256
    x = H.normal(90, (Cc, S)); w = H.normal(91, Cc, 1.0, 0.02); dy = H.normal(92, (Cc, S))
    out = np.empty_like(x)
    br.lib.mi355_rmsnorm(_p(out), _p(x), _p(w), Cc, S)
    assert H.rel_err(out, O.rmsnorm(x, w)) <= TOL
    dx = np.zeros_like(x); dw = H.normal(93, Cc); dw_in = dw.copy()
    br.lib.mi355_rmsnorm_bwd(_p(dx), _p(dw), _p(dy), _p(x), _p(w), Cc, S)
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, dw=dw_in)
    assert H.rel_err(dx, rdx) <= TOL and H.rel_err(dw, rdw) <= TOL

    V = 5000
    logits = H.normal(94, (V, S), 0, 2.0)
    tg = np.random.default_rng(95).integers(0, V, S).astype(np.uint16)
    dl = np.empty_like(logits)
    loss = br.lib.mi355_cross_entropy_loss(_p(dl), _p(logits), _p(tg), V, S)
    rl, rd = O.cross_entropy(logits, tg.astype(np.int32))
    assert abs(loss - rl) <= TOL * abs(rl) and H.rel_err(dl, rd) <= TOL

    D = 96
    E = H.normal(96, (V, D), 0, 0.02)
    tok = H.zipf_ids(97, S, V).astype(np.uint16)
    xo = np.zeros((D, S), np.float32)
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()
    E2 = E.copy(); E2[tok[0]] += 1                                     # the optimizer changed the table
    E[...] = E2
    br.lib.mi355_host_table_invalidate(_p(E))
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()
    g = H.normal(98, (D, S)); dE = H.normal(99, (V, D)); dE_in = dE.copy()
    br.lib.mi355_embed_backward(_p(dE), _p(g), _p(tok), V, D, S)
    assert dE.tobytes() == O.embed_backward(dE_in, g[None], tok.astype(np.int32)[None]).tobytes()

    dq = H.normal(100, (12 * 64, S)); dq_in = dq.copy()
    br.lib.mi355_rope_backward_inplace(_p(dq), S, 12 * 64, 64)
    assert np.array_equal(dq, O.rope(dq_in, 64, 10000.0, -1))


def test_host_vocab_dropins_and_table_coherence(br):
    """vocab_map_build / vocab_compact_embed / vocab_scatter_grads / vocab_update_full on host arrays
    (training/training_dynamic/cpu_ops.h:96-148), and the resident copy of the embedding table staying current when
    adam_update rewrites the host table (training/training_dynamic/train.m:869-871 followed by :405 of the next step)."""
    V, D, S = 3000, 96, 64
    data = H.zipf_ids(110, 5000, V).astype(np.uint16)
    f2c = np.full(V, 7, np.int32); c2f = np.full(V, -5, np.int32)
    cv = br.lib.mi355_vocab_map_build(_p(f2c), _p(c2f), _p(data), data.size, V)
    rf2c, rc2f = O.vocab_map_build(data, V)
    assert cv == rc2f.size and np.array_equal(f2c, rf2c) and np.array_equal(c2f[:cv], rc2f)
    E = H.normal(111, (V, D), 0, 0.02)
    ce = np.zeros((cv, D), np.float32)
    br.lib.mi355_vocab_compact_embed(_p(ce), _p(E), _p(c2f), cv, V, D)
    assert ce.tobytes() == O.vocab_compact_embed(E, rc2f).tobytes()
    G = H.normal(112, (V, D)); G_in = G.copy(); gc = H.normal(113, (cv, D))
    br.lib.mi355_vocab_scatter_grads(_p(G), _p(gc), _p(c2f), cv, V, D)
    assert G.tobytes() == O.vocab_scatter_grads(G_in, gc, rc2f).tobytes()
    # the table is resident now; an Adam step on the host array must reach the next lookup and the next compaction
    tok = data[:S].copy()
    xo = np.zeros((D, S), np.float32)
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()
    g = H.normal(114, (V, D)); m = np.zeros((V, D), np.float32); v = np.zeros((V, D), np.float32)
    E_before = E.copy()
    br.lib.mi355_adam_update(_p(E), _p(g), _p(m), _p(v), E.size, 1, 1e-2, 0.9, 0.95, 1e-8, 0.1)
    assert np.abs(E - E_before).max() > 1e-3
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()      # not the rows of before
    br.lib.mi355_vocab_compact_embed(_p(ce), _p(E), _p(c2f), cv, V, D)
    assert ce.tobytes() == O.vocab_compact_embed(E, rc2f).tobytes()
    # ... also a step on some rows only (the resident copy takes them on the device), and one on a range that runs
    # past the table's end (the copy is uploaded again)
    rows = slice(100, 1200)
    n_sub = E[rows].size
    br.lib.mi355_adam_update(_p(E[rows]), _p(g[rows]), _p(m[rows]), _p(v[rows]), n_sub, 2, 1e-2, 0.9, 0.95, 1e-8, 0.1)
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()
    big = np.concatenate([E.ravel(), np.zeros(D, np.float32)]); E2 = big[:V * D].reshape(V, D)
    br.lib.mi355_embed_lookup(_p(xo), _p(E2), _p(tok), V, D, S)                         # a second resident table
    tail = big[(V - 3) * D:]; zt = np.zeros_like(tail)
    br.lib.mi355_adam_update(_p(tail), _p(np.ones_like(tail)), _p(zt), _p(zt.copy()), tail.size, 1, 1e-2, 0.9, 0.95, 1e-8, 0.0)
    tok2 = np.full(S, V - 1, np.uint16)
    br.lib.mi355_embed_lookup(_p(xo), _p(E2), _p(tok2), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E2, tok2.astype(np.int32))[0][0].tobytes()
    # update_full writes the host rows and keeps the resident copy current
    new = (ce * np.float32(0.5)).astype(np.float32); E_in = E.copy()
    br.lib.mi355_vocab_update_full(_p(E), _p(new), _p(c2f), cv, V, D)
    assert E.tobytes() == O.vocab_update_full(E_in, new, rc2f).tobytes()
    br.lib.mi355_embed_lookup(_p(xo), _p(E), _p(tok), V, D, S)
    assert xo.tobytes() == O.embed_lookup(E, tok.astype(np.int32))[0][0].tobytes()
    # data with ids past the vocabulary are ignored (the reference's scan would write out of bounds)
    small_v = 1000
    f2 = np.zeros(small_v, np.int32); c2 = np.zeros(small_v, np.int32)
    cv2 = br.lib.mi355_vocab_map_build(_p(f2), _p(c2), _p(data), data.size, small_v)
    rf2, rc2 = O.vocab_map_build(data[data < small_v], small_v)
    assert cv2 == rc2.size and np.array_equal(f2, rf2) and np.array_equal(c2[:cv2], rc2)


@pytest.mark.parametrize("V,S", [(32000, 256), (37, 12), (1000, 5), (4099, 64)])
def test_column_softmax_and_nll_from_probs(br, V, S):
    """The two halves of the classifier loss as training/train_large_ane.m:508-530 runs them."""
    say("softmax_cols / nll_from_probs V=%d S=%d" % (V, S))
    logits = H.normal(120, (V, S), 0, 2.0)
    tgt = np.random.default_rng(121).integers(0, V, S).astype(np.int32)
    if S > 4:
        tgt[1] = V; tgt[3] = -1
    ld, td = dev(br, logits), dev(br, tgt)
    pd = br.DevArray(logits.shape); dd = br.DevArray(logits.shape); lossd = br.DevArray(1)
    br.check(br.lib.mi355_softmax_cols_dev(pd.ptr, ld.ptr, V, S))
    p = pd.numpy()
    rp = O.softmax_cols(logits)
    assert H.err_elem(p, rp) <= TOL
    l64 = logits.astype(np.float64); e = np.exp(l64 - l64.max(axis=0))
    assert H.err_elem(p, e / e.sum(axis=0)) <= TOL
    br.check(br.lib.mi355_nll_from_probs_dev(dd.ptr, lossd.ptr, pd.ptr, td.ptr, V, S))
    rl, rd = O.nll_from_probs(p, tgt)                   # same probabilities in: the op is exact fp32 arithmetic
    assert abs(float(lossd.numpy()[0]) - rl) <= TOL * abs(rl)
    assert np.array_equal(dd.numpy(), rd)
    # against the fused op on valid targets
    ok = (tgt >= 0) & (tgt < V)
    fl, fd = O.cross_entropy(logits, np.where(ok, tgt, 0).astype(np.int32))
    assert H.err_std(dd.numpy()[:, ok], fd[:, ok]) <= TOL
    # in place: probabilities over the logits, gradient over the probabilities
    br.check(br.lib.mi355_softmax_cols_dev(ld.ptr, ld.ptr, V, S))
    assert np.array_equal(ld.numpy(), p)
    br.check(br.lib.mi355_nll_from_probs_dev(ld.ptr, lossd.ptr, ld.ptr, td.ptr, V, S))
    assert np.array_equal(ld.numpy(), rd) and abs(float(lossd.numpy()[0]) - rl) <= TOL * abs(rl)


def test_bad_arguments_fail_cleanly(br):
    x = dev(br, np.ones((4, 8), np.float32)); y = dev(br, np.full((4, 8), 5.0, np.float32))
    w = dev(br, np.ones(4, np.float32))
    assert br.lib.mi355_rmsnorm_fwd_dev(y.ptr, None, w.ptr, 4, 8, 1, 1e-5) == -1
    assert "NULL" in br.last_error()
    assert br.lib.mi355_rmsnorm_fwd_dev(y.ptr, x.ptr, w.ptr, 0, 8, 1, 1e-5) == -1
    assert br.lib.mi355_rmsnorm_bwd_dev(y.ptr, w.ptr, x.ptr, x.ptr, w.ptr, 4, 8, 1, 1e-5, 2) == -1
    assert br.lib.mi355_swiglu_fwd_dev(y.ptr, x.ptr, x.ptr, 0) == -1
    assert br.lib.mi355_axpby_dev(y.ptr, x.ptr, None, 1.0, 32, 0) == -1
    assert br.lib.mi355_axpby_dev(y.ptr, x.ptr, x.ptr, 1.0, 32, 5) == -1
    assert br.lib.mi355_softmax_ce_dev(y.ptr, None, x.ptr, x.ptr, 4, 8, 1.0) == -1
    assert br.lib.mi355_int8_quant_dev(y.ptr, x.ptr, w.ptr, 32, 3) == -1
    assert br.lib.mi355_rope_dev(y.ptr, None, x.ptr, None, 1, 0, 3, 8, 1, x.ptr, x.ptr, 1) == -1     # odd head_dim
    assert br.lib.mi355_embed_gather_dev(y.ptr, x.ptr, None, 4, 8, 1, 1) == -1
    assert np.array_equal(y.numpy(), np.full((4, 8), 5.0, np.float32))   # outputs untouched
    assert br.lib.mi355_tune_set(b"no_such_knob", 1) == -1
    # buffer accessors ignore bad ranges, as the reference's write_input/read_output do
    junk = np.zeros(4, np.float32)
    br.lib.mi355_buf_write(y.handle, 10 ** 9, junk.ctypes.data, 16)
    br.lib.mi355_buf_read(None, 0, junk.ctypes.data, 16)
    br.lib.mi355_buf_free(None)
    assert np.array_equal(y.numpy(), np.full((4, 8), 5.0, np.float32))
