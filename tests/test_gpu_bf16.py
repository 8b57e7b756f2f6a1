"""Optional bfloat16-storage variants: parity with the fp32 oracle run on the same bf16-representable inputs,
within 5e-3 (the tolerance stated for bf16 variants); the converts themselves are bit-exact."""
import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu
TOL16 = 5e-3


def bf(a):
    """fp32 array -> (bf16 bit patterns, the fp32 values they stand for)."""
    bits = O.cvt_f32_bf16(a)
    return bits, O.cvt_bf16_f32(bits)


def dev(br, a):
    return br.DevArray.from_numpy(a)


def back(d):
    return O.cvt_bf16_f32(d.numpy())


@pytest.mark.parametrize("rows,cols,dst_ld,src_ld", [(1, 1 << 20, 1 << 20, 1 << 20), (7, 13, 19, 13), (5, 16, 16, 24)])
def test_bf16_converts_bit_exact(br, rows, cols, dst_ld, src_ld):
    src = H.normal(200, (rows, src_ld), 0, 30.0)
    if cols >= 4096:
        b = H.f16_boundary_values()
        ties = (np.arange(0x3f80, 0x4080, dtype=np.uint32) << 16 | 0x8000).view(np.float32)
        src[0, :b.size] = b; src[0, b.size:b.size + ties.size] = ties
    dst0 = np.random.default_rng(201).integers(0, 65536, (rows, dst_ld)).astype(np.uint16)
    sd, dd = dev(br, src), dev(br, dst0)
    br.check(br.lib.mi355_cvt_f32_bf16_dev(dd.ptr, dst_ld, sd.ptr, src_ld, rows, cols))
    want = dst0.copy(); want[:, :cols] = O.cvt_f32_bf16(src[:, :cols])
    assert np.array_equal(dd.numpy(), want)
    b0 = H.normal(202, (rows, src_ld)); bd = dev(br, b0)
    br.check(br.lib.mi355_cvt_bf16_f32_dev(bd.ptr, src_ld, dd.ptr, dst_ld, rows, cols))
    wb = b0.copy(); wb[:, :cols] = O.cvt_bf16_f32(want[:, :cols])
    assert np.array_equal(bd.numpy().view(np.uint32), wb.view(np.uint32))


@pytest.mark.parametrize("n", [16 * 3072 * 256, 2048 * 256, 1003, 8])
def test_swiglu_and_residual_bf16(br, n):
    print("[case] bf16 swiglu/axpby n=%d" % n, flush=True)
    (h1b, h1), (h3b, h3), (db, d) = bf(H.normal(210, n)), bf(H.normal(211, n)), bf(H.normal(212, n))
    h1d, h3d, dd = dev(br, h1b), dev(br, h3b), dev(br, db)
    out, o1, o3 = (br.DevArray(n, np.uint16) for _ in range(3))
    br.check(br.lib.mi355_swiglu_fwd_bf16_dev(out.ptr, h1d.ptr, h3d.ptr, n))
    assert H.rel_err(back(out), O.swiglu_fwd(h1, h3)) <= TOL16
    br.check(br.lib.mi355_swiglu_bwd_bf16_dev(o1.ptr, o3.ptr, dd.ptr, h1d.ptr, h3d.ptr, n))
    r1, r3 = O.swiglu_bwd(d, h1, h3)
    assert H.rel_err(back(o1), r1) <= TOL16 and H.rel_err(back(o3), r3) <= TOL16
    # the stored values are the correctly rounded fp32 results: identical to rounding the oracle's output
    assert np.mean(out.numpy() == O.cvt_f32_bf16(O.swiglu_fwd(h1, h3))) > 0.999
    al = np.float32(24 ** 0.25)
    for mode, ref in ((0, O.axpby(h1, h3, al, 0)), (1, O.axpby(h1, None, al, 1)), (2, O.axpby(h1, h3, 0.0, 2))):
        y = br.DevArray(n, np.uint16)
        br.check(br.lib.mi355_axpby_bf16_dev(y.ptr, h1d.ptr, None if mode == 1 else h3d.ptr, al, n, mode))
        assert np.array_equal(y.numpy(), O.cvt_f32_bf16(ref))          # exact fp32 arithmetic, one rounding
    br.check(br.lib.mi355_axpby_bf16_dev(h1d.ptr, h1d.ptr, h3d.ptr, al, n, 0))          # in place
    assert np.array_equal(h1d.numpy(), O.cvt_f32_bf16(O.axpby(h1, h3, al, 0)))


@pytest.mark.parametrize("B,C,S", [(16, 1024, 256), (1, 768, 256), (2, 100, 37), (3, 48, 24), (2, 5000, 64), (5, 128, 256),
                                   (2, 300, 16), (1, 2048, 8), (1, 1, 8), (64, 1024, 256), (70, 640, 256)])
def test_rmsnorm_bf16(br, B, C, S):
    print("[case] bf16 rmsnorm B=%d C=%d S=%d" % (B, C, S), flush=True)
    (xb, x), (dyb, dy) = bf(H.normal(220, (B, C, S))), bf(H.normal(221, (B, C, S)))
    w = H.normal(222, C, 1.0, 0.02); dw0 = H.normal(223, C)
    xd, dyd, wd = dev(br, xb), dev(br, dyb), dev(br, w)
    y, dx = br.DevArray(x.shape, np.uint16), br.DevArray(x.shape, np.uint16)
    br.check(br.lib.mi355_rmsnorm_fwd_bf16_dev(y.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5))
    assert H.rel_err(back(y), O.rmsnorm(x, w)) <= TOL16
    for variant in (0, 1):
        dwd = dev(br, dw0)
        br.check(br.lib.mi355_rmsnorm_bwd_bf16_dev(dx.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5, variant))
        rdx, rdw = O.rmsnorm_bwd(dy, x, w, variant=variant, dw=dw0)
        assert H.rel_err(back(dx), rdx) <= TOL16
        assert H.rel_err(dwd.numpy(), rdw) <= 1e-5                      # fp32 in, fp32 sums, fp32 out


@pytest.mark.parametrize("B,C,S", [(16, 1024, 256), (1, 768, 256), (2, 1000, 200), (3, 520, 136), (1, 2048, 8), (2, 100, 37),
                                   (3, 48, 24), (2, 5000, 64), (40, 1024, 256)])
def test_rmsnorm_residual_fusions_bf16(br, B, C, S):
    """The residual add fused with the RMSNorm after it (training/training_dynamic/train.m:460-461) and the RMSNorm
    backward with the backward residual and the scaled copy riding along (train.m:586-595), bf16 storage: within 5e-3
    of the fp32 oracle run on the same bf16-representable inputs; y itself equals the rounded oracle sum to the bit;
    the clustered kernels give the same bits whichever way their exchange goes; in place (y over a, dx over res, dx
    over dy) the same values."""
    print("[case] bf16 residual+rmsnorm fusions B=%d C=%d S=%d" % (B, C, S), flush=True)
    (ab, a), (bb, b) = bf(H.normal(260, (B, C, S))), bf(H.normal(261, (B, C, S)))
    (dyb, dy), (rb, res) = bf(H.normal(262, (B, C, S))), bf(H.normal(263, (B, C, S)))
    w = H.normal(264, C, 1.0, 0.02); dw0 = H.normal(265, C)
    alpha = np.float32(1 / np.sqrt(2 * 28))
    ad, bd, dyd, rd, wd = (dev(br, v) for v in (ab, bb, dyb, rb, w))
    ysum = O.axpby(a, b, alpha, 0)
    yb_ref, y_ref = bf(ysum)                                             # the stored y: the fp32 sum rounded once
    yn_ref = O.rmsnorm(y_ref, w)
    rdx, rdw = O.rmsnorm_bwd(dy, a, w, dw=dw0)
    dx_ref = O.axpby(rdx, res, 0.0, 2)
    dxs_ref = O.axpby(dx_ref, None, alpha, 1)

    def run_all(in_place=0):
        y, yn = br.DevArray(a.shape, np.uint16), br.DevArray(a.shape, np.uint16)
        dx, dxs = br.DevArray(a.shape, np.uint16), br.DevArray(a.shape, np.uint16)
        dwd = dev(br, dw0)
        a2 = dev(br, ab) if in_place else ad
        r2 = dev(br, rb) if in_place == 1 else rd
        g2 = dev(br, dyb) if in_place == 2 else dyd
        yo = a2 if in_place else y
        dxo = r2 if in_place == 1 else g2 if in_place == 2 else dx
        br.check(br.lib.mi355_residual_rmsnorm_fwd_bf16_dev(yo.ptr, yn.ptr, a2.ptr, bd.ptr, alpha, wd.ptr, C, S, B, 1e-5))
        br.check(br.lib.mi355_rmsnorm_bwd_residual_bf16_dev(dxo.ptr, dxs.ptr, dwd.ptr, g2.ptr, ad.ptr, wd.ptr, r2.ptr, alpha,
                                                           C, S, B, 1e-5, 0))
        return [v.numpy() for v in (yo, yn, dxo, dxs, dwd)]

    def check(out, what):
        y, yn, dx, dxs, dwv = out
        assert np.array_equal(y, yb_ref), what
        assert H.rel_err(O.cvt_bf16_f32(yn), yn_ref) <= TOL16, what
        assert H.rel_err(O.cvt_bf16_f32(dx), dx_ref) <= TOL16 and H.rel_err(O.cvt_bf16_f32(dxs), dxs_ref) <= TOL16, what
        assert H.rel_err(dwv, rdw) <= 1e-5, what

    try:
        got = run_all()
        check(got, "out of place")
        expired = br.exchange_fallbacks()[0]
        again = run_all()
        assert all(u.tobytes() == v.tobytes() for u, v in zip(got, again))
        assert br.exchange_fallbacks()[0] == expired
        br.tune("xch_take_nothing", 1)                                   # every workgroup computes its partners' sums itself
        refused = run_all()
        assert all(u.tobytes() == v.tobytes() for u, v in zip(got, refused))
        if (B, C, S) == (16, 1024, 256):
            assert br.exchange_fallbacks()[0] > expired                  # (the named shape runs clustered)
        br.tune("xch_take_nothing", 0)
        for mode in (1, 2):
            check(run_all(mode), "in place %d" % mode)
        dwd = dev(br, dw0); dx = br.DevArray(a.shape, np.uint16)         # no scaled copy asked for
        br.check(br.lib.mi355_rmsnorm_bwd_residual_bf16_dev(dx.ptr, None, dwd.ptr, dyd.ptr, ad.ptr, wd.ptr, rd.ptr, alpha, C, S,
                                                           B, 1e-5, 1))
        rdx1, _ = O.rmsnorm_bwd(dy, a, w, variant=1, dw=dw0)
        assert H.rel_err(back(dx), O.axpby(rdx1, res, 0.0, 2)) <= TOL16
    finally:
        br.tune("xch_take_nothing", 0)
    assert br.lib.mi355_rmsnorm_bwd_residual_bf16_dev(ad.ptr, None, wd.ptr, dyd.ptr, ad.ptr, wd.ptr, rd.ptr, alpha, C, S, B,
                                                      1e-5, 0) == -1      # dx over x
    y = br.DevArray(a.shape, np.uint16)
    assert br.lib.mi355_residual_rmsnorm_fwd_bf16_dev(y.ptr, y.ptr, ad.ptr, bd.ptr, alpha, wd.ptr, C, S, B, 1e-5) == -1


@pytest.mark.parametrize("B,C,S", [(16, 1024, 256), (1, 768, 256), (2, 1000, 200), (3, 520, 136), (1, 2048, 8)])
def test_rmsnorm_bf16_clustered_every_split_and_the_expired_wait(br, B, C, S):
    """The bf16-storage norm with the channel axis split over 2, 4 or 8 cooperating workgroups (and the library's own
    choice): against the oracle, equal to the bit whatever the split's bounded wait does, and run-to-run."""
    print("[case] bf16 rmsnorm clustered B=%d C=%d S=%d" % (B, C, S), flush=True)
    (xb, x), (dyb, dy) = bf(H.normal(230, (B, C, S))), bf(H.normal(231, (B, C, S)))
    w = H.normal(232, C, 1.0, 0.02); dw0 = H.normal(233, C)
    xd, dyd, wd = dev(br, xb), dev(br, dyb), dev(br, w)
    ry = O.rmsnorm(x, w)
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, dw=dw0)

    def run_all():
        y, dx = br.DevArray(x.shape, np.uint16), br.DevArray(x.shape, np.uint16)
        dwd = dev(br, dw0)
        br.check(br.lib.mi355_rmsnorm_fwd_bf16_dev(y.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5))
        br.check(br.lib.mi355_rmsnorm_bwd_bf16_dev(dx.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5, 0))
        return [a.numpy() for a in (y, dx, dwd)]

    try:
        for split in (0, 2, 4, 8):
            br.tune("rms_cluster", split); br.tune("rms_cluster_spin", 0)
            got = run_all()
            y, dx, dwv = got
            assert H.rel_err(O.cvt_bf16_f32(y), ry) <= TOL16, split
            assert H.rel_err(O.cvt_bf16_f32(dx), rdx) <= TOL16 and H.rel_err(dwv, rdw) <= 1e-5, split
            expired = br.exchange_fallbacks()[0]
            again = run_all()
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, again)), split
            assert br.exchange_fallbacks()[0] == expired, split         # every column sum came from the partners
            br.tune("rms_cluster_spin", -1)                              # the wait expires before it starts
            alone = run_all()
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, alone)), split
            br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 1)
            refused = run_all()                                          # every workgroup computes its partners' sums itself
            assert all(a.tobytes() == b.tobytes() for a, b in zip(got, refused)), split
            moved = br.exchange_fallbacks()[0] - expired
            if (split == 0 and (B, C, S) == (16, 1024, 256)) or (split and -(-C // split) <= 256):
                assert moved > 0, split      # (a member holds at most 256 rows; the library splits the named shape itself)
            br.tune("xch_take_nothing", 0)
    finally:
        br.tune("rms_cluster", 0); br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)
    br.tune("rms_cluster", -1)                                           # never clustered: the single-workgroup tiles
    try:
        y, dx, dwv = run_all()
        assert H.rel_err(O.cvt_bf16_f32(y), ry) <= TOL16 and H.rel_err(O.cvt_bf16_f32(dx), rdx) <= TOL16
    finally:
        br.tune("rms_cluster", 0)
    # in place (dx over dy) the single-workgroup tile runs
    dy2 = dev(br, dyb); dwd = dev(br, dw0)
    br.check(br.lib.mi355_rmsnorm_bwd_bf16_dev(dy2.ptr, dwd.ptr, dy2.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5, 0))
    assert H.rel_err(back(dy2), rdx) <= TOL16


@pytest.mark.parametrize("V,S", [(4099, 64), (32000, 256), (151936, 256), (700, 128), (9000, 1024), (5000, 192)])
def test_softmax_ce_bf16_one_launch_and_its_expired_wait(br, V, S):
    """The bf16 instance of the kernel that keeps the logits on the chip between the passes (every row of
    [151936,256] fits): against the oracle, the same bits run to run, with the bounded wait expired at once and with
    no partner's value taken at all; close to the three-launch form."""
    print("[case] bf16 softmax_ce one launch V=%d S=%d" % (V, S), flush=True)
    lb, logits = bf(H.normal(250, (V, S), 0, 2.0))
    tgt = np.random.default_rng(251).integers(0, V, S).astype(np.int32)
    tgt[1] = V; tgt[S - 2] = -1
    ld, td = dev(br, lb), dev(br, tgt)

    def run():
        dl, lossd = br.DevArray((V, S), np.uint16), br.DevArray(1)
        br.check(br.lib.mi355_softmax_ce_bf16_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
        return lossd.numpy().copy(), dl.numpy()

    try:
        br.tune("ce_resident", 1); br.tune("rms_cluster_spin", 0)
        loss, dl = run()
        rl, rd = O.cross_entropy(logits, tgt)
        assert abs(float(loss[0]) - rl) <= 1e-5 * abs(rl) and H.rel_err(O.cvt_bf16_f32(dl), rd) <= TOL16
        expired = br.exchange_fallbacks()[1]
        loss2, dl2 = run()
        assert loss.tobytes() == loss2.tobytes() and dl.tobytes() == dl2.tobytes()
        assert br.exchange_fallbacks()[1] == expired                     # every partial was handed over
        for spin, refuse in ((-1, 0), (0, 1)):
            br.tune("rms_cluster_spin", spin); br.tune("xch_take_nothing", refuse)
            loss3, dl3 = run()
            assert loss.tobytes() == loss3.tobytes() and dl.tobytes() == dl3.tobytes(), (spin, refuse)
        assert br.exchange_fallbacks()[1] > expired
        br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)
        br.tune("ce_resident", -1)                                       # the three-launch form
        loss4, dl4 = run()
        assert abs(float(loss4[0]) - float(loss[0])) <= 2e-6 * abs(float(loss[0]))
        assert H.rel_err(O.cvt_bf16_f32(dl4), O.cvt_bf16_f32(dl)) <= TOL16
    finally:
        br.tune("ce_resident", 0); br.tune("rms_cluster_spin", 0); br.tune("xch_take_nothing", 0)


def test_bf16_bad_arguments(br):
    a = br.DevArray(64, np.uint16); w = br.DevArray(8)
    assert br.lib.mi355_rmsnorm_fwd_bf16_dev(a.ptr, a.ptr, None, 8, 8, 1, 1e-5) == -1
    assert br.lib.mi355_rmsnorm_bwd_bf16_dev(a.ptr, w.ptr, a.ptr, a.ptr, w.ptr, 8, 8, 1, 1e-5, 2) == -1
    a2, a3 = br.DevArray(64, np.uint16), br.DevArray(64, np.uint16)
    assert br.lib.mi355_rmsnorm_bwd_bf16_dev(a.ptr, w.ptr, a2.ptr, a.ptr, w.ptr, 8, 8, 1, 1e-5, 0) == -1     # dx over x
    assert "alias" in br.last_error()
    assert br.lib.mi355_rmsnorm_bwd_bf16_dev(a2.ptr, w.ptr, a2.ptr, a3.ptr, w.ptr, 8, 8, 1, 1e-5, 0) == 0    # dx over dy
    assert br.lib.mi355_swiglu_fwd_bf16_dev(a.ptr, a.ptr, a.ptr, 0) == -1
    assert br.lib.mi355_axpby_bf16_dev(a.ptr, a.ptr, None, 1.0, 64, 0) == -1
    assert br.lib.mi355_cvt_f32_bf16_dev(a.ptr, 4, w.ptr, 8, 1, 8) == -1
    assert "bf16" in br.last_error()


@pytest.mark.parametrize("B,heads,kvh,hd,S", [(16, 16, 8, 128, 256), (2, 12, 12, 64, 256), (2, 3, 2, 16, 24), (1, 2, 1, 8, 10),
                                              (1, 2, 1, 512, 16), (2, 4, 2, 256, 32), (1, 1, 1, 1024, 8), (1, 4, 0, 32, 16)])
def test_rope_and_qknorm_rope_bf16(br, B, heads, kvh, hd, S):
    print("[case] bf16 qknorm_rope B=%d heads=%d/%d hd=%d S=%d" % (B, heads, kvh, hd, S), flush=True)
    theta = 1e6
    kv = max(kvh, 1)
    (qb, q), (kb, k) = bf(H.normal(230, (B, heads * hd, S))), bf(H.normal(231, (B, kv * hd, S)))
    (gqb, gq), (gkb, gk) = bf(H.normal(232, q.shape)), bf(H.normal(233, k.shape))
    wq = H.normal(234, hd, 1.0, 0.02); wk = H.normal(235, hd, 1.0, 0.02)
    dwq0 = H.normal(236, hd); dwk0 = H.normal(237, hd)
    cd, sd = br.rope_tables_dev(S, hd, theta)
    qd, kd, gqd, gkd, wqd, wkd = (dev(br, a) for a in (qb, kb, gqb, gkb, wq, wk))
    K = lambda a: a.ptr if kvh else None
    # stand-alone rotation, both directions
    for direction in (+1, -1):
        qo, ko = br.DevArray(q.shape, np.uint16), br.DevArray(k.shape, np.uint16)
        br.check(br.lib.mi355_rope_bf16_dev(qo.ptr, K(ko), qd.ptr, K(kd), heads, kvh, hd, S, B, cd, sd, direction))
        assert H.rel_err(back(qo), O.rope(q, hd, theta, direction)) <= TOL16
        if kvh:
            assert H.rel_err(back(ko), O.rope(k, hd, theta, direction)) <= TOL16
    small = hd / 2 > 64 and S % 8 != 0          # beyond the scalar-column register tile: refused
    qo, ko = br.DevArray(q.shape, np.uint16), br.DevArray(k.shape, np.uint16)
    rc = br.lib.mi355_qknorm_rope_fwd_bf16_dev(qo.ptr, K(ko), qd.ptr, K(kd), wqd.ptr, K(wkd), heads, kvh, hd, S, B, cd, sd, 1e-5)
    assert rc == (-1 if small else 0)
    if small:
        return
    assert H.rel_err(back(qo), O.qknorm_rope_fwd(q, wq, hd, theta)) <= TOL16
    if kvh:
        assert H.rel_err(back(ko), O.qknorm_rope_fwd(k, wk, hd, theta)) <= TOL16
    for variant in (0, 1):
        dq, dk = br.DevArray(q.shape, np.uint16), br.DevArray(k.shape, np.uint16)
        dwq, dwk = dev(br, dwq0), dev(br, dwk0)
        br.check(br.lib.mi355_qknorm_rope_bwd_bf16_dev(dq.ptr, K(dk), dwq.ptr, K(dwk), gqd.ptr, K(gkd), qd.ptr, K(kd), wqd.ptr,
                                                       K(wkd), heads, kvh, hd, S, B, cd, sd, 1e-5, variant))
        rdq, rdwq = O.qknorm_rope_bwd(gq, q, wq, hd, theta, variant=variant, dw=dwq0)
        tol = TOL16 if hd >= 16 else 2e-2
        assert H.rel_err(back(dq), rdq) <= tol and H.rel_err(dwq.numpy(), rdwq) <= 1e-5
        if kvh:
            rdk, rdwk = O.qknorm_rope_bwd(gk, k, wk, hd, theta, variant=variant, dw=dwk0)
            assert H.rel_err(back(dk), rdk) <= tol and H.rel_err(dwk.numpy(), rdwk) <= 1e-5


@pytest.mark.parametrize("V,S", [(32000, 256), (151936, 256), (37, 12), (1000, 5), (300, 1024)])
def test_softmax_ce_bf16(br, V, S):
    print("[case] bf16 softmax_ce V=%d S=%d" % (V, S), flush=True)
    lb, logits = bf(H.normal(240, (V, S), 0, 2.0))
    tgt = np.random.default_rng(241).integers(0, V, S).astype(np.int32)
    if S > 8:
        tgt[3] = V; tgt[5] = -1                                         # out-of-range targets are skipped
    ld, td = dev(br, lb), dev(br, tgt)
    for scale in (1.0, 256.0):
        dl, lossd = br.DevArray((V, S), np.uint16), br.DevArray(1)
        br.check(br.lib.mi355_softmax_ce_bf16_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, scale))
        rl, rd = O.cross_entropy(logits, tgt, grad_scale=scale)
        assert abs(float(lossd.numpy()[0]) - rl) <= 1e-5 * abs(rl)        # fp32 all the way
        assert H.rel_err(back(dl), rd) <= TOL16
    br.check(br.lib.mi355_softmax_ce_bf16_dev(ld.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))     # in place
    assert H.rel_err(back(ld), O.cross_entropy(logits, tgt)[1]) <= TOL16
