"""Seeded random shapes for the tile kernels: every branch of the tile pickers (register tiles of each width,
the two-sweep variant, scalar columns, odd sizes) has to agree with the oracle."""
import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-5


def dev(br, a):
    return br.DevArray.from_numpy(a)


def _rms_shapes():
    rng = np.random.default_rng(2024)
    out = []
    for _ in range(18):
        C = int(rng.choice([rng.integers(1, 64), rng.integers(64, 600), rng.integers(600, 2200), rng.integers(2200, 6000)]))
        S = int(rng.choice([rng.integers(1, 40), 4 * rng.integers(1, 80), 256]))
        B = int(rng.integers(1, 5))
        out.append((B, C, S))
    # the last three have enough columns for the 128-byte strips (fp32 and bf16 pickers switch on strips x batch)
    return out + [(1, 2048, 256), (3, 2049, 12), (2, 4096, 64), (7, 16, 1024), (32, 1024, 256), (40, 768, 256), (9, 600, 1024)]


@pytest.mark.parametrize("B,C,S", _rms_shapes())
def test_rmsnorm_random_shapes(br, B, C, S):
    print("[case] rmsnorm B=%d C=%d S=%d" % (B, C, S), flush=True)
    x = H.normal(1, (B, C, S)); w = H.normal(2, C, 1.0, 0.02); dy = H.normal(3, (B, C, S)); b2 = H.normal(4, (B, C, S))
    dw0 = H.normal(5, C)
    xd, wd, dyd, bd = (dev(br, a) for a in (x, w, dy, b2))
    yd, dxd, dwd = br.DevArray(x.shape), br.DevArray(x.shape), dev(br, dw0)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5))
    assert H.rel_err(yd.numpy(), O.rmsnorm(x, w)) <= TOL
    br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5, 0))
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, dw=dw0)
    assert H.rel_err(dxd.numpy(), rdx) <= TOL and H.rel_err(dwd.numpy(), rdw) <= TOL
    # residual + norm in one launch equals the two separate oracle steps
    y2, yn = br.DevArray(x.shape), br.DevArray(x.shape)
    al = np.float32(24 ** 0.25)
    br.check(br.lib.mi355_residual_rmsnorm_fwd_dev(y2.ptr, yn.ptr, xd.ptr, bd.ptr, al, wd.ptr, C, S, B, 1e-5))
    r2 = O.axpby(x, b2, al, 0)
    assert np.array_equal(y2.numpy(), r2) and H.rel_err(yn.numpy(), O.rmsnorm(r2, w)) <= TOL


def _qk_shapes():
    rng = np.random.default_rng(77)
    out = []
    for _ in range(10):
        hd = int(rng.choice([2, 8, 16, 32, 64, 96, 128, 256, 512]))
        kvh = int(rng.integers(1, 4)); heads = kvh * int(rng.integers(1, 4))
        S = int(rng.choice([4 * rng.integers(1, 70), rng.integers(1, 30)]))
        out.append((int(rng.integers(1, 4)), heads, kvh, hd, S))
    return out


@pytest.mark.parametrize("B,heads,kvh,hd,S", _qk_shapes())
def test_qknorm_rope_random_shapes(br, B, heads, kvh, hd, S):
    print("[case] qknorm_rope B=%d heads=%d/%d hd=%d S=%d" % (B, heads, kvh, hd, S), flush=True)
    theta = 1e6
    q = H.normal(10, (B, heads * hd, S)); k = H.normal(11, (B, kvh * hd, S))
    wq = H.normal(12, hd, 1.0, 0.02); wk = H.normal(13, hd, 1.0, 0.02)
    gq = H.normal(14, q.shape); gk = H.normal(15, k.shape)
    cd, sd = br.rope_tables_dev(S, hd, theta)
    qd, kd, wqd, wkd, gqd, gkd = (dev(br, a) for a in (q, k, wq, wk, gq, gk))
    qo, ko = br.DevArray(q.shape), br.DevArray(k.shape)
    br.check(br.lib.mi355_qknorm_rope_fwd_dev(qo.ptr, ko.ptr, qd.ptr, kd.ptr, wqd.ptr, wkd.ptr, heads, kvh, hd, S, B, cd, sd,
                                              1e-5))
    assert H.rel_err(qo.numpy(), O.qknorm_rope_fwd(q, wq, hd, theta)) <= TOL
    assert H.rel_err(ko.numpy(), O.qknorm_rope_fwd(k, wk, hd, theta)) <= TOL
    dq, dk, dwq, dwk = br.DevArray(q.shape), br.DevArray(k.shape), br.DevArray(hd), br.DevArray(hd)
    br.check(br.lib.mi355_qknorm_rope_bwd_dev(dq.ptr, dk.ptr, dwq.ptr, dwk.ptr, gqd.ptr, gkd.ptr, qd.ptr, kd.ptr, wqd.ptr,
                                              wkd.ptr, heads, kvh, hd, S, B, cd, sd, 1e-5, 0))
    rdq, rdwq = O.qknorm_rope_bwd(gq, q, wq, hd, theta)
    rdk, rdwk = O.qknorm_rope_bwd(gk, k, wk, hd, theta)
    # with two channels per head the backward cancels almost exactly and fp32 itself is off by more than 1e-5
    tol = TOL if hd >= 16 else 1e-3
    assert H.rel_err(dq.numpy(), rdq) <= tol and H.rel_err(dk.numpy(), rdk) <= tol
    assert H.rel_err(dwq.numpy(), rdwq) <= TOL and H.rel_err(dwk.numpy(), rdwk) <= TOL


def _ce_shapes():
    rng = np.random.default_rng(5)
    return [(int(rng.integers(2, 9000)), int(rng.choice([rng.integers(1, 70), 4 * rng.integers(1, 130)]))) for _ in range(8)]


@pytest.mark.parametrize("V,S", _ce_shapes())
def test_softmax_ce_random_shapes(br, V, S):
    print("[case] softmax_ce V=%d S=%d" % (V, S), flush=True)
    logits = H.normal(20, (V, S), 0, 2.0)
    tgt = np.random.default_rng(21).integers(-1, V + 1, S).astype(np.int32)      # a few out-of-range targets
    ld, td = dev(br, logits), dev(br, tgt)
    dl, lossd = br.DevArray(logits.shape), br.DevArray(1)
    br.check(br.lib.mi355_softmax_ce_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
    rl, rd = O.cross_entropy(logits, tgt)
    assert abs(float(lossd.numpy()[0]) - rl) <= TOL * max(abs(rl), 1e-3) and H.rel_err(dl.numpy(), rd) <= TOL
