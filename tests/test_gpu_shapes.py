"""Seeded random shapes for the tile kernels: every branch of the tile pickers (register tiles of each width,
the two-sweep variant, scalar columns, odd sizes) has to agree with the oracle.

MI355_RANDOM_CASES=k draws k times as many shapes of every family and MI355_RANDOM_SEED=s draws other ones (the default,
1 and 0, is what the suite runs; a longer campaign is `MI355_RANDOM_CASES=8 MI355_RANDOM_SEED=1 pytest tests/test_gpu_shapes.py`)."""
import os

import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-5
MORE = max(1, int(os.environ.get("MI355_RANDOM_CASES", "1")))
SEED = int(os.environ.get("MI355_RANDOM_SEED", "0"))


def dev(br, a):
    return br.DevArray.from_numpy(a)


def _rms_shapes():
    rng = np.random.default_rng(2024 + SEED)
    out = []
    for _ in range(18 * MORE):
        C = int(rng.choice([rng.integers(1, 64), rng.integers(64, 600), rng.integers(600, 2200), rng.integers(2200, 6000)]))
        S = int(rng.choice([rng.integers(1, 40), 4 * rng.integers(1, 80), 256]))
        B = int(rng.integers(1, 5))
        out.append((B, C, S))
    # the last three have enough columns for the 128-byte strips (fp32 and bf16 pickers switch on strips x batch)
    return out + [(1, 2048, 256), (3, 2049, 12), (2, 4096, 64), (7, 16, 1024), (32, 1024, 256), (40, 768, 256), (9, 600, 1024),
                  (128, 384, 256)]      # 32768 columns below 512 channels: 16-lane strips on 512 threads


@pytest.mark.parametrize("B,C,S", _rms_shapes())
def test_rmsnorm_random_shapes(br, B, C, S):
    print("[case] rmsnorm B=%d C=%d S=%d" % (B, C, S), flush=True)
    x = H.normal(1, (B, C, S)); w = H.normal(2, C, 1.0, 0.02); dy = H.normal(3, (B, C, S)); b2 = H.normal(4, (B, C, S))
    dw0 = H.normal(5, C)
    xd, wd, dyd, bd = (dev(br, a) for a in (x, w, dy, b2))
    yd, dxd, dwd = br.DevArray(x.shape), br.DevArray(x.shape), dev(br, dw0)
    br.check(br.lib.mi355_rmsnorm_fwd_dev(yd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5))
    assert H.err_elem(yd.numpy(), O.rmsnorm(x, w)) <= TOL
    br.check(br.lib.mi355_rmsnorm_bwd_dev(dxd.ptr, dwd.ptr, dyd.ptr, xd.ptr, wd.ptr, C, S, B, 1e-5, 0))
    rdx, rdw = O.rmsnorm_bwd(dy, x, w, dw=dw0)
    assert H.rel_err(dxd.numpy(), rdx) <= TOL and H.rel_err(dwd.numpy(), rdw) <= TOL
    # residual + norm in one launch equals the two separate oracle steps
    y2, yn = br.DevArray(x.shape), br.DevArray(x.shape)
    al = np.float32(24 ** 0.25)
    br.check(br.lib.mi355_residual_rmsnorm_fwd_dev(y2.ptr, yn.ptr, xd.ptr, bd.ptr, al, wd.ptr, C, S, B, 1e-5))
    r2 = O.axpby(x, b2, al, 0)
    assert np.array_equal(y2.numpy(), r2) and H.err_elem(yn.numpy(), O.rmsnorm(r2, w)) <= TOL
    # backward with the residual riding along (8-row tiles, or the two-sweep variant)
    dx3, dw3 = br.DevArray(x.shape), dev(br, dw0)
    br.check(br.lib.mi355_rmsnorm_bwd_residual_dev(dx3.ptr, None, dw3.ptr, dyd.ptr, xd.ptr, wd.ptr, bd.ptr, 1.0, C, S, B,
                                                   1e-5, 0))
    assert H.rel_err(dx3.numpy(), O.axpby(rdx, b2, 0.0, 2)) <= TOL and H.rel_err(dw3.numpy(), rdw) <= TOL


def _qk_shapes():
    rng = np.random.default_rng(77 + SEED)
    out = []
    for _ in range(10 * MORE):
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
    rng = np.random.default_rng(5 + SEED)
    return [(int(rng.integers(2, 9000)), int(rng.choice([rng.integers(1, 70), 4 * rng.integers(1, 130)]))) for _ in range(8 * MORE)]


@pytest.mark.parametrize("V,S", _ce_shapes())
def test_softmax_ce_random_shapes(br, V, S):
    print("[case] softmax_ce V=%d S=%d" % (V, S), flush=True)
    logits = H.normal(20, (V, S), 0, 2.0)
    tgt = np.random.default_rng(21).integers(-1, V + 1, S).astype(np.int32)      # a few out-of-range targets
    ld, td = dev(br, logits), dev(br, tgt)
    dl, lossd = br.DevArray(logits.shape), br.DevArray(1)
    br.check(br.lib.mi355_softmax_ce_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
    rl, rd = O.cross_entropy(logits, tgt)
    assert abs(float(lossd.numpy()[0]) - rl) <= TOL * max(abs(rl), 1e-3) and H.err_std(dl.numpy(), rd) <= TOL


def _ce_one_launch_shapes():
    rng = np.random.default_rng(6 + SEED)
    return [(int(rng.integers(1, 30000)), 64 * int(rng.integers(1, 17))) for _ in range(10 * MORE)] + [(3, 64), (130, 256), (65, 1024)]


@pytest.mark.parametrize("V,S", _ce_one_launch_shapes())
def test_softmax_ce_one_launch_random_shapes(br, V, S):
    """The one-launch form on every shape it accepts (any V, S = 64 .. 1024): members with ragged, single and no
    rows, 1 to 16 strips; against the oracle and, to the bit, against itself with every partner's value refused."""
    print("[case] softmax_ce one launch V=%d S=%d" % (V, S), flush=True)
    logits = H.normal(22, (V, S), 0, 2.0)
    tgt = np.random.default_rng(23).integers(-1, V + 1, S).astype(np.int32)
    ld, td = dev(br, logits), dev(br, tgt)
    rl, rd = O.cross_entropy(logits, tgt)
    try:
        br.tune("ce_resident", 1)
        out = []
        for refuse in (0, 1):
            br.tune("xch_take_nothing", refuse)
            expired = br.exchange_fallbacks()[1]
            dl, lossd = br.DevArray(logits.shape), br.DevArray(1)
            br.check(br.lib.mi355_softmax_ce_dev(dl.ptr, lossd.ptr, ld.ptr, td.ptr, V, S, 1.0))
            out.append((lossd.numpy().tobytes(), dl.numpy().tobytes()))
            assert abs(float(lossd.numpy()[0]) - rl) <= TOL * max(abs(rl), 1e-3) and H.err_std(dl.numpy(), rd) <= TOL
            assert (br.exchange_fallbacks()[1] > expired) == bool(refuse)
        assert out[0] == out[1]
    finally:
        br.tune("ce_resident", 0); br.tune("xch_take_nothing", 0)


def _embed_cases():
    """Seeded random shapes and id distributions for the gather and the ordered scatter-add: uniform ids, Zipf ids,
    two or three hot tokens, ids of which a third are out of range, one token only; sequence lengths that are not
    multiples of 4 or 64, row widths on both sides of the 128-bit and 256-float paths, vocabularies around the
    planner's 2^18 limit, and every fifth case beyond its 16384 positions (library sort)."""
    rng = np.random.default_rng(12345 + SEED)
    out = []
    for case in range(36 * MORE):
        kind = int(rng.integers(0, 5))
        S = int(rng.choice([1, 3, 4, 8, 16, 37, 64, 100, 256, 257, 512]))
        B = int(rng.integers(1, max(2, min(300, 17000 // S))))
        if case % 5 == 4:
            B = max(1, 20000 // S)
        D = int(rng.choice([1, 3, 4, 8, 20, 32, 33, 64, 96, 128, 256, 260, 768, 1024]))
        if B * S * D > 12_000_000:
            D = max(1, 12_000_000 // (B * S))
        V = int(rng.choice([1, 2, 5, 37, 256, 1000, 32000, 151936, 262143, 262144, 400000]))
        if V * D > 40_000_000:
            V = max(1, 40_000_000 // D)
        out.append((case, kind, V, D, B, S, int(rng.integers(1 << 30))))
    return out


@pytest.mark.parametrize("case,kind,V,D,B,S,seed", _embed_cases())
def test_embed_gather_scatter_random_shapes(br, case, kind, V, D, B, S, seed):
    print("[case] embed %d kind=%d V=%d D=%d B=%d S=%d" % (case, kind, V, D, B, S), flush=True)
    rng = np.random.default_rng(seed)
    N = B * S
    if kind == 0: ids = rng.integers(0, V, N)
    elif kind == 1: ids = H.zipf_ids(seed, N, V)
    elif kind == 2: ids = rng.integers(0, max(1, min(V, 3)), N)
    elif kind == 3: ids = np.where(rng.random(N) < 0.3, rng.integers(-5, V + 5, N), rng.integers(0, V, N))
    else: ids = np.full(N, rng.integers(0, V))
    ids = ids.astype(np.int32).reshape(B, S)
    E = (rng.standard_normal((V, D)) * 0.02).astype(np.float32)
    # gather: a copy, bit for bit; columns of skipped ids keep what the output held
    x0 = np.full((B, D, S), 7.0, np.float32)
    Ed, idd, xd = dev(br, E), dev(br, ids), dev(br, x0)
    br.check(br.lib.mi355_embed_gather_dev(xd.ptr, Ed.ptr, idd.ptr, V, D, S, B))
    want, _ = O.embed_lookup(E, ids, out=x0.copy())
    assert xd.numpy().tobytes() == want.tobytes()
    # scatter-add: the reference loop's order, bit for bit, by default; the opt-in tree order within each row's scale
    dx = (rng.standard_normal((B, D, S)) * 3).astype(np.float32)
    dE0 = rng.standard_normal((V, D)).astype(np.float32)
    dxd, dEd = dev(br, dx), dev(br, dE0)
    tree = case % 7 == 6
    br.tune("scatter_tree", int(tree))
    br.tune("scatter_cols", (0, -1, 1)[case % 3])       # the form chosen for the shape / token-major rows / columns of dE
    try:
        br.check(br.lib.mi355_embed_scatter_add_dev(dEd.ptr, dxd.ptr, idd.ptr, V, D, S, B))
    finally:
        br.tune("scatter_tree", 0)
        br.tune("scatter_cols", 0)
    got, ref = dEd.numpy(), O.embed_backward(dE0, dx, ids)
    if not tree:
        assert got.tobytes() == ref.tobytes()
    else:
        # a reordered fp32 sum of n terms of scale 3: each row is judged against the size of its own partial sums, and
        # against the exact (float64) sum: the reference's chain of n fp32 additions is itself ~sqrt(n)/2 ulps of that
        # size away from it (1.2e-5 of the scale at 20000 positions on one token), the tree ~log2(n) ulps
        cnt = np.bincount(ids[(ids >= 0) & (ids < V)].ravel(), minlength=V).astype(np.float64)
        scale = np.maximum(np.sqrt(np.mean(ref.astype(np.float64) ** 2, axis=1)), 3.0 * np.sqrt(np.maximum(cnt, 1.0)))
        exact = H.np_embed_backward(dE0, dx, ids)
        assert np.max(np.max(np.abs(got - exact), axis=1) / scale) <= TOL
        chain = np.max(np.abs(ref - exact), axis=1)
        assert np.max((np.max(np.abs(got.astype(np.float64) - ref), axis=1) - chain) / scale) <= TOL
        assert np.array_equal(got[cnt <= 96], ref[cnt <= 96])          # short segments keep the reference order


def _stream_cases():
    """Lengths on both sides of the 128-bit path's tail and of one workgroup's share, with pointers 0-3 elements off a
    16-byte boundary (the inputs and the outputs separately), for the element-wise and reduction kernels."""
    rng = np.random.default_rng(901 + SEED)
    out = []
    for _ in range(12 * MORE):
        n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 70000), rng.integers(70000, 3_000_000)]))
        out.append((n, int(rng.integers(0, 4)), int(rng.integers(0, 4)), int(rng.integers(1 << 30))))
    return out


class _Off:
    """A device array of n elements that starts `off` elements into its allocation."""

    def __init__(self, br, n, off, dtype=np.float32, data=None):
        self.n, self.off, self.dtype = n, off, np.dtype(dtype)
        host = np.zeros(n + off, dtype)
        if data is not None:
            host[off:] = data
        self.d = br.DevArray.from_numpy(host)
        self.ptr = self.d.ptr + off * self.dtype.itemsize

    def numpy(self):
        return self.d.numpy()[self.off:]


@pytest.mark.parametrize("n,oi,oo,seed", _stream_cases())
def test_streaming_ops_random_lengths_and_offsets(br, n, oi, oo, seed):
    print("[case] streaming n=%d offsets in=%d out=%d seed=%d" % (n, oi, oo, seed), flush=True)
    a = H.normal(seed, n); b = H.normal(seed + 1, n); d = H.normal(seed + 2, n)
    ad, bd, dd = (_Off(br, n, oi, data=v) for v in (a, b, d))
    o1, o2 = _Off(br, n, oo), _Off(br, n, oo)
    # SwiGLU (within 1e-5 of the oracle; the gate's gradient against the tensor's scale, where its factor cancels)
    br.check(br.lib.mi355_swiglu_fwd_dev(o1.ptr, ad.ptr, bd.ptr, n))
    assert H.err_elem(o1.numpy(), O.swiglu_fwd(a, b)) <= TOL
    br.check(br.lib.mi355_swiglu_bwd_dev(o1.ptr, o2.ptr, dd.ptr, ad.ptr, bd.ptr, n))
    r1, r3 = O.swiglu_bwd(d, a, b)
    assert H.rel_err(o1.numpy(), r1) <= TOL and H.err_elem(o2.numpy(), r3) <= TOL
    # the residual family: bit for bit
    al = np.float32(1 / np.sqrt(2 * 28))
    for mode, second in ((0, bd), (1, None), (2, bd)):
        br.check(br.lib.mi355_axpby_dev(o1.ptr, ad.ptr, second.ptr if second else None, al, n, mode))
        assert np.array_equal(o1.numpy(), O.axpby(a, b if second else None, al, mode))
    # INT8: scale, both roundings, dequantize, and the fused scale+quantize — bit for bit
    x3 = a * np.float32(3.0)
    xd = _Off(br, n, oi, data=x3)
    sd, s2 = br.DevArray(1), br.DevArray(1)
    br.check(br.lib.mi355_int8_scale_dev(sd.ptr, xd.ptr, n))
    scale = sd.numpy()[0]
    assert scale == np.float32(O.int8_scale(x3))
    for rounding in (0, 1):
        q, q2 = _Off(br, n, oo, np.int8), _Off(br, n, oo, np.int8)
        br.check(br.lib.mi355_int8_quant_dev(q.ptr, xd.ptr, sd.ptr, n, rounding))
        want = O.int8_quant(x3, scale, rounding)
        assert np.array_equal(q.numpy(), want)
        br.check(br.lib.mi355_int8_quantize_dynamic_dev(q2.ptr, s2.ptr, xd.ptr, n, rounding))
        assert s2.numpy()[0] == scale and np.array_equal(q2.numpy(), want)
        br.check(br.lib.mi355_int8_dequant_dev(o1.ptr, q.ptr, sd.ptr, n))
        assert np.array_equal(o1.numpy(), O.int8_dequant(want, scale))
    # range diagnostics: exact
    mm = br.DevArray(3)
    br.check(br.lib.mi355_minmax_dev(mm.ptr, xd.ptr, n))
    assert mm.numpy().tobytes() == O.minmax(x3).tobytes()
    # optimizer tail: sum of squares, then AdamW with the clip scale read on the device
    w = H.normal(seed + 3, n, 0, 0.05); m = H.normal(seed + 4, n, 0, 0.01); v = np.abs(H.normal(seed + 5, n, 0, 0.01))
    g = a * np.float32(40.0)
    wd_, gd, md, vd = (_Off(br, n, o, data=t) for o, t in ((oo, w), (oi, g), (oo, m), (oi, v)))
    ss = dev(br, np.zeros(1, np.float32)); cs = br.DevArray(1)
    gsc = np.float32(1.0 / 256.0)
    br.check(br.lib.mi355_sumsq_accum_dev(ss.ptr, gd.ptr, n, gsc))
    t64 = float(np.sum((g * gsc).astype(np.float64) ** 2))
    assert abs(ss.numpy()[0] - t64) <= TOL * t64
    br.check(br.lib.mi355_clip_scale_dev(cs.ptr, ss.ptr, np.float32(1e-3)))
    r_cs = O.clip_scale(float(ss.numpy()[0]), np.float32(1e-3))
    assert cs.numpy()[0] == np.float32(r_cs)
    br.check(br.lib.mi355_adam_update_dev(wd_.ptr, gd.ptr, md.ptr, vd.ptr, n, 3, 3e-4, 0.9, 0.95, 1e-8, 0.1, gsc, cs.ptr, 1))
    rw, rm, rv = O.adam_update(w, (g * gsc) * np.float32(r_cs), m, v, 3, 3e-4, 0.9, 0.95, 1e-8, 0.1)
    assert H.rel_err(md.numpy(), rm) <= TOL and H.rel_err(vd.numpy(), rv) <= TOL and H.rel_err(wd_.numpy(), rw) <= TOL
    assert not gd.numpy().any()


def _bf16_shapes():
    rng = np.random.default_rng(333 + SEED)
    out = []
    for _ in range(6 * MORE):
        C = int(rng.choice([rng.integers(1, 64), rng.integers(64, 600), rng.integers(600, 2200), rng.integers(2200, 5200)]))
        S = int(rng.choice([rng.integers(1, 40), 8 * rng.integers(1, 40), 256]))
        out.append((int(rng.integers(1, 5)), C, S))
    return out


@pytest.mark.parametrize("B,C,S", _bf16_shapes())
def test_bf16_norms_random_shapes(br, B, C, S):
    """The bfloat16-storage RMSNorm kernels and their residual fusions on random shapes: the checks of the named shapes
    (within 5e-3 of the fp32 oracle on the same bf16-representable inputs, y and the exchange-free rerun to the bit)."""
    import test_gpu_bf16 as BF
    BF.test_rmsnorm_bf16(br, B, C, S)
    BF.test_rmsnorm_residual_fusions_bf16(br, B, C, S)


def _bf16_qk_shapes():
    rng = np.random.default_rng(444 + SEED)
    out = []
    for _ in range(4 * MORE):
        hd = int(rng.choice([16, 32, 64, 96, 128, 256]))
        kvh = int(rng.integers(1, 4)); heads = kvh * int(rng.integers(1, 4))
        S = int(rng.choice([8 * rng.integers(1, 40), rng.integers(1, 30)]))
        out.append((int(rng.integers(1, 4)), heads, kvh, hd, S))
    return out


@pytest.mark.parametrize("B,heads,kvh,hd,S", _bf16_qk_shapes())
def test_bf16_rope_random_shapes(br, B, heads, kvh, hd, S):
    import test_gpu_bf16 as BF
    BF.test_rope_and_qknorm_rope_bf16(br, B, heads, kvh, hd, S)


@pytest.mark.parametrize("V,S", [(v, s) for v, s in _ce_shapes()[:4 * MORE]])
def test_bf16_softmax_ce_random_shapes(br, V, S):
    import test_gpu_bf16 as BF
    BF.test_softmax_ce_bf16(br, V, S)


def _helper_cases():
    """Random shapes for the helpers either side of the path (bit-exact ops): GQA tile / reduce, fp16 rectangle converts
    with pitches, vocabulary compaction rows, the map build and the one-pass attention-gradient finish."""
    rng = np.random.default_rng(555 + SEED)
    out = []
    for _ in range(5 * MORE):
        kvh = int(rng.integers(1, 5)); ratio = int(rng.integers(1, 5))
        hd = int(rng.choice([2, 4, 6, 8, 16, 64, 128])); S = int(rng.choice([rng.integers(1, 40), 4 * rng.integers(1, 70)]))
        rows = int(rng.integers(1, 300)); cols = int(rng.integers(1, 600))
        out.append((int(rng.integers(1, 4)), kvh, ratio, hd, S, rows, cols, cols + int(rng.integers(0, 40)),
                    cols + int(rng.integers(0, 40)), int(rng.choice([5, 300, 1031, 32000])),
                    int(rng.choice([1, 6, 64, 250, 1024])), int(rng.integers(1, 5000)), int(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("B,kvh,ratio,hd,S,rows,cols,dst_ld,src_ld,V,D,ntok,in_f16", _helper_cases())
def test_helper_ops_random_shapes(br, B, kvh, ratio, hd, S, rows, cols, dst_ld, src_ld, V, D, ntok, in_f16):
    print("[case] helpers B=%d kvh=%d ratio=%d hd=%d S=%d | cvt %dx%d ld %d/%d | vocab V=%d D=%d ntok=%d | f16 in %d"
          % (B, kvh, ratio, hd, S, rows, cols, dst_ld, src_ld, V, D, ntok, in_f16), flush=True)
    import test_gpu_parity as P
    P.test_gqa_tile_reduce(br, B, kvh, ratio, hd, S)
    P.test_cvt_rectangles(br, rows, cols, dst_ld, src_ld)
    P.test_vocab_compaction_bit_exact(br, V, D, ntok)
    P.test_vocab_map_build_and_remap_exact(br, V, ntok)
    P.test_attn_grads_finish_equals_separate_steps(br, B, kvh * ratio, kvh, hd, S, in_f16)
