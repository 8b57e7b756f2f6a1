"""Pins the C oracle (oracle/oracle.c) without running the reference: against the committed golden
vectors (inputs from the reference's own test recipes), float64 closed forms written independently
in helpers.py, finite differences, invariants and hand-computable special cases.  CPU only."""
import os

import numpy as np
import pytest

import helpers as H
import oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "kat_small.npz"))
F32_FAITHFUL = 3e-6     # sequential float32 evaluation vs the float64 closed form


# ---------------------------------------------------------------------------------------------
# input recipes
# ---------------------------------------------------------------------------------------------
def test_drand48_recipes_match_the_posix_lcg():
    # training/test_rmsnorm_bwd.m:26-33 — x and dy drawn interleaved, then w
    n, d = 64, 5
    x, dy, w = O.recipe_drand48(0, 42, n, d)
    g = H.Drand48(42)
    for i in range(n):
        assert x[i] == np.float32(g.next() * 2 - 1) * np.float32(0.5)
        assert dy[i] == np.float32(g.next() * 2 - 1) * np.float32(0.1)
    for i in range(d):
        assert w[i] == np.float32(g.next() * 0.5 + 0.75)
    # first drand48() after srand48(0) is a published constant of the LCG
    assert abs(H.Drand48(0).next() - 0.17082803610628972) < 1e-15
    # training/test_classifier.m:132-134
    x2, _, _ = O.recipe_drand48(2, 999, 16, 0)
    g = H.Drand48(999)
    assert np.array_equal(x2, np.array([np.float32(g.next() * 10 - 5) for _ in range(16)], np.float32))
    # training/test_classifier.m:60-62 and :205-207 — one array, then the next, from the same stream
    for recipe, seed, sx in ((3, 123, 0.1), (4, 456, 0.01)):
        x3, _, w3 = O.recipe_drand48(recipe, seed, 10, 7)
        g = H.Drand48(seed)
        assert np.array_equal(x3, np.array([np.float32(g.next() * 2 - 1) * np.float32(sx) for _ in range(10)], np.float32))
        assert np.array_equal(w3, np.array([np.float32(g.next() * 2 - 1) * np.float32(0.02) for _ in range(7)], np.float32))


# ---------------------------------------------------------------------------------------------
# RMSNorm
# ---------------------------------------------------------------------------------------------
def test_rmsnorm_golden_and_closed_form():
    y = O.rmsnorm(GOLD["rms_x"], GOLD["rms_w"])
    assert H.rel_err(y, GOLD["rms_y"]) < F32_FAITHFUL
    x = H.normal(0, (3, 768, 32)); w = H.normal(1, 768, 1.0, 0.02)
    assert H.rel_err(O.rmsnorm(x, w), H.np_rmsnorm(x, w)) < F32_FAITHFUL


def test_rmsnorm_known_answers():
    C, S = 40, 7
    w = H.normal(3, C, 1.0, 0.3)
    y = O.rmsnorm(np.ones((C, S), np.float32), w)                  # x == 1 -> y = w / sqrt(1+eps)
    assert np.allclose(y, (w / np.sqrt(1 + 1e-5))[:, None], rtol=3e-7)
    x = H.normal(4, (C, S))
    y = O.rmsnorm(x, np.ones(C, np.float32)).astype(np.float64)    # w == 1 -> mean y^2 = ms/(ms+eps)
    ms = np.mean(x.astype(np.float64) ** 2, axis=0)
    assert np.allclose(np.mean(y * y, axis=0), ms / (ms + 1e-5), rtol=2e-6)
    # a transposed operand or a reduction over the wrong axis fails here: scale one column only
    x2 = x.copy(); x2[:, 3] *= 10
    y2 = O.rmsnorm(x2, np.ones(C, np.float32))
    assert np.allclose(np.delete(y2, 3, 1), np.delete(y.astype(np.float32), 3, 1), rtol=1e-6)
    assert np.allclose(y2[:, 3], y[:, 3], rtol=1e-4)               # scale invariance of that column


def _loss64(x, w, dy, eps=1e-5):
    return float(np.sum(np.asarray(dy, np.float64) * H.np_rmsnorm(x, w, eps)))


def test_closed_form_gradient_is_the_derivative():
    """Pins helpers.np_rmsnorm_bwd (variant 1) and dw by central differences in float64."""
    rng = np.random.default_rng(5)
    C, S = 6, 3
    x = rng.standard_normal((C, S)); dy = rng.standard_normal((C, S)); w = 1 + 0.3 * rng.standard_normal(C)
    dx1, dw = H.np_rmsnorm_bwd(dy, x, w, variant=1)
    h = 1e-6
    for (c, s) in [(0, 0), (2, 1), (5, 2)]:
        xp = x.copy(); xm = x.copy(); xp[c, s] += h; xm[c, s] -= h
        fd = (_loss64(xp, w, dy) - _loss64(xm, w, dy)) / (2 * h)
        assert abs(fd - dx1[c, s]) < 1e-7 * max(1, abs(fd))
    for c in range(C):
        wp = w.copy(); wm = w.copy(); wp[c] += h; wm[c] -= h
        fd = (_loss64(x, wp, dy) - _loss64(x, wm, dy)) / (2 * h)
        assert abs(fd - dw[c]) < 1e-7 * max(1, abs(fd))


def test_rmsnorm_bwd_golden_and_variants():
    x, dy, w = GOLD["rms_x"], GOLD["rms_dy"], GOLD["rms_w"]
    dx0, dw0 = O.rmsnorm_bwd(dy, x, w, variant=0)
    dx1, dw1 = O.rmsnorm_bwd(dy, x, w, variant=1)
    assert H.rel_err(dx0, GOLD["rms_dx_v0"]) < F32_FAITHFUL
    assert H.rel_err(dx1, GOLD["rms_dx_v1"]) < F32_FAITHFUL
    assert H.rel_err(dw0, GOLD["rms_dw"]) < F32_FAITHFUL and np.array_equal(dw0, dw1)
    # the reference op (variant 0) is NOT the exact gradient once w != 1 ...
    assert H.rel_err(dx0, GOLD["rms_dx_v1"]) > 1e-3
    # ... and is exactly it when w == 1
    one = np.ones_like(w)
    a, _ = O.rmsnorm_bwd(dy, x, one, variant=0)
    b, _ = O.rmsnorm_bwd(dy, x, one, variant=1)
    assert H.rel_err(a, b) < 1e-6
    # What the reference's operand order does to the exact gradient, derived from training/stories_cpu_ops.h:35-46
    # without retyping its formula: it multiplies the whole bracket by w instead of dy alone, so
    #   variant0 = variant1 + x * (1 - w) * (rr^2 / C) * sum_c dy*y,   y = the forward output, rr^2 = 1/(mean x^2 + eps).
    # Variant 1 is pinned by finite differences below and y by the forward tests, so a dropped term, a wrong sign or
    # a misplaced w in the oracle's variant 0 fails here.
    x64, dy64, w64 = x.astype(np.float64), dy.astype(np.float64), w.astype(np.float64)
    y64 = O.rmsnorm(x, w).astype(np.float64)
    rr2 = 1.0 / (np.mean(x64 * x64, axis=0, keepdims=True) + 1e-5)
    corr = x64 * (1.0 - w64)[:, None] * (rr2 / x.shape[0]) * np.sum(dy64 * y64, axis=0, keepdims=True)
    assert H.rel_err(dx0, dx1.astype(np.float64) + corr) < 1e-5
    assert np.max(np.abs(corr)) > 1e-3 * np.max(np.abs(dx1))            # the correction is not a rounding artefact
    # and variant 1 with dw against central differences of L = sum dy * rmsnorm(x, w), at a few entries
    def loss(xx, ww):
        return float(np.sum(dy64 * H.np_rmsnorm(xx, ww)))
    h = 1e-5
    rng = np.random.default_rng(5)
    for _ in range(6):
        c, t = int(rng.integers(x.shape[0])), int(rng.integers(x.shape[1]))
        xp, xm = x64.copy(), x64.copy(); xp[c, t] += h; xm[c, t] -= h
        assert abs((loss(xp, w64) - loss(xm, w64)) / (2 * h) - dx1[c, t]) < 2e-4 * max(1.0, abs(dx1[c, t]))
        wp, wm = w64.copy(), w64.copy(); wp[c] += h; wm[c] -= h
        assert abs((loss(x64, wp) - loss(x64, wm)) / (2 * h) - dw0[c]) < 2e-4 * max(1.0, abs(dw0[c]))


def test_rmsnorm_bwd_assigns_dx_accumulates_dw_over_batch():
    B, C, S = 3, 32, 8
    x = H.normal(7, (B, C, S)); dy = H.normal(8, (B, C, S)); w = H.normal(9, C, 1.0, 0.02)
    dw_in = H.normal(10, C)
    dx, dw = O.rmsnorm_bwd(dy, x, w, dw=dw_in)
    rdx, rdw = H.np_rmsnorm_bwd(dy, x, w, variant=0)
    assert H.rel_err(dx, rdx) < F32_FAITHFUL
    assert H.rel_err(dw, dw_in.astype(np.float64) + rdw) < F32_FAITHFUL
    # threads > 1 (the multi-core baseline path) gives the same answer
    dx_t, dw_t = O.rmsnorm_bwd(dy, x, w, dw=dw_in, threads=3)
    assert np.array_equal(dx, dx_t) and H.rel_err(dw_t, dw) < 1e-6


# ---------------------------------------------------------------------------------------------
# SwiGLU
# ---------------------------------------------------------------------------------------------
def test_swiglu_golden_closed_form_and_finite_differences():
    h1, h3, d = GOLD["sw_h1"], GOLD["sw_h3"], GOLD["sw_d"]
    assert H.rel_err(O.swiglu_fwd(h1, h3), GOLD["sw_out"]) < F32_FAITHFUL
    dh1, dh3 = O.swiglu_bwd(d, h1, h3)
    assert H.rel_err(dh1, GOLD["sw_dh1"]) < F32_FAITHFUL
    assert H.rel_err(dh3, GOLD["sw_dh3"]) < F32_FAITHFUL
    # the closed form itself is the derivative of the forward (float64 central differences)
    a = h1[:16].astype(np.float64); b = h3[:16].astype(np.float64); g = d[:16].astype(np.float64)
    h = 1e-6
    fd1 = g * (H.np_swiglu_fwd(a + h, b) - H.np_swiglu_fwd(a - h, b)) / (2 * h)
    fd3 = g * (H.np_swiglu_fwd(a, b + h) - H.np_swiglu_fwd(a, b - h)) / (2 * h)
    r1, r3 = H.np_swiglu_bwd(g, a, b)
    assert np.allclose(fd1, r1, rtol=1e-7, atol=1e-9) and np.allclose(fd3, r3, rtol=1e-7, atol=1e-9)
    # scalar formulation of training/forward.h:101 (x/(1+exp(-x))) agrees with the sigmoid-mul form
    alt = (h1.astype(np.float64) / (1 + np.exp(-h1.astype(np.float64)))) * h3
    assert H.rel_err(O.swiglu_fwd(h1, h3), alt) < F32_FAITHFUL
    # known values: silu(0) = 0, d silu(0) = 1/2
    z = np.zeros(4, np.float32); o = np.ones(4, np.float32)
    assert np.array_equal(O.swiglu_fwd(z, o), z)
    assert np.allclose(O.swiglu_bwd(o, z, o)[0], 0.5)


# ---------------------------------------------------------------------------------------------
# RoPE and QK-norm
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("theta,tag", [(10000.0, "1e4"), (1e6, "1e6")])
def test_rope_golden_and_invariants(theta, tag):
    x = GOLD["rope_x"]; hd = 16
    f = O.rope(x, hd, theta, +1); b = O.rope(x, hd, theta, -1)
    assert H.rel_err(f, GOLD["rope_fwd_" + tag]) < 1e-5      # float32 angles vs float64 angles
    assert H.rel_err(b, GOLD["rope_bwd_" + tag]) < 1e-5
    assert np.array_equal(f[:, 0], x[:, 0]) and np.array_equal(b[:, 0], x[:, 0])     # position 0: identity
    assert H.rel_err(O.rope(f, hd, theta, -1), x) < 1e-6                             # bwd o fwd = identity
    pairs = lambda a: (a.reshape(-1, 2, a.shape[-1]).astype(np.float64) ** 2).sum(axis=1)
    assert np.allclose(pairs(f), pairs(x), rtol=1e-6)                                # rotations keep pair norms
    # a wrong sign shows up here: forward then forward is a rotation by twice the angle, not identity
    assert H.rel_err(O.rope(f, hd, theta, +1), x) > 1e-2


def test_rope_tables_and_rotation_with_exact_table_angles():
    S, hd, theta = 64, 32, 1e6
    c, s = O.rope_tables(S, hd, theta)
    ang = H.np_rope_angles(S, hd, theta)
    # the float32 angle p*(1/powf(theta,2i/hd)) carries up to ~|angle|*2^-23 of error
    assert np.max(np.abs(c - np.cos(ang))) < 63 * 3e-7 and np.max(np.abs(s - np.sin(ang))) < 63 * 3e-7
    assert np.allclose(c.astype(np.float64) ** 2 + s.astype(np.float64) ** 2, 1.0, atol=3e-7)
    # layout: [pair][position]; pair 0 has frequency 1 -> angle = position
    assert np.allclose(c[0], np.cos(np.arange(S)), atol=1e-6)
    # rotating with exactly the tabulated float32 angles is float32-faithful
    x = H.normal(11, (2, 3 * hd, S))
    ang32 = np.arctan2(s.astype(np.float64), c.astype(np.float64))
    ref = H.np_rope(x, hd, theta, +1, angles=ang32)
    assert H.rel_err(O.rope(x, hd, theta, +1), ref) < F32_FAITHFUL


def test_rope_matches_row_major_formula():
    """training/forward.h:55-70 written for [S, nheads*hd]: out[t,h,i]=x0*cos - x1*sin with
    freq = 1/10000^(i/hd) for even i."""
    S, nh, hd = 9, 2, 8
    x = H.normal(12, (nh * hd, S))
    rm = x.T.astype(np.float64).copy()          # [S, nh*hd]
    for t in range(S):
        for h in range(nh):
            for i in range(0, hd, 2):
                val = t / 10000.0 ** (i / hd)
                o = h * hd + i
                a, b = rm[t, o], rm[t, o + 1]
                rm[t, o] = a * np.cos(val) - b * np.sin(val)
                rm[t, o + 1] = a * np.sin(val) + b * np.cos(val)
    assert H.rel_err(O.rope(x, hd, 10000.0, +1), rm.T) < 3e-6


def test_qknorm_rope_golden_and_composition():
    x, w, dy = GOLD["rope_x"], GOLD["qk_w"], GOLD["qk_dy"]
    assert H.rel_err(O.qknorm_rope_fwd(x, w, 16, 1e6), GOLD["qk_fwd"]) < 1e-5
    dx, dw = O.qknorm_rope_bwd(dy, x, w, 16, 1e6)
    assert H.rel_err(dx, GOLD["qk_dx_v0"]) < 1e-5 and H.rel_err(dw, GOLD["qk_dw"]) < 1e-5
    # equals "rmsnorm per head slab, then rope"
    y = np.concatenate([O.rmsnorm(x[h * 16:(h + 1) * 16], w) for h in range(4)])
    assert np.array_equal(O.qknorm_rope_fwd(x, w, 16, 1e6), O.rope(y, 16, 1e6, +1))


# ---------------------------------------------------------------------------------------------
# residual, GQA, Adam
# ---------------------------------------------------------------------------------------------
def test_axpby_is_exact_float32_arithmetic():
    a = H.normal(13, 1001); b = H.normal(14, 1001); al = np.float32(24 ** 0.25)
    assert np.array_equal(O.axpby(a, b, al, 0), (b * al) + a)      # two roundings, vDSP_vsma restated
    assert np.array_equal(O.axpby(a, None, al, 1), a * al)
    assert np.array_equal(O.axpby(a, b, 0.0, 2), a + b)


def test_gqa_tile_reduce():
    kvh, ratio, hd, S = 2, 3, 4, 5
    k = H.normal(15, (kvh * hd, S))
    t = O.gqa_tile(k, kvh, ratio, hd)
    for q in range(kvh * ratio):
        assert np.array_equal(t[q * hd:(q + 1) * hd], k[(q // ratio) * hd:(q // ratio + 1) * hd])
    g = H.normal(16, (kvh * ratio * hd, S))
    r = O.gqa_reduce(g, kvh, ratio, hd)
    ref = g.reshape(kvh, ratio, hd, S).astype(np.float64).sum(axis=1).reshape(kvh * hd, S)
    assert H.rel_err(r, ref) < 1e-6
    # reduce is the adjoint of tile: <tile(k), g> = <k, reduce(g)>
    assert abs(np.vdot(t.astype(np.float64), g) - np.vdot(k.astype(np.float64), r)) < 1e-4


def test_fp16_converts_match_ieee_binary16():
    """cvt_f32_f16 / cvt_f16_f32 (training/training_dynamic/io.h:33-50) are the IEEE conversions; numpy's float16
    is an independent implementation of the same standard."""
    allh = np.arange(65536, dtype=np.uint16)
    f = O.cvt_f16_f32(allh)
    ref = allh.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(f), nan)
    assert np.array_equal(f[~nan].view(np.uint32), ref[~nan].view(np.uint32))              # exact, signed zeros included
    # every half survives the round trip
    assert np.array_equal(O.cvt_f32_f16(f[~nan]), allh[~nan])

    v = H.f16_boundary_values()
    with np.errstate(over="ignore"):
        assert np.array_equal(O.cvt_f32_f16(v), v.astype(np.float16).view(np.uint16))      # ties, subnormals, overflow
        rnd = np.random.default_rng(5).integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
        rnd = rnd[~np.isnan(rnd)]
        assert np.array_equal(O.cvt_f32_f16(rnd), rnd.astype(np.float16).view(np.uint16))
    got = O.cvt_f32_f16(np.array([np.nan, -np.nan], np.float32)).view(np.float16)
    assert np.isnan(got).all()


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_sgemm_is_the_row_major_product(ta, tb):
    M, N, K = 37, 29, 53
    A = H.normal(150, (K, M) if ta else (M, K)); B = H.normal(151, (N, K) if tb else (K, N)); C0 = H.normal(152, (M, N))
    ref = 0.75 * ((A.T if ta else A).astype(np.float64) @ (B.T if tb else B).astype(np.float64)) - 0.5 * C0
    got = O.sgemm(ta, tb, 0.75, A, B, -0.5, C0)
    assert H.rel_err(got, ref) < 2e-7                                   # one rounding of the exact value
    # beta = 0 must not read C (cblas semantics): NaNs in C are overwritten
    assert np.isfinite(O.sgemm(ta, tb, 1.0, A, B, 0.0, np.full((M, N), np.nan, np.float32))).all()


def test_bf16_converts_match_an_independent_implementation():
    """torch's bfloat16 is an independent round-to-nearest-even implementation."""
    import torch
    v = np.concatenate([H.f16_boundary_values(),
                        np.random.default_rng(8).integers(0, 2 ** 32, 1_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    # exact ties of bf16: patterns ending in 0x8000, both parities of the kept part
    ties = (np.arange(0x3f80, 0x4080, dtype=np.uint32) << 16 | 0x8000).view(np.float32)
    v = np.concatenate([v, ties, -ties, np.array([3.3895314e38, 3.4028235e38, np.inf, -np.inf, 0.0, -0.0, 1e-45], np.float32)])
    v = v[~np.isnan(v)]
    ref = torch.from_numpy(v.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.cvt_f32_bf16(v)
    assert np.array_equal(got, ref)
    allb = np.arange(65536, dtype=np.uint16)
    back = O.cvt_bf16_f32(allb)
    assert np.array_equal(back.view(np.uint32), allb.astype(np.uint32) << 16)
    assert np.isnan(O.cvt_bf16_f32(O.cvt_f32_bf16(np.array([np.nan], np.float32)))).all()


def test_adam_matches_formula():
    n = 257
    w = H.normal(17, n); g = H.normal(18, n); m = H.normal(19, n, 0, 0.1); v = np.abs(H.normal(20, n, 0, 0.1))
    t, lr, b1, b2, eps, wd = 3, 1e-3, 0.9, 0.999, 1e-8, 0.01
    w2, m2, v2 = O.adam_update(w, g, m, v, t, lr, b1, b2, eps, wd)
    lr, b1, b2, eps, wd = (float(np.float32(c)) for c in (lr, b1, b2, eps, wd))   # the op holds them as floats
    m64 = b1 * m.astype(np.float64) + (1 - b1) * g
    v64 = b2 * v.astype(np.float64) + (1 - b2) * g.astype(np.float64) ** 2
    w64 = w - lr * ((m64 / (1 - b1 ** t)) / (np.sqrt(v64 / (1 - b2 ** t)) + eps) + wd * w)
    assert H.rel_err(m2, m64) < 2e-6 and H.rel_err(v2, v64) < 2e-6 and H.rel_err(w2, w64) < 2e-6


def test_vocab_compaction():
    V, D = 300, 6
    data = H.zipf_ids(41, 500, V).astype(np.uint16)
    f2c, c2f = O.vocab_map_build(data, V)
    used = np.unique(data)
    assert np.array_equal(c2f, used)                                   # compact ids in ascending id order
    assert np.array_equal(f2c[used], np.arange(used.size)) and (np.delete(f2c, used) == -1).all()
    E = H.normal(42, (V, D)); ce = O.vocab_compact_embed(E, c2f)
    assert np.array_equal(ce, E[used])
    g = H.normal(43, (used.size, D)); G0 = H.normal(44, (V, D))
    G1 = O.vocab_scatter_grads(G0, g, c2f)
    ref = G0.copy(); ref[used] += g
    assert np.array_equal(G1, ref)
    E2 = O.vocab_update_full(E, ce * 2, c2f)
    ref = E.copy(); ref[used] = ce * 2
    assert np.array_equal(E2, ref)


def test_sumsq_and_clip_scale():
    g = H.normal(40, 100003) * 3
    gsc = np.float32(1.0 / 256.0)
    ref = float(np.sum((g * gsc).astype(np.float64) ** 2))          # the scale pass rounds to float32 first
    assert abs(O.sumsq_scaled(g, gsc) - ref) <= 2e-6 * ref
    assert O.sumsq_scaled(np.array([3.0, 4.0], np.float32), 1.0) == 25.0
    assert O.clip_scale(25.0, 1.0) == np.float32(1.0) / np.float32(5.0)   # norm 5 > clip 1 -> 1/5
    assert O.clip_scale(25.0, 10.0) == 1.0 and O.clip_scale(25.0, 0.0) == 1.0


# ---------------------------------------------------------------------------------------------
# embedding
# ---------------------------------------------------------------------------------------------
def test_embed_lookup_bit_exact_and_skips_out_of_range():
    V, D, B, S = 50, 12, 3, 9
    E = H.normal(21, (V, D), 0, 0.02)
    ids = H.zipf_ids(22, B * S, V).reshape(B, S)
    x, skipped = O.embed_lookup(E, ids)
    assert skipped == 0 and np.array_equal(x, E[ids].transpose(0, 2, 1))
    ids2 = ids.copy(); ids2[1, 4] = V; ids2[2, 0] = -1
    pre = H.normal(23, (B, D, S))
    x2, skipped = O.embed_lookup(E, ids2, out=pre)
    assert skipped == 2
    assert np.array_equal(x2[1, :, 4], pre[1, :, 4]) and np.array_equal(x2[2, :, 0], pre[2, :, 0])
    ok = (ids2 >= 0) & (ids2 < V)
    assert np.array_equal(x2.transpose(0, 2, 1)[ok], E[ids2[ok]])


def test_embed_backward_is_the_ordered_float32_sum():
    V, D, B, S = 40, 10, 4, 16
    ids = H.zipf_ids(24, B * S, V).reshape(B, S)
    ids[0, 3] = V + 5                                   # skipped
    dx = H.normal(25, (B, D, S)) * np.float32(1e3)      # large values make the order visible in the last bits
    dE0 = H.normal(26, (V, D))
    got = O.embed_backward(dE0, dx, ids)
    assert np.array_equal(got, H.np_embed_backward_f32(dE0, dx, ids))
    # the float64 sum agrees to rounding, and untouched rows are untouched
    ref = dE0.astype(np.float64)
    for b in range(B):
        for t in range(S):
            if 0 <= ids[b, t] < V:
                ref[ids[b, t]] += dx[b, :, t]
    assert H.rel_err(got, ref) < 1e-5
    untouched = np.setdiff1d(np.arange(V), ids[(ids >= 0) & (ids < V)])
    assert np.array_equal(got[untouched], dE0[untouched])


# ---------------------------------------------------------------------------------------------
# softmax + cross-entropy
# ---------------------------------------------------------------------------------------------
def test_cross_entropy_golden_and_properties():
    logits, tgt = GOLD["ce_logits"], GOLD["ce_targets"]
    loss, dl = O.cross_entropy(logits, tgt)
    assert abs(loss - float(GOLD["ce_loss"])) < 1e-6 * abs(float(GOLD["ce_loss"]))
    assert H.rel_err(dl, GOLD["ce_dlogits"]) < F32_FAITHFUL
    V, S = logits.shape
    assert np.max(np.abs(dl.astype(np.float64).sum(axis=0))) < 1e-7          # sum_v (p - onehot) = 0
    # shift invariance per column
    shift = H.normal(27, S)[None, :] * 3
    loss2, dl2 = O.cross_entropy(logits + shift, tgt)
    assert abs(loss2 - loss) < 1e-5 and H.rel_err(dl2, dl) < 1e-5
    # uniform logits: loss = -log(1/V + 1e-10)
    lu, du = O.cross_entropy(np.full((V, S), 0.7, np.float32), tgt)
    assert abs(lu - (-np.log(1.0 / V + 1e-10))) < 1e-6
    assert np.allclose(du[tgt, np.arange(S)], (1.0 / V - 1) / S, rtol=1e-6)
    # grad_scale multiplies dlogits only (training/training_dynamic/train.m:497)
    loss3, dl3 = O.cross_entropy(logits, tgt, grad_scale=256.0)
    assert loss3 == loss and np.array_equal(dl3, dl * np.float32(256.0))


def test_cross_entropy_matches_scalar_softmax_of_reference_test():
    """The scalar softmax loop of training/test_classifier.m:139-151 (max, exp, sum, divide)."""
    V, S = 101, 6
    x, _, _ = O.recipe_drand48(2, 999, V * S, 0)
    logits = x.reshape(V, S)
    tgt = np.full(S, -1, np.int32)                      # all skipped: dlogits is the plain softmax
    loss, p = O.cross_entropy(logits, tgt)
    assert loss == 0.0
    l64 = logits.astype(np.float64)
    e = np.exp(l64 - l64.max(axis=0))
    assert H.rel_err(p, e / e.sum(axis=0)) < F32_FAITHFUL
    assert np.allclose(p.astype(np.float64).sum(axis=0), 1.0, atol=1e-6)


def test_cross_entropy_out_of_range_target_policy():
    V, S = 23, 5
    logits = H.normal(28, (V, S), 0, 2)
    tgt = np.array([1, V, 3, -2, 22], np.int32)
    loss, dl = O.cross_entropy(logits, tgt)
    rl, rd = H.np_cross_entropy(logits, tgt)
    assert abs(loss - rl) < 1e-6 and H.rel_err(dl, rd) < F32_FAITHFUL
    assert abs(dl[:, 1].astype(np.float64).sum() - 1.0) < 1e-6      # skipped column = unscaled softmax


def test_column_softmax_and_nll_on_probabilities():
    """The halves of the op as training/train_large_ane.m:508-530 runs them: pinned by the float64 closed form, by
    the column sums, by the recipe of training/test_classifier.m:132-134, and against the fused op (the two
    formulations of the reference must agree: p*(1/sum) there, p/sum here)."""
    V, S = 101, 6
    x, _, _ = O.recipe_drand48(2, 999, V * S, 0)
    logits = x.reshape(V, S)
    p = O.softmax_cols(logits)
    l64 = logits.astype(np.float64)
    e = np.exp(l64 - l64.max(axis=0))
    p64 = e / e.sum(axis=0)
    assert H.err_elem(p, p64) < F32_FAITHFUL
    assert np.allclose(p.astype(np.float64).sum(axis=0), 1.0, atol=1e-6)
    assert np.all(p.argmax(axis=0) == logits.argmax(axis=0))
    tgt = np.array([3, 100, 0, 57, 57, 1], np.int32)
    loss, dl = O.nll_from_probs(p, tgt)
    cols = np.arange(S)
    assert abs(loss - (-np.log(p64[tgt, cols] + 1e-10).mean())) < 1e-6
    d64 = p64.copy(); d64[tgt, cols] -= 1.0; d64 /= S
    assert H.err_std(dl, d64) < F32_FAITHFUL
    assert np.max(np.abs(dl.astype(np.float64).sum(axis=0))) < 1e-7
    # same numbers as the fused op
    floss, fdl = O.cross_entropy(logits, tgt)
    assert abs(floss - loss) < 1e-6 and H.err_std(dl, fdl) < 1e-6
    # hand-computable: two classes, logits (0, ln 3) -> probs (1/4, 3/4)
    p2 = O.softmax_cols(np.array([[0.0], [np.log(3.0)]], np.float32))
    assert np.allclose(p2[:, 0], [0.25, 0.75], rtol=1e-6)
    l2, d2 = O.nll_from_probs(p2, np.array([1], np.int32))
    assert abs(l2 - (-np.log(0.75 + 1e-10))) < 1e-6 and np.allclose(d2[:, 0], [0.25, -0.25], rtol=1e-6)
    # a target outside the vocabulary: no loss term, no one-hot, column still scaled by 1/S
    l3, d3 = O.nll_from_probs(p, np.array([3, V, 0, -1, 57, 1], np.int32))
    assert np.allclose(d3[:, 1], p[:, 1] / S, rtol=1e-6) and np.allclose(d3[:, 3], p[:, 3] / S, rtol=1e-6)
    assert abs(l3 - (-(np.log(p64[[3, 0, 57, 1], [0, 2, 4, 5]] + 1e-10)).sum() / S)) < 1e-6


# ---------------------------------------------------------------------------------------------
# INT8
# ---------------------------------------------------------------------------------------------
def test_int8_golden_ties_and_bounds():
    x = GOLD["i8_x"]
    s = O.int8_scale(x)
    assert s == 1.0
    assert np.array_equal(O.int8_quant(x, s, 0), GOLD["i8_rne"])
    assert np.array_equal(O.int8_quant(x, s, 1), GOLD["i8_away"])
    assert O.int8_scale(np.zeros(5, np.float32)) == 1.0                 # all-zero tensor -> scale 1
    y = H.normal(29, 4099) * 3
    s = O.int8_scale(y)
    assert s == np.float32(np.max(np.abs(y))) / np.float32(127.0)
    for mode in (0, 1):
        q = O.int8_quant(y, s, mode)
        assert q.min() >= -127 and q.max() <= 127 and (np.abs(q) == 127).any()
        assert np.max(np.abs(O.int8_dequant(q, s).astype(np.float64) - y)) <= s / 2 * (1 + 1e-6)
    # clamp: values beyond the scale saturate at -128 / 127
    assert np.array_equal(O.int8_quant(np.array([1e6, -1e6], np.float32), 1.0, 0), np.array([127, -128], np.int8))
    q = O.int8_quant(y, s, 0)
    assert np.array_equal(q, np.clip(np.rint(y / np.float32(s)), -128, 127).astype(np.int8))


def test_minmax_matches_numpy_and_skips_nan():
    """orc_minmax (the loop's vDSP_minv / vDSP_maxv / vDSP_maxmgv diagnostics) against numpy's reductions."""
    x = H.normal(70, 10007) * np.float32(3.0)
    lo, hi, mg = O.minmax(x)
    assert lo == x.min() and hi == x.max() and mg == np.abs(x).max()
    assert tuple(O.minmax(np.array([-2.5], np.float32))) == (-2.5, -2.5, 2.5)
    y = x.copy(); y[5] = np.nan; y[100] = -50.0
    lo, hi, mg = O.minmax(y)
    assert lo == -50.0 and hi == np.nanmax(y) and mg == 50.0
