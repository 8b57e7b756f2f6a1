"""The C mirror of the reference's training-step op sequence (ane_amd/host/train_step_mirror.c), run
on the GPU through the reference-named ops of include/mi355_cpu_ops.h, against a replay of the same
sequence with the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "ane_amd", "host", "train_step_mirror")

DIM, HIDDEN, HEADS, KV_HEADS, HD, SEQ, NLAYERS, VOCAB = 64, 160, 4, 2, 16, 32, 2, 500
Q_DIM, KV_DIM = HEADS * HD, KV_HEADS * HD
f32 = np.float32


class Lcg:
    def __init__(self):
        self.s = 12345

    def frand(self):
        self.s = (self.s * 1664525 + 1013904223) & 0xFFFFFFFF
        return f32(f32(self.s >> 8) * f32(1.0 / 16777216.0) - f32(0.5))


def stage(inp, n_out, salt):
    inp = np.ascontiguousarray(inp, f32).ravel()
    i = np.arange(n_out, dtype=np.int64)
    a = inp[(i * 7 + salt) % inp.size] * f32(0.5)
    b = f32(0.25) * inp[(i * 13 + 3 * salt) % inp.size]
    return (a + b).astype(f32)


CLS_GAIN = f32(16.0)
NSTEPS, NTOKENS = 2, 4 * SEQ + 1


def host_gemm(A, B):
    """The mirror's stand-in for cblas_sgemm: double accumulation, rounded once, times the gain."""
    return ((A.astype(np.float64) @ B.astype(np.float64)).astype(f32) * CLS_GAIN).astype(f32)


def replay():
    """Both steps of the mirror with the CPU oracle; returns (CV, [per-step dict])."""
    g = Lcg()
    embed = np.array([f32(0.04) * g.frand() for _ in range(VOCAB * DIM)], f32).reshape(VOCAB, DIM)
    rms_att, rms_ffn = [], []
    for _ in range(NLAYERS):
        a = np.empty(DIM, f32); b = np.empty(DIM, f32)
        for i in range(DIM):
            a[i] = f32(1.0) + f32(0.1) * g.frand()
            b[i] = f32(1.0) + f32(0.1) * g.frand()
        rms_att.append(a); rms_ffn.append(b)
    rms_final = np.array([f32(1.0) + f32(0.1) * g.frand() for _ in range(DIM)], f32)
    data = np.array([(7 * t + 13) % 256 + 1 for t in range(NTOKENS)], np.uint16)
    data[5] = data[2]
    alpha = f32(1.0) / np.sqrt(f32(2.0 * NLAYERS), dtype=f32)
    DS, HS, QS, KS = DIM * SEQ, HIDDEN * SEQ, Q_DIM * SEQ, KV_DIM * SEQ

    f2c, c2f = O.vocab_map_build(data, VOCAB)
    CV = c2f.size
    cembed = O.vocab_compact_embed(embed, c2f)
    z = np.zeros_like
    st = dict(final=(z(rms_final), z(rms_final)), embed=(z(embed), z(embed)),
              att=[(z(w), z(w)) for w in rms_att], ffn=[(z(w), z(w)) for w in rms_ffn])
    steps = []
    for step in range(NSTEPS):
        tok = data[17 * step:17 * step + SEQ].astype(np.int32)
        ctgt = f2c[data[17 * step + 1:17 * step + 1 + SEQ]].astype(np.int32)
        x_cur = O.embed_lookup(embed, tok[None])[0][0]
        out = {"x": x_cur.copy()}
        acts = []
        for L in range(NLAYERS):
            ac = {"layer_in": x_cur.copy()}
            ac["xnorm"] = O.rmsnorm(x_cur, rms_att[L])
            attn_out = stage(ac["xnorm"], QS, 1 + L)
            o_out = stage(attn_out, DS, 2 + L).reshape(DIM, SEQ)
            ac["x2"] = O.axpby(x_cur, o_out, alpha, 0)
            x2norm = O.rmsnorm(ac["x2"], rms_ffn[L])
            ac["h1"] = stage(x2norm, HS, 3 + L); ac["h3"] = stage(x2norm, HS, 4 + L)
            silu = O.swiglu_fwd(ac["h1"], ac["h3"])
            ffn_out = stage(silu, DS, 5 + L).reshape(DIM, SEQ)
            x_cur = O.axpby(ac["x2"], ffn_out, alpha, 0)
            acts.append(ac)
        x_final = O.rmsnorm(x_cur, rms_final)
        logits = host_gemm(cembed, x_final)
        loss, dlogits = O.cross_entropy(logits, ctgt)
        dlogits = O.axpby(dlogits, None, f32(256.0), 1)
        dy = host_gemm(cembed.T, dlogits)
        gcembed = host_gemm(dlogits, x_final.T)
        dy, grms_final = O.rmsnorm_bwd(dy, x_cur, rms_final)
        g_att = [None] * NLAYERS; g_ffn = [None] * NLAYERS
        for L in reversed(range(NLAYERS)):
            ac = acts[L]
            dffn = O.axpby(dy, None, alpha, 1)
            dsilu = stage(dffn, HS, 8 + L)
            dh1, dh3 = O.swiglu_bwd(dsilu, ac["h1"], ac["h3"])
            dx_ffn = stage(np.concatenate([dh1, dh3]), DS, 9 + L).reshape(DIM, SEQ)
            dx2, g_ffn[L] = O.rmsnorm_bwd(dx_ffn, ac["x2"], rms_ffn[L])
            dx2 = O.axpby(dx2, dy, 0.0, 2)
            dx2s = O.axpby(dx2, None, alpha, 1)
            da = stage(dx2s, QS, 10 + L)
            dq = O.rope(stage(da, QS, 11 + L).reshape(Q_DIM, SEQ), HD, 10000.0, -1)
            dk = O.rope(stage(da, KS, 12 + L).reshape(KV_DIM, SEQ), HD, 10000.0, -1)
            dx_attn = O.axpby(stage(dq, DS, 13 + L), stage(dk, DS, 14 + L), 0.0, 2).reshape(DIM, SEQ)
            dx_rms, g_att[L] = O.rmsnorm_bwd(dx_attn, ac["layer_in"], rms_att[L])
            dy = O.axpby(dx_rms, dx2, 0.0, 2)
        gembed = O.embed_backward(np.zeros((VOCAB, DIM), f32), dy[None], tok[None])
        # optimizer tail: 1/loss_scale, compact classifier gradient scattered into the full one, Adam
        gsc = f32(1.0) / f32(256.0)
        g_att = [g * gsc for g in g_att]; g_ffn = [g * gsc for g in g_ffn]
        grms_final = grms_final * gsc
        gembed = O.vocab_scatter_grads(gembed, gcembed, c2f) * gsc
        out.update(loss=loss, dy=dy, grms_final=grms_final, g_att=g_att, g_ffn=g_ffn, gembed=gembed)
        hp = dict(t=step + 1, lr=3e-4, b1=0.9, b2=0.95, eps=1e-8)
        for L in range(NLAYERS):
            rms_att[L], *st["att"][L] = O.adam_update(rms_att[L], g_att[L], *st["att"][L], wd=0.0, **hp)
            rms_ffn[L], *st["ffn"][L] = O.adam_update(rms_ffn[L], g_ffn[L], *st["ffn"][L], wd=0.0, **hp)
        rms_final, *st["final"] = O.adam_update(rms_final, grms_final, *st["final"], wd=0.0, **hp)
        embed, *st["embed"] = O.adam_update(embed, gembed, *st["embed"], wd=0.1, **hp)
        cembed = O.vocab_compact_embed(embed, c2f)
        out.update(w_final=rms_final.copy(), w_att=[w.copy() for w in rms_att], w_ffn=[w.copy() for w in rms_ffn],
                   w_embed=embed.copy(), cembed=cembed.copy())
        steps.append(out)
    return CV, steps


def test_training_step_mirror_matches_oracle_replay(tmp_path):
    assert os.path.exists(BIN), "build it first: python -m ane_amd.build"
    out = tmp_path / "mirror.bin"
    r = subprocess.run([BIN, str(out)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    raw = np.fromfile(out, f32)
    CV, steps = replay()
    assert int(raw[0]) == CV
    DS, VD = DIM * SEQ, VOCAB * DIM
    per_step = [DS, 1, DS, DIM] + [DIM] * (2 * NLAYERS) + [VD] + [DIM] + [DIM] * (2 * NLAYERS) + [VD, CV * DIM]
    assert raw.size == 1 + NSTEPS * sum(per_step)
    data = np.array([(7 * t + 13) % 256 + 1 for t in range(NTOKENS)])
    data[5] = data[2]
    # a chain of ~40 ops per step: each is held to 1e-5 on its own (test_gpu_parity.py); the chain to 1e-4
    tol = 1e-4
    pos = 1
    prev_embed = None
    for step, ref in enumerate(steps):
        parts = []
        for n in per_step:
            parts.append(raw[pos:pos + n]); pos += n
        it = iter(parts)
        # the gather is a copy of the table the mirror holds: the initial one at step 0, afterwards the rows that
        # the previous step's adam_update wrote (a resident device copy that missed the update would show here)
        x = next(it)
        tok = data[17 * step:17 * step + SEQ]
        want_x = ref["x"] if prev_embed is None else np.ascontiguousarray(prev_embed[tok].T)
        assert x.tobytes() == want_x.tobytes(), "step %d: embed_lookup read stale rows" % step
        assert H.rel_err(x, ref["x"]) <= 1e-5
        assert abs(next(it)[0] - ref["loss"]) <= 1e-5 * abs(ref["loss"])
        assert H.rel_err(next(it), ref["dy"]) <= tol
        assert H.rel_err(next(it), ref["grms_final"]) <= tol
        for L in range(NLAYERS):
            assert H.rel_err(next(it), ref["g_att"][L]) <= tol
            assert H.rel_err(next(it), ref["g_ffn"][L]) <= tol
        ge = next(it)
        assert H.rel_err(ge, ref["gembed"]) <= tol
        untouched = np.setdiff1d(np.arange(VOCAB), np.unique(data))
        assert not ge.reshape(VOCAB, DIM)[untouched].any()
        # weights after the Adam step (the update is ~lr*sign(g) at first, so these are tight)
        assert H.rel_err(next(it), ref["w_final"]) <= 1e-5
        for L in range(NLAYERS):
            assert H.rel_err(next(it), ref["w_att"][L]) <= 1e-5
            assert H.rel_err(next(it), ref["w_ffn"][L]) <= 1e-5
        we = next(it)
        assert H.rel_err(we, ref["w_embed"]) <= 1e-5
        ce = next(it)
        # the re-compacted classifier table is a row copy of the table the mirror itself holds
        _, c2f = O.vocab_map_build(data.astype(np.uint16), VOCAB)
        assert ce.tobytes() == we.reshape(VOCAB, DIM)[c2f].tobytes()
        prev_embed = we.reshape(VOCAB, DIM).copy()
    if NSTEPS > 1:
        assert not np.array_equal(steps[0]["w_embed"], steps[1]["w_embed"])
