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


def replay():
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
    tok = np.array([(7 * t + 13) % 256 + 1 for t in range(SEQ)], np.int32)
    tgt = np.array([(7 * (t + 1) + 13) % 256 + 1 for t in range(SEQ)], np.int32)
    tok[5] = tok[2]
    alpha = f32(1.0) / np.sqrt(f32(2.0 * NLAYERS), dtype=f32)
    DS, HS, QS, KS, VS = DIM * SEQ, HIDDEN * SEQ, Q_DIM * SEQ, KV_DIM * SEQ, VOCAB * SEQ

    x_cur = O.embed_lookup(embed, tok[None])[0][0]
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
    logits = (stage(x_final, VS, 6) * f32(4.0)).reshape(VOCAB, SEQ)
    loss, dlogits = O.cross_entropy(logits, tgt)
    dlogits = O.axpby(dlogits, None, f32(256.0), 1)
    dy = stage(dlogits, DS, 7).reshape(DIM, SEQ)
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
    # optimizer tail: scale by 1/loss_scale, then one Adam step (AdamW with wd on the embedding only)
    gsc = f32(1.0) / f32(256.0)
    g_att = [g * gsc for g in g_att]; g_ffn = [g * gsc for g in g_ffn]
    grms_final = grms_final * gsc; gembed = gembed * gsc
    hp = dict(t=1, lr=3e-4, b1=0.9, b2=0.95, eps=1e-8)
    z = lambda a: np.zeros_like(a)
    w_att = [O.adam_update(rms_att[L], g_att[L], z(rms_att[L]), z(rms_att[L]), wd=0.0, **hp)[0] for L in range(NLAYERS)]
    w_ffn = [O.adam_update(rms_ffn[L], g_ffn[L], z(rms_ffn[L]), z(rms_ffn[L]), wd=0.0, **hp)[0] for L in range(NLAYERS)]
    w_final = O.adam_update(rms_final, grms_final, z(rms_final), z(rms_final), wd=0.0, **hp)[0]
    w_embed = O.adam_update(embed, gembed, z(embed), z(embed), wd=0.1, **hp)[0]
    return loss, dy, grms_final, g_att, g_ffn, gembed, w_final, w_att, w_ffn, w_embed


def test_training_step_mirror_matches_oracle_replay(tmp_path):
    assert os.path.exists(BIN), "build it first: python -m ane_amd.build"
    out = tmp_path / "mirror.bin"
    r = subprocess.run([BIN, str(out)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    raw = np.fromfile(out, f32)
    DS = DIM * SEQ
    sizes = [1, DS, DIM] + [DIM] * (2 * NLAYERS) + [VOCAB * DIM] + [DIM] + [DIM] * (2 * NLAYERS) + [VOCAB * DIM]
    assert raw.size == sum(sizes)
    parts = np.split(raw, np.cumsum(sizes)[:-1])
    loss, dy, grms_final, g_att, g_ffn, gembed, w_final, w_att, w_ffn, w_embed = replay()
    # a chain of ~40 ops: each is held to 1e-5 on its own (test_gpu_parity.py); the chain to 1e-4
    tol = 1e-4
    assert abs(parts[0][0] - loss) <= 1e-5 * abs(loss)
    assert H.rel_err(parts[1], dy) <= tol
    assert H.rel_err(parts[2], grms_final) <= tol
    for L in range(NLAYERS):
        assert H.rel_err(parts[3 + 2 * L], g_att[L]) <= tol
        assert H.rel_err(parts[4 + 2 * L], g_ffn[L]) <= tol
    ge = 3 + 2 * NLAYERS
    assert H.rel_err(parts[ge], gembed) <= tol
    touched = np.unique([(7 * t + 13) % 256 + 1 for t in range(SEQ)])
    untouched = np.setdiff1d(np.arange(VOCAB), touched)
    assert not parts[ge].reshape(VOCAB, DIM)[untouched].any()
    # weights after the Adam step (first step: the update is ~lr*sign(g), so compare the CHANGE as well)
    assert H.rel_err(parts[ge + 1], w_final) <= 1e-6
    for L in range(NLAYERS):
        assert H.rel_err(parts[ge + 2 + 2 * L], w_att[L]) <= 1e-6
        assert H.rel_err(parts[ge + 3 + 2 * L], w_ffn[L]) <= 1e-6
    assert H.rel_err(parts[-1], w_embed) <= 1e-5
