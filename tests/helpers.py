"""Shared test helpers: error metric, seeded inputs, and float64 closed forms written
independently of the C oracle (they pin it; see test_oracle_*.py)."""
import numpy as np

TOL_F32 = 1e-5          # the fp32 parity bound of this path


def rel_err(a, ref, floor=1.0):
    """max_i |a_i - ref_i| / max(|ref_i|, floor * rms(ref)).

    Element-wise relative error; `floor` (in units of the tensor's RMS) bounds the denominator from below.
    floor = 1: entries that are small by cancellation are judged against the scale of the tensor — used only
    for outputs whose formula subtracts nearly equal terms (RMSNorm dx, the rotation after a norm) or sums
    thousands of signed terms (dw, loss gradients through GEMMs).  See err_std and err_elem for the others."""
    a = np.asarray(a, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    assert a.shape == ref.shape
    if a.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    den = np.maximum(np.abs(ref), floor * (rms if rms > 0 else 1.0))
    den = np.maximum(den, 1.1754944e-38)        # entries below the smallest normal fp32 are judged against it
    diff = np.abs(a - ref)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(diff == 0.0, 0.0, diff / den)
    return float(np.max(q))


def err_std(a, ref):
    """The metric of this path: max |a - ref| / max(|ref|, 1e-3 * rms(ref))."""
    return rel_err(a, ref, 1e-3)


def err_elem(a, ref):
    """Pure element-wise relative error (no floor): for outputs that are products of the inputs with no
    subtraction (RMSNorm forward, SwiGLU forward, dh3, INT8 dequantize)."""
    return rel_err(a, ref, 0.0)


def normal(seed, shape, mean=0.0, std=1.0):
    return (mean + std * np.random.default_rng(seed).standard_normal(shape)).astype(np.float32)


def zipf_ids(seed, n, vocab, s=1.1):
    """n ids in [0, vocab): rank r (1-based) has probability proportional to r^-s; id = rank-1.
    Inverse-CDF sampling on a seeded uniform stream."""
    w = np.arange(1, vocab + 1, dtype=np.float64) ** (-s)
    cdf = np.cumsum(w / w.sum())
    u = np.random.default_rng(seed).random(n)
    return np.minimum(np.searchsorted(cdf, u, side="right"), vocab - 1).astype(np.int32)


# ---- the POSIX 48-bit LCG behind srand48/drand48, restated from its definition ----------------
class Drand48:
    A = 0x5DEECE66D
    C = 0xB
    M = 1 << 48

    def __init__(self, seed):
        self.x = ((seed & 0xFFFFFFFF) << 16) | 0x330E

    def next(self):
        self.x = (self.A * self.x + self.C) % self.M
        return self.x / float(self.M)

    def take(self, n):
        return np.array([self.next() for _ in range(n)], np.float64)


# ---- float64 closed forms (channel-first [.., C, S]) ----------------------------------------
def np_rrms(x, eps):
    x = np.asarray(x, np.float64)
    return 1.0 / np.sqrt(np.mean(x * x, axis=-2, keepdims=True) + eps)


def np_rmsnorm(x, w, eps=1e-5):
    x = np.asarray(x, np.float64)
    w = np.asarray(w, np.float64)
    return x * np_rrms(x, eps) * w[:, None]


def np_rmsnorm_bwd(dy, x, w, eps=1e-5, variant=0):
    """variant 0: dx = w*rr*(dy - x*dot), dot = rr^2/C * sum_c dy*x*w  (the reference CPU op);
    variant 1: dx = rr*(w*dy - x*dot)  (the exact gradient).  dw = sum_{b,s} dy*x*rr."""
    dy = np.asarray(dy, np.float64); x = np.asarray(x, np.float64); w = np.asarray(w, np.float64)
    C = x.shape[-2]
    rr = np_rrms(x, eps)
    wc = w[:, None]
    dot = (rr * rr / C) * np.sum(dy * x * wc, axis=-2, keepdims=True)
    if variant == 0:
        dx = wc * rr * (dy - x * dot)
    else:
        dx = rr * (wc * dy - x * dot)
    dw = np.sum((dy * x * rr).reshape(-1, C, x.shape[-1]), axis=(0, 2))
    return dx, dw


def np_sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def np_swiglu_fwd(h1, h3):
    h1 = np.asarray(h1, np.float64)
    return h1 * np_sigmoid(h1) * np.asarray(h3, np.float64)


def np_swiglu_bwd(d, h1, h3):
    d = np.asarray(d, np.float64); h1 = np.asarray(h1, np.float64); h3 = np.asarray(h3, np.float64)
    s = np_sigmoid(h1)
    return d * h3 * s * (1 + h1 * (1 - s)), d * h1 * s


def np_rope_angles(S, hd, theta):
    """[hd/2, S] angles p / theta^(2i/hd) in float64."""
    i = np.arange(hd // 2, dtype=np.float64)[:, None]
    p = np.arange(S, dtype=np.float64)[None, :]
    return p / np.power(float(theta), 2.0 * i / hd)


def np_rope(x, hd, theta, direction=+1, angles=None):
    """x [.., nheads*hd, S]; interleaved pairs (2i, 2i+1).  `angles` overrides the float64 angles
    (pass the float32-rounded ones to separate rotation error from angle error)."""
    x = np.asarray(x, np.float64)
    S = x.shape[-1]
    ang = np_rope_angles(S, hd, theta) if angles is None else np.asarray(angles, np.float64)
    c, s = np.cos(ang), direction * np.sin(ang)
    xs = x.reshape(x.shape[:-2] + (-1, hd // 2, 2, S))
    x0, x1 = xs[..., 0, :], xs[..., 1, :]
    out = np.stack([x0 * c - x1 * s, x0 * s + x1 * c], axis=-2)
    return out.reshape(x.shape)


def np_qknorm_rope_fwd(x, w, hd, theta, eps=1e-5, angles=None):
    x = np.asarray(x, np.float64)
    xs = x.reshape(x.shape[:-2] + (-1, hd, x.shape[-1]))
    y = np_rmsnorm(xs, w, eps).reshape(x.shape)
    return np_rope(y, hd, theta, +1, angles)


def np_qknorm_rope_bwd(dy, x, w, hd, theta, eps=1e-5, variant=0, angles=None):
    x = np.asarray(x, np.float64)
    g = np_rope(dy, hd, theta, -1, angles)
    S = x.shape[-1]
    xs = x.reshape(-1, hd, S); gs = g.reshape(-1, hd, S)
    dx, dw = np_rmsnorm_bwd(gs, xs, w, eps, variant)
    return dx.reshape(x.shape), dw


def np_cross_entropy(logits, targets, grad_scale=1.0):
    """logits [V,S]; returns (loss, dlogits) with the reference's +1e-10 inside the log and the
    skip of out-of-range targets (column left as the unscaled softmax)."""
    l = np.asarray(logits, np.float64)
    V, S = l.shape
    e = np.exp(l - l.max(axis=0, keepdims=True))
    p = e / e.sum(axis=0, keepdims=True)
    t = np.asarray(targets)
    ok = (t >= 0) & (t < V)
    cols = np.arange(S)
    loss = -np.sum(np.log(p[t[ok], cols[ok]] + 1e-10)) / S
    d = p.copy()
    d[t[ok], cols[ok]] -= 1.0
    d[:, ok] /= S
    return loss, d * grad_scale


def np_embed_backward_f32(dE, dx, tokens):
    """Sequential float32 accumulation in ascending (b, t) order — the definition of the op."""
    dE = np.array(dE, np.float32, copy=True)
    dx = np.asarray(dx, np.float32)
    B, D, S = dx.shape
    V = dE.shape[0]
    tok = np.asarray(tokens).reshape(B, S)
    for b in range(B):
        for t in range(S):
            k = int(tok[b, t])
            if 0 <= k < V:
                dE[k] = dE[k] + dx[b, :, t]
    return dE


def f16_boundary_values():
    """float32 inputs on and around every rounding boundary of binary16."""
    h = np.arange(0x0000, 0x7c01, dtype=np.uint16).view(np.float16).astype(np.float64)     # all finite halves >= 0, inf
    mids = (h[:-1] + h[1:]) / 2                                                            # the exact ties
    mids = mids[np.isfinite(mids)]
    near = np.concatenate([mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                           np.nextafter(mids.astype(np.float32), np.float32(-np.inf))]).astype(np.float32)
    extra = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                      2.0 ** -25 * 1.0000001, 2.0 ** -26, 1e-40, 5.9604645e-08, 6.1035156e-05, 6.0975552e-05],
                     np.float32)
    v = np.concatenate([h[np.isfinite(h)].astype(np.float32), near, extra])
    return np.concatenate([v, -v])


# ---- checkpoints: the file as save_checkpoint writes it, and the offsets as the dashboard reads it ----
CKPT_MAGIC = 0x424C5A54


def ckpt_sizes(cfg):
    """Element counts of the nine per-layer tensors in file order (train.m:118-122 of the dynamic loop)."""
    dim, hid, qd, kvd = cfg["dim"], cfg["hidden"], cfg["q_dim"], cfg["kv_dim"]
    return [qd * dim, kvd * dim, kvd * dim, dim * qd, hid * dim, dim * hid, hid * dim, dim, dim]


def ckpt_header_bytes(cfg, version, step=7, total_steps=100, lr=3e-4, loss=2.5, adam_t=9):
    import struct
    tail = (cfg["kv_heads"], cfg["head_dim"], cfg["q_dim"]) if version == 4 else (0, 0, 0)
    return struct.pack("<10i2f3d3i3i", CKPT_MAGIC, version, step, total_steps, cfg["layers"], cfg["vocab"], cfg["dim"],
                       cfg["hidden"], cfg["heads"], cfg["seq"], lr, loss, 1.5, 2.5, 3.5, 11, 12, adam_t, *tail)


def ckpt_write_like_reference(path, cfg, version, seed=0):
    """Writes header + tensors with sequential writes in save_checkpoint's order; returns {(layer, tensor, part): array}."""
    rng = np.random.default_rng(seed)
    tensors = {}
    with open(path, "wb") as f:
        f.write(ckpt_header_bytes(cfg, version))
        sizes = ckpt_sizes(cfg)
        for L in range(cfg["layers"]):
            for t, n in enumerate(sizes):                       # the nine weights
                a = rng.standard_normal(n).astype(np.float32); tensors[(L, t, 0)] = a; f.write(a.tobytes())
            for t, n in enumerate(sizes):                       # then (m, v) of each
                for part in (1, 2):
                    a = rng.standard_normal(n).astype(np.float32); tensors[(L, t, part)] = a; f.write(a.tobytes())
        for t, n in ((9, cfg["dim"]), (10, cfg["vocab"] * cfg["dim"])):
            for part in (0, 1, 2):
                a = rng.standard_normal(n).astype(np.float32); tensors[(0, t, part)] = a; f.write(a.tobytes())
    return tensors


def ckpt_weight_offsets_like_dashboard(cfg):
    """Byte offsets of the weights as training/dashboard.py:141-174 walks the file: 96-byte header, nine weights
    per layer, a seek over the layer's Adam block, rms_final, a seek over its Adam pair, embed."""
    sizes = ckpt_sizes(cfg)
    adam_per_layer = 2 * sum(sizes)
    off, out = 96, {}
    for L in range(cfg["layers"]):
        for t, n in enumerate(sizes):
            out[(L, t)] = off; off += 4 * n
        off += 4 * adam_per_layer
    out[(0, 9)] = off; off += 4 * cfg["dim"] + 4 * 2 * cfg["dim"]
    out[(0, 10)] = off
    return out


def np_embed_backward(dE0, dx, ids):
    """dE0 + per-token sums of dx columns in float64 (the exact value both summation orders approximate)."""
    B, D, S = dx.shape
    V = dE0.shape[0]
    out = dE0.astype(np.float64).copy()
    flat = ids.reshape(-1)
    cols = dx.transpose(0, 2, 1).reshape(B * S, D).astype(np.float64)
    ok = (flat >= 0) & (flat < V)
    np.add.at(out, flat[ok], cols[ok])
    return out
