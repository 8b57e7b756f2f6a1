"""ctypes loader for the CPU oracle (``liboracle.so``, built from ``oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the CPU-baseline
leg of ``bench.py``.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(dtype=np.int8, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile liboracle.so with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)


def _stale():
    if not os.path.exists(_SO):
        return True
    built = os.path.getmtime(_SO)
    return any(os.path.getmtime(os.path.join(_HERE, f)) > built for f in ("oracle.c", "Makefile"))


def _load():
    if _stale():
        build(force=True)
    lib = C.CDLL(_SO)
    sig = {
        "orc_rmsnorm": (None, [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_float]),
        "orc_rmsnorm_bwd": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_float, C.c_int]),
        "orc_swiglu_fwd": (None, [_f32p, _f32p, _f32p, C.c_size_t]),
        "orc_swiglu_bwd": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_size_t]),
        "orc_rope_tables": (None, [_f32p, _f32p, C.c_int, C.c_int, C.c_float]),
        "orc_rope_bwd": (None, [_f32p, C.c_int, C.c_int, C.c_int, C.c_float]),
        "orc_rope_fwd": (None, [_f32p, C.c_int, C.c_int, C.c_int, C.c_float]),
        "orc_qknorm_rope_fwd": (None, [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float]),
        "orc_qknorm_rope_bwd": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int,
                                       C.c_float, C.c_float, C.c_int]),
        "orc_axpby": (None, [_f32p, _f32p, C.c_void_p, C.c_float, C.c_size_t, C.c_int]),
        "orc_embed_lookup": (C.c_int, [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int]),
        "orc_embed_backward": (None, [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int]),
        "orc_cross_entropy": (C.c_float, [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_float]),
        "orc_softmax_cols": (None, [_f32p, _f32p, C.c_int, C.c_int]),
        "orc_nll_from_probs": (C.c_float, [_f32p, _f32p, _i32p, C.c_int, C.c_int]),
        "orc_minmax": (None, [_f32p, _f32p, C.c_size_t]),
        "orc_int8_scale": (C.c_float, [_f32p, C.c_size_t]),
        "orc_int8_quant": (None, [_i8p, _f32p, C.c_size_t, C.c_float, C.c_int]),
        "orc_int8_dequant": (None, [_f32p, _i8p, C.c_size_t, C.c_float]),
        "orc_gqa_tile": (None, [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]),
        "orc_gqa_reduce": (None, [_f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]),
        "orc_sgemm": (None, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _f32p, C.c_int, _f32p, C.c_int,
                             C.c_float, _f32p, C.c_int, C.c_int]),
        "orc_cvt_f32_bf16": (None, [_u16p, _f32p, C.c_size_t]),
        "orc_cvt_bf16_f32": (None, [_f32p, _u16p, C.c_size_t]),
        "orc_cvt_f32_f16": (None, [_u16p, C.c_size_t, _f32p, C.c_size_t, C.c_size_t, C.c_size_t]),
        "orc_cvt_f16_f32": (None, [_f32p, C.c_size_t, _u16p, C.c_size_t, C.c_size_t, C.c_size_t]),
        "orc_adam_update": (None, [_f32p, _f32p, _f32p, _f32p, C.c_size_t, C.c_int, C.c_float,
                                   C.c_float, C.c_float, C.c_float, C.c_float]),
        "orc_rmsnorm_batched": (None, [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int]),
        "orc_rmsnorm_bwd_batched": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int,
                                           C.c_float, C.c_int, C.c_int]),
        "orc_qknorm_rope_fwd_batched": (None, [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.c_float, C.c_float, C.c_int]),
        "orc_qknorm_rope_bwd_batched": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int,
                                               C.c_int, C.c_float, C.c_float, C.c_int, C.c_int]),
        "orc_rope_batched": (None, [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int]),
        "orc_swiglu_fwd_mt": (None, [_f32p, _f32p, _f32p, C.c_size_t, C.c_int]),
        "orc_swiglu_bwd_mt": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, C.c_size_t, C.c_int]),
        "orc_axpby_mt": (None, [_f32p, _f32p, C.c_void_p, C.c_float, C.c_size_t, C.c_int, C.c_int]),
        "orc_embed_lookup_batched": (C.c_int, [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int]),
        "orc_embed_backward_batched": (None, [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int]),
        "orc_sumsq_scaled": (C.c_float, [_f32p, C.c_size_t, C.c_float]),
        "orc_clip_scale": (C.c_float, [C.c_float, C.c_float]),
        "orc_vocab_map_build": (C.c_int, [_i32p, _i32p, np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS"),
                                          C.c_size_t, C.c_int]),
        "orc_vocab_compact_embed": (None, [_f32p, _f32p, _i32p, C.c_int, C.c_int]),
        "orc_vocab_scatter_grads": (None, [_f32p, _f32p, _i32p, C.c_int, C.c_int]),
        "orc_vocab_update_full": (None, [_f32p, _f32p, _i32p, C.c_int, C.c_int]),
        "orc_recipe_drand48": (None, [C.c_int, C.c_long, _f32p, _f32p, _f32p, C.c_size_t, C.c_int]),
        "orc_now_s": (C.c_double, []),
        "orc_max_threads": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


# ---- numpy-level wrappers (inputs are not modified unless stated) --------------------------------

def rmsnorm(x, w, eps=1e-5, threads=1):
    """x [B,C,S] or [C,S] -> y of the same shape."""
    x = _f32(x); w = _f32(w)
    x3 = x.reshape((-1,) + x.shape[-2:])
    out = np.empty_like(x3)
    lib.orc_rmsnorm_batched(out, x3, w, x3.shape[1], x3.shape[2], x3.shape[0], eps, threads)
    return out.reshape(x.shape)


def rmsnorm_bwd(dy, x, w, eps=1e-5, variant=0, dw=None, threads=1):
    """Returns (dx, dw); dw accumulates onto the given array (copied) or zeros."""
    dy = _f32(dy); x = _f32(x); w = _f32(w)
    x3 = x.reshape((-1,) + x.shape[-2:]); dy3 = dy.reshape(x3.shape)
    dx = np.empty_like(x3)
    dwo = np.zeros_like(w) if dw is None else _f32(dw).copy()
    lib.orc_rmsnorm_bwd_batched(dx, dwo, dy3, x3, w, x3.shape[1], x3.shape[2], x3.shape[0], eps, variant, threads)
    return dx.reshape(x.shape), dwo


def swiglu_fwd(h1, h3, threads=1):
    h1 = _f32(h1); h3 = _f32(h3)
    out = np.empty_like(h1)
    lib.orc_swiglu_fwd_mt(out, h1, h3, h1.size, threads)
    return out


def swiglu_bwd(dsilu, h1, h3, threads=1):
    dsilu = _f32(dsilu); h1 = _f32(h1); h3 = _f32(h3)
    dh1 = np.empty_like(h1); dh3 = np.empty_like(h1)
    lib.orc_swiglu_bwd_mt(dh1, dh3, dsilu, h1, h3, h1.size, threads)
    return dh1, dh3


def rope_tables(S, hd, theta):
    c = np.empty((hd // 2, S), np.float32); s = np.empty((hd // 2, S), np.float32)
    lib.orc_rope_tables(c, s, S, hd, theta)
    return c, s


def rope(x, hd, theta, direction=+1, threads=1):
    """x [B,dim,S] or [dim,S]; returns the rotated copy (direction +1 forward, -1 backward)."""
    x = _f32(x).copy()
    x3 = x.reshape((-1,) + x.shape[-2:])
    lib.orc_rope_batched(x3, x3.shape[2], x3.shape[1], hd, x3.shape[0], theta, direction, threads)
    return x


def qknorm_rope_fwd(x, w, hd, theta, eps=1e-5, threads=1):
    x = _f32(x); w = _f32(w)
    x3 = x.reshape((-1,) + x.shape[-2:])
    out = np.empty_like(x3)
    lib.orc_qknorm_rope_fwd_batched(out, x3, w, x3.shape[1] // hd, hd, x3.shape[2], x3.shape[0], theta, eps, threads)
    return out.reshape(x.shape)


def qknorm_rope_bwd(dy, x, w, hd, theta, eps=1e-5, variant=0, dw=None, threads=1):
    dy = _f32(dy); x = _f32(x); w = _f32(w)
    x3 = x.reshape((-1,) + x.shape[-2:]); dy3 = dy.reshape(x3.shape)
    dx = np.empty_like(x3)
    dwo = np.zeros_like(w) if dw is None else _f32(dw).copy()
    lib.orc_qknorm_rope_bwd_batched(dx, dwo, dy3, x3, w, x3.shape[1] // hd, hd, x3.shape[2], x3.shape[0],
                                    theta, eps, variant, threads)
    return dx.reshape(x.shape), dwo


def axpby(a, b, alpha, mode, threads=1):
    a = _f32(a)
    y = np.empty_like(a)
    bp = None if b is None else _f32(b)
    lib.orc_axpby_mt(y, a, None if bp is None else bp.ctypes.data, alpha, a.size, mode, threads)
    return y


def embed_lookup(embed, tokens, out=None):
    """embed [V,D], tokens [B,S] or [S] -> x [B,D,S]; returns (x, skipped)."""
    embed = _f32(embed); tokens = _i32(tokens)
    t2 = tokens.reshape(-1, tokens.shape[-1])
    B, S = t2.shape
    V, D = embed.shape
    x = np.zeros((B, D, S), np.float32) if out is None else _f32(out).copy().reshape(B, D, S)
    skipped = lib.orc_embed_lookup_batched(x, embed, t2, V, D, S, B)
    return x, skipped


def embed_backward(d_embed, dx, tokens):
    """Accumulates onto a copy of d_embed [V,D]; dx [B,D,S]; tokens [B,S]."""
    dE = _f32(d_embed).copy(); dx = _f32(dx); tokens = _i32(tokens)
    t2 = tokens.reshape(-1, tokens.shape[-1])
    B, S = t2.shape
    V, D = dE.shape
    lib.orc_embed_backward_batched(dE, dx.reshape(B, D, S), t2, V, D, S, B)
    return dE


def cross_entropy(logits, targets, grad_scale=1.0):
    logits = _f32(logits); targets = _i32(targets)
    V, S = logits.shape
    dl = np.empty_like(logits)
    loss = lib.orc_cross_entropy(dl, logits, targets, V, S, grad_scale)
    return float(loss), dl


def softmax_cols(logits):
    """Column softmax of logits [V,S] — train_large_ane.m:508-516."""
    logits = _f32(logits)
    V, S = logits.shape
    p = np.empty_like(logits)
    lib.orc_softmax_cols(p, logits, V, S)
    return p


def nll_from_probs(probs, targets):
    """(loss, dlogits) from probabilities [V,S] — train_large_ane.m:519-530."""
    probs = _f32(probs); targets = _i32(targets)
    V, S = probs.shape
    dl = np.empty_like(probs)
    loss = lib.orc_nll_from_probs(dl, probs, targets, V, S)
    return float(loss), dl


def minmax(x):
    """(min, max, max|x|) of a tensor — train.m:664-666,738-742."""
    x = _f32(x)
    out = np.empty(3, np.float32)
    lib.orc_minmax(out, x.reshape(-1), x.size)
    return out


def int8_scale(x):
    x = _f32(x)
    return float(lib.orc_int8_scale(x.reshape(-1), x.size))


def int8_quant(x, scale, rounding=0):
    x = _f32(x)
    q = np.empty(x.shape, np.int8)
    lib.orc_int8_quant(q.reshape(-1), x.reshape(-1), x.size, scale, rounding)
    return q


def int8_dequant(q, scale):
    q = np.ascontiguousarray(q, np.int8)
    x = np.empty(q.shape, np.float32)
    lib.orc_int8_dequant(x.reshape(-1), q.reshape(-1), q.size, scale)
    return x


def sgemm(ta, tb, alpha, A, B, beta=0.0, Cin=None, threads=8):
    """Row-major C = alpha*op(A)*op(B) + beta*C on 2-D arrays (leading dimensions = row lengths)."""
    A = _f32(A); B = _f32(B)
    M, K = (A.shape[1], A.shape[0]) if ta else A.shape
    N = B.shape[0] if tb else B.shape[1]
    out = np.zeros((M, N), np.float32) if Cin is None else _f32(Cin).copy()
    lib.orc_sgemm(int(ta), int(tb), M, N, K, alpha, A.reshape(-1), A.shape[1], B.reshape(-1), B.shape[1], beta,
                  out.reshape(-1), N, threads)
    return out


def cvt_f32_bf16(x):
    """fp32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    lib.orc_cvt_f32_bf16(out.reshape(-1), x.reshape(-1), x.size)
    return out


def cvt_bf16_f32(h):
    h = np.ascontiguousarray(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.orc_cvt_bf16_f32(out.reshape(-1), h.reshape(-1), h.size)
    return out


def cvt_f32_f16(x):
    """fp32 -> fp16 bit patterns (uint16), same shape."""
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    lib.orc_cvt_f32_f16(out.reshape(-1), x.size, x.reshape(-1), x.size, 1, x.size)
    return out


def cvt_f16_f32(h):
    """fp16 bit patterns (uint16) -> fp32, same shape."""
    h = np.ascontiguousarray(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.orc_cvt_f16_f32(out.reshape(-1), h.size, h.reshape(-1), h.size, 1, h.size)
    return out


def gqa_tile(x, kv_heads, ratio, hd):
    x = _f32(x)
    S = x.shape[-1]
    out = np.empty((kv_heads * ratio * hd, S), np.float32)
    lib.orc_gqa_tile(out, x, kv_heads, ratio, hd, S)
    return out


def gqa_reduce(x, kv_heads, ratio, hd):
    x = _f32(x)
    S = x.shape[-1]
    out = np.empty((kv_heads * hd, S), np.float32)
    lib.orc_gqa_reduce(out, x, kv_heads, ratio, hd, S)
    return out


def adam_update(w, g, m, v, t, lr, b1, b2, eps, wd=0.0):
    w = _f32(w).copy(); m = _f32(m).copy(); v = _f32(v).copy(); g = _f32(g)
    lib.orc_adam_update(w.reshape(-1), g.reshape(-1), m.reshape(-1), v.reshape(-1), w.size, t, lr, b1, b2, eps, wd)
    return w, m, v


def recipe_drand48(recipe, seed, n, d):
    x = np.zeros(n, np.float32); dy = np.zeros(n, np.float32); w = np.zeros(max(d, 1), np.float32)
    lib.orc_recipe_drand48(recipe, seed, x, dy, w, n, d)
    return x, dy, w


def sumsq_scaled(g, pre_scale=1.0):
    g = _f32(g)
    return float(lib.orc_sumsq_scaled(g.reshape(-1), g.size, pre_scale))


def clip_scale(sumsq, grad_clip):
    return float(lib.orc_clip_scale(sumsq, grad_clip))


def vocab_map_build(data, full_vocab):
    """Returns (full_to_compact [V], compact_to_full [CV])."""
    data = np.ascontiguousarray(data, np.uint16)
    f2c = np.empty(full_vocab, np.int32); c2f = np.empty(full_vocab, np.int32)
    cv = lib.orc_vocab_map_build(f2c, c2f, data, data.size, full_vocab)
    return f2c, c2f[:cv].copy()


def vocab_compact_embed(full, c2f):
    full = _f32(full); c2f = _i32(c2f)
    ce = np.empty((c2f.size, full.shape[1]), np.float32)
    lib.orc_vocab_compact_embed(ce, full, c2f, c2f.size, full.shape[1])
    return ce


def vocab_scatter_grads(full_g, compact_g, c2f):
    out = _f32(full_g).copy(); c2f = _i32(c2f)
    lib.orc_vocab_scatter_grads(out, _f32(compact_g), c2f, c2f.size, out.shape[1])
    return out


def vocab_update_full(full, compact, c2f):
    out = _f32(full).copy(); c2f = _i32(c2f)
    lib.orc_vocab_update_full(out, _f32(compact), c2f, c2f.size, out.shape[1])
    return out
