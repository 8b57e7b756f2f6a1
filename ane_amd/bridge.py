"""ctypes binding of ``libmi355_ops.so`` — the C-ABI declared in ``include/mi355_bridge.h``.

There is no CPU fallback: if the library is missing, importing this module raises, and if no
gfx950 device is present every op returns -1 / raises ``BridgeError``.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355_ops.so")


class BridgeError(RuntimeError):
    pass


if not os.path.exists(LIB_PATH):
    raise ImportError(
        "%s not found: build it with `python -m ane_amd.build` (needs hipcc); there is no CPU fallback" % LIB_PATH)

lib = C.CDLL(LIB_PATH)

_p = C.c_void_p
_i = C.c_int
_f = C.c_float
_z = C.c_size_t
_u64 = C.c_uint64
_s = C.c_char_p


class CkptHdr(C.Structure):
    """The 96-byte checkpoint header (``mi355_ckpt_hdr``)."""
    _fields_ = ([(n, C.c_int) for n in ("magic", "version", "step", "total_steps", "n_layers", "vocab_size", "dim",
                                         "hidden_dim", "n_heads", "seq_len")] +
                [("lr", C.c_float), ("loss", C.c_float)] +
                [(n, C.c_double) for n in ("cum_compile", "cum_train", "cum_wall")] +
                [(n, C.c_int) for n in ("cum_steps", "cum_batches", "adam_t", "kv_heads", "head_dim", "q_dim")])


CK_TENSORS = ("WQ", "WK", "WV", "WO", "W1", "W2", "W3", "RMS_ATT", "RMS_FFN", "RMS_FINAL", "EMBED")

# name -> (restype, argtypes); every symbol include/mi355_bridge.h declares
SIGNATURES = {
    "mi355_init": (_i, []),
    "mi355_shutdown": (None, []),
    "mi355_last_error": (C.c_char_p, []),
    "mi355_device_info": (_i, [C.c_char_p, _z, C.POINTER(C.c_double), C.POINTER(_i)]),
    "mi355_set_stream": (_i, [_p]),
    "mi355_sync": (_i, []),
    "mi355_workspace_reserve": (_i, [_z]),
    "mi355_tune_set": (_i, [C.c_char_p, _i]),
    "mi355_exchange_stats": (_i, [C.POINTER(C.c_longlong), C.POINTER(C.c_longlong)]),
    "mi355_buf_alloc": (_p, [_z]),
    "mi355_buf_free": (None, [_p]),
    "mi355_buf_devptr": (_p, [_p]),
    "mi355_buf_bytes": (_z, [_p]),
    "mi355_buf_write": (None, [_p, _z, _p, _z]),
    "mi355_buf_read": (None, [_p, _z, _p, _z]),
    "mi355_buf_zero": (_i, [_p]),
    "mi355_event_create": (_p, []),
    "mi355_event_destroy": (None, [_p]),
    "mi355_event_record": (_i, [_p]),
    "mi355_event_elapsed_ms": (_f, [_p, _p]),
    "mi355_fill_normal_dev": (_i, [_p, _z, C.c_uint64, _f, _f]),
    "mi355_fill_randint_dev": (_i, [_p, _z, C.c_uint64, C.c_int32, C.c_int32]),
    "mi355_rmsnorm_fwd_dev": (_i, [_p, _p, _p, _i, _i, _i, _f]),
    "mi355_rmsnorm_bwd_dev": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _f, _i]),
    "mi355_dw_defer": (_i, [_i]),
    "mi355_dw_flush": (_i, []),
    "mi355_rmsnorm_bwd_residual_dev": (_i, [_p, _p, _p, _p, _p, _p, _p, _f, _i, _i, _i, _f, _i]),
    "mi355_residual_rmsnorm_fwd_dev": (_i, [_p, _p, _p, _p, _f, _p, _i, _i, _i, _f]),
    "mi355_swiglu_fwd_dev": (_i, [_p, _p, _p, _z]),
    "mi355_swiglu_bwd_dev": (_i, [_p, _p, _p, _p, _p, _z]),
    "mi355_rope_tables": (_i, [_p, _p, _i, _i, _f]),
    "mi355_rope_tables_dev": (_i, [C.POINTER(_p), C.POINTER(_p), _i, _i, _f]),
    "mi355_rope_dev": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i]),
    "mi355_qknorm_rope_fwd_dev": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _f]),
    "mi355_qknorm_rope_bwd_dev": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _f, _i]),
    "mi355_axpby_dev": (_i, [_p, _p, _p, _f, _z, _i]),
    "mi355_embed_gather_dev": (_i, [_p, _p, _p, _i, _i, _i, _i]),
    "mi355_embed_scatter_add_dev": (_i, [_p, _p, _p, _i, _i, _i, _i]),
    "mi355_embed_scatter_add_form": (_i, [_i, _i, _i, _i, _i]),
    "mi355_softmax_ce_dev": (_i, [_p, _p, _p, _p, _i, _i, _f]),
    "mi355_minmax_dev": (_i, [_p, _p, _z]),
    "mi355_int8_scale_dev": (_i, [_p, _p, _z]),
    "mi355_int8_quantize_dynamic_dev": (_i, [_p, _p, _p, _z, _i]),
    "mi355_int8_quant_dev": (_i, [_p, _p, _p, _z, _i]),
    "mi355_int8_dequant_dev": (_i, [_p, _p, _p, _z]),
    "mi355_sumsq_accum_dev": (_i, [_p, _p, _z, _f]),
    "mi355_clip_scale_dev": (_i, [_p, _p, _f]),
    "mi355_adam_update_dev": (_i, [_p, _p, _p, _p, _z, _i, _f, _f, _f, _f, _f, _f, _p, _i]),
    "mi355_sumsq_accum_multi_dev": (_i, [_p, _p, _p, _i, _f]),
    "mi355_adam_update_multi_dev": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _f, _f, _f, _f, _f, _p, _i]),
    "mi355_rmsnorm_tile": (_i, [_i, _i, _i, _i, _i, _p]),
    "mi355_softmax_ce_noalloc_dev": (_i, [_p, _p, _p, _p, _i, _i, _f]),
    "mi355_softmax_cols_dev": (_i, [_p, _p, _i, _i]),
    "mi355_nll_from_probs_dev": (_i, [_p, _p, _p, _p, _i, _i]),
    "mi355_vocab_map_build_dev": (_i, [_p, _p, _p, _p, _z, _i]),
    "mi355_vocab_remap_dev": (_i, [_p, _p, _p, _z, _i]),
    "mi355_vocab_compact_embed_dev": (_i, [_p, _p, _p, _i, _i, _i]),
    "mi355_vocab_update_full_dev": (_i, [_p, _p, _p, _i, _i, _i]),
    "mi355_vocab_scatter_grads_dev": (_i, [_p, _p, _p, _i, _i, _i]),
    "mi355_gqa_tile_dev": (_i, [_p, _p, _i, _i, _i, _i, _i]),
    "mi355_gqa_reduce_dev": (_i, [_p, _p, _i, _i, _i, _i, _i]),
    "mi355_ckpt_read_header": (_i, [_s, C.POINTER(CkptHdr)]),
    "mi355_ckpt_locate": (_i, [C.POINTER(CkptHdr), _i, _i, _i, C.POINTER(_u64), C.POINTER(_u64)]),
    "mi355_ckpt_file_bytes": (_u64, [C.POINTER(CkptHdr)]),
    "mi355_ckpt_create": (_i, [_s, C.POINTER(CkptHdr)]),
    "mi355_ckpt_load_dev": (_i, [_s, _u64, _p, _u64]),
    "mi355_ckpt_store_dev": (_i, [_s, _u64, _p, _u64]),
    "mi355_cvt_f32_bf16_dev": (_i, [_p, _z, _p, _z, _z, _z]),
    "mi355_cvt_bf16_f32_dev": (_i, [_p, _z, _p, _z, _z, _z]),
    "mi355_rmsnorm_fwd_bf16_dev": (_i, [_p, _p, _p, _i, _i, _i, _f]),
    "mi355_rmsnorm_bwd_bf16_dev": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _f, _i]),
    "mi355_residual_rmsnorm_fwd_bf16_dev": (_i, [_p, _p, _p, _p, _f, _p, _i, _i, _i, _f]),
    "mi355_rmsnorm_bwd_residual_bf16_dev": (_i, [_p, _p, _p, _p, _p, _p, _p, _f, _i, _i, _i, _f, _i]),
    "mi355_swiglu_fwd_bf16_dev": (_i, [_p, _p, _p, _z]),
    "mi355_swiglu_bwd_bf16_dev": (_i, [_p, _p, _p, _p, _p, _z]),
    "mi355_axpby_bf16_dev": (_i, [_p, _p, _p, _f, _z, _i]),
    "mi355_softmax_ce_bf16_dev": (_i, [_p, _p, _p, _p, _i, _i, _f]),
    "mi355_rope_bf16_dev": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i]),
    "mi355_qknorm_rope_fwd_bf16_dev": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _f]),
    "mi355_qknorm_rope_bwd_bf16_dev": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _f, _i]),
    "mi355_workspace_size": (_z, []),
    "mi355_graph_begin": (_i, []),
    "mi355_graph_end": (_p, []),
    "mi355_graph_launch": (_i, [_p]),
    "mi355_graph_free": (None, [_p]),
    "mi355_sgemm_dev": (_i, [_i, _i, _i, _i, _i, _f, _p, _i, _p, _i, _f, _p, _i]),
    "mi355_cvt_f32_f16_dev": (_i, [_p, _z, _p, _z, _z, _z]),
    "mi355_cvt_f16_f32_dev": (_i, [_p, _z, _p, _z, _z, _z]),
    "mi355_attn_grads_finish_dev": (_i, [_p, _p, _p, _p, _p, _p, _i, _z, _z, _z, _i, _i, _i, _i, _i, _p, _p]),
    "mi355_adam_update": (None, [_p, _p, _p, _p, _z, _i, _f, _f, _f, _f, _f]),
    "mi355_vocab_map_build": (_i, [_p, _p, _p, _z, _i]),
    "mi355_vocab_compact_embed": (None, [_p, _p, _p, _i, _i, _i]),
    "mi355_vocab_scatter_grads": (None, [_p, _p, _p, _i, _i, _i]),
    "mi355_vocab_update_full": (None, [_p, _p, _p, _i, _i, _i]),
    "mi355_rmsnorm": (None, [_p, _p, _p, _i, _i]),
    "mi355_rmsnorm_bwd": (None, [_p, _p, _p, _p, _p, _i, _i]),
    "mi355_cross_entropy_loss": (_f, [_p, _p, _p, _i, _i]),
    "mi355_embed_lookup": (None, [_p, _p, _p, _i, _i, _i]),
    "mi355_host_table_invalidate": (None, [_p]),
    "mi355_embed_backward": (None, [_p, _p, _p, _i, _i, _i]),
    "mi355_rope_backward_inplace": (None, [_p, _i, _i, _i]),
    "mi355_swiglu_bwd": (None, [_p, _p, _p, _p, _p, _z]),
    "mi355_swiglu_fwd": (None, [_p, _p, _p, _z]),
    "mi355_axpby": (None, [_p, _p, _p, _f, _z, _i]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)          # AttributeError here = the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args


def last_error():
    return lib.mi355_last_error().decode()


def check(rc, what="mi355 call"):
    if rc != 0:
        raise BridgeError("%s failed: %s" % (what, last_error()))


def init():
    check(lib.mi355_init(), "mi355_init")


def sync():
    check(lib.mi355_sync(), "mi355_sync")


def device_info():
    name = C.create_string_buffer(256)
    peak = C.c_double(0)
    cus = C.c_int(0)
    check(lib.mi355_device_info(name, 256, C.byref(peak), C.byref(cus)), "mi355_device_info")
    return name.value.decode(), peak.value, cus.value


def tune(key, value):
    if lib.mi355_tune_set(key.encode(), int(value)) != 0:
        raise BridgeError("unknown tuning knob %r" % key)


def exchange_fallbacks():
    """(shared exchange area, one-launch softmax-CE): workgroups whose bounded wait for a partner expired, ever."""
    a, c = C.c_longlong(0), C.c_longlong(0)
    check(lib.mi355_exchange_stats(C.byref(a), C.byref(c)), "mi355_exchange_stats")
    return a.value, c.value


class DevArray:
    """A device buffer with a numpy-style shape/dtype; thin wrapper over ``mi355_buf``."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__len__") else (shape,)))
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = max(self.size * self.dtype.itemsize, 1)
        self.handle = lib.mi355_buf_alloc(self.nbytes)
        if not self.handle:
            raise BridgeError("mi355_buf_alloc(%d) failed: %s" % (self.nbytes, last_error()))
        self.ptr = lib.mi355_buf_devptr(self.handle)

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        d.upload(a)
        return d

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.size == self.size, (a.shape, self.shape)
        if a.size:
            lib.mi355_buf_write(self.handle, 0, a.ctypes.data, a.nbytes)
        return self

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if out.size:
            lib.mi355_buf_read(self.handle, 0, out.ctypes.data, out.nbytes)
        return out

    def zero(self):
        check(lib.mi355_buf_zero(self.handle), "mi355_buf_zero")
        return self

    def free(self):
        if self.handle:
            lib.mi355_buf_free(self.handle)
            self.handle = None
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Event:
    def __init__(self):
        self.handle = lib.mi355_event_create()
        if not self.handle:
            raise BridgeError("mi355_event_create failed: %s" % last_error())

    def record(self):
        check(lib.mi355_event_record(self.handle), "mi355_event_record")
        return self

    def elapsed_ms(self, stop):
        ms = lib.mi355_event_elapsed_ms(self.handle, stop.handle)
        if ms < 0:
            raise BridgeError("mi355_event_elapsed_ms failed")
        return ms

    def __del__(self):
        try:
            if self.handle:
                lib.mi355_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def rope_tables_dev(S, hd, theta):
    c = _p()
    s = _p()
    check(lib.mi355_rope_tables_dev(C.byref(c), C.byref(s), S, hd, theta), "mi355_rope_tables_dev")
    return c.value, s.value
