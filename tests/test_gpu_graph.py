"""Recorded graphs of the device-resident ops: every replay must equal the same ops run eagerly, with the
program's own eager work and waits between replays."""
import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu

C_, S, B, HID, HEADS, KVH, HD, V = 256, 64, 2, 512, 4, 2, 32, 1031
VE = 5                     # embedding rows: few, so that the scatter-add has long segments too
ALPHA = np.float32(24 ** 0.25)


def make(br):
    """One set of operands for the sequence below; identical for every call."""
    f = lambda seed, *shape: br.DevArray.from_numpy(H.normal(seed, shape))
    w = lambda seed, n: br.DevArray.from_numpy(H.normal(seed, n, 1.0, 0.02))
    z = lambda *shape: br.DevArray(shape)
    d = dict(x=f(1, B, C_, S), o=f(2, B, C_, S), w1=w(3, C_), w2=w(4, C_), xn=z(B, C_, S), x2=z(B, C_, S), x2n=z(B, C_, S),
             q=f(5, B, HEADS * HD, S), k=f(6, B, KVH * HD, S), wq=w(7, HD), wk=w(8, HD), qr=z(B, HEADS * HD, S),
             kr=z(B, KVH * HD, S), h1=f(9, B, HID, S), h3=f(10, B, HID, S), act=z(B, HID, S), ds=f(11, B, HID, S),
             dh1=z(B, HID, S), dh3=z(B, HID, S), dy=f(12, B, C_, S), dx=z(B, C_, S), dw2=f(13, C_),
             gq=f(14, B, HEADS * HD, S), gk=f(15, B, KVH * HD, S), dq=z(B, HEADS * HD, S), dk=z(B, KVH * HD, S),
             dwq=f(16, HD), dwk=f(17, HD), logits=br.DevArray.from_numpy(H.normal(18, (V, S), 0, 2.0)),
             tgt=br.DevArray.from_numpy(np.random.default_rng(19).integers(0, V, S).astype(np.int32)),
             dl=z(V, S), loss=z(1), scale=z(1), q8=br.DevArray(B * C_ * S, np.int8), deq=z(B, C_, S),
             h16=br.DevArray((B, HEADS * HD, S), np.uint16), fq=z(B, HEADS * HD, S), fk=z(B, KVH * HD, S),
             fv=z(B, KVH * HD, S), ssq=z(1), clip=z(1), m=z(C_), v=z(C_), scratch=f(20, 4096),
             E=f(21, VE, C_), ids=br.DevArray.from_numpy(H.zipf_ids(22, B * S, VE).reshape(B, S)), emb=z(B, C_, S),
             dE=f(23, VE, C_))
    return d


def run(br, d, cos, sin):
    """A layer's worth of ops: forward, backward with accumulating weight gradients, loss, INT8, staging, optimizer."""
    L, ck = br.lib, br.check
    n_c, n_h = B * C_ * S, B * HID * S
    ck(L.mi355_embed_gather_dev(d["emb"].ptr, d["E"].ptr, d["ids"].ptr, VE, C_, S, B))
    ck(L.mi355_embed_scatter_add_dev(d["dE"].ptr, d["dy"].ptr, d["ids"].ptr, VE, C_, S, B))    # accumulates per run
    ck(L.mi355_rmsnorm_fwd_dev(d["xn"].ptr, d["x"].ptr, d["w1"].ptr, C_, S, B, 1e-5))
    ck(L.mi355_qknorm_rope_fwd_dev(d["qr"].ptr, d["kr"].ptr, d["q"].ptr, d["k"].ptr, d["wq"].ptr, d["wk"].ptr, HEADS, KVH, HD,
                                   S, B, cos, sin, 1e-5))
    ck(L.mi355_axpby_dev(d["x2"].ptr, d["x"].ptr, d["o"].ptr, ALPHA, n_c, 0))
    ck(L.mi355_residual_rmsnorm_fwd_dev(d["x2"].ptr, d["x2n"].ptr, d["x"].ptr, d["o"].ptr, ALPHA, d["w2"].ptr, C_, S, B, 1e-5))
    ck(L.mi355_swiglu_fwd_dev(d["act"].ptr, d["h1"].ptr, d["h3"].ptr, n_h))
    ck(L.mi355_swiglu_bwd_dev(d["dh1"].ptr, d["dh3"].ptr, d["ds"].ptr, d["h1"].ptr, d["h3"].ptr, n_h))
    ck(L.mi355_rmsnorm_bwd_dev(d["dx"].ptr, d["dw2"].ptr, d["dy"].ptr, d["x2"].ptr, d["w2"].ptr, C_, S, B, 1e-5, 0))
    ck(L.mi355_rmsnorm_bwd_residual_dev(d["xn"].ptr, d["deq"].ptr, d["dw2"].ptr, d["dy"].ptr, d["x2"].ptr, d["w2"].ptr,
                                        d["o"].ptr, ALPHA, C_, S, B, 1e-5, 0))
    ck(L.mi355_qknorm_rope_bwd_dev(d["dq"].ptr, d["dk"].ptr, d["dwq"].ptr, d["dwk"].ptr, d["gq"].ptr, d["gk"].ptr, d["q"].ptr,
                                   d["k"].ptr, d["wq"].ptr, d["wk"].ptr, HEADS, KVH, HD, S, B, cos, sin, 1e-5, 0))
    ck(L.mi355_softmax_ce_dev(d["dl"].ptr, d["loss"].ptr, d["logits"].ptr, d["tgt"].ptr, V, S, 256.0))
    ck(L.mi355_int8_scale_dev(d["scale"].ptr, d["xn"].ptr, n_c))
    ck(L.mi355_int8_quant_dev(d["q8"].ptr, d["xn"].ptr, d["scale"].ptr, n_c, 0))
    ck(L.mi355_int8_dequant_dev(d["deq"].ptr, d["q8"].ptr, d["scale"].ptr, n_c))
    nq = B * HEADS * HD * S
    ck(L.mi355_cvt_f32_f16_dev(d["h16"].ptr, nq, d["gq"].ptr, nq, 1, nq))
    ck(L.mi355_attn_grads_finish_dev(d["fq"].ptr, d["fk"].ptr, d["fv"].ptr, d["h16"].ptr, d["h16"].ptr, d["h16"].ptr, 1, 0, 0, 0,
                                     HEADS, KVH, HD, S, B, cos, sin))
    ck(L.mi355_buf_zero(d["ssq"].handle))
    ck(L.mi355_dw_flush())                                   # the norm below reads dw2
    ck(L.mi355_sumsq_accum_dev(d["ssq"].ptr, d["dw2"].ptr, C_, 1.0))
    ck(L.mi355_clip_scale_dev(d["clip"].ptr, d["ssq"].ptr, 1e-3))
    ck(L.mi355_adam_update_dev(d["w2"].ptr, d["dw2"].ptr, d["m"].ptr, d["v"].ptr, C_, 3, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1.0,
                               d["clip"].ptr, 0))


def snapshot(d):
    return {k: a.numpy().tobytes() for k, a in d.items()}


@pytest.mark.parametrize("defer", [0, 1])
def test_graph_replays_equal_eager_runs(br, defer):
    L = br.lib
    cos, sin = br.rope_tables_dev(S, HD, 1e4)
    br.check(L.mi355_dw_defer(defer))
    try:
        warm, eager, rec = make(br), make(br), make(br)
        run(br, warm, cos, sin)                               # sizes every workspace
        br.sync()
        before = snapshot(rec)
        br.check(L.mi355_graph_begin())
        run(br, rec, cos, sin)
        assert L.mi355_sync() == -1 and L.mi355_buf_alloc(64) is None     # refused, and the recording goes on
        g = L.mi355_graph_end()
        assert g, br.last_error()
        assert snapshot(rec) == before                        # recording ran nothing
        other = br.DevArray.from_numpy(H.normal(30, (2, 2 * 4 * 8, 16)))
        tiled = br.DevArray((2, 2 * 2 * 4 * 8, 16))
        for rep in range(3):
            run(br, eager, cos, sin)
            br.check(L.mi355_graph_launch(g))
            want, got = snapshot(eager), snapshot(rec)        # reads wait for the stream
            bad = [k for k in want if want[k] != got[k]]
            assert not bad, (rep, bad)
            # the program's own eager work and a wait between replays
            br.check(L.mi355_gqa_tile_dev(tiled.ptr, other.ptr, 2 * 4, 2, 8, 16, 2))
            br.check(L.mi355_axpby_dev(rec["scratch"].ptr, rec["scratch"].ptr, None, 1.5, 4096, 1))
            br.check(L.mi355_axpby_dev(eager["scratch"].ptr, eager["scratch"].ptr, None, 1.5, 4096, 1))
            br.sync()
        # a workspace reallocated after the recording invalidates it
        br.check(L.mi355_workspace_reserve(L.mi355_workspace_size() + (1 << 20)))
        assert L.mi355_graph_launch(g) == -1 and "record it again" in br.last_error()
        L.mi355_graph_free(g)
    finally:
        L.mi355_dw_defer(0)


def test_graph_capture_refuses_ops_that_allocate(br):
    L = br.lib
    dE = br.DevArray((50, 16)); dx = br.DevArray.from_numpy(H.normal(40, (1, 16, 8)))
    ids = br.DevArray.from_numpy(np.arange(8, dtype=np.int32))
    br.check(L.mi355_embed_scatter_add_dev(dE.ptr, dx.ptr, ids.ptr, 1 << 20, 16, 8, 1))   # sizes the workspace
    br.sync()
    a = br.DevArray(64)
    br.check(L.mi355_graph_begin())
    assert L.mi355_graph_begin() == -1
    assert L.mi355_embed_scatter_add_dev(dE.ptr, dx.ptr, ids.ptr, 1 << 20, 16, 8, 1) == -1    # library-sort path
    assert L.mi355_sgemm_dev(0, 0, 4, 4, 4, 1.0, a.ptr, 4, a.ptr, 4, 0.0, a.ptr, 4) == -1
    assert L.mi355_exchange_stats(None, None) == -1                     # it waits for the stream and copies to the host
    assert "captured" in br.last_error()
    br.check(L.mi355_axpby_dev(a.ptr, a.ptr, None, 2.0, 64, 1))
    g = L.mi355_graph_end()
    assert g
    assert L.mi355_graph_end() is None                        # no capture open any more
    br.check(L.mi355_graph_launch(g))
    br.sync()
    L.mi355_graph_free(g)
    L.mi355_graph_free(None)


def test_graph_records_a_scatter_add_beyond_16384_positions(br):
    """Eagerly such an input takes the library sort, which cannot be recorded; during a capture the entry point takes
    the form with the columns of dE owned by workgroups instead: same bits, replayed three times."""
    L = br.lib
    V, D, B, S = 3000, 24, 80, 256                            # 20480 positions
    ids = H.zipf_ids(5, B * S, V).astype(np.int32).reshape(B, S)
    dx = H.normal(41, (B, D, S)); dE0 = H.normal(42, (V, D))
    idd, dxd = br.DevArray.from_numpy(ids), br.DevArray.from_numpy(dx)
    eager = br.DevArray.from_numpy(dE0)
    br.check(L.mi355_embed_scatter_add_dev(eager.ptr, dxd.ptr, idd.ptr, V, D, S, B))     # also sizes the workspace
    br.sync()
    assert eager.numpy().tobytes() == O.embed_backward(dE0, dx, ids).tobytes()
    rec = br.DevArray.from_numpy(dE0)
    br.check(L.mi355_graph_begin())
    br.check(L.mi355_embed_scatter_add_dev(rec.ptr, dxd.ptr, idd.ptr, V, D, S, B))
    g = L.mi355_graph_end()
    assert g
    try:
        want = dE0
        for rep in range(3):
            br.check(L.mi355_graph_launch(g))
            want = O.embed_backward(want, dx, ids)
            assert rec.numpy().tobytes() == want.tobytes(), rep
            br.check(L.mi355_axpby_dev(eager.ptr, eager.ptr, None, 1.0, 64, 1))          # eager work between replays
            br.sync()
    finally:
        L.mi355_graph_free(g)


def test_graph_replays_the_one_launch_cross_entropy(br):
    """The cross-entropy kernel whose workgroups exchange partials inside the launch, recorded without a warm-up
    call (it allocates nothing: its slots and launch counters live in a device array of the library that is
    never cleared) and replayed between eager runs of the same op on other shapes: same bits every time."""
    L = br.lib
    V, S = 4608, 128
    logits = br.DevArray.from_numpy(H.normal(50, (V, S), 0, 2.0))
    tgt = br.DevArray.from_numpy(np.random.default_rng(51).integers(0, V, S).astype(np.int32))
    dl_g, loss_g = br.DevArray((V, S)), br.DevArray(1)
    dl_n, loss_n = br.DevArray((V, S)), br.DevArray(1)
    ws_before = L.mi355_workspace_size()
    br.check(L.mi355_graph_begin())
    br.check(L.mi355_softmax_ce_dev(dl_g.ptr, loss_g.ptr, logits.ptr, tgt.ptr, V, S, 2.0))
    br.check(L.mi355_softmax_ce_noalloc_dev(dl_n.ptr, loss_n.ptr, logits.ptr, tgt.ptr, V, S, 2.0))
    g = L.mi355_graph_end()
    assert g, br.last_error()
    assert L.mi355_workspace_size() == ws_before
    dl_e, loss_e = br.DevArray((V, S)), br.DevArray(1)
    V2, S2 = 9000, 256                                           # another shape: other workgroup numbers take part
    lg2 = br.DevArray.from_numpy(H.normal(52, (V2, S2), 0, 2.0))
    tg2 = br.DevArray.from_numpy(np.random.default_rng(53).integers(0, V2, S2).astype(np.int32))
    dl2, loss2 = br.DevArray((V2, S2)), br.DevArray(1)
    for rep in range(3):
        br.check(L.mi355_softmax_ce_dev(dl_e.ptr, loss_e.ptr, logits.ptr, tgt.ptr, V, S, 2.0))
        br.check(L.mi355_graph_launch(g))
        want = (dl_e.numpy().tobytes(), loss_e.numpy().tobytes())
        assert (dl_g.numpy().tobytes(), loss_g.numpy().tobytes()) == want, rep
        assert (dl_n.numpy().tobytes(), loss_n.numpy().tobytes()) == want, rep
        br.check(L.mi355_softmax_ce_dev(dl2.ptr, loss2.ptr, lg2.ptr, tg2.ptr, V2, S2, 1.0))
        br.check(L.mi355_buf_zero(dl_g.handle)); br.check(L.mi355_buf_zero(dl_n.handle))
        br.sync()
    rl, rd = O.cross_entropy(logits.numpy(), tgt.numpy(), 2.0)
    assert H.err_std(dl_e.numpy(), rd) <= 1e-5 and abs(float(loss_e.numpy()[0]) - rl) <= 1e-5 * abs(rl)
    L.mi355_graph_free(g)
