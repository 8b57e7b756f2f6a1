"""mi355_softmax_ce_noalloc_dev, the entry point that allocates nothing (its scratch is a fixed device array of the
library), against mi355_softmax_ce_dev: same bits out, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest

import helpers as H
import oracle as O

pytestmark = pytest.mark.gpu


def _both(br, V, S, seed, grad_scale):
    logits = H.normal(seed, (V, S), 0, 2.0)
    tgt = np.random.default_rng(seed + 1).integers(0, V, S).astype(np.int32)
    if S > 8:
        tgt[2] = V; tgt[5] = -1                       # out-of-range targets are skipped in both
    ld, td = br.DevArray.from_numpy(logits), br.DevArray.from_numpy(tgt)
    d_ref, l_ref = br.DevArray(logits.shape), br.DevArray(1)
    br.check(br.lib.mi355_softmax_ce_dev(d_ref.ptr, l_ref.ptr, ld.ptr, td.ptr, V, S, grad_scale))
    want_d, want_l = d_ref.numpy(), l_ref.numpy()
    d_new, l_new = br.DevArray(logits.shape), br.DevArray(1)
    d_new.upload(np.full(logits.shape, 9.0, np.float32))
    ws_before = br.lib.mi355_workspace_size()
    br.check(br.lib.mi355_softmax_ce_noalloc_dev(d_new.ptr, l_new.ptr, ld.ptr, td.ptr, V, S, grad_scale))
    assert br.lib.mi355_workspace_size() == ws_before
    got_d, got_l = d_new.numpy(), l_new.numpy()
    assert got_d.tobytes() == want_d.tobytes() and got_l.tobytes() == want_l.tobytes(), (V, S)
    rl, rd = O.cross_entropy(logits, tgt, grad_scale)
    assert abs(float(got_l[0]) - rl) <= 1e-5 * abs(rl) and H.err_std(got_d, rd) <= 1e-5
    return ld, td


def test_softmax_ce_without_allocation_matches_the_allocating_entry_point(br):
    print("[case] softmax_ce_noalloc V=151936 S=256, then V=4099 S=64, then V=37 S=12", flush=True)
    _both(br, 151936, 256, 300, 1.0)                  # BASELINE config 4's classifier shape
    _both(br, 4099, 64, 302, 256.0)                   # a smaller input right behind it: the scratch keeps old contents
    _both(br, 37, 12, 304, 1.0)                       # scalar columns
    ld, td = _both(br, 32000, 256, 306, 1.0)
    # in place, as the allocating entry point allows (both then take the three-launch form)
    ref = br.DevArray.from_numpy(ld.numpy()); lref = br.DevArray(1); lnew = br.DevArray(1)
    br.check(br.lib.mi355_softmax_ce_dev(ref.ptr, lref.ptr, ref.ptr, td.ptr, 32000, 256, 1.0))
    br.check(br.lib.mi355_softmax_ce_noalloc_dev(ld.ptr, lnew.ptr, ld.ptr, td.ptr, 32000, 256, 1.0))
    assert ld.numpy().tobytes() == ref.numpy().tobytes() and lnew.numpy().tobytes() == lref.numpy().tobytes()


def test_softmax_ce_without_allocation_rejects_what_does_not_fit(br):
    # S = 4096 columns x 64 row blocks of partials is beyond the fixed 2 MiB: a clear error, nothing launched
    V, S = 4096, 4096
    big = br.DevArray((V, S)); out = br.DevArray((V, S)); loss = br.DevArray(1)
    tgt = br.DevArray.from_numpy(np.zeros(S, np.int32))
    out.upload(np.full((V, S), 3.0, np.float32))
    assert br.lib.mi355_softmax_ce_noalloc_dev(out.ptr, loss.ptr, big.ptr, tgt.ptr, V, S, 1.0) == -1
    assert "scratch" in br.last_error()
    assert np.all(out.numpy() == 3.0)
    assert br.lib.mi355_softmax_ce_dev(out.ptr, loss.ptr, big.ptr, tgt.ptr, V, S, 1.0) == 0      # the growing one takes it
