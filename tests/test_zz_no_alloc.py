"""The allocation-free forward (csk_moe_forward_noalloc) against csk_moe_forward: same
kernels out of a workspace that is part of the library image, so the outputs must be
equal bit for bit -- on two calls in a row, the second with a smaller batch (the shared
array still holds the first call's lists, rows and descriptors)."""
import numpy as np
import pytest

from coalsack_amd import capi, synth
from tests.helpers import build_layer

pytestmark = pytest.mark.gpu


def _both(lib, layer, hidden, flags):
    T, H = hidden.shape
    d_in, d_a, d_b = lib.to_device(hidden), lib.dev_alloc(hidden.nbytes), lib.dev_alloc(hidden.nbytes)
    try:
        layer.forward_device(d_in, T, d_a, flags)
        want = lib.to_host(d_a, (T, H))
        counts_w, toks_w = layer.last_dispatch(T)
        layer.forward_device_noalloc(d_in, T, d_b, flags)
        got = lib.to_host(d_b, (T, H))
        counts_g, toks_g = layer.last_dispatch(T)
    finally:
        for d in (d_in, d_a, d_b):
            lib.dev_free(d)
    assert np.all(np.isfinite(want))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(counts_g, counts_w) and np.array_equal(toks_g, toks_w)
    return got


@pytest.mark.parametrize("opts", [dict(), dict(weight_before_ffn=True), dict(norm=True)])
def test_noalloc_forward_equals_forward_twice(lib, opts):
    opts = dict(opts)
    norm = opts.pop("norm", False)
    flags = (capi.FWD_RMSNORM | capi.FWD_RESIDUAL) if norm else 0
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=811, with_norm=True)
    with build_layer(lib, L, norm=True, device_weights=True, **opts) as layer:
        _both(lib, layer, synth.hidden_states(64, L.H, seed=5), flags)   # fills the shared array
        _both(lib, layer, synth.hidden_states(3, L.H, seed=6), flags)    # smaller batch over its leftovers
        _both(lib, layer, synth.hidden_states(16, L.H, seed=7), flags)


def test_noalloc_forward_allocates_nothing(lib):
    """The property the entry point exists for: across calls of it the library makes no
    device allocation (every allocation of the library is counted) and the runtime reports
    the same free device memory -- also on the first call at a new batch size, where
    csk_moe_forward grows its workspace."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=812, with_norm=True)
    with build_layer(lib, L, norm=True, device_weights=True) as layer:
        hs = {T: synth.hidden_states(T, L.H, seed=T) for T in (1, 7, 64, 33)}
        d_in = {T: lib.to_device(h) for T, h in hs.items()}
        d_out = lib.dev_alloc(hs[64].nbytes)
        try:
            lib.synchronize()
            n0, (free0, _) = lib.alloc_count(), lib.device_memory()
            for T in (1, 7, 64, 33, 1):
                for flags in (0, capi.FWD_RMSNORM | capi.FWD_RESIDUAL):
                    layer.forward_device_noalloc(d_in[T], T, d_out, flags)
            lib.synchronize()
            assert lib.alloc_count() == n0
            assert lib.device_memory()[0] == free0
            # the counter is alive: an allocation made through the library moves it
            extra = lib.dev_alloc(4096)
            assert lib.alloc_count() == n0 + 1
            lib.dev_free(extra)
        finally:
            for d in d_in.values():
                lib.dev_free(d)
            lib.dev_free(d_out)


def test_last_dispatch_is_per_layer(lib):
    """A layer's dispatch lists are gone once another forward has used the workspace: asking
    for them then is an error, not another layer's lists."""
    La, Lb = synth.LayerInputs(8, 2, 128, 160, seed=1), synth.LayerInputs(8, 2, 128, 160, seed=2)
    with build_layer(lib, La) as a, build_layer(lib, Lb) as b:
        ha, hb = synth.hidden_states(5, La.H, seed=1), synth.hidden_states(9, Lb.H, seed=2)
        a.forward(ha)
        ca, _ = a.last_dispatch(5)
        assert ca.sum() == 5 * La.k
        b.forward(hb)
        with pytest.raises(capi.CskError, match="another forward has run") as ei:
            a.last_dispatch(5)
        assert ei.value.code == capi.ERR_STATE
        cb, _ = b.last_dispatch(9)
        assert cb.sum() == 9 * Lb.k
        d_in, d_out = lib.to_device(ha), lib.dev_alloc(ha.nbytes)
        try:
            a.forward_device_noalloc(d_in, 5, d_out, 0)  # the fixed workspace: b's lists stay valid
            assert np.array_equal(a.last_dispatch(5)[0], ca)
            assert np.array_equal(b.last_dispatch(9)[0], cb)
        finally:
            lib.dev_free(d_in)
            lib.dev_free(d_out)


def test_noalloc_forward_small_shape_then_limits(lib):
    L = synth.LayerInputs(8, 2, 128, 160, seed=9)
    with build_layer(lib, L) as layer:
        _both(lib, layer, synth.hidden_states(21, L.H, seed=1), 0)
        _both(lib, layer, synth.hidden_states(1, L.H, seed=2), 0)
        d = lib.dev_alloc(65 * L.H * 4)
        try:
            with pytest.raises(capi.CskError, match="at most 64 tokens") as ei:
                layer.forward_device_noalloc(d, 65, d)
            assert ei.value.code == capi.ERR_ARG
        finally:
            lib.dev_free(d)
    L = synth.LayerInputs(4, 2, 3200, 64, seed=23)   # rows longer than the fixed workspace holds
    with build_layer(lib, L) as layer:
        d = lib.dev_alloc(2 * L.H * 4)
        try:
            with pytest.raises(capi.CskError, match="up to 3072"):
                layer.forward_device_noalloc(d, 2, d)
        finally:
            lib.dev_free(d)
    L = synth.LayerInputs(32, 16, 64, 96, seed=3)    # 64 tokens x top-16 = 1024 assignments
    with build_layer(lib, L) as layer:
        d = lib.dev_alloc(64 * L.H * 4)
        try:
            with pytest.raises(capi.CskError, match="512 token-expert assignments"):
                layer.forward_device_noalloc(d, 64, d)
            _both(lib, layer, synth.hidden_states(32, L.H, seed=4), 0)  # 512 assignments: the limit itself
        finally:
            lib.dev_free(d)
