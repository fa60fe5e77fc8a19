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
