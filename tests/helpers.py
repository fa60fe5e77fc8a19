"""Shared helpers of the GPU parity tests."""
import numpy as np

from coalsack_amd import synth


def all_blocks(L, which):
    return np.concatenate([L.blocks(e, which) for e in range(L.E)])


def build_layer(lib, L, bias=True, norm=False, device_weights=False, **opts):
    """Populate a resident layer from LayerInputs; weights either uploaded from
    the host replay of the generator or generated on the device."""
    layer = lib.layer(L.E, L.k, L.H, L.F)
    layer.set_router(L.gate_w, L.gate_b)
    if device_weights:
        layer.fill_synthetic(L.seed, L.layer)
        for e in range(L.E):
            if bias:
                layer.set_expert(e, None, None, None, L.b_up[e], L.b_gate[e], L.b_down[e])
    else:
        for e in range(L.E):
            b = (L.b_up[e], L.b_gate[e], L.b_down[e]) if bias else (None, None, None)
            layer.set_expert(e, L.blocks(e, 0), L.blocks(e, 1), L.blocks(e, 2), *b)
    if norm:
        layer.set_norm(L.norm_w, 1e-5)
    if opts:
        layer.set_options(**opts)
    return layer


def oracle_layer(oracle, L, hidden, bias=True, norm=False, residual=False, max_tokens=-1, **opts):
    return oracle.moe_layer(
        hidden, L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, all_blocks(L, 0), all_blocks(L, 1),
        all_blocks(L, 2), L.b_up if bias else None, L.b_gate if bias else None,
        L.b_down if bias else None, norm_w=L.norm_w if norm else None, norm_eps=1e-5,
        residual=residual, max_tokens=max_tokens, **opts)


def classify_index_mismatches(oracle, hidden, L, got_pairs, want_pairs):
    """Returns (real, near_tie): tokens whose expert indices differ from the
    oracle's, split by whether float64 logits show a rank boundary closer than
    fp32 summation noise (gap < 1e-5 * |logit| + 1e-6)."""
    gi, wi = got_pairs[..., 0].astype(int), want_pairs[..., 0].astype(int)
    bad = np.nonzero(np.any(gi != wi, axis=1))[0]
    if bad.size == 0:
        return 0, 0
    logits = hidden[bad].astype(np.float64) @ L.gate_w.astype(np.float64).T + L.gate_b
    real = near = 0
    k = L.k
    for r in range(bad.size):
        srt = np.sort(logits[r])[::-1][:k + 1]
        gaps = np.abs(np.diff(srt))
        tol = 1e-5 * np.abs(srt[:-1]) + 1e-6
        if np.any(gaps < tol):
            near += 1
        else:
            real += 1
    return real, near


def assert_layer_close(got, want, tol=1e-3):
    """max|d| / max(1e-6, max|want|) <= tol and |d| <= tol * max(1, |want|) per element."""
    d = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(np.isfinite(got))
    assert d.max() / max(1e-6, np.abs(want).max()) <= tol, d.max()
    assert np.all(d <= tol * np.maximum(1.0, np.abs(want))), d.max()
    return d.max()


def nbits_differ(a, b):
    """Number of elements whose fp32 bit patterns differ."""
    a = np.ascontiguousarray(a, np.float32).reshape(-1).view(np.uint32)
    b = np.ascontiguousarray(b, np.float32).reshape(-1).view(np.uint32)
    return int(np.count_nonzero(a != b))


# |w_gpu - w_cpu| for a routing weight.  The two sets of logits differ by summation order:
# test_router_logits_distance_from_sequential_sums holds each logit within 3 units of
# 2^-24 sqrt(H) max(1, |logit|) of the reference's sequential sum -- 9.6e-6 max(1, |logit|)
# at H = 2880.  A softmax (or sigmoid) weight moves by at most w (1 - w) <= 1/4 per unit of
# logit difference between two experts, i.e. by up to 1/4 x 2 x 9.6e-6 = 4.8e-6 for logits
# of magnitude <= 1 and proportionally more for larger ones (observed: 5.5e-6 at 257
# tokens).  1e-5 is that bound for the logit magnitudes of these configurations; 1e-6
# would need every logit in the reference's sequential order, which the library computes
# only where a selection depends on it (close calls).
ROUTING_WEIGHT_TOL = 1e-5


def oracle_layer_tokens(oracle, L, hidden, idx, threads=16):
    """Oracle output and router pairs for the tokens hidden[idx] (any index set), replaying on
    the host only the experts those tokens select; the tokens are farmed over threads (the
    checker releases the interpreter lock inside a call and tokens are independent)."""
    import threading
    idx = np.asarray(idx, dtype=np.int64)
    sub = np.ascontiguousarray(hidden[idx])
    pairs = oracle.router(sub, L.gate_w, L.gate_b, L.k)
    used = sorted(set(pairs[..., 0].astype(int).ravel().tolist()))
    per_gu, per_d = L.F * (L.H // 32) * 17, L.H * (L.F // 32) * 17
    wu = np.zeros(L.E * per_gu, np.uint8)
    wg = np.zeros(L.E * per_gu, np.uint8)
    wd = np.zeros(L.E * per_d, np.uint8)
    for e in used:
        wu[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 0)
        wg[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 1)
        wd[e * per_d:(e + 1) * per_d] = L.blocks(e, 2)
    out = np.zeros((idx.size, L.H), np.float32)
    opairs = np.zeros((idx.size, L.k, 2), np.float32)
    chunks = [c for c in np.array_split(np.arange(idx.size), max(1, min(threads, idx.size))) if c.size]

    def work(c):
        o, p = oracle.moe_layer(np.ascontiguousarray(sub[c]), L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, wu, wg, wd,
                                L.b_up, L.b_gate, L.b_down)
        out[c], opairs[c] = o, p
    ts = [threading.Thread(target=work, args=(c,)) for c in chunks]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    return out, opairs


def oracle_layer_subset(oracle, L, hidden, ntok, norm=False, residual=False, **opts):
    """Oracle output for the first ntok tokens, replaying on the host only the
    experts those tokens select (the others stay zero and are never read)."""
    xin = oracle.rmsnorm(hidden[:ntok], L.norm_w, 1e-5) if norm else hidden[:ntok]
    pairs = oracle.router(xin, L.gate_w, L.gate_b, L.k, opts.get("sigmoid", False))
    used = sorted(set(pairs[..., 0].astype(int).ravel().tolist()))
    per_gu, per_d = L.F * (L.H // 32) * 17, L.H * (L.F // 32) * 17
    wu = np.zeros(L.E * per_gu, np.uint8)
    wg = np.zeros(L.E * per_gu, np.uint8)
    wd = np.zeros(L.E * per_d, np.uint8)
    for e in used:
        wu[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 0)
        wg[e * per_gu:(e + 1) * per_gu] = L.blocks(e, 1)
        wd[e * per_d:(e + 1) * per_d] = L.blocks(e, 2)
    return oracle.moe_layer(hidden[:ntok], L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, wu, wg, wd,
                            L.b_up, L.b_gate, L.b_down, norm_w=L.norm_w if norm else None,
                            norm_eps=1e-5, residual=residual, **opts)
