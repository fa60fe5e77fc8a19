"""GPU parity: the HIP path through the C ABI against the CPU oracle on the same
seeded inputs.  Bit-exact for bytes / dequantised weights / expert indices
(outside fp32-noise ties), <= 1e-3 for layer outputs."""
import numpy as np
import pytest

from coalsack_amd import capi, synth
from tests.helpers import (ROUTING_WEIGHT_TOL, all_blocks, assert_layer_close, build_layer,
                           classify_index_mismatches, oracle_layer, nbits_differ,
                           oracle_layer_subset, oracle_layer_tokens)

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ codec

def test_dequant_bit_exact_and_roundtrip(lib, oracle):
    rng = np.random.default_rng(0)
    for rows, K in [(16, 32), (37, 96), (64, 2880), (2880, 2880)]:
        blocks = rng.integers(0, 256, (rows * (K // 32), 17), dtype=np.uint8)
        blocks[:, 0] = rng.integers(2, 255, blocks.shape[0])  # every exactly representable scale
        blocks = blocks.reshape(-1)
        h = lib.mxfp4_upload(blocks, rows, K)
        try:
            got = lib.mxfp4_dequant(h, rows, K)
            want = oracle.dequant(blocks, rows * K).reshape(rows, K)
            assert nbits_differ(got, want) == 0, (rows, K)
            assert np.count_nonzero(lib.mxfp4_export(h, rows, K) != blocks) == 0
        finally:
            lib.mxfp4_free(h)


def test_dequant_every_scale_and_code(lib, oracle):
    """Every scale byte the reference decodes to finite values, 0 and 1 (fp32 denormals)
    included, with all 16 codes in both nibble positions: bit-exact against the fixture
    written from the reference's own codec."""
    g = np.load(__file__.replace("test_gpu_parity.py", "golden/mxfp4_codec.npz"))
    blocks = g["blocks"][64:64 + 255]  # scale bytes 0..254
    assert blocks[0, 0] == 0 and blocks[254, 0] == 254
    n = blocks.shape[0]
    h = lib.mxfp4_upload(blocks.reshape(-1), n, 32)
    try:
        got = lib.mxfp4_dequant(h, n, 32)
        want = g["values"].reshape(-1, 32)[64:64 + 255]
        assert nbits_differ(got, want.view(np.float32)) == 0
        assert np.array_equal(lib.mxfp4_export(h, n, 32), blocks.reshape(-1))
    finally:
        lib.mxfp4_free(h)


def test_scale_byte_255_finite_values_exact_larger_codes_refused(lib, oracle):
    """Scale byte 255 is 2^127 on the doubled code table (gguf_dequant.h:419-433): codes 0 and
    +-0.5 decode to 0 and +-2^127, bit for bit as the oracle does; the resident copy keeps
    them as byte 254 with the codes doubled, which is what the export returns.  Any larger
    code overflows fp32 in the reference itself: refused."""
    blk = np.zeros(17, np.uint8)
    blk[0] = 255
    blk[1:] = [0x00, 0x08, 0x80, 0x88, 0x01, 0x10, 0x91, 0x19] * 2
    want = oracle.dequant(blk, 32)
    assert np.all(np.isfinite(want)) and np.abs(want).max() == 2.0 ** 127
    h = lib.mxfp4_upload(blk, 1, 32)
    try:
        got = lib.mxfp4_dequant(h, 1, 32).reshape(-1)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        back = lib.mxfp4_export(h, 1, 32)
        assert back[0] == 254
        assert np.array_equal(back[1:], [0x00, 0x08, 0x80, 0x88, 0x02, 0x20, 0xA2, 0x2A] * 2)
        assert np.array_equal(oracle.dequant(back, 32).view(np.uint32), want.view(np.uint32))
    finally:
        lib.mxfp4_free(h)
    blk[5] = 0x20
    with pytest.raises(capi.CskError, match="overflows fp32") as ei:
        lib.mxfp4_upload(blk, 1, 32)
    assert ei.value.code == capi.ERR_SCALE


@pytest.mark.parametrize("T", [5, 130])
def test_layer_with_zero_and_denormal_scale_blocks(lib, oracle, T):
    """A checkpoint as ggml writes it: all-zero blocks carry scale byte 0; a few non-zero
    blocks with scale bytes 0 and 1 (values below 1e-37) are thrown in.  Both regimes must
    accept the layer and match the CPU path."""
    L = synth.LayerInputs(4, 2, 128, 96, seed=57)
    rng = np.random.default_rng(5)
    W = {}
    for e in range(L.E):
        for which in range(3):
            b = L.blocks(e, which).reshape(-1, 17).copy()
            zero = rng.random(b.shape[0]) < 0.2
            b[zero, 1:] = 0
            b[zero, 0] = 0
            tiny = rng.random(b.shape[0]) < 0.05
            b[tiny, 0] = rng.integers(0, 2, int(tiny.sum()))
            W[(e, which)] = b.reshape(-1)
    hidden = synth.hidden_states(T, L.H, seed=T)
    layer = lib.layer(L.E, L.k, L.H, L.F)
    try:
        layer.set_router(L.gate_w, L.gate_b)
        for e in range(L.E):
            layer.set_expert(e, W[(e, 0)], W[(e, 1)], W[(e, 2)], L.b_up[e], L.b_gate[e], L.b_down[e])
            assert nbits_differ(layer.dequant(e, 2), oracle.dequant(W[(e, 2)], L.H * L.F).reshape(L.H, L.F)) == 0
        got = layer.forward(hidden)
    finally:
        layer.close()
    cat = lambda w: np.concatenate([W[(e, w)] for e in range(L.E)])  # noqa: E731
    want, _ = oracle.moe_layer(hidden, L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, cat(0), cat(1), cat(2),
                               L.b_up, L.b_gate, L.b_down)
    assert_layer_close(got, want)


def test_device_generator_matches_host_replay(lib):
    L = synth.LayerInputs(3, 2, 64, 96, seed=77, layer=5)
    with build_layer(lib, L, device_weights=True) as layer:
        for e in range(3):
            for which in range(3):
                assert np.count_nonzero(layer.export(e, which) != L.blocks(e, which)) == 0, (e, which)


# ----------------------------------------------------------------- router

def test_router_known_answer(lib):
    # test/test_moe_router.cpp:82-138
    H, E, k = 4, 6, 3
    h = np.ones((1, H), np.float32)
    g = np.repeat((np.arange(E, dtype=np.float32) / H)[:, None], H, axis=1)
    out = lib.moe_router(h, g, np.zeros(E, np.float32), k)
    assert out[0, :, 0].astype(int).tolist() == [5, 4, 3]


@pytest.mark.parametrize("T,H,E,k,bias,sigmoid", [
    (2, 4, 8, 2, True, False), (8, 128, 32, 4, True, False), (33, 2880, 128, 4, True, False),
    (5, 96, 7, 3, False, False), (64, 2880, 32, 4, True, True), (700, 256, 200, 8, True, False),
    (100, 96, 40, 3, True, False), (65, 32, 5, 1, False, True), (257, 2880, 128, 4, True, False)])
def test_router_matches_oracle(lib, oracle, T, H, E, k, bias, sigmoid):
    rng = np.random.default_rng(T * 1000 + E)
    h = rng.normal(0, 1, (T, H)).astype(np.float32)
    g = rng.normal(0, 0.05, (E, H)).astype(np.float32)
    b = rng.normal(0, 0.01, E).astype(np.float32) if bias else None
    got = lib.moe_router(h, g, b, k, sigmoid)
    want = oracle.router(h, g, b, k, sigmoid)
    same = np.all(got[..., 0] == want[..., 0], axis=1)

    class _L:  # adapter for classify_index_mismatches
        pass
    L = _L()
    L.k, L.gate_w, L.gate_b = k, g, (b if b is not None else np.zeros(E, np.float32))
    real, near = classify_index_mismatches(oracle, h, L, got, want)
    assert (real, near) == (0, 0)
    # weights inherit the difference between the two fp32 summation orders of the logits
    assert np.max(np.abs(got[same, :, 1] - want[same, :, 1])) <= ROUTING_WEIGHT_TOL
    assert np.all(got[..., 1] > 0) and np.allclose(got[..., 1].sum(axis=1), 1.0, atol=1e-5) or sigmoid


@pytest.mark.parametrize("T,E,k", [(1, 8, 4), (3, 8, 8), (20, 32, 4), (100, 128, 4), (300, 7, 3)])
def test_router_nonfinite_logits_still_select_k_distinct_experts(lib, oracle, T, E, k):
    """Tokens whose logits are NaN, +inf or -inf: the k experts returned are distinct and in
    range (the dispatch relies on it), the weights are NaN where the reference's softmax
    gives NaN (moe_router_node.h:176-200), and the other tokens of the batch are untouched."""
    H = 64
    rng = np.random.default_rng(E * 100 + T)
    h = rng.normal(0, 1, (T, H)).astype(np.float32)
    g = rng.normal(0, 0.05, (E, H)).astype(np.float32)
    g[:, 3] = np.abs(g[:, 3]) + 0.01          # column 3 positive: an infinity there drives every logit to it
    b = rng.normal(0, 0.01, E).astype(np.float32)
    clean = lib.moe_router(h, g, b, k)
    kinds = {0: np.nan, T // 2: np.inf, T - 1: -np.inf}
    for t, v in kinds.items():
        h[t, 3] = v
    got = lib.moe_router(h, g, b, k)
    with np.errstate(all="ignore"):
        want = oracle.router(h, g, b, k)
    for t in range(T):
        ids = got[t, :, 0].astype(int)
        assert len(set(ids.tolist())) == k and ids.min() >= 0 and ids.max() < E, (t, ids)
        if t in kinds:
            assert np.all(np.isnan(want[t, :, 1])), "oracle weights finite?"
            assert np.all(np.isnan(got[t, :, 1])), (t, got[t])
        else:
            assert np.array_equal(got[t], clean[t])


@pytest.mark.parametrize("T,bias", [(1, True), (16, False), (300, True)])
def test_router_with_resident_gate_equals_host_gate(lib, T, bias):
    """csk_moe_router_resident (gate kept in device memory by the caller) is csk_moe_router."""
    rng = np.random.default_rng(T)
    E, H, k = 32, 2880, 4
    h = rng.normal(0, 1, (T, H)).astype(np.float32)
    g = rng.normal(0, 0.02, (E, H)).astype(np.float32)
    b = rng.normal(0, 0.01, E).astype(np.float32) if bias else None
    dg = lib.to_device(g)
    db = lib.to_device(b) if bias else None
    try:
        got = lib.moe_router_resident(h, dg, E, db, k)
    finally:
        lib.dev_free(dg)
        if db:
            lib.dev_free(db)
    assert np.array_equal(got, lib.moe_router(h, g, b, k))


@pytest.mark.parametrize("T,E,H,sg", [(2048, 32, 2880, 0.02), (1024, 128, 2880, 0.02), (16, 32, 2880, 0.02),
                                      (2048, 32, 512, 0.05), (300, 200, 256, 0.05)])
def test_router_logits_distance_from_sequential_sums(lib, oracle, T, E, H, sg):
    """The close-call threshold of the top-k selection (8 units of 2^-24 sqrt(H)) assumes
    that no tree-ordered logit is further than 3 units from the reference's sequential sum."""
    rng = np.random.default_rng(T + E)
    h = rng.normal(0, 1, (T, H)).astype(np.float32)
    g = rng.normal(0, sg, (E, H)).astype(np.float32)
    b = rng.normal(0, 0.01, E).astype(np.float32)
    got, want = lib.moe_router_logits(h, g, b), oracle.router_logits(h, g, b)
    rel = np.abs(got.astype(np.float64) - want) / np.maximum(1.0, np.abs(want))
    assert rel.max() <= 3.0 * 5.96e-8 * np.sqrt(H), rel.max() / (5.96e-8 * np.sqrt(H))


def _near_tie_gate(E, H, seed):
    """Gate rows in near-identical pairs: experts 2i and 2i+1 differ by a few 1e-7 relative,
    so their logits sit within an ulp or two of each other and the order of the fp32
    additions decides which one ranks first."""
    rng = np.random.default_rng(seed)
    g = rng.normal(0, 0.05, (E, H)).astype(np.float32)
    for e in range(0, E - 1, 2):
        g[e + 1] = g[e] * np.float32(1.0 + rng.choice([-3e-7, -1e-7, 1e-7, 3e-7]))
        g[e + 1, rng.integers(0, H, 8)] += np.float32(1e-7)
    return g


def _no_exact_tie_rows(logits, k):
    srt = -np.sort(-logits, axis=1)[:, :k + 1]
    return np.all(srt[:, :-1] != srt[:, 1:], axis=1)


@pytest.mark.parametrize("T,E,k,H", [(48, 16, 4, 2880), (300, 32, 4, 2880), (200, 10, 3, 96)])
def test_router_near_ties_follow_reference_order(lib, oracle, T, E, k, H):
    """Logits closer than summation-order noise: the indices and their slot order must
    still be the reference's (sequential-order recomputation of close calls); only exact
    ties of the reference's own logits are exempt."""
    rng = np.random.default_rng(T + E)
    h = rng.normal(0, 1, (T, H)).astype(np.float32)
    g = _near_tie_gate(E, H, seed=E * 7 + k)
    b = rng.normal(0, 0.01, E).astype(np.float32)
    b[1::2] = b[0:E - 1:2][:len(b[1::2])]  # same bias within a pair
    got = lib.moe_router(h, g, b, k)
    want = oracle.router(h, g, b, k)
    ok = _no_exact_tie_rows(oracle.router_logits(h, g, b), k)
    assert ok.sum() > T // 2
    # the pairs really are close calls: a float64 ranking disagrees with the reference's on some tokens
    l64 = h.astype(np.float64) @ g.astype(np.float64).T + b
    top64 = np.argsort(-l64, axis=1)[:, :k]
    assert np.any(top64[ok] != want[ok, :, 0].astype(int))
    assert np.array_equal(got[ok, :, 0], want[ok, :, 0])
    assert np.max(np.abs(got[ok, :, 1] - want[ok, :, 1])) <= ROUTING_WEIGHT_TOL


@pytest.mark.parametrize("T", [16, 4, 1])
def test_layer_small_batch_near_ties_follow_reference_order(lib, oracle, T):
    """The same through the small-batch routing kernels of the layer forward (up to four
    tokens: one wave per token; beyond: the single-workgroup kernel)."""
    E, k, H, F = 8, 2, 2880, 32
    L = synth.LayerInputs(E, k, H, F, seed=4)
    L.gate_w = _near_tie_gate(E, H, seed=5)
    L.gate_b[1::2] = L.gate_b[0::2]
    hidden = synth.hidden_states(T, H, seed=6)
    with build_layer(lib, L) as layer:
        _, pairs = layer.forward(hidden, want_pairs=True)
    want = oracle.router(hidden, L.gate_w, L.gate_b, k)
    ok = _no_exact_tie_rows(oracle.router_logits(hidden, L.gate_w, L.gate_b), k)
    assert ok.sum() >= (T + 1) // 2
    assert np.array_equal(pairs[ok, :, 0], want[ok, :, 0])


# ------------------------------------------------------------- expert MLP

def _const_matrix(rows, K, code_diag=None):
    nb = K // 32
    m = np.zeros((rows, nb, 17), np.uint8)
    m[:, :, 0] = 128
    if code_diag is not None:
        for r in range(min(rows, K)):
            blk, j = divmod(r, 32)
            if j < 16:
                m[r, blk, 1 + j] |= code_diag
            else:
                m[r, blk, 1 + j - 16] |= code_diag << 4
    return m.reshape(-1)


def test_expert_activation_known_answer(lib):
    # test/test_expert_mlp.cpp:118-200 recast for MXFP4 (gate = 1.0, up = 1.5, identity down)
    H = F = 32
    wz, wd = _const_matrix(F, H), _const_matrix(H, F, code_diag=1)
    out = lib.expert_token(np.ones(H, np.float32), wz, wz, wd, np.full(F, 1.5, np.float32),
                           np.full(F, 1.0, np.float32), np.zeros(H, np.float32), H, F)
    want = 1.0 / (1.0 + np.exp(-1.702)) * 2.5
    assert np.allclose(out, want, atol=1e-3)  # the reference test's own tolerance
    assert np.allclose(out, want, rtol=2e-5)  # activations travel as three FP6 terms: 2^-14.7 of a block's maximum


@pytest.mark.parametrize("H,F,bias,act", [(64, 96, True, 0), (256, 128, False, 0),
                                          (2880, 2880, True, 0), (128, 64, True, 1)])
def test_expert_token_matches_oracle(lib, oracle, H, F, bias, act):
    rng = np.random.default_rng(H + F)
    w = [synth.mxfp4_blocks(1, 0, 0, i, F if i < 2 else H, H if i < 2 else F) for i in range(3)]
    x = rng.normal(0, 1, H).astype(np.float32)
    b = [rng.normal(0, 0.01, n).astype(np.float32) if bias else None for n in (F, F, H)]
    got = lib.expert_token(x, *w, *b, H, F, act)
    want = oracle.expert_token(x, *w, *b, H, F, act)
    assert_layer_close(got, want)
    assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("wbf,T", [(False, 37), (True, 37), (False, 150), (True, 150), (True, 20000)])
def test_expert_node_rows_and_empty(lib, oracle, wbf, T):
    """T = 37 runs the streaming kernels, T = 150 the grouped GEMM; 20000 tokens are two passes
    whose inputs are too large for the pinned staging area and go up piece by piece."""
    H, F, k = 64, 96, 2
    rng = np.random.default_rng(1)
    w = [synth.mxfp4_blocks(3, 0, 4, i, F if i < 2 else H, H if i < 2 else F) for i in range(3)]
    hs = [lib.mxfp4_upload(w[0], F, H), lib.mxfp4_upload(w[1], F, H), lib.mxfp4_upload(w[2], H, F)]
    try:
        hidden = rng.normal(0, 1, (T, H)).astype(np.float32)
        pairs = np.zeros((T, k, 2), np.float32)
        for t in range(T):
            pairs[t, :, 0] = rng.choice(6, k, replace=False)
        pairs[..., 1] = rng.uniform(0.1, 0.9, (T, k))
        assert lib.expert_mlp(9, hidden, F, *hs, None, None, None, pairs) is None
        b = [rng.normal(0, 0.01, n).astype(np.float32) for n in (F, F, H)]
        for eid in (4, 0):
            got = lib.expert_mlp(eid, hidden, F, *hs, *b, pairs, weight_before_ffn=wbf)
            want = oracle.expert_mlp(eid, hidden, F, *w, *b, pairs, weight_before_ffn=wbf)
            sel = np.any(pairs[..., 0] == eid, axis=1)
            assert np.all(got[~sel] == 0)
            assert_layer_close(got, want)
    finally:
        for h in hs:
            lib.mxfp4_free(h)


# ------------------------------------------------------------------ merge

def test_merge_matches_oracle_bit_exact(lib, oracle):
    T, k, E, H = 9, 3, 5, 2880
    rng = np.random.default_rng(2)
    outs = [rng.normal(0, 1, (T, H)).astype(np.float32) for _ in range(E)]
    outs[3] = None
    pairs = np.zeros((T, k, 2), np.float32)
    for t in range(T):
        pairs[t, :, 0] = rng.choice(E, k, replace=False)
    pairs[..., 1] = rng.uniform(0, 1, (T, k))
    for pre in (False, True):
        rc, want = oracle.expert_merge(pairs, outs, H, pre_weighted=pre)
        assert rc == 0
        assert np.array_equal(lib.expert_merge(pairs, outs, H, pre_weighted=pre), want)
    with pytest.raises(capi.CskError) as ei:
        lib.expert_merge(pairs, [None] * E, H)
    assert ei.value.code == capi.ERR_ALL_EMPTY and "no non-empty expert outputs" in ei.value.message
    bad = pairs.copy()
    bad[0, 0, 0] = E
    with pytest.raises(capi.CskError) as ei:
        lib.expert_merge(bad, outs, H)
    assert ei.value.code == capi.ERR_RANGE


def test_rmsnorm_and_add(lib, oracle):
    x = np.array([[1, 2, 3, 4]], np.float32)
    w = np.array([2, 0.5, 1.5, 1], np.float32)
    assert np.allclose(lib.rmsnorm(x, w, 0.0), x / np.sqrt(7.5) * w, atol=1e-5)  # test_rmsnorm.cpp:74-115
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (5, 2880)).astype(np.float32)
    w = rng.normal(1, 0.02, 2880).astype(np.float32)
    assert np.allclose(lib.rmsnorm(x, w, 1e-5), oracle.rmsnorm(x, w, 1e-5), atol=1e-6, rtol=1e-6)
    assert np.array_equal(lib.add(x, x), oracle.add(x, x))


def test_rmsnorm_f64_equals_cpu_bit_for_bit(lib, oracle):
    """rmsnorm_node's float64 branch (rmsnorm_node.h:49-50): every operation is a double one
    in the reference's order, so the result is the CPU's."""
    assert lib.rmsnorm_f64(np.array([[5.0]]), np.array([2.0]), 0.0)[0, 0] == 2.0  # test_rmsnorm.cpp:118-142
    rng = np.random.default_rng(11)
    for T, H in ((1, 1), (3, 7), (9, 512), (5, 513), (17, 2880), (2, 5000)):
        x = rng.normal(0, 2, (T, H))
        w = rng.normal(1, 0.1, H)
        for eps in (0.0, 1e-5):
            assert np.array_equal(lib.rmsnorm_f64(x, w, eps), oracle.rmsnorm_f64(x, w, eps)), (T, H, eps)
    x = np.zeros((2, 64))
    assert np.array_equal(lib.rmsnorm_f64(x, np.ones(64), 1e-5), x)
    got = lib.rmsnorm_f64(x, np.ones(64), 0.0)  # 0 / 0, as the reference computes it
    assert np.all(np.isnan(got))


# ------------------------------------------------------------ whole layer

def _check_layer(lib, oracle, L, T, bias=True, norm=False, residual=False, device_weights=False,
                 oracle_tokens=-1, subset=False, **opts):
    """subset: the oracle replays only the experts the batch selects (real-shape layers whose
    weights were generated on the device)."""
    hidden = synth.hidden_states(T, L.H, seed=T + 17)
    flags = (capi.FWD_RMSNORM if norm else 0) | (capi.FWD_RESIDUAL if residual else 0)
    with build_layer(lib, L, bias=bias, norm=norm, device_weights=device_weights, **opts) as layer:
        got, pairs = layer.forward(hidden, flags, want_pairs=True)
        counts, toks = layer.last_dispatch(T)
    oopts = {}
    if "act" in opts:
        oopts["act"] = opts["act"]
    if "sigmoid" in opts:
        oopts["sigmoid"] = opts["sigmoid"]
    if "weight_before_ffn" in opts:
        oopts["weight_before_ffn"] = opts["weight_before_ffn"]
    if subset:
        assert bias and oracle_tokens < 0
        want, wpairs = oracle_layer_subset(oracle, L, hidden, T, norm=norm, residual=residual, **oopts)
    else:
        want, wpairs = oracle_layer(oracle, L, hidden, bias=bias, norm=norm, residual=residual,
                                    max_tokens=oracle_tokens, **oopts)
    xin = oracle.rmsnorm(hidden, L.norm_w, 1e-5) if norm else hidden
    real, near = classify_index_mismatches(oracle, xin, L, pairs, wpairs)
    assert real == 0, (real, near)
    if not norm:
        # the router sees the reference's own input: close calls are recomputed in the
        # reference's summation order, so not even a near-tie may come out differently
        assert near == 0, near
    same = np.all(pairs[..., 0] == wpairs[..., 0], axis=1)
    assert np.max(np.abs(pairs[same, :, 1] - wpairs[same, :, 1])) <= ROUTING_WEIGHT_TOL
    # dispatch: per-expert token lists are {t : e in topk(t)} ascending, counts sum to T*k
    ids = pairs[..., 0].astype(int)
    assert counts.sum() == T * L.k
    off = 0
    for e in range(L.E):
        want_t = np.nonzero(np.any(ids == e, axis=1))[0]
        assert counts[e] == want_t.size
        assert np.array_equal(toks[off:off + counts[e]], want_t)
        off += counts[e]
    n = T if oracle_tokens < 0 else min(T, oracle_tokens)
    rows = np.nonzero(same[:n])[0]
    return assert_layer_close(got[rows], want[rows])


def test_layer_config1_20b_8_tokens(lib, oracle):
    """BASELINE config 1: 20b shape, 8 tokens -- the parity configuration."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=1234)
    _check_layer(lib, oracle, L, 8)


def test_layer_config1_dequant_all_planes(lib, oracle):
    """Dequantised weights bit-exact, config 1 in full: every expert, all three planes."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=1234)
    with build_layer(lib, L) as layer:
        for e in range(L.E):
            for which in range(3):
                want = oracle.dequant(L.blocks(e, which), 2880 * 2880).reshape(2880, 2880)
                assert nbits_differ(layer.dequant(e, which), want) == 0, (e, which)


def test_layer_120b_dequant_sampled_experts(lib, oracle):
    """Dequantised weights bit-exact at the 120b shape (configs 4 / 5), weights generated on
    the device: a hot expert, a cold one and the last, against the host replay of the
    generator through the CPU codec."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=78, hot_experts=8)
    hot = int(np.argmax(L.gate_b))
    cold = int(np.argmin(L.gate_b))
    assert L.gate_b[hot] > 1.5 > 0.5 > L.gate_b[cold]
    with build_layer(lib, L, device_weights=True) as layer:
        for e in sorted({hot, cold, L.E - 1}):
            for which in range(3):
                want = oracle.dequant(L.blocks(e, which), 2880 * 2880).reshape(2880, 2880)
                assert nbits_differ(layer.dequant(e, which), want) == 0, (e, which)


@pytest.mark.parametrize("T", [1, 2, 4, 16])
def test_layer_config2_20b_decode_sweep(lib, oracle, T):
    """BASELINE config 2 at its real shape: the decode sweep's batch sizes that no other test of
    the 20b shape meets (8 is config 1, 32 and 64 follow below), against the CPU path."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=1234 + T)
    _check_layer(lib, oracle, L, T, device_weights=True, subset=True)


@pytest.mark.parametrize("T", [1, 2, 4, 16, 32])
def test_layer_decode_sweep_small_shape(lib, oracle, T):
    L = synth.LayerInputs(32, 4, 256, 192, seed=5)
    _check_layer(lib, oracle, L, T)


@pytest.mark.parametrize("T", [1, 9, 150])
def test_layer_nan_and_inf_tokens_propagate(lib, oracle, T):
    """A NaN or an infinity in a token's hidden state comes out as a non-finite output row,
    as in the reference's fp32 arithmetic (expert_mlp_node.h:651-732 has no clamp), in the
    streaming and in the grouped-GEMM regime; the other tokens of the batch still match the
    oracle.  (Which experts a token with NaN logits selects is unspecified in the reference
    -- its partial sort compares NaNs -- so only finiteness is compared for those rows.)"""
    L = synth.LayerInputs(8, 2, 128, 160, seed=9)
    hidden = synth.hidden_states(T, L.H, seed=T + 3)
    bad_nan, bad_inf = 0, (T - 1 if T > 1 else None)
    hidden[bad_nan, 37] = np.nan
    if bad_inf is not None:
        hidden[bad_inf, 5] = np.inf
    with build_layer(lib, L) as layer:
        got = layer.forward(hidden, 0)
    with np.errstate(all="ignore"):
        want, _ = oracle_layer(oracle, L, hidden)
    bad = [bad_nan] + ([bad_inf] if bad_inf is not None else [])
    for t in bad:
        assert not np.any(np.isfinite(want[t])), "oracle row finite?"
        assert not np.any(np.isfinite(got[t])), (t, got[t][:8])
    good = [t for t in range(T) if t not in bad]
    if good:
        assert_layer_close(got[good], want[good])


@pytest.mark.parametrize("opts", [dict(act=1), dict(sigmoid=True), dict(weight_before_ffn=True),
                                  dict(bias=False), dict(norm=True, residual=True)])
def test_layer_variants(lib, oracle, opts):
    opts = dict(opts)
    bias = opts.pop("bias", True)
    norm = opts.pop("norm", False)
    residual = opts.pop("residual", False)
    L = synth.LayerInputs(8, 2, 128, 160, seed=9, with_norm=True)
    _check_layer(lib, oracle, L, 21, bias=bias, norm=norm, residual=residual, **opts)


@pytest.mark.parametrize("opts", [dict(), dict(act=1), dict(sigmoid=True), dict(weight_before_ffn=True),
                                  dict(bias=False), dict(norm=True, residual=True),
                                  dict(weight_before_ffn=True, sigmoid=True, norm=True, residual=True)])
@pytest.mark.parametrize("shape", [(8, 2, 128, 160), (128, 4, 256, 192), (5, 5, 64, 96), (200, 16, 96, 64)])
def test_layer_one_token_variants(lib, oracle, opts, shape):
    """One token: the gate/up kernel selects the experts itself (no routing launch in front);
    every option of the layer, few and many experts, top_k = E and the largest top_k."""
    opts = dict(opts)
    bias = opts.pop("bias", True)
    norm = opts.pop("norm", False)
    residual = opts.pop("residual", False)
    E, k, H, F = shape
    L = synth.LayerInputs(E, k, H, F, seed=E + k, with_norm=True)
    _check_layer(lib, oracle, L, 1, bias=bias, norm=norm, residual=residual, **opts)


@pytest.mark.parametrize("opts", [dict(act=1), dict(sigmoid=True), dict(weight_before_ffn=True),
                                  dict(bias=False), dict(norm=True, residual=True),
                                  dict(weight_before_ffn=True, norm=True, residual=True)])
def test_layer_variants_grouped_gemm(lib, oracle, opts):
    """The same variants at a batch that takes the grouped-GEMM path (T > 64), on a shape
    whose expert count, feature count and K are not multiples of the tile sizes."""
    opts = dict(opts)
    bias = opts.pop("bias", True)
    norm = opts.pop("norm", False)
    residual = opts.pop("residual", False)
    L = synth.LayerInputs(7, 3, 160, 224, seed=19, with_norm=True)
    _check_layer(lib, oracle, L, 131, bias=bias, norm=norm, residual=residual, **opts)


def test_layer_few_tokens_long_rows(lib, oracle):
    """Rows longer than the streaming kernel's LDS budget: few tokens still take the GEMM."""
    L = synth.LayerInputs(4, 2, 3200, 64, seed=23, with_norm=True)
    _check_layer(lib, oracle, L, 6, norm=True, residual=True)
    L = synth.LayerInputs(4, 2, 64, 3200, seed=24)
    _check_layer(lib, oracle, L, 5)
    # rows longer than 4096: the prologue + logits kernel reads them in several rounds instead of holding them
    L = synth.LayerInputs(6, 2, 4608, 64, seed=25, with_norm=True)
    _check_layer(lib, oracle, L, 3, norm=True, residual=True)
    _check_layer(lib, oracle, L, 7)


@pytest.mark.parametrize("H,F", [(3072, 3072), (32, 3072), (3072, 32), (32, 32), (3040, 2976)])
@pytest.mark.parametrize("T", [3, 23])
def test_layer_streaming_row_length_limits(lib, oracle, H, F, T):
    """The streaming kernels at the ends of the row lengths they accept: 3072 (every block
    of the activation rows in LDS holds data, none is a zero tail), one block of 32, and
    lengths whose last 128-wide step is partly past the row."""
    L = synth.LayerInputs(5, 2, H, F, seed=11 + H // 32 + F // 64, with_norm=True)
    _check_layer(lib, oracle, L, T, norm=True, residual=True)


def test_layer_many_tokens_per_expert(lib, oracle):
    """More than 64 tokens on one expert: several passes of the M tiles."""
    L = synth.LayerInputs(4, 2, 128, 96, seed=3)
    _check_layer(lib, oracle, L, 300)


def test_layer_120b_shape_skewed_16_tokens(lib, oracle):
    """BASELINE config 4 at T=16: 128 experts, 8 hot experts with +2.0 bias;
    weights generated on the device, replayed on the host for the oracle."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=42, hot_experts=8)
    _check_layer(lib, oracle, L, 16, device_weights=True)


@pytest.mark.parametrize("T", [32, 64])
def test_layer_20b_shape_wide_token_groups(lib, oracle, T):
    """BASELINE config 2 above 16 tokens: the wide-group streaming kernels at K = 2880."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=52)
    _check_layer(lib, oracle, L, T, device_weights=True, subset=True)


@pytest.mark.parametrize("T", [1, 64])
def test_layer_120b_shape_skewed_1_and_64_tokens(lib, oracle, T):
    """BASELINE config 4 / 5 shape at the ends of the decode range, with the skewed bias."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=43, hot_experts=8)
    _check_layer(lib, oracle, L, T, device_weights=True, subset=True)


@pytest.mark.parametrize("T", [160, 320])
def test_layer_120b_shape_many_experts_few_tokens_each(lib, oracle, T):
    """More than 64 tokens, but at most ten assignments per expert on average: such a batch
    still takes the streaming kernels (groups of seven tokens; the hot experts take many)."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=44, hot_experts=8)
    _check_layer(lib, oracle, L, T, device_weights=True, subset=True)


@pytest.mark.parametrize("opts", [dict(weight_before_ffn=True, sigmoid=True), dict(act=1)])
def test_layer_many_small_experts_beyond_64_tokens(lib, oracle, opts):
    L = synth.LayerInputs(64, 4, 128, 96, seed=45)
    _check_layer(lib, oracle, L, 150, **opts)


# ----------------------------------------------------- prefill (grouped GEMM)

def _prefill_case(lib, oracle, L, T, ntok_oracle):
    hidden = synth.hidden_states(T, L.H, seed=T + 3)
    with build_layer(lib, L, device_weights=True) as layer:
        got, pairs = layer.forward(hidden, want_pairs=True)
        counts, toks = layer.last_dispatch(T)
        again = layer.forward(hidden)
        # a token's result does not depend on its place in the batch: permuting the
        # tokens permutes the outputs bit for bit
        perm = np.random.default_rng(1).permutation(T)
        got_p = layer.forward(hidden[perm])
        # ... nor on the kernels its batch takes: every token of the batch, sixteen at a time
        # through the weight-streaming kernels (themselves checked against the CPU path on
        # their own), selects the same experts and gives the same result to a fifth of the bar
        for t0 in range(0, T, 16):
            small, spairs = layer.forward(hidden[t0:t0 + 16], want_pairs=True)
            assert np.array_equal(spairs[..., 0], pairs[t0:t0 + 16, :, 0]), t0
            assert_layer_close(got[t0:t0 + 16], small, tol=2e-4)
    assert nbits_differ(got, again) == 0
    assert nbits_differ(got_p, got[perm]) == 0
    ids = pairs[..., 0].astype(int)
    assert counts.sum() == T * L.k and np.array_equal(counts, np.bincount(ids.ravel(), minlength=L.E))
    off = np.concatenate([[0], np.cumsum(counts)])
    for e in range(L.E):
        assert np.array_equal(toks[off[e]:off[e + 1]], np.nonzero(np.any(ids == e, axis=1))[0])
    assert np.allclose(pairs[..., 1].sum(axis=1), 1.0, atol=1e-5)
    # against the CPU path: a sample strided over the batch, plus the tokens of the last
    # (ragged) M tile of the expert with the most tokens and of the one with the fewest --
    # rows that sit beside padding in a 64- and in a 32-token work unit
    busiest = int(np.argmax(counts))
    fewest = int(np.argmin(np.where(counts > 0, counts, T * L.k + 1)))
    idx = set(np.linspace(0, T - 1, ntok_oracle).astype(int).tolist())
    for e in (busiest, fewest):
        lst = toks[off[e]:off[e + 1]]
        idx |= set(lst[64 * ((lst.size - 1) // 64):].tolist())
    idx = np.array(sorted(idx))
    assert idx.size >= 64 or idx.size == T
    want, wpairs = oracle_layer_tokens(oracle, L, hidden, idx)
    real, near = classify_index_mismatches(oracle, hidden[idx], L, pairs[idx], wpairs)
    assert (real, near) == (0, 0)
    same = np.all(pairs[idx, :, 0] == wpairs[..., 0], axis=1)
    assert np.max(np.abs(pairs[idx][same, :, 1] - wpairs[same, :, 1])) <= ROUTING_WEIGHT_TOL
    assert_layer_close(got[idx][same], want[same])
    return counts


def test_prefill_20b_2048_tokens(lib, oracle):
    """BASELINE config 3: 20b shape, 2048 tokens (about 256 tokens per expert)."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=77)
    counts = _prefill_case(lib, oracle, L, 2048, 48)
    assert counts.min() > 64  # natural routing: every expert sees several M tiles


def test_prefill_120b_skewed_4096_tokens(lib, oracle):
    """BASELINE config 4 at T=4096: 8 hot experts take about half of the assignments."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=78, hot_experts=8)
    counts = _prefill_case(lib, oracle, L, 4096, 48)
    hot = np.sort(counts)[-8:].sum() / counts.sum()
    assert 0.4 < hot < 0.75, hot  # +2.0 logit offset on logits of std ~1.1


@pytest.mark.parametrize("T,seed", [(512, 80), (1024, 79)])
def test_prefill_repeatable_with_many_small_experts(lib, T, seed):
    """128 experts with a skewed router at a few hundred tokens: most experts hold a handful
    of tokens, so most M tiles are ragged and their padding rows repeat the last token --
    the timing in which a load that the compiler does not track, or a register moved while
    such a load is in flight, shows as a few wrong rows in some runs.  Every run must give
    the same bits."""
    L = synth.LayerInputs(128, 4, 2880, 2880, seed=seed, hot_experts=8)
    hidden = synth.hidden_states(T, L.H, seed=T + 3)
    with build_layer(lib, L, device_weights=True) as layer:
        first = layer.forward(hidden)
        assert np.all(np.isfinite(first))
        for _ in range(11):
            assert nbits_differ(layer.forward(hidden), first) == 0


def test_prefill_ragged_small_shape(lib, oracle):
    """Token counts that are not multiples of the 64-token M tile, N not a multiple of
    the 128-feature N tile, K not a multiple of the 128-element K step."""
    L = synth.LayerInputs(5, 2, 96, 160, seed=31)
    hidden = synth.hidden_states(333, L.H, seed=2)
    with build_layer(lib, L) as layer:
        got, pairs = layer.forward(hidden, want_pairs=True)
    want, wpairs = oracle_layer(oracle, L, hidden)
    real, near = classify_index_mismatches(oracle, hidden, L, pairs, wpairs)
    assert (real, near) == (0, 0)
    assert_layer_close(got, want)


def test_concurrent_forwards_equal_sequential(lib):
    """Two threads, each driving its own layer through the C ABI at the same time (ctypes
    releases the interpreter lock during a call): the library serialises the calls, so every
    result is bit-identical to the one the same call gives when made alone."""
    import threading
    shapes = [(8, 2, 128, 160, 21), (16, 4, 256, 192, 150)]
    layers, hiddens, wants = [], [], []
    for i, (E, k, H, F, T) in enumerate(shapes):
        L = synth.LayerInputs(E, k, H, F, seed=40 + i)
        layer = build_layer(lib, L)
        hidden = synth.hidden_states(T, H, seed=i)
        layers.append(layer), hiddens.append(hidden), wants.append(layer.forward(hidden))
    bad = [0, 0]

    def work(i):
        for _ in range(20):
            if not np.array_equal(layers[i].forward(hiddens[i]), wants[i]):
                bad[i] += 1

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for layer in layers:
        layer.close()
    assert bad == [0, 0]


@pytest.mark.parametrize("E,k,H,F,T,n_layers", [(8, 2, 128, 160, 1, 4), (8, 2, 128, 160, 8, 4), (16, 4, 256, 192, 64, 3),
                                                (128, 4, 2880, 2880, 1, 2), (128, 4, 2880, 2880, 8, 2)])
def test_stack_config5(lib, oracle, E, k, H, F, T, n_layers):
    """BASELINE config 5: h <- h + MoE(RMSNorm(h)) through several layers on the device
    (csk_moe_stack_forward).  The stack equals the same layers called one at a time bit for
    bit, and every layer's output matches the CPU path fed with that layer's actual input
    (so that a routing near-tie in one layer is not carried into the next comparison)."""
    from coalsack_amd.capi import stack_forward
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    big = H >= 2048
    Ls = [synth.LayerInputs(E, k, H, F, seed=77, layer=i, with_norm=True) for i in range(n_layers)]
    layers = [build_layer(lib, L, norm=True, device_weights=big) for L in Ls]
    hidden = synth.hidden_states(T, H, seed=3)
    d_h = lib.to_device(hidden)
    try:
        stack_forward(lib, layers, d_h, T)
        got_stack = lib.to_host(d_h, hidden.shape)
        h = hidden
        for L, layer in zip(Ls, layers):
            nxt, pairs = layer.forward(h, flags, want_pairs=True)
            n = T if not big else min(T, 3)
            if big:  # replay only the experts the first tokens select
                want, wpairs = oracle_layer_subset(oracle, L, h, n, norm=True, residual=True)
            else:
                want, wpairs = oracle_layer(oracle, L, h, norm=True, residual=True)
            xin = oracle.rmsnorm(h[:n], L.norm_w, 1e-5)
            real, near = classify_index_mismatches(oracle, xin, L, pairs[:n], wpairs[:n])
            assert real == 0, (real, near)  # the router input carries the GPU's RMSNorm rounding: near-ties are tolerated
            same = np.all(pairs[:n, :, 0] == wpairs[:n, :, 0], axis=1)
            assert_layer_close(nxt[:n][same], want[:n][same])
            h = nxt
        assert np.array_equal(got_stack, h)
    finally:
        lib.dev_free(d_h)
        for layer in layers:
            layer.close()


def test_stack_config5_36_resident_layers(lib, oracle):
    """BASELINE config 5 as stated: 36 layers of the 120b shape resident at once (61 GB of
    expert planes, generated on the device), decode batches of 1, 8 and 64 tokens.  The stack
    call equals the layers called one at a time bit for bit; on sampled layers the output of
    the layer matches the CPU path fed with that layer's actual input, on sampled tokens
    (the host replays only the experts those tokens select)."""
    from coalsack_amd.capi import stack_forward
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    E, k, H, F, n_layers = 128, 4, 2880, 2880, 36
    Ls = [synth.LayerInputs(E, k, H, F, seed=91, layer=i, hot_experts=8, with_norm=True) for i in range(n_layers)]
    layers = []
    try:
        for L in Ls:
            layers.append(build_layer(lib, L, norm=True, device_weights=True))
        for T, sampled in ((1, (0, 17, 35)), (8, (1, 20, 35)), (64, (2, 35))):
            hidden = synth.hidden_states(T, H, seed=30 + T)
            d_h = lib.to_device(hidden)
            try:
                stack_forward(lib, layers, d_h, T)
                got_stack = lib.to_host(d_h, hidden.shape)
            finally:
                lib.dev_free(d_h)
            h = hidden
            n = min(T, 4)
            for i, (L, layer) in enumerate(zip(Ls, layers)):
                nxt, pairs = layer.forward(h, flags, want_pairs=True)
                if i in sampled:
                    want, wpairs = oracle_layer_subset(oracle, L, h, n, norm=True, residual=True)
                    xin = oracle.rmsnorm(h[:n], L.norm_w, 1e-5)
                    real, near = classify_index_mismatches(oracle, xin, L, pairs[:n], wpairs)
                    assert real == 0, (T, i, real, near)
                    same = np.all(pairs[:n, :, 0] == wpairs[..., 0], axis=1)
                    assert same.any(), (T, i)
                    # the residual stream grows through the stack: compare the layer's own
                    # contribution (output minus residual input) to the bar as well
                    assert_layer_close(nxt[:n][same], want[same])
                    assert_layer_close((nxt[:n] - h[:n])[same], (want - h[:n])[same])
                h = nxt
            assert np.all(np.isfinite(got_stack))
            assert np.array_equal(got_stack, h), T
    finally:
        for layer in layers:
            layer.close()


def test_long_batch_in_passes(lib, oracle):
    """A batch longer than the pass size is taken in passes of equal size (tokens are
    independent): same result bit for bit while the passes use the kernels the whole batch
    would, same router output, and the CPU path's result in any case."""
    L = synth.LayerInputs(8, 2, 128, 160, seed=21, with_norm=True)
    T = 333
    hidden = synth.hidden_states(T, L.H, seed=9)
    flags = capi.FWD_RMSNORM | capi.FWD_RESIDUAL
    with build_layer(lib, L, norm=True) as layer:
        whole, pairs = layer.forward(hidden, flags, want_pairs=True)
        layer.last_dispatch(T)
        try:
            lib.set_pass_tokens(100)  # four passes of 84, 84, 84, 81 tokens: grouped GEMM, as the whole batch
            got, gpairs = layer.forward(hidden, flags, want_pairs=True)
            assert np.array_equal(got, whole) and np.array_equal(gpairs, pairs)
            assert np.array_equal(layer.forward(hidden, flags), whole)
            with pytest.raises(capi.CskError, match="several passes"):
                layer.last_dispatch(T)
            lib.set_pass_tokens(50)   # seven passes of 48 tokens: the streaming kernels
            small, spairs = layer.forward(hidden, flags, want_pairs=True)
        finally:
            lib.set_pass_tokens(32768)
        with pytest.raises(capi.CskError):
            lib.set_pass_tokens(0)
    # other kernels, another summation order: the same experts (no near-tie in this batch), weights to rounding
    assert np.array_equal(spairs[..., 0], pairs[..., 0]) and np.max(np.abs(spairs[..., 1] - pairs[..., 1])) < 1e-5
    want, wpairs = oracle_layer(oracle, L, hidden, norm=True, residual=True)
    real, near = classify_index_mismatches(oracle, oracle.rmsnorm(hidden, L.norm_w, 1e-5), L, pairs, wpairs)
    assert real == 0, (real, near)
    same = np.all(pairs[..., 0] == wpairs[..., 0], axis=1)
    assert_layer_close(small[same], want[same])
    assert_layer_close(whole[same], want[same])


@pytest.mark.parametrize("E,T,norm", [(128, 64, True), (128, 64, False), (200, 40, True), (130, 33, False)])
def test_layer_many_experts_small_batch(lib, oracle, E, T, norm):
    """Small batches over many experts: the prologue + logits kernel then gives a workgroup
    four experts (the one-expert workgroups would not all be resident), with expert counts
    that are not multiples of four and ragged token tiles."""
    L = synth.LayerInputs(E, 4, 128, 96, seed=61, with_norm=True)
    _check_layer(lib, oracle, L, T, norm=norm, residual=norm)


@pytest.mark.parametrize("T", [3, 4, 5, 32, 33, 64, 65, 200])
def test_layer_maximum_experts_and_top_k(lib, oracle, T):
    """The limits of a layer: 256 experts, top-16 -- four tokens fill the one-wave-per-token
    router (64 assignments), 32 are the most the single-workgroup one takes (512 assignments),
    33 to 64 go through the multi-workgroup selection and the dispatch kernel behind the fused
    norm + logits kernel, 65 through the separate kernels, 200 take the grouped GEMM."""
    L = synth.LayerInputs(256, 16, 64, 96, seed=71)
    _check_layer(lib, oracle, L, T)
