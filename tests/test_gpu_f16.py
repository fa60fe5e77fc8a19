"""GPU parity of the fp16 expert path (csk_f16_*, csk_expert_mlp_f16, fp16 layers) against
the CPU restatement, through the C ABI.  Tolerance: 1e-3 of the output scale, as for the
MXFP4 path; measured differences are ~1e-6."""
import numpy as np
import pytest

from coalsack_amd import capi, synth
from tests.helpers import assert_layer_close
from tests.test_oracle_expert import modified_swiglu_ref
from tests.test_oracle_expert_f16 import random_f16_expert

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,K", [(16, 32), (37, 45), (1, 1), (200, 2880), (2880, 96)])
def test_f16_upload_export_round_trip(lib, rows, K):
    rng = np.random.default_rng([rows, K])
    w = rng.standard_normal((rows, K)).astype(np.float16)
    w.reshape(-1)[:4] = np.array([0.0, -0.0, 65504.0, 6e-8], np.float16)[:min(4, w.size)]
    h = lib.f16_upload(w)
    try:
        back = lib.f16_export(h, rows, K)
    finally:
        lib.f16_free(h)
    assert np.array_equal(back.view(np.uint16), w.view(np.uint16))


@pytest.mark.parametrize("kind,ty", [("q4_k", 12), ("q6_k", 14)])
@pytest.mark.parametrize("rows,K", [(16, 256), (48, 160), (37, 256), (2880, 512)])
def test_kquant_upload_equals_weight_provider_halves(lib, oracle, kind, ty, rows, K):
    """csk_f16_upload_ggml on a Q4_K / Q6_K stream leaves exactly the halves the reference's
    provider computes (dequantize, then the truncating fp32 -> fp16), also when super-blocks
    straddle rows (K = 160)."""
    from tests.golden.make_kquant_golden import random_blocks
    rng = np.random.default_rng([rows, K, ty])
    blocks = random_blocks(rng, kind, rows * K // 256).reshape(-1)
    want = oracle.kquant_to_fp16(kind, blocks, rows * K).reshape(rows, K)
    h = lib.f16_upload_ggml(ty, blocks, rows, K)
    try:
        got = lib.f16_export(h, rows, K)
    finally:
        lib.f16_free(h)
    assert np.array_equal(got.view(np.uint16), want)


def test_kquant_upload_fixture_and_errors(lib):
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "kquant_codec.npz"))
    for tag, ty in (("q4", 12), ("q6", 14)):
        b = gold[tag + "_blocks"]
        h = lib.f16_upload_ggml(ty, b.reshape(-1), 48, 256)
        try:
            assert np.array_equal(lib.f16_export(h, 48, 256).view(np.uint16).reshape(-1), gold[tag + "_f16"])
        finally:
            lib.f16_free(h)
    with pytest.raises(capi.CskError, match="multiple of 256"):
        lib.f16_upload_ggml(12, np.zeros(144, np.uint8), 3, 100)
    with pytest.raises(capi.CskError, match="ggml types"):
        lib.f16_upload_ggml(13, np.zeros(176, np.uint8), 16, 16)


def test_reference_known_answer_two_by_two(lib):
    # test/test_expert_mlp.cpp:118-200
    x = np.array([[1.0, 0.5]], np.float32)
    w_up = np.zeros((2, 2), np.float16)
    w_gate = np.zeros((2, 2), np.float16)
    w_down = np.zeros((2, 2), np.float16)
    w_up[0, 0] = 1.0
    w_gate[0, 0] = 1.0
    w_down.reshape(-1)[0] = 1.0
    w_down.reshape(-1)[2] = 1.0
    b_up = np.array([0.5, 0.0], np.float32)
    zero = np.zeros(2, np.float32)
    pairs = np.array([[[0, 1.0], [1, 0.0], [2, 0.0], [3, 0.0]]], np.float32)
    out = lib.expert_mlp_f16(0, x, w_up, w_gate, w_down, b_up, zero, zero, pairs)
    assert abs(out[0, 0] - modified_swiglu_ref(1.0, 1.5)) < 1e-3  # the reference's own tolerance
    assert abs(out[0, 0] - modified_swiglu_ref(1.0, 1.5)) < 1e-6


@pytest.mark.parametrize("T,H,F", [(5, 64, 96), (7, 37, 29), (3, 2880, 2880), (150, 96, 160),
                                   (70, 45, 50), (18000, 64, 32)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("act,wbf", [(0, False), (1, False), (0, True)])
def test_expert_node_matches_oracle(lib, oracle, T, H, F, bias, act, wbf):
    if H == 2880 and (bias or act or wbf):
        pytest.skip("large shape: one variant is enough")
    if T == 18000 and (act or not bias):
        pytest.skip("long batch (two passes, inputs past the pinned staging area): two variants are enough")
    rng = np.random.default_rng([T, H, F, act])
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    w = random_f16_expert(rng, H, F, 0.1)
    b = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)] if bias else [None] * 3
    k = 2
    pairs = np.zeros((T, k, 2), np.float32)
    sel = rng.random(T) < 0.6
    sel[0] = True
    pairs[:, 0, 0] = np.where(sel, 4, 1)
    pairs[:, 1, 0] = 2
    pairs[..., 1] = rng.random((T, k)).astype(np.float32)
    got = lib.expert_mlp_f16(4, hidden, *w, *b, pairs, act=act, weight_before_ffn=wbf)
    want = oracle.expert_mlp_f16(4, hidden, *w, *b, pairs, act=act, weight_before_ffn=wbf)
    assert_layer_close(got, want)
    assert not got[~sel].any()
    assert lib.expert_mlp_f16(9, hidden, *w, *b, pairs, act=act, weight_before_ffn=wbf) is None


def test_expert_node_shape_errors(lib):
    hidden = np.zeros((2, 8), np.float32)
    pairs = np.zeros((2, 1, 2), np.float32)
    good = np.zeros((4, 8), np.float16), np.zeros((4, 8), np.float16), np.zeros((8, 4), np.float16)
    with pytest.raises(capi.CskError, match="w_down must be"):
        lib.expert_mlp_f16(0, hidden, good[0], good[1], np.zeros((8, 5), np.float16), None, None, None, pairs)
    with pytest.raises(capi.CskError, match="w_gate must be"):
        lib.expert_mlp_f16(0, hidden, good[0], np.zeros((4, 7), np.float16), good[2], None, None, None, pairs)
    with pytest.raises(capi.CskError, match="biases"):
        lib.expert_mlp_f16(0, hidden, *good, np.zeros(4, np.float32), None, None, pairs)


def _f16_layer(lib, L, ws, bias=True, norm=False, **opts):
    layer = lib.layer(L.E, L.k, L.H, L.F, f16=True)
    layer.set_router(L.gate_w, L.gate_b)
    for e in range(L.E):
        b = (L.b_up[e], L.b_gate[e], L.b_down[e]) if bias else (None, None, None)
        layer.set_expert_f16(e, *ws[e], *b)
    if norm:
        layer.set_norm(L.norm_w, 1e-5)
    if opts:
        layer.set_options(**opts)
    return layer


def _oracle_f16_layer(oracle, L, ws, hidden, bias=True, norm=False, residual=False, **opts):
    w_up = np.stack([w[0] for w in ws])
    w_gate = np.stack([w[1] for w in ws])
    w_down = np.stack([w[2] for w in ws])
    return oracle.moe_layer(hidden, L.E, L.k, L.H, L.F, L.gate_w, L.gate_b, w_up, w_gate, w_down,
                            L.b_up if bias else None, L.b_gate if bias else None,
                            L.b_down if bias else None, norm_w=L.norm_w if norm else None,
                            norm_eps=1e-5, residual=residual, **opts)


@pytest.mark.parametrize("T", [1, 5, 33, 64, 65, 200])
def test_f16_layer_matches_oracle(lib, oracle, T):
    L = synth.LayerInputs(8, 2, 96, 160, seed=17, with_norm=True)
    rng = np.random.default_rng(17)
    ws = [random_f16_expert(rng, L.H, L.F, 0.1) for _ in range(L.E)]
    hidden = synth.hidden_states(T, L.H)
    with _f16_layer(lib, L, ws, norm=True) as layer:
        for flags in (0, capi.FWD_RMSNORM | capi.FWD_RESIDUAL):
            got, pairs = layer.forward(hidden, flags=flags, want_pairs=True)
            want, wpairs = _oracle_f16_layer(oracle, L, ws, hidden, norm=bool(flags),
                                             residual=bool(flags))
            assert np.array_equal(pairs[..., 0], wpairs[..., 0])
            assert_layer_close(got, want)
            counts, _ = layer.last_dispatch(T)
            assert counts.sum() == T * L.k


@pytest.mark.parametrize("opts", [dict(sigmoid=True), dict(act=1), dict(weight_before_ffn=True),
                                  dict(sigmoid=True, act=1, weight_before_ffn=True)])
@pytest.mark.parametrize("T", [6, 130])
def test_f16_layer_variants(lib, oracle, opts, T):
    L = synth.LayerInputs(6, 3, 64, 96, seed=23)
    rng = np.random.default_rng(23)
    ws = [random_f16_expert(rng, L.H, L.F, 0.1) for _ in range(L.E)]
    hidden = synth.hidden_states(T, L.H)
    with _f16_layer(lib, L, ws, **opts) as layer:
        got = layer.forward(hidden)
        want, _ = _oracle_f16_layer(oracle, L, ws, hidden, **opts)
        assert_layer_close(got, want)


def test_f16_layer_20b_shape_device_weights(lib, oracle):
    """20b-shaped layer (32 experts, top-4, 2880 x 2880) with weights generated on the GPU;
    the oracle gets them back through the export, only for the experts the tokens select."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=31)
    T = 4
    hidden = synth.hidden_states(T, L.H)
    with lib.layer(L.E, L.k, L.H, L.F, f16=True) as layer:
        layer.set_router(L.gate_w, L.gate_b)
        layer.fill_synthetic(31, 0)
        for e in range(L.E):
            layer.set_expert_f16(e, None, None, None, L.b_up[e], L.b_gate[e], L.b_down[e])
        got, pairs = layer.forward(hidden, want_pairs=True)
        want_pairs = oracle.router(hidden, L.gate_w, L.gate_b, L.k)
        assert np.array_equal(pairs[..., 0], want_pairs[..., 0])
        want = np.zeros_like(got)
        for t in range(T):
            for j in range(L.k):
                e = int(want_pairs[t, j, 0])
                w = [layer.export_f16(e, which) for which in (capi.W_UP, capi.W_GATE, capi.W_DOWN)]
                assert np.abs(w[0].astype(np.float32)).max() <= 0.125
                y = oracle.expert_token_f16(hidden[t], *w, L.b_up[e], L.b_gate[e], L.b_down[e])
                want[t] += want_pairs[t, j, 1] * y
        assert_layer_close(got, want)


def test_f16_layer_20b_shape_many_tokens(lib, oracle):
    """The same layer at 1024 tokens (grouped GEMM, about 128 tokens per expert): the first
    tokens against the CPU path, and every token against the same layer run sixteen tokens at
    a time through the decode kernels -- same experts, same result to a fifth of the bar."""
    L = synth.LayerInputs(32, 4, 2880, 2880, seed=31)
    T = 1024
    hidden = synth.hidden_states(T, L.H, seed=5)
    with lib.layer(L.E, L.k, L.H, L.F, f16=True) as layer:
        layer.set_router(L.gate_w, L.gate_b)
        layer.fill_synthetic(31, 0)
        for e in range(L.E):
            layer.set_expert_f16(e, None, None, None, L.b_up[e], L.b_gate[e], L.b_down[e])
        got, pairs = layer.forward(hidden, want_pairs=True)
        for t0 in range(0, T, 16):
            small, spairs = layer.forward(hidden[t0:t0 + 16], want_pairs=True)
            assert np.array_equal(spairs[..., 0], pairs[t0:t0 + 16, :, 0]), t0
            assert_layer_close(got[t0:t0 + 16], small, tol=2e-4)
        nt = 2
        want_pairs = oracle.router(hidden[:nt], L.gate_w, L.gate_b, L.k)
        assert np.array_equal(pairs[:nt, :, 0], want_pairs[..., 0])
        want = np.zeros_like(got[:nt])
        for t in range(nt):
            for j in range(L.k):
                e = int(want_pairs[t, j, 0])
                w = [layer.export_f16(e, which) for which in (capi.W_UP, capi.W_GATE, capi.W_DOWN)]
                y = oracle.expert_token_f16(hidden[t], *w, L.b_up[e], L.b_gate[e], L.b_down[e])
                want[t] += want_pairs[t, j, 1] * y
        assert_layer_close(got[:nt], want)


def test_layer_kinds_do_not_mix(lib):
    with lib.layer(2, 1, 32, 32, f16=True) as layer:
        with pytest.raises(capi.CskError, match="fp16 experts"):
            layer.set_expert(0, np.zeros(32 * 17, np.uint8), np.zeros(32 * 17, np.uint8),
                             np.zeros(32 * 17, np.uint8))
    with lib.layer(2, 1, 32, 32) as layer:
        with pytest.raises(capi.CskError, match="MXFP4 experts"):
            layer.set_expert_f16(0, *[np.zeros((32, 32), np.float16)] * 3)


@pytest.mark.parametrize("T,H,F", [(1, 64, 96), (7, 37, 29), (64, 96, 160), (65, 96, 160), (300, 128, 72),
                                   (3, 1024, 2048)])
@pytest.mark.parametrize("bias", ["none", "all", "down_only"])
def test_dense_ffn_matches_oracle(lib, oracle, T, H, F, bias):
    """The shared expert (dense_ffn_node): every token through one fp16 gated MLP."""
    rng = np.random.default_rng([T, H, F])
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    w_up, w_gate, w_down = random_f16_expert(rng, H, F, 0.1)
    bg, bu, bd = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)]
    if bias == "none":
        bg = bu = bd = None
    elif bias == "down_only":
        bg = bu = None
    got = lib.dense_ffn_f16(hidden, w_gate, w_up, w_down, bg, bu, bd)
    want = oracle.dense_ffn_f16(hidden, w_gate, w_up, w_down, bg, bu, bd)
    assert_layer_close(got, want)


def test_dense_ffn_shape_errors(lib):
    hidden = np.zeros((2, 8), np.float32)
    g, u, d = np.zeros((4, 8), np.float16), np.zeros((4, 8), np.float16), np.zeros((8, 4), np.float16)
    with pytest.raises(capi.CskError, match="gate_w/up_w shape mismatch"):
        lib.dense_ffn_f16(hidden, g, np.zeros((5, 8), np.float16), d)
    with pytest.raises(capi.CskError, match="down_w shape mismatch, expected"):
        lib.dense_ffn_f16(hidden, g, u, np.zeros((8, 5), np.float16))


@pytest.mark.parametrize("M,K,N", [(1, 64, 96), (7, 37, 29), (64, 2880, 512), (65, 96, 160), (300, 128, 72),
                                   (2, 5120, 1024)])
def test_matmul_transpose_matches_oracle(lib, oracle, M, K, N):
    """matmul_transpose_mixed_node with a float16 weight (the engine's linear projections)."""
    rng = np.random.default_rng([M, K, N])
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.1).astype(np.float16)
    got = lib.matmul_transpose_f16(a, w)
    want = oracle.matmul_transpose_f16(a, w)
    assert got.shape == (M, N)
    assert_layer_close(got, want)
    with pytest.raises(capi.CskError, match="incompatible dimensions"):
        lib.matmul_transpose_f16(a[:, :K - 1] if K > 1 else a, w)


@pytest.mark.parametrize("T,H,F", [(1, 64, 96), (7, 37, 29), (65, 96, 160), (3, 1024, 2048)])
@pytest.mark.parametrize("bias", ["none", "all"])
def test_dense_ffn_float32_weights_match_oracle(lib, oracle, T, H, F, bias):
    """dense_ffn_node's FLOAT32 weight branch (dense_ffn_node.h:102-113): the weights travel as two
    fp16 terms, so they are exact to 2^-25 absolute; the result is held to the layer bar against
    the oracle's scalar fp32 loops and to 2e-5 of the largest output against float64."""
    rng = np.random.default_rng([T, H, F, 32])
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    w_gate, w_up = [(rng.standard_normal((F, H)) * 0.1).astype(np.float32) for _ in range(2)]
    w_down = (rng.standard_normal((H, F)) * 0.1).astype(np.float32)
    bg, bu, bd = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)]
    if bias == "none":
        bg = bu = bd = None
    got = lib.dense_ffn_f16(hidden, w_gate, w_up, w_down, bg, bu, bd)
    want = oracle.dense_ffn_f32(hidden, w_gate, w_up, w_down, bg, bu, bd)
    assert_layer_close(got, want)
    x = hidden.astype(np.float64)
    g = x @ w_gate.astype(np.float64).T + (0 if bg is None else bg)
    u = x @ w_up.astype(np.float64).T + (0 if bu is None else bu)
    ref = (g / (1 + np.exp(-g)) * u) @ w_down.astype(np.float64).T + (0 if bd is None else bd)
    assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


def test_dense_ffn_weight_types_must_agree(lib):
    hidden = np.zeros((2, 8), np.float32)
    h16 = [lib.f16_upload(np.zeros(s, np.float16)) for s in ((4, 8), (4, 8))]
    h32 = lib.f16_upload_f32(np.zeros((8, 4), np.float32))
    out = np.empty((2, 8), np.float32)
    try:
        rc = lib.dll.csk_dense_ffn_f16(hidden.ctypes.data, 2, 8, 4, h16[0], h16[1], h32, None, None, None,
                                       out.ctypes.data)
        assert rc == capi.ERR_ARG
        assert "weight tensors must all be FLOAT16 or all FLOAT32" in lib.dll.csk_last_error().decode()
    finally:
        for h in h16 + [h32]:
            lib.f16_free(h)


@pytest.mark.parametrize("M,K,N", [(1, 64, 96), (7, 37, 29), (64, 2880, 512), (65, 96, 160), (2, 5120, 1024)])
def test_matmul_transpose_float32_weight_matches_oracle(lib, oracle, M, K, N):
    """matmul_transpose_mixed_node's fp32 B (matmul_transpose_mixed_node.h:83-92)."""
    rng = np.random.default_rng([M, K, N, 32])
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    got = lib.matmul_transpose_f16(a, w)
    want = oracle.matmul_transpose_f32(a, w)
    assert got.shape == (M, N)
    assert_layer_close(got, want)
    ref = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()
    with pytest.raises(capi.CskError, match="incompatible dimensions"):
        lib.matmul_transpose_f16(a[:, :K - 1] if K > 1 else a, w)


@pytest.mark.parametrize("scale", [1e-6, 1e5, 3e-30, 1e30])
def test_float32_weights_of_any_magnitude(lib, oracle, scale):
    """fp32 weights far outside the fp16 range (matmul_transpose_mixed_node.h:83-92 and
    dense_ffn_node.h:102-113 take any fp32): the matrix travels as two fp16 terms of
    w / 2^s, 2^s chosen per matrix, so tiny and huge weights keep the same relative accuracy
    as weights of order one."""
    rng = np.random.default_rng(int(abs(np.log10(scale))))
    M, K, N = 9, 160, 96
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * scale).astype(np.float32)
    got = lib.matmul_transpose_f16(a, w)
    want = oracle.matmul_transpose_f32(a, w)
    ref = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()
    assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()
    if 1e-6 <= scale <= 1e5:
        # dense FFN: gate and up of one magnitude, down of its inverse, so the three scales differ
        T, H, F = 5, 64, 96
        hidden = rng.standard_normal((T, H)).astype(np.float32)
        w_gate = (rng.standard_normal((F, H)) * scale).astype(np.float32)
        w_up = (rng.standard_normal((F, H)) * 0.1).astype(np.float32)
        w_down = (rng.standard_normal((H, F)) / scale).astype(np.float32)
        got = lib.dense_ffn_f16(hidden, w_gate, w_up, w_down, None, None, None)
        want = oracle.dense_ffn_f32(hidden, w_gate, w_up, w_down, None, None, None)
        x = hidden.astype(np.float64)
        g = x @ w_gate.astype(np.float64).T
        u = x @ w_up.astype(np.float64).T
        with np.errstate(over="ignore"):
            ref = (g / (1 + np.exp(-g)) * u) @ w_down.astype(np.float64).T
        assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


def test_float32_weight_upload_refuses_non_finite_weights(lib):
    w = np.ones((4, 8), np.float32)
    w[2, 3] = 1e6   # beyond fp16 by itself: fine, the matrix is scaled
    lib.f16_free(lib.f16_upload_f32(w))
    for bad in (np.nan, np.inf, -np.inf):
        w[2, 3] = bad
        with pytest.raises(capi.CskError, match="holds a NaN or an infinity"):
            lib.f16_upload_f32(w)
