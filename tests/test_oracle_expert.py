"""Pins oracle expert MLP, merge, RMSNorm and add (oracle/moe_oracle.c) against
float64 evaluations over weights dequantised with the pinned codec, the
reference's activation known answer and structural properties."""
import numpy as np
import pytest

from coalsack_amd import synth


def modified_swiglu_ref(g, u):
    # test/test_expert_mlp.cpp:37-46
    x = np.minimum(g, 7.0)
    y = np.clip(u, -7.0, 7.0)
    return x / (1.0 + np.exp(1.702 * (-x))) * (y + 1.0)


def standard_swiglu_ref(g, u):
    return g / (1.0 + np.exp(-g)) * u


def mlp_f64(oracle, x, w_up, w_gate, w_down, b_up, b_gate, b_down, H, F, act=0):
    Wu = oracle.dequant(w_up, F * H).reshape(F, H).astype(np.float64)
    Wg = oracle.dequant(w_gate, F * H).reshape(F, H).astype(np.float64)
    Wd = oracle.dequant(w_down, H * F).reshape(H, F).astype(np.float64)
    x = x.astype(np.float64)
    up = Wu @ x + (0 if b_up is None else b_up)
    gate = Wg @ x + (0 if b_gate is None else b_gate)
    a = modified_swiglu_ref(gate, up) if act == 0 else standard_swiglu_ref(gate, up)
    return Wd @ a + (0 if b_down is None else b_down)


def const_matrix(rows, K, code_diag=None, scale=128):
    """All-zero MXFP4 matrix; code_diag puts that code on the diagonal."""
    nb = K // 32
    m = np.zeros((rows, nb, 17), np.uint8)
    m[:, :, 0] = scale
    if code_diag is not None:
        for r in range(min(rows, K)):
            blk, j = divmod(r, 32)
            if j < 16:
                m[r, blk, 1 + j] |= code_diag
            else:
                m[r, blk, 1 + j - 16] |= code_diag << 4
    return m.reshape(-1)


def test_activation_known_answer(oracle):
    """test/test_expert_mlp.cpp:118-200 recast for MXFP4: gate = 1.0 and up = 1.5
    through an identity down projection."""
    H = F = 32
    # gate/up weights zero, biases carry the pre-activations; down = identity (code 1 * 2^0)
    wz = const_matrix(F, H)
    wd = const_matrix(H, F, code_diag=1)
    x = np.ones(H, np.float32)
    out = oracle.expert_token(x, wz, wz, wd, np.full(F, 1.5, np.float32), np.full(F, 1.0, np.float32),
                              np.zeros(H, np.float32), H, F)
    want = modified_swiglu_ref(np.float64(1.0), np.float64(1.5))
    assert np.allclose(out, want, atol=1e-3)
    assert np.allclose(out, want, rtol=1e-6)



def test_activation_clipping_and_standard(oracle):
    H = F = 32
    wz = const_matrix(F, H)
    wd = const_matrix(H, F, code_diag=1)
    x = np.ones(H, np.float32)
    zeros = np.zeros(H, np.float32)
    for g, u in [(9.0, -9.0), (-3.0, 0.25), (7.0, 7.0), (0.0, 2.0)]:
        out = oracle.expert_token(x, wz, wz, wd, np.full(F, u, np.float32), np.full(F, g, np.float32),
                                  zeros, H, F, act=0)
        assert np.allclose(out, modified_swiglu_ref(np.float64(g), np.float64(u)), rtol=1e-6, atol=1e-7)
        out = oracle.expert_token(x, wz, wz, wd, np.full(F, u, np.float32), np.full(F, g, np.float32),
                                  zeros, H, F, act=1)
        assert np.allclose(out, standard_swiglu_ref(np.float64(g), np.float64(u)), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("H,F,bias,act", [(64, 96, True, 0), (256, 128, False, 0), (2880, 2880, True, 0),
                                          (128, 64, True, 1)])
def test_token_against_float64(oracle, H, F, bias, act):
    rng = np.random.default_rng(H + F)
    w_up = synth.mxfp4_blocks(1, 0, 0, 0, F, H)
    w_gate = synth.mxfp4_blocks(1, 0, 0, 1, F, H)
    w_down = synth.mxfp4_blocks(1, 0, 0, 2, H, F)
    x = rng.normal(0, 1, H).astype(np.float32)
    b_up = rng.normal(0, 0.01, F).astype(np.float32) if bias else None
    b_gate = rng.normal(0, 0.01, F).astype(np.float32) if bias else None
    b_down = rng.normal(0, 0.01, H).astype(np.float32) if bias else None
    got = oracle.expert_token(x, w_up, w_gate, w_down, b_up, b_gate, b_down, H, F, act)
    want = mlp_f64(oracle, x, w_up, w_gate, w_down, b_up, b_gate, b_down, H, F, act)
    assert np.max(np.abs(got - want)) <= 2e-5 * max(1.0, np.max(np.abs(want)))


def test_gate_and_up_are_not_swapped(oracle):
    """A transposed gate/up argument order changes the result: the modified
    activation is not symmetric."""
    H = F = 64
    rng = np.random.default_rng(0)
    w_up = synth.mxfp4_blocks(2, 0, 0, 0, F, H)
    w_gate = synth.mxfp4_blocks(2, 0, 0, 1, F, H)
    w_down = synth.mxfp4_blocks(2, 0, 0, 2, H, F)
    x = rng.normal(0, 4, H).astype(np.float32)
    a = oracle.expert_token(x, w_up, w_gate, w_down, None, None, None, H, F)
    b = oracle.expert_token(x, w_gate, w_up, w_down, None, None, None, H, F)
    assert not np.allclose(a, b)
    assert np.allclose(a, mlp_f64(oracle, x, w_up, w_gate, w_down, None, None, None, H, F), atol=1e-4)


def test_expert_node_rows_and_empty(oracle):
    """expert_mlp_node.h:441-443, 509-512: {0} tensor when no token selects the
    expert; zero rows for tokens that did not; selected rows equal the
    single-token computation."""
    H, F, T, k = 64, 64, 5, 2
    rng = np.random.default_rng(1)
    w = [synth.mxfp4_blocks(3, 0, 4, i, F if i < 2 else H, H if i < 2 else F) for i in range(3)]
    hidden = rng.normal(0, 1, (T, H)).astype(np.float32)
    pairs = np.zeros((T, k, 2), np.float32)
    pairs[:, 0, 0], pairs[:, 1, 0] = [4, 1, 2, 4, 0], [0, 4, 3, 2, 1]
    pairs[..., 1] = rng.uniform(0.1, 0.9, (T, k))
    assert oracle.expert_mlp(7, hidden, F, *w, None, None, None, pairs) is None
    out = oracle.expert_mlp(4, hidden, F, *w, None, None, None, pairs)
    for t in range(T):
        if 4 in pairs[t, :, 0]:
            assert np.array_equal(out[t], oracle.expert_token(hidden[t], *w, None, None, None, H, F))
        else:
            assert np.all(out[t] == 0)
    # weight_before_ffn scales the input by the routing weight (:515-522)
    outw = oracle.expert_mlp(4, hidden, F, *w, None, None, None, pairs, weight_before_ffn=True)
    wt = pairs[0, 0, 1]
    assert np.array_equal(outw[0], oracle.expert_token(hidden[0] * wt, *w, None, None, None, H, F))


def test_merge_definition_and_special_cases(oracle):
    T, k, E, H = 6, 2, 4, 16
    rng = np.random.default_rng(2)
    outs = [rng.normal(0, 1, (T, H)).astype(np.float32) for _ in range(E)]
    pairs = np.zeros((T, k, 2), np.float32)
    for t in range(T):
        pairs[t, :, 0] = rng.choice(E, k, replace=False)
    pairs[..., 1] = rng.uniform(0, 1, (T, k))
    rc, got = oracle.expert_merge(pairs, outs, H)
    assert rc == 0
    want = np.zeros((T, H))
    for t in range(T):
        for s in range(k):
            want[t] += np.float64(pairs[t, s, 1]) * outs[int(pairs[t, s, 0])][t]
    assert np.allclose(got, want, atol=1e-6)
    # one-hot weights reduce to a copy
    p1 = pairs.copy()
    p1[:, 0, 1], p1[:, 1, 1] = 1.0, 0.0
    rc, got = oracle.expert_merge(p1, outs, H)
    for t in range(T):
        assert np.array_equal(got[t], outs[int(p1[t, 0, 0])][t])
    # pre-weighted: plain sum (expert_merge_node.h:119-123)
    rc, got = oracle.expert_merge(pairs, outs, H, pre_weighted=True)
    for t in range(T):
        assert np.array_equal(got[t], (0 + outs[int(pairs[t, 0, 0])][t]) + outs[int(pairs[t, 1, 0])][t])
    # empty experts are skipped (:111-113); all empty is an error (:60-62); bad index (:102-105)
    e_empty = int(pairs[0, 0, 0])
    outs2 = list(outs)
    outs2[e_empty] = None
    rc, got = oracle.expert_merge(pairs, outs2, H)
    assert rc == 0
    assert np.allclose(got[0], pairs[0, 1, 1] * outs[int(pairs[0, 1, 0])][0], atol=1e-7)
    rc, _ = oracle.expert_merge(pairs, [None] * E, H)
    assert rc == 3
    bad = pairs.copy()
    bad[0, 0, 0] = E
    rc, _ = oracle.expert_merge(bad, outs, H)
    assert rc == 2


def test_rmsnorm_known_answers(oracle):
    # test/test_rmsnorm.cpp:74-115 and :118-142
    x = np.array([[1, 2, 3, 4]], np.float32)
    w = np.array([2, 0.5, 1.5, 1], np.float32)
    rms = np.sqrt(np.float32(30.0) / np.float32(4.0))
    assert np.allclose(oracle.rmsnorm(x, w, 0.0), x / rms * w, atol=1e-5)
    assert np.allclose(oracle.rmsnorm(np.array([[5.0]], np.float32), np.array([2.0], np.float32), 0.0), 2.0, atol=1e-5)
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (3, 2880)).astype(np.float32)
    w = rng.normal(1, 0.02, 2880).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-5) * w
    assert np.allclose(oracle.rmsnorm(x, w, 1e-5), want, atol=1e-5)
    assert np.array_equal(oracle.add(x, x), x + x)


def test_rmsnorm_f64_pinned(oracle):
    """rmsnorm_node.h:49-50 / :62-83 with T = double.  Known answers in double; rows on which
    every operation is exact or a single correctly rounded one (so Python's own IEEE double
    arithmetic states the answer without restating the loop); the sum of squares against
    math.fsum; exact scale covariance; agreement with the float32 function."""
    import math
    # test_rmsnorm.cpp:118-142 and :74-115 in double
    assert oracle.rmsnorm_f64(np.array([[5.0]]), np.array([2.0]), 0.0)[0, 0] == 2.0
    x = np.array([[1.0, 2.0, 3.0, 4.0]])
    w = np.array([2.0, 0.5, 1.5, 1.0])
    rms = math.sqrt(30.0 / 4.0)  # 30 and 7.5 are exact; one rounding in the root
    assert np.array_equal(oracle.rmsnorm_f64(x, w, 0.0), np.array([[(v / rms) * g for v, g in zip(x[0], w)]]))
    # rows of +-c: sum of squares H c^2 exact for small integers, mean = c^2 exact, eps widened from float
    for c, H in ((3.0, 8), (0.5, 64), (7.0, 2880)):
        eps = float(np.float32(1e-5))
        row = np.array([[c if j % 2 == 0 else -c for j in range(H)]])
        wv = np.linspace(0.5, 1.5, H)
        r = math.sqrt(c * c + eps)
        want = np.array([[(v / r) * g for v, g in zip(row[0], wv)]])
        assert np.array_equal(oracle.rmsnorm_f64(row, wv, 1e-5), want)
    # a dropped term, a wrong divisor or a float accumulator would show here
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, (4, 2880))
    w = rng.normal(1, 0.02, 2880)
    got = oracle.rmsnorm_f64(x, w, 1e-5)
    for i in range(4):
        ss = math.fsum(float(v) * float(v) for v in x[i])  # (rounded products, exactly summed)
        r = math.sqrt(ss / 2880 + float(np.float32(1e-5)))
        want = x[i] / r * w
        assert np.max(np.abs(got[i] - want) / np.abs(want)) < 1e-13  # sequential vs compensated sum: a few ulp
    # eps = 0: scaling the row by a power of two changes nothing (every operation scales exactly)
    a = oracle.rmsnorm_f64(x, w, 0.0)
    assert np.array_equal(oracle.rmsnorm_f64(x * 1024.0, w, 0.0), a)
    assert np.array_equal(oracle.rmsnorm_f64(x, w * 0.25, 0.0), a * 0.25)
    # against the float32 function on float32 data
    xf, wf = x.astype(np.float32), w.astype(np.float32)
    assert np.allclose(oracle.rmsnorm_f64(xf, wf, 1e-5), oracle.rmsnorm(xf, wf, 1e-5), rtol=2e-6, atol=1e-6)


def test_layer_composition_equals_node_chain(oracle):
    """orc_moe_layer (token-by-token evaluation) is bit-identical to the node
    chain the reference wires: router -> E expert nodes -> merge."""
    E, k, H, F, T = 6, 2, 64, 96, 7
    L = synth.LayerInputs(E, k, H, F, seed=11)
    hidden = synth.hidden_states(T, H, seed=5)
    wu = np.concatenate([L.blocks(e, 0) for e in range(E)])
    wg = np.concatenate([L.blocks(e, 1) for e in range(E)])
    wd = np.concatenate([L.blocks(e, 2) for e in range(E)])
    for wbf in (False, True):
        out, pairs = oracle.moe_layer(hidden, E, k, H, F, L.gate_w, L.gate_b, wu, wg, wd, L.b_up,
                                      L.b_gate, L.b_down, weight_before_ffn=wbf)
        assert np.array_equal(pairs, oracle.router(hidden, L.gate_w, L.gate_b, k))
        outs = [oracle.expert_mlp(e, hidden, F, L.blocks(e, 0), L.blocks(e, 1), L.blocks(e, 2),
                                  L.b_up[e], L.b_gate[e], L.b_down[e], pairs, weight_before_ffn=wbf)
                for e in range(E)]
        rc, want = oracle.expert_merge(pairs, outs, H, pre_weighted=wbf)
        assert rc == 0
        assert np.array_equal(out, want)
    # norm + residual wiring (llm_engine.cpp:714-777): h + moe(rmsnorm(h))
    norm_w = np.linspace(0.9, 1.1, H).astype(np.float32)
    out, _ = oracle.moe_layer(hidden, E, k, H, F, L.gate_w, L.gate_b, wu, wg, wd, L.b_up, L.b_gate,
                              L.b_down, norm_w=norm_w, norm_eps=1e-5, residual=True)
    xn = oracle.rmsnorm(hidden, norm_w, 1e-5)
    inner, _ = oracle.moe_layer(xn, E, k, H, F, L.gate_w, L.gate_b, wu, wg, wd, L.b_up, L.b_gate, L.b_down)
    assert np.array_equal(out, oracle.add(hidden, inner))
