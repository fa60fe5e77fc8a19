"""Pins the oracle's fp16 expert path (oracle/moe_oracle.c: orc_expert_token_f16,
orc_expert_mlp_f16, fp16 weights in orc_moe_layer) against the reference's known answer,
float64 evaluations, and the already pinned MXFP4 functions on weights both formats hold
exactly."""
import numpy as np
import pytest

from coalsack_amd import synth
from tests.test_oracle_expert import modified_swiglu_ref, standard_swiglu_ref


def mlp_f64(x, w_up, w_gate, w_down, b_up, b_gate, b_down, act=0):
    x = x.astype(np.float64)
    up = w_up.astype(np.float64) @ x + (0 if b_up is None else b_up)
    gate = w_gate.astype(np.float64) @ x + (0 if b_gate is None else b_gate)
    a = modified_swiglu_ref(gate, up) if act == 0 else standard_swiglu_ref(gate, up)
    return w_down.astype(np.float64) @ a + (0 if b_down is None else b_down)


def random_f16_expert(rng, H, F, scale=0.05):
    return ((rng.standard_normal((F, H)) * scale).astype(np.float16),
            (rng.standard_normal((F, H)) * scale).astype(np.float16),
            (rng.standard_normal((H, F)) * scale).astype(np.float16))


def test_reference_known_answer_two_by_two(oracle):
    # test/test_expert_mlp.cpp:118-200: hidden_dim = expert_ffn_dim = 2, every element goes
    # through the scalar remainder loop; gate = 1, up = 1.5, w_down flat indices 0 and 2 set
    x = np.array([1.0, 0.5], np.float32)
    w_up = np.zeros((2, 2), np.float16)
    w_gate = np.zeros((2, 2), np.float16)
    w_down = np.zeros((2, 2), np.float16)
    w_up[0, 0] = 1.0
    w_gate[0, 0] = 1.0
    w_down.reshape(-1)[0] = 1.0
    w_down.reshape(-1)[2] = 1.0
    b_up = np.array([0.5, 0.0], np.float32)
    zero = np.zeros(2, np.float32)
    out = oracle.expert_token_f16(x, w_up, w_gate, w_down, b_up, zero, zero, act=0)
    want = modified_swiglu_ref(1.0, 1.5)
    assert abs(out[0] - want) < 1e-6
    assert abs(out[1] - want) < 1e-6  # flat index 2 is w_down[1][0]


@pytest.mark.parametrize("H,F", [(8, 8), (37, 29), (64, 96), (250, 130)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("act", [0, 1])
def test_token_against_float64(oracle, H, F, bias, act):
    rng = np.random.default_rng([H, F, act, bias])
    x = rng.standard_normal(H).astype(np.float32)
    w_up, w_gate, w_down = random_f16_expert(rng, H, F, 0.2)
    b = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)] if bias else [None] * 3
    got = oracle.expert_token_f16(x, w_up, w_gate, w_down, *b, act=act)
    want = mlp_f64(x, w_up, w_gate, w_down, *b, act=act)
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


def test_gate_and_up_are_not_swapped(oracle):
    rng = np.random.default_rng(5)
    H = F = 16
    x = rng.standard_normal(H).astype(np.float32)
    w_up, w_gate, w_down = random_f16_expert(rng, H, F, 0.5)
    a = oracle.expert_token_f16(x, w_up, w_gate, w_down, None, None, None, act=0)
    b = oracle.expert_token_f16(x, w_gate, w_up, w_down, None, None, None, act=0)
    assert np.abs(a - b).max() > 1e-3


def test_bit_identical_to_mxfp4_path_on_shared_weights(oracle):
    """Every MXFP4 value with a moderate scale is an fp16 value, and the two reference loops
    put element i of a row into accumulator lane i % 8 in the same order
    (expert_mlp_node.h:551-572 and :259-266), so on such weights the two oracle functions
    must agree to the last bit."""
    H, F = 96, 64
    blocks = [synth.mxfp4_blocks(11, 0, 0, w, *((H, F) if w == 2 else (F, H))) for w in range(3)]
    deq = [oracle.dequant(blocks[w], F * H).reshape((H, F) if w == 2 else (F, H)) for w in range(3)]
    halves = [d.astype(np.float16) for d in deq]
    for d, h in zip(deq, halves):
        assert np.array_equal(h.astype(np.float32), d)
    rng = np.random.default_rng(3)
    x = rng.standard_normal(H).astype(np.float32)
    b = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)]
    for act in (0, 1):
        a = oracle.expert_token(x, blocks[0], blocks[1], blocks[2], *b, H, F, act)
        c = oracle.expert_token_f16(x, halves[0], halves[1], halves[2], *b, act=act)
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32))


def test_expert_node_rows_and_empty(oracle):
    rng = np.random.default_rng(8)
    T, H, F, k = 6, 40, 24, 2
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    w = random_f16_expert(rng, H, F, 0.2)
    pairs = np.zeros((T, k, 2), np.float32)
    pairs[:, 0, 0] = [3, 1, 3, 0, 2, 3]
    pairs[:, 1, 0] = [1, 0, 2, 1, 0, 1]
    pairs[:, 0, 1] = 0.75
    pairs[:, 1, 1] = 0.25
    out = oracle.expert_mlp_f16(3, hidden, *w, None, None, None, pairs)
    for t in range(T):
        if t in (0, 2, 5):
            want = oracle.expert_token_f16(hidden[t], *w, None, None, None)
            assert np.array_equal(out[t], want)
        else:
            assert not out[t].any()
    assert oracle.expert_mlp_f16(7, hidden, *w, None, None, None, pairs) is None
    # weight_before_ffn scales the token by its routing weight first (:766-772)
    out_w = oracle.expert_mlp_f16(3, hidden, *w, None, None, None, pairs, weight_before_ffn=True)
    want = oracle.expert_token_f16(hidden[0] * np.float32(0.75), *w, None, None, None)
    assert np.array_equal(out_w[0], want)


def test_layer_with_fp16_experts_equals_node_chain(oracle):
    rng = np.random.default_rng(21)
    E, k, H, F, T = 6, 2, 64, 32, 9
    L = synth.LayerInputs(E, k, H, F, seed=5)
    hidden = synth.hidden_states(T, H)
    ws = [random_f16_expert(rng, H, F, 0.2) for _ in range(E)]
    w_up = np.stack([w[0] for w in ws])
    w_gate = np.stack([w[1] for w in ws])
    w_down = np.stack([w[2] for w in ws])
    out, pairs = oracle.moe_layer(hidden, E, k, H, F, L.gate_w, L.gate_b, w_up, w_gate, w_down,
                                  L.b_up, L.b_gate, L.b_down)
    assert np.array_equal(pairs, oracle.router(hidden, L.gate_w, L.gate_b, k))
    outs = [oracle.expert_mlp_f16(e, hidden, *ws[e], L.b_up[e], L.b_gate[e], L.b_down[e], pairs)
            for e in range(E)]
    rc, merged = oracle.expert_merge(pairs, outs, H)
    assert rc == 0
    assert np.array_equal(out, merged)


@pytest.mark.parametrize("T,H,F", [(1, 8, 8), (5, 37, 29), (3, 64, 96)])
@pytest.mark.parametrize("bias", [False, True])
def test_dense_ffn_against_float64(oracle, T, H, F, bias):
    """dense_ffn_node.h:163-218: every token, standard SwiGLU, weight order gate, up, down."""
    rng = np.random.default_rng([T, H, F, bias])
    hidden = rng.standard_normal((T, H)).astype(np.float32)
    w_up, w_gate, w_down = random_f16_expert(rng, H, F, 0.2)
    b = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)] if bias else [None] * 3
    got = oracle.dense_ffn_f16(hidden, w_gate, w_up, w_down, *b)
    for t in range(T):
        want = mlp_f64(hidden[t], w_up, w_gate, w_down, b[1], b[0], b[2], act=1)
        assert np.abs(got[t] - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
        assert np.array_equal(got[t], oracle.expert_token_f16(hidden[t], w_up, w_gate, w_down, b[1], b[0], b[2], act=1))


@pytest.mark.parametrize("M,K,N", [(1, 8, 4), (3, 37, 5), (5, 64, 7), (2, 24, 9), (4, 100, 16)])
def test_matmul_transpose_against_float64(oracle, M, K, N):
    """matmul_transpose_mixed_node.h:198-308 with a float16 weight: both column paths (tiles of
    four, remainder columns) and every K remainder."""
    rng = np.random.default_rng([M, K, N])
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.3).astype(np.float16)
    got = oracle.matmul_transpose_f16(a, w)
    want = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - want).max() <= 2e-6 * np.sqrt(K) * max(1.0, np.abs(want).max())
    eye = np.eye(N, K, dtype=np.float16)
    assert np.array_equal(oracle.matmul_transpose_f16(a, eye), a[:, :N] if N <= K else np.pad(a, ((0, 0), (0, N - K))))
