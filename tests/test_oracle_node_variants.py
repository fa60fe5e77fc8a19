"""Pins the oracle's restatements of the node branches beside the main path: fp32-weight
matmul / dense FFN, batched matmul, broadcasting add and the float64 router."""
import math

import numpy as np
import pytest


@pytest.mark.parametrize("M,K,N", [(1, 64, 96), (7, 37, 29), (3, 16, 4), (5, 8, 7), (2, 1, 1), (4, 50, 9)])
def test_matmul_f32_against_float64_and_f16_twin(oracle, M, K, N):
    """matmul_transpose_mixed_node.h:116-196: tiles of four columns and remainder columns, K in
    steps of 16, 8 and 1."""
    rng = np.random.default_rng([M, K, N])
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    got = oracle.matmul_transpose_f32(a, w)
    ref = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - ref).max() <= 1e-6 * max(1.0, np.abs(ref).max()) * math.sqrt(K)
    # weights that fp16 holds exactly: the fp32 function and the fp16 one run the same sums
    w16 = w.astype(np.float16)
    assert np.array_equal(oracle.matmul_transpose_f32(a, w16.astype(np.float32)), oracle.matmul_transpose_f16(a, w16))
    # a one-hot weight row copies a column of A exactly
    eye = np.zeros((N, K), np.float32)
    for j in range(min(N, K)):
        eye[j, j] = 1
    assert np.array_equal(oracle.matmul_transpose_f32(a, eye)[:, :min(N, K)], a[:, :min(N, K)])


@pytest.mark.parametrize("b_dtype", [np.float16, np.float32])
def test_matmul_batched_follows_numpy_where_modulus_and_broadcast_agree(oracle, b_dtype):
    rng = np.random.default_rng(5)
    for sa, sb in [((3, 4, 16), (5, 16)), ((2, 3, 4, 16), (5, 16)), ((3, 4, 16), (3, 5, 16)), ((4, 16), (3, 5, 16)),
                   ((2, 3, 4, 16), (3, 5, 16)), ((1, 4, 16), (6, 5, 16))]:
        a = rng.standard_normal(sa).astype(np.float32)
        b = (rng.standard_normal(sb) * 0.1).astype(b_dtype)
        got = oracle.matmul_transpose_batched(a, b)
        ref = a.astype(np.float64) @ np.swapaxes(b.astype(np.float64), -1, -2)
        assert got.shape == ref.shape
        assert np.abs(got - ref).max() <= 1e-5
        # and each matrix is the 2-D function of its operands
        a3, b3 = a.reshape(-1, 4, 16), b.reshape(-1, 5, 16)
        g3 = got.reshape(-1, 4, 5)
        two_d = oracle.matmul_transpose_f16 if b_dtype == np.float16 else oracle.matmul_transpose_f32
        for i in range(g3.shape[0]):
            assert np.array_equal(g3[i], two_d(a3[i % a3.shape[0]], b3[i % b3.shape[0]]))


def test_matmul_batched_modulus_rule_where_it_differs_from_broadcasting(oracle):
    """A [2,1,M,K] with B [1,3,N,K]: the node pairs output matrix i with A[i % 2] and B[i % 3]
    (matmul_transpose_mixed_node.h:76-78), not with A[i // 3]."""
    rng = np.random.default_rng(6)
    a = rng.standard_normal((2, 1, 2, 8)).astype(np.float32)
    b = rng.standard_normal((1, 3, 3, 8)).astype(np.float32)
    got = oracle.matmul_transpose_batched(a, b).reshape(6, 2, 3)
    for i in range(6):
        assert np.array_equal(got[i], oracle.matmul_transpose_f32(a.reshape(2, 2, 8)[i % 2], b.reshape(3, 3, 8)[i % 3]))


@pytest.mark.parametrize("T,H,F", [(1, 8, 6), (3, 37, 29), (2, 64, 96)])
@pytest.mark.parametrize("bias", [False, True])
def test_dense_ffn_f32_against_sequential_float32_and_float64(oracle, T, H, F, bias):
    """dense_ffn_node.h:122-153: scalar loops, every product and sum rounded on its own."""
    rng = np.random.default_rng([T, H, F, bias])
    x = rng.standard_normal((T, H)).astype(np.float32)
    wg, wu = [(rng.standard_normal((F, H)) * 0.2).astype(np.float32) for _ in range(2)]
    wd = (rng.standard_normal((H, F)) * 0.2).astype(np.float32)
    b = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in (F, F, H)] if bias else [None] * 3
    got = oracle.dense_ffn_f32(x, wg, wu, wd, *b)

    f32 = np.float32
    def seq_dot(u, v):
        s = f32(0)
        for p in (u * v):  # float32 products, rounded
            s = f32(s + p)
        return s
    want = np.empty((T, H), np.float32)
    for t in range(T):
        act = np.empty(F, np.float32)
        for o in range(F):
            g, u = seq_dot(x[t], wg[o]), seq_dot(x[t], wu[o])
            if bias:
                g, u = f32(g + b[0][o]), f32(u + b[1][o])
            act[o] = f32(g / f32(f32(1) + np.exp(f32(-g), dtype=np.float32))) * u
        for o in range(H):
            s = seq_dot(act, wd[o])
            want[t, o] = f32(s + b[2][o]) if bias else s
    # expf may differ from numpy's by an ulp; everything else is the same arithmetic
    assert np.allclose(got, want, rtol=2e-6, atol=2e-6)
    x64 = x.astype(np.float64)
    g = x64 @ wg.astype(np.float64).T + (b[0] if bias else 0)
    u = x64 @ wu.astype(np.float64).T + (b[1] if bias else 0)
    ref = (g / (1 + np.exp(-g)) * u) @ wd.astype(np.float64).T + (b[2] if bias else 0)
    assert np.abs(got - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_add_broadcast_is_numpys(oracle, dtype):
    rng = np.random.default_rng(7)
    def rand(shape):
        if np.issubdtype(dtype, np.integer):
            info = np.iinfo(dtype)
            return rng.integers(info.min, info.max, shape, dtype=dtype, endpoint=True)
        return rng.standard_normal(shape).astype(dtype)
    for sa, sb in [((4, 5), (4, 5)), ((4, 5), (5,)), ((5,), (4, 5)), ((4, 1), (1, 5)), ((2, 3, 4), (3, 1)),
                   ((2, 1, 4), (1, 3, 1)), ((), (3,)), ((3,), ()), ((1,), (1,)), ((2, 0, 3), (1, 3)),
                   ((0,), (1,)), ((1, 2, 3, 4, 5), (4, 1)), ((7,), (1, 1, 1, 7))]:
        a, b = rand(sa), rand(sb)
        got = oracle.add_broadcast(a, b)
        with np.errstate(over="ignore"):
            want = a + b
        assert got.shape == want.shape and got.dtype == want.dtype
        assert np.array_equal(got, want)
    for sa, sb in [((4, 5), (4,)), ((2, 3), (3, 2)), ((2, 3, 4), (2, 4))]:
        assert oracle.add_broadcast(rand(sa), rand(sb)) is None


def test_router_f64_known_answer_and_ties(oracle):
    # test/test_moe_router.cpp:82-138 widened to float64
    H, E, k = 4, 6, 3
    h = np.ones((1, H))
    g = np.repeat((np.arange(E) / H)[:, None], H, axis=1)
    out = oracle.router_f64(h, g, np.zeros(E, np.float32), k)
    assert out.dtype == np.float32 and out[0, :, 0].astype(int).tolist() == [5, 4, 3]
    ex = np.exp(np.array([0.0, -1.0, -2.0]))
    assert np.allclose(out[0, :, 1], ex / ex.sum(), atol=1e-6)
    # all-equal logits: the same libstdc++ order as the float32 instantiation
    for E in (8, 32, 128):
        o32 = oracle.router(np.zeros((1, 16), np.float32), np.ones((E, 16), np.float32), None, 4)
        o64 = oracle.router_f64(np.zeros((1, 16)), np.ones((E, 16)), None, 4)
        assert np.array_equal(o32, o64) and o64[0, :, 0].astype(int).tolist() == [1, 3, 0, 2]


@pytest.mark.parametrize("sigmoid", [False, True])
def test_router_f64_against_exact_sums(oracle, sigmoid):
    rng = np.random.default_rng(11)
    for (T, H, E, k, bias) in [(16, 64, 32, 4, True), (6, 2880, 128, 4, True), (5, 96, 7, 3, False), (3, 5, 4, 4, True)]:
        h = rng.standard_normal((T, H))
        g = rng.standard_normal((E, H)) * 0.02
        b = (rng.standard_normal(E) * 0.01).astype(np.float32) if bias else None
        out, logits = oracle.router_f64(h, g, b, k, sigmoid=sigmoid, want_logits=True)
        exact = np.array([[math.fsum(h[t] * g[e]) + (float(b[e]) if bias else 0.0) for e in range(E)] for t in range(T)])
        assert np.abs(logits - exact).max() <= 1e-12
        # the first few logits follow the sequential rule exactly
        for t, e in [(0, 0), (T - 1, E - 1)]:
            s = 0.0
            for d in range(H):
                s += h[t, d] * g[e, d]
            assert logits[t, e] == s + (float(b[e]) if bias else 0.0)
        order = np.argsort(-logits, axis=1, kind="stable")[:, :k]
        assert np.array_equal(out[..., 0].astype(int), order)
        top = np.take_along_axis(logits, order, axis=1)
        if sigmoid:
            w = 1 / (1 + np.exp(-top))
        else:
            ex = np.exp(top - top.max(axis=1, keepdims=True))
            w = ex / ex.sum(axis=1, keepdims=True)
        assert np.allclose(out[..., 1], w, atol=2e-6)
