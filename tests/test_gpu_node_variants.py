"""GPU parity of the node branches beside the main path: the float64 router and the
broadcasting add, through the C ABI, bit-exact against the oracle."""
import numpy as np
import pytest

from coalsack_amd import capi

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("sigmoid", [False, True])
@pytest.mark.parametrize("T,H,E,k,bias", [(1, 64, 32, 4, True), (16, 2880, 128, 4, True), (5, 96, 7, 3, False),
                                          (3, 5, 4, 4, True), (130, 37, 70, 9, True), (4, 33, 300, 20, False)])
def test_router_float64_bit_exact(lib, oracle, T, H, E, k, bias, sigmoid):
    """moe_router_node.h:115-118: logits are the sequential float64 sums bit for bit, so the
    selected experts are the oracle's without any near-tie allowance."""
    rng = np.random.default_rng([T, H, E, k])
    h = rng.standard_normal((T, H))
    g = rng.standard_normal((E, H)) * 0.02
    b = (rng.standard_normal(E) * 0.01).astype(np.float32) if bias else None
    got, logits = lib.moe_router_f64(h, g, b, k, sigmoid=sigmoid, want_logits=True)
    want, want_logits = oracle.router_f64(h, g, b, k, sigmoid=sigmoid, want_logits=True)
    assert np.array_equal(logits, want_logits)
    assert np.array_equal(got[..., 0], want[..., 0])
    assert np.allclose(got[..., 1], want[..., 1], rtol=1e-6, atol=1e-7)


def test_router_float64_ties_and_known_answer(lib, oracle):
    for E in (8, 32, 128):
        out = lib.moe_router_f64(np.zeros((2, 16)), np.ones((E, 16)), None, 4)
        assert out[0, :, 0].astype(int).tolist() == [1, 3, 0, 2]
        assert np.array_equal(out[..., 1], np.full((2, 4), 0.25, np.float32))
    # ties between some experts only: duplicate gate rows
    rng = np.random.default_rng(3)
    g = rng.standard_normal((16, 24))
    g[5] = g[2]
    g[11] = g[2]
    g[9] = g[4]
    h = rng.standard_normal((40, 24))
    assert np.array_equal(lib.moe_router_f64(h, g, None, 6)[..., 0], oracle.router_f64(h, g, None, 6)[..., 0])
    # test/test_moe_router.cpp:82-138 in float64
    H, E, k = 4, 6, 3
    out = lib.moe_router_f64(np.ones((1, H)), np.repeat((np.arange(E) / H)[:, None], H, axis=1), np.zeros(E, np.float32), k)
    assert out[0, :, 0].astype(int).tolist() == [5, 4, 3]
    with pytest.raises(capi.CskError):
        lib.moe_router_f64(np.ones((1, 4)), np.ones((2, 4)), None, 3)


def test_router_float64_many_tokens(lib, oracle):
    rng = np.random.default_rng(9)
    h = rng.standard_normal((20000, 32))
    g = rng.standard_normal((8, 32))
    got = lib.moe_router_f64(h, g, None, 2)
    want = oracle.router_f64(h, g, None, 2)
    assert np.array_equal(got[..., 0], want[..., 0])
    assert np.allclose(got[..., 1], want[..., 1], rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_add_broadcast_bit_exact(lib, oracle, dtype):
    """add_node.h:16-50 through elementwise_helpers.h:9-66, every element type."""
    rng = np.random.default_rng(7)

    def rand(shape):
        if np.issubdtype(dtype, np.integer):
            info = np.iinfo(dtype)
            return rng.integers(info.min, info.max, shape, dtype=dtype, endpoint=True)
        return rng.standard_normal(shape).astype(dtype)
    for sa, sb in [((4, 5), (4, 5)), ((4, 5), (5,)), ((5,), (4, 5)), ((4, 1), (1, 5)), ((2, 3, 4), (3, 1)),
                   ((2, 1, 4), (1, 3, 1)), ((), (3,)), ((3,), ()), ((1,), (1,)), ((1, 2, 3, 4, 5), (4, 1)),
                   ((7,), (1, 1, 1, 7)), ((3, 1, 2880), (1, 17, 2880)), ((1000, 1), (1, 777)),
                   ((2, 1, 2, 1, 2, 1, 2, 1), (1, 3, 1, 3, 1, 3, 1, 3))]:
        a, b = rand(sa), rand(sb)
        got = lib.add_broadcast(a, b)
        want = oracle.add_broadcast(a, b)
        assert got.shape == want.shape and got.dtype == want.dtype
        assert np.array_equal(got, want)
    # a zero-sized dimension gives an empty result, not an error
    assert lib.add_broadcast(rand((2, 0, 3)), rand((1, 3))).shape == (2, 0, 3)


def test_add_broadcast_errors_carry_the_reference_text(lib):
    a, b = np.zeros((4, 5), np.float32), np.zeros((4,), np.float32)
    with pytest.raises(capi.CskError, match=r"Broadcast failed: Shape A=\[4,5\], Shape B=\[4\]"):
        lib.add_broadcast(a, b)
    with pytest.raises(capi.CskError, match=r"Broadcast failed: Shape A=\[2,3,4\], Shape B=\[2,4\]"):
        lib.add_broadcast(np.zeros((2, 3, 4), np.int64), np.zeros((2, 4), np.int64))
    with pytest.raises(capi.CskError, match="more than 8 dimensions"):
        lib.add_broadcast(np.zeros((1,) * 9, np.float32), np.zeros((1,), np.float32))
