"""Pins the oracle's conv-layer glue (elementwise ops, Repeat, Sum) against
numpy -- the library routine each reduces to -- and against brute force where
the reference's native template departs from numpy (sign(0), sequential fp32
summation order)."""
import numpy as np
import pytest

from oracle import oracle as O


def _x(n=1000, seed=0):
    rs = np.random.RandomState(seed)
    return (rs.randn(n) * 2).astype(np.float32)


NP_UNARY = {"abs": np.abs, "cos": np.cos, "exp": np.exp, "log": np.log, "neg": np.negative, "sin": np.sin,
            "square": np.square, "sqrt": np.sqrt, "tanh": np.tanh, "sigmoid": lambda v: 1.0 / (1.0 + np.exp(-v))}


@pytest.mark.parametrize("op", sorted(NP_UNARY))
def test_unary_vs_numpy(op):
    x = _x()
    if op in ("log", "sqrt"):
        x = np.abs(x) + 0.01
    ref = NP_UNARY[op](x.astype(np.float64)).astype(np.float32)     # double math, rounded once: the C template's path
    got = O.elwise_unary(op, x)
    if op in ("abs", "neg", "square", "sqrt"):
        assert np.array_equal(got, ref)
    else:
        np.testing.assert_allclose(got, ref, rtol=2e-7, atol=0)


def test_sign_follows_native_template():
    # 2*(x>0)-1 (cgt/core.py:1127): -1 at zero, where numpy's sign gives 0
    x = np.array([-2.5, -0.0, 0.0, 1e-30, 3.0], np.float32)
    assert np.array_equal(O.elwise_unary("sign", x), np.array([-1, -1, -1, 1, 1], np.float32))


NP_BINARY = {"*": np.multiply, "+": np.add, "-": np.subtract, "/": np.divide, "<": np.less, ">": np.greater,
             "<=": np.less_equal, ">=": np.greater_equal, "==": np.equal, "!=": np.not_equal}


@pytest.mark.parametrize("op", sorted(NP_BINARY))
@pytest.mark.parametrize("mask", [(False, False), (True, False), (False, True)])
def test_binary_ff_vs_numpy(op, mask):
    x, y = _x(seed=1), _x(seed=2)
    y[::7] = x[::7]                     # ties for the comparisons
    if mask[0]:
        x = x[3].reshape(())
    if mask[1]:
        y = y[5].reshape(())
    got = O.elwise_binary(op, x, y)
    ref = NP_BINARY[op](x, y)
    assert got.dtype == (np.int8 if ref.dtype == bool else np.float32)
    assert np.array_equal(got, ref.astype(got.dtype))


def test_binary_pow():
    x, y = np.abs(_x(seed=3)) + 0.1, _x(seed=4)
    np.testing.assert_allclose(O.elwise_binary("**", x, y), np.power(x.astype(np.float64), y.astype(np.float64)),
                               rtol=2e-7)


def test_binary_mixed_types_promote():
    x = _x(seed=5)
    m = (x >= 0).astype(np.int8)
    assert np.array_equal(O.elwise_binary("*", x, m), x * m)                  # relu = x * (x >= 0)
    assert np.array_equal(O.elwise_binary("*", m, x), m * x)
    assert O.elwise_binary("*", m, m).dtype == np.int8
    assert np.array_equal(O.elwise_binary("+", m, m), (m + m).astype(np.int8))
    d = O.elwise_binary("/", m, (m + 1).astype(np.int8))                      # "/" always gives floatX
    assert d.dtype == np.float32 and np.array_equal(d, (m / (m + 1.0)).astype(np.float32))
    assert np.array_equal(O.elwise_binary(">=", x, np.float32(0).reshape(())), m)


@pytest.mark.parametrize("shape,axes,reps", [((1, 5, 1, 1), (0, 2, 3), (3, 4, 2)), ((4, 1), (1,), (6,)),
                                             ((1, 6), (0,), (5,)), ((2, 1, 3, 1, 2), (1, 3), (4, 5)),
                                             ((1, 1), (0, 1), (3, 2)), ((3, 4), (), ())])
def test_repeat_vs_numpy(shape, axes, reps):
    rs = np.random.RandomState(6)
    for dtype in (np.float32, np.int8):
        x = (rs.randn(*shape) * 10).astype(dtype)
        oshape = list(shape)
        for a, r in zip(axes, reps):
            oshape[a] = r
        assert np.array_equal(O.repeat(x, axes, reps), np.broadcast_to(x, oshape))


@pytest.mark.parametrize("shape,axes", [((3, 5, 4, 2), (0, 2, 3)), ((7, 9), (0,)), ((7, 9), (1,)), ((7, 9), (0, 1)),
                                        ((2, 3, 4, 5, 2), (1, 3)), ((6,), ()), ((2, 1, 3), (1,))])
def test_sum_vs_numpy_and_bruteforce(shape, axes):
    rs = np.random.RandomState(7)
    x64 = rs.randn(*shape)
    ref = x64.sum(axis=axes, keepdims=True) if axes else x64
    np.testing.assert_allclose(O.sum_keepdims(x64, axes), ref, rtol=1e-12, atol=1e-12)
    # float32: one running sum per output cell, input walked in row-major order
    x = x64.astype(np.float32)
    out = np.zeros([1 if a in axes else s for a, s in enumerate(shape)], np.float32)
    for idx in np.ndindex(*shape):
        o = tuple(0 if a in axes else i for a, i in enumerate(idx))
        out[o] = np.float32(out[o] + x[idx])
    assert np.array_equal(O.sum_keepdims(x, axes), out)


def test_sum_order_is_sequential():
    # (1e8 + 1) - 1e8 in fp32 is 0; any pairing that adds 1e8 and -1e8 first gives 1
    x = np.array([1e8, 1.0, -1e8], np.float32)
    assert O.sum_keepdims(x, (0,))[0] == 0.0
    x = np.array([1e8, -1e8, 1.0], np.float32)
    assert O.sum_keepdims(x, (0,))[0] == 1.0
