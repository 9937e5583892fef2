"""Parity of the conv-layer glue kernels (elementwise unary / binary, Repeat,
Sum, Fill), called through the C ABI, with the CPU oracle on the same inputs.

Bars: bit-exact where the arithmetic is exactly rounded on both sides
(+ - * / compares, abs neg square sqrt sign, Repeat, Fill); relative error
<= 2e-6 per element for the transcendental functions (device libm vs the
oracle's double-precision libm rounded to float); relative <= 1e-5 against a
float64 sum for Sum, whose fp32 summation order differs from the reference's
single running sum by design (and is tighter than it).
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

SIZES = [1, 7, 8, 2048, 2049, 100003, 1 << 22]


@pytest.fixture(scope="module")
def K():
    from cgt_amd import capi, kernels
    capi.require_gpu()
    return kernels


def gpu(a):
    from cgt_amd.gpuarray import to_gpu
    return to_gpu(a)


def bits_equal(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


EXACT_UNARY = ("abs", "neg", "square", "sqrt", "sign")


@pytest.mark.parametrize("op", O.UNARY_OPS)
def test_elwise_unary(K, op):
    rs = np.random.RandomState(0)
    for n in SIZES:
        x = (rs.randn(n) * 3).astype(np.float32)
        if op in ("log", "sqrt"):
            x = np.abs(x) + 1e-3
        x[: min(n, 3)] = [0.0, 1.0, 2.5][: min(n, 3)] if op not in ("log",) else [1.0, 1.0, 2.5][: min(n, 3)]
        got, ref = K.elwise_unary(op, gpu(x)).get(), O.elwise_unary(op, x)
        if op in EXACT_UNARY:
            assert bits_equal(got, ref), (op, n)
        else:
            np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-7, err_msg="%s n=%d" % (op, n))


@pytest.mark.parametrize("op", O.BINARY_OPS)
@pytest.mark.parametrize("mask", [(False, False), (True, False), (False, True)])
def test_elwise_binary_ff(K, op, mask):
    rs = np.random.RandomState(1)
    for n in SIZES:
        x = (rs.randn(n) * 3).astype(np.float32)
        y = (rs.randn(n) * 3).astype(np.float32)
        y[::5] = x[::5]
        if op == "**":
            x = np.abs(x) + 0.1
        if mask[0]:
            x = x[0].reshape(())
        if mask[1]:
            y = y[-1].reshape(())
        got, ref = K.elwise_binary(op, gpu(x), gpu(y)).get(), O.elwise_binary(op, x, y)
        if op == "**":
            assert got.dtype == ref.dtype
            np.testing.assert_allclose(got, ref, rtol=2e-6, err_msg="n=%d" % n)
        else:
            assert bits_equal(got, ref), (op, mask, n)


@pytest.mark.parametrize("op", ["*", "+", "-", "/", ">=", "=="])
def test_elwise_binary_mixed_types(K, op):
    rs = np.random.RandomState(2)
    for n in [5, 2048, 100003]:
        x = (rs.randn(n) * 3).astype(np.float32)
        b = rs.randint(0, 2, n).astype(np.int8)
        c = rs.randint(1, 3, n).astype(np.int8)
        for lhs, rhs in [(x, b + 1), (b + 1, x), (b, c), (x, np.int8(1).reshape(())), (np.int8(1).reshape(()), x)]:
            lhs, rhs = np.asarray(lhs), np.asarray(rhs)
            if lhs.dtype != np.float32:
                lhs = lhs.astype(np.int8)
            if rhs.dtype != np.float32:
                rhs = rhs.astype(np.int8)
            got, ref = K.elwise_binary(op, gpu(lhs), gpu(rhs)).get(), O.elwise_binary(op, lhs, rhs)
            assert bits_equal(got, ref), (op, n, lhs.dtype, rhs.dtype)


def test_rectify_and_gradient_composition(K):
    # nn.rectify = x * (x >= 0) (cgt/nn.py:44-45); its pullback multiplies the cotangent by the same mask
    rs = np.random.RandomState(3)
    x = rs.randn(64, 32, 15, 15).astype(np.float32)
    x[0, 0, 0, :5] = [0.0, -0.0, 1.0, -1.0, 0.0]
    zero = gpu(np.float32(0).reshape(()))
    xg = gpu(x)
    mask = K.elwise_binary(">=", xg, zero)
    y = K.elwise_binary("*", xg, mask)
    assert bits_equal(y.get(), O.rectify(x))
    g = rs.randn(*x.shape).astype(np.float32)
    gx = K.elwise_binary("*", mask, gpu(g))
    assert bits_equal(gx.get(), (x >= 0).astype(np.float32) * g)


def test_binary_shape_mismatch_raises(K):
    with pytest.raises(ValueError):
        K.elwise_binary("+", gpu(np.zeros((2, 3), np.float32)), gpu(np.zeros((3, 2), np.float32)))


REPEAT_CASES = [((1, 96, 1, 1), (0, 2, 3), (8, 55, 55)),      # bias over an AlexNet activation
                ((1, 128, 1, 1), (0, 2, 3), (4, 56, 56)),
                ((1, 5, 1, 1), (0, 2, 3), (3, 4, 2)),
                ((4, 1), (1,), (1000,)), ((1, 777), (0,), (33,)), ((1, 1), (0, 1), (300, 301)),
                ((2, 1, 3, 1, 2), (1, 3), (4, 5)),               # generic pattern
                ((3, 4), (), ()), ((5, 1, 7), (1,), (1,))]


@pytest.mark.parametrize("shape,axes,reps", REPEAT_CASES)
@pytest.mark.parametrize("dtype", [np.float32, np.int8])
def test_repeat(K, shape, axes, reps, dtype):
    rs = np.random.RandomState(4)
    x = (rs.randn(*shape) * 10).astype(dtype)
    assert bits_equal(K.repeat(gpu(x), axes, reps).get(), O.repeat(x, axes, reps))


SUM_CASES = [((8, 96, 55, 55), (0, 2, 3)),       # bias gradient
             ((4, 128, 56, 56), (0, 2, 3)),
             ((3, 5, 4, 2), (0, 2, 3)),
             ((64, 10), (0,)), ((64, 10), (1,)), ((1000, 333), (0,)), ((333, 1000), (1,)),
             ((8, 96, 55, 55), (0, 1, 2, 3)),     # scalar loss
             ((1 << 22,), (0,)), ((100003,), (0,)),
             ((2, 3, 4, 5, 2), (1, 3)),           # generic pattern
             ((6, 7), ()), ((2, 1, 3), (1,))]


@pytest.mark.parametrize("shape,axes", SUM_CASES)
def test_sum(K, shape, axes):
    rs = np.random.RandomState(5)
    x = rs.randn(*shape).astype(np.float32) + 0.25
    xg = gpu(x)
    got = K.sum_keepdims(xg, axes).get()
    ref64 = x.astype(np.float64).sum(axis=axes, keepdims=True) if axes else x.astype(np.float64)
    scale = np.abs(x.astype(np.float64)).sum(axis=axes, keepdims=True) if axes else np.abs(ref64)
    assert got.shape == ref64.shape
    assert np.all(np.abs(got - ref64) <= 1e-5 * scale + 1e-30)
    # the reference's own (sequential fp32) result is inside the same band around the exact sum
    seq = O.sum_keepdims(x, axes)
    n_red = max(x.size // max(got.size, 1), 1)
    assert np.all(np.abs(seq - ref64) <= n_red * 6e-8 * scale + 1e-30)
    # fixed order: a second launch gives the same bits
    assert bits_equal(K.sum_keepdims(xg, axes).get(), got)


def test_sum_empty_and_fill(K):
    from cgt_amd.gpuarray import empty
    out = K.sum_keepdims(empty((0, 5)), (0,)).get()
    assert out.shape == (1, 5) and np.array_equal(out, np.zeros((1, 5), np.float32))
    f = K.fill(2.5, (3, 1001)).get()
    assert np.array_equal(f, np.full((3, 1001), 2.5, np.float32))
