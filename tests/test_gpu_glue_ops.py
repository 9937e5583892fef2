"""The conv-layer glue through the Op API: ElwiseUnary / ElwiseBinary / Repeat /
Sum / Fill closures fired on device arrays, `broadcast`, `sum`, `rectify`,
`SpatialConvolution`, and `grad` through all of them from a scalar cost -- one
SpatialConvolution + ReLU + max-pool training step checked against a float64
restatement built from the oracle's pieces.
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-4


@pytest.fixture(scope="module")
def cgt():
    import cgt_amd
    from cgt_amd import capi
    capi.require_gpu()
    return cgt_amd


def relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


def test_operators_and_types(cgt):
    rs = np.random.RandomState(0)
    x, y = rs.randn(3, 50).astype(np.float32), rs.randn(3, 50).astype(np.float32)
    xn, yn = cgt.constant(x), cgt.constant(y)
    assert np.array_equal((xn + yn).get(), x + y)
    assert np.array_equal((xn - yn).get(), x - y)
    assert np.array_equal((xn * yn).get(), x * y)
    assert np.array_equal((xn / yn).get(), x / y)
    assert np.array_equal((xn * 2.0).get(), x * np.float32(2))
    assert np.array_equal((1 - xn).get(), np.float32(1) - x)
    assert np.array_equal((-xn).get(), -x)
    m = xn >= 0
    assert m.dtype == "i1" and np.array_equal(m.get(), (x >= 0).astype(np.int8))
    assert (xn * m).dtype == "f4"
    with pytest.raises(ValueError):
        xn + cgt.constant(np.zeros((50, 3), np.float32))


@pytest.mark.parametrize("opname", ["abs", "cos", "exp", "log", "sin", "square", "sqrt", "tanh", "sigmoid"])
def test_unary_grad_matches_finite_difference(cgt, opname):
    rs = np.random.RandomState(1)
    x = (np.abs(rs.randn(4, 33)) + 0.5).astype(np.float32)
    f = getattr(cgt, opname)
    xn = cgt.constant(x)
    yn = f(xn)
    np.testing.assert_allclose(yn.get(), O.elwise_unary(opname, x), rtol=2e-6, atol=1e-7)
    g = rs.randn(*x.shape).astype(np.float32)
    (gx,) = cgt.grad(yn, [xn], goutput=g)
    eps = 1e-3
    x64 = x.astype(np.float64)
    ref = {"abs": np.abs, "cos": np.cos, "exp": np.exp, "log": np.log, "sin": np.sin, "square": np.square,
           "sqrt": np.sqrt, "tanh": np.tanh, "sigmoid": lambda v: 1 / (1 + np.exp(-v))}[opname]
    fd = (ref(x64 + eps) - ref(x64 - eps)) / (2 * eps) * g
    assert relfro(gx.get(), fd) <= 1e-4


def test_broadcast_sum_mean(cgt):
    rs = np.random.RandomState(2)
    x = rs.randn(4, 6, 5, 7).astype(np.float32)
    b = rs.randn(1, 6, 1, 1).astype(np.float32)
    xn, bn = cgt.constant(x), cgt.constant(b)
    z = cgt.broadcast("+", xn, bn, "xxxx,1x11")
    assert np.array_equal(z.get(), x + b)
    z2 = cgt.broadcast("*", bn, xn, "1x11,xxxx")
    assert np.array_equal(z2.get(), b * x)
    s = cgt.sum(xn, axis=(0, 2, 3), keepdims=True)
    assert s.shape == (1, 6, 1, 1) and relfro(s.get(), x.astype(np.float64).sum((0, 2, 3), keepdims=True)) <= 1e-6
    s = cgt.sum(xn, axis=1)
    assert s.shape == (4, 5, 7) and relfro(s.get(), x.astype(np.float64).sum(1)) <= 1e-6
    tot = cgt.sum(xn)
    assert tot.shape == () and abs(float(tot.get()) - x.astype(np.float64).sum()) <= 1e-4
    mu = cgt.mean(xn, axis=(0, 2, 3), keepdims=True)
    assert relfro(mu.get(), x.astype(np.float64).mean((0, 2, 3), keepdims=True)) <= 1e-6
    # pullbacks: Repeat <-> Sum
    g = rs.randn(*x.shape).astype(np.float32)
    gx, gb = cgt.grad(z, [xn, bn], goutput=g)
    assert np.array_equal(gx.get(), g)
    assert gb.shape == b.shape and relfro(gb.get(), g.astype(np.float64).sum((0, 2, 3), keepdims=True)) <= 1e-6
    (gx,) = cgt.grad(cgt.sum(xn * xn), [xn])
    assert relfro(gx.get(), 2.0 * x) <= 1e-6
    assert np.array_equal(cgt.fill(3.0, [2, 5]).get(), np.full((2, 5), 3.0, np.float32))
    assert np.array_equal(cgt.zeros_like(xn).get(), np.zeros_like(x))


def test_rectify_forward_backward(cgt):
    from cgt_amd import nn
    rs = np.random.RandomState(3)
    x = rs.randn(8, 16, 9, 9).astype(np.float32)
    x[0, 0, 0, :3] = [0.0, -0.0, -1.0]
    xn = cgt.constant(x)
    y = nn.rectify(xn)
    assert np.array_equal(y.get().view(np.uint32), O.rectify(x).view(np.uint32))
    g = rs.randn(*x.shape).astype(np.float32)
    (gx,) = cgt.grad(y, [xn], goutput=g)
    assert np.array_equal(gx.get(), g * (x >= 0))


def _layer_reference(x, w, b, pad, stride, pool):
    """float64 restatement of SpatialConvolution -> rectify -> max_pool -> sum and its gradients."""
    x, w, b = x.astype(np.float64), w.astype(np.float64), b.astype(np.float64)
    conv = O.conv2d(x, w, pad, stride)
    pre = conv + b
    act = pre * (pre >= 0)
    pooled, mask = O.max_pool(act, *pool)
    loss = pooled.sum()
    gact = O.max_pool_pullback(act.shape, mask, np.ones_like(pooled))
    gpre = gact * (pre >= 0)
    gb = gpre.sum((0, 2, 3), keepdims=True)
    gx, gw = O.conv2d_pullback(x, w, gpre, pad, stride)
    return loss, act, gx, gw, gb


@pytest.mark.parametrize("case", [
    dict(x=(4, 3, 20, 20), L=8, k=(5, 5), pad=(2, 2), stride=(1, 1), pool=((3, 3), (0, 0), (2, 2))),
    dict(x=(3, 16, 14, 14), L=24, k=(3, 3), pad=(1, 1), stride=(1, 1), pool=((2, 2), (0, 0), (2, 2))),
    dict(x=(2, 3, 43, 43), L=12, k=(11, 11), pad=(0, 0), stride=(4, 4), pool=((3, 3), (0, 0), (2, 2))),
])
def test_spatial_convolution_training_step(cgt, case):
    from cgt_amd import nn
    rs = np.random.RandomState(4)
    x = rs.randn(*case["x"]).astype(np.float32)
    C = case["x"][1]
    w = (rs.randn(case["L"], C, *case["k"]) / np.sqrt(C * case["k"][0] * case["k"][1])).astype(np.float32)
    b = (0.1 * rs.randn(1, case["L"], 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(C, case["L"], case["k"], case["pad"], case["stride"], weight_init=w, bias_init=b)
    xn = cgt.constant(x)
    act = nn.rectify(layer(xn))
    pooled = nn.max_pool_2d(act, *case["pool"])
    loss = cgt.sum(pooled)
    gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
    rloss, ract, rgx, rgw, rgb = _layer_reference(x, w, b, case["pad"], case["stride"], case["pool"])
    assert relfro(act.get(), ract) <= TOL
    assert abs(float(loss.get()) - rloss) <= TOL * abs(rloss)
    assert gb.shape == b.shape
    assert relfro(gx.get(), rgx) <= TOL and relfro(gw.get(), rgw) <= TOL and relfro(gb.get(), rgb) <= TOL
