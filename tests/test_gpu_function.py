"""`cgt.function`: a traced graph replayed by the C++ interpreter (LoadArgument /
Alloc / BuildTup / ReturnByRef / ReturnByVal) gives the same bits as evaluating
the nodes one by one from python, for new argument values, with weights bound by
reference and output buffers reused between calls."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cgt():
    import cgt_amd
    from cgt_amd import capi
    capi.require_gpu()
    return cgt_amd


def _graph(cgt, nn, xn, layer):
    act = nn.rectify(layer(xn))
    act = nn.cross_channel_lrn(act, 5, 1e-3, 0.75)
    pooled = nn.max_pool_2d(act, (3, 3), (0, 0), (2, 2))
    loss = cgt.sum(pooled * pooled)
    gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
    return pooled, loss, gx, gw, gb


def test_function_replays_training_step(cgt):
    from cgt_amd import nn
    rs = np.random.RandomState(0)
    x0 = rs.randn(4, 8, 17, 17).astype(np.float32)
    w = (rs.randn(16, 8, 3, 3) / 8).astype(np.float32)
    b = (0.1 * rs.randn(1, 16, 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(8, 16, (3, 3), (1, 1), weight_init=w, bias_init=b)
    xn = cgt.constant(x0)
    outs = _graph(cgt, nn, xn, layer)
    f = cgt.function([xn], list(outs))
    assert f.n_instructions > 40
    # same argument: same bits as the node-by-node evaluation
    for got, node in zip(f(x0), outs):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    # new argument values: compare with a fresh node-by-node evaluation
    x1 = rs.randn(*x0.shape).astype(np.float32)
    fresh = _graph(cgt, nn, cgt.constant(x1), layer)
    for got, node in zip(f(x1), fresh):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    # weights are bound by reference: an in-place update is seen by the next call
    w2 = (w * 0.5).astype(np.float32)
    layer.weight.value.set(w2)
    fresh = _graph(cgt, nn, cgt.constant(x1), layer)
    for got, node in zip(f(x1), fresh):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    # and the whole thing agrees with the oracle's pieces in float64
    conv = O.conv2d(x1.astype(np.float64), w2.astype(np.float64), (1, 1), (1, 1)) + b
    act = conv * (conv >= 0)
    top, _ = O.lrn_fwd(act, 5, 1e-3, 0.75)
    pooled, _ = O.max_pool(top, (3, 3), (0, 0), (2, 2))
    assert abs(float(f(x1)[1]) - (pooled ** 2).sum()) <= 1e-4 * (pooled ** 2).sum()


def test_function_device_outputs_reuse_buffers_and_check_shapes(cgt):
    from cgt_amd import nn
    rs = np.random.RandomState(1)
    x0 = rs.randn(2, 3, 12, 12).astype(np.float32)
    fl = rs.randn(5, 3, 3, 3).astype(np.float32)
    xn, fn = cgt.constant(x0), cgt.constant(fl)
    y = nn.conv2d(xn, fn, (3, 3), (1, 1))
    pool, = [nn.max_pool_2d(y, (2, 2), (0, 0), (2, 2))]
    f = cgt.function([xn, fn], [y, pool], device_outputs=True)
    y1, p1 = f(x0, fl)
    ptrs = (y1.ptr, p1.ptr)
    assert np.array_equal(y1.get(), y.get()) and np.array_equal(p1.get(), pool.get())
    y2, p2 = f(cgt.to_gpu(x0 * 2), fl)                  # device array argument: no copy
    assert (y2.ptr, p2.ptr) == ptrs
    assert np.allclose(y2.get(), 2 * y.get(), rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError):
        f(x0[:1], fl)
    with pytest.raises(TypeError):
        f(x0)
    single = cgt.function([xn, fn], y)
    assert isinstance(single(x0, fl), np.ndarray)


def test_function_dispatch_is_cheaper_than_node_by_node(cgt):
    # many tiny ops: the interpreter's per-instruction cost against python's per-node cost
    import time
    from cgt_amd import capi
    x0 = np.linspace(-1, 1, 256, dtype=np.float32).reshape(16, 16)
    xn = cgt.constant(x0)

    def chain(x):
        y = x
        for _ in range(50):
            y = cgt.tanh(y * 1.01 + 0.001)
        return y
    y = chain(xn)
    f = cgt.function([xn], y, device_outputs=True)
    xg = cgt.to_gpu(x0)
    f(xg)
    capi.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        f(xg)
    capi.synchronize()
    t_fn = (time.perf_counter() - t0) / 20
    t0 = time.perf_counter()
    for _ in range(5):
        chain(cgt.constant(xg))
    capi.synchronize()
    t_py = (time.perf_counter() - t0) / 5
    print("150 ops: compiled function %.3f ms, node by node %.3f ms" % (t_fn * 1e3, t_py * 1e3))
    assert np.array_equal(f(xg).get(), y.get())
    assert t_fn < t_py


def test_function_with_sgd_updates_trains_in_place(cgt):
    # loss = sum((pool(relu(conv(x) + b)))^2); five SGD steps on W and b through one compiled
    # function against the same steps in float64 built from the oracle's pieces
    from cgt_amd import nn
    rs = np.random.RandomState(2)
    x = rs.randn(4, 3, 12, 12).astype(np.float32)
    w = (rs.randn(6, 3, 3, 3) / 5).astype(np.float32)
    b = (0.1 * rs.randn(1, 6, 1, 1)).astype(np.float32)
    lr = 1e-3
    layer = nn.SpatialConvolution(3, 6, (3, 3), (1, 1), weight_init=w, bias_init=b)
    xn = cgt.constant(x)
    pooled = nn.max_pool_2d(nn.rectify(layer(xn)), (2, 2), (0, 0), (2, 2))
    loss = cgt.sum(pooled * pooled)
    params = [layer.weight, layer.bias]
    step = cgt.function([xn], loss, updates=nn.sgd(loss, params, lr))
    wptr = layer.weight.value.ptr

    w64, b64, x64 = w.astype(np.float64), b.astype(np.float64), x.astype(np.float64)
    losses, ref_losses = [], []
    for _ in range(5):
        losses.append(float(step(x)))
        pre = O.conv2d(x64, w64, (1, 1), (1, 1)) + b64
        act = pre * (pre >= 0)
        p, mask = O.max_pool(act, (2, 2), (0, 0), (2, 2))
        ref_losses.append(float((p * p).sum()))
        gact = O.max_pool_pullback(act.shape, mask, 2 * p)
        gpre = gact * (pre >= 0)
        _, gw = O.conv2d_pullback(x64, w64, gpre, (1, 1), (1, 1))
        w64 = w64 - lr * gw
        b64 = b64 - lr * gpre.sum((0, 2, 3), keepdims=True)
    assert layer.weight.value.ptr == wptr                       # updated in place
    assert np.allclose(losses, ref_losses, rtol=1e-4)
    assert losses[-1] < losses[0]
    assert np.linalg.norm(layer.weight.get() - w64) <= 1e-4 * np.linalg.norm(w64)
    assert np.linalg.norm(layer.bias.get() - b64) <= 1e-4 * np.linalg.norm(b64)


def test_function_as_hip_graph_matches_eager_on_every_replay(cgt):
    # an MNIST-sized block (launch-bound: a dozen kernels of a few microseconds) recorded into a
    # HIP graph; several replays with other work and synchronisations in between, each checked
    import time
    from cgt_amd import capi, nn
    rs = np.random.RandomState(3)
    xs = [rs.randn(64, 1, 28, 28).astype(np.float32) for _ in range(4)]
    w = (0.1 * rs.randn(32, 1, 3, 3)).astype(np.float32)
    layer = nn.SpatialConvolution(1, 32, (3, 3), (1, 1), weight_init=w)

    def build(xn):
        pooled = nn.max_pool_2d(nn.rectify(layer(xn)), (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gw, gb = cgt.grad(loss, [layer.weight, layer.bias])
        return pooled, loss, gw, gb
    xn = cgt.constant(xs[0])
    outs = build(xn)
    plain = cgt.function([xn], list(outs))
    graph = cgt.function([xn], list(outs), use_graph=True)
    for rep in range(6):
        x = xs[rep % len(xs)]
        want = plain(x)
        other = (cgt.constant(x) * 2.0).get()              # unrelated eager work between replays
        capi.synchronize()
        got = graph(x)
        for g, wnt in zip(got, want):
            assert np.array_equal(g.view(np.uint32), wnt.view(np.uint32)), rep
        assert np.array_equal(other, x * 2)
    # one launch per call instead of one per kernel (informational: on this stack a replay takes as
    # long as the interpreter's own asynchronous launches)
    xg = cgt.to_gpu(xs[1])
    plain_dev = cgt.function([xn], list(outs), device_outputs=True)
    graph_dev = cgt.function([xn], list(outs), device_outputs=True, use_graph=True)
    plain_dev(xg), graph_dev(xg), graph_dev(xg)

    def timeit(f, n=50):
        capi.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            f(xg)
        capi.synchronize()
        return (time.perf_counter() - t0) / n * 1e3
    t_plain, t_graph = timeit(plain_dev), timeit(graph_dev)
    print("MNIST block fwd+bwd: interpreter %.3f ms/call, HIP graph %.3f ms/call (%d instructions)"
          % (t_plain, t_graph, plain.n_instructions))
    for a, b in zip(graph_dev(xg), plain_dev(xg)):
        assert np.array_equal(a.get(), b.get())
