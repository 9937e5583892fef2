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
        f(x0[0], fl)                                    # wrong rank
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


def test_function_is_shape_generic(cgt):
    # compiled at batch 4, called at batch 7 and at batch 4 again: extents that depend on the
    # argument are recomputed by Size / integer-op instructions, Alloc follows them
    # (src/execution.cpp:251-264), and every output has the bits of a fresh evaluation
    from cgt_amd import nn
    rs = np.random.RandomState(5)
    w = (rs.randn(16, 8, 3, 3) / 8).astype(np.float32)
    b = (0.1 * rs.randn(1, 16, 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(8, 16, (3, 3), (1, 1), weight_init=w, bias_init=b)

    def graph(xn):
        act = nn.rectify(layer(xn))
        act = nn.cross_channel_lrn(act, 5, 1e-3, 0.75)
        pooled = nn.max_pool_2d(act, (3, 3), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
        return [pooled, loss, gx, gw, gb]

    x4 = rs.randn(4, 8, 17, 17).astype(np.float32)
    xn = cgt.constant(x4)
    f = cgt.function([xn], graph(xn), device_outputs=True)
    assert f.shape_generic and f.n_shape_instructions > 0
    ptrs = {}
    for batch in (4, 7, 4, 4, 2):
        xb = rs.randn(batch, 8, 17, 17).astype(np.float32)
        got = f(xb)
        want = graph(cgt.constant(xb))
        for g, node in zip(got, want):
            assert g.shape == node.shape
            assert np.array_equal(g.get().view(np.uint32), node.get().view(np.uint32)), batch
        ptrs.setdefault(batch, []).append([g.ptr for g in got])
    # the buffers that grew for batch 7 serve the smaller batches after it: no new allocation
    assert ptrs[4][1] == ptrs[7][0] and ptrs[4][2] == ptrs[7][0] and ptrs[2][0] == ptrs[7][0]
    # spatial extents are symbolic too
    xs = rs.randn(3, 8, 21, 13).astype(np.float32)
    for g, node in zip(f(xs), graph(cgt.constant(xs))):
        assert np.array_equal(g.get().view(np.uint32), node.get().view(np.uint32))


def test_extents_used_as_values_follow_the_call_shapes(cgt):
    # the reference's cgt.size is a symbolic scalar, so sum(x) / size(x, 0), x * x.shape[1] and
    # mean() are right at any shape (cgt/core.py:1614-1640); here an extent that depends on an
    # argument enters a value through ExtentAsFloat, which a compiled function re-evaluates per call
    from cgt_amd import core
    x0 = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    xn = cgt.constant(x0)

    def graph(xn):
        return [cgt.mean(xn * xn), cgt.sum(xn) / cgt.size(xn, 0), xn * xn.shape[1],
                (cgt.size(xn, 0) * cgt.size(xn, 2) - 1) * cgt.sum(xn, axis=0), cgt.mean(xn, axis=(0, 2))]

    f = cgt.function([xn], graph(xn))
    assert f.shape_generic
    assert any(isinstance(n.op, core.ExtentAsFloat) for n in f._order)
    rs = np.random.RandomState(3)
    for shape in [(2, 3, 4), (5, 3, 4), (1, 7, 2), (2, 3, 4)]:
        xv = rs.randn(*shape).astype(np.float32)
        got = f(xv)
        want = graph(cgt.constant(xv))                    # node-by-node evaluation at this shape
        ref = [np.mean(xv.astype(np.float64) ** 2), xv.sum(dtype=np.float64) / shape[0], xv * shape[1],
               (shape[0] * shape[2] - 1) * xv.sum(axis=0, dtype=np.float64), xv.mean(axis=(0, 2), dtype=np.float64)]
        for g, w, r in zip(got, want, ref):
            assert np.array_equal(np.asarray(g).view(np.uint32), w.get().view(np.uint32)), shape
            assert np.allclose(np.asarray(g), r, rtol=1e-5, atol=1e-5), shape
    # an extent of a weight (not an argument) is a constant
    wn = cgt.constant(np.ones((3, 4), np.float32))
    g = cgt.function([xn], cgt.sum(xn * 2.0) * cgt.mean(wn))
    assert g.shape_generic
    assert abs(float(g(x0[:1])) - 2 * x0[:1].sum()) <= 1e-3


def test_function_with_a_baked_extent_keeps_the_traced_shapes(cgt):
    # a value computed outside the graph from an extent (a node flagged shape_baked) cannot follow
    # the call's shapes: such a function refuses other shapes instead of using the wrong count
    from cgt_amd import core
    x0 = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    xn = cgt.constant(x0)
    n = cgt.size(xn, 0) * cgt.size(xn, 1)
    divisor = cgt.constant(np.float32(1.0 / n))
    divisor.shape_baked, divisor.baked_expr = True, core.ShapeInt._lift(n).expr
    f = cgt.function([xn], cgt.sum(xn) * divisor)
    assert not f.shape_generic
    assert abs(float(f(x0)) - x0.sum() / 6) <= 1e-4 * x0.sum()
    with pytest.raises(ValueError):
        f(x0[:1])


def test_function_transports_follow_the_gpu_deref_mask(cgt):
    # conv2d + bias + grad built from HOST leaves: the placement rule (reference
    # cgt/compilation.py:45-80, 285-304, with the gpu_deref_mask of core.py:748 honoured) puts
    # one Transport in front of x and one in front of W; Col2Im's four int64 scalars, the
    # Reshape operands and Repeat's counts are read in place on the host
    from cgt_amd import core, nn, rt
    rs = np.random.RandomState(6)
    x0 = rs.randn(3, 4, 9, 9).astype(np.float32)
    w0 = (rs.randn(6, 4, 3, 3) / 6).astype(np.float32)
    b0 = (0.1 * rs.randn(1, 6, 1, 1)).astype(np.float32)

    def graph(xn, wn, bn):
        y = core.broadcast("+", nn.conv2d(xn, wn, (3, 3), (1, 1)), bn, "xxxx,1x11")
        gy = cgt.constant(np.cos(np.arange(y.get().size, dtype=np.float32)).reshape(y.get().shape))
        gx, gw, gb = cgt.grad(y, [xn, wn, bn], goutput=gy)
        return [y, gx, gw, gb]

    xh, wh = cgt.constant(x0, devtype="cpu"), cgt.constant(w0, devtype="cpu")
    bn = cgt.constant(b0)
    assert xh.devtype == "cpu" and wh.devtype == "cpu"
    outs_h = graph(xh, wh, bn)
    outs_d = graph(cgt.constant(x0), cgt.constant(w0), bn)
    for a, b in zip(outs_h, outs_d):                     # node by node: same bits as the all-device graph
        assert np.array_equal(a.get().view(np.uint32), b.get().view(np.uint32))
    # the gradient of a host leaf comes back to the host (the pullback of a Transport is the
    # reverse Transport); y and the bias gradient stay on the device
    assert [o.devtype for o in outs_h] == ["gpu", "cpu", "cpu", "gpu"]
    f = cgt.function([xh, wh], outs_h)
    assert f.n_transports == 4 and f.n_arg_transports == 0
    steps = f.plan_steps()
    transports = [s for s in steps if s[0] == "byref" and s[4] == "transport"]
    assert sorted((s[2][0][1], s[3][1]) for s in transports) == [(rt.CPU, rt.GPU)] * 2 + [(rt.GPU, rt.CPU)] * 2
    seen = set()
    for s in steps:
        if s[0] != "byref" or s[4] != "op":
            continue
        name = s[1].op_str
        devs = [loc[1] for loc in s[2]]
        if name.startswith("Col2Im"):
            assert devs == [rt.GPU] + [rt.CPU] * 4
            seen.add("col2im")
        elif name.startswith("Repeat"):
            assert devs[0] == rt.GPU and all(d == rt.CPU for d in devs[1:])
            seen.add("repeat")
        else:
            assert all(d == rt.GPU for d in devs), name
    assert seen == {"col2im", "repeat"}
    x1 = rs.randn(*x0.shape).astype(np.float32)
    want = graph(cgt.constant(x1), cgt.constant(w0), bn)
    for got, node in zip(f(x1, w0), want):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    # an input that lives on the device may be handed over as a device array (no copy) or as a
    # numpy array: LoadArgument + an argument transport inside the instruction list make the
    # copy, not python, and both ways share the function's buffers
    xd, wd = cgt.constant(x0), cgt.constant(w0)
    fd = cgt.function([xd, wd], graph(xd, wd, bn), device_outputs=True)
    assert fd.n_transports == 0 and fd.n_arg_transports == 2
    got_h = fd(x1, w0)
    ptrs = [g.ptr for g in got_h]
    for got, node in zip(got_h, want):
        assert np.array_equal(got.get().view(np.uint32), node.get().view(np.uint32))
    x1_dev = cgt.to_gpu(x1 * 0.5)
    got_d = fd(x1_dev, w0)
    assert [g.ptr for g in got_d] == ptrs
    want_half = graph(cgt.constant(x1 * 0.5), cgt.constant(w0), bn)
    for got, node in zip(got_d, want_half):
        assert np.array_equal(got.get().view(np.uint32), node.get().view(np.uint32))
    assert np.array_equal(x1_dev.get(), x1 * 0.5)        # the caller's device array is only read
    for got, node in zip(fd(x1, w0), want):               # host again: the staging buffer, not the caller's array
        assert np.array_equal(got.get().view(np.uint32), node.get().view(np.uint32))
    assert np.array_equal(x1_dev.get(), x1 * 0.5)


def test_function_momentum_updates_read_the_new_value(cgt):
    # v := 0.9 v - lr g ; p := p + v_new.  The second update reads the NEW velocity, and the
    # function also returns an expression of the updated parameter: every reader of an update's
    # right-hand side must see the new value, every reader of the parameter the old one
    rs = np.random.RandomState(7)
    x = rs.randn(5, 6).astype(np.float32)
    p0 = rs.randn(6, 3).astype(np.float32)
    v0 = (0.1 * rs.randn(6, 3)).astype(np.float32)
    lr, mu = 0.05, 0.9
    xn = cgt.constant(x)
    p, v = cgt.constant(p0), cgt.constant(v0)
    y = cgt.dot(xn, p)
    loss = cgt.sum(y * y)
    g, = cgt.grad(loss, [p])
    v_new = v * mu - g * lr
    p_new = p + v_new
    probe = cgt.sum(p_new * p_new)               # an output computed from the updated parameter
    step = cgt.function([xn], [loss, probe], updates=[(v, v_new), (p, p_new)])
    pptr, vptr = p.value.ptr, v.value.ptr
    p64, v64, x64 = p0.astype(np.float64), v0.astype(np.float64), x.astype(np.float64)
    for _ in range(4):
        got_loss, got_probe = step(x)
        y64 = x64 @ p64
        g64 = 2 * x64.T @ y64
        v64 = mu * v64 - lr * g64
        want_loss = (y64 * y64).sum()
        p64 = p64 + v64
        assert abs(float(got_loss) - want_loss) <= 1e-4 * want_loss
        assert abs(float(got_probe) - (p64 * p64).sum()) <= 1e-4 * (p64 * p64).sum()
        assert np.linalg.norm(p.get() - p64) <= 1e-4 * np.linalg.norm(p64)
        assert np.linalg.norm(v.get() - v64) <= 1e-4 * np.linalg.norm(v64)
    assert (p.value.ptr, v.value.ptr) == (pptr, vptr)
    kinds = [s[4] for s in step.plan_steps() if s[0] == "byref"]
    assert kinds[-1] == "update-copy" or kinds[-2] == "update-copy"
    # two parameters whose updates read each other's OLD value
    a, b = cgt.constant(np.float32([[1.0, 2.0]])), cgt.constant(np.float32([[10.0, 20.0]]))
    swap = cgt.function([], [], updates=[(a, b * 1.0), (b, a * 1.0)])
    swap()
    assert np.array_equal(a.get(), [[10.0, 20.0]]) and np.array_equal(b.get(), [[1.0, 2.0]])


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


def test_kept_device_outputs_survive_a_later_call_that_needs_larger_buffers(cgt):
    # device_outputs=True hands out the interpreter's own buffers.  A later call at a larger shape
    # makes the interpreter drop those buffers for larger ones; an output kept from the earlier
    # call holds a reference on its buffer (a view holds one on the buffer it shows), so it still
    # reads the values of its call
    from cgt_amd import nn
    rs = np.random.RandomState(12)
    w = (rs.randn(16, 16, 3, 3) / 12).astype(np.float32)
    wn = cgt.constant(w)

    def graph(xn):
        y = nn.conv2d(xn, wn, (3, 3), pad=(1, 1))
        return [y, cgt.reshape(y * 2.0, [cgt.size(y, 0), cgt.size(y, 1) * cgt.size(y, 2) * cgt.size(y, 3)])]

    x_small = rs.randn(2, 16, 9, 9).astype(np.float32)
    xn = cgt.constant(x_small)
    f = cgt.function([xn], graph(xn), device_outputs=True)
    kept = f(x_small)
    want = [g.get().copy() for g in kept]
    ptr_small = kept[0].ptr
    for batch in (5, 9, 33):                       # each call outgrows the buffers of the one before
        big = f(rs.randn(batch, 16, 9, 9).astype(np.float32))
        assert big[0].shape[0] == batch
    assert big[0].ptr != ptr_small
    # allocate and scribble: freed memory would be handed out again
    from cgt_amd.gpuarray import to_gpu
    junk = [to_gpu(np.full(want[0].shape, 7.0, np.float32)) for _ in range(8)]
    for g, w_ in zip(kept, want):
        assert np.array_equal(g.get().view(np.uint32), w_.view(np.uint32))
    del junk, kept, big
    # a smaller call after the growth is a view of the large buffer; keeping it keeps that buffer
    small_again = f(x_small)
    del f
    assert np.array_equal(small_again[0].get().view(np.uint32), want[0].view(np.uint32))
