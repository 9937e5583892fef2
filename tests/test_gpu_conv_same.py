"""conv2d without a column buffer (stride 1, pad = (kernel - 1) / 2): forward, data
gradient and weight gradient read the image operand from a zero-padded copy.  They must
compute what the reference's composition im2col -> Mul22 -> transpose computes
(cgt/nn.py:95-100) and what its autodiff derives for the gradients: compared here with
the float64 oracle chain at 1e-4 relative Frobenius error, and bit for bit where the
operation is a copy (the padding) or the same fp32 operations (fused bias add + rectify).
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-4


@pytest.fixture(scope="module")
def K():
    from cgt_amd import capi, kernels
    capi.require_gpu()
    return kernels


def relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def _padded_reference(x, kernel, total):
    B, C, H, W = x.shape
    ph, pw = (kernel[0] - 1) // 2, (kernel[1] - 1) // 2
    # a plane: pw zeros, then H + 2 ph rows of W + pw floats (W pixels, pw zeros)
    Hp, Wp = H + 2 * ph, W + pw
    plane = (pw + Hp * Wp + 16 + 15) // 16 * 16
    ref = np.zeros(total, np.float32)
    body = ref[:B * C * plane].reshape(B * C, plane)
    img = np.zeros((B * C, Hp, Wp), np.float32)
    img[:, ph:ph + H, :W] = x.reshape(B * C, H, W)
    body[:, pw:pw + Hp * Wp] = img.reshape(B * C, -1)
    return ref


CASES = [
    # B, C, H, W, L, kernel
    (2, 64, 9, 11, 128, (3, 3)),
    (2, 128, 6, 9, 256, (3, 3)),
    (1, 256, 5, 5, 128, (3, 3)),
    (3, 128, 14, 14, 128, (3, 3)),
    (2, 64, 7, 20, 128, (5, 5)),
    (1, 128, 56, 56, 128, (3, 3)),
    (5, 64, 3, 70, 128, (3, 5)),
    (2, 128, 1, 1, 128, (3, 3)),
    # filters / channels that do not fill the last tile of rows, tiles that span several taps
    (4, 32, 15, 15, 64, (5, 5)),            # the second convolution of the CIFAR stack
    (2, 16, 8, 9, 16, (3, 3)),
    (2, 48, 7, 12, 80, (3, 3)),
    (1, 160, 6, 6, 96, (3, 3)),
    (2, 96, 5, 13, 208, (1, 3)),
    (3, 64, 13, 13, 64, (3, 3)),
    # many K pieces of a small weight gradient (the kernel that sums them stores the filters' layout)
    (48, 16, 20, 22, 16, (3, 3)),
    (40, 32, 15, 15, 48, (5, 3)),
]


@pytest.mark.parametrize("B,C,H,W,L,kernel", CASES)
def test_conv_same_forward_and_gradients_vs_oracle(K, B, C, H, W, L, kernel):
    from cgt_amd.gpuarray import to_gpu
    pad = ((kernel[0] - 1) // 2, (kernel[1] - 1) // 2)
    assert K.conv_same_supported(C, L, kernel, pad, (1, 1))
    rs = np.random.RandomState(B * 1000 + C + H)
    x = rs.randn(B, C, H, W).astype(np.float32)
    f = (rs.randn(L, C, *kernel) / np.sqrt(C * kernel[0] * kernel[1])).astype(np.float32)
    gy = rs.randn(B, L, H, W).astype(np.float32)
    xg, fg, gyg = to_gpu(x), to_gpu(f), to_gpu(gy)
    xpad = K.conv_same_pad(xg, kernel)
    # the padding is a copy: bit-exact, and every float of the buffer is written
    assert np.array_equal(xpad.get().view(np.uint32), _padded_reference(x, kernel, xpad.size).view(np.uint32))
    d = np.float64
    y64 = O.conv2d(x.astype(d), f.astype(d), pad, (1, 1))
    y = K.conv_same_fwd(xpad, fg, x.shape)
    assert relfro(y.get(), y64) <= TOL
    # against the im2col path of the same library: agreement to rounding
    y_col = K.conv2d(xg, fg, pad, (1, 1))
    assert relfro(y.get(), y_col.get()) <= 1e-5
    gx64, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), gy.astype(d), pad, (1, 1))
    gypad = K.conv_same_pad(gyg, kernel)
    gx = K.conv_same_bwd_data(gypad, fg, x.shape)
    gf = K.conv_same_bwd_filter(gypad, xpad, x.shape, f.shape)
    assert relfro(gx.get(), gx64) <= TOL
    assert relfro(gf.get(), gf64) <= TOL
    # a second call into the same (reused, uncleared) outputs gives the same bits
    y2 = K.conv_same_fwd(xpad, fg, x.shape, out=y)
    assert y2 is y and np.array_equal(K.conv_same_bwd_filter(gypad, xpad, x.shape, f.shape, out=gf).get(), gf.get())


@pytest.mark.parametrize("B,C,H,W,L", [(3, 64, 10, 13, 128), (11, 64, 56, 56, 128)])
def test_conv_same_fused_bias_and_rectify_match_the_separate_ops(K, B, C, H, W, L):
    # the second size has 286 pixel tiles on 256 CUs: its last 30 go through the tail split,
    # whose reduce kernel applies the bias and the rectify too
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(11)
    x = rs.randn(B, C, H, W).astype(np.float32)
    f = (rs.randn(L, C, 3, 3) / 24).astype(np.float32)
    b = rs.randn(L).astype(np.float32)
    xpad = K.conv_same_pad(to_gpu(x), (3, 3))
    plain = K.conv_same_fwd(xpad, to_gpu(f), x.shape).get()
    fused = K.conv_same_fwd(xpad, to_gpu(f), x.shape, bias=to_gpu(b), relu=True).get()
    pre = plain + b.reshape(1, L, 1, 1)
    want = pre * (pre >= 0).astype(np.float32)            # x * (x >= 0), cgt/nn.py:44-45
    assert np.array_equal(fused.view(np.uint32), want.view(np.uint32))
    only_bias = K.conv_same_fwd(xpad, to_gpu(f), x.shape, bias=to_gpu(b)).get()
    assert np.array_equal(only_bias.view(np.uint32), pre.view(np.uint32))
    if B > 4:
        y64 = O.conv2d(x[-1:].astype(np.float64), f.astype(np.float64), (1, 1), (1, 1))
        assert relfro(plain[-1:], y64) <= TOL


def test_conv_same_supported_rule(K):
    assert K.conv_same_supported(128, 128, (3, 3), (1, 1), (1, 1))
    assert K.conv_same_supported(64, 128, (5, 5), (2, 2), (1, 1))
    assert K.conv_same_supported(256, 512, (3, 3), (1, 1), (1, 1))
    assert K.conv_same_supported(32, 64, (5, 5), (2, 2), (1, 1))          # tiles padded in both products
    assert K.conv_same_supported(16, 16, (3, 3), (1, 1), (1, 1))
    assert K.conv_same_supported(48, 80, (1, 3), (0, 1), (1, 1))
    assert not K.conv_same_supported(24, 128, (5, 5), (2, 2), (1, 1))     # channels: not a multiple of 16
    assert not K.conv_same_supported(128, 72, (5, 5), (2, 2), (1, 1))     # filters (channels of the data gradient)
    assert not K.conv_same_supported(3, 96, (11, 11), (0, 0), (4, 4))     # AlexNet conv1: strided
    assert not K.conv_same_supported(3, 32, (5, 5), (2, 2), (1, 1))       # 3 channels: not a multiple of 16
    assert not K.conv_same_supported(128, 128, (3, 3), (0, 0), (1, 1))    # valid padding
    assert not K.conv_same_supported(128, 128, (2, 2), (0, 0), (1, 1))    # even kernel


def test_nn_conv2d_takes_the_fused_ops_and_grad_goes_through_them(K):
    # nn.conv2d picks the fused ops for a layer they cover; grad walks ConvForward's own
    # pullback (ConvPad of the cotangent, ConvBackwardData, ConvBackwardFilter); a compiled
    # function replays the same closures and serves another batch size
    import cgt_amd as cgt
    from cgt_amd import nn
    from cgt_amd.nn_ops import conv_same
    rs = np.random.RandomState(3)
    x = rs.randn(3, 64, 12, 10).astype(np.float32)
    f = (rs.randn(128, 64, 3, 3) / 24).astype(np.float32)

    def graph(xn, fn):
        y = nn.conv2d(xn, fn, (3, 3), pad=(1, 1))
        pooled = nn.max_pool_2d(nn.rectify(y), (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gf = cgt.grad(loss, [xn, fn])
        return y, loss, gx, gf

    xn, fn = cgt.constant(x), cgt.constant(f)
    y, loss, gx, gf = graph(xn, fn)
    assert isinstance(y.op, conv_same.ConvForward) and isinstance(gx.op, conv_same.ConvBackwardData)
    assert isinstance(gf.op, conv_same.ConvBackwardFilter)
    # the cotangent comes out of the pool: its pullback writes the padded copy itself, rectify mask included
    assert isinstance(gx.parents[0].op, conv_same.ConvPadPoolPullback) and gx.parents[0].op.has_relu
    assert gf.parents[0] is gx.parents[0]
    d = np.float64
    y64 = O.conv2d(x.astype(d), f.astype(d), (1, 1), (1, 1))
    r64 = y64 * (y64 >= 0)
    p64, mask = O.max_pool(r64, (2, 2), (0, 0), (2, 2))
    gr = O.max_pool_pullback(r64.shape, mask, 2 * p64) * (y64 >= 0)
    gx64, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), gr, (1, 1), (1, 1))
    assert relfro(y.get(), y64) <= TOL and abs(float(loss.get()) - (p64 ** 2).sum()) <= TOL * (p64 ** 2).sum()
    assert relfro(gx.get(), gx64) <= TOL and relfro(gf.get(), gf64) <= TOL
    # the im2col composition of the same layer: same results to rounding
    old = nn.conv_algo("im2col")
    try:
        y_c, loss_c, gx_c, gf_c = graph(cgt.constant(x), cgt.constant(f))
        assert not isinstance(y_c.op, conv_same.ConvForward)
    finally:
        nn.conv_algo(old)
    assert relfro(y.get(), y_c.get()) <= 1e-5 and relfro(gx.get(), gx_c.get()) <= 1e-4 and relfro(gf.get(), gf_c.get()) <= 1e-4
    fun = cgt.function([xn], [y, loss, gx, gf])
    for got, node in zip(fun(x), (y, loss, gx, gf)):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    x5 = rs.randn(5, 64, 12, 10).astype(np.float32)
    fresh = graph(cgt.constant(x5), fn)
    for got, node in zip(fun(x5), fresh):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))


def test_spatial_convolution_bias_and_rectify_fused_have_the_bits_of_the_separate_ops(K):
    # SpatialConvolution's bias add and the nn.rectify behind it go into the product's epilogue;
    # values, loss and all three gradients are bit-identical to the graph with the separate
    # Repeat / add / >= / * ops, and the compiled function is shorter
    import cgt_amd as cgt
    from cgt_amd import nn
    from cgt_amd.nn_ops import conv_same
    rs = np.random.RandomState(8)
    x = rs.randn(3, 64, 11, 9).astype(np.float32)
    w = (rs.randn(128, 64, 3, 3) / 24).astype(np.float32)
    b = (0.3 * rs.randn(1, 128, 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(64, 128, (3, 3), (1, 1), weight_init=w, bias_init=b)

    def graph(xn):
        act = nn.rectify(layer(xn))
        pooled = nn.max_pool_2d(act, (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
        return [act, loss, gx, gw, gb]

    xn = cgt.constant(x)
    fused = graph(xn)
    producer = fused[0].parents[0].op                       # act = TupleIndex(0) of the fused op's (y, mask)
    assert isinstance(producer, conv_same.ConvForward) and producer.relu and producer.has_bias
    old = nn.conv_fusion(False)
    try:
        xu = cgt.constant(x)
        unfused = graph(xu)
        assert isinstance(unfused[0].op, cgt.ElwiseBinary)
    finally:
        nn.conv_fusion(old)
    for a, u in zip(fused, unfused):
        assert np.array_equal(a.get().view(np.uint32), u.get().view(np.uint32))
    # and against the float64 chain
    d = np.float64
    pre = O.conv2d(x.astype(d), w.astype(d), (1, 1), (1, 1)) + b
    act64 = pre * (pre >= 0)
    p64, mask = O.max_pool(act64, (2, 2), (0, 0), (2, 2))
    gpre = O.max_pool_pullback(act64.shape, mask, 2 * p64) * (pre >= 0)
    gx64, gw64 = O.conv2d_pullback(x.astype(d), w.astype(d), gpre, (1, 1), (1, 1))
    assert relfro(fused[0].get(), act64) <= TOL and relfro(fused[2].get(), gx64) <= TOL
    assert relfro(fused[3].get(), gw64) <= TOL and relfro(fused[4].get(), gpre.sum((0, 2, 3), keepdims=True)) <= TOL
    f_fused, f_unfused = cgt.function([xn], fused), cgt.function([xu], unfused)
    launches = lambda f: sum(1 for s in f.plan_steps() if s[0] == "byref")      # noqa: E731
    assert launches(f_fused) <= launches(f_unfused) - 4          # Repeat, +, >=, * are gone
    x2 = rs.randn(5, 64, 11, 9).astype(np.float32)
    for a, u in zip(f_fused(x2), f_unfused(x2)):
        assert np.array_equal(a.view(np.uint32), u.view(np.uint32))


POOLS = [((2, 2), (0, 0), (2, 2)), ((3, 3), (0, 0), (2, 2)), ((3, 3), (1, 1), (2, 2)), ((4, 3), (1, 0), (3, 2)),
         ((2, 2), (0, 0), (1, 1)), ((1, 1), (0, 0), (2, 3))]


@pytest.mark.parametrize("pk,pp,ps", POOLS)
@pytest.mark.parametrize("shape,kernel", [((3, 5, 14, 12), (3, 3)), ((2, 3, 55, 55), (5, 5)), ((1, 7, 9, 31), (1, 7)), ((2, 4, 6, 5), (7, 3)),
                                          ((41, 101, 6, 5), (3, 3)),        # many small planes: several per workgroup, the last one short
                                          ((64, 128, 56, 56), (3, 3))])     # the VGG layer at full size
def test_pool_pullback_written_into_the_padded_layout_is_bit_exact(K, pk, pp, ps, shape, kernel):
    # one pass instead of MaxPoolPullback -> (rectify mask *) -> ConvPad: the same bits, every float of
    # the padded buffer written (it starts out poisoned)
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(sum(shape) + pk[0] * 7 + ps[1])
    act = rs.randn(*shape).astype(np.float32)
    act *= (act >= 0)                                   # ties at zero, as after a rectify
    top, mask = K.max_pool(to_gpu(act), pk, pp, ps)
    if top.size == 0:
        pytest.skip("the pool has no output for this shape")
    gtop_h = (rs.randn(*top.shape) * 10.0 ** rs.randint(-3, 4, top.shape)).astype(np.float32)
    gtop_h[rs.rand(*top.shape) < 0.05] = -0.0           # 0 + (-0) = +0 in the reference's scatter-add
    gtop = to_gpu(gtop_h)
    rmask = to_gpu((rs.rand(*shape) < 0.6).astype(np.int8))
    want_plain = K.conv_same_pad(K.max_pool_pullback(shape, mask, gtop, pk, pp, ps), kernel).get()
    want_relu = K.conv_same_pad(K.elwise_binary("*", rmask, K.max_pool_pullback(shape, mask, gtop, pk, pp, ps)), kernel).get()
    # what the oracle says the unpadded pullback is
    assert np.array_equal(K.max_pool_pullback(shape, mask, gtop, pk, pp, ps).get().view(np.uint32),
                          O.max_pool_pullback(shape, mask.get(), gtop.get()).view(np.uint32))
    poison = to_gpu(np.full(want_plain.shape, np.nan, np.float32))
    got = K.conv_same_pad_pool_pullback(shape, mask, gtop, pk, pp, ps, kernel, out=poison).get()
    assert np.array_equal(got.view(np.uint32), want_plain.view(np.uint32))
    poison = to_gpu(np.full(want_plain.shape, np.nan, np.float32))
    got = K.conv_same_pad_pool_pullback(shape, mask, gtop, pk, pp, ps, kernel, relu_mask=rmask, out=poison).get()
    assert np.array_equal(got.view(np.uint32), want_relu.view(np.uint32))


def test_pool_pullback_fusion_leaves_the_gradients_bit_identical(K):
    # conv -> rectify -> pool: gradients through ConvPadPoolPullback against the graph with the
    # separate MaxPoolPullback, mask multiply and ConvPad; and the compiled function is shorter
    import cgt_amd as cgt
    from cgt_amd import nn
    from cgt_amd.nn_ops import conv_same
    rs = np.random.RandomState(21)
    x = rs.randn(3, 32, 13, 14).astype(np.float32)
    f = (rs.randn(48, 32, 3, 3) / 17).astype(np.float32)

    def graph(xn, fn, relu):
        y = nn.conv2d(xn, fn, (3, 3), pad=(1, 1))
        pooled = nn.max_pool_2d(nn.rectify(y) if relu else y, (3, 3), (0, 0), (2, 2))
        gx, gf = cgt.grad(cgt.sum(pooled * pooled), [xn, fn])
        return [pooled, gx, gf]

    for relu in (True, False):
        xn, fn = cgt.constant(x), cgt.constant(f)
        fused = graph(xn, fn, relu)
        assert isinstance(fused[1].parents[0].op, conv_same.ConvPadPoolPullback)
        conv_same.FUSE_POOL_PULLBACK = False
        try:
            xu, fu = cgt.constant(x), cgt.constant(f)
            plain = graph(xu, fu, relu)
            assert isinstance(plain[1].parents[0].op, conv_same.ConvPad)
        finally:
            conv_same.FUSE_POOL_PULLBACK = True
        for a, u in zip(fused, plain):
            assert np.array_equal(a.get().view(np.uint32), u.get().view(np.uint32))
        f_fused, f_plain = cgt.function([xn], fused), cgt.function([xu], plain)
        launches = lambda fun: sum(1 for s in fun.plan_steps() if s[0] == "byref")      # noqa: E731
        assert launches(f_fused) == launches(f_plain) - (2 if relu else 1)
        x2 = rs.randn(5, 32, 13, 14).astype(np.float32)
        for a, u in zip(f_fused(x2), f_plain(x2)):
            assert np.array_equal(a.view(np.uint32), u.view(np.uint32))


def test_vgg_layer_full_size_through_the_fused_ops(K):
    # the headline layer at full size: slices against the float64 oracle, the rest through
    # the adjoint identity <conv(x), gy> = <x, conv^T(gy)> and linearity in the filters
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(0)
    B, C, H, W, L = 64, 128, 56, 56, 128
    x = rs.randn(B, C, H, W).astype(np.float32)
    f = (rs.randn(L, C, 3, 3) * np.sqrt(1.0 / (C * 9))).astype(np.float32)
    gy = rs.randn(B, L, H, W).astype(np.float32)
    xg, fg = to_gpu(x), to_gpu(f)
    xpad, gypad = K.conv_same_pad(xg, (3, 3)), K.conv_same_pad(to_gpu(gy), (3, 3))
    y = K.conv_same_fwd(xpad, fg, x.shape).get()
    gx = K.conv_same_bwd_data(gypad, fg, x.shape).get()
    gf = K.conv_same_bwd_filter(gypad, xpad, x.shape, f.shape).get()
    d = np.float64
    for b in (0, 37, 63):
        y64 = O.conv2d(x[b:b + 1].astype(d), f.astype(d), (1, 1), (1, 1))
        gx64, _ = O.conv2d_pullback(x[b:b + 1].astype(d), f.astype(d), gy[b:b + 1].astype(d), (1, 1), (1, 1))
        assert relfro(y[b:b + 1], y64) <= TOL and relfro(gx[b:b + 1], gx64) <= TOL
    lhs = float(np.vdot(y.astype(d), gy.astype(d)))
    assert abs(lhs - float(np.vdot(x.astype(d), gx.astype(d)))) <= 1e-5 * abs(lhs)
    assert abs(lhs - float(np.vdot(f.astype(d), gf.astype(d)))) <= 1e-5 * abs(lhs)
    # the weight gradient itself: sampled (channel, tap) columns over all filters and the whole batch
    # against float64 -- gf[l, c, ho, wo] = sum over (b, h, w) of gy[b, l, h, w] * x[b, c, h + ho - 1, w + wo - 1];
    # every tap, first / last / interior channels of the blocks of 16 the product walks
    gy64 = gy.astype(d)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    samples = [(c, ho, wo) for c in (0, 15, 16, 77, 127) for ho in range(3) for wo in range(3)][::2]
    got = np.stack([gf[:, c, ho, wo] for c, ho, wo in samples], 1)
    want = np.stack([np.einsum("blhw,bhw->l", gy64, xp[:, c, ho:ho + H, wo:wo + W].astype(d)) for c, ho, wo in samples], 1)
    assert relfro(got, want) <= TOL
    assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
    # the same launches again: same bits (split-K partial sums are reduced in a fixed order)
    assert np.array_equal(K.conv_same_bwd_filter(gypad, xpad, x.shape, f.shape).get().view(np.uint32), gf.view(np.uint32))
    assert np.array_equal(K.conv_same_fwd(xpad, fg, x.shape).get().view(np.uint32), y.view(np.uint32))
    assert np.array_equal(K.conv_same_bwd_data(gypad, fg, x.shape).get().view(np.uint32), gx.view(np.uint32))
