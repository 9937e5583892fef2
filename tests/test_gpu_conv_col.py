"""conv2d over the column buffer with the NCHW side read / written by the GEMMs
themselves: the forward product writes [B,L,m,n] directly (no [B*m*n, L] matrix, no
Transpose{0,3,1,2}), the two gradient products read the NCHW cotangent directly (no
Transpose{0,2,3,1}).  They must compute what the reference's composition
im2col -> Mul22(F,T) -> reshape -> transpose computes (cgt/nn.py:95-100) and what its
autodiff derives for it (cgt/core.py:2143-2175): compared with the float64 oracle at 1e-4
relative Frobenius error, and with the literal composition of this library to rounding.
The fused bias add + rectify is bit-identical to the separate fp32 operations.
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


CASES = [
    # B, C, H, W, L, kernel, pad, stride
    (4, 3, 47, 47, 96, (11, 11), (0, 0), (4, 4)),       # AlexNet conv1 in miniature: ragged K = 363, 96-row tiles
    (8, 3, 32, 32, 32, (5, 5), (2, 2), (1, 1)),         # CIFAR conv1: 32 filters, K = 75
    (6, 1, 28, 28, 32, (3, 3), (1, 1), (1, 1)),         # MNIST: K = 9
    (37, 2, 7, 7, 20, (3, 3), (0, 0), (1, 1)),          # 25 pixels per image: a tile of columns spans 6 images; 20 filters
    (3, 5, 9, 13, 130, (3, 2), (1, 0), (2, 1)),         # two row tiles, the second nearly empty
    (1, 4, 5, 5, 7, (5, 5), (0, 0), (1, 1)),            # one pixel per image
    (12, 16, 56, 56, 64, (5, 5), (2, 2), (1, 1)),       # 294 column tiles: the last 38 go through the tail split
    (2, 24, 30, 30, 48, (3, 3), (1, 1), (1, 1)),
    (5, 3, 20, 17, 33, (4, 6), (3, 5), (3, 2)),         # padding wider than half the kernel, patches hanging over every edge
    (2, 6, 40, 40, 200, (7, 7), (3, 3), (2, 2)),
    (10, 2, 63, 57, 100, (10, 11), (9, 9), (2, 2)),     # the two weight-gradient variants pick different tile shapes
    # few filters and short patches: the gathered weight gradient is the reduction kernel (bands of output
    # rows staged in LDS) -- bands that do not divide the rows, 17 filters, patches of exactly 128, a
    # stride, more (image, band) units than workgroups, rows too wide for it (the tiled product again)
    (3, 3, 33, 70, 32, (5, 5), (2, 2), (1, 1)),
    (5, 2, 31, 29, 17, (8, 8), (3, 3), (2, 2)),
    (1300, 1, 6, 6, 8, (3, 3), (1, 1), (1, 1)),
    (2, 1, 9, 300, 32, (3, 3), (1, 1), (1, 1)),
    (4, 3, 24, 24, 1, (3, 5), (0, 2), (1, 3)),
]


@pytest.mark.parametrize("B,C,H,W,L,kernel,pad,stride", CASES)
def test_conv_col_products_vs_oracle(K, B, C, H, W, L, kernel, pad, stride):
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(B * 100 + C * 10 + L)
    x = rs.randn(B, C, H, W).astype(np.float32)
    f = (rs.randn(L, C, *kernel) / np.sqrt(C * kernel[0] * kernel[1])).astype(np.float32)
    d = np.float64
    y64 = O.conv2d(x.astype(d), f.astype(d), pad, stride)
    gy = rs.randn(*y64.shape).astype(np.float32)
    xg, fg, gyg = to_gpu(x), to_gpu(f), to_gpu(gy)
    col = K.im2col(xg, kernel, pad, stride)
    y = K.conv_col_fwd(col, fg)
    assert y.shape == y64.shape
    assert relfro(y.get(), y64) <= TOL
    # the literal composition (GEMM into [B*m*n, L], then a transpose): same sums, agreement to rounding
    assert relfro(y.get(), K.conv2d(xg, fg, pad, stride).get()) <= 2e-6
    gx64, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), gy.astype(d), pad, stride)
    gcol = K.conv_col_bwd_data(gyg, fg)
    assert gcol.shape == col.shape
    want_gcol = np.einsum("blmn,lz->bmnz", gy.astype(d), f.reshape(L, -1).astype(d))
    assert relfro(gcol.get(), want_gcol) <= TOL
    gx = K.col2im(gcol, x.shape, kernel, pad, stride)
    assert relfro(gx.get(), gx64) <= TOL
    gf = K.conv_col_bwd_filter(gyg, col, f.shape)
    assert relfro(gf.get(), gf64) <= TOL
    gx_lit, gf_lit = K.conv2d_pullback(xg, fg, gyg, pad, stride)
    assert relfro(gf.get(), gf_lit.get()) <= 2e-6 and relfro(gx.get(), gx_lit.get()) <= 2e-6
    # the same two products with the patches gathered from x inside the GEMM (no column buffer): the
    # same operand values in the same order.  Forward: the same bits.  Weight gradient: the same sums
    # cut into the same K pieces when both variants take the same tile shape (the gathered one has
    # tiles of 128 or 64 columns only) -- the same bits then, the same result to rounding otherwise.
    assert K.conv_patch_supported(x.shape, kernel, pad, stride)
    y_p = K.conv_patch_fwd(xg, fg, pad, stride)
    assert np.array_equal(y_p.get().view(np.uint32), y.get().view(np.uint32))
    gf_p = K.conv_patch_bwd_filter(gyg, xg, f.shape, pad, stride)
    assert relfro(gf_p.get(), gf.get()) <= 2e-6 and relfro(gf_p.get(), gf64) <= TOL
    assert np.array_equal(K.conv_patch_bwd_filter(gyg, xg, f.shape, pad, stride).get().view(np.uint32), gf_p.get().view(np.uint32))
    # a second call into the same (reused, uncleared) outputs gives the same bits
    first = (y.get(), gcol.get(), gf.get())
    K.conv_col_fwd(col, fg, out=y)
    K.conv_col_bwd_data(gyg, fg, out=gcol)
    K.conv_col_bwd_filter(gyg, col, f.shape, out=gf)
    for a, b in zip(first, (y.get(), gcol.get(), gf.get())):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("B,C,H,W,L,kernel,pad,stride", [CASES[0], CASES[3], CASES[6]])
def test_conv_col_fused_bias_and_rectify_match_the_separate_ops(K, B, C, H, W, L, kernel, pad, stride):
    from cgt_amd.gpuarray import empty, to_gpu
    rs = np.random.RandomState(5)
    x = rs.randn(B, C, H, W).astype(np.float32)
    f = (rs.randn(L, C, *kernel) / np.sqrt(C * kernel[0] * kernel[1])).astype(np.float32)
    b = rs.randn(L).astype(np.float32)
    col = K.im2col(to_gpu(x), kernel, pad, stride)
    plain = K.conv_col_fwd(col, to_gpu(f)).get()
    mask = empty(plain.shape, np.int8)
    fused = K.conv_col_fwd(col, to_gpu(f), bias=to_gpu(b), relu=True, mask=mask).get()
    pre = plain + b.reshape(1, L, 1, 1)
    want = pre * (pre >= 0).astype(np.float32)            # x * (x >= 0), cgt/nn.py:44-45
    assert np.array_equal(fused.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(mask.get(), (pre >= 0).astype(np.int8))
    only_bias = K.conv_col_fwd(col, to_gpu(f), bias=to_gpu(b)).get()
    assert np.array_equal(only_bias.view(np.uint32), pre.view(np.uint32))
    # and without the column buffer
    mask2 = empty(plain.shape, np.int8)
    fused2 = K.conv_patch_fwd(to_gpu(x), to_gpu(f), pad, stride, bias=to_gpu(b), relu=True, mask=mask2).get()
    assert np.array_equal(fused2.view(np.uint32), want.view(np.uint32)) and np.array_equal(mask2.get(), mask.get())


def test_conv_col_full_size_alexnet_conv1(K):
    # 128 x 3 x 227 x 227, 96 11x11 filters, stride 4: parity on image slices against the oracle,
    # and the weight gradient (a sum over all 128 x 3025 pixels) against the literal composition
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(0)
    x = rs.randn(128, 3, 227, 227).astype(np.float32)
    f = (0.01 * rs.randn(96, 3, 11, 11)).astype(np.float32)
    xg, fg = to_gpu(x), to_gpu(f)
    col = K.im2col(xg, (11, 11), (0, 0), (4, 4))
    y = K.conv_col_fwd(col, fg)
    assert y.shape == (128, 96, 55, 55)
    yh = y.get()
    d = np.float64
    for b in (0, 77, 127):
        assert relfro(yh[b:b + 1], O.conv2d(x[b:b + 1].astype(d), f.astype(d), (0, 0), (4, 4))) <= TOL
    gy = rs.randn(128, 96, 55, 55).astype(np.float32)
    gyg = to_gpu(gy)
    gcol = K.conv_col_bwd_data(gyg, fg)
    gx = K.col2im(gcol, x.shape, (11, 11), (0, 0), (4, 4)).get()
    gf = K.conv_col_bwd_filter(gyg, col, f.shape).get()
    assert np.array_equal(K.conv_patch_fwd(xg, fg, (0, 0), (4, 4)).get().view(np.uint32), yh.view(np.uint32))
    assert np.array_equal(K.conv_patch_bwd_filter(gyg, xg, f.shape, (0, 0), (4, 4)).get().view(np.uint32), gf.view(np.uint32))   # same tile shape
    del gcol
    gf64 = np.zeros(f.shape, d)
    for b in (3, 126):
        gxb, _ = O.conv2d_pullback(x[b:b + 1].astype(d), f.astype(d), gy[b:b + 1].astype(d), (0, 0), (4, 4))
        assert relfro(gx[b:b + 1], gxb) <= TOL
    # float64 weight gradient: per image gy_b [L, P] . col_b [P, Z], summed over the batch
    colh = col.get().reshape(128, 3025, 363)
    for b in range(128):
        gf64 += (gy[b].reshape(96, 3025).astype(d) @ colh[b].astype(d)).reshape(f.shape)
    assert relfro(gf, gf64) <= TOL


def test_nn_conv2d_builds_the_column_buffer_ops_for_a_strided_layer():
    # a layer the padded-image products do not cover (stride 2, 20 channels): Im2Col stays, one
    # fused op follows it, grad walks its pullback and Im2Col's own (Col2Im); a compiled function
    # replays the same closures and serves another batch size; the literal composition agrees
    import cgt_amd as cgt
    from cgt_amd import capi, nn
    from cgt_amd.nn_ops import conv_col
    capi.require_gpu()
    rs = np.random.RandomState(4)
    x = rs.randn(3, 20, 23, 19).astype(np.float32)
    f = (rs.randn(40, 20, 5, 5) / 22).astype(np.float32)

    def graph(xn, fn):
        y = nn.conv2d(xn, fn, (5, 5), pad=(1, 2), stride=(2, 2))
        pooled = nn.max_pool_2d(nn.rectify(y), (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gf = cgt.grad(loss, [xn, fn])
        return y, loss, gx, gf

    xn, fn = cgt.constant(x), cgt.constant(f)
    y, loss, gx, gf = graph(xn, fn)
    assert isinstance(y.op, conv_col.ConvColForward) and type(y.parents[0].op).__name__ == "Im2Col"
    assert type(gx.op).__name__ == "Col2Im" and isinstance(gx.parents[0].op, conv_col.ConvColBackwardData)
    assert isinstance(gf.op, conv_col.ConvColBackwardFilter)
    d = np.float64
    y64 = O.conv2d(x.astype(d), f.astype(d), (1, 2), (2, 2))
    r64 = y64 * (y64 >= 0)
    p64, mask = O.max_pool(r64, (2, 2), (0, 0), (2, 2))
    gr = O.max_pool_pullback(r64.shape, mask, 2 * p64) * (y64 >= 0)
    gx64, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), gr, (1, 2), (2, 2))
    assert relfro(y.get(), y64) <= TOL and abs(float(loss.get()) - (p64 ** 2).sum()) <= TOL * (p64 ** 2).sum()
    assert relfro(gx.get(), gx64) <= TOL and relfro(gf.get(), gf64) <= TOL
    old = nn.conv_algo("im2col")
    try:
        y_c, loss_c, gx_c, gf_c = graph(cgt.constant(x), cgt.constant(f))
        assert isinstance(y_c.op, cgt.Transpose)
    finally:
        nn.conv_algo(old)
    assert relfro(y.get(), y_c.get()) <= 1e-5 and relfro(gx.get(), gx_c.get()) <= 1e-4 and relfro(gf.get(), gf_c.get()) <= 1e-4
    fun = cgt.function([xn], [y, loss, gx, gf])
    for got, node in zip(fun(x), (y, loss, gx, gf)):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))
    x5 = rs.randn(5, 20, 23, 19).astype(np.float32)
    fresh = graph(cgt.constant(x5), fn)
    for got, node in zip(fun(x5), fresh):
        assert np.array_equal(got.view(np.uint32), node.get().view(np.uint32))


def test_spatial_convolution_over_the_column_buffer_fuses_bias_and_rectify():
    # SpatialConvolution's bias add and the nn.rectify behind it go into the product's epilogue:
    # values, loss and all three gradients have the bits of the graph with the separate ops
    import cgt_amd as cgt
    from cgt_amd import capi, nn
    from cgt_amd.nn_ops import conv_col
    capi.require_gpu()
    rs = np.random.RandomState(9)
    x = rs.randn(4, 17, 21, 21).astype(np.float32)
    w = (rs.randn(24, 17, 7, 7) / 29).astype(np.float32)
    b = (0.3 * rs.randn(1, 24, 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(17, 24, (7, 7), (0, 0), stride=(2, 2), weight_init=w, bias_init=b)

    def graph(xn):
        act = nn.rectify(layer(xn))
        pooled = nn.max_pool_2d(act, (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
        return [act, loss, gx, gw, gb]

    xn = cgt.constant(x)
    fused = graph(xn)
    producer = fused[0].parents[0].op                       # act = TupleIndex(0) of the fused op's (y, mask)
    assert isinstance(producer, conv_col.ConvColForward) and producer.relu and producer.has_bias
    old = nn.conv_fusion(False)
    try:
        xu = cgt.constant(x)
        unfused = graph(xu)
        assert isinstance(unfused[0].op, cgt.ElwiseBinary)
    finally:
        nn.conv_fusion(old)
    for a, u in zip(fused, unfused):
        assert np.array_equal(a.get().view(np.uint32), u.get().view(np.uint32))
    d = np.float64
    pre = O.conv2d(x.astype(d), w.astype(d), (0, 0), (2, 2)) + b
    act64 = pre * (pre >= 0)
    p64, mask = O.max_pool(act64, (2, 2), (0, 0), (2, 2))
    gpre = O.max_pool_pullback(act64.shape, mask, 2 * p64) * (pre >= 0)
    gx64, gw64 = O.conv2d_pullback(x.astype(d), w.astype(d), gpre, (0, 0), (2, 2))
    assert relfro(fused[0].get(), act64) <= TOL and relfro(fused[2].get(), gx64) <= TOL
    assert relfro(fused[3].get(), gw64) <= TOL and relfro(fused[4].get(), gpre.sum((0, 2, 3), keepdims=True)) <= TOL
    f_fused, f_unfused = cgt.function([xn], fused), cgt.function([xu], unfused)
    launches = lambda f: sum(1 for s in f.plan_steps() if s[0] == "byref")      # noqa: E731
    assert launches(f_fused) <= launches(f_unfused) - 4          # Repeat, +, >=, * are gone
    x2 = rs.randn(6, 17, 21, 21).astype(np.float32)
    for a, u in zip(f_fused(x2), f_unfused(x2)):
        assert np.array_equal(a.view(np.uint32), u.view(np.uint32))


def test_nn_conv2d_gathers_patches_for_a_layer_with_few_channels():
    # 3 input channels, stride 2, padding: no Im2Col in the graph -- the forward product and the
    # weight gradient read x themselves, the data gradient goes through the column buffer's
    # cotangent and Col2Im.  Values and gradients have the bits of the graph over the column buffer
    # (the same products on the same operand values; 40 filters give both weight gradients the same
    # tile shape and therefore the same K pieces), SpatialConvolution's bias and a rectify ride
    # in the epilogue, and the compiled function serves another batch size.
    import cgt_amd as cgt
    from cgt_amd import capi, nn
    from cgt_amd.nn_ops import conv_col
    capi.require_gpu()
    rs = np.random.RandomState(14)
    x = rs.randn(4, 3, 29, 23).astype(np.float32)
    w = (rs.randn(40, 3, 5, 7) / 10).astype(np.float32)
    b = (0.3 * rs.randn(1, 40, 1, 1)).astype(np.float32)
    layer = nn.SpatialConvolution(3, 40, (5, 7), (2, 1), stride=(2, 3), weight_init=w, bias_init=b)

    def graph(xn):
        act = nn.rectify(layer(xn))
        pooled = nn.max_pool_2d(act, (2, 2), (0, 0), (2, 2))
        loss = cgt.sum(pooled * pooled)
        gx, gw, gb = cgt.grad(loss, [xn, layer.weight, layer.bias])
        return [act, loss, gx, gw, gb]

    xn = cgt.constant(x)
    patch = graph(xn)
    producer = patch[0].parents[0].op
    assert isinstance(producer, conv_col.ConvPatchForward) and producer.relu and producer.has_bias
    assert type(patch[2].op).__name__ == "Col2Im" and isinstance(patch[2].parents[0].op, conv_col.ConvPatchBackwardData)
    assert isinstance(patch[3].op, conv_col.ConvPatchBackwardFilter)
    old = nn.conv_algo("col")
    try:
        xc = cgt.constant(x)
        col = graph(xc)
        assert isinstance(col[0].parents[0].op, conv_col.ConvColForward)
    finally:
        nn.conv_algo(old)
    for a, u in zip(patch, col):
        assert np.array_equal(a.get().view(np.uint32), u.get().view(np.uint32))
    d = np.float64
    pre = O.conv2d(x.astype(d), w.astype(d), (2, 1), (2, 3)) + b
    act64 = pre * (pre >= 0)
    p64, mask = O.max_pool(act64, (2, 2), (0, 0), (2, 2))
    gpre = O.max_pool_pullback(act64.shape, mask, 2 * p64) * (pre >= 0)
    gx64, gw64 = O.conv2d_pullback(x.astype(d), w.astype(d), gpre, (2, 1), (2, 3))
    assert relfro(patch[0].get(), act64) <= TOL and relfro(patch[2].get(), gx64) <= TOL
    assert relfro(patch[3].get(), gw64) <= TOL and relfro(patch[4].get(), gpre.sum((0, 2, 3), keepdims=True)) <= TOL
    f_patch, f_col = cgt.function([xn], patch), cgt.function([xc], col)
    launches = lambda f: sum(1 for s in f.plan_steps() if s[0] == "byref")      # noqa: E731
    assert launches(f_patch) == launches(f_col) - 1              # no Im2Col
    x2 = rs.randn(7, 3, 29, 23).astype(np.float32)
    for a, u in zip(f_patch(x2), f_col(x2)):
        assert np.array_equal(a.view(np.uint32), u.view(np.uint32))


def test_weight_gradient_of_a_large_batch_runs_in_groups_of_images(K):
    # the weight gradient's K axis is cut per image, one [L][Z] block of partial sums per image:
    # 2000 images x 64 x 576 floats is more than the 256 MiB those may take, so the batch runs in two
    # groups whose results are added in order -- the same entry point, any batch size
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(8)
    B, C, H, W, L = 2000, 64, 4, 4, 64
    x = rs.randn(B, C, H, W).astype(np.float32)
    gy = rs.randn(B, L, 2, 2).astype(np.float32)
    f = (rs.randn(L, C, 3, 3) / 24).astype(np.float32)
    assert B * L * C * 9 * 4 > 256 << 20
    col = K.im2col(to_gpu(x), (3, 3), (0, 0), (1, 1))
    gf = K.conv_col_bwd_filter(to_gpu(gy), col, f.shape)
    d = np.float64
    _, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), gy.astype(d), (0, 0), (1, 1))
    assert relfro(gf.get(), gf64) <= TOL
    # deterministic, and the gathered form (no column buffer) groups the same way
    assert np.array_equal(K.conv_col_bwd_filter(to_gpu(gy), col, f.shape).get().view(np.uint32), gf.get().view(np.uint32))
    x3 = rs.randn(1500, 3, 9, 9).astype(np.float32)
    gy3 = rs.randn(1500, 512, 3, 3).astype(np.float32)
    assert 1500 * 512 * 3 * 49 * 4 > 256 << 20
    gf3 = K.conv_patch_bwd_filter(to_gpu(gy3), to_gpu(x3), (512, 3, 7, 7), (0, 0), (1, 1))
    _, gf64 = O.conv2d_pullback(x3.astype(d), np.zeros((512, 3, 7, 7), d), gy3.astype(d), (0, 0), (1, 1))
    assert relfro(gf3.get(), gf64) <= TOL


def test_nn_conv2d_falls_through_when_a_layer_outgrows_the_fused_products(K):
    # a 16-channel 1449 x 1449 same-padding layer: its padded plane has more than 2^21 floats, which the
    # products over the padded image do not index; nn.conv2d then builds the products over a column
    # buffer (and beyond their limits the literal composition) instead of raising
    import cgt_amd as cgt
    from cgt_amd import nn
    from cgt_amd.nn_ops import conv_col, conv_same
    assert K.conv_same_fits((1, 16, 1440, 1440), 16, (3, 3)) and not K.conv_same_fits((1, 16, 1449, 1449), 16, (3, 3))
    assert K.conv_same_fits((64, 128, 56, 56), 128, (3, 3))
    assert not K.conv_same_fits((1, 1024, 1024, 1024), 16, (3, 3))          # one image's channels: 2^30 floats
    assert K.conv_col_fits((128, 3, 227, 227), 96, (11, 11), (0, 0), (4, 4))
    assert not K.conv_col_fits((1, 16, 2048, 2048), 256, (3, 3), (1, 1), (1, 1))   # L * P = 2^30
    rs = np.random.RandomState(9)
    x = rs.randn(1, 16, 1449, 1449).astype(np.float32)
    f = (rs.randn(16, 16, 3, 3) / 12).astype(np.float32)
    xn, fn = cgt.constant(x), cgt.constant(f)
    y = nn.conv2d(xn, fn, (3, 3), pad=(1, 1))
    assert isinstance(y.op, conv_col.ConvColForward) and not isinstance(y.op, conv_same.ConvForward)
    gy = rs.randn(*y.shape).astype(np.float32)
    gx, gf = cgt.grad(y, [xn, fn], goutput=gy)
    yv, gxv, gfv = y.get(), gx.get(), gf.get()
    d = np.float64
    # rows of the result against a float64 correlation of the rows they read
    xp = np.pad(x[0].astype(d), ((0, 0), (1, 1), (1, 1)))
    for h in (0, 700, 1448):
        want = np.einsum("lcij,cijw->lw", f.astype(d),
                         np.stack([np.stack([xp[:, h + i, j:j + 1449] for j in range(3)], 1) for i in range(3)], 1))
        assert relfro(yv[0, :, h, :], want) <= TOL
    lhs = float(np.vdot(yv.astype(d), gy.astype(d)))
    assert abs(lhs - float(np.vdot(x.astype(d), gxv.astype(d)))) <= 1e-5 * abs(lhs)
    assert abs(lhs - float(np.vdot(f.astype(d), gfv.astype(d)))) <= 1e-5 * abs(lhs)
