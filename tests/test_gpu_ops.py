"""The hot path through CGT's Op API on the GPU: nn.conv2d / max_pool_2d /
cross_channel_lrn, Mul22 / BatchedMul22, each op's compiled closure fired on
cgtArray views of device memory, gradients through the ops' own pullback
rules.  The cases mirror the reference's tests (cgt/tests/test_conv.py,
test_imgproc.py, test_affine.py, test_einsum.py) with the CPU oracle or the
reference's own numpy/scipy expressions as the expected values.
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
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def test_conv(cgt):
    # cgt/tests/test_conv.py:7-33
    import scipy.signal
    from cgt_amd import nn
    np.random.seed(0)
    x = np.random.randn(2, 2, 5, 17)
    filt = np.random.randn(3, 2, 4, 7)
    filtrows, filtcols = filt.shape[2:]
    out = np.zeros((2, 3, x.shape[2] + filtrows - 1, x.shape[3] + filtcols - 1))
    for b in range(x.shape[0]):
        for inchan in range(x.shape[1]):
            for outchan in range(filt.shape[0]):
                out[b, outchan] += scipy.signal.convolve2d(x[b, inchan], filt[outchan, inchan][::-1, ::-1], mode="full")
    y = nn.conv2d(cgt.constant(x), cgt.constant(filt), kernelshape=(filtrows, filtcols), pad=(filtrows - 1, filtcols - 1))
    np.testing.assert_allclose(out, y.get(), atol=1e-3)


def test_pool(cgt):
    # cgt/tests/test_imgproc.py:40-57: gradient of (y*h).sum() wrt x, here as the
    # pullback of cotangent h, against the oracle (itself pinned by finite differences)
    from cgt_amd.nn import max_pool_2d
    np.random.seed(0)
    xval = np.random.randn(2, 3, 5, 7).astype(np.float32)
    x = cgt.constant(xval)
    y = max_pool_2d(x, (4, 4), (0, 0), (1, 1))
    assert y.shape == (2, 3, 1, 3)
    hval = np.random.randn(*y.shape).astype(np.float32)
    gana = cgt.grad(y, [x], goutput=hval)[0]
    top, mask = O.max_pool(xval, (4, 4), (0, 0), (1, 1))
    assert np.array_equal(y.get(), top)
    assert np.array_equal(gana.get(), O.max_pool_pullback(xval.shape, mask, hval))


def test_im2col(cgt):
    # cgt/tests/test_imgproc.py:59-77: Col2Im is the adjoint of Im2Col
    from cgt_amd.nn_ops.im2col import im2col
    for settings in [((4, 4), (0, 0), (1, 1)), ((3, 3), (1, 1), (2, 2)), ((3, 3), (1, 1), (3, 3))]:
        xval = np.arange(2 * 1 * 28 * 28).reshape(2, 1, 28, 28).astype(np.float32)
        x = cgt.constant(xval)
        y = im2col(x, *settings)
        assert np.array_equal(y.get()[0, 0, 0], xval[0, :, 0:settings[0][0], 0:settings[0][1]].flatten()) or settings[1] != (0, 0)
        hval = np.random.RandomState(0).randn(*y.shape).astype(np.float32)
        gana = cgt.grad(y, [x], goutput=hval)[0].get()
        assert np.array_equal(gana, O.col2im(hval, xval.shape, *settings))
        # adjoint identity in float64 on the host: <im2col(x), h> == <x, col2im(h)>
        lhs = float((y.get().astype(np.float64) * hval).sum())
        rhs = float((xval.astype(np.float64) * gana).sum())
        assert abs(lhs - rhs) <= 1e-5 * abs(lhs)


@pytest.mark.parametrize("top_only", [True, False])
def test_lrn(cgt, top_only, monkeypatch):
    # cgt/tests/test_imgproc.py:79-97: randn(4,8,16,16), localsize 4, alpha .1, beta .5; as the op
    # that stores top alone (what cross_channel_lrn builds) and as the reference's tuple-valued op
    from cgt_amd.nn import cross_channel_lrn
    from cgt_amd.nn_ops import cross_channel_lrn as L
    monkeypatch.setattr(L, "STORE_TOP_ONLY", top_only)
    np.random.seed(0)
    Xval = np.random.randn(4, 8, 16, 16).astype(np.float32)
    X = cgt.constant(Xval)
    y = cross_channel_lrn(X, localsize=4, alpha=.1, beta=.5)
    sums = [float(cross_channel_lrn(X, localsize=4, alpha=.1, beta=.5).get().sum()) for _ in range(3)]
    assert np.isfinite(sums[0]) and sums[0] == sums[1] == sums[2]
    top64, scale64 = O.lrn_fwd(Xval.astype(np.float64), 4, .1, .5)
    assert relfro(y.get(), top64) <= TOL
    a = np.random.rand(*y.shape).astype(np.float32)
    g = cgt.grad(y, [X], goutput=a)[0]
    assert type(y.op).__name__ == ("CrossChannelLRNTop" if top_only else "TupleIndex")
    assert type(g.op).__name__ == ("CrossChannelLRNBackwardFromX" if top_only else "CrossChannelLRNBackward")
    assert relfro(g.get(), O.lrn_bwd(Xval.astype(np.float64), top64, scale64, a.astype(np.float64), 4, .1, .5)) <= TOL


def test_lrn_k_extension(cgt):
    import torch
    import torch.nn.functional as F
    from cgt_amd.nn import cross_channel_lrn
    Xval = np.random.RandomState(1).randn(2, 16, 5, 6).astype(np.float32)
    X = cgt.constant(Xval)
    y = cross_channel_lrn(X, 5, 1e-2, .75, k=2.0)
    xt = torch.from_numpy(Xval).double().requires_grad_(True)
    ref = F.local_response_norm(xt, 5, alpha=1e-2, beta=.75, k=2.0)
    assert relfro(y.get(), ref.detach().numpy()) <= TOL
    # the gradient forms the scale again from X: k goes into it
    a = np.random.RandomState(2).rand(*Xval.shape).astype(np.float32)
    ref.backward(torch.from_numpy(a).double())
    assert relfro(cgt.grad(y, [X], goutput=a)[0].get(), xt.grad.numpy()) <= TOL


@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
def test_mul22_and_pullback(cgt, tA, tB):
    # cgt/tests/test_affine.py matmat cases (M23, M35) and their gradients
    rs = np.random.RandomState(0)
    M23, M35 = rs.randn(2, 3).astype(np.float32), rs.randn(3, 5).astype(np.float32)
    Aval = M23.T.copy() if tA else M23
    Bval = M35.T.copy() if tB else M35
    A, B = cgt.constant(Aval), cgt.constant(Bval)
    C = cgt.Result(cgt.Mul22(tA, tB), [A, B])
    np.testing.assert_allclose(C.get(), M23.dot(M35), rtol=1e-5, atol=1e-6)
    G = rs.randn(2, 5).astype(np.float32)
    gA, gB = cgt.grad(C, [A, B], goutput=G)
    wantA, wantB = G.dot(M35.T), M23.T.dot(G)
    np.testing.assert_allclose(gA.get(), wantA.T if tA else wantA, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gB.get(), wantB.T if tB else wantB, rtol=1e-5, atol=1e-6)


def test_mul22_shape_mismatch_is_an_error(cgt):
    from cgt_amd.capi import CgtAmdError
    A, B = cgt.constant(np.zeros((3, 4), np.float32)), cgt.constant(np.zeros((5, 6), np.float32))
    with pytest.raises(CgtAmdError, match="shape mismatch"):
        cgt.Result(cgt.Mul22(False, False), [A, B])


def test_mul22_output_extent_mismatch_does_not_launch(cgt):
    # the closure is handed a write array whose M (or N) does not fit A (or B): it must
    # report the mismatch and launch nothing -- with extents taken from C the kernel
    # would read A or B past their rows
    from cgt_amd import core
    from cgt_amd.capi import CgtAmdError
    from cgt_amd.gpuarray import to_gpu
    T2 = core.TensorType("f4", 2)
    call = core.get_callable(core.Mul22(False, False), [T2, T2])
    A, B = to_gpu(np.ones((3, 4), np.float32)), to_gpu(np.ones((4, 6), np.float32))
    for cshape in [(7, 6), (3, 9)]:
        sentinel = np.full(cshape, 123.0, np.float32)
        C = to_gpu(sentinel)
        with pytest.raises(CgtAmdError, match="shape mismatch"):
            call.call([A, B], C)
        assert np.array_equal(C.get(), sentinel)
    bcall = core.get_callable(core.BatchedMul22(False, False), [core.TensorType("f4", 3)] * 2)
    A3, B3 = to_gpu(np.ones((2, 3, 4), np.float32)), to_gpu(np.ones((2, 4, 6), np.float32))
    for cshape in [(2, 7, 6), (2, 3, 9), (3, 3, 6)]:
        sentinel = np.full(cshape, 123.0, np.float32)
        C = to_gpu(sentinel)
        with pytest.raises(CgtAmdError, match="shape mismatch"):
            bcall.call([A3, B3], C)
        assert np.array_equal(C.get(), sentinel)


def test_batched_matmul(cgt):
    # cgt/tests/test_einsum.py, test_affine.py batchedmatmul: (2,3,5) x (2,5,7)
    rs = np.random.RandomState(0)
    x, y = rs.randn(2, 3, 5).astype(np.float32), rs.randn(2, 5, 7).astype(np.float32)
    X, Y = cgt.constant(x), cgt.constant(y)
    Z = cgt.batched_matmul(X, Y)
    np.testing.assert_allclose(Z.get(), np.einsum("nij,njk->nik", x, y), atol=1e-3)
    G = rs.randn(2, 3, 7).astype(np.float32)
    gX, gY = cgt.grad(Z, [X, Y], goutput=G)
    np.testing.assert_allclose(gX.get(), np.einsum("nik,njk->nij", G, y), atol=1e-3)
    np.testing.assert_allclose(gY.get(), np.einsum("nij,nik->njk", x, G), atol=1e-3)


@pytest.mark.parametrize("xshape,fshape,pad,stride", [
    ((4, 1, 28, 28), (32, 1, 3, 3), (1, 1), (1, 1)),
    ((2, 3, 32, 32), (32, 3, 5, 5), (2, 2), (1, 1)),
    ((2, 3, 67, 67), (96, 3, 11, 11), (0, 0), (4, 4)),
    ((2, 32, 28, 28), (48, 32, 3, 3), (1, 1), (1, 1)),
])
def test_conv2d_grad_through_op_pullbacks(cgt, xshape, fshape, pad, stride):
    from cgt_amd import nn
    rs = np.random.RandomState(2)
    xval = rs.randn(*xshape).astype(np.float32)
    fval = (rs.randn(*fshape) / np.sqrt(np.prod(fshape[1:]))).astype(np.float32)
    x, f = cgt.constant(xval), cgt.constant(fval)
    y = nn.conv2d(x, f, kernelshape=fshape[2:], pad=pad, stride=stride)
    y64 = O.conv2d(xval.astype(np.float64), fval.astype(np.float64), pad, stride)
    assert relfro(y.get(), y64) <= TOL
    gy = rs.randn(*y.shape).astype(np.float32)
    gx, gf = cgt.grad(y, [x, f], goutput=gy)
    gx64, gf64 = O.conv2d_pullback(xval.astype(np.float64), fval.astype(np.float64), gy.astype(np.float64), pad, stride)
    assert gx.shape == xshape and gf.shape == fshape
    assert relfro(gx.get(), gx64) <= TOL and relfro(gf.get(), gf64) <= TOL


@pytest.mark.parametrize("shape,axes", [((5, 7), (1, 0)), ((3, 4, 5), (2, 0, 1)), ((3, 4, 5), (0, 2, 1)), ((6,), (0,)),
                                        ((2, 3, 4, 5), (3, 1, 0, 2)), ((1, 9), (1, 0))])
def test_transpose_of_fewer_than_four_axes(cgt, shape, axes):
    # the reference's Transpose takes any rank (cgt/core.py:1559-1594); the device kernel is 4-d, fewer axes
    # ride along as leading extents of 1.  Values, gradient, and a compiled replay at another leading extent
    rs = np.random.RandomState(len(shape))
    xv = rs.randn(*shape).astype(np.float32)
    x = cgt.constant(xv)
    y = cgt.transpose(x, axes)
    assert np.array_equal(y.get(), xv.transpose(axes))
    g = rs.randn(*y.shape).astype(np.float32)
    gx, = cgt.grad(y, [x], goutput=g)
    assert np.array_equal(gx.get(), g.transpose(np.argsort(axes)))
    f = cgt.function([x], y)
    x2 = rs.randn(*((shape[0] + 2,) + shape[1:])).astype(np.float32)
    assert np.array_equal(f(x2), x2.transpose(axes))
    with pytest.raises(ValueError):
        cgt.transpose(x, (axes[0],) * len(axes) if len(axes) > 1 else (1,))        # not a permutation
    with pytest.raises(NotImplementedError):
        cgt.Transpose((0, 1, 2, 3, 4))


def test_conv2d_rejects_a_kernel_larger_than_the_padded_image(cgt):
    from cgt_amd import nn
    x = cgt.constant(np.zeros((2, 3, 4, 9), np.float32))
    f = cgt.constant(np.zeros((5, 3, 5, 5), np.float32))
    with pytest.raises(ValueError, match="larger than"):
        nn.conv2d(x, f, (5, 5))                       # 4 rows, no padding
    assert nn.conv2d(x, f, (5, 5), pad=(1, 0)).shape == (2, 5, 2, 5)
    with pytest.raises(ValueError, match="channels"):
        nn.conv2d(x, cgt.constant(np.zeros((5, 4, 3, 3), np.float32)), (3, 3))
    with pytest.raises(ValueError, match="larger than"):
        nn.SpatialConvolution(3, 5, (5, 5), (0, 0))(x)


def test_cifar_shaped_stack_forward_backward(cgt):
    # the CIFAR-shaped stack in miniature: conv 5x5 p2 -> pool 3x3/2 -> LRN(5,1e-4,.75) -> conv 5x5 p2,
    # loss = sum of outputs; gradients wrt input and both weights.  (The ReLU between
    # conv and pool is an elementwise op outside the hot path and is left out on both sides.)
    from cgt_amd import nn
    rs = np.random.RandomState(0)
    xval = rs.rand(4, 3, 32, 32).astype(np.float32)
    w1 = (0.01 * rs.randn(32, 3, 5, 5)).astype(np.float32)
    w2 = (0.01 * rs.randn(64, 32, 5, 5)).astype(np.float32)
    x, W1, W2 = cgt.constant(xval), cgt.constant(w1), cgt.constant(w2)
    h1 = nn.conv2d(x, W1, (5, 5), pad=(2, 2))
    p1 = nn.max_pool_2d(h1, (3, 3), (0, 0), (2, 2))
    n1 = nn.cross_channel_lrn(p1, 5, 1e-4, 0.75)
    out = nn.conv2d(n1, W2, (5, 5), pad=(2, 2))
    assert p1.shape == (4, 32, 15, 15) and out.shape == (4, 64, 15, 15)
    gx, gW1, gW2 = cgt.grad(out, [x, W1, W2], goutput=np.ones(out.shape, np.float32))
    # the same chain on the oracle, in float64
    d = np.float64
    oh1 = O.conv2d(xval.astype(d), w1.astype(d), (2, 2), (1, 1))
    op1, omask = O.max_pool(oh1, (3, 3), (0, 0), (2, 2))
    on1, oscale = O.lrn_fwd(op1, 5, 1e-4, 0.75)
    oout = O.conv2d(on1, w2.astype(d), (2, 2), (1, 1))
    assert relfro(out.get(), oout) <= TOL
    gn1, ogW2 = O.conv2d_pullback(on1, w2.astype(d), np.ones_like(oout), (2, 2), (1, 1))
    gp1 = O.lrn_bwd(op1, on1, oscale, gn1, 5, 1e-4, 0.75)
    gh1 = O.max_pool_pullback(oh1.shape, omask, gp1)
    ogx, ogW1 = O.conv2d_pullback(xval.astype(d), w1.astype(d), gh1, (2, 2), (1, 1))
    assert np.array_equal(p1.parents[0].value[1].get(), omask), "argmax must match for the gradients to be comparable"
    assert relfro(gW2.get(), ogW2) <= TOL and relfro(gW1.get(), ogW1) <= TOL and relfro(gx.get(), ogx) <= TOL


def test_interpreter_replays_conv_forward_with_buffer_reuse(cgt):
    # Alloc + ReturnByRef instructions fired by the C++ interpreter on device buffers
    from cgt_amd import core, rt
    from cgt_amd.nn_ops.im2col import Im2Col, Im2ColInfo
    rs = np.random.RandomState(3)
    xval = rs.randn(2, 3, 9, 9).astype(np.float32)
    fval = rs.randn(4, 27).astype(np.float32)
    T4, T2 = core.TensorType("f4", 4), core.TensorType("f4", 2)
    im2col_call = core.get_callable(Im2Col(Im2ColInfo(3, 3, 1, 1, 1, 1)), [T4])
    gemm_call = core.get_callable(core.Mul22(False, True), [T2, T2])
    it = rt.Interpreter(12)
    cpu, gpu = rt.CPU, rt.GPU
    it.load_argument(0, (0, gpu))
    it.load_argument(1, (1, gpu))
    for slot, v in [(2, 2), (3, 9), (4, 9), (5, 27), (6, 162), (7, 4)]:
        it.set_slot(slot, v)
    it.alloc(np.float32, [(2, cpu), (3, cpu), (4, cpu), (5, cpu)], (8, gpu))
    it.return_byref(im2col_call, [(0, gpu)], (8, gpu))
    it.alloc(np.float32, [(6, cpu), (7, cpu)], (9, gpu))
    x, f = cgt.to_gpu(xval), cgt.to_gpu(fval)
    ref = O.im2col(xval, (3, 3), (1, 1), (1, 1))
    it.run([x, f])
    assert np.array_equal(it.get_array(8).get(), ref)
    p1 = it.get_array(8).ptr
    it.run([x, f])
    assert it.get_array(8).ptr == p1
    # the GEMM reads the column buffer as [B*m*n, Z]: a reshaped view placed in a slot
    it2 = rt.Interpreter(6)
    it2.load_argument(0, (0, gpu))
    it2.load_argument(1, (1, gpu))
    it2.set_slot(2, 162)
    it2.set_slot(3, 4)
    it2.alloc(np.float32, [(2, cpu), (3, cpu)], (4, gpu))
    it2.return_byref(gemm_call, [(0, gpu), (1, gpu)], (4, gpu))
    it2.run([it.get_array(8).reshape(162, 27), f])
    want = ref.reshape(162, 27).astype(np.float64) @ fval.astype(np.float64).T
    assert relfro(it2.get_array(4).get(), want) <= TOL
