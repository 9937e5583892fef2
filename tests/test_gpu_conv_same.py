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
    Hp, Wp = H + 2 * ph, W + 2 * pw
    plane = (Hp * Wp + 16 + 15) // 16 * 16
    ref = np.zeros(total, np.float32)
    body = ref[:B * C * plane].reshape(B * C, plane)
    img = np.zeros((B * C, Hp, Wp), np.float32)
    img[:, ph:ph + H, pw:pw + W] = x.reshape(B * C, H, W)
    body[:, :Hp * Wp] = img.reshape(B * C, -1)
    return ref


CASES = [
    # B, C, H, W, L, kernel
    (2, 32, 9, 11, 128, (3, 3)),
    (3, 128, 14, 14, 128, (3, 3)),
    (2, 64, 7, 20, 128, (5, 5)),
    (1, 128, 56, 56, 128, (3, 3)),
    (5, 32, 3, 70, 128, (3, 5)),
    (2, 128, 1, 1, 128, (3, 3)),
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


def test_conv_same_fused_bias_and_rectify_match_the_separate_ops(K):
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(11)
    B, C, H, W, L = 3, 64, 10, 13, 128
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


def test_conv_same_supported_rule(K):
    assert K.conv_same_supported(128, 128, (3, 3), (1, 1), (1, 1))
    assert K.conv_same_supported(32, 128, (5, 5), (2, 2), (1, 1))
    assert not K.conv_same_supported(3, 96, (11, 11), (0, 0), (4, 4))     # AlexNet conv1: strided
    assert not K.conv_same_supported(3, 32, (5, 5), (2, 2), (1, 1))       # 3 channels: not a multiple of 16
    assert not K.conv_same_supported(128, 128, (3, 3), (0, 0), (1, 1))    # valid padding
    assert not K.conv_same_supported(128, 128, (2, 2), (0, 0), (1, 1))    # even kernel
    assert not K.conv_same_supported(32, 64, (5, 5), (2, 2), (1, 1))      # 64 filters: no weight-gradient tile
