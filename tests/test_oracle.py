"""Pins the CPU oracle (oracle/cgt_oracle.c) before anything is compared to it.

Three kinds of evidence, none of which retypes the oracle's own formula:
  * the golden vectors written from the reference's own im2col.h / pooling.h
    (tests/golden/*.npz), and the compiled reference itself where it is built;
  * library routines that compute the same thing by other means
    (torch unfold / max_pool2d / local_response_norm / conv2d + autograd,
    scipy.signal.convolve2d as the reference's own test_conv does, np.matmul);
  * what the mathematics fixes: the adjoint identity <im2col x, y> = <x, col2im y>,
    finite differences (the reference's own method for pool / LRN), brute force
    on tiny inputs.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O
from oracle import ref as R

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _load(name):
    z = np.load(os.path.join(GOLD, name))
    return z, json.loads(str(z["meta"]))


def _kps(g):
    return tuple(g[0:2]), tuple(g[2:4]), tuple(g[4:6])


# ---------------------------------------------------------------- goldens

def test_im2col_col2im_golden_bit_exact():
    z, meta = _load("im2col_col2im.npz")
    assert len(meta) >= 14
    for i, m in enumerate(meta):
        k, p, s = _kps(m["geom"])
        x = z["c%d_x" % i]
        col = O.im2col(x, k, p, s)
        assert col.shape == z["c%d_col" % i].shape
        assert np.array_equal(col.view(np.uint32), z["c%d_col" % i].view(np.uint32)), m
        gim = O.col2im(z["c%d_gcol" % i], x.shape, k, p, s)
        assert np.array_equal(gim.view(np.uint32), z["c%d_gim" % i].view(np.uint32)), m


def test_max_pool_golden_bit_exact():
    z, meta = _load("max_pool.npz")
    assert len(meta) >= 11
    for i, m in enumerate(meta):
        k, p, s = _kps(m["geom"])
        x = z["c%d_x" % i]
        top, mask = O.max_pool(x, k, p, s)
        assert np.array_equal(mask, z["c%d_mask" % i]), m
        assert np.array_equal(top.view(np.uint32), z["c%d_top" % i].view(np.uint32)), m
        gb = O.max_pool_pullback(x.shape, mask, z["c%d_gtop" % i])
        assert np.array_equal(gb.view(np.uint32), z["c%d_gbottom" % i].view(np.uint32)), m


def test_golden_layout_fact_from_reference_test():
    # cgt/tests/test_imgproc.py:75-77: col[0,0,0] == x[0,:,0:4,0:4].flatten()
    z, meta = _load("im2col_col2im.npz")
    x, col = z["c0_x"], z["c0_col"]
    assert meta[0]["geom"] == [4, 4, 0, 0, 1, 1]
    assert np.array_equal(col[0, 0, 0], x[0, :, 0:4, 0:4].flatten())


@pytest.mark.skipif(not R.available(), reason="oracle/_ref not built (no reference tree)")
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_oracle_vs_compiled_reference(dtype):
    rs = np.random.RandomState(7)
    for g in R.GEOMS:
        k, p, s = _kps(g)
        H, W = rs.randint(max(k[0], 3), 20), rs.randint(max(k[1], 3), 20)
        x = rs.randn(2, 3, H, W).astype(dtype)
        col = O.im2col(x, k, p, s)
        assert np.array_equal(col, R.im2col(x, k, p, s)), g
        gcol = (rs.randn(*col.shape) * 10.0 ** rs.uniform(-5, 5, col.shape)).astype(dtype)
        assert np.array_equal(O.col2im(gcol, x.shape, k, p, s), R.col2im(gcol, x.shape, k, p, s)), g
        if H + 2 * p[0] > k[0] and W + 2 * p[1] > k[1]:
            top, mask = O.max_pool(x, k, p, s)
            rtop, rmask = R.max_pool(x, k, p, s)
            assert np.array_equal(mask, rmask) and np.array_equal(top, rtop), g
            gt = rs.randn(*top.shape).astype(dtype)
            assert np.array_equal(O.max_pool_pullback(x.shape, mask, gt),
                                  R.max_pool_pullback(x.shape, rmask, gt)), g


# ---------------------------------------------------------------- shape rules

def test_shape_rules():
    # pooled = ceil((H+2p-k)/s), no +1: reference test_pool gets (2,3,1,3)
    assert O.max_pool(np.zeros((2, 3, 5, 7), np.float32), (4, 4), (0, 0), (1, 1))[0].shape == (2, 3, 1, 3)
    assert O.pool_outsize(28, 2, 0, 2) == 13
    assert O.pool_outsize(32, 3, 0, 2) == 15
    assert O.pool_outsize(55, 3, 0, 2) == 26
    assert O.pool_outsize(56, 2, 0, 2) == 27
    assert O.conv_outsize(227, 11, 0, 4) == 55
    assert O.conv_outsize(56, 3, 1, 1) == 56
    assert O.im2col(np.zeros((2, 3, 9, 11), np.float32), (3, 3), (1, 1), (2, 2)).shape == (2, 5, 6, 27)


# ---------------------------------------------------------------- im2col / col2im identities

GEOMS = [((3, 3), (1, 1), (1, 1)), ((5, 5), (2, 2), (1, 1)), ((11, 11), (0, 0), (4, 4)),
         ((4, 7), (3, 6), (1, 1)), ((2, 3), (0, 1), (3, 2)), ((3, 2), (1, 0), (2, 1))]


@pytest.mark.parametrize("k,p,s", GEOMS)
def test_im2col_equals_torch_unfold(k, p, s):
    rs = np.random.RandomState(3)
    x = rs.randn(2, 3, 23, 19).astype(np.float32)
    col = O.im2col(x, k, p, s)
    B, m, n, Z = col.shape
    u = F.unfold(torch.from_numpy(x), k, padding=p, stride=s)  # [B, Z, m*n], Z = (c, kh, kw)
    assert np.array_equal(col.reshape(B, m * n, Z), u.transpose(1, 2).numpy())


@pytest.mark.parametrize("k,p,s", GEOMS)
def test_col2im_is_adjoint_of_im2col(k, p, s):
    rs = np.random.RandomState(4)
    x = rs.randn(2, 2, 17, 21)
    col = O.im2col(x, k, p, s)
    y = rs.randn(*col.shape)
    lhs = float((col * y).sum())
    rhs = float((x * O.col2im(y, x.shape, k, p, s)).sum())
    assert abs(lhs - rhs) <= 1e-10 * max(1.0, abs(lhs))
    # and equals torch fold (sum of overlapping patches)
    B, m, n, Z = col.shape
    fold = F.fold(torch.from_numpy(y.reshape(B, m * n, Z)).transpose(1, 2), x.shape[2:], k,
                  padding=p, stride=s).numpy()
    np.testing.assert_allclose(O.col2im(y, x.shape, k, p, s), fold, rtol=1e-12, atol=1e-12)


def test_col2im_add_order_is_ascending_z():
    # One pixel fed by three taps whose magnitudes make the result depend on
    # the order: ((0 + 1e8) + -1e8) + 1 = 1, while 1e8 + (-1e8 + 1) = 0.
    # 1x3 kernel, pad 1: pixel wp=1 receives col[w=2, wo=0], col[w=1, wo=1],
    # col[w=0, wo=2], i.e. z = 0, 1, 2 in the reference's outer loop.
    a, b, c = np.float32(1e8), np.float32(-1e8), np.float32(1.0)
    k, p, s = (1, 3), (0, 1), (1, 1)
    col = np.zeros((1, 1, 3, 3), np.float32)
    col[0, 0, 2, 0], col[0, 0, 1, 1], col[0, 0, 0, 2] = a, b, c
    im = O.col2im(col, (1, 1, 1, 3), k, p, s)
    assert im[0, 0, 0, 1] == np.float32(1.0)
    assert np.float32(a + np.float32(b + c)) == np.float32(0.0)  # the other order differs


# ---------------------------------------------------------------- pooling identities

POOLS = [((2, 2), (0, 0), (2, 2)), ((3, 3), (0, 0), (2, 2)), ((4, 4), (0, 0), (1, 1)),
         ((3, 3), (1, 1), (2, 2)), ((2, 3), (0, 1), (2, 1))]


@pytest.mark.parametrize("k,p,s", POOLS)
def test_max_pool_equals_torch_cropped(k, p, s):
    rs = np.random.RandomState(5)
    x = rs.randn(2, 3, 14, 17).astype(np.float32)
    top, mask = O.max_pool(x, k, p, s)
    t, idx = F.max_pool2d(torch.from_numpy(x), k, stride=s, padding=p, return_indices=True)
    PH, PW = top.shape[2:]
    assert np.array_equal(top, t.numpy()[:, :, :PH, :PW])
    assert np.array_equal(mask, idx.numpy()[:, :, :PH, :PW].astype(np.int32))


def test_max_pool_brute_force_ties_and_padding():
    rs = np.random.RandomState(6)
    x = rs.randint(-2, 3, size=(2, 2, 7, 8)).astype(np.float32)  # many ties
    k, p, s = (3, 3), (1, 1), (2, 2)
    top, mask = O.max_pool(x, k, p, s)
    N, C, PH, PW = top.shape
    assert (PH, PW) == (3, 4)
    for n in range(N):
        for c in range(C):
            for y in range(PH):
                for xx in range(PW):
                    best, arg = None, -1
                    for h in range(y * s[0] - p[0], y * s[0] - p[0] + k[0]):
                        for w in range(xx * s[1] - p[1], xx * s[1] - p[1] + k[1]):
                            if 0 <= h < 7 and 0 <= w < 8 and (best is None or x[n, c, h, w] > best):
                                best, arg = x[n, c, h, w], h * 8 + w
                    assert top[n, c, y, xx] == best and mask[n, c, y, xx] == arg


def test_max_pool_pullback_finite_difference():
    # the reference's test_pool: (2,3,5,7), k=4, s=1, double, numeric grad of (y*h).sum()
    np.random.seed(0)
    x = np.random.randn(2, 3, 5, 7)
    k, p, s = (4, 4), (0, 0), (1, 1)
    top, mask = O.max_pool(x, k, p, s)
    h = np.random.randn(*top.shape)
    gana = O.max_pool_pullback(x.shape, mask, h)
    gnum = np.zeros_like(x)
    eps = 1e-6
    for i in range(x.size):
        xp = x.copy().ravel(); xp[i] += eps
        xm = x.copy().ravel(); xm[i] -= eps
        fp = (O.max_pool(xp.reshape(x.shape), k, p, s)[0] * h).sum()
        fm = (O.max_pool(xm.reshape(x.shape), k, p, s)[0] * h).sum()
        gnum.ravel()[i] = (fp - fm) / (2 * eps)
    assert np.allclose(gnum, gana, atol=1e-6)


def test_max_pool_pullback_equals_torch_autograd():
    rs = np.random.RandomState(8)
    x = rs.randn(2, 3, 11, 13)
    k, p, s = (3, 3), (0, 0), (2, 2)
    top, mask = O.max_pool(x, k, p, s)
    g = rs.randn(*top.shape)
    xt = torch.from_numpy(x).requires_grad_()
    t = F.max_pool2d(xt, k, stride=s, padding=p)[:, :, :top.shape[2], :top.shape[3]]
    (t * torch.from_numpy(g)).sum().backward()
    np.testing.assert_allclose(O.max_pool_pullback(x.shape, mask, g), xt.grad.numpy(), rtol=1e-13, atol=1e-13)


# ---------------------------------------------------------------- LRN

def _lrn_window_direct(x, size, alpha, k, pre, post):
    """scale by direct window sum with explicit window [c-pre, c+post]."""
    N, C, H, W = x.shape
    sq = x.astype(np.float64) ** 2
    scale = np.empty_like(sq)
    for c in range(C):
        lo, hi = max(0, c - pre), min(C - 1, c + post)
        scale[:, c] = k + (alpha / size) * sq[:, lo:hi + 1].sum(axis=1)
    return scale


@pytest.mark.parametrize("size,C", [(5, 32), (3, 7), (5, 5), (1, 4)])
@pytest.mark.parametrize("k", [1.0, 2.0])
def test_lrn_fwd_equals_torch_odd_sizes(size, C, k):
    rs = np.random.RandomState(9)
    x = rs.randn(2, C, 6, 5)
    alpha, beta = 0.1, 0.75
    top, scale = O.lrn_fwd(x, size, alpha, beta, k)
    ref = F.local_response_norm(torch.from_numpy(x), size, alpha=alpha, beta=beta, k=k).numpy()
    np.testing.assert_allclose(top, ref, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(top, x * scale ** (-beta), rtol=1e-13)


def test_lrn_fwd_even_size_window_alignment():
    # size 4 (the reference's test_lrn): forward window is [c-1, c+2]
    # (pre_pad = (size-1)/2 = 1, post_pad = 2, lrn.cuh:15-16)
    rs = np.random.RandomState(10)
    x = rs.randn(2, 8, 4, 4)
    top, scale = O.lrn_fwd(x, 4, 0.1, 0.5)
    np.testing.assert_allclose(scale, _lrn_window_direct(x, 4, 0.1, 1.0, 1, 2), rtol=1e-13)
    wrong = _lrn_window_direct(x, 4, 0.1, 1.0, 2, 1)
    assert not np.allclose(scale, wrong, rtol=1e-6)


def test_lrn_fwd_f32_close_to_f64():
    rs = np.random.RandomState(11)
    x = rs.randn(3, 16, 5, 7)
    t64, s64 = O.lrn_fwd(x, 5, 1e-4, 0.75)
    t32, s32 = O.lrn_fwd(x.astype(np.float32), 5, 1e-4, 0.75)
    assert np.linalg.norm(t32 - t64) / np.linalg.norm(t64) < 1e-6
    assert np.linalg.norm(s32 - s64) / np.linalg.norm(s64) < 1e-6


@pytest.mark.parametrize("size", [4, 5, 3])
def test_lrn_bwd_finite_difference(size):
    # the reference's test_lrn: randn(4,8,16,16) (smaller plane here), alpha .1, beta .5, double, eps 1e-5
    np.random.seed(0)
    x = np.random.randn(2, 8, 3, 4)
    alpha, beta = 0.1, 0.5
    top, scale = O.lrn_fwd(x, size, alpha, beta)
    a = np.random.rand(*top.shape)
    gana = O.lrn_bwd(x, top, scale, a, size, alpha, beta)
    gnum = np.zeros_like(x)
    eps = 1e-5
    for i in range(x.size):
        xp = x.copy().ravel(); xp[i] += eps
        xm = x.copy().ravel(); xm[i] -= eps
        fp = (O.lrn_fwd(xp.reshape(x.shape), size, alpha, beta)[0] * a).sum()
        fm = (O.lrn_fwd(xm.reshape(x.shape), size, alpha, beta)[0] * a).sum()
        gnum.ravel()[i] = (fp - fm) / (2 * eps)
    assert np.allclose(gnum, gana, atol=1e-8)


def test_lrn_bwd_equals_torch_autograd_odd():
    rs = np.random.RandomState(12)
    x = rs.randn(2, 12, 5, 6)
    size, alpha, beta = 5, 0.3, 0.75
    top, scale = O.lrn_fwd(x, size, alpha, beta)
    g = rs.randn(*x.shape)
    xt = torch.from_numpy(x).requires_grad_()
    (F.local_response_norm(xt, size, alpha=alpha, beta=beta, k=1.0) * torch.from_numpy(g)).sum().backward()
    np.testing.assert_allclose(O.lrn_bwd(x, top, scale, g, size, alpha, beta), xt.grad.numpy(), rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- GEMM

@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
def test_mul22_equals_numpy(tA, tB):
    rs = np.random.RandomState(13)
    M, N, K = 7, 11, 13
    A = rs.randn(K, M) if tA else rs.randn(M, K)
    B = rs.randn(N, K) if tB else rs.randn(K, N)
    ref = (A.T if tA else A) @ (B.T if tB else B)
    np.testing.assert_allclose(O.mul22(A, B, tA, tB), ref, rtol=1e-13)
    A32, B32 = A.astype(np.float32), B.astype(np.float32)
    np.testing.assert_allclose(O.mul22(A32, B32, tA, tB), ref, rtol=1e-5, atol=1e-5)


def test_batched_mul22_equals_einsum():
    # reference test_einsum / batchedmatmul: (2,3,5) x (2,5,7)
    rs = np.random.RandomState(14)
    x, y = rs.randn(2, 3, 5), rs.randn(2, 5, 7)
    np.testing.assert_allclose(O.batched_mul22(x, y), np.einsum("nij,njk->nik", x, y), rtol=1e-13)
    np.testing.assert_allclose(O.batched_mul22(x.transpose(0, 2, 1).copy(), y, tA=True),
                               np.einsum("nij,njk->nik", x, y), rtol=1e-13)
    np.testing.assert_allclose(O.batched_mul22(x, y.transpose(0, 2, 1).copy(), tB=True),
                               np.einsum("nij,njk->nik", x, y), rtol=1e-13)


def test_transpose4():
    x = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    for axes in [(0, 3, 1, 2), (0, 2, 3, 1), (3, 2, 1, 0)]:
        assert np.array_equal(O.transpose4(x, axes), x.transpose(axes))


# ---------------------------------------------------------------- conv2d composition

def test_conv2d_reference_known_answer():
    # cgt/tests/test_conv.py:14-33, same legacy RNG stream and shapes
    import scipy.signal
    np.random.seed(0)
    x = np.random.randn(2, 2, 5, 17)
    filt = np.random.randn(3, 2, 4, 7)
    out = np.zeros((2, 3, 5 + 4 - 1, 17 + 7 - 1))
    for b in range(2):
        for ic in range(2):
            for oc in range(3):
                out[b, oc] += scipy.signal.convolve2d(x[b, ic], filt[oc, ic][::-1, ::-1], mode="full")
    np.testing.assert_allclose(O.conv2d(x, filt, pad=(3, 6)), out, atol=1e-6)
    np.testing.assert_allclose(O.conv2d(x.astype(np.float32), filt.astype(np.float32), pad=(3, 6)), out, atol=1e-3)


@pytest.mark.parametrize("k,p,s", [((3, 3), (1, 1), (1, 1)), ((5, 5), (2, 2), (1, 1)), ((11, 11), (0, 0), (4, 4)), ((3, 2), (1, 0), (2, 1))])
def test_conv2d_fwd_bwd_equals_torch(k, p, s):
    rs = np.random.RandomState(15)
    x = rs.randn(2, 3, 19, 23)
    f = rs.randn(4, 3, *k)
    y = O.conv2d(x, f, p, s)
    xt, ft = torch.from_numpy(x).requires_grad_(), torch.from_numpy(f).requires_grad_()
    yt = F.conv2d(xt, ft, stride=s, padding=p)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-11, atol=1e-11)
    gy = rs.randn(*y.shape)
    (yt * torch.from_numpy(gy)).sum().backward()
    gx, gf = O.conv2d_pullback(x, f, gy, p, s)
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(gf, ft.grad.numpy(), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape,kernel", [((2, 3, 5, 7), (3, 3)), ((1, 2, 4, 9), (5, 3)), ((3, 1, 6, 6), (1, 7)), ((1, 1, 1, 1), (3, 5))])
def test_padded_plane_layout_puts_every_tap_at_a_plain_offset(shape, kernel):
    # the layout the column-buffer-free products read (no reference counterpart): tap (ho, wo) of the
    # padded-grid pixel q = h * Wp + w must be the float at q + ho * Wp + wo of its plane, equal to
    # x[h + ho - ph, w + wo - pw] or zero outside the image -- checked against numpy's own padding
    from cgt_amd import capi
    B, C, H, W = shape
    kh, kw = kernel
    ph, pw = (kh - 1) // 2, (kw - 1) // 2
    rs = np.random.RandomState(kh * 10 + W)
    x = rs.randn(*shape).astype(np.float32)
    total = capi.lib().cgt_amd_conv_same_padded_size(B * C, H, W, kh, kw)
    flat = O.conv_same_padded(x, kernel, total)
    Wp = W + pw
    plane = (total - (256 + kh * Wp + 3) // 4 * 4) // (B * C)
    assert plane * B * C + (256 + kh * Wp + 3) // 4 * 4 == total and plane % 16 == 0
    ref = np.pad(x.reshape(B * C, H, W), ((0, 0), (ph, ph), (pw, pw)))
    planes = np.concatenate([flat, np.zeros(kh * Wp + kw, np.float32)])      # reads of the last plane's taps run into the tail
    for p in range(B * C):
        for ho in range(kh):
            for wo in range(kw):
                for h in range(H):
                    got = planes[p * plane + h * Wp + ho * Wp + wo: p * plane + h * Wp + ho * Wp + wo + W]
                    assert np.array_equal(got, ref[p, h + ho, wo:wo + W]), (p, ho, wo, h)
    # everything that is not a pixel is zero, and every pixel appears exactly once
    assert np.count_nonzero(flat) == np.count_nonzero(x) and abs(float(flat.sum(dtype=np.float64)) - float(x.sum(dtype=np.float64))) < 1e-3
