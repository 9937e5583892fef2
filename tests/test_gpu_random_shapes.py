"""Seeded random shapes and geometries against the oracle: the hand-picked
cases elsewhere aim at known code paths, these sweep the space between them
(kernel / pad / stride combinations the launchers pick tilings for at run
time, ragged extents, channel counts around the chunk sizes).  Bars as
everywhere: bit-exact for im2col / col2im / pooling, relative Frobenius
<= 1e-4 for GEMM and LRN."""
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


def gpu(a):
    from cgt_amd.gpuarray import to_gpu
    return to_gpu(a)


def bits_equal(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


def _conv_cases(n, seed):
    rs = np.random.RandomState(seed)
    hot = [(3, 3, 1, 1, 1, 1), (5, 5, 2, 2, 1, 1), (11, 11, 0, 0, 4, 4), (3, 3, 0, 0, 1, 1), (1, 1, 0, 0, 1, 1)]
    cases = []
    while len(cases) < n:
        if rs.rand() < 0.5:
            kh, kw, ph, pw, sh, sw = hot[rs.randint(len(hot))]
        else:
            kh, kw = rs.randint(1, 8, 2)
            ph, pw = rs.randint(0, kh), rs.randint(0, kw)
            sh, sw = rs.randint(1, 5, 2)
        B, C = rs.randint(1, 4), int(rs.choice([1, 2, 3, 4, 7, 8, 9, 16, 33, 40]))
        H, W = rs.randint(kh, kh + 40), rs.randint(kw, kw + 70)
        if H + 2 * ph < kh or W + 2 * pw < kw or C * kh * kw * H * W * B > 6e6:
            continue
        cases.append(((B, C, int(H), int(W)), (int(kh), int(kw)), (int(ph), int(pw)), (int(sh), int(sw))))
    return cases


@pytest.mark.parametrize("xshape,k,p,s", _conv_cases(48, 11))
def test_im2col_col2im_random(K, xshape, k, p, s):
    print("case", xshape, k, p, s, flush=True)
    rs = np.random.RandomState(0)
    x = rs.randn(*xshape).astype(np.float32)
    ref = O.im2col(x, k, p, s)
    assert bits_equal(K.im2col(gpu(x), k, p, s).get(), ref)
    gcol = (rs.randn(*ref.shape) * 10.0 ** rs.uniform(-3, 3, ref.shape)).astype(np.float32)
    assert bits_equal(K.col2im(gpu(gcol), xshape, k, p, s).get(), O.col2im(gcol, xshape, k, p, s))


def _pool_cases(n, seed):
    rs = np.random.RandomState(seed)
    hot = [(2, 2, 0, 0, 2, 2), (3, 3, 0, 0, 2, 2), (3, 3, 1, 1, 2, 2)]
    cases = []
    while len(cases) < n:
        if rs.rand() < 0.5:
            kh, kw, ph, pw, sh, sw = hot[rs.randint(len(hot))]
        else:
            kh, kw = rs.randint(1, 6, 2)
            ph, pw = rs.randint(0, kh), rs.randint(0, kw)
            sh, sw = rs.randint(1, 4, 2)
        N, C = rs.randint(1, 4), rs.randint(1, 20)
        H, W = rs.randint(kh + 1, kh + 60), rs.randint(kw + 1, kw + 60)
        PH, PW = O.pool_outsize(H, kh, ph, sh), O.pool_outsize(W, kw, pw, sw)
        # the op's shape rule must give windows that start inside the image
        if PH < 1 or PW < 1 or (PH - 1) * sh - ph >= H or (PW - 1) * sw - pw >= W:
            continue
        cases.append(((int(N), int(C), int(H), int(W)), (int(kh), int(kw)), (int(ph), int(pw)), (int(sh), int(sw))))
    return cases


@pytest.mark.parametrize("xshape,k,p,s", _pool_cases(40, 12))
def test_max_pool_random(K, xshape, k, p, s):
    print("case", xshape, k, p, s, flush=True)
    rs = np.random.RandomState(1)
    x = np.round(rs.randn(*xshape) * 2).astype(np.float32) / 2          # plenty of ties
    rtop, rmask = O.max_pool(x, k, p, s)
    top, mask = K.max_pool(gpu(x), k, p, s)
    assert np.array_equal(mask.get(), rmask) and bits_equal(top.get(), rtop)
    g = (rs.randn(*rtop.shape) * 10.0 ** rs.uniform(-3, 3, rtop.shape)).astype(np.float32)
    assert bits_equal(K.max_pool_pullback(xshape, mask, gpu(g), k, p, s).get(), O.max_pool_pullback(xshape, rmask, g))


def _lrn_cases(n, seed):
    rs = np.random.RandomState(seed)
    cases = []
    for _ in range(n):
        size = int(rs.randint(1, 12))
        C = int(size + rs.randint(0, 40))
        cases.append(((int(rs.randint(1, 4)), C, int(rs.randint(1, 30)), int(rs.randint(1, 30))), size,
                      float(10.0 ** rs.uniform(-4, -1)), float(rs.choice([0.5, 0.75, 1.0])), float(rs.choice([1.0, 2.0]))))
    return cases


@pytest.mark.parametrize("shape,size,alpha,beta,k", _lrn_cases(24, 13))
def test_lrn_random(K, shape, size, alpha, beta, k):
    print("case", shape, size, alpha, beta, k, flush=True)
    rs = np.random.RandomState(2)
    x = rs.randn(*shape).astype(np.float32)
    rtop, rscale = O.lrn_fwd(x, size, alpha, beta, k)
    top, scale = K.lrn_fwd(gpu(x), size, alpha, beta, k)
    assert relfro(top.get(), rtop) <= TOL and relfro(scale.get(), rscale) <= TOL
    g = rs.randn(*shape).astype(np.float32)
    ref = O.lrn_bwd(x, rtop, rscale, g, size, alpha, beta)
    assert relfro(K.lrn_bwd(gpu(x), gpu(rtop), gpu(rscale), gpu(g), size, alpha, beta).get(), ref) <= TOL


def _gemm_cases(n, seed):
    rs = np.random.RandomState(seed)
    cases = []
    for _ in range(n):
        kind = rs.randint(4)
        if kind == 0:
            M, N, Kd = rs.randint(1, 300, 3)
        elif kind == 1:      # tall and thin, conv forward / data gradient
            M, N, Kd = rs.randint(2000, 60000), rs.randint(1, 200), rs.randint(1, 400)
        elif kind == 2:      # weight gradient: long K, split along K
            M, N, Kd = rs.randint(1, 200), rs.randint(1, 500), rs.randint(1500, 40000)
        else:
            M, N, Kd = rs.randint(100, 1500, 3)
        cases.append((int(M), int(N), int(Kd), bool(rs.randint(2)), bool(rs.randint(2))))
    return cases


@pytest.mark.parametrize("M,N,Kd,tA,tB", _gemm_cases(40, 14))
def test_mul22_random(K, M, N, Kd, tA, tB):
    print("case", M, N, Kd, tA, tB, flush=True)
    rs = np.random.RandomState(3)
    A = rs.uniform(-1, 1, (Kd, M) if tA else (M, Kd)).astype(np.float32)
    B = rs.uniform(-1, 1, (N, Kd) if tB else (Kd, N)).astype(np.float32)
    ref = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
    C = K.mul22(gpu(A), gpu(B), tA, tB).get()
    assert C.shape == (M, N) and relfro(C, ref) <= 2e-6
