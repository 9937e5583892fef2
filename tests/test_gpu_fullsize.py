"""Full-size runs of the two headline layers (AlexNet conv1 at batch 128, the
VGG 128x56x56 3x3 layer at batch 64), checked where the CPU oracle cannot
cover the whole array in seconds:

* every stage is independent per image (or per row of the GEMM), so the oracle
  is run on a few images / rows of the SAME full-size launch -- first, middle,
  last -- and must match that slice of the device result: bit-exact for
  im2col, col2im, pool values, masks and pool pullback; relative Frobenius
  <= 1e-4 for the GEMMs, conv outputs/gradients and LRN;
* size-independent properties over the whole arrays: <im2col(x), c> equals
  <x, col2im(c)> (adjointness), every mask entry names a cell inside its
  window that holds the pooled value, the pool pullback conserves the sum of
  its cotangent, transposes round-trip bit-exactly.

This is what exercises the launch geometry only large shapes reach (XCD
remapping, row bands, split-K and tail splits, multi-round grids).
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-4

LAYERS = {
    # name: x shape, filter shape, pad, stride, pool (kernel, pad, stride), lrn (size, alpha, beta, k)
    "alexnet_conv1": ((128, 3, 227, 227), (96, 3, 11, 11), (0, 0), (4, 4), ((3, 3), (0, 0), (2, 2)), (5, 1e-4, 0.75, 2.0)),
    "vgg_mid": ((64, 128, 56, 56), (128, 128, 3, 3), (1, 1), (1, 1), ((2, 2), (0, 0), (2, 2)), None),
}


@pytest.fixture(scope="module")
def K():
    from cgt_amd import capi, kernels
    capi.require_gpu()
    return kernels


def gpu(a):
    from cgt_amd.gpuarray import to_gpu
    return to_gpu(a)


def relfro(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300)


def bits_equal(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("name", sorted(LAYERS))
def test_layer_fullsize(K, name):
    xs, fs, pad, stride, pool, lrn = LAYERS[name]
    print("full-size layer", name, xs, fs, flush=True)
    rs = np.random.RandomState(0)
    x = rs.randn(*xs).astype(np.float32)
    f = (rs.randn(*fs) * np.sqrt(1.0 / np.prod(fs[1:]))).astype(np.float32)
    B, C, H, W = xs
    L, _, r, c = fs
    m, n = K.conv_outsize(H, r, pad[0], stride[0]), K.conv_outsize(W, c, pad[1], stride[1])
    Z = C * r * c
    imgs = [0, B // 2 + 1, B - 1]

    # ---- im2col: slices vs oracle (bit-exact)
    xg, fg = gpu(x), gpu(f)
    colg = K.im2col(xg, (r, c), pad, stride)
    col = colg.get()
    for b in imgs:
        assert bits_equal(col[b:b + 1], O.im2col(x[b:b + 1], (r, c), pad, stride)), "im2col image %d" % b

    # ---- forward GEMM (NT): sampled rows vs float64
    y2g = K.mul22(colg.reshape(B * m * n, Z), fg.reshape(L, Z), False, True)
    y2 = y2g.get()
    rows = np.unique(np.concatenate([np.arange(0, 300), rs.randint(0, B * m * n, 1500), np.arange(B * m * n - 300, B * m * n)]))
    ref = col.reshape(-1, Z)[rows].astype(np.float64) @ f.reshape(L, Z).astype(np.float64).T
    assert relfro(y2[rows], ref) <= TOL

    # ---- transpose {0,3,1,2}: whole array, bit-exact
    yg = K.transpose4(y2g.reshape(B, m, n, L), (0, 3, 1, 2))
    y = yg.get()
    assert bits_equal(y, np.ascontiguousarray(y2.reshape(B, m, n, L).transpose(0, 3, 1, 2)))
    del y2

    # ---- LRN forward/backward: slices vs oracle
    act_g, act = yg, y
    if lrn:
        size, alpha, beta, k = lrn
        topg, scaleg = K.lrn_fwd(yg, size, alpha, beta, k)
        top, scale = topg.get(), scaleg.get()
        for b in imgs:
            rt, rsx = O.lrn_fwd(y[b:b + 1], size, alpha, beta, k)
            assert relfro(top[b:b + 1], rt) <= TOL and relfro(scale[b:b + 1], rsx) <= TOL, "lrn_fwd image %d" % b
        act_g, act = topg, top

    # ---- max pool: slices vs oracle (bit-exact) + whole-array mask property
    pk, pp, ps = pool
    poolg, maskg = K.max_pool(act_g, pk, pp, ps)
    pooled, mask = poolg.get(), maskg.get()
    for b in imgs:
        rp, rm = O.max_pool(act[b:b + 1], pk, pp, ps)
        assert np.array_equal(mask[b:b + 1], rm) and bits_equal(pooled[b:b + 1], rp), "max_pool image %d" % b
    PH, PW = pooled.shape[2:]
    assert mask.min() >= 0 and mask.max() < m * n
    mh, mw = mask // n, mask % n
    ph_idx = np.arange(PH).reshape(1, 1, PH, 1) * ps[0] - pp[0]
    pw_idx = np.arange(PW).reshape(1, 1, 1, PW) * ps[1] - pp[1]
    assert np.all((mh >= ph_idx) & (mh < ph_idx + pk[0]) & (mw >= pw_idx) & (mw < pw_idx + pk[1]))
    picked = np.take_along_axis(act.reshape(B, L, m * n), mask.reshape(B, L, PH * PW), axis=2)
    assert bits_equal(picked.reshape(pooled.shape), pooled)

    # ---- pool pullback: slices vs oracle (bit-exact) + conservation of the cotangent
    gpool = rs.randn(*pooled.shape).astype(np.float32)
    gactg = K.max_pool_pullback(act.shape, maskg, gpu(gpool), pk, pp, ps)
    gact = gactg.get()
    for b in imgs:
        assert bits_equal(gact[b:b + 1], O.max_pool_pullback((1,) + act.shape[1:], mask[b:b + 1], gpool[b:b + 1])), \
            "pool pullback image %d" % b
    assert abs(gact.astype(np.float64).sum() - gpool.astype(np.float64).sum()) <= 1e-6 * np.abs(gpool).sum()

    # ---- LRN backward
    gyg, gy = gactg, gact
    if lrn:
        gyg = K.lrn_bwd(yg, topg, scaleg, gactg, size, alpha, beta)
        gy = gyg.get()
        for b in imgs:
            ref = O.lrn_bwd(y[b:b + 1], top[b:b + 1], scale[b:b + 1], gact[b:b + 1], size, alpha, beta)
            assert relfro(gy[b:b + 1], ref) <= TOL, "lrn_bwd image %d" % b
        del top, scale

    # ---- transpose {0,2,3,1}
    gcg = K.transpose4(gyg, (0, 2, 3, 1))
    gc = gcg.get()
    assert bits_equal(gc, np.ascontiguousarray(gy.transpose(0, 2, 3, 1)))
    gc2g = gcg.reshape(B * m * n, L)

    # ---- data-gradient GEMM (NN): sampled rows vs float64
    gcolg = K.mul22(gc2g, fg.reshape(L, Z), False, False)
    gcol = gcolg.get()
    ref = gc.reshape(-1, L)[rows].astype(np.float64) @ f.reshape(L, Z).astype(np.float64)
    assert relfro(gcol.reshape(-1, Z)[rows], ref) <= TOL

    # ---- col2im: slices vs oracle (bit-exact: same add order) + adjointness over the whole arrays
    gxg = K.col2im(gcolg.reshape(B, m, n, Z), xs, (r, c), pad, stride)
    gx = gxg.get()
    for b in imgs:
        assert bits_equal(gx[b:b + 1], O.col2im(gcol.reshape(B, m, n, Z)[b:b + 1], (1,) + xs[1:], (r, c), pad, stride)), \
            "col2im image %d" % b
    lhs = float(np.dot(col.reshape(-1).astype(np.float64), gcol.reshape(-1).astype(np.float64)))
    rhs = float(np.dot(x.reshape(-1).astype(np.float64), gx.reshape(-1).astype(np.float64)))
    scale_ = float(np.linalg.norm(col.reshape(-1).astype(np.float64)) * np.linalg.norm(gcol.reshape(-1).astype(np.float64)))
    assert abs(lhs - rhs) <= 1e-6 * scale_, (lhs, rhs)

    # ---- weight-gradient GEMM (TN, K = B*m*n, split along K): sampled columns vs float64
    gfg = K.mul22(gc2g, colg.reshape(B * m * n, Z), True, False)
    gf = gfg.get()
    cols = np.unique(np.concatenate([np.arange(0, 8), rs.randint(0, Z, 24), np.arange(Z - 8, Z)]))
    ref = gc.reshape(-1, L).astype(np.float64).T @ col.reshape(-1, Z)[:, cols].astype(np.float64)
    assert relfro(gf[:, cols], ref) <= TOL
    # the split-K reduction is ordered: a second launch gives the same bits
    assert bits_equal(K.mul22(gc2g, colg.reshape(B * m * n, Z), True, False).get(), gf)


def test_raw_gemm_fullsize(K):
    """Mul22 4096^3, all four transpose variants, and BatchedMul22 64 x 512^3:
    sampled rows against float64."""
    rs = np.random.RandomState(1)
    n = 4096
    A = rs.uniform(-1, 1, (n, n)).astype(np.float32)
    Bm = rs.uniform(-1, 1, (n, n)).astype(np.float32)
    Ag, Bg = gpu(A), gpu(Bm)
    rows = np.unique(np.concatenate([np.arange(0, 130), rs.randint(0, n, 120), np.arange(n - 130, n)]))
    A64, B64 = A.astype(np.float64), Bm.astype(np.float64)
    for tA in (False, True):
        for tB in (False, True):
            print("Mul22 4096^3", tA, tB, flush=True)
            C = K.mul22(Ag, Bg, tA, tB).get()
            opA = A64.T[rows] if tA else A64[rows]
            ref = opA @ (B64.T if tB else B64)
            assert relfro(C[rows], ref) <= TOL
    P, nb = 64, 512
    bA = rs.uniform(-1, 1, (P, nb, nb)).astype(np.float32)
    bB = rs.uniform(-1, 1, (P, nb, nb)).astype(np.float32)
    C = K.batched_mul22(gpu(bA), gpu(bB)).get()
    ref = np.einsum("pij,pjk->pik", bA.astype(np.float64), bB.astype(np.float64))
    assert relfro(C, ref) <= TOL
