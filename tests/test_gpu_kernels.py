"""Parity of the HIP kernels (through the C ABI in libcgt_amd.so) with the CPU
oracle and the reference-compiled golden vectors, on the same seeded inputs.

Bars: bit-exact for im2col / col2im / pool values, argmax masks and pool
pullback; relative Frobenius error <= 1e-4 for GEMM, conv and LRN outputs and
gradients (TOL below).
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-4  # relative Frobenius bound for fp32 GEMM / conv / LRN
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def K():
    from cgt_amd import capi, kernels
    capi.require_gpu()
    print("device:", capi.device_name(), flush=True)
    return kernels


def gpu(a, dtype=None):
    from cgt_amd.gpuarray import to_gpu
    return to_gpu(a, dtype)


def relfro(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    d = np.linalg.norm(a - b)
    n = np.linalg.norm(b)
    return d / n if n > 0 else d


def bits_equal(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def _load(name):
    z = np.load(os.path.join(GOLD, name))
    return z, json.loads(str(z["meta"]))


def _kps(g):
    return tuple(g[0:2]), tuple(g[2:4]), tuple(g[4:6])


# ---------------------------------------------------------------- golden vectors

def test_im2col_col2im_golden(K):
    z, meta = _load("im2col_col2im.npz")
    for i, m in enumerate(meta):
        print("golden im2col case", i, m, flush=True)
        k, p, s = _kps(m["geom"])
        x = z["c%d_x" % i]
        col = K.im2col(gpu(x), k, p, s).get()
        assert bits_equal(col, z["c%d_col" % i]), m
        gim = K.col2im(gpu(z["c%d_gcol" % i]), x.shape, k, p, s).get()
        assert bits_equal(gim, z["c%d_gim" % i]), m


def test_max_pool_golden(K):
    z, meta = _load("max_pool.npz")
    for i, m in enumerate(meta):
        print("golden pool case", i, m, flush=True)
        k, p, s = _kps(m["geom"])
        x = z["c%d_x" % i]
        top, mask = K.max_pool(gpu(x), k, p, s)
        assert np.array_equal(mask.get(), z["c%d_mask" % i]), m
        assert bits_equal(top.get(), z["c%d_top" % i]), m
        gb = K.max_pool_pullback(x.shape, mask, gpu(z["c%d_gtop" % i]), k, p, s).get()
        assert bits_equal(gb, z["c%d_gbottom" % i]), m


# ---------------------------------------------------------------- im2col / col2im vs oracle

IM2COL_CASES = [
    # (xshape, kernel, pad, stride)  -- miniatures of the configured layers first
    ((4, 1, 28, 28), (3, 3), (1, 1), (1, 1)),      # MNIST conv
    ((3, 3, 32, 32), (5, 5), (2, 2), (1, 1)),      # CIFAR conv1
    ((2, 32, 15, 15), (5, 5), (2, 2), (1, 1)),     # CIFAR conv2 (odd plane, Z=800)
    ((2, 3, 227, 227), (11, 11), (0, 0), (4, 4)),  # AlexNet conv1, full plane
    ((1, 128, 56, 56), (3, 3), (1, 1), (1, 1)),    # VGG mid layer, full plane (channel chunks)
    ((2, 130, 20, 24), (3, 3), (1, 1), (1, 1)),    # C not a multiple of the chunk
    ((2, 7, 13, 9), (3, 3), (0, 0), (1, 1)),       # Z = 63: scalar-store path
    ((2, 5, 10, 11), (1, 1), (0, 0), (1, 1)),
    ((2, 2, 5, 17), (4, 7), (3, 6), (1, 1)),       # runtime geometry, full padding
    ((2, 2, 10, 11), (2, 3), (0, 1), (3, 2)),      # stride > kernel
    ((2, 4, 13, 14), (5, 3), (2, 1), (2, 3)),
    ((1, 1, 3, 20000), (3, 3), (1, 1), (1, 1)),    # row too wide for LDS staging
    ((1, 2, 4, 6), (4, 6), (0, 0), (1, 1)),        # single output pixel
    ((2, 6, 30, 40), (5, 5), (2, 2), (1, 1)),      # 5x5 row-streamed col2im, partial channel chunk
    ((1, 20, 17, 70), (3, 3), (0, 0), (1, 1)),     # two column tiles, partial row tile
    ((1, 16, 56, 56), (3, 3), (1, 1), (1, 1)),
    ((1, 3, 100, 300), (11, 11), (0, 0), (4, 4)),  # three column tiles at stride 4
    ((1, 2, 5, 2000), (3, 3), (1, 1), (1, 1)),     # rows longer than one pipelined staging buffer
    ((2, 40, 9, 30), (3, 3), (1, 1), (1, 1)),      # several channel chunks, last one partial
    ((3, 20, 11, 12), (3, 3), (1, 1), (1, 1)),     # narrow image: 16 lanes per row, 4 channels abreast, partial chunk
    ((2, 9, 7, 20), (3, 3), (0, 0), (1, 1)),       # 32 lanes per row
    ((2, 6, 9, 20), (5, 5), (2, 2), (1, 1)),       # 5x5, 32 lanes per row, partial chunk
    ((2, 12, 10, 10), (5, 5), (2, 2), (1, 1)),     # 5x5, 16 lanes per row, partial chunk
    ((4, 64, 15, 15), (5, 5), (2, 2), (1, 1)),     # CIFAR conv2 at full channel count
    # col2im with a tile as wide as the image: finished rows leave through LDS in batches of 8 per channel
    ((2, 10, 37, 45), (3, 3), (1, 1), (1, 1)),     # odd width: batches start at any alignment, partial chunk, partial top batch
    ((2, 8, 19, 64), (3, 3), (0, 0), (1, 1)),      # full 64-wide tile, no padding
    ((1, 4, 70, 33), (5, 5), (2, 2), (1, 1)),      # 5x5, 32 lanes per row, several bands
    # odd Z with every channel staged at once: the row's region is written as aligned 16-byte units
    ((5, 3, 23, 27), (11, 11), (0, 0), (4, 4)),    # Z = 363, regions of 1815 floats: every start alignment
    ((3, 5, 9, 11), (3, 3), (1, 1), (1, 1)),       # Z = 45, a region shorter than one pass
    ((6, 1, 6, 7), (3, 3), (0, 0), (1, 1)),        # Z = 9: a unit straddles pixels, three LDS rows in all
    ((2, 13, 20, 57), (11, 11), (0, 0), (4, 4)),   # Z = 1573 > one pass of 1024 floats
    ((3, 7, 40, 41), (5, 5), (2, 2), (1, 1)),      # Z = 175, several passes per region
]


@pytest.mark.parametrize("xshape,k,p,s", IM2COL_CASES)
def test_im2col_col2im_vs_oracle(K, xshape, k, p, s):
    print("im2col case", xshape, k, p, s, flush=True)
    rs = np.random.RandomState(0)
    x = rs.randn(*xshape).astype(np.float32)
    ref = O.im2col(x, k, p, s)
    col = K.im2col(gpu(x), k, p, s).get()
    assert bits_equal(col, ref)
    gcol = (rs.randn(*ref.shape) * 10.0 ** rs.uniform(-4, 4, ref.shape)).astype(np.float32)
    gim = K.col2im(gpu(gcol), xshape, k, p, s).get()
    assert bits_equal(gim, O.col2im(gcol, xshape, k, p, s))


def test_im2col_output_fully_overwritten(K):
    # the interpreter reuses output buffers without clearing them
    from cgt_amd.gpuarray import empty
    rs = np.random.RandomState(1)
    x = rs.randn(2, 3, 9, 9).astype(np.float32)
    k, p, s = (3, 3), (1, 1), (2, 2)
    ref = O.im2col(x, k, p, s)
    out = empty(ref.shape).fill_u32(0x7FC00000)  # NaN
    K.im2col(gpu(x), k, p, s, out=out)
    assert bits_equal(out.get(), ref)
    im = empty(x.shape).fill_u32(0x7FC00000)
    K.col2im(gpu(ref), x.shape, k, p, s, out=im)
    assert bits_equal(im.get(), O.col2im(ref, x.shape, k, p, s))


# ---------------------------------------------------------------- pooling vs oracle

POOL_CASES = [
    ((4, 32, 28, 28), (2, 2), (0, 0), (2, 2)),     # MNIST block -> 13x13
    ((2, 32, 32, 32), (3, 3), (0, 0), (2, 2)),     # CIFAR -> 15x15
    ((2, 96, 55, 55), (3, 3), (0, 0), (2, 2)),     # AlexNet -> 26x26
    ((2, 128, 56, 56), (2, 2), (0, 0), (2, 2)),    # VGG -> 27x27
    ((2, 3, 5, 7), (4, 4), (0, 0), (1, 1)),        # reference test_pool
    ((2, 3, 9, 10), (3, 3), (1, 1), (2, 2)),       # padding
    ((3, 2, 9, 13), (2, 3), (0, 1), (2, 1)),
    ((1, 2, 130, 120), (3, 3), (0, 0), (2, 2)),    # plane too large for LDS staging
    ((1, 1, 3, 3), (2, 2), (0, 0), (2, 2)),        # one output
    ((2, 3, 11, 13), (3, 3), (1, 1), (2, 2)),      # compiled-in geometry, odd extents, padding
    ((3, 4, 7, 9), (2, 2), (0, 0), (2, 2)),        # odd width: no paired stores in the pullback
    ((600, 9, 6, 6), (2, 2), (0, 0), (2, 2)),      # many small planes per workgroup
    ((2, 3, 12, 16), (3, 3), (1, 1), (2, 2)),      # W % 4 == 0: the pullback writes 16-byte rows (overlapping windows, padding)
    ((3, 5, 4, 4), (2, 2), (0, 0), (2, 2)),        # one 16-byte unit per row
    ((2, 2, 9, 8), (3, 3), (0, 0), (2, 2)),
    # odd planes, overlapping windows: the pullback goes through LDS in runs of planes that start at
    # every 16-byte phase; input runs whose last 16-byte unit is cut by the end of the arrays
    ((7, 3, 5, 7), (3, 3), (0, 0), (2, 2)),
    ((5, 13, 9, 11), (3, 3), (1, 1), (2, 2)),
    ((1, 1, 3, 5), (3, 3), (0, 0), (2, 2)),
    ((37, 59, 7, 7), (3, 3), (0, 0), (2, 2)),      # several planes per workgroup, the last workgroup short
    ((3, 1, 55, 55), (3, 3), (0, 0), (2, 2)),
    ((1, 5, 1, 9), (3, 3), (1, 1), (2, 2)),
]


@pytest.mark.parametrize("xshape,k,p,s", POOL_CASES)
@pytest.mark.parametrize("kind", ["randn", "relu_ties"])
def test_max_pool_vs_oracle(K, xshape, k, p, s, kind):
    print("pool case", xshape, k, p, s, kind, flush=True)
    rs = np.random.RandomState(2)
    x = rs.randn(*xshape).astype(np.float32)
    if kind == "relu_ties":
        x = O.rectify(np.round(x * 2) / 2).astype(np.float32)   # many exact ties and zeros
    rtop, rmask = O.max_pool(x, k, p, s)
    top, mask = K.max_pool(gpu(x), k, p, s)
    assert np.array_equal(mask.get(), rmask)
    assert bits_equal(top.get(), rtop)
    gtop = (rs.randn(*rtop.shape) * 10.0 ** rs.uniform(-4, 4, rtop.shape)).astype(np.float32)
    gb = K.max_pool_pullback(xshape, mask, gpu(gtop), k, p, s).get()
    assert bits_equal(gb, O.max_pool_pullback(xshape, rmask, gtop))


def test_max_pool_all_negative_and_constant(K):
    x = -np.ones((1, 2, 6, 6), np.float32)
    x[0, 1] = -3.5
    for k, p, s in [((2, 2), (0, 0), (2, 2)), ((3, 3), (1, 1), (2, 2))]:
        rtop, rmask = O.max_pool(x, k, p, s)
        top, mask = K.max_pool(gpu(x), k, p, s)
        assert np.array_equal(mask.get(), rmask) and bits_equal(top.get(), rtop)


@pytest.mark.parametrize("xshape,k,p,s", [((2, 3, 13, 17), (3, 3), (0, 0), (2, 2)), ((2, 16, 56, 56), (2, 2), (0, 0), (2, 2)),
                                         ((1, 96, 55, 55), (3, 3), (0, 0), (2, 2)), ((2, 5, 9, 9), (3, 3), (1, 1), (1, 1)),
                                         ((3, 4, 20, 31), (4, 4), (0, 0), (1, 1))])
def test_max_pool_and_im2col_with_nan_and_infinite_inputs(K, xshape, k, p, s):
    # the reference's scan starts from -FLT_MAX / index -1 and keeps a cell only if it compares
    # greater (include/pooling.h:46-54): NaN and -inf never win, a window of nothing else yields
    # (-FLT_MAX, -1).  Selection and copying carry the bits through unchanged.
    rs = np.random.RandomState(7)
    x = rs.randn(*xshape).astype(np.float32)
    m = rs.rand(*xshape)
    x[m < 0.15] = np.nan
    x[(m >= 0.15) & (m < 0.25)] = -np.inf
    x[(m >= 0.25) & (m < 0.3)] = np.inf
    x[0, 0, :4, :4] = np.nan
    x[0, 0, 4:8, :4] = -np.inf
    rtop, rmask = O.max_pool(x, k, p, s)
    assert rmask.min() == -1 and (rtop == -np.finfo(np.float32).max).any()
    top, mask = K.max_pool(gpu(x), k, p, s)
    assert np.array_equal(mask.get(), rmask) and bits_equal(top.get(), rtop)
    assert bits_equal(K.im2col(gpu(x), k, p, s).get(), O.im2col(x, k, p, s))


# ---------------------------------------------------------------- LRN vs oracle

LRN_CASES = [
    # (shape, size, alpha, beta, k)
    ((4, 32, 15, 15), 5, 1e-4, 0.75, 1.0),   # CIFAR block
    ((2, 96, 55, 55), 5, 1e-4, 0.75, 1.0),   # AlexNet block, full plane
    ((2, 96, 55, 55), 5, 1e-4, 0.75, 2.0),   # k = 2 (extension)
    ((4, 8, 16, 16), 4, 0.1, 0.5, 1.0),      # reference test_lrn (even size)
    ((2, 5, 7, 9), 5, 0.1, 0.75, 1.0),       # C == size
    ((2, 9, 6, 5), 1, 0.3, 0.75, 1.0),
    ((2, 9, 6, 5), 2, 0.3, 0.75, 1.0),
    ((2, 10, 6, 5), 3, 0.3, 0.5, 1.0),
    ((2, 20, 6, 5), 6, 0.3, 0.75, 1.0),
    ((2, 20, 6, 5), 7, 0.3, 0.75, 1.0),
    ((2, 20, 6, 5), 8, 0.3, 0.75, 1.0),
    ((2, 20, 6, 5), 9, 0.3, 0.75, 1.0),
    ((2, 24, 6, 5), 11, 0.3, 0.75, 1.0),     # generic window length
    ((1, 64, 33, 31), 5, 1.0, 0.75, 1.0),    # large alpha: scale far from 1
]


@pytest.mark.parametrize("shape,size,alpha,beta,k", LRN_CASES)
def test_lrn_vs_oracle(K, shape, size, alpha, beta, k):
    print("lrn case", shape, size, alpha, beta, k, flush=True)
    rs = np.random.RandomState(3)
    x = rs.randn(*shape).astype(np.float32)
    rtop, rscale = O.lrn_fwd(x, size, alpha, beta, k)
    x64 = x.astype(np.float64)
    ttop, tscale = O.lrn_fwd(x64, size, alpha, beta, k)   # float64 truth
    top, scale = K.lrn_fwd(gpu(x), size, alpha, beta, k)
    top, scale = top.get(), scale.get()
    assert relfro(scale, rscale) <= TOL and relfro(top, rtop) <= TOL
    # and no further from the float64 result than a few fp32 roundings
    assert relfro(scale, tscale) <= 1e-6 and relfro(top, ttop) <= 5e-6
    assert np.max(np.abs(top - ttop) / (np.abs(ttop) + 1e-6)) <= 1e-4
    if k == 1.0:
        g = rs.rand(*shape).astype(np.float32)
        rgb = O.lrn_bwd(x, rtop, rscale, g, size, alpha, beta)
        tgb = O.lrn_bwd(x64, ttop, tscale, g.astype(np.float64), size, alpha, beta)
        gb = K.lrn_bwd(gpu(x), gpu(rtop), gpu(rscale), gpu(g), size, alpha, beta).get()
        assert relfro(gb, rgb) <= TOL
        assert relfro(gb, tgb) <= 1e-5
    # the variant that does not read `top` (what the Op's closure calls): top is formed again from
    # x and scale, so on the pair the forward kernel wrote it has the bits of the five-array kernel
    g = rs.rand(*shape).astype(np.float32)
    xg, gg = gpu(x), gpu(g)
    dtop, dscale = K.lrn_fwd(xg, size, alpha, beta, k)
    with_top = K.lrn_bwd(xg, dtop, dscale, gg, size, alpha, beta).get()
    recomputed = K.lrn_bwd(xg, None, dscale, gg, size, alpha, beta).get()
    assert np.array_equal(recomputed.view(np.uint32), with_top.view(np.uint32))
    tgb = O.lrn_bwd(x64, ttop, tscale, g.astype(np.float64), size, alpha, beta)
    assert relfro(recomputed, tgb) <= 1e-5
    # without a stored scale: top alone has the bits of the pair's top where the same kernel wrote
    # both; the gradient from x and the cotangent alone forms the scale again (k goes in)
    top_only = K.lrn_fwd(xg, size, alpha, beta, k, want_scale=False).get()
    assert relfro(top_only, ttop) <= 5e-6
    if x.size < (16 << 20):
        assert np.array_equal(top_only.view(np.uint32), top.view(np.uint32))
    from_x = K.lrn_bwd_from_x(xg, gg, size, alpha, beta, k).get()
    assert relfro(from_x, tgb) <= 1e-5 and relfro(from_x, with_top) <= 1e-6


@pytest.mark.parametrize("shape,size", [((5, 7, 701, 685), 5), ((5, 7, 701, 685), 4), ((2, 9, 1024, 1024), 3)])
def test_lrn_forward_large_arrays(K, shape, size):
    # >= 16 M floats: the forward pass takes the kernel that owns aligned units of
    # the flat array.  Odd plane and odd total (units that straddle planes, a
    # partial last unit), few channels (window mostly clipped), and an aligned case.
    print("lrn large case", shape, size, flush=True)
    rs = np.random.RandomState(4)
    x = rs.randn(*shape).astype(np.float32)
    rtop, rscale = O.lrn_fwd(x, size, 0.3, 0.75, 1.0)
    top, scale = K.lrn_fwd(gpu(x), size, 0.3, 0.75, 1.0)
    top, scale = top.get(), scale.get()
    assert relfro(scale, rscale) <= 1e-6 and relfro(top, rtop) <= 5e-6
    assert np.max(np.abs(scale - rscale) / rscale) <= 1e-5
    assert np.max(np.abs(top - rtop) / (np.abs(rtop) + 1e-6)) <= 1e-4
    # top alone (no scale array): the pixel-per-lane kernel at this size too
    top_only = K.lrn_fwd(gpu(x), size, 0.3, 0.75, 1.0, want_scale=False).get()
    assert relfro(top_only, rtop) <= 5e-6 and np.max(np.abs(top_only - rtop) / (np.abs(rtop) + 1e-6)) <= 1e-4


def test_lrn_confines_non_finite_inputs_to_their_windows(K):
    # A documented difference.  The reference keeps a running window sum down the channels
    # (include/lrn.cuh:22-50: add the entering square, subtract the leaving one), so once an
    # infinite or NaN input has entered, inf - inf leaves NaN in the sum for every later channel
    # of that pixel.  The kernels here sum every window afresh: the same values wherever the
    # reference's are finite, and non-finite results only for the windows that hold the input.
    rs = np.random.RandomState(3)
    x = rs.randn(2, 16, 9, 9).astype(np.float32)
    x[0, 3, 2, 2], x[1, 5, 4, 4], x[1, 7, 1, 1] = np.inf, np.nan, -np.inf
    rtop, rscale = O.lrn_fwd(x, 5, 1e-4, 0.75)
    top, scale = K.lrn_fwd(gpu(x), 5, 1e-4, 0.75)
    top, scale = top.get(), scale.get()
    fin = np.isfinite(rtop) & np.isfinite(rscale)
    assert fin.sum() > 0.9 * fin.size
    assert np.allclose(top[fin], rtop[fin], rtol=1e-5, atol=1e-7) and np.allclose(scale[fin], rscale[fin], rtol=1e-6)
    bad = ~np.isfinite(scale)
    assert not (bad & np.isfinite(rscale)).any()            # never non-finite where the reference is finite
    for (n, c, h, w) in [(0, 3, 2, 2), (1, 5, 4, 4), (1, 7, 1, 1)]:
        assert bad[n, max(0, c - 2):c + 3, h, w].all()      # the windows that contain the input
        assert np.isfinite(scale[n, c + 3:, h, w]).all() and not np.isfinite(rscale[n, c + 3:, h, w]).any()


def test_lrn_window_sums_do_not_inherit_the_running_sums_cancellation(K):
    # The second documented difference, same cause.  One channel of 1e4 among ones: the
    # reference's running sum holds 1e8 while that square is in the window, the ones added
    # meanwhile fall below its last bit, and after the subtraction the sum is 0 (later even
    # negative) where it should be 5.  The oracle, which restates the reference, shows it; the
    # kernels match the float64 window sums.  (On inputs of ordinary range the two agree to
    # rounding: every other LRN test compares the kernels with the oracle.)
    x = np.ones((1, 12, 3, 3), np.float32)
    x[0, 0] = 1e4
    _, rscale = O.lrn_fwd(x, 5, 0.1, 0.75)
    _, scale = K.lrn_fwd(gpu(x), 5, 0.1, 0.75)
    sq = x.astype(np.float64) ** 2
    exact = np.stack([1 + 0.1 / 5 * sq[0, max(0, c - 2):c + 3].sum(axis=0) for c in range(12)])[None]
    assert np.allclose(scale.get(), exact, rtol=1e-6)
    assert abs(rscale[0, 5, 0, 0] - 1.0) < 1e-6 and abs(exact[0, 5, 0, 0] - 1.1) < 1e-12 and rscale[0, 11, 0, 0] < 1.0


def test_lrn_rejects_size_above_channels(K):
    from cgt_amd.capi import CgtAmdError
    x = gpu(np.zeros((1, 3, 2, 2), np.float32))
    with pytest.raises(CgtAmdError):
        K.lrn_fwd(x, 5, 1e-4, 0.75)


# ---------------------------------------------------------------- GEMM vs oracle

GEMM_SHAPES = [
    # (M, N, K)
    (7, 11, 13), (128, 128, 16), (129, 127, 17), (64, 192, 100), (300, 70, 33),
    (256, 256, 256), (1, 1, 1), (5, 300, 2), (1000, 96, 363),   # AlexNet conv1 skew
    (2048, 32, 9),                                             # MNIST conv skew
    (200, 64, 800), (96, 363, 3000),                           # split-K range
    (128, 1152, 4100),                                         # VGG weight gradient in miniature
    (38400, 128, 512),                                         # 300 tiles: whole round + K-split tail
    (33000, 96, 363),                                          # 258 tiles of 128x96, unaligned K, clipped tail tile
]


@pytest.mark.parametrize("M,N,Kd", GEMM_SHAPES)
@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
def test_mul22_vs_oracle(K, M, N, Kd, tA, tB):
    print("gemm case", M, N, Kd, tA, tB, flush=True)
    rs = np.random.RandomState(4)
    A = rs.uniform(-1, 1, (Kd, M) if tA else (M, Kd)).astype(np.float32)
    B = rs.uniform(-1, 1, (N, Kd) if tB else (Kd, N)).astype(np.float32)
    if M * N * Kd <= 40e6:
        ref = O.mul22(A, B, tA, tB)
    else:   # textbook product in float64 (what the oracle computes, via BLAS for speed)
        ref = ((A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)).astype(np.float32)
    C = K.mul22(gpu(A), gpu(B), tA, tB).get()
    assert C.shape == (M, N)
    assert relfro(C, ref) <= TOL
    assert relfro(C, ref) <= 2e-6   # what fp32 accumulation should give at these K


def test_mul22_shape_mismatch_raises(K):
    with pytest.raises(ValueError):
        K.mul22(gpu(np.zeros((3, 4), np.float32)), gpu(np.zeros((5, 6), np.float32)))


@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
def test_batched_mul22_vs_oracle(K, tA, tB):
    rs = np.random.RandomState(5)
    P, M, N, Kd = 3, 70, 130, 45
    A = rs.uniform(-1, 1, (P, Kd, M) if tA else (P, M, Kd)).astype(np.float32)
    B = rs.uniform(-1, 1, (P, N, Kd) if tB else (P, Kd, N)).astype(np.float32)
    ref = O.batched_mul22(A, B, tA, tB)
    C = K.batched_mul22(gpu(A), gpu(B), tA, tB).get()
    assert relfro(C, ref) <= 2e-6
    # the reference's einsum case: (2,3,5) x (2,5,7)
    x, y = rs.randn(2, 3, 5).astype(np.float32), rs.randn(2, 5, 7).astype(np.float32)
    np.testing.assert_allclose(K.batched_mul22(gpu(x), gpu(y)).get(), np.einsum("nij,njk->nik", x, y), atol=1e-5)


def test_mul22_deterministic_split_k(K):
    rs = np.random.RandomState(6)
    A = gpu(rs.uniform(-1, 1, (5000, 128)).astype(np.float32))
    B = gpu(rs.uniform(-1, 1, (5000, 200)).astype(np.float32))
    c1 = K.mul22(A, B, True, False).get()
    c2 = K.mul22(A, B, True, False).get()
    assert bits_equal(c1, c2)


# ---------------------------------------------------------------- transpose / conv2d composition

@pytest.mark.parametrize("axes", [(0, 3, 1, 2), (0, 2, 3, 1), (3, 2, 1, 0), (0, 1, 2, 3), (1, 0, 3, 2)])
def test_transpose4(K, axes):
    rs = np.random.RandomState(7)
    x = rs.randn(3, 70, 9, 65).astype(np.float32)
    assert bits_equal(K.transpose4(gpu(x), axes).get(), np.ascontiguousarray(x.transpose(axes)))


# conv-glue shapes where the filter count is the short extent: thin-tile path
# (vector and scalar variants, ragged last tile, long extent odd)
@pytest.mark.parametrize("shape", [(2, 55, 55, 96), (3, 19, 17, 75), (2, 16, 16, 128), (1, 23, 13, 4),
                                   (2, 31, 9, 1), (2, 20, 20, 100)])
@pytest.mark.parametrize("axes", [(0, 3, 1, 2), (0, 2, 3, 1)])
def test_transpose4_conv_glue(K, shape, axes):
    rs = np.random.RandomState(8)
    if axes == (0, 2, 3, 1):
        shape = (shape[0], shape[3], shape[1], shape[2])      # [B, L, m, n]
    x = rs.randn(*shape).astype(np.float32)
    assert bits_equal(K.transpose4(gpu(x), axes).get(), np.ascontiguousarray(x.transpose(axes)))


def test_conv2d_reference_known_answer(K):
    # cgt/tests/test_conv.py:14-33 (single precision tolerance atol 1e-3)
    import scipy.signal
    np.random.seed(0)
    x = np.random.randn(2, 2, 5, 17)
    filt = np.random.randn(3, 2, 4, 7)
    out = np.zeros((2, 3, 8, 23))
    for b in range(2):
        for ic in range(2):
            for oc in range(3):
                out[b, oc] += scipy.signal.convolve2d(x[b, ic], filt[oc, ic][::-1, ::-1], mode="full")
    y = K.conv2d(gpu(x, np.float32), gpu(filt, np.float32), pad=(3, 6)).get()
    np.testing.assert_allclose(y, out, atol=1e-3)


CONV_CASES = [
    # (xshape, fshape, pad, stride): one miniature per configured layer
    ((4, 1, 28, 28), (32, 1, 3, 3), (1, 1), (1, 1)),
    ((3, 3, 32, 32), (32, 3, 5, 5), (2, 2), (1, 1)),
    ((2, 32, 15, 15), (64, 32, 5, 5), (2, 2), (1, 1)),
    ((2, 3, 227, 227), (96, 3, 11, 11), (0, 0), (4, 4)),
    ((1, 128, 28, 28), (128, 128, 3, 3), (1, 1), (1, 1)),
    ((2, 3, 11, 13), (5, 3, 3, 2), (1, 0), (2, 1)),
]


@pytest.mark.parametrize("xshape,fshape,p,s", CONV_CASES)
def test_conv2d_fwd_bwd_vs_oracle(K, xshape, fshape, p, s):
    print("conv case", xshape, fshape, p, s, flush=True)
    rs = np.random.RandomState(8)
    x = rs.randn(*xshape).astype(np.float32)
    f = (rs.randn(*fshape) * np.sqrt(1.0 / np.prod(fshape[1:]))).astype(np.float32)
    # float64 oracle as truth; the float32 oracle differs from it by accumulation order only
    y64 = O.conv2d(x.astype(np.float64), f.astype(np.float64), p, s)
    keep = {}
    y = K.conv2d(gpu(x), gpu(f), p, s, keep=keep).get()
    assert y.shape == y64.shape
    assert relfro(y, y64) <= TOL
    gy = rs.randn(*y64.shape).astype(np.float32)
    gx64, gf64 = O.conv2d_pullback(x.astype(np.float64), f.astype(np.float64), gy.astype(np.float64), p, s)
    gx, gf = K.conv2d_pullback(gpu(x), gpu(f), gpu(gy), p, s, col=keep["col"])
    assert relfro(gx.get(), gx64) <= TOL
    assert relfro(gf.get(), gf64) <= TOL
