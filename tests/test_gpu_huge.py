"""Arrays of more than 2^31 elements (8 GiB of float32) through every entry point of the path.

The reference computes strides in `int` (include/cgt_common.h:107-117) and stops there; a 288 GB
device holds arrays well past that, so the kernels carry 64-bit offsets and these tests walk them
across the 2^31-element line.  The operands are a 64 MB random pattern tiled over the array on
the device (its period is odd, so it lines up with no plane, row or tile), which makes every
element known on the host without an 8 GiB transfer: the checks read back the slices around
element 0, element 2^31 and the end, and compare them with the oracle on the same slices.
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

P = (1 << 24) + 3
N31 = 1 << 31


@pytest.fixture(scope="module")
def K():
    from cgt_amd import capi, kernels
    capi.require_gpu()
    return kernels


@pytest.fixture(scope="module")
def pattern(K):
    from cgt_amd.gpuarray import to_gpu
    chunk = np.random.RandomState(5).randn(P).astype(np.float32)
    return chunk, to_gpu(chunk)


def view(a, start, shape):
    from cgt_amd.gpuarray import GpuArray
    return GpuArray(shape, a.dtype, _buffer=a._buffer, _offset=a._offset + start * a.dtype.itemsize)


def tiled(pattern, shape):
    """Device array of `shape` whose flat element i is chunk[i % P]."""
    from cgt_amd import capi
    from cgt_amd.gpuarray import empty
    _, dchunk = pattern
    a = empty(shape)
    at = 0
    while at < a.size:
        k = min(P, a.size - at)
        capi.check(capi.lib().cgt_amd_memcpy(capi.GPU, capi.GPU, a.ptr + 4 * at, dchunk.ptr, 4 * k))
        at += k
    return a


def expect(pattern, start, shape):
    n = int(np.prod(shape))
    return pattern[0][(start + np.arange(n, dtype=np.int64)) % P].reshape(shape)


def same(a, b):
    return np.array_equal(np.asarray(a).view(np.uint32), np.asarray(b).view(np.uint32))


def rel(a, b):
    return float(np.linalg.norm(np.asarray(a, np.float64) - b) / np.linalg.norm(b))


def test_elementwise_fill_repeat(K, pattern):
    from cgt_amd.gpuarray import to_gpu
    n = N31 + 4099
    spots = (0, N31 - 3000, n - 6000)
    x = tiled(pattern, (n,))
    y = K.elwise_unary("square", x)
    for s in spots:
        assert same(view(y, s, (6000,)).get(), np.square(expect(pattern, s, (6000,)))), s
    z = K.elwise_binary("*", x, y, out=y)
    for s in spots:
        e = expect(pattern, s, (6000,))
        assert same(view(z, s, (6000,)).get(), e * np.square(e)), s
    m = K.elwise_binary(">=", x, to_gpu(np.float32(0.0)))
    for s in spots:
        assert np.array_equal(view(m, s, (6000,)).get(), (expect(pattern, s, (6000,)) >= 0).astype(np.int8)), s
    K.fill(1.5, (n,), out=y)
    assert np.all(view(y, n - 6000, (6000,)).get() == 1.5) and np.all(view(y, N31 - 10, (20,)).get() == 1.5)
    row = pattern[0][:4104]
    r = K.repeat(to_gpu(row.reshape(1, 4104)), (0,), (523777,))
    assert r.size > N31
    for i in (0, 523263, 523776):
        assert same(view(r, i * 4104, (4104,)).get(), row), i


def test_sum(K, pattern):
    shape = (65537, 8, 4096)
    n = int(np.prod(shape))
    assert n > N31
    x = tiled(pattern, shape)
    c64 = pattern[0].astype(np.float64)
    mean_abs = np.abs(c64).mean()
    # all axes: whole periods of the pattern plus a remainder
    got = float(K.sum_keepdims(x.reshape(n), (0,)).get()[0])
    want = (n // P) * c64.sum() + c64[: n % P].sum()
    assert abs(got - want) <= 1e-6 * n * mean_abs
    # keep the middle axis: row (r0, k) starts at ((r0 * 8 + k) * 4096) % P of the pattern
    cs = np.concatenate([[0.0], np.cumsum(np.concatenate([c64, c64[:4096]]))])
    starts = ((np.arange(shape[0], dtype=np.int64)[:, None] * 8 + np.arange(8)[None, :]) * 4096) % P
    want = (cs[starts + 4096] - cs[starts]).sum(axis=0)
    got = K.sum_keepdims(x, (0, 2)).get().reshape(8)
    assert np.abs(got - want).max() <= 1e-6 * shape[0] * 4096 * mean_abs
    # keep the innermost axis: eight of its columns
    idx = ((np.arange(shape[0] * 8, dtype=np.int64)[:, None] * 4096) + np.arange(0, 4096, 512)[None, :]) % P
    got = K.sum_keepdims(x, (0, 1)).get().reshape(4096)[::512]
    assert np.abs(got - c64[idx].sum(axis=0)).max() <= 1e-6 * shape[0] * 8 * mean_abs


def test_transposes(K, pattern):
    shape = (2049, 32, 32, 1024)
    per = 32 * 32 * 1024
    x = tiled(pattern, shape)
    y = K.transpose4(x, (0, 3, 1, 2))
    for b in (0, 2047, 2048):
        assert same(view(y, b * per, (1024, 32, 32)).get(), expect(pattern, b * per, (32, 32, 1024)).transpose(2, 0, 1)), b
    y = K.transpose4(x.reshape(2049, 1024, 32, 32), (0, 2, 3, 1), out=y.reshape(shape))
    for b in (0, 2047, 2048):
        assert same(view(y, b * per, (32, 32, 1024)).get(), expect(pattern, b * per, (1024, 32, 32)).transpose(1, 2, 0)), b


@pytest.mark.parametrize("geom", [((2, 2), (0, 0), (2, 2)), ((3, 3), (0, 0), (2, 2)), ((4, 3), (1, 0), (3, 2))])
def test_max_pool_and_pullback(K, pattern, geom):
    shape = (2049, 16, 256, 256)
    HW = 256 * 256
    x = tiled(pattern, shape)
    top, mask = K.max_pool(x, *geom)
    gb = K.max_pool_pullback(shape, mask, top, *geom)
    PP = top.shape[2] * top.shape[3]
    for pl in (0, 32767, 32768, 2049 * 16 - 1):           # plane 32768 starts at element 2^31
        xe = expect(pattern, pl * HW, (1, 1, 256, 256))
        rt, rm = O.max_pool(xe, *geom)
        assert same(view(top, pl * PP, rt.shape).get(), rt), pl
        assert np.array_equal(view(mask, pl * PP, rm.shape).get(), rm), pl
        assert same(view(gb, pl * HW, xe.shape).get(), O.max_pool_pullback(xe.shape, rm, rt)), pl


@pytest.mark.parametrize("size", [5, 4])
def test_lrn(K, pattern, size):
    shape = (2049, 16, 256, 256)
    per = 16 * 256 * 256
    x = tiled(pattern, shape)
    top, scale = K.lrn_fwd(x, size, 1e-2, 0.75)
    gb = K.lrn_bwd(x, top, scale, x, size, 1e-2, 0.75)
    gb2 = K.lrn_bwd(x, None, scale, x, size, 1e-2, 0.75)
    for b in (0, 2047, 2048):                             # image 2048 starts at element 2^31
        xe = expect(pattern, b * per, (1, 16, 256, 256))
        rt, rsc = O.lrn_fwd(xe, size, 1e-2, 0.75)
        assert rel(view(top, b * per, xe.shape).get(), rt) <= 1e-5, b
        assert rel(view(scale, b * per, xe.shape).get(), rsc) <= 1e-5, b
        g = view(gb, b * per, xe.shape).get()
        assert rel(g, O.lrn_bwd(xe, rt, rsc, xe, size, 1e-2, 0.75)) <= 1e-4, b
        assert same(g, view(gb2, b * per, xe.shape).get()), b


@pytest.mark.parametrize("shape,kernel,pad,stride", [((600, 128, 56, 56), (3, 3), (1, 1), (1, 1)),
                                                     ((11200, 3, 99, 99), (11, 11), (0, 0), (4, 4))])
def test_im2col_col2im(K, pattern, shape, kernel, pad, stride):
    x = tiled(pattern, shape)
    col = K.im2col(x, kernel, pad, stride)
    assert col.size > N31
    gx = K.col2im(col, shape, kernel, pad, stride)
    per, cper = int(np.prod(shape[1:])), int(np.prod(col.shape[1:]))
    for b in (0, N31 // cper, N31 // cper + 1, shape[0] - 1):       # image N31 // cper straddles the line
        xe = expect(pattern, b * per, (1,) + shape[1:])
        ce = O.im2col(xe, kernel, pad, stride)
        assert same(view(col, b * cper, ce.shape).get(), ce), b
        assert same(view(gx, b * per, xe.shape).get(), O.col2im(ce, xe.shape, kernel, pad, stride)), b


def test_mul22(K, pattern):
    chunk, dchunk = pattern
    M, N, Kd = (1 << 21) + 64, 1032, 48
    assert M * N > N31
    rows = (0, N31 // N - 2, M - 200)
    A = tiled(pattern, (M, Kd))
    Bh = chunk[7:7 + Kd * N].reshape(Kd, N).astype(np.float64)
    C = K.mul22(A, view(dchunk, 7, (Kd, N)))                          # the result crosses the line
    for r in rows:
        assert rel(view(C, r * N, (200, N)).get(), expect(pattern, r * Kd, (200, Kd)).astype(np.float64) @ Bh) <= 2e-6, r
    C2 = K.mul22(view(dchunk, 11, (Kd, N)), C, tB=True).get()         # [48, M] = A2 . C^T: the B operand does
    A2 = chunk[11:11 + Kd * N].reshape(Kd, N).astype(np.float64)
    for r in rows:
        assert rel(C2[:, r:r + 200], A2 @ view(C, r * N, (200, N)).get().astype(np.float64).T) <= 2e-6, r
    C3 = K.mul22(C, A, tA=True).get()                                 # [N, 48] = C^T . A: K = M, cut into splits
    cols = [0, 17, 47]
    acc = np.zeros((N, len(cols)))
    for r0 in range(0, M, 1 << 17):
        r1 = min(M, r0 + (1 << 17))
        acc += view(C, r0 * N, (r1 - r0, N)).get().astype(np.float64).T @ expect(pattern, r0 * Kd, (r1 - r0, Kd))[:, cols].astype(np.float64)
    assert rel(C3[:, cols], acc) <= 2e-6


def test_conv_products_without_a_column_buffer(K, pattern):
    from cgt_amd.gpuarray import to_gpu
    d = np.float64
    B, C, H, W, L = 5600, 16, 56, 56, 128
    per, yper = C * H * W, L * H * W
    assert B * yper > N31
    x = tiled(pattern, (B, C, H, W))
    f = to_gpu((pattern[0][100:100 + L * C * 9].reshape(L, C, 3, 3) / 12).astype(np.float32))
    fh = f.get().astype(d)
    xpad = K.conv_same_pad(x, (3, 3))
    y = K.conv_same_fwd(xpad, f, x.shape)
    gypad = K.conv_same_pad(y, (3, 3))
    assert gypad.size > N31
    gx = K.conv_same_bwd_data(gypad, f, x.shape)
    for b in (0, N31 // yper, N31 // yper + 1, B - 1):
        xe = expect(pattern, b * per, (1, C, H, W)).astype(d)
        ye = view(y, b * yper, (1, L, H, W)).get()
        assert rel(ye, O.conv2d(xe, fh, (1, 1), (1, 1))) <= 1e-5, b
        assert rel(view(gx, b * per, (1, C, H, W)).get(), O.conv2d_pullback(xe, fh, ye.astype(d), (1, 1), (1, 1))[0]) <= 1e-5, b
    # the weight gradient sums over every image: the same kernel over four quarters of the batch
    # (each below the line, the size the other tests pin), added in float64
    gf = K.conv_same_bwd_filter(gypad, xpad, x.shape, f.shape).get()
    acc = np.zeros(gf.shape)
    q = B // 4
    for b0 in range(0, B, q):
        xq, yq = view(x, b0 * per, (q, C, H, W)), view(y, b0 * yper, (q, L, H, W))
        acc += K.conv_same_bwd_filter(K.conv_same_pad(yq, (3, 3)), K.conv_same_pad(xq, (3, 3)), xq.shape, f.shape).get()
    assert rel(gf, acc) <= 2e-6


def test_conv_products_over_a_column_buffer(K, pattern):
    from cgt_amd.gpuarray import to_gpu
    d = np.float64
    B, C, H, W, L = 600, 128, 56, 56, 32
    per, yper, cper = C * H * W, L * H * W, H * W * C * 9
    x = tiled(pattern, (B, C, H, W))
    col = K.im2col(x, (3, 3), (1, 1), (1, 1))
    assert col.size > N31
    f = to_gpu((pattern[0][50:50 + L * C * 9].reshape(L, C, 3, 3) / 34).astype(np.float32))
    fh = f.get().astype(d)
    y = K.conv_col_fwd(col, f)
    gcol = K.conv_col_bwd_data(y, f)
    for b in (0, N31 // cper, N31 // cper + 1, B - 1):
        xe = expect(pattern, b * per, (1, C, H, W)).astype(d)
        yb = view(y, b * yper, (1, L, H, W)).get()
        assert rel(yb, O.conv2d(xe, fh, (1, 1), (1, 1))) <= 1e-5, b
        want = yb.astype(d).transpose(0, 2, 3, 1).reshape(H * W, L) @ fh.reshape(L, -1)
        assert rel(view(gcol, b * cper, (H * W, C * 9)).get(), want) <= 1e-5, b
    gf = K.conv_col_bwd_filter(y, col, f.shape).get()
    acc = np.zeros(gf.shape)
    q = B // 4
    for b0 in range(0, B, q):
        acc += K.conv_col_bwd_filter(view(y, b0 * yper, (q, L, H, W)), view(col, b0 * cper, (q, H, W, C * 9)), f.shape).get()
    assert rel(gf, acc) <= 2e-6
