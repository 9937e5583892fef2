"""Edge behaviour of the C ABI itself, called with raw pointers as a foreign
host would: empty inputs are accepted and touch nothing, bad arguments come
back as CGT_AMD_ERR_ARG with a message (the reference's kernels print and carry
on, include/cgt_cuda.h:11-21; here nothing is launched), and the library stays
usable after an error."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

OK, ERR_ARG = 0, 1


@pytest.fixture(scope="module")
def L():
    from cgt_amd import capi
    capi.require_gpu()
    return capi.lib()


def gpu(a):
    from cgt_amd.gpuarray import to_gpu
    return to_gpu(a)


def _err(L):
    return L.cgt_amd_last_error().decode()


def test_empty_inputs_are_ok(L):
    x = gpu(np.zeros((4,), np.float32))
    p = x.ptr
    assert L.cgt_amd_im2col_f32(p, 0, 3, 8, 8, 3, 3, 1, 1, 1, 1, p, None) == OK
    assert L.cgt_amd_col2im_f32(p, 0, 3, 8, 8, 3, 3, 1, 1, 1, 1, p, None) == OK
    assert L.cgt_amd_max_pool_f32(p, 0, 3, 8, 8, 2, 2, 0, 0, 2, 2, 3, 3, p, p, None) == OK
    assert L.cgt_amd_lrn_fwd_f32(p, 0, 8, 4, 4, 5, 1e-4, 0.75, 1.0, p, p, None) == OK
    assert L.cgt_amd_sgemm(0, 0, 0, 5, 7, p, 7, p, 5, p, 5, None) == OK
    assert L.cgt_amd_sgemm_batched(0, 0, 0, 4, 4, 4, p, 4, 16, p, 4, 16, p, 4, 16, None) == OK
    assert L.cgt_amd_elwise_unary_f32(0, 0, p, p, None) == OK
    assert L.cgt_amd_elwise_binary(1, 11, 11, 0, p, 0, p, 0, p, None) == OK
    assert L.cgt_amd_fill_f32(p, 1.0, 0, None) == OK
    assert np.array_equal(x.get(), np.zeros(4, np.float32))


def test_gemm_with_k_zero_writes_zeros(L):
    # C = A[M,0] . B[0,N] is all zeros, and C must be overwritten, not skipped
    c = gpu(np.full((5, 7), 3.0, np.float32))
    a = gpu(np.zeros((1,), np.float32))
    assert L.cgt_amd_sgemm(0, 0, 5, 7, 0, a.ptr, 0, a.ptr, 7, c.ptr, 7, None) == OK
    assert np.array_equal(c.get(), np.zeros((5, 7), np.float32))


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_with_huge_leading_dimension(L, tA, tB):
    # rows 2^23 floats apart: the 32-bit tile offsets of the steady-state loads do not
    # reach, so every tile has to take the 64-bit tested loads; results must not change
    ld = 1 << 23
    M, N, K = 130, 140, 37
    rs = np.random.RandomState(5)
    a = rs.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    b = rs.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    wide_a = np.zeros((a.shape[0], ld), np.float32)
    wide_a[:, :a.shape[1]] = a
    ga, gb = gpu(wide_a), gpu(b)
    del wide_a
    c = gpu(np.zeros((M, N), np.float32))
    assert L.cgt_amd_sgemm(tA, tB, M, N, K, ga.ptr, ld, gb.ptr, b.shape[1], c.ptr, N, None) == OK
    ref = (a.T if tA else a).astype(np.float64) @ (b.T if tB else b).astype(np.float64)
    err = np.linalg.norm(c.get() - ref) / np.linalg.norm(ref)
    assert err <= 1e-4     # relative Frobenius bar of the GEMM tests


@pytest.mark.parametrize("M,N,K", [(300, 260, 70),        # whole and edge tiles
                                   (2100, 2100, 300),     # 289 tiles: the last partial round is cut along K
                                   (100, 200, 5000),      # few tiles, long K: split along K
                                   (1024, 96, 363),       # 128x96 tiles, ragged K
                                   (600, 500, 700)])      # edge tiles in the two-slices-in-flight loop
@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_with_padded_leading_dimensions(L, M, N, K, tA, tB):
    # operands and result live inside wider arrays: rows are lda / ldb / ldc apart, the
    # columns beyond the matrices hold NaN (operands) or a sentinel (result) and must
    # neither reach the sums nor be written
    rs = np.random.RandomState(M * 7 + N * 3 + K + tA * 2 + tB)
    pa, pb, pc = 5, 9, 13
    a = rs.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    b = rs.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    wa = np.full((a.shape[0], a.shape[1] + pa), np.nan, np.float32)
    wa[:, :a.shape[1]] = a
    wb = np.full((b.shape[0], b.shape[1] + pb), np.nan, np.float32)
    wb[:, :b.shape[1]] = b
    wc = np.full((M, N + pc), -7.0, np.float32)
    ga, gb, gc = gpu(wa), gpu(wb), gpu(wc)
    assert L.cgt_amd_sgemm(tA, tB, M, N, K, ga.ptr, wa.shape[1], gb.ptr, wb.shape[1], gc.ptr, N + pc, None) == OK
    out = gc.get()
    ref = (a.T if tA else a).astype(np.float64) @ (b.T if tB else b).astype(np.float64)
    assert np.array_equal(out[:, N:], np.full((M, pc), -7.0, np.float32))
    assert np.linalg.norm(out[:, :N] - ref) / np.linalg.norm(ref) <= 1e-4


def test_batched_gemm_with_strides_and_shared_operand(L):
    # batch strides larger than the matrices, and a batch stride of zero (one operand
    # shared by every product, as a conv layer's filters would be)
    rs = np.random.RandomState(11)
    P, M, N, K = 5, 150, 70, 45
    a = rs.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rs.uniform(-1, 1, (P, K + 2, N + 3)).astype(np.float32)      # each product uses b[p, :K, :N]
    c = np.full((P, M + 1, N + 4), 3.0, np.float32)
    ga, gb, gc = gpu(a), gpu(b), gpu(c)
    assert L.cgt_amd_sgemm_batched(0, 0, P, M, N, K, ga.ptr, K, 0, gb.ptr, N + 3, (K + 2) * (N + 3),
                                   gc.ptr, N + 4, (M + 1) * (N + 4), None) == OK
    out = gc.get()
    for p in range(P):
        ref = a.astype(np.float64) @ b[p, :K, :N].astype(np.float64)
        assert np.linalg.norm(out[p, :M, :N] - ref) / np.linalg.norm(ref) <= 1e-4
    assert np.all(out[:, M:, :] == 3.0) and np.all(out[:, :, N:] == 3.0)


@pytest.mark.parametrize("M,N,K", [(256, 256, 16 * 9 + 5), (128, 96, 363), (384, 128, 11), (128, 128, 16),
                                   # one round of workgroups with >= 32 K slices each: the loop that keeps
                                   # two slices of loads in flight (whole slices only / ragged last slice)
                                   (512, 384, 640), (512, 384, 16 * 40 + 5)])
@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_whole_tiles_with_ragged_k(L, M, N, K, tA, tB):
    # every tile is inside C, so the untested loads run for all full K slices and only
    # the last, ragged slice is bounds-tested; memory right behind the operands is
    # poisoned with NaN so a read past a row end that reached the sum would show
    rs = np.random.RandomState(M + N + K)
    a = rs.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    b = rs.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    pad = np.full(64, np.nan, np.float32)
    ga = gpu(np.concatenate([a.ravel(), pad]))
    gb = gpu(np.concatenate([b.ravel(), pad]))
    c = gpu(np.zeros((M, N), np.float32))
    assert L.cgt_amd_sgemm(tA, tB, M, N, K, ga.ptr, a.shape[1], gb.ptr, b.shape[1], c.ptr, N, None) == OK
    ref = (a.T if tA else a).astype(np.float64) @ (b.T if tB else b).astype(np.float64)
    out = c.get()
    assert np.isfinite(out).all()
    assert np.linalg.norm(out - ref) / np.linalg.norm(ref) <= 1e-4


@pytest.mark.parametrize("call,needle", [
    (lambda L, p: L.cgt_amd_im2col_f32(p, 1, 1, 2, 2, 5, 5, 0, 0, 1, 1, p, None), "kernel larger"),
    (lambda L, p: L.cgt_amd_im2col_f32(p, 1, 1, 8, 8, 3, 3, 0, 0, 0, 1, p, None), "geometry"),
    (lambda L, p: L.cgt_amd_im2col_f32(None, 1, 1, 8, 8, 3, 3, 0, 0, 1, 1, p, None), "null"),
    (lambda L, p: L.cgt_amd_col2im_f32(p, 1, -1, 8, 8, 3, 3, 0, 0, 1, 1, p, None), "negative"),
    (lambda L, p: L.cgt_amd_max_pool_f32(p, 1, 1, 8, 8, 2, 2, 0, 0, 2, 2, 9, 4, p, p, None), "does not fit"),
    (lambda L, p: L.cgt_amd_max_pool_pullback_f32(p, p, 1, 1, 8, 8, 2, 2, 0, 0, -2, 2, 4, 4, p, None), "geometry"),
    (lambda L, p: L.cgt_amd_lrn_fwd_f32(p, 1, 3, 4, 4, 5, 1e-4, 0.75, 1.0, p, p, None), "size"),
    (lambda L, p: L.cgt_amd_lrn_fwd_f32(p, 1, 8, 4, 4, 5, 1e-4, 0.75, 0.0, p, p, None), "k must be positive"),
    (lambda L, p: L.cgt_amd_lrn_bwd_f32(p, p, p, p, 1, 8, 4, 4, 0, 1e-4, 0.75, p, None), "size"),
    (lambda L, p: L.cgt_amd_lrn_fwd_f32(p, 1, 8, 4, 4, 5, 1e-4, 0.75, 1.0, None, None, None), "null"),     # top may not be null (scale may)
    (lambda L, p: L.cgt_amd_lrn_bwd_from_x_f32(p, p, 1, 8, 4, 4, 5, 1e-4, 0.75, 0.0, p, None), "k must be positive"),
    (lambda L, p: L.cgt_amd_lrn_bwd_from_x_f32(p, None, 1, 8, 4, 4, 5, 1e-4, 0.75, 1.0, p, None), "null"),
    (lambda L, p: L.cgt_amd_lrn_bwd_from_x_f32(p, p, 1, 3, 4, 4, 5, 1e-4, 0.75, 1.0, p, None), "size"),
    (lambda L, p: L.cgt_amd_lrn_bwd_recompute_f32(p, None, p, 1, 8, 4, 4, 5, 1e-4, 0.75, p, None), "null"),
    (lambda L, p: L.cgt_amd_conv_same_pad_pool_pullback_f32(p, p, None, 2, 4, 4, 2, 2, 0, 0, 2, 2, 2, 2, 4, 4, p, None), "odd"),
    (lambda L, p: L.cgt_amd_sgemm(0, 0, 4, 4, 4, p, 3, p, 4, p, 4, None), "leading dimension"),
    (lambda L, p: L.cgt_amd_sgemm(0, 0, 4, 4, 4, p, 4, p, 4, None, 4, None), "null"),
    (lambda L, p: L.cgt_amd_sgemm(0, 0, -1, 4, 4, p, 4, p, 4, p, 4, None), "negative"),
    (lambda L, p: L.cgt_amd_transpose4_f32(p, (ctypes.c_long * 4)(1, 2, 3, 4), (ctypes.c_int * 4)(0, 1, 1, 3), p, None),
     "permutation"),
    (lambda L, p: L.cgt_amd_elwise_unary_f32(99, 4, p, p, None), "unknown op"),
    (lambda L, p: L.cgt_amd_elwise_binary(99, 11, 11, 4, p, 0, p, 0, p, None), "unknown op"),
    (lambda L, p: L.cgt_amd_elwise_binary(1, 7, 11, 4, p, 0, p, 0, p, None), "unsupported dtypes"),
    (lambda L, p: L.cgt_amd_repeat(p, 2, 1, (ctypes.c_long * 1)(4), (ctypes.c_int * 1)(0), p, None), "itemsize"),
    (lambda L, p: L.cgt_amd_repeat(p, 4, 9, (ctypes.c_long * 9)(*[1] * 9), (ctypes.c_int * 9)(*[0] * 9), p, None), "ndim"),
    (lambda L, p: L.cgt_amd_sum_f32(p, 1, (ctypes.c_long * 1)(-4), (ctypes.c_int * 1)(1), p, None), "negative"),
    (lambda L, p: L.cgt_amd_fill_u32(None, 0, 4, None), "null"),
])
def test_bad_arguments_are_reported_not_launched(L, call, needle):
    buf = gpu(np.arange(256, dtype=np.float32))
    rc = call(L, buf.ptr)
    assert rc == ERR_ARG, _err(L)
    assert needle in _err(L), _err(L)
    # nothing was written and the library still works
    assert np.array_equal(buf.get(), np.arange(256, dtype=np.float32))
    assert L.cgt_amd_fill_f32(buf.ptr, 2.0, 256, None) == OK
    assert np.array_equal(buf.get(), np.full(256, 2.0, np.float32))


def test_pool_outsize_rule(L):
    # ceil((H + 2p - k) / s), no "+1" (cgt/nn_ops/max_pool_2d.py:40-41)
    assert L.cgt_amd_pool_outsize(28, 2, 0, 2) == 13
    assert L.cgt_amd_pool_outsize(55, 3, 0, 2) == 26
    assert L.cgt_amd_pool_outsize(56, 2, 0, 2) == 27
    assert L.cgt_amd_pool_outsize(32, 3, 0, 2) == 15
    assert L.cgt_amd_pool_outsize(2, 5, 0, 1) == 0
    assert L.cgt_amd_pool_outsize(8, 2, 0, 0) == 0


@pytest.mark.parametrize("loads_in_flight", [8, 4, 16])
def test_stream_copy_any_alignment_and_size(L, loads_in_flight):
    # the copy kernel behind device-to-device transports: bytes before the first and after the
    # last whole 16-byte unit, source and destination aligned differently (no units at all),
    # sizes around the region of one workgroup; everything outside the range stays untouched
    assert L.cgt_amd_stream_copy_tune(8192, loads_in_flight) == OK
    try:
        rs = np.random.RandomState(7)
        total = 3 * 65536 + 64
        src_h = rs.randint(0, 256, total).astype(np.int8)
        src = gpu(src_h)
        for so, do, n in [(0, 0, 0), (0, 0, 1), (3, 3, 15), (5, 5, 16), (5, 5, 17), (0, 0, 8192), (16, 32, 8192 + 16),
                          (1, 1, 65536 + 5), (7, 23, 3 * 8192 - 1), (9, 10, 40000), (0, 16, 2 * 65536 + 48), (4, 0, 65536 * 2 + 33)]:
            dst = gpu(np.full(total, 0x55, np.int8))
            assert L.cgt_amd_stream_copy(dst.ptr + do, src.ptr + so, n, None) == OK, _err(L)
            want = np.full(total, 0x55, np.int8)
            want[do:do + n] = src_h[so:so + n]
            assert np.array_equal(dst.get(), want), (so, do, n)
        assert L.cgt_amd_stream_copy(src.ptr + 8, src.ptr, 100, None) == ERR_ARG and "overlap" in _err(L)
        assert L.cgt_amd_stream_copy(None, src.ptr, 100, None) == ERR_ARG
        assert L.cgt_amd_stream_copy_tune(5000, 8) == ERR_ARG and L.cgt_amd_stream_copy_tune(8192, 3) == ERR_ARG
    finally:
        assert L.cgt_amd_stream_copy_tune(16384, 4) == OK


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_tiles_loaded_straight_into_lds_match_the_register_path(L, tA, tB):
    # Whole tiles reach LDS through global_load_lds_dwordx4, whose LDS base travels in m0 and is set
    # from inline asm (the compiler is not told: it reserves m0 and refuses it in a clobber list).
    # If a toolchain ever kept a value of its own in m0 across that asm, or scheduled around it, the
    # direct loads would land in the wrong place -- in whole tiles only.  Edge tiles take the
    # register path (ordinary loads + ds_write), which does not touch m0: the same product with one
    # row / column fewer computes the same dot products in the same order, so its rows and columns
    # must have the bits of the whole-tile product.  Several K so that the pipelined loop (both
    # operands k-contiguous, many tiles), the plain loop and a ragged last slice are all covered.
    rs = np.random.RandomState(31)
    for M, N, K in [(256, 256, 256), (384, 1664, 96), (256, 128, 363)]:
        A = rs.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
        B = rs.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)

        def product(m, n):
            a = np.ascontiguousarray(A[:, :m] if tA else A[:m])
            b = np.ascontiguousarray(B[:n] if tB else B[:, :n])
            ga, gb, gc = gpu(a), gpu(b), gpu(np.full((m, n), np.nan, np.float32))
            assert L.cgt_amd_sgemm(tA, tB, m, n, K, ga.ptr, a.shape[1], gb.ptr, b.shape[1], gc.ptr, n, None) == OK, _err(L)
            return gc.get()

        whole = product(M, N)
        ref = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
        assert np.linalg.norm(whole - ref) <= 1e-5 * np.linalg.norm(ref)
        fewer_rows, fewer_cols = product(M - 1, N), product(M, N - 1)
        assert np.array_equal(fewer_rows.view(np.uint32), whole[:M - 1].view(np.uint32)), (tA, tB, M, N, K)
        assert np.array_equal(fewer_cols.view(np.uint32), whole[:, :N - 1].view(np.uint32)), (tA, tB, M, N, K)


def test_workspaces_of_rising_sizes_do_not_pile_up(L):
    # split-K products whose partial sums grow call by call (a shape-generic function fed rising batch
    # sizes): the stream's workspace grows geometrically and blocks it has outgrown are freed at the
    # next synchronize -- the memory held afterwards is about the largest workspace, not the sum of all
    from cgt_amd import capi
    def free_bytes():
        f, t = ctypes.c_long(), ctypes.c_long()
        assert L.cgt_amd_mem_info(ctypes.byref(f), ctypes.byref(t)) == OK
        return f.value
    s = capi.Stream()
    K = 64 * 1024
    sizes = [64 + 16 * i for i in range(24)]              # M = N: 64 .. 432, 112 splits each -> 1.8 .. 84 MB of partials
    a = gpu(np.ones((max(sizes), K), np.float32))
    b = gpu(np.ones((max(sizes), K), np.float32))
    c = gpu(np.zeros((max(sizes), max(sizes)), np.float32))
    L.cgt_amd_synchronize(None)
    before = free_bytes()
    total_asked = 0
    for m in sizes:
        assert L.cgt_amd_sgemm(0, 1, m, m, K, a.ptr, K, b.ptr, K, c.ptr, m, s.handle) == OK, _err(L)
        total_asked += m * m * 4 * 64
    assert L.cgt_amd_synchronize(s.handle) == OK
    held = before - free_bytes()
    assert np.array_equal(c.get().reshape(-1)[:sizes[-1] ** 2], np.full(sizes[-1] ** 2, K, np.float32))
    largest = sizes[-1] ** 2 * 4 * 256        # an upper bound on one call's workspace (<= 256 MiB cap)
    assert held <= min(2 * largest, 600 << 20), (held, largest, total_asked)
    del s


def test_host_threads_on_their_own_streams_get_the_bits_of_the_calls_made_alone(L):
    # the library keeps per-stream workspaces and a thread-local error string: four host threads,
    # each launching a mixed sequence (fused conv products with their split-K / tail workspaces,
    # pooling, im2col / col2im, LRN, ragged Mul22) on a stream of its own, must neither disturb each
    # other nor change a bit of what the same calls give one after another on the null stream
    import threading
    from cgt_amd import capi, kernels as K

    def work(seed, stream, out):
        rs = np.random.RandomState(seed)
        res = []
        for _ in range(6):
            B, C, Lf = rs.randint(1, 9), 16 * rs.randint(1, 5), 16 * rs.randint(1, 5)
            H, W = rs.randint(5, 40), rs.randint(5, 40)
            x = rs.randn(B, C, H, W).astype(np.float32)
            f = (rs.randn(Lf, C, 3, 3) / 12).astype(np.float32)
            xg, fg = gpu(x), gpu(f)
            xpad = K.conv_same_pad(xg, (3, 3), stream=stream)
            y = K.conv_same_fwd(xpad, fg, x.shape, stream=stream)
            top, mask = K.max_pool(y, (2, 2), (0, 0), (2, 2), stream=stream)
            gyp = K.conv_same_pad(gpu(rs.randn(*y.shape).astype(np.float32)), (3, 3), stream=stream)
            gx = K.conv_same_bwd_data(gyp, fg, x.shape, stream=stream)
            gf = K.conv_same_bwd_filter(gyp, xpad, x.shape, f.shape, stream=stream)
            col = K.im2col(xg, (3, 3), (1, 1), (1, 1), stream=stream)
            im = K.col2im(col, x.shape, (3, 3), (1, 1), (1, 1), stream=stream)
            lt, ls = K.lrn_fwd(y, 5, 1e-4, 0.75, stream=stream)
            M, N, Kk = rs.randint(1, 300), rs.randint(1, 300), rs.randint(1, 3000)
            c = K.mul22(gpu(rs.randn(M, Kk).astype(np.float32)), gpu(rs.randn(Kk, N).astype(np.float32)), stream=stream)
            capi.synchronize(stream)
            res.append([t.get() for t in (y, top, mask, gx, gf, col, im, lt, ls, c)])
        out[seed] = res

    alone, together = {}, {}
    for s in range(4):
        work(s, None, alone)
    streams = [capi.Stream() for _ in range(4)]
    threads = [threading.Thread(target=work, args=(s, streams[s].handle, together)) for s in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert sorted(together) == [0, 1, 2, 3]
    for s in range(4):
        for ra, rb in zip(alone[s], together[s]):
            for a, b in zip(ra, rb):
                assert a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))
