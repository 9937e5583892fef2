"""cgt_amd_sgemm_noalloc -- the GEMM entry point that allocates nothing (its
split-K partials live in a 64 MiB device array inside the library) -- called
through the C ABI and compared, bit for bit, with cgt_amd_sgemm, whose split
plan and kernels it shares: two calls in a row on the shared scratch, the
second with a smaller input, for both workspace users (split-K and the tail
split), plus the refusal of a product whose plan needs more scratch than the
array holds.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from cgt_amd import capi
    capi.require_gpu()
    return capi


def _pair(api, tA, tB, M, N, K, seed):
    """(C from cgt_amd_sgemm_noalloc, C from cgt_amd_sgemm) on the same seeded operands."""
    from cgt_amd.gpuarray import empty, to_gpu
    rs = np.random.RandomState(seed)
    A = to_gpu(rs.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32))
    B = to_gpu(rs.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32))
    lib = api.lib()
    outs = []
    for fn in (lib.cgt_amd_sgemm_noalloc, lib.cgt_amd_sgemm):
        C = empty((M, N), np.float32)
        C.fill_u32(0x7fc00000)                      # NaN: every element must be overwritten
        api.check(fn(int(tA), int(tB), M, N, K, A.ptr, A.shape[1], B.ptr, B.shape[1], C.ptr, N, None))
        api.synchronize()
        outs.append(C.get())
    ref = (A.get().T if tA else A.get()).astype(np.float64) @ (B.get().T if tB else B.get()).astype(np.float64)
    return outs[0], outs[1], ref


def _same(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_split_k_two_calls_second_smaller(api):
    # weight-gradient shapes (TN, few tiles, long K): split-K partials go through the scratch
    got, want, ref = _pair(api, True, False, 96, 363, 40000, 0)
    assert _same(got, want)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-4
    # a smaller product right after: must not see what the first one left in the scratch
    got, want, ref = _pair(api, True, False, 32, 75, 9000, 1)
    assert _same(got, want)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-4


def test_tail_split_two_calls_second_smaller(api):
    # 300 then 260 tiles of 128x128 on 256 CUs: the partial last round is cut along K
    got, want, ref = _pair(api, False, True, 300 * 128, 128, 512, 2)
    assert _same(got, want)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-4
    got, want, ref = _pair(api, False, True, 260 * 128 - 5, 120, 256, 3)
    assert _same(got, want)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-4


def test_no_split_needs_no_scratch(api):
    got, want, _ = _pair(api, False, False, 257, 131, 77, 4)
    assert _same(got, want)


def test_plan_that_needs_more_than_the_static_scratch_is_refused(api):
    # 475 tiles: the 219 tail tiles would be cut into 7 pieces each = 1533 pieces of 64 KiB > 64 MiB
    from cgt_amd.gpuarray import empty
    M, N, K = 475 * 128, 128, 1008      # K < 1024: no split-K, the tail split applies
    A, B, C = empty((M, K), np.float32), empty((N, K), np.float32), empty((M, N), np.float32)
    lib = api.lib()
    rc = lib.cgt_amd_sgemm_noalloc(0, 1, M, N, K, A.ptr, K, B.ptr, K, C.ptr, N, None)
    assert rc == 1 and "static buffer holds" in api.last_error()
    # the allocating entry point takes the same product
    api.check(lib.cgt_amd_sgemm(0, 1, M, N, K, A.ptr, K, B.ptr, K, C.ptr, N, None))
    api.synchronize()
