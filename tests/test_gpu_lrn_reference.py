"""Cross-channel LRN against the reference's own device kernels.

The reference has no CPU LRN: include/lrn.cuh is its only definition.  hipcc
compiles that file unchanged (oracle/ref_lrn_shim.hip -> oracle/_ref/
liblrn_ref.so, built where the reference tree exists), so on the GPU box the
real reference kernels pin (1) the CPU oracle's line-by-line restatement,
including the even-size window alignment that no library routine shares, and
(2) the product kernels.
"""
import numpy as np
import pytest

from oracle import oracle as O
from oracle import ref_lrn as RL

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not RL.available(), reason="oracle/_ref/liblrn_ref.so not built (no reference tree)")]

CASES = [
    # (shape, size, alpha, beta)
    ((4, 8, 16, 16), 4, 0.1, 0.5),      # the reference's test_lrn
    ((2, 32, 15, 15), 5, 1e-4, 0.75),   # CIFAR block
    ((2, 96, 27, 27), 5, 1e-4, 0.75),   # AlexNet block (smaller plane)
    ((2, 6, 5, 7), 6, 0.3, 0.75),       # C == size, even
    ((2, 9, 5, 7), 2, 0.5, 0.5),
    ((2, 9, 5, 7), 3, 0.5, 0.5),
    ((1, 12, 4, 4), 1, 0.5, 0.75),
]


def relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / np.linalg.norm(b)


@pytest.mark.parametrize("shape,size,alpha,beta", CASES)
def test_oracle_restatement_matches_reference_kernels(shape, size, alpha, beta):
    rs = np.random.RandomState(0)
    x = rs.randn(*shape)
    g = rs.rand(*shape)
    # double: same arithmetic, same order -> agreement to rounding of pow()
    rtop, rscale = RL.lrn_fwd(x, size, alpha, beta)
    otop, oscale = O.lrn_fwd(x, size, alpha, beta)
    np.testing.assert_allclose(oscale, rscale, rtol=1e-14)
    np.testing.assert_allclose(otop, rtop, rtol=1e-13)
    np.testing.assert_allclose(O.lrn_bwd(x, otop, oscale, g, size, alpha, beta),
                               RL.lrn_bwd(x, rtop, rscale, g, size, alpha, beta), rtol=1e-11, atol=1e-14)
    # single: the device may contract a*a+acc into an fma, the CPU build may not
    x32, g32 = x.astype(np.float32), g.astype(np.float32)
    rtop, rscale = RL.lrn_fwd(x32, size, alpha, beta)
    otop, oscale = O.lrn_fwd(x32, size, alpha, beta)
    assert relfro(oscale, rscale) <= 1e-6 and relfro(otop, rtop) <= 1e-6
    assert relfro(O.lrn_bwd(x32, otop, oscale, g32, size, alpha, beta),
                  RL.lrn_bwd(x32, rtop, rscale, g32, size, alpha, beta)) <= 1e-5


@pytest.mark.parametrize("shape,size,alpha,beta", CASES)
def test_product_kernels_match_reference_kernels(shape, size, alpha, beta):
    from cgt_amd import kernels as K
    from cgt_amd.gpuarray import to_gpu
    rs = np.random.RandomState(1)
    x = rs.randn(*shape).astype(np.float32)
    g = rs.rand(*shape).astype(np.float32)
    rtop, rscale = RL.lrn_fwd(x, size, alpha, beta)
    top, scale = K.lrn_fwd(to_gpu(x), size, alpha, beta)
    assert relfro(scale.get(), rscale) <= 1e-4 and relfro(top.get(), rtop) <= 1e-4
    rgb = RL.lrn_bwd(x, rtop, rscale, g, size, alpha, beta)
    gb = K.lrn_bwd(to_gpu(x), to_gpu(rtop), to_gpu(rscale), to_gpu(g), size, alpha, beta)
    assert relfro(gb.get(), rgb) <= 1e-4
