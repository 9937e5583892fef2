"""Writes the golden vectors under tests/golden/ from the REFERENCE's own CPU
code (include/im2col.h, include/pooling.h), compiled in place into
oracle/_ref/libcgt_ref.so by `make -C oracle`.  Runs only where
/root/reference exists; the fixtures it writes are committed, the reference is
not.  The reference ships no golden files of its own (its tests are
gradient-consistency checks), so these vectors are what pins the restatement
in oracle/cgt_oracle.c on machines without the reference tree.

    python tests/golden/make_golden.py

Each .npz holds, per case i, the inputs, the reference outputs and a JSON
`meta` entry with the geometry.  Cases follow the reference tests' shapes
(cgt/tests/test_imgproc.py:40-77, cgt/tests/test_conv.py:14-16) plus the edge
cases each kernel has (padding on all sides, strides that do not divide,
stride > kernel, non-square, ties, all-negative windows, shared argmax).
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

from oracle import ref  # noqa: E402


def wide_range(rs, shape):
    """fp32 values spanning ~12 decades so that a different add order shows."""
    return (rs.randn(*shape) * 10.0 ** rs.uniform(-6, 6, size=shape)).astype(np.float32)


def im2col_cases():
    rs = np.random.RandomState(0)
    ar = np.arange(2 * 1 * 28 * 28, dtype=np.float32).reshape(2, 1, 28, 28)
    cases = [
        # the three settings of the reference's test_im2col on arange(2*1*28*28)
        (ar, (4, 4, 0, 0, 1, 1)),
        (ar, (3, 3, 1, 1, 2, 2)),
        (ar, (3, 3, 1, 1, 3, 3)),
        # C > 1: Z ordering (channel, kh, kw)
        (rs.randn(2, 3, 9, 11).astype(np.float32), (3, 3, 1, 1, 1, 1)),
        (rs.randn(1, 4, 8, 8).astype(np.float32), (3, 3, 0, 0, 1, 1)),
        # 5x5 pad 2 (CIFAR block) and 11x11 stride 4 (AlexNet conv1) miniatures
        (rs.randn(2, 3, 12, 10).astype(np.float32), (5, 5, 2, 2, 1, 1)),
        (rs.randn(2, 3, 35, 31).astype(np.float32), (11, 11, 0, 0, 4, 4)),
        # non-square kernel on a non-square image, full padding (test_conv shape)
        (rs.randn(2, 2, 5, 17).astype(np.float32), (4, 7, 3, 6, 1, 1)),
        # stride > kernel: holes, col2im leaves zeros
        (rs.randn(2, 2, 10, 11).astype(np.float32), (2, 3, 0, 1, 3, 2)),
        # 1x1, 2x2/s2, mixed
        (rs.randn(2, 5, 4, 6).astype(np.float32), (1, 1, 0, 0, 1, 1)),
        (rs.randn(2, 3, 7, 9).astype(np.float32), (2, 2, 0, 0, 2, 2)),
        (rs.randn(1, 2, 9, 8).astype(np.float32), (3, 2, 1, 0, 2, 1)),
        (rs.randn(2, 2, 13, 14).astype(np.float32), (5, 3, 2, 1, 2, 3)),
        (rs.randn(1, 3, 5, 5).astype(np.float32), (2, 2, 1, 1, 1, 1)),
    ]
    out = {}
    meta = []
    for i, (x, g) in enumerate(cases):
        k, p, s = g[0:2], g[2:4], g[4:6]
        col = ref.im2col(x, k, p, s)
        gcol = wide_range(rs, col.shape)
        gim = ref.col2im(gcol, x.shape, k, p, s)
        out["c%d_x" % i] = x
        out["c%d_col" % i] = col
        out["c%d_gcol" % i] = gcol
        out["c%d_gim" % i] = gim
        meta.append({"geom": list(g), "xshape": list(x.shape)})
    out["meta"] = np.array(json.dumps(meta))
    return out


def pool_cases():
    rs = np.random.RandomState(1)
    relu = lambda a: (a * (a >= 0)).astype(np.float32)  # noqa: E731
    ties = np.zeros((1, 2, 6, 6), np.float32)
    ties[0, 1] = 3.0
    cases = [
        # reference test_pool: (2,3,5,7), k=4, s=1 -> pooled (1,3)
        (rs.randn(2, 3, 5, 7).astype(np.float32), (4, 4, 0, 0, 1, 1)),
        # k2/s2 on even H: last window dropped (size rule has no +1)
        (rs.randn(2, 3, 8, 8).astype(np.float32), (2, 2, 0, 0, 2, 2)),
        # k3/s2 overlapping windows, odd and even extents
        (rs.randn(2, 2, 11, 11).astype(np.float32), (3, 3, 0, 0, 2, 2)),
        (rs.randn(2, 2, 12, 10).astype(np.float32), (3, 3, 0, 0, 2, 2)),
        # padding: clamp order, padded cells never selected
        (rs.randn(2, 2, 7, 7).astype(np.float32), (3, 3, 1, 1, 2, 2)),
        (-np.abs(rs.randn(1, 2, 6, 7)).astype(np.float32) - 1, (3, 3, 1, 1, 1, 1)),
        # ties: post-ReLU zeros, and all-equal planes -> first (h,w)
        (relu(rs.randn(2, 3, 9, 9)), (3, 3, 0, 0, 2, 2)),
        (ties, (2, 2, 0, 0, 2, 2)),
        (ties, (3, 3, 1, 1, 2, 2)),
        # non-square window / stride
        (rs.randn(1, 3, 9, 13).astype(np.float32), (2, 3, 0, 1, 2, 1)),
        (rs.randn(1, 2, 10, 9).astype(np.float32), (3, 2, 1, 0, 3, 2)),
    ]
    out = {}
    meta = []
    for i, (x, g) in enumerate(cases):
        k, p, s = g[0:2], g[2:4], g[4:6]
        top, mask = ref.max_pool(x, k, p, s)
        gtop = wide_range(rs, top.shape)
        gb = ref.max_pool_pullback(x.shape, mask, gtop)
        out["c%d_x" % i] = x
        out["c%d_top" % i] = top
        out["c%d_mask" % i] = mask
        out["c%d_gtop" % i] = gtop
        out["c%d_gbottom" % i] = gb
        meta.append({"geom": list(g), "xshape": list(x.shape)})
    out["meta"] = np.array(json.dumps(meta))
    return out


def main():
    if not ref.available():
        raise SystemExit("oracle/_ref/libcgt_ref.so missing: run `make -C oracle` where "
                         "/root/reference exists")
    np.savez_compressed(os.path.join(HERE, "im2col_col2im.npz"), **im2col_cases())
    np.savez_compressed(os.path.join(HERE, "max_pool.npz"), **pool_cases())
    for f in ("im2col_col2im.npz", "max_pool.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
