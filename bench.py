#!/usr/bin/env python3
"""Benchmark of the CGT CNN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--no-cpu]

A step is one forward+backward pass of one configured layer over one batch of
synthetic input, every buffer resident in HBM before the timed region:
    conv2d forward  = im2col -> GEMM(NT) -> transpose{0,3,1,2}
    [cross-channel LRN forward] -> max-pool forward (values + argmax)
    max-pool pullback -> [LRN backward]
    conv2d backward = transpose{0,2,3,1} -> GEMM(NN) -> col2im, GEMM(TN)
Prints ONE JSON line: the headline conv2d fwd+bwd TFLOP/s over the whole
step, a per-kernel table (HIP-event timed on the launch stream) with GB/s or
TFLOP/s against the MI355X roofs, the roofline of the dominant kernel (the
MFMA GEMM, its HBM traffic read from the counter summaries under profiles/)
and the CPU path timed on this box's host cores on a bounded sample.  The
headline workload is the VGG-style layer; the default run then measures the
other configurations the same way (AlexNet conv1 with LRN and pool, the raw
Mul22 / BatchedMul22 products, the CIFAR and MNIST first layers, whose GEMMs
sit under the HBM roof and are reported against both roofs) under "workloads".
"""
import argparse
import gc
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published

WORKLOADS = {
    # VGG-style mid layer (the headline configuration)
    "vgg_mid_conv3x3_128x56x56_b64": dict(
        x=(64, 128, 56, 56), f=(128, 128, 3, 3), pad=(1, 1), stride=(1, 1),
        fscale="he", lrn=None, pool=((2, 2), (0, 0), (2, 2))),
    # AlexNet conv1 -> LRN (k = 2, as the configuration states it; the reference's own LRN
    # has k fixed at 1, the kernel and its cost are the same) -> pool
    "alexnet_conv1_11x11s4_3x227x227_b128": dict(
        x=(128, 3, 227, 227), f=(96, 3, 11, 11), pad=(0, 0), stride=(4, 4),
        fscale=0.01, lrn=(5, 1e-4, 0.75, 2.0), pool=((3, 3), (0, 0), (2, 2))),
    # first conv of the CIFAR stack: K = 75, N = 32 -- a GEMM under the HBM roof
    "cifar_conv1_5x5_3x32x32_b128": dict(
        x=(128, 3, 32, 32), f=(32, 3, 5, 5), pad=(2, 2), stride=(1, 1),
        fscale=0.01, lrn=None, pool=((3, 3), (0, 0), (2, 2))),
    # second conv of the CIFAR stack (with its pool + LRN input side)
    "cifar_conv2_5x5_32x15x15_b128": dict(
        x=(128, 32, 15, 15), f=(64, 32, 5, 5), pad=(2, 2), stride=(1, 1),
        fscale=0.01, lrn=None, pool=None),
    # MNIST conv block (conv + pool)
    "mnist_conv3x3_1x28x28_b64": dict(
        x=(64, 1, 28, 28), f=(32, 1, 3, 3), pad=(1, 1), stride=(1, 1),
        fscale=0.1, lrn=None, pool=((2, 2), (0, 0), (2, 2))),
}
# raw dense contraction
GEMM_WORKLOAD = "raw_gemm_4096_and_batched_64x512"
DEFAULT_WORKLOAD = "vgg_mid_conv3x3_128x56x56_b64"

# The workloads the default run reports beside the headline one, under "workloads"; the
# headline layer once more as the im2col -> Mul22 -> col2im composition, which is how
# layers the fused ops do not cover run and where the VGG-sized im2col / col2im figures are
IM2COL_SUFFIX = "/im2col"
# ... and AlexNet conv1 once more over a column buffer ("/col": im2col + the fused products over it), which is
# where the AlexNet-sized im2col figure is now that the layer itself runs without one
COL_SUFFIX = "/col"
EXTRA_WORKLOADS = [DEFAULT_WORKLOAD + IM2COL_SUFFIX, "alexnet_conv1_11x11s4_3x227x227_b128",
                   "alexnet_conv1_11x11s4_3x227x227_b128" + COL_SUFFIX, GEMM_WORKLOAD,
                   "cifar_conv1_5x5_3x32x32_b128", "cifar_conv2_5x5_32x15x15_b128", "mnist_conv3x3_1x28x28_b64"]


def split_workload(workload):
    """(base workload, forced conv algorithm or None) of a name with an algorithm suffix."""
    for suffix, algo in ((IM2COL_SUFFIX, "im2col"), (COL_SUFFIX, "col")):
        if workload.endswith(suffix):
            return workload[:-len(suffix)], algo
    return workload, None

# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries of this script, per workload
PROFILE_PREFIX = {
    "vgg_mid_conv3x3_128x56x56_b64": "vgg_mid_conv3x3_b64",
    "alexnet_conv1_11x11s4_3x227x227_b128": "alexnet_conv1_b128",
}


def _pmc_rows(path):
    """(scale, rows) of a counter summary: `scale` is the calibration factor its header
    states ("factor: X"), rows are (kernel name, MB per launch) in the file's order, which is
    the order of first launch inside a step."""
    import re
    scale, rows = None, []
    with open(path) as fh:
        for line in fh:
            m = re.match(r"factor:\s*([0-9.]+)", line)
            if m:
                scale = float(m.group(1))
                continue
            parts = line.rstrip("\n").rsplit(None, 4)
            if len(parts) == 5 and "kernel" in parts[0] and parts[0].strip() != "kernel":
                try:
                    rows.append((parts[0].strip(), float(parts[4])))
                except ValueError:
                    pass
    return scale, rows


def profile_prefix(workload, algo):
    base, _ = split_workload(workload)
    prefix = PROFILE_PREFIX.get(base)
    if prefix is None or (base != DEFAULT_WORKLOAD and algo not in (None, "patch")):
        return None             # AlexNet conv1: the summaries are of the layer as nn.conv2d builds it
    return prefix + ("_im2col" if algo == "im2col" and base == DEFAULT_WORKLOAD else "")


def traffic_from_profiles(workload, algo=None, stage_names=("gemm_fwd_NT", "gemm_dgrad_NN", "gemm_wgrad_TN"), profiles_dir=None):
    """HBM bytes per launch of each GEMM stage of a step, read from the committed counter
    summaries: stage -> calibrated FETCH_SIZE + WRITE_SIZE bytes of the sgemm launch and of
    the reduce kernel that follows it (split-K / tail partials).  The summaries list kernels
    in launch order, so the sgemm rows are, in order, the forward product, the data gradient
    and the weight gradient.  {} when the workload has no summaries."""
    prefix = profile_prefix(workload, algo)
    profiles_dir = profiles_dir or os.path.join(ROOT, "profiles")
    if prefix is None:
        return {}
    total = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        path = os.path.join(profiles_dir, "%s_pmc_%s.txt" % (prefix, counter))
        if not os.path.exists(path):
            return {}
        scale, rows = _pmc_rows(path)
        if scale is None:
            return {}
        order = iter(stage_names)
        stage = None
        for name, mb in rows:
            if "sgemm_kernel" in name:
                stage = next(order, None)
            elif "reduce_" not in name:
                stage = None if stage is None else "-"     # another kernel: later reduce rows are not this GEMM's
            # splitk_reduce_kernel, tail_reduce_kernel, tail_reduce_conv_kernel: the partials' second pass
            if stage not in (None, "-") and ("sgemm_kernel" in name or "reduce_" in name):
                total[stage] = total.get(stage, 0.0) + scale * mb * 1e6
    return {k: int(round(v)) for k, v in total.items()}


def make_inputs(cfg, batch=None, seed=0):
    """Seeded synthetic inputs: legacy RandomState stream, input then weights."""
    rs = np.random.RandomState(seed)
    xs = list(cfg["x"])
    if batch is not None:
        xs[0] = batch
    x = rs.randn(*xs).astype(np.float32)
    f = rs.randn(*cfg["f"])
    if cfg["fscale"] == "he":
        f = f * np.sqrt(1.0 / np.prod(cfg["f"][1:]))
    else:
        f = f * cfg["fscale"]
    return x, f.astype(np.float32)


class Stage(object):
    def __init__(self, name, kernel, fn, work, bound, operand_bytes=None, ref_bytes=None):
        self.name, self.kernel, self.fn, self.work, self.bound = name, kernel, fn, work, bound
        self.operand_bytes = operand_bytes      # GEMM stages: 4 * (|A| + |B| + |C|), the compulsory traffic
        # HBM stages whose op moves fewer arrays than the reference's algorithm does (`work` is what
        # the op as built has to move): the reference algorithm's bytes, the unit its figures are quoted in
        self.ref_bytes = ref_bytes
        self.ms = self.ms_median = self.ms_min = self.ms_in_step = self.ms_copy_in_step = None


class LayerOnGpu(object):
    """One configured layer with every buffer pre-allocated on the device."""

    def __init__(self, cfg, overlap=False, glue=False, algo="auto", batch=None, seed=0, cotangent="ones"):
        """batch / seed: another batch size and input stream than the configured ones (the parity
        gate runs the very stage list that is timed on a 2-image slice); cotangent "ones" is the
        configured loss (sum of outputs), "random" a seeded N(0,1) one for the gate."""
        from cgt_amd import capi, kernels as K
        from cgt_amd.gpuarray import empty, to_gpu
        # two streams (default priority): the weight-gradient GEMM depends only on
        # the transposed output gradient and the column buffer, so step() runs
        # it beside the data-gradient GEMM + col2im
        self._main, self._side = capi.Stream(), capi.Stream()
        self._fork, self._join = capi.Event(), capi.Event()
        self.overlap = overlap
        stream = self._main.handle
        self._wgrad_stream = stream
        self.cfg, self.K, self.stream = cfg, K, stream
        x, f = make_inputs(cfg, batch, seed)
        cot_rs = np.random.RandomState(seed + 1000)
        self._cot = (lambda shape: np.ones(shape, np.float32)) if cotangent == "ones" else \
                    (lambda shape: cot_rs.randn(*shape).astype(np.float32))
        B, C, H, W = x.shape
        L, _, r, c = f.shape
        pad, stride = cfg["pad"], cfg["stride"]
        m, n = K.conv_outsize(H, r, pad[0], stride[0]), K.conv_outsize(W, c, pad[1], stride[1])
        Z = C * r * c
        Bmn = B * m * n
        self.dims = dict(B=B, C=C, H=H, W=W, L=L, r=r, c=c, m=m, n=n, Z=Z, Bmn=Bmn)
        self.x, self.f = to_gpu(x), to_gpu(f)
        self.f_LZ = self.f.reshape(L, Z)
        nelem = lambda a: int(np.prod(a.shape))  # noqa: E731
        # what nn.conv2d builds for this layer: the fused ops without a column buffer where they
        # apply (stride 1, same padding, channel counts in multiples of 16), else im2col and the fused
        # products over the column buffer ("col"); "im2col" is the literal composition with Mul22 and
        # the two transposes
        if algo == "auto":
            self.algo = ("direct" if K.conv_same_supported(C, L, (r, c), pad, stride) else
                         "patch" if C < 16 and K.conv_patch_supported(x.shape, (r, c), pad, stride) else "col")
        else:
            self.algo = algo
        patch = self.algo == "patch"          # no column buffer for the forward product and the weight gradient
        fused_col = self.algo in ("col", "patch")
        if self.algo == "direct":
            self.overlap = False
            self.glue = glue
            self._direct_stages(K, cfg, nelem)
            return
        self.col = None if patch else empty((B, m, n, Z))
        self.col2 = None if patch else self.col.reshape(Bmn, Z)
        self.y_mnL = None if fused_col else empty((Bmn, L))
        self.y = empty((B, L, m, n))
        act = self.y
        st = []
        s = stream
        gemm_bytes = 4 * (Bmn * Z + L * Z + Bmn * L)      # the three conv products touch the same three matrices
        if not patch:
            st.append(Stage("im2col", "im2col_linear_kernel or im2col_pipe_kernel", lambda: K.im2col(self.x, (r, c), pad, stride, out=self.col, stream=s),
                            4 * (nelem(self.x) + nelem(self.col)), "hbm"))
        patch_bytes = 4 * (nelem(self.x) + L * Z + Bmn * L)      # image + filters + result
        if patch:           # the product gathers the patches from x and writes [B,L,m,n] itself
            st.append(Stage("gemm_fwd", "sgemm_kernel", lambda: K.conv_patch_fwd(self.x, self.f, pad, stride, out=self.y, stream=s),
                            2 * Bmn * L * Z, "mfma", patch_bytes))
        elif fused_col:     # the product writes [B,L,m,n] itself
            st.append(Stage("gemm_fwd", "sgemm_kernel", lambda: K.conv_col_fwd(self.col, self.f, out=self.y, stream=s),
                            2 * Bmn * L * Z, "mfma", gemm_bytes))
        else:
            st.append(Stage("gemm_fwd_NT", "sgemm_kernel", lambda: K.mul22(self.col2, self.f_LZ, False, True, out=self.y_mnL, stream=s),
                            2 * Bmn * L * Z, "mfma", gemm_bytes))
            st.append(Stage("transpose_0312", "thin_transpose_kernel or batched_transpose_kernel",
                            lambda: K.transpose4(self.y_mnL.reshape(B, m, n, L), (0, 3, 1, 2), out=self.y, stream=s),
                            2 * 4 * nelem(self.y), "hbm"))
        if cfg["lrn"]:
            size, alpha, beta, k = cfg["lrn"]
            # what nn.cross_channel_lrn builds beside the fused conv ops: only `top` is stored and the
            # gradient forms the scale again from x (two arrays forward, three backward); the literal
            # composition keeps the reference's (top, scale) pair (three forward, four backward: `top`
            # is formed again).  The reference's algorithm moves three and five.
            lean_lrn = patch or fused_col
            self.top = empty(self.y.shape)
            self.scale = None if lean_lrn else empty(self.y.shape)
            if lean_lrn:
                st.append(Stage("lrn_fwd", "lrn_fwd_kernel", lambda: K.lrn_fwd(self.y, size, alpha, beta, k, out=self.top, stream=s, want_scale=False),
                                2 * 4 * nelem(self.y), "hbm", ref_bytes=3 * 4 * nelem(self.y)))
            else:
                st.append(Stage("lrn_fwd", "lrn_fwd_flat_kernel or lrn_fwd_kernel", lambda: K.lrn_fwd(self.y, size, alpha, beta, k, out=(self.top, self.scale), stream=s),
                                3 * 4 * nelem(self.y), "hbm"))
            act = self.top
        if cfg["pool"]:
            pk, pp, ps = cfg["pool"]
            PH, PW = K.pool_outsize(m, pk[0], pp[0], ps[0]), K.pool_outsize(n, pk[1], pp[1], ps[1])
            self.pool, self.mask = empty((B, L, PH, PW)), empty((B, L, PH, PW), np.int32)
            self.gpool = to_gpu(self._cot((B, L, PH, PW)))
            self.gact = empty(self.y.shape)
            pool_in = act
            st.append(Stage("max_pool_fwd", "max_pool_fwd_kernel", lambda: K.max_pool(pool_in, pk, pp, ps, out=(self.pool, self.mask), stream=s),
                            4 * (nelem(self.y) + 2 * nelem(self.pool)), "hbm"))
            st.append(Stage("max_pool_bwd", "max_pool_bwd_block_kernel",
                            lambda: K.max_pool_pullback(self.y.shape, self.mask, self.gpool, pk, pp, ps, out=self.gact, stream=s),
                            4 * (2 * nelem(self.pool) + nelem(self.y)), "hbm"))
            gy = self.gact
        else:
            gy = to_gpu(self._cot(self.y.shape))   # "ones": loss = sum of outputs
        if cfg["lrn"]:
            self.gy_lrn = empty(self.y.shape)
            g_in = gy
            if lean_lrn:    # x and the cotangent in, one array out
                st.append(Stage("lrn_bwd", "lrn_bwd_x_kernel",
                                lambda: K.lrn_bwd_from_x(self.y, g_in, size, alpha, beta, k, out=self.gy_lrn, stream=s),
                                3 * 4 * nelem(self.y), "hbm", ref_bytes=5 * 4 * nelem(self.y)))
            else:           # as the Op's closure calls it: `top` is formed again from x and scale, not read
                st.append(Stage("lrn_bwd", "lrn_bwd_kernel",
                                lambda: K.lrn_bwd(self.y, None, self.scale, g_in, size, alpha, beta, out=self.gy_lrn, stream=s),
                                4 * 4 * nelem(self.y), "hbm", ref_bytes=5 * 4 * nelem(self.y)))
            gy = self.gy_lrn
        self.gy = gy
        self.gcol = empty((Bmn, Z))
        self.gx = empty(self.x.shape)
        self.gf = empty((L, Z))
        col2im = Stage("col2im", "col2im_stream_kernel",
                       lambda: K.col2im(self.gcol.reshape(B, m, n, Z), self.x.shape, (r, c), pad, stride, out=self.gx, stream=s),
                       4 * (nelem(self.x) + nelem(self.gcol)), "hbm")
        if fused_col:       # both gradient products read the NCHW cotangent themselves
            self.overlap = False
            gcol4, gf4 = self.gcol.reshape(B, m, n, Z), self.gf.reshape(L, C, r, c)
            st.append(Stage("gemm_dgrad", "sgemm_kernel", lambda: K.conv_col_bwd_data(self.gy, self.f, out=gcol4, stream=s),
                            2 * Bmn * L * Z, "mfma", gemm_bytes))
            st.append(col2im)
            if patch:
                st.append(Stage("gemm_wgrad", "sgemm_kernel", lambda: K.conv_patch_bwd_filter(self.gy, self.x, self.f.shape, pad, stride, out=gf4, stream=s),
                                2 * Bmn * L * Z, "mfma", patch_bytes))
            else:
                st.append(Stage("gemm_wgrad", "sgemm_kernel", lambda: K.conv_col_bwd_filter(self.gy, self.col, self.f.shape, out=gf4, stream=s),
                                2 * Bmn * L * Z, "mfma", gemm_bytes))
        else:
            self.gc = empty((B, m, n, L))
            self.gc2 = self.gc.reshape(Bmn, L)
            st.append(Stage("transpose_0231", "thin_transpose_kernel or batched_transpose_kernel", lambda: K.transpose4(self.gy, (0, 2, 3, 1), out=self.gc, stream=s),
                            2 * 4 * nelem(self.y), "hbm"))
            st.append(Stage("gemm_dgrad_NN", "sgemm_kernel", lambda: K.mul22(self.gc2, self.f_LZ, False, False, out=self.gcol, stream=s),
                            2 * Bmn * L * Z, "mfma", gemm_bytes))
            st.append(col2im)
            st.append(Stage("gemm_wgrad_TN", "sgemm_kernel", lambda: K.mul22(self.gc2, self.col2, True, False, out=self.gf, stream=self._wgrad_stream),
                            2 * Bmn * L * Z, "mfma", gemm_bytes))
        self.stages = st
        self.conv_flops = 6 * Bmn * L * Z
        # The glue a SpatialConvolution training step adds around this layer
        # (bias add, ReLU = x*(x>=0), their gradients, scalar loss): timed in the
        # per-kernel table only, never part of step() / `value`.
        self.extra_stages = []
        if glue:
            ex = self.extra_stages
            ny = nelem(self.y)
            self.bias = to_gpu(np.zeros((1, L, 1, 1), np.float32))
            self.zero = to_gpu(np.float32(0).reshape(()))
            self.bias_full, self.pre, self.act = empty(self.y.shape), empty(self.y.shape), empty(self.y.shape)
            self.mask_ge = empty(self.y.shape, np.int8)
            self.gpre, self.gbias, self.loss = empty(self.y.shape), empty((1, L, 1, 1)), empty((1, 1, 1, 1))
            ex.append(Stage("repeat_bias", "repeat_rkr_kernel",
                            lambda: K.repeat(self.bias, (0, 2, 3), (B, m, n), out=self.bias_full, stream=s), 4 * ny, "hbm"))
            ex.append(Stage("add_bias", "elwise_binary_kernel",
                            lambda: K.elwise_binary("+", self.y, self.bias_full, out=self.pre, stream=s), 12 * ny, "hbm"))
            ex.append(Stage("relu_mask_ge", "elwise_binary_kernel",
                            lambda: K.elwise_binary(">=", self.pre, self.zero, out=self.mask_ge, stream=s), 5 * ny, "hbm"))
            ex.append(Stage("relu_mul", "elwise_binary_kernel",
                            lambda: K.elwise_binary("*", self.pre, self.mask_ge, out=self.act, stream=s), 9 * ny, "hbm"))
            ex.append(Stage("relu_grad_mul", "elwise_binary_kernel",
                            lambda: K.elwise_binary("*", self.mask_ge, self.gy, out=self.gpre, stream=s), 9 * ny, "hbm"))
            ex.append(Stage("bias_grad_sum", "sum_rkr_kernel",
                            lambda: K.sum_keepdims(self.gpre, (0, 2, 3), out=self.gbias, stream=s), 4 * ny, "hbm"))
            ex.append(Stage("loss_sum", "sum_rkr_kernel",
                            lambda: K.sum_keepdims(self.act, (0, 1, 2, 3), out=self.loss, stream=s), 4 * ny, "hbm"))

    def _direct_stages(self, K, cfg, nelem):
        """The same layer without a column buffer: pad -> GEMM over the padded image (writes
        NCHW itself), pool both ways, pad of the cotangent -> data-gradient GEMM, weight-gradient
        GEMM.  Every stage is one kernel (plus the weight gradient's split-K reduce kernel)."""
        from cgt_amd import capi
        from cgt_amd.gpuarray import empty, to_gpu
        lib = capi.lib()
        d = self.dims
        B, C, H, W, L, r, c, Bmn, Z = d["B"], d["C"], d["H"], d["W"], d["L"], d["r"], d["c"], d["Bmn"], d["Z"]
        s = self.stream
        self.xpad = empty((K.conv_same_padded_size(B * C, H, W, (r, c)),))
        self.gypad = empty((K.conv_same_padded_size(B * L, H, W, (r, c)),))
        self.fk, self.fflip = empty((L, r * c, C)), empty((C, r * c, L))
        self.y, self.gx, self.gf = empty((B, L, H, W)), empty(self.x.shape), empty(self.f.shape)

        def call(fn, *a):
            capi.check(fn(*a))
        gemm_flops = 2 * Bmn * L * Z
        gemm_bytes = 4 * (nelem(self.x) + L * Z + Bmn * L)       # image + filters + result: no column buffer
        st = []
        st.append(Stage("pad_x", "pad_planes_kernel", lambda: K.conv_same_pad(self.x, (r, c), out=self.xpad, stream=s),
                        4 * (nelem(self.x) + nelem(self.xpad)), "hbm"))
        st.append(Stage("filter_fwd", "batched_transpose_kernel",
                        lambda: call(lib.cgt_amd_conv_same_filter_f32, self.f.ptr, L, C, r, c, 0, self.fk.ptr, s), 8 * L * Z, "hbm"))
        st.append(Stage("gemm_fwd", "sgemm_kernel",
                        lambda: call(lib.cgt_amd_conv_same_product_f32, self.xpad.ptr, self.fk.ptr, None, 0, B, C, H, W, L, r, c, self.y.ptr, None, s),
                        gemm_flops, "mfma", gemm_bytes))
        act = self.y
        if cfg["pool"]:
            pk, pp, ps = cfg["pool"]
            PH, PW = K.pool_outsize(H, pk[0], pp[0], ps[0]), K.pool_outsize(W, pk[1], pp[1], ps[1])
            self.pool, self.mask = empty((B, L, PH, PW)), empty((B, L, PH, PW), np.int32)
            self.gpool = to_gpu(self._cot((B, L, PH, PW)))
            st.append(Stage("max_pool_fwd", "max_pool_fwd_kernel", lambda: K.max_pool(act, pk, pp, ps, out=(self.pool, self.mask), stream=s),
                            4 * (nelem(self.y) + 2 * nelem(self.pool)), "hbm"))
            # the pool's pullback writes the padded cotangent itself (what the Op graph builds:
            # ConvPadPoolPullback in the place of MaxPoolPullback -> ConvPad)
            st.append(Stage("max_pool_bwd_padded", "max_pool_bwd_padded_kernel",
                            lambda: K.conv_same_pad_pool_pullback(self.y.shape, self.mask, self.gpool, pk, pp, ps, (r, c),
                                                                  out=self.gypad, stream=s),
                            4 * (2 * nelem(self.pool) + nelem(self.gypad)), "hbm"))
        else:
            self.gy = to_gpu(self._cot(self.y.shape))
            st.append(Stage("pad_gy", "pad_planes_kernel", lambda: K.conv_same_pad(self.gy, (r, c), out=self.gypad, stream=s),
                            4 * (nelem(self.y) + nelem(self.gypad)), "hbm"))
        st.append(Stage("filter_flip", "flip_filters_kernel",
                        lambda: call(lib.cgt_amd_conv_same_filter_f32, self.f.ptr, L, C, r, c, 1, self.fflip.ptr, s), 8 * L * Z, "hbm"))
        st.append(Stage("gemm_dgrad", "sgemm_kernel",
                        lambda: call(lib.cgt_amd_conv_same_product_f32, self.gypad.ptr, self.fflip.ptr, None, 0, B, L, H, W, C, r, c, self.gx.ptr, None, s),
                        gemm_flops, "mfma", gemm_bytes))
        # (the kernel that sums the product's K pieces stores the gradient in the filters' own layout)
        st.append(Stage("gemm_wgrad", "sgemm_kernel", lambda: call(lib.cgt_amd_conv_same_bwd_filter_f32, self.gypad.ptr, self.xpad.ptr, B, C, H, W, L, r, c, self.gf.ptr, s),
                        gemm_flops, "mfma", gemm_bytes))
        self.stages = st
        self.conv_flops = 6 * Bmn * L * Z
        self.extra_stages = []
        if self.glue:
            # bias add + rectify: inside the forward product's epilogue (one launch, the mask of the
            # rectify's gradient written beside the result) against the separate passes of the unfused graph
            ex = self.extra_stages
            ny = nelem(self.y)
            self.bias = to_gpu(np.zeros((1, L, 1, 1), np.float32))
            self.zero = to_gpu(np.float32(0).reshape(()))
            self.bias_full, self.pre, self.act = empty(self.y.shape), empty(self.y.shape), empty(self.y.shape)
            self.mask_ge = empty(self.y.shape, np.int8)
            ex.append(Stage("gemm_fwd_bias_relu_fused", "sgemm_kernel",
                            lambda: call(lib.cgt_amd_conv_same_product_f32, self.xpad.ptr, self.fk.ptr, self.bias.ptr, 1, B, C, H, W, L,
                                         r, c, self.act.ptr, self.mask_ge.ptr, s), gemm_bytes + ny, "hbm"))
            ex.append(Stage("gemm_fwd_plain", "sgemm_kernel",
                            lambda: call(lib.cgt_amd_conv_same_product_f32, self.xpad.ptr, self.fk.ptr, None, 0, B, C, H, W, L,
                                         r, c, self.y.ptr, None, s), gemm_bytes, "hbm"))
            ex.append(Stage("repeat_bias", "repeat_rkr_kernel",
                            lambda: K.repeat(self.bias, (0, 2, 3), (B, H, W), out=self.bias_full, stream=s), 4 * ny, "hbm"))
            ex.append(Stage("add_bias", "elwise_binary_kernel",
                            lambda: K.elwise_binary("+", self.y, self.bias_full, out=self.pre, stream=s), 12 * ny, "hbm"))
            ex.append(Stage("relu_mask_ge", "elwise_binary_kernel",
                            lambda: K.elwise_binary(">=", self.pre, self.zero, out=self.mask_ge, stream=s), 5 * ny, "hbm"))
            ex.append(Stage("relu_mul", "elwise_binary_kernel",
                            lambda: K.elwise_binary("*", self.pre, self.mask_ge, out=self.act, stream=s), 9 * ny, "hbm"))

    def step(self):
        from cgt_amd import capi
        if not self.overlap:
            for st in self.stages:
                st.fn()
            return
        main, side = self._main.handle, self._side.handle
        for st in self.stages:
            if st.name == "gemm_wgrad_TN":       # join: the next step overwrites its operands
                capi.stream_wait_event(main, self._join)
                continue
            st.fn()
            if st.name == "gemm_dgrad_NN":
                # fork after the data-gradient GEMM: the weight-gradient GEMM (matrix
                # cores) then shares the chip with col2im (HBM), not with another GEMM
                self._fork.record(main)
                capi.stream_wait_event(side, self._fork)
                self._wgrad_stream = side
                self.stages[-1].fn()
                self._wgrad_stream = main
                self._join.record(side)

    def time_stages_in_step(self, steps):
        """Each stage's duration inside real steps: an event between every two stages of `steps`
        consecutive steps (one stream).  A stage launched back to back with itself, as in
        time_stages, finds its operands and its output buffer in the last-level cache when they
        fit, and its stores can drain while the next copy runs; inside a step neither holds."""
        from cgt_amd import capi
        if self.overlap:
            return
        n = len(self.stages)
        ev = [[capi.Event() for _ in range(n + 1)] for _ in range(steps)]
        self.step()
        for k in range(steps):
            ev[k][0].record(self.stream)
            for i, st in enumerate(self.stages):
                st.fn()
                ev[k][i + 1].record(self.stream)
        capi.synchronize()
        for i, st in enumerate(self.stages):
            st.ms_in_step = sum(ev[k][i].elapsed_ms(ev[k][i + 1]) for k in range(steps)) / steps

    def time_copy_in_step(self, steps, min_bytes=4e6):
        """The yardstick for the HBM-bound stages: each one in turn is replaced by this library's
        streaming copy moving the same number of bytes (half read, half written, between two
        scratch arrays) and that copy is timed where the stage runs, with the same kernels in
        front of it and behind it.  -> st.ms_copy_in_step"""
        from cgt_amd import capi
        from cgt_amd.gpuarray import empty
        if self.overlap:
            return
        todo = [st for st in self.stages if st.bound == "hbm" and st.work >= min_bytes]
        if not todo:
            return
        half = max(st.work for st in todo) // 2 // 16 * 16
        src, dst = empty((half // 4,)), empty((half // 4,))
        self.K.fill(1.0, src.shape, out=src, stream=self.stream)
        lib, keep = capi.lib(), [st.ms_in_step for st in self.stages]
        for st in todo:
            nbytes = st.work // 2 // 16 * 16
            fn, st.fn = st.fn, (lambda nbytes=nbytes: capi.check(lib.cgt_amd_stream_copy(dst.ptr, src.ptr, nbytes, self.stream)))
            try:
                self.time_stages_in_step(steps)
                st.ms_copy_in_step = st.ms_in_step
            finally:
                st.fn = fn
        for st, ms in zip(self.stages, keep):
            st.ms_in_step = ms
        self.step()         # every buffer holds a real step's values again
        capi.synchronize()

    def time_stages(self, reps):
        from cgt_amd import capi
        for st in self.stages + getattr(self, "extra_stages", []):
            for _ in range(5):          # warm-up launches of this kernel (clock and caches settle)
                st.fn()
            e0, e1 = capi.Event(), capi.Event()
            e0.record(self.stream)
            for _ in range(reps):
                st.fn()
            e1.record(self.stream)
            st.ms = e0.elapsed_ms(e1) / reps
            # the same launches once more with an event after each one: median and
            # minimum of the individual durations (each includes the gap to the
            # previous launch, a few microseconds)
            ev = [capi.Event() for _ in range(reps + 1)]
            ev[0].record(self.stream)
            for i in range(reps):
                st.fn()
                ev[i + 1].record(self.stream)
            capi.synchronize()
            each = sorted(ev[i].elapsed_ms(ev[i + 1]) for i in range(reps))
            st.ms_median, st.ms_min = each[len(each) // 2], each[0]


class GemmOnGpu(object):
    """Mul22 4096^3 in all four transpose variants + BatchedMul22 64 x 512^3, operands ~ U(-1,1)."""

    def __init__(self, stream=None, n=4096, P=64, nb=512):
        from cgt_amd import kernels as K
        from cgt_amd.gpuarray import empty, to_gpu
        rs = np.random.RandomState(0)
        self.stream = stream
        self.A = to_gpu(rs.uniform(-1, 1, (n, n)).astype(np.float32))
        self.B = to_gpu(rs.uniform(-1, 1, (n, n)).astype(np.float32))
        self.C = empty((n, n))
        self.bA = to_gpu(rs.uniform(-1, 1, (P, nb, nb)).astype(np.float32))
        self.bB = to_gpu(rs.uniform(-1, 1, (P, nb, nb)).astype(np.float32))
        self.bC = empty((P, nb, nb))
        s = stream
        st = []
        for tA, tB, name in [(False, False, "NN"), (False, True, "NT"), (True, False, "TN"), (True, True, "TT")]:
            st.append(Stage("mul22_%s_%d" % (name, n), "sgemm_kernel",
                            (lambda tA=tA, tB=tB: K.mul22(self.A, self.B, tA, tB, out=self.C, stream=s)),
                            2 * n ** 3, "mfma", 12 * n * n))
        st.append(Stage("batched_mul22_%dx%d" % (P, nb), "sgemm_kernel",
                        lambda: K.batched_mul22(self.bA, self.bB, out=self.bC, stream=s), 2 * P * nb ** 3, "mfma",
                        12 * P * nb * nb))
        self.stages = st
        self.overlap = False
        self.conv_flops = sum(x.work for x in st)

    step = LayerOnGpu.step
    time_stages = LayerOnGpu.time_stages


def hbm_reference(reps=10):
    """What plain streaming kernels of this library reach on this box, measured in the same
    run on arrays (1 GiB each) far larger than the 256 MB last-level cache: the library's
    device-to-device copy kernel (workgroup-contiguous regions, 8 x 16-byte loads in flight
    per lane, non-temporal stores), the runtime's own memcpy beside it, a pure write (fill),
    a pure read (sum) and an elementwise add (two reads, one write).  The HBM-bound stages are
    priced against the published 8 TB/s; these rows say how much of that a kernel with no
    index arithmetic at all gets here."""
    from cgt_amd import capi, kernels as K
    from cgt_amd.gpuarray import empty
    n = 1 << 28
    a, b, c = empty((n,)), empty((n,)), empty((n,))
    s = capi.Stream()
    st = s.handle
    K.fill(1.0, (n,), out=a, stream=st)
    K.fill(2.0, (n,), out=b, stream=st)
    lib = capi.lib()
    small = empty((1,))
    rows = {}

    def timed(name, fn, nbytes):
        for _ in range(2):
            fn()
        e0, e1 = capi.Event(), capi.Event()
        e0.record(st)
        for _ in range(reps):
            fn()
        e1.record(st)
        ms = e0.elapsed_ms(e1) / reps
        rows[name] = {"ms": round(ms, 4), "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                      "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}

    timed("copy_kernel_1GiB", lambda: capi.check(lib.cgt_amd_stream_copy(c.ptr, a.ptr, 4 * n, st)), 8 * n)
    # overlapping ranges keep the runtime's copy (memmove semantics): this row is hipMemcpyAsync itself
    timed("runtime_memcpy_1GiB", lambda: capi.check(lib.cgt_amd_memcpy_async(capi.GPU, capi.GPU, a.ptr + 4096, a.ptr, 4 * n - 4096, st)), 8 * n)
    timed("write_fill_1GiB", lambda: K.fill(3.0, (n,), out=c, stream=st), 4 * n)
    timed("read_sum_1GiB", lambda: K.sum_keepdims(a, (0,), out=small, stream=st), 4 * n)
    timed("add_2r1w_1GiB", lambda: K.elwise_binary("+", a, b, out=c, stream=st), 12 * n)
    s.synchronize()
    return rows


def _relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def _same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return bool(a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint32), b.view(np.uint32)))


TOL = 1e-4      # relative Frobenius error allowed for GEMM, conv and LRN results (north_star)


def check_gemm_against_oracle(layer, rows=24):
    """Parity gate of the raw products, on the operands and launches that are timed: after one
    step every variant's result is compared, on `rows` sampled rows (and 2 sampled batches),
    with the oracle's product in float64 (reference argument mapping, cgt/core.py:2196-2205,
    2272-2285)."""
    from cgt_amd import capi
    from oracle import oracle as O
    A, B = layer.A.get().astype(np.float64), layer.B.get().astype(np.float64)
    rs = np.random.RandomState(5)
    pick = np.sort(rs.choice(A.shape[0], rows, replace=False))
    worst = 0.0
    for st, (tA, tB) in zip(layer.stages[:4], [(False, False), (False, True), (True, False), (True, True)]):
        st.fn()
        capi.synchronize()
        got = layer.C.get()[pick]
        Asub = np.ascontiguousarray(A[:, pick] if tA else A[pick])
        worst = max(worst, _relfro(got, O.mul22(Asub, B, tA, tB)))
    layer.stages[4].fn()
    capi.synchronize()
    bA, bB, bC = layer.bA.get().astype(np.float64), layer.bB.get().astype(np.float64), layer.bC.get()
    for p in (0, bA.shape[0] - 1):
        worst = max(worst, _relfro(bC[p], O.batched_mul22(bA[p:p + 1], bB[p:p + 1])[0]))
    return {"mul22_x4_batched_rel_fro": worst, "ok": bool(worst <= TOL)}


def check_layer_against_oracle(cfg, algo):
    """Parity gate run with every measurement: the stage list that is timed (same algorithm,
    same entry points, same geometry) runs once on a 2-image slice with a random cotangent, and
    every stage's output is compared with the oracle applied to that stage's inputs.  Bit-exact:
    im2col, col2im, padding, pool values, int32 mask, pool pullback (also where it is written
    into the padded layout).  Relative Frobenius <= 1e-4 against float64: conv output, LRN
    top / scale / gradient, data gradient, weight gradient.  Reference: cgt/nn.py:87-111,
    include/im2col.h:6-50, include/pooling.h:24-106, include/lrn.cuh:3-114."""
    from cgt_amd import capi
    from oracle import oracle as O
    layer = LayerOnGpu(cfg, algo=algo, batch=2, seed=1, cotangent="random")
    layer.step()
    capi.synchronize()
    d = np.float64
    pad, stride = tuple(cfg["pad"]), tuple(cfg["stride"])
    x, f = layer.x.get(), layer.f.get()
    r, c = f.shape[2:]
    exact, err = {}, {}
    y = layer.y.get()
    err["conv_fwd"] = _relfro(y, O.conv2d(x.astype(d), f.astype(d), pad, stride))
    if layer.algo == "direct":
        exact["pad"] = _same_bits(layer.xpad.get(), O.conv_same_padded(x, (r, c), layer.xpad.size))
    elif getattr(layer, "col", None) is not None:
        exact["im2col"] = _same_bits(layer.col.get(), O.im2col(x, (r, c), pad, stride))
    act = y
    if cfg["lrn"]:
        size, alpha, beta, k = cfg["lrn"]
        top64, scale64 = O.lrn_fwd(y.astype(d), size, alpha, beta, k)
        act = layer.top.get()
        err["lrn_fwd"] = _relfro(act, top64)
        if getattr(layer, "scale", None) is not None:
            err["lrn_fwd"] = max(err["lrn_fwd"], _relfro(layer.scale.get(), scale64))
    if cfg["pool"]:
        pk, pp, ps = cfg["pool"]
        opool, omask = O.max_pool(act, pk, pp, ps)
        mask = layer.mask.get()
        exact["pool_values"] = _same_bits(layer.pool.get(), opool)
        exact["pool_mask"] = _same_bits(mask, omask)
        g = O.max_pool_pullback(act.shape, mask, layer.gpool.get())
        if layer.algo == "direct":      # written straight into the padded cotangent
            exact["pool_bwd_padded"] = _same_bits(layer.gypad.get(), O.conv_same_padded(g, (r, c), layer.gypad.size))
        else:
            exact["pool_bwd"] = _same_bits(layer.gact.get(), g)
    else:
        g = layer.gy.get()
        if layer.algo == "direct":
            exact["pad_gy"] = _same_bits(layer.gypad.get(), O.conv_same_padded(g, (r, c), layer.gypad.size))
    if cfg["lrn"]:
        got = layer.gy_lrn.get()
        err["lrn_bwd"] = _relfro(got, O.lrn_bwd(y.astype(d), top64, scale64, g.astype(d), size, alpha, beta))
        g = got
    gx64, gf64 = O.conv2d_pullback(x.astype(d), f.astype(d), g.astype(d), pad, stride)
    err["conv_dgrad"] = _relfro(layer.gx.get(), gx64)
    err["conv_wgrad"] = _relfro(layer.gf.get().reshape(f.shape), gf64)
    if getattr(layer, "gcol", None) is not None:
        B, C, H, W = x.shape
        gcol = layer.gcol.get().reshape(B, layer.dims["m"], layer.dims["n"], layer.dims["Z"])
        exact["col2im"] = _same_bits(layer.gx.get(), O.col2im(gcol, x.shape, (r, c), pad, stride))
    ok = all(exact.values()) and all(v <= TOL for v in err.values())
    return {"ok": bool(ok), "algo": layer.algo, "images": 2, "bit_exact": exact,
            "rel_fro": {k: float("%.2e" % v) for k, v in err.items()}}


def settle_clock(step, settle_ms):
    """Untimed steps until the device has been under load for settle_ms milliseconds.  After an
    idle stretch (the host-side parity gate, compilation) the power manager takes about 25 ms of
    load to reach the clock it then sustains: the first step runs 14 % slower than the sixteenth,
    and five warm-up steps of 1.4 ms end in the middle of that ramp.  Returns the steps run."""
    from cgt_amd import capi
    n, t0 = 0, time.perf_counter()
    while settle_ms > 0 and (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(5):
            step()
        capi.synchronize()
        n += 5
    return n


def op_api_step_ms(cfg, steps, warmup, settle_ms=0):
    """The same layer built with the Op API (nn.conv2d / cross_channel_lrn /
    max_pool_2d, grad through the ops' pullbacks), compiled with cgt.function and
    replayed by the C++ interpreter on one stream: ms per step."""
    import cgt_amd as cgt
    from cgt_amd import capi, nn
    x, f = make_inputs(cfg)
    xn, fn = cgt.constant(x), cgt.constant(f)
    out = nn.conv2d(xn, fn, tuple(cfg["f"][2:]), tuple(cfg["pad"]), tuple(cfg["stride"]))
    if cfg["lrn"]:
        size, alpha, beta, k = cfg["lrn"]
        out = nn.cross_channel_lrn(out, size, alpha, beta, k)
    if cfg["pool"]:
        pk, pp, ps = cfg["pool"]
        out = nn.max_pool_2d(out, pk, pp, ps)
    gx, gf = cgt.grad(out, [xn, fn], goutput=cgt.ones(cgt.shape(out)))
    fun = cgt.function([xn, fn], [out, gx, gf], device_outputs=True)
    args = (xn.value, fn.value)
    del out, gx, gf
    settle_clock(lambda: fun(*args), settle_ms)
    for _ in range(warmup):
        fun(*args)
    capi.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fun(*args)
    capi.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3, fun.n_instructions


def cpu_baseline(cfg, sample_batch):
    """The CPU path (oracle stages + OpenBLAS sgemm) on a bounded sample of the workload."""
    from oracle import cpu_baseline as CB
    from oracle import oracle as O
    threads = CB.set_threads(min(CB.host_cores(), 16))
    x, f = make_inputs(cfg, batch=sample_batch)
    pad, stride = cfg["pad"], cfg["stride"]
    L, C, r, c = f.shape
    m = O.conv_outsize(x.shape[2], r, pad[0], stride[0])
    n = O.conv_outsize(x.shape[3], c, pad[1], stride[1])
    gy = np.ones((sample_batch, L, m, n), np.float32)
    # the reference's own loops where they were compiled here (im2col_cpu / col2im_cpu with this
    # geometry as template constants, pooling.h), the oracle's restatement elsewhere
    conv_kind = CB.conv_impl((r, c), pad, stride)[1]
    P, pool_kind = CB.pool_impl()
    from_reference = ([s for s in ("im2col", "col2im") if conv_kind == "reference"] +
                      [s for s in ("max_pool_fwd", "max_pool_bwd") if pool_kind == "reference" and cfg["pool"]])

    def run():
        y, gx, gf = CB.conv2d_fwd_bwd(x, f, gy, pad, stride)
        act = y
        if cfg["lrn"]:
            size, alpha, beta, k = cfg["lrn"]
            act, scale = O.lrn_fwd(y, size, alpha, beta, k)
        if cfg["pool"]:
            pk, pp, ps = cfg["pool"]
            pool, mask = P.max_pool(act, pk, pp, ps)
            g = P.max_pool_pullback(act.shape, mask, np.ones_like(pool))
            if cfg["lrn"]:
                O.lrn_bwd(y, act, scale, g, size, alpha, beta)

    best, reps = CB.timed(run, min_seconds=8.0, max_reps=20)
    flops = 6 * sample_batch * m * n * L * C * r * c
    # the same stages one by one (GB/s for the single-threaded C loops, TFLOP/s for OpenBLAS)
    per_stage = {}
    for name, (sec, work) in CB.stage_times(x, f, gy, pad, stride, cfg["pool"], cfg["lrn"]).items():
        if name.startswith("gemm"):
            per_stage[name] = {"ms": round(sec * 1e3, 3), "TFLOPs": round(work / sec / 1e12, 4)}
        else:
            per_stage[name] = {"ms": round(sec * 1e3, 3), "GBps": round(work / sec / 1e9, 3),
                               "impl": "reference" if name in from_reference else "port"}
    # "port": not every stage is the reference's own code (its GEMM library is a build-time download,
    # its transpose generated C, its LRN CUDA only); `reference_stages` names the ones that are
    return {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port", "stages": per_stage,
            "reference_stages": from_reference,
            "sample_short": "%d of %d images, best of %d passes (%.2f s each); 1-thread C loops (%s: the reference's own, -O3), "
                            "GEMM %s x%d threads; %s" % (sample_batch, cfg["x"][0], reps, best, "/".join(from_reference) or "none",
                                                         " ".join(CB.blas_config().split()[:2]), threads, CB.cpu_model()),
            "sample": "%d of %d images of the workload, best of %d passes (%.2f s each); single-threaded C: %s the "
                      "reference's own loops compiled -O3 (geometry as template constants), transposes/LRN%s the "
                      "oracle's restatement; GEMM %s with %d threads; host %s, %d cores usable"
                      % (sample_batch, cfg["x"][0], reps, best, "/".join(from_reference) if from_reference else "none of them",
                         "" if from_reference else "/im2col/col2im/pool",
                         CB.blas_config(), threads, CB.cpu_model(), CB.host_cores())}


def cpu_gemm_baseline(n=2048):
    from oracle import cpu_baseline as CB
    threads = CB.set_threads(min(CB.host_cores(), 16))
    rs = np.random.RandomState(0)
    A = rs.uniform(-1, 1, (n, n)).astype(np.float32)
    B = rs.uniform(-1, 1, (n, n)).astype(np.float32)
    best, reps = CB.timed(lambda: CB.sgemm(A, B), min_seconds=8.0, max_reps=200)
    return {"value": 2 * n ** 3 / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "Mul22 NN %d^3 (1/8 of the 4096^3 work), best of %d; %s with %d threads; host %s"
                      % (n, reps, CB.blas_config(), threads, CB.cpu_model())}


def measure(workload, args, primary):
    """Run one workload: timed steps, both stage clocks, the stage table.  Returns the
    fields of the JSON line that describe it (the caller adds the Op API and CPU legs)."""
    from cgt_amd import capi
    is_gemm = workload == GEMM_WORKLOAD
    if is_gemm:
        cfg = {"x": [4096, 4096], "f": [4096, 4096], "pad": [], "stride": []}
        layer = GemmOnGpu()
        parity = {"ok": True, "skipped": True} if args.no_check else check_gemm_against_oracle(layer)
    else:
        base, forced = split_workload(workload)
        cfg = WORKLOADS[base]
        layer = LayerOnGpu(cfg, overlap=primary and args.overlap and not args.no_overlap, glue=primary and args.glue,
                           algo=forced or args.conv_algo)
        parity = {"ok": True, "skipped": True} if args.no_check else check_layer_against_oracle(cfg, forced or args.conv_algo)

    settle_steps = settle_clock(layer.step, args.settle_ms)
    for _ in range(args.warmup):
        layer.step()
    capi.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        layer.step()
    capi.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    # Two clocks per stage.  "ms_in_step": events between the stages of real steps (what a
    # launch costs where it runs: after another kernel, operands wherever that left them) --
    # the roofline figure uses this one.  "ms": the same launch repeated back to back, the
    # kernel's own steady state (HBM kernels look better there than inside a step: repeated on
    # the same buffers they find part of them in the 256 MB last-level cache; GEMMs look worse:
    # the chip holds a lower clock under sustained matrix load).  --stage-reps 0 skips the second.
    in_step_steps = max(5, min(args.steps, 20))
    stage_reps = args.stage_reps if primary or is_gemm else 0      # extra layers: the in-step clock only
    if stage_reps > 0 or is_gemm or (primary and args.glue) or getattr(layer, "overlap", False):
        layer.time_stages(max(stage_reps, 1))
    if not is_gemm:
        layer.time_stages_in_step(in_step_steps)
        if not args.no_copy_yardstick:
            layer.time_copy_in_step(in_step_steps)

    def clock(st):          # the stage's duration for the roofline: inside the step where measured
        t = getattr(st, "ms_in_step", None)
        return t if t is not None else st.ms

    stages = []
    gemm_flops = gemm_ms = 0.0
    dominant = max((st for st in layer.stages if st.bound == "mfma"), key=clock)
    for st in layer.stages:
        row = {"stage": st.name, "kernel": st.kernel, "bound": st.bound}
        peak = HBM_PEAK_GBS if st.bound == "hbm" else FP32_MFMA_PEAK_TFLOPS
        unit, scale = ("GBps", 1e9) if st.bound == "hbm" else ("TFLOPs", 1e12)
        row["bytes" if st.bound == "hbm" else "flops"] = st.work
        if st.ms is not None:
            rate = st.work / (st.ms * 1e-3) / scale
            row.update({"ms": round(st.ms, 4), "ms_median": round(st.ms_median, 4), "ms_min": round(st.ms_min, 4),
                        unit: round(rate, 2), "frac": round(rate / peak, 4)})
        if getattr(st, "ms_in_step", None) is not None:
            rate = st.work / (st.ms_in_step * 1e-3) / scale
            row.update({"ms_in_step": round(st.ms_in_step, 4), unit + "_in_step": round(rate, 2),
                        "frac_in_step": round(rate / peak, 4)})
        if getattr(st, "ms_copy_in_step", None) is not None and getattr(st, "ms_in_step", None):
            # the same bytes moved by the plain streaming copy at this place in the step
            row.update({"ms_copy_same_bytes_in_step": round(st.ms_copy_in_step, 4),
                        "frac_copy_same_bytes_in_step": round(st.work / (st.ms_copy_in_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                        "vs_copy_in_step": round(st.ms_copy_in_step / st.ms_in_step, 3)})
        if st.bound == "hbm" and getattr(st, "ref_bytes", None):
            row.update({"bytes_reference_algorithm": st.ref_bytes,
                        "GBps_in_reference_bytes": round(st.ref_bytes / (clock(st) * 1e-3) / 1e9, 1)})
        if st.bound == "mfma":
            gemm_flops += st.work
            gemm_ms += clock(st)
            # both roofs: a product with a short K (the CIFAR / MNIST first layers) moves more
            # bytes per flop than the chip's 19.7 flop/byte balance and sits under the HBM roof
            if getattr(st, "operand_bytes", None):
                gbs = st.operand_bytes / (clock(st) * 1e-3) / 1e9
                intensity = st.work / st.operand_bytes
                row.update({"bytes": st.operand_bytes, "GBps_operands": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                            "flop_per_byte": round(intensity, 2),
                            "roof": "hbm" if intensity < FP32_MFMA_PEAK_TFLOPS * 1e3 / HBM_PEAK_GBS else "mfma"})
        stages.append(row)
    glue_stages = []
    for st in getattr(layer, "extra_stages", []):
        gbs = st.work / (st.ms * 1e-3) / 1e9
        glue_stages.append({"stage": st.name, "kernel": st.kernel, "ms": round(st.ms, 4), "bound": "hbm",
                            "bytes": st.work, "GBps": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4)})
    gemm_tf = gemm_flops / (gemm_ms * 1e-3) / 1e12
    value = layer.conv_flops / (ms_per_step * 1e-3) / 1e12
    mfma_stages = [st.name for st in layer.stages if st.bound == "mfma"]
    algo = getattr(layer, "algo", None)
    traffic = traffic_from_profiles(workload, algo, mfma_stages).get(dominant.name)
    config = {"workload": workload, "x": list(cfg["x"]), "filters": list(cfg["f"]),
              "pad": list(cfg["pad"]), "stride": list(cfg["stride"]),
              "value_is": "conv GEMM flops 6*B*m*n*L*Z / whole step time, every stage counted: " +
                          ", ".join(st.name for st in layer.stages if st.bound == "hbm"),
              "schedule": ("one stream" if not getattr(layer, "overlap", False) else
                           "weight-gradient GEMM on a second stream beside col2im")}
    if algo:
        config["conv_algo"] = {"direct": "fused ops, no column buffer (pad -> GEMM over the padded image -> NCHW)",
                               "col": "im2col -> fused products over the column buffer (NCHW written / read by the GEMMs) -> col2im",
                               "patch": "forward product and weight gradient gather their patches from the image (no column buffer, "
                                        "NCHW written / read by the GEMMs); data gradient over a column buffer -> col2im",
                               "im2col": "im2col -> Mul22 -> transpose; transpose -> Mul22 -> col2im, Mul22"}[algo]
    if is_gemm:
        config["value_is"] = "flops of Mul22 4096^3 x {NN,NT,TN,TT} + BatchedMul22 64x512^3 / step time"
    elif cfg.get("lrn"):
        config["lrn"] = dict(zip(("size", "alpha", "beta", "k"), cfg["lrn"]))
    res = {
        "value": round(value, 3), "ms_per_step": round(ms_per_step, 4), "config": config,
        # untimed steps run before the warm-up steps so that the timed ones see the sustained clock
        "clock_settle": {"ms": args.settle_ms, "steps": settle_steps},
        "frac_fp32_mfma_peak": round(value / FP32_MFMA_PEAK_TFLOPS, 4),
        # the dominant kernel: the slowest MFMA GEMM launch of a step
        "roofline": {"bound": "mfma", "kernel": dominant.kernel, "stage": dominant.name,
                     "achieved": round(dominant.work / (clock(dominant) * 1e-3) / 1e12, 2),
                     "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(dominant.work / (clock(dominant) * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4),
                     "flops_per_launch": dominant.work, "avg_launch_ms": round(clock(dominant), 4),
                     "timing": ("HIP events around the launch inside %d consecutive steps" % in_step_steps
                                if getattr(dominant, "ms_in_step", None) is not None else
                                "HIP events around %d back-to-back launches" % max(stage_reps, 1)),
                     "avg_launch_ms_back_to_back": None if dominant.ms is None else round(dominant.ms, 4),
                     "traffic": traffic,
                     "traffic_source": None if traffic is None else
                     "profiles/%s_pmc_{FETCH,WRITE}_SIZE.txt, calibrated" % profile_prefix(workload, algo)},
        "gemm_all_launches": {"TFLOPs": round(gemm_tf, 2), "frac": round(gemm_tf / FP32_MFMA_PEAK_TFLOPS, 4)},
        "stages": stages,
        "glue_stages": glue_stages,
        "parity": parity,
    }
    del layer, dominant, st
    gc.collect()            # the stage closures and the layer reference each other
    return res, cfg


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="milliseconds of untimed steps before the warm-up steps (0: none): the device reaches the "
                         "clock it sustains only after about 25 ms under load")
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS) + [GEMM_WORKLOAD])
    ap.add_argument("--stage-reps", type=int, default=20)
    ap.add_argument("--cpu-sample", type=int, default=16, help="images in the CPU baseline sample")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--overlap", action="store_true",
                    help="issue the weight-gradient GEMM on a second stream beside col2im (default: one stream, "
                         "which measures faster since the GEMM epilogues were trimmed)")
    ap.add_argument("--no-overlap", action="store_true", help="accepted for older command lines: one stream is the default")
    ap.add_argument("--glue", action="store_true",
                    help="also time the conv-layer glue kernels (bias add, ReLU, their gradients, loss sum) on the "
                         "layer's activation; they appear in `glue_stages`, outside the step")
    ap.add_argument("--no-op-api", action="store_true", help="skip timing the same step through the Op API")
    ap.add_argument("--no-copy-yardstick", action="store_true",
                    help="skip timing a plain copy of the same bytes in place of each HBM-bound stage")
    ap.add_argument("--no-check", action="store_true",
                    help="skip the parity gate (profiling runs: keeps its small launches out of the kernel statistics)")
    ap.add_argument("--conv-algo", default="auto", choices=["auto", "patch", "col", "im2col"],
                    help="auto: what nn.conv2d builds (the fused ops without a column buffer where they apply, else "
                         "im2col + the fused products over the column buffer); col: the latter for every layer; "
                         "im2col: always the literal im2col -> Mul22 -> transpose composition")
    ap.add_argument("--detail-file", default=None, help="also write the full JSON (stage tables of every workload) here")
    ap.add_argument("--hbm-reference-only", action="store_true",
                    help="run only the plain streaming kernels (copy, fill, sum, add over 1 GiB) and print their table")
    ap.add_argument("--only", action="store_true",
                    help="measure --workload alone (profiling runs); by default the headline workload is followed by "
                         "the other configurations, reported under `workloads`")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (the hot path has no "
                 "multi-GPU part: it would shard the batch axis)" % args.gpus)

    from cgt_amd import capi
    capi.require_gpu()
    if args.hbm_reference_only:
        print(json.dumps({"hbm_reference": hbm_reference(), "peak_GBps": HBM_PEAK_GBS, "device": capi.device_name()}))
        return
    is_gemm = args.workload == GEMM_WORKLOAD
    res, cfg = measure(args.workload, args, primary=True)
    out = {
        "metric": "conv2d fwd+bwd TFLOP/s (% fp32 MFMA peak); pool/LRN/im2col GB/s (% HBM)",
        "value": res["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
    }
    out.update({k: v for k, v in res.items() if k not in ("value", "ms_per_step")})
    out["device"] = capi.device_name()
    parity_ok = res["parity"]["ok"]
    if not is_gemm and not args.no_op_api:
        ms, n_instr = op_api_step_ms(cfg, args.steps, args.warmup, args.settle_ms)
        out["op_api_step"] = {"ms_per_step": round(ms, 4), "TFLOPs": round(res["value"] * res["ms_per_step"] / ms, 3),
                              "instructions": n_instr,
                              "what": "the same step through nn.conv2d / cross_channel_lrn / max_pool_2d + grad, compiled "
                                      "with cgt.function and replayed by the C++ interpreter (one stream)"}
    # the other configurations, same measurement (their stage tables carry the in-step clock;
    # the raw GEMMs, which have no step around them, the back-to-back one)
    if not args.only and args.workload == DEFAULT_WORKLOAD:
        out["hbm_reference"] = hbm_reference()
        out["workloads"] = {}
        for name in EXTRA_WORKLOADS:
            r, _ = measure(name, args, primary=False)
            parity_ok = parity_ok and r["parity"]["ok"]
            r["unit"] = "TFLOP/s"
            out["workloads"][name] = r
    if "hbm_reference" in out:
        # every HBM-bound stage also against what this library's streaming copy reaches in this run
        copy = out["hbm_reference"]["copy_kernel_1GiB"]["GBps"]
        for table in [out["stages"]] + [w["stages"] for w in out["workloads"].values()]:
            for row in table:
                if row["bound"] == "hbm" and "GBps_in_step" in row:
                    row["vs_measured_copy"] = round(row["GBps_in_step"] / copy, 3)
    if not args.no_cpu and not is_gemm:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample)
    elif not args.no_cpu:
        out["cpu_baseline"] = cpu_gemm_baseline()
    # stdout carries ONE compact line (the contract fields, the roofline, the CPU baseline, the parity
    # gate and one summary row per other workload); the full stage tables go to stderr as one JSON
    # line behind the word "detail", and to --detail-file when given
    detail = json.dumps(out)
    sys.stderr.write("detail " + detail + "\n")
    sys.stderr.flush()
    if args.detail_file:
        with open(args.detail_file, "w") as fh:
            fh.write(detail + "\n")
    print(json.dumps(compact_line(out), separators=(",", ":")))
    sys.stdout.flush()
    if not parity_ok:
        sys.exit("bench.py: parity gate failed")


MAX_LINE = 3500     # characters of the stdout line (a longer one has been cut by a harness that captures a tail)


def _clock_frac(row):
    return row.get("frac_in_step", row.get("frac"))


def _summary(res):
    """One short row per workload: whole-step value, its slowest GEMM launch as fraction of the
    fp32 MFMA peak, the HBM-bound stage furthest from 8 TB/s, and the gate's verdict."""
    # (stages that move less than 4 MB -- the filter permutes -- are launches, not bandwidth figures)
    hbm = [(r["stage"], _clock_frac(r), r.get("vs_copy_in_step")) for r in res["stages"]
           if r["bound"] == "hbm" and _clock_frac(r) is not None and r.get("bytes", 0) >= 4e6]
    row = {"value": res["value"], "ms_per_step": res["ms_per_step"], "gemm_frac": res["roofline"]["frac"],
           "parity_ok": res["parity"]["ok"]}
    if hbm:
        best, worst = max(hbm, key=lambda t: t[1]), min(hbm, key=lambda t: t[1])
        # [stage, fraction of 8 TB/s, fraction of what a plain copy of the same bytes reaches there]
        row["hbm_best"], row["hbm_worst"] = ([t[0], round(t[1], 3)] + ([t[2]] if t[2] is not None else []) for t in (best, worst))
    return row


def compact_line(out):
    """The stdout line: the contract fields in full, everything else boiled down."""
    keep = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data", "device")
    line = {k: out[k] for k in keep if k in out}
    cfg = out["config"]
    line["config"] = {k: cfg[k] for k in ("workload", "x", "filters", "pad", "stride", "conv_algo", "value_is", "lrn") if k in cfg}
    roof = out["roofline"]
    line["roofline"] = {k: roof[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "stage",
                                             "flops_per_launch", "avg_launch_ms", "timing")}
    line["frac_fp32_mfma_peak"] = out["frac_fp32_mfma_peak"]
    if "clock_settle" in out:       # untimed steps before the warm-up steps: {"ms": asked for, "steps": run}
        line["clock_settle"] = out["clock_settle"]
    if "cpu_baseline" in out:
        cpu = out["cpu_baseline"]
        line["cpu_baseline"] = {k: cpu[k] for k in ("value", "unit", "cores", "kind") if k in cpu}
        line["cpu_baseline"]["value"] = round(cpu["value"], 4)
        line["cpu_baseline"]["sample"] = cpu.get("sample_short", cpu["sample"])[:220]
    par = out["parity"]
    line["parity"] = {"ok": bool(par["ok"] and all(w["parity"]["ok"] for w in out.get("workloads", {}).values()))}
    for k in ("bit_exact", "rel_fro", "mul22_x4_batched_rel_fro", "skipped"):
        if k in par:
            line["parity"][k] = par[k]
    # stage -> [ms inside the step, fraction of its roof (8 TB/s or 157.3 TFLOP/s)]
    # (HBM stages: and the time of a plain copy of the same bytes at that place in the step / the stage's time)
    line["stages"] = {r["stage"]: [r.get("ms_in_step", r.get("ms")), _clock_frac(r)] +
                      ([r["vs_copy_in_step"]] if "vs_copy_in_step" in r else []) for r in out["stages"]}
    if "op_api_step" in out:
        line["op_api_step"] = {k: out["op_api_step"][k] for k in ("ms_per_step", "TFLOPs")}
    if "hbm_reference" in out:      # fraction of 8 TB/s that plain streaming kernels reach in this run
        line["hbm_reference"] = {k: v["frac"] for k, v in out["hbm_reference"].items()}
    if "workloads" in out:
        line["workloads"] = {name: _summary(r) for name, r in out["workloads"].items()}
    line["detail"] = "stderr"
    # never longer than a tail capture holds: drop the optional parts, least needed first
    for drop in (None, "stages", "hbm_reference", "op_api_step", "workloads"):
        if drop:
            line.pop(drop, None)
        if len(json.dumps(line, separators=(",", ":"))) <= MAX_LINE:
            break
    return line


if __name__ == "__main__":
    main()
