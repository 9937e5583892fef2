"""The C-ABI library loads and exports every symbol include/cgt_amd.h declares
(no compute calls: this runs without a GPU)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cgt_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cgt_amd_\w+)\s*\(", text)))


def test_header_declares_the_hot_path():
    syms = declared_symbols()
    for need in ["cgt_amd_im2col_f32", "cgt_amd_col2im_f32", "cgt_amd_max_pool_f32",
                 "cgt_amd_max_pool_pullback_f32", "cgt_amd_lrn_fwd_f32", "cgt_amd_lrn_bwd_f32",
                 "cgt_amd_sgemm", "cgt_amd_sgemm_batched", "cgt_amd_transpose4_f32",
                 "cgt_amd_alloc", "cgt_amd_free", "cgt_amd_memcpy"]:
        assert need in syms


def test_library_exports_every_declared_symbol():
    from cgt_amd import capi
    if not os.path.exists(capi.libpath()):
        pytest.fail("libcgt_amd.so is not built: run `python -m cgt_amd.build`")
    handle = capi.lib()
    syms = declared_symbols()
    assert sorted(capi.PROTOTYPES) == syms, "capi.PROTOTYPES and include/cgt_amd.h disagree"
    for name in syms:
        assert getattr(handle, name) is not None


def test_no_compute_needed_for_host_only_entry_points():
    from cgt_amd import capi
    lib = capi.lib()
    assert lib.cgt_amd_version() >= 100
    assert lib.cgt_amd_pool_outsize(28, 2, 0, 2) == 13
    assert lib.cgt_amd_pool_outsize(55, 3, 0, 2) == 26
    assert lib.cgt_amd_pool_outsize(5, 4, 0, 1) == 1
    assert lib.cgt_amd_pool_outsize(2, 3, 0, 1) == 0
    assert capi.device_count() >= 0


def test_staged_pool_kernels_stay_inside_their_index_range():
    # the LDS-staged kernels split flat indices by reciprocal multiplication, exact below 2^21:
    # the launcher must fall back to the direct kernels beyond that
    from cgt_amd import capi
    lib = capi.lib()
    limit = 1 << 21
    cases = [(55, 55, 26, 26), (56, 56, 27, 27), (2100, 2100, 65, 65), (1, 1, 1001, 1001), (3, 3, 700, 700),
             (110, 110, 54, 54), (4000, 3, 124, 1), (1, 1, 1, 1), (40000, 40000, 10, 10)]
    for H, W, PH, PW in cases:
        for backward in (0, 1):
            ppw = lib.cgt_amd_pool_staged_planes(backward, H, W, PH, PW)
            assert ppw >= 0
            if ppw:
                assert ppw * H * W < limit and ppw * PH * PW < limit, (backward, H, W, PH, PW, ppw)
                assert (PH * PW * 8 if backward else H * W * 4) <= 48 * 1024
    assert lib.cgt_amd_pool_staged_planes(0, 55, 55, 26, 26) >= 1       # the AlexNet planes stay staged
    assert lib.cgt_amd_pool_staged_planes(1, 2100, 2100, 65, 65) == 0   # 4.4 M cells per plane: direct kernel
    assert lib.cgt_amd_pool_staged_planes(0, 1, 1, 1001, 1001) in (0, 1, 2)


def test_conv_same_host_side_rules():
    # which layers the im2col-free products cover, and the padded layout's size: host code only
    from cgt_amd import capi, core
    from cgt_amd.nn_ops import conv_same
    lib = capi.lib()
    ok = lambda C, L, k, p, s: lib.cgt_amd_conv_same_supported(C, L, k, k, p, p, s, s)      # noqa: E731
    assert ok(128, 128, 3, 1, 1) and ok(64, 128, 5, 2, 1) and ok(256, 512, 3, 1, 1) and ok(128, 256, 7, 3, 1)
    assert not ok(3, 96, 11, 0, 4) and not ok(128, 128, 3, 0, 1) and not ok(128, 128, 3, 1, 2)
    # channels and filters in multiples of 16 (tiles that are not whole are padded)
    assert ok(32, 64, 5, 2, 1) and ok(128, 96, 3, 1, 1) and ok(16, 16, 3, 1, 1) and ok(48, 80, 1, 0, 1)
    assert not ok(120, 128, 3, 1, 1) and not ok(128, 72, 3, 1, 1) and not ok(3, 32, 5, 2, 1)
    assert not lib.cgt_amd_conv_same_supported(128, 128, 2, 2, 0, 0, 1, 1)
    # pw zeros, then H + 2 ph rows of W + pw floats, rounded up past 16 zeros to a multiple of 16; + tail
    plane = (1 + 58 * 57 + 16 + 15) // 16 * 16
    tail = (256 + 3 * 57 + 3) // 4 * 4
    assert lib.cgt_amd_conv_same_padded_size(1, 56, 56, 3, 3) == plane + tail
    assert lib.cgt_amd_conv_same_padded_size(64 * 128, 56, 56, 3, 3) == 64 * 128 * plane + tail
    assert lib.cgt_amd_conv_same_padded_size(5, 9, 20, 5, 3) == 5 * ((1 + 13 * 21 + 31) // 16 * 16) + (256 + 5 * 21 + 3) // 4 * 4
    assert lib.cgt_amd_conv_same_padded_size(1, 56, 56, 2, 2) == -1
    # the Op's shape rule is the same number, symbolically
    info = conv_same.ConvSameInfo(3, 3)
    B = core.ShapeInt(64, ("size", object(), 0))
    n = conv_same.padded_size(B * 128, 56, 56, info)
    assert n == 64 * 128 * plane + tail and not n.is_constant()
    rc = lib.cgt_amd_conv_same_fwd_f32(None, None, None, 0, 1, 128, 8, 8, 128, 3, 3, None, None, None)
    assert rc == 1 and "null" in capi.last_error()
    rc = lib.cgt_amd_conv_same_bwd_filter_f32(None, None, 1, 128, 8, 8, 128, 4, 4, None, None)
    assert rc == 1 and "odd" in capi.last_error()


def test_argument_errors_are_reported_not_fatal():
    # argument validation happens on the host before any launch
    from cgt_amd import capi
    lib = capi.lib()
    rc = lib.cgt_amd_im2col_f32(None, 1, 1, 4, 4, 0, 3, 0, 0, 1, 1, None, None)
    assert rc == 1 and "geometry" in capi.last_error()
    rc = lib.cgt_amd_lrn_fwd_f32(None, 1, 3, 2, 2, 5, 1e-4, 0.75, 1.0, None, None, None)
    assert rc == 1 and "size" in capi.last_error()
    rc = lib.cgt_amd_sgemm(0, 0, 4, 4, 4, None, 2, None, 4, None, 4, None)
    assert rc == 1


def test_conv_col_and_patch_host_side_rules():
    # the column-buffer and patch-gather products validate on the host before any launch
    from cgt_amd import capi
    lib = capi.lib()
    ok = lambda B, C, H, W, k, p, s: lib.cgt_amd_conv_patch_supported(B, C, H, W, k, k, p, p, s, s)      # noqa: E731
    assert ok(128, 3, 227, 227, 11, 0, 4) and ok(64, 1, 28, 28, 3, 1, 1) and ok(1, 3, 5, 5, 5, 0, 1)
    assert not ok(1, 3, 4, 4, 5, 0, 1)                  # kernel larger than the padded image
    assert not ok(1, 1, 3000, 3000, 3, 1, 1)            # 9 M output pixels per image: beyond the gather's pixel walk
    assert not ok(4096, 64, 64, 64, 3, 1, 1)            # 2^30 floats: byte offsets into x would not fit 32 bits
    assert not ok(1, 3, 40000, 8, 3, 1, 1) and not ok(1, 3, 8, 8, 3, 1, 0)
    rc = lib.cgt_amd_conv_patch_fwd_f32(None, None, None, 0, 2, 3, 9, 9, 8, 3, 3, 1, 1, 1, 1, None, None, None)
    assert rc == 1 and "null" in capi.last_error()
    rc = lib.cgt_amd_conv_patch_fwd_f32(None, None, None, 0, 2, 3, 2, 2, 8, 3, 3, 0, 0, 1, 1, None, None, None)
    assert rc == 1 and "out of range" in capi.last_error()
    rc = lib.cgt_amd_conv_patch_bwd_filter_f32(None, None, 2, 3, 9, 9, 8, 3, 3, 1, 1, 1, 1, None, None)
    assert rc == 1 and "null" in capi.last_error()
    # empty batches and empty filter banks are not errors and launch nothing
    assert lib.cgt_amd_conv_patch_fwd_f32(None, None, None, 0, 0, 3, 9, 9, 8, 3, 3, 1, 1, 1, 1, None, None, None) == 0
    assert lib.cgt_amd_conv_col_fwd_f32(None, None, None, 0, 0, 49, 27, 8, None, None, None) == 0
    assert lib.cgt_amd_conv_col_bwd_data_f32(None, None, 0, 49, 27, 8, None, None) == 0
    rc = lib.cgt_amd_conv_col_fwd_f32(None, None, None, 0, 2, 49, 27, 8, None, None, None)
    assert rc == 1 and "null" in capi.last_error()
    rc = lib.cgt_amd_conv_col_bwd_filter_f32(None, None, 2, 49, 27, 8, None, None)
    assert rc == 1 and "null" in capi.last_error()
    rc = lib.cgt_amd_conv_col_fwd_f32(None, None, None, 0, -1, 49, 27, 8, None, None, None)
    assert rc == 1 and "negative" in capi.last_error()
