"""Seeded random layer graphs through the Op API: what nn builds by default (the fused
convolution families, the pool pullback written into the padded cotangent, LRN without a
stored scale) against the reference's literal composition (cgt/nn.py:87-100: im2col ->
Mul22 -> transpose, separate bias / rectify / pool / LRN ops), and one compiled function
replayed at other batch and image sizes against fresh node-by-node evaluation.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cgt():
    import cgt_amd
    from cgt_amd import capi
    capi.require_gpu()
    return cgt_amd


def relfro(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def same_bits(a, b):
    a, b = np.asarray(a), np.asarray(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def random_layer(rs, family):
    """A conv layer geometry of the family nn.conv2d picks an op for."""
    if family == "same":        # stride 1, same padding, channel counts in multiples of 16
        C, L = 16 * rs.randint(1, 4), 16 * rs.randint(1, 5)
        k = (2 * rs.randint(0, 3) + 1, 2 * rs.randint(0, 3) + 1)
        pad, stride = ((k[0] - 1) // 2, (k[1] - 1) // 2), (1, 1)
    elif family == "patch":     # few input channels: patches gathered inside the product
        C, L = rs.randint(1, 8), rs.randint(1, 70)
        k = (rs.randint(1, 8), rs.randint(1, 8))
        pad, stride = (rs.randint(0, 3), rs.randint(0, 3)), (rs.randint(1, 4), rs.randint(1, 4))
    else:                       # products over the column buffer
        C, L = rs.randint(17, 40), rs.randint(1, 70)
        k = (rs.randint(1, 6), rs.randint(1, 6))
        pad, stride = (rs.randint(0, 3), rs.randint(0, 3)), (2, rs.randint(1, 3))
    return dict(C=int(C), L=int(L), k=k, pad=pad, stride=stride,
                bias=bool(rs.rand() < 0.5), relu=bool(rs.rand() < 0.6), lrn=bool(rs.rand() < 0.4 and L >= 5),
                pool=[None, ((2, 2), (0, 0), (2, 2)), ((3, 3), (0, 0), (2, 2)), ((3, 3), (1, 1), (1, 1))][rs.randint(4)])


def random_size(rs, spec, hi):
    """(H, W) that leave the convolution at least 4 x 4 outputs (every pool has something to do)."""
    lo = [k + 3 * s for k, s in zip(spec["k"], spec["stride"])]
    return int(rs.randint(lo[0], lo[0] + hi)), int(rs.randint(lo[1], lo[1] + hi))


def build(cgt, spec, x, w, b):
    from cgt_amd import nn
    xn, wn, bn = cgt.constant(x), cgt.constant(w), cgt.constant(b)
    h = nn.conv2d(xn, wn, spec["k"], spec["pad"], spec["stride"])
    if spec["bias"]:
        h = cgt.broadcast("+", h, bn, "xxxx,1x11")
    if spec["relu"]:
        h = nn.rectify(h)
    if spec["lrn"]:
        h = nn.cross_channel_lrn(h, 5, 1e-2, 0.75)
    if spec["pool"]:
        h = nn.max_pool_2d(h, *spec["pool"])
    loss = cgt.sum(h * h)
    return xn, [h, loss] + list(cgt.grad(loss, [xn, wn] + ([bn] if spec["bias"] else [])))


CASES = [(family, seed) for family in ("same", "patch", "col") for seed in range(6)]


@pytest.mark.parametrize("family,seed", CASES)
def test_fused_graph_agrees_with_the_literal_composition(cgt, family, seed):
    from cgt_amd import nn
    rs = np.random.RandomState(100 * seed + len(family))
    spec = random_layer(rs, family)
    H, W = random_size(rs, spec, 28)
    B = rs.randint(1, 6)
    print(family, seed, spec, (B, H, W), flush=True)
    # dyadic inputs: every product and sum of the forward convolution is exact in fp32, so both graphs
    # pool the same bits (a maximum between two nearly equal activations would otherwise flip with the
    # forward product's rounding, which moves the gradient discretely)
    x = (np.round(rs.randn(B, spec["C"], H, W) * 4) / 4).astype(np.float32)
    w = (np.round(rs.randn(spec["L"], spec["C"], *spec["k"]) * 8) / 64).astype(np.float32)
    b = (np.round(rs.randn(1, spec["L"], 1, 1) * 8) / 8).astype(np.float32)
    _, fused = build(cgt, spec, x, w, b)
    old_algo, old_fusion = nn.conv_algo("im2col"), nn.conv_fusion(False)
    try:
        _, literal = build(cgt, spec, x, w, b)
    finally:
        nn.conv_algo(old_algo)
        nn.conv_fusion(old_fusion)
    names = ["output", "loss", "grad x", "grad w", "grad b"]
    for name, a, u in zip(names, fused, literal):
        assert relfro(a.get(), u.get()) <= 2e-5, name
    if not spec["lrn"]:
        assert same_bits(fused[0].get(), literal[0].get())     # exact products: the fused epilogues change no bit


@pytest.mark.parametrize("family,seed", CASES[::2])
def test_compiled_function_at_other_batch_and_image_sizes(cgt, family, seed):
    rs = np.random.RandomState(1000 + 100 * seed + len(family))
    spec = random_layer(rs, family)
    sizes = [(int(rs.randint(1, 5)),) + random_size(rs, spec, 24) for _ in range(3)]
    print(family, seed, spec, sizes, flush=True)
    w = (rs.randn(spec["L"], spec["C"], *spec["k"]) / np.sqrt(spec["C"] * spec["k"][0] * spec["k"][1])).astype(np.float32)
    b = (0.1 * rs.randn(1, spec["L"], 1, 1)).astype(np.float32)
    B, H, W = sizes[0]
    xn, outs = build(cgt, spec, rs.randn(B, spec["C"], H, W).astype(np.float32), w, b)
    f = cgt.function([xn], outs)
    for B, H, W in sizes[1:] + sizes[:1]:
        x = rs.randn(B, spec["C"], H, W).astype(np.float32)
        got = f(x)
        want = [o.get() for o in build(cgt, spec, x, w, b)[1]]
        for a, u in zip(got, want):
            assert same_bits(a, u), (B, H, W)
