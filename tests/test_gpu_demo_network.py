"""The reference's convolutional example as a caller of the whole path.

examples/demo_cifar.py:30-57 builds conv 5x5 -> rectify -> pool 3x3/2 (twice), conv 5x5 -> pool -> rectify,
flatten, Affine, logsoftmax, the mean negative log-likelihood, and trains it with the RMSProp updates of
demo_cifar.py:7-17 through one cgt.function(inputs, [loss], updates=...).  Here the same network is built
with cgt_amd on synthetic CIFAR-shaped batches and trained for a few steps; every loss and every
parameter afterwards is compared with the same steps in float64 (torch autograd on the CPU).  The
label gather `logprobs[arange(B), y]` is written as a product with the one-hot labels (the same
numbers; integer indexing is outside the path).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
F = torch.nn.functional


@pytest.fixture(scope="module")
def cgt():
    import cgt_amd
    from cgt_amd import capi
    capi.require_gpu()
    return cgt_amd


def init(rs):
    # demo_cifar.py:37-47: IIDGaussian(1e-4) for the first layer, 0.01 for the others, zero biases;
    # the example leaves the Affine weights at zero, which keeps every gradient below it at zero on the
    # first step -- a small random matrix here, so that all layers learn from step one
    return {
        "w1": (1e-4 * rs.randn(32, 3, 5, 5)).astype(np.float32), "b1": np.zeros((1, 32, 1, 1), np.float32),
        "w2": (0.01 * rs.randn(32, 32, 5, 5)).astype(np.float32), "b2": np.zeros((1, 32, 1, 1), np.float32),
        "w3": (0.01 * rs.randn(64, 32, 5, 5)).astype(np.float32), "b3": np.zeros((1, 64, 1, 1), np.float32),
        "wo": (0.01 * rs.randn(256, 10)).astype(np.float32), "bo": np.zeros((1, 10), np.float32),
    }


def torch_steps(params, batches, stepsize, rho, eps, want_grads=False):
    p = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in params.items()}
    acc = {k: torch.zeros_like(v) for k, v in p.items()}
    losses = []

    def pool(h):
        # CGT keeps ceil((H - k) / s) windows per axis, one fewer than the Caffe rule its comment
        # quotes (cgt/nn_ops/max_pool_2d.py:36-41): 32 -> 15 -> 6 -> 2
        n = -(-(h.shape[2] - 3) // 2)
        return F.max_pool2d(h, 3, 2, ceil_mode=True)[:, :, :n, :n]

    for x, onehot in batches:
        x, onehot = torch.tensor(x, dtype=torch.float64), torch.tensor(onehot, dtype=torch.float64)
        h = pool(F.relu(F.conv2d(x, p["w1"], padding=2) + p["b1"]))
        h = pool(F.relu(F.conv2d(h, p["w2"], padding=2) + p["b2"]))
        h = F.relu(pool(F.conv2d(h, p["w3"], padding=2) + p["b3"]))
        logits = h.reshape(h.shape[0], -1) @ p["wo"] + p["bo"]
        e = torch.exp(logits)
        logprobs = torch.log(e / e.sum(1, keepdim=True))
        loss = -(logprobs * onehot).sum() / x.shape[0]
        grads = torch.autograd.grad(loss, [p[k] for k in sorted(p)])
        losses.append(float(loss.detach()))
        if want_grads:
            return losses, {k: g.numpy() for k, g in zip(sorted(p), grads)}
        with torch.no_grad():
            for k, g in zip(sorted(p), grads):
                acc[k] = rho * acc[k] + (1 - rho) * g * g
                p[k] -= stepsize * g / torch.sqrt(acc[k] + eps)
    return losses, {k: v.detach().numpy() for k, v in p.items()}


def test_the_reference_cifar_example_trains_as_in_float64(cgt):
    from cgt_amd import nn
    rs = np.random.RandomState(0)
    params = init(rs)
    stepsize, rho, eps = 1e-3, 0.9, 1e-6
    sizes = [16, 16, 16, 8, 24]              # one compiled function, three batch sizes
    batches = []
    for B in sizes:
        x = rs.rand(B, 3, 32, 32).astype(np.float32)
        y = rs.randint(0, 10, B)
        batches.append((x, np.eye(10, dtype=np.float32)[y]))

    X, Y = cgt.constant(batches[0][0]), cgt.constant(batches[0][1])
    conv1 = nn.SpatialConvolution(3, 32, (5, 5), (2, 2), weight_init=params["w1"], bias_init=params["b1"])
    conv2 = nn.SpatialConvolution(32, 32, (5, 5), (2, 2), weight_init=params["w2"], bias_init=params["b2"])
    conv3 = nn.SpatialConvolution(32, 64, (5, 5), (2, 2), weight_init=params["w3"], bias_init=params["b3"])
    ip1 = nn.Affine(256, 10, weight_init=params["wo"], bias_init=params["bo"])
    pool1 = nn.max_pool_2d(nn.rectify(conv1(X)), (3, 3), (0, 0), (2, 2))
    pool2 = nn.max_pool_2d(nn.rectify(conv2(pool1)), (3, 3), (0, 0), (2, 2))
    relu3 = nn.rectify(nn.max_pool_2d(conv3(pool2), (3, 3), (0, 0), (2, 2)))
    d0, d1, d2, d3 = relu3.shape
    assert (d1, d2, d3) == (64, 2, 2)
    logprobs = nn.logsoftmax(ip1(relu3.reshape([d0, d1 * d2 * d3])))
    loss = -(cgt.sum(logprobs * Y) / cgt.size(X, 0))
    nodes = {"w1": conv1.weight, "b1": conv1.bias, "w2": conv2.weight, "b2": conv2.bias,
             "w3": conv3.weight, "b3": conv3.bias, "wo": ip1.weight, "bo": ip1.bias}
    names = sorted(nodes)
    grads = cgt.grad(loss, [nodes[k] for k in names])
    updates = []
    for k, g in zip(names, grads):          # demo_cifar.py:7-17
        acc = cgt.constant(np.zeros_like(params[k]))
        acc_new = acc * rho + cgt.square(g) * (1 - rho)
        updates.append((acc, acc_new))
        updates.append((nodes[k], nodes[k] - g / cgt.sqrt(acc_new + eps) * stepsize))
    train = cgt.function([X, Y], [loss], updates=updates)

    # gradients at the initial parameters, node by node, before any update
    _, g0 = torch_steps(params, batches[:1], stepsize, rho, eps, want_grads=True)
    for k, g in zip(names, grads):
        err = np.linalg.norm(g.get().astype(np.float64) - g0[k]) / np.linalg.norm(g0[k])
        # w1 sits under the first pool: where two cells of a window agree to the last bits of the fp32
        # convolution, float64 picks the other one, the cotangent lands one pixel aside (the bias
        # gradient, a plain sum, does not notice) and that one term moves the filter gradient by ~1e-3
        assert err <= (5e-3 if k == "w1" else 1e-5), (k, err)

    losses = [float(train(x, onehot)[0]) for x, onehot in batches]
    want_losses, want = torch_steps(params, batches, stepsize, rho, eps)
    assert np.allclose(losses, want_losses, rtol=1e-5), (losses, want_losses)
    assert abs(want_losses[0] - np.log(10)) < 0.05 and min(losses) < losses[0]
    for k in names:
        # RMSProp divides by sqrt(acc + 1e-6): steps of gradients far below 1e-3 keep their relative
        # error, but five of them largely cancel, so the net displacement is compared by direction
        # and loosely by length
        got, moved = nodes[k].get().astype(np.float64) - params[k], want[k] - params[k]
        cos = (got * moved).sum() / (np.linalg.norm(got) * np.linalg.norm(moved))
        assert cos >= 0.97 and np.linalg.norm(got - moved) <= 0.3 * np.linalg.norm(moved), (k, cos)
