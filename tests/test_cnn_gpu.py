"""One training step of the network of the reference's examples/mnist_cnn_example.cpp:31-63 on the GPU, op by op
through the Python mirror (conv1 1->32 k3, ReLU, conv2 32->64 k3, ReLU, max_pool2d(2, 2, 0), flatten, Linear
9216->128, ReLU, Linear 128->10; dropout left out, a squared-error sum as the loss), with the backward pass written
out as the reference's autograd would run it (conv2d_backward, pool backward, ReLU mask `x < 0 -> 0 else 1`,
dA = dC.B^T / dB = A^T.dC), against the same step over the CPU oracle.

fp64 on small-integer data: every intermediate up to the pooling backward is an integer below 2^53, so both sides are
exact there and must be bit-identical (ReLU masks and pooling ties included); behind the pooling backward (which
divides among ties) the fp64 tolerance of the path applies.  An fp32 run on real-valued data checks the forward output
within the path's tolerance.
"""
import numpy as np
import pytest

from helpers import max_rel_error

pytestmark = pytest.mark.gpu


def make_net(rng, dtype, integer):
    def draw(*shape, scale=1.0):
        if integer:
            return rng.integers(-1, 2, shape).astype(dtype)
        return (rng.normal(0, scale, shape)).astype(dtype)
    return dict(w1=draw(32, 1, 3, 3, scale=0.3), b1=draw(32, scale=0.1), w2=draw(64, 32, 3, 3, scale=0.06), b2=draw(64, scale=0.1),
                W3=draw(9216, 128, scale=0.01), b3=draw(128, scale=0.1), W4=draw(128, 10, scale=0.09), b4=draw(10, scale=0.1))


def cpu_step(oracle, x, t, p, backward=True):
    z1 = oracle.conv2d_forward(x, p["w1"], p["b1"], 1, 0)
    a1 = np.maximum(z1, 0)
    z2 = oracle.conv2d_forward(a1, p["w2"], p["b2"], 1, 0)
    a2 = np.maximum(z2, 0)
    pooled = oracle.pool2d_forward(a2, "max", 2, 2, 0)
    flat = pooled.reshape(pooled.shape[0], -1)
    z3 = oracle.matmul(flat, p["W3"]) + p["b3"]
    a3 = np.maximum(z3, 0)
    y = oracle.matmul(a3, p["W4"]) + p["b4"]
    out = {"y": y}
    if not backward:
        return out
    gy = 2 * (y - t)
    out["loss"] = np.sum((y - t) ** 2)
    out["db4"] = gy.sum(0)
    da3, out["dW4"] = (v[0] for v in oracle.matmul_backward(a3[None], p["W4"][None], gy[None]))
    dz3 = da3 * np.where(z3 < 0, 0, 1).astype(x.dtype)
    out["db3"] = dz3.sum(0)
    dflat, out["dW3"] = (v[0] for v in oracle.matmul_backward(flat[None], p["W3"][None], dz3[None]))
    da2 = oracle.pool2d_backward(np.ascontiguousarray(dflat.reshape(pooled.shape)), a2, pooled, "max", 2, 2, 0)
    dz2 = da2 * np.where(z2 < 0, 0, 1).astype(x.dtype)
    da1, out["dw2"], out["db2"] = oracle.conv2d_backward(dz2, a1, p["w2"], True, 1, 0)
    dz1 = da1 * np.where(z1 < 0, 0, 1).astype(x.dtype)
    out["dx"], out["dw1"], out["db1"] = oracle.conv2d_backward(dz1, x, p["w1"], True, 1, 0)
    return out


def relu_mask(tt, z):
    """where(z < 0, 0, 1) in z's dtype (autograd/unary_ops.cpp:568-573)."""
    return tt.where(z < 0.0, tt.full(z.shape, 0.0, z.dtype), tt.full(z.shape, 1.0, z.dtype))


def gpu_step(tt, x, t, p, backward=True):
    d = {k: tt.Tensor.from_numpy(v) for k, v in p.items()}
    tx, tt_ = tt.Tensor.from_numpy(x), tt.Tensor.from_numpy(t)
    z1 = tt.conv2d(tx, d["w1"], d["b1"], 1, 0)
    a1 = z1.relu()
    z2 = tt.conv2d(a1, d["w2"], d["b2"], 1, 0)
    a2 = z2.relu()
    pooled = tt.max_pool2d(a2, 2, 2, 0)
    flat = pooled.flatten(1)
    z3 = tt.linear(flat, d["W3"], d["b3"])
    a3 = z3.relu()
    y = tt.linear(a3, d["W4"], d["b4"])
    out = {"y": y.to_numpy()}
    if not backward:
        return out
    diff = y - tt_
    out["loss"] = (diff * diff).sum().to_numpy().reshape(-1)[0]
    gy = diff * 2.0
    out["db4"] = gy.sum(0).to_numpy()
    da3, dW4 = tt.matmul_backward(a3.unsqueeze(0), d["W4"].unsqueeze(0), gy.unsqueeze(0))
    out["dW4"] = dW4.to_numpy()[0]
    dz3 = da3.squeeze(0) * relu_mask(tt, z3)
    out["db3"] = dz3.sum(0).to_numpy()
    dflat, dW3 = tt.matmul_backward(flat.unsqueeze(0), d["W3"].unsqueeze(0), dz3.unsqueeze(0))
    out["dW3"] = dW3.to_numpy()[0]
    da2 = tt.pool2d_backward(dflat.squeeze(0).reshape(list(pooled.shape)), a2, pooled, "max", 2, 2, 0)
    dz2 = da2 * relu_mask(tt, z2)
    da1, dw2, db2 = tt.conv2d_backward(dz2, a1, d["w2"], d["b2"], 1, 0)
    out["dw2"], out["db2"] = dw2.to_numpy(), db2.to_numpy()
    dz1 = da1 * relu_mask(tt, z1)
    dx, dw1, db1 = tt.conv2d_backward(dz1, tx, d["w1"], d["b1"], 1, 0)
    out["dx"], out["dw1"], out["db1"] = dx.to_numpy(), dw1.to_numpy(), db1.to_numpy()
    return out


def test_mnist_cnn_training_step_exact_in_fp64(tt, oracle):
    rng = np.random.default_rng(7)
    x = rng.integers(0, 3, (6, 1, 28, 28)).astype(np.float64)
    t = rng.integers(-5, 6, (6, 10)).astype(np.float64)
    p = make_net(rng, np.float64, integer=True)
    want = cpu_step(oracle, x, t, p)
    got = gpu_step(tt, x, t, p)
    assert np.abs(want["dw1"]).max() < 2.0 ** 53 and np.abs(want["y"]).max() > 0  # exact range, non-trivial values
    for key in ("y", "db4", "dW4", "db3", "dW3"):
        assert got[key].shape == want[key].shape, key
        assert np.array_equal(got[key], want[key]), key
    assert float(got["loss"]) == float(want["loss"])
    # max-pool backward divides a gradient among tied window elements (thirds appear), so what lies behind it is no
    # longer integer-valued: the fp64 tolerance of the path applies there
    for key in ("dw2", "db2", "dx", "dw1", "db1"):
        assert got[key].shape == want[key].shape, key
        assert max_rel_error(got[key], want[key]) <= 1e-12, key


def test_mnist_cnn_forward_fp32(tt, oracle):
    rng = np.random.default_rng(8)
    x = rng.uniform(0, 1, (16, 1, 28, 28)).astype(np.float32)
    p = make_net(rng, np.float32, integer=False)
    want = cpu_step(oracle, x, None, p, backward=False)["y"]
    got = gpu_step(tt, x, np.zeros((16, 10), np.float32), p, backward=False)["y"]
    assert got.shape == want.shape == (16, 10)
    assert max_rel_error(got, want) <= 1e-4
