"""Every entry point takes the stream it launches on.  These tests run a small Linear training fragment (fused
bias + ReLU GEMM with a split reduction, GEMMs on transposed views, elementwise kernels, a two-stage sum, conv2d
forward and backward, max pooling forward and backward) on a stream of their own and then inside a HIP graph captured from that stream, and compare every replay
with the eager result on the same inputs.  The graph is replayed several times with eager work, host copies and
synchronisation in between: the library only records kernels (its zero fill is a kernel, not a memset node), takes
its scratch from per-stream buffers that the warm-up run has grown, and allocates nothing while capturing.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def fragment(tt, be, x, w1, b1, w2, target, img, filt):
    """Forward of Linear-ReLU-Linear with a squared-error sum, the two weight gradients' GEMMs, and a conv2d with ReLU
    and max pooling, forward and backward."""
    h = be.batched_matmul(x, w1, bias=b1, bias_mode=1, relu=True)  # 256x512x256: split reduction + fused epilogue
    y = be.batched_matmul(h, w2)
    d = be.binary(y, target, "sub")
    loss = be.sum(be.binary(d, d, "mul"))
    gw2 = be.batched_matmul(h.permute(0, 2, 1), d)   # A^T . B on a view
    gh = be.batched_matmul(d, w2.permute(0, 2, 1))   # A . B^T on a view
    c = be.conv2d(img, filt, None, 1, 1)
    a = c.relu()
    pooled = tt.max_pool2d(a, 2, 2, 0)
    ga = tt.pool2d_backward(pooled, a, pooled, "max", 2, 2, 0)
    gimg, gfilt, _ = be.conv2d_backward(ga, img, filt, None, 1, 1)  # workspace from the allocator's cache, no wait
    return [h, y, loss, gw2, gh, c, pooled, ga, gimg, gfilt]


def make_inputs(tt, seed):
    rng = np.random.default_rng(seed)
    f = np.float32
    host = dict(x=rng.uniform(-1, 1, (1, 256, 512)).astype(f), w1=rng.uniform(-0.1, 0.1, (1, 512, 256)).astype(f),
                b1=rng.uniform(-1, 1, (256,)).astype(f), w2=rng.uniform(-0.1, 0.1, (1, 256, 64)).astype(f),
                target=rng.uniform(-1, 1, (1, 256, 64)).astype(f), img=rng.normal(0, 1, (4, 8, 12, 12)).astype(f),
                filt=rng.normal(0, 0.2, (16, 8, 3, 3)).astype(f))
    return host


def test_launches_follow_the_stream_argument(tt):
    be = tt.get_backend(tt.kAMD)
    stream = tt.graph.Stream()
    try:
        host = make_inputs(tt, 0)
        dev = {k: tt.Tensor.from_numpy(v) for k, v in host.items()}
        want = [t.to_numpy() for t in fragment(tt, be, **dev)]  # default stream
        got = stream.run(lambda: fragment(tt, be, **dev))
        stream.synchronize()
        for g, w in zip(got, want):
            assert np.array_equal(g.to_numpy(), w)  # same kernels, same inputs: identical bits
        # a value check of the chain itself, so that "equal" cannot mean "equally wrong"
        h = np.maximum(host["x"][0].astype(np.float64) @ host["w1"][0] + host["b1"], 0)
        y = h @ host["w2"][0]
        assert np.allclose(want[1][0], y, rtol=1e-4, atol=1e-4)
        assert np.isclose(float(want[2].reshape(-1)[0]), float(((y - host["target"][0]) ** 2).sum()), rtol=1e-4)
    finally:
        stream.close()


def test_captured_graph_replays_match_eager(tt):
    be = tt.get_backend(tt.kAMD)
    stream = tt.graph.Stream()
    graph = None
    try:
        host = make_inputs(tt, 1)
        dev = {k: tt.Tensor.from_numpy(v) for k, v in host.items()}
        graph = tt.graph.Graph(stream, lambda: fragment(tt, be, **dev))  # warms up on the stream, then captures
        assert graph.num_nodes() >= 8, f"expected the fragment's kernels as graph nodes, got {graph.num_nodes()}"
        first = None
        for replay in range(4):
            fresh = make_inputs(tt, 100 + replay)
            for k in ("x", "target", "img"):  # new inputs into the captured buffers (blocking copies)
                graph.copy_in(dev[k], fresh[k])
            graph.launch()
            stream.synchronize()
            got = [t.to_numpy() for t in graph.outputs]
            # eager on the default stream with the same inputs (also the "work between replays")
            eager = [t.to_numpy() for t in fragment(tt, be, **dev)]
            for i, (g, w) in enumerate(zip(got, eager)):
                assert np.array_equal(g, w), f"replay {replay}: output {i} differs from the eager result"
            be.synchronize(0)
            first = got if first is None else first
        assert not np.array_equal(first[1], got[1])  # the replays really ran on different inputs
    finally:
        if graph is not None:
            graph.close()
        stream.close()
