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
    h = be.batched_matmul(x, w1, bias=b1, bias_mode=1, relu=True)  # 320x512x416: split reduction + fused epilogue
    y = be.batched_matmul(h, w2)                     # 320x416x64: the kernel for small outputs
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
    host = dict(x=rng.uniform(-1, 1, (1, 320, 512)).astype(f), w1=rng.uniform(-0.1, 0.1, (1, 512, 416)).astype(f),
                b1=rng.uniform(-1, 1, (416,)).astype(f), w2=rng.uniform(-0.1, 0.1, (1, 416, 64)).astype(f),
                target=rng.uniform(-1, 1, (1, 320, 64)).astype(f), img=rng.normal(0, 1, (4, 8, 12, 12)).astype(f),
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


def test_blocks_allocated_between_replays_are_not_overwritten(tt):
    """Temporaries of the captured function are freed when it returns; their blocks must stay the graph's own, or a
    tensor allocated afterwards in the same size class would be overwritten by the next replay."""
    be = tt.get_backend(tt.kAMD)
    stream = tt.graph.Stream()
    graph = None
    try:
        host = make_inputs(tt, 2)
        dev = {k: tt.Tensor.from_numpy(v) for k, v in host.items()}
        graph = tt.graph.Graph(stream, lambda: fragment(tt, be, **dev))
        graph.launch()
        stream.synchronize()
        first = [t.to_numpy() for t in graph.outputs]
        # fresh tensors in the size classes of the fragment's temporaries and results (d, a, the conv workspace, ...)
        rng = np.random.default_rng(7)
        guards = []
        for shape in ((1, 256, 64), (4, 16, 12, 12), (1, 256, 256), (4, 16, 6, 6), (16, 8, 3, 3), (4, 8, 12, 12), (1, 64, 256)) * 3:
            h = rng.normal(0, 1, shape).astype(np.float32)
            guards.append((h, tt.Tensor.from_numpy(h)))
        for _ in range(2):
            graph.launch()
            stream.synchronize()
        for h, t in guards:
            assert np.array_equal(t.to_numpy(), h)
        for g, w in zip(graph.outputs, first):
            assert np.array_equal(g.to_numpy(), w)
    finally:
        if graph is not None:
            graph.close()
        stream.close()


def test_scratch_growth_after_a_capture_keeps_the_recorded_buffer(tt):
    """A captured split-k product has its scratch address recorded; a later, larger split-k product on the same stream
    grows the scratch.  The outgrown buffer must stay valid for the replays."""
    be = tt.get_backend(tt.kAMD)
    stream = tt.graph.Stream()
    graph = None
    try:
        rng = np.random.default_rng(3)
        a = tt.Tensor.from_numpy(rng.integers(-3, 4, (1, 320, 512)).astype(np.float32))
        b = tt.Tensor.from_numpy(rng.integers(-3, 4, (1, 512, 416)).astype(np.float32))
        assert "splitk" in be.batched_matmul_variant(a, b)
        graph = tt.graph.Graph(stream, lambda: [be.batched_matmul(a, b)])
        graph.launch()
        stream.synchronize()
        want = graph.outputs[0].to_numpy()
        assert np.array_equal(want[0], (a.to_numpy()[0].astype(np.float64) @ b.to_numpy()[0]).astype(np.float32))
        # 3 x 320 x 1024 x 384 splits three ways: 4.2 MiB of partial tiles, more than the stream's first 4 MiB buffer
        big_a = tt.Tensor.from_numpy(rng.integers(-3, 4, (3, 320, 1024)).astype(np.float32))
        big_b = tt.Tensor.from_numpy(rng.integers(-3, 4, (3, 1024, 384)).astype(np.float32))
        assert "splitk3" in be.batched_matmul_variant(big_a, big_b)
        big = stream.run(lambda: be.batched_matmul(big_a, big_b))
        stream.synchronize()
        assert np.array_equal(big.to_numpy(), np.matmul(big_a.to_numpy().astype(np.float64), big_b.to_numpy()).astype(np.float32))
        for _ in range(2):
            graph.launch()
            stream.synchronize()
            assert np.array_equal(graph.outputs[0].to_numpy(), want)
    finally:
        if graph is not None:
            graph.close()
        stream.close()


def test_block_freed_on_one_stream_is_not_reused_on_another_while_in_flight(tt):
    """A tensor is released right after work that reads it has been enqueued on a (non-blocking) stream; an allocation
    of the same size for the default stream, made while that work is still running, must not receive its block."""
    be = tt.get_backend(tt.kAMD)
    assert tt._capi.lib.ttamd_empty_cache(0) == 0  # so that the block released below is the only cached one of its size
    stream = tt.graph.Stream(non_blocking=True)
    try:
        n = 2048
        rng = np.random.default_rng(4)
        a_h = rng.integers(-2, 3, (1, n, n)).astype(np.float32)
        b_h = rng.integers(-2, 3, (1, n, n)).astype(np.float32)
        b = tt.Tensor.from_numpy(b_h)
        outs = [tt.Tensor.empty((1, n, n), tt._capi.F32) for _ in range(4)]
        want = (a_h[0].astype(np.float64) @ b_h[0]).astype(np.float32)  # small integers: exact in any order
        be.synchronize(0)

        def enqueue():
            a = tt.Tensor.from_numpy(a_h)          # allocated for `stream` (the upload itself is a blocking copy)
            for _ in range(60):                    # tens of milliseconds of GEMMs that read `a`
                for o in outs:
                    be.batched_matmul(a, b, out=o)
            return a.storage.ptr                   # `a` is released here, with the work still queued

        freed_ptr = stream.run(enqueue)
        # default stream, same size class, while the GEMMs run: other data
        other_h = np.full((1, n, n), 7.0, np.float32)
        other = tt.Tensor.from_numpy(other_h)
        in_flight_reuse = other.storage.ptr == freed_ptr
        still_busy = not stream.is_idle()          # asked AFTER the allocation: the GEMMs were running when it was served
        stream.synchronize()
        for o in outs:
            assert np.array_equal(o.to_numpy()[0], want)
        assert np.array_equal(other.to_numpy(), other_h)
        if still_busy:                             # (on a box that drained the queue already, reuse would be legitimate)
            assert not in_flight_reuse
        # once the stream is idle the block serves any stream again (which request gets it is the cache's business)
        again = tt.Tensor.from_numpy(other_h)
        assert np.array_equal(again.to_numpy(), other_h)
    finally:
        stream.close()


def test_blocks_of_a_closed_stream_serve_later_requests(tt):
    """Blocks allocated and freed for a stream stay in the cache under its handle; once the stream has been closed
    (Stream.close releases the handle first) a request for another stream takes such a block without touching the
    stream that no longer exists, and a block that outlives its allocation stream is freed and reused as well."""
    assert tt._capi.lib.ttamd_empty_cache(0) == 0
    stream = tt.graph.Stream()
    kept = stream.run(lambda: tt.Tensor.from_numpy(np.arange(3000, dtype=np.float32)))      # outlives the stream
    freed_ptr = stream.run(lambda: tt.Tensor.from_numpy(np.ones(5000, np.float32)).storage.ptr)  # freed for the stream
    stream.close()
    again = tt.Tensor.from_numpy(np.full(5000, 2.0, np.float32))  # default stream, the cached block's size class
    assert again.storage.ptr == freed_ptr
    assert np.array_equal(again.to_numpy(), np.full(5000, 2.0, np.float32))
    assert np.array_equal(kept.to_numpy(), np.arange(3000, dtype=np.float32))
    del kept                                                       # freed for the default stream, allocated for the closed one
    other = tt.graph.Stream()
    try:
        # (whether this request gets that block depends on whether the event it records on the default stream has
        # already completed; either way it must not touch the closed stream)
        reuse = other.run(lambda: tt.Tensor.from_numpy(np.full(3000, 5.0, np.float32)))
        other.synchronize()
        assert np.array_equal(reuse.to_numpy(), np.full(3000, 5.0, np.float32))
        del reuse
        assert tt._capi.lib.ttamd_device_synchronize(0) == 0
    finally:
        other.close()


def test_scalar_operands_are_filled_once(tt):
    """A scalar operand of an element-wise call is a stride-0 view of a one-element tensor that is kept per value: the
    recorded graph of a function that has run before holds no fill kernels, 0.0 and -0.0 are different constants, and
    full() still hands out storage of its own."""
    x = tt.Tensor.from_numpy(np.array([[-1.5, 2.0, 0.0, 3.0]], np.float32))
    stream = tt.graph.Stream()
    graph = None
    try:
        graph = tt.graph.Graph(stream, lambda: [x * 2.0, tt.where(x < 0.0, 0.0, 1.0), x * 2.0])
        assert graph.num_nodes() == 4   # mul, lt, where, mul: no fills
        graph.launch()
        stream.synchronize()
        assert np.array_equal(graph.outputs[0].to_numpy(), x.to_numpy() * 2)
        assert np.array_equal(graph.outputs[1].to_numpy(), np.where(x.to_numpy() < 0, 0, 1).astype(np.float32))
        assert np.array_equal(graph.outputs[2].to_numpy(), x.to_numpy() * 2)
    finally:
        if graph is not None:
            graph.close()
        stream.close()
    pos, neg = (x * 0.0).to_numpy(), (x * -0.0).to_numpy()
    assert np.array_equal(np.signbit(pos), np.signbit(x.to_numpy() * np.float32(0.0)))
    assert np.array_equal(np.signbit(neg), np.signbit(x.to_numpy() * np.float32(-0.0)))
    a, b = tt.full((2, 2), 7.0), tt.full((2, 2), 7.0)
    assert a.storage is not b.storage and np.array_equal(a.to_numpy(), np.full((2, 2), 7, np.float32))
    ints = tt.Tensor.from_numpy(np.arange(6, dtype=np.int32))
    assert np.array_equal((ints * 3).to_numpy(), np.arange(6) * 3) and np.array_equal((ints * 3).to_numpy(), np.arange(6) * 3)

