"""The hot path recorded into a HIP graph and replayed: callers that keep a training or serving loop
in a captured graph need every entry point on the path to enqueue kernels only (no allocation, no
memset node, no synchronisation once the library's workspace has grown to its size).  Each case runs
its call sequence eagerly, records the same sequence on a capture stream, and replays the graph
several times with eager work and synchronisations of its own between the replays; every replay must
reproduce the eager results bit for bit (all kernels on the path are deterministic)."""
import numpy as np
import pytest

from gpu_util import driver, dev, empty, host, tuning

pytestmark = pytest.mark.gpu
RM, N_, T_ = 101, 111, 112


def _record(fn):
    """fn() eagerly on a side stream (default priority) as warm-up, then once more under capture."""
    import torch
    drv = driver()
    main = torch.cuda.current_stream()
    side = torch.cuda.Stream()
    side.wait_stream(main)
    graph = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.stream(side):
            drv.set_stream(side.cuda_stream)
            fn()   # the workspace, the arrival counters and the LDS grants reach their final size here
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                fn()
    finally:
        drv.set_stream(main.cuda_stream)
    torch.cuda.synchronize()
    return graph


def _check_replays(graph, outputs, eager_work, replays=3):
    """outputs: tensors the sequence writes.  Their eager values are taken first; before each replay
    they are poisoned so that a replay that skipped a kernel is noticed."""
    import torch
    want = [host(t).copy() for t in outputs]
    for r in range(replays):
        for t in outputs:
            t.fill_(float("nan") if t.dtype.is_floating_point else -7)
        eager_work()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (t, w) in enumerate(zip(outputs, want)):
            np.testing.assert_array_equal(host(t), w, err_msg="replay %d, output %d" % (r, i))


def test_lowering_path_in_a_graph():
    """lower_cube, the three GEMMs (the weight gradient split over the contraction, with its reduction),
    remap, forward bias, and inverse_lower_cube fused with the split bias-gradient reduction (arrival
    counters, partial sums in the library's workspace)."""
    from caffecontroll_amd.driver import conv_pmap, remap_pmap, lift_args
    drv = driver()
    rng = np.random.default_rng(71)
    b, d, n, k, s, p, o = 32, 16, 27, 5, 1, 2, 32
    m = (n + 2 * p - k) // s + 1
    kkd, bmm = k * k * d, b * m * m
    x = dev(rng.standard_normal((b, d, n, n)).astype(np.float32))
    w = dev((rng.standard_normal((o, kkd)) * 0.1).astype(np.float32))
    bias = dev(rng.standard_normal(o).astype(np.float32))
    og = dev(rng.standard_normal((b, o, m, m)).astype(np.float32))
    lowered, tmp, out = empty((bmm, kkd)), empty((o, bmm)), empty((b, o, m, m))
    og_t, lg, dx, db, dwg = empty((o, bmm)), empty((kkd, bmm)), empty((b, d, n, n)), empty((o,)), empty((o, kkd))

    def seq():
        drv.lower_cube(lowered, x, conv_pmap(b, d, n, k, s, p))
        drv.sgemm(RM, N_, T_, o, bmm, kkd, 1.0, w, kkd, lowered, kkd, 0.0, tmp, bmm)
        drv.remap(out, tmp, remap_pmap(m, m, o, b))
        drv.forward_bias(bias, out, m * m, o, b)
        drv.remap(og_t, og, remap_pmap(m, m, b, o))
        drv.sgemm(RM, T_, N_, kkd, bmm, o, 1.0, w, kkd, og_t, bmm, 0.0, lg, bmm)
        drv.inverse_lower_cube_bias_backward(dx, lg, lift_args(b, d, n, k, s, p), db, og, m * m, o, b)
        drv.sgemm(RM, N_, N_, o, kkd, bmm, 1.0, og_t, bmm, lowered, kkd, 0.0, dwg, kkd)

    seq()
    outputs = [lowered, out, dx, db, dwg]
    graph = _record(seq)

    def eager_work():
        # the library's own kernels on other data between the replays: workspace and counters are shared
        y = empty((o, kkd))
        drv.sgemm(RM, N_, N_, o, kkd, bmm, 1.0, og_t, bmm, lowered, kkd, 0.0, y, kkd)
        drv.backward_bias(empty((o,)), og, m * m, o, b)

    _check_replays(graph, outputs, eager_work)


@pytest.mark.parametrize("shape", [(16, 16, 13, 3, 1, 32), (8, 8, 27, 5, 2, 48), (16, 64, 14, 3, 1, 128),
                                   (6, 32, 28, 5, 2, 64), (4, 4, 100, 3, 1, 8), (4, 8, 20, 7, 3, 16)])
def test_direct_kernels_in_a_graph(shape):
    """Weight re-layout, forward (bias and ReLU in the epilogue), data gradient and weight gradient (partial
    sums over step ranges in the workspace, fixed-order reduction) of the direct path: the generic kernels, two
    compile-time weight-gradient instances, an image in column bands, a 7 x 7 layer."""
    drv = driver()
    b, d, n, k, p, o = shape
    if not drv.conv_direct_supported(b, d, n, k, 1, p, o):
        pytest.skip("geometry outside the direct kernels")
    rng = np.random.default_rng(72)
    m = n + 2 * p - k + 1
    x = dev(rng.standard_normal((b, d, n, n)).astype(np.float32))
    w = dev((rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32))
    bias = dev(rng.standard_normal(o).astype(np.float32))
    og = dev(rng.standard_normal((b, o, m, m)).astype(np.float32))
    sf = empty((drv.conv_direct_slab_floats(o, d, k, False),))
    sb = empty((drv.conv_direct_slab_floats(o, d, k, True),))
    out, dx, dw, db = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, d, k, k)), empty((o,))

    def seq():
        drv.conv_direct_slabs(sf, w, o, d, k, False)
        drv.conv_direct_slabs(sb, w, o, d, k, True)
        drv.conv_direct_forward(out, x, sf, bias, b, d, n, k, p, o, relu=True)
        drv.conv_direct_backward_data(dx, og, sb, b, d, n, k, p, o)
        drv.conv_direct_backward_weights(dw, og, x, b, d, n, k, p, o, db=db)

    seq()
    graph = _record(seq)

    def eager_work():
        drv.conv_direct_backward_weights(empty((o, d, k, k)), og, x, b, d, n, k, p, o, db=empty((o,)))

    _check_replays(graph, [out, dx, dw, db], eager_work)


@pytest.mark.parametrize("shape", [(8, 32, 13, 48), (5, 64, 8, 64)])
def test_pointwise_products_in_a_graph(shape):
    """1 x 1 layers: one product per image forward and for the data gradient, one product summed over the images
    (partial sums in the workspace, fixed-order reduction) plus the bias gradient for the weights."""
    drv = driver()
    b, d, n, o = shape
    rng = np.random.default_rng(74)
    x = dev(rng.standard_normal((b, d, n, n)).astype(np.float32))
    w = dev((rng.standard_normal((o, d)) * 0.1).astype(np.float32))
    bias = dev(rng.standard_normal(o).astype(np.float32))
    og = dev(rng.standard_normal((b, o, n, n)).astype(np.float32))
    out, dx, dw, db = empty((b, o, n, n)), empty((b, d, n, n)), empty((o, d)), empty((o,))

    def seq():
        drv.conv1x1_forward(out, x, w, bias, b, d, n * n, o, relu=True)
        drv.conv1x1_backward_data(dx, og, w, b, d, n * n, o)
        drv.conv1x1_backward_weights(dw, og, x, b, d, n * n, o, db=db)

    seq()
    graph = _record(seq)

    def eager_work():
        drv.conv1x1_backward_weights(empty((o, d)), og, x, b, d, n * n, o, db=empty((o,)))

    _check_replays(graph, [out, dx, dw, db], eager_work)


def test_elementwise_operators_in_a_graph():
    """Plane-tiled pooling forward / backward, LRN forward / backward, ReLU, softmax loss, SGD update."""
    import torch
    drv = driver()
    rng = np.random.default_rng(73)
    B, D, n = 16, 32, 27
    mo = (n - 3) // 2 + 1
    x = dev(rng.standard_normal((B, D, n, n)).astype(np.float32))
    pooled, idx = empty((B, D, mo, mo)), empty((B, D, mo, mo), dtype=torch.int32)
    pog = dev(rng.standard_normal((B, D, mo, mo)).astype(np.float32))
    pgrad = empty((B, D, n, n))
    y, den, lgrad = empty((B, D, mo, mo)), empty((B, D, mo, mo)), empty((B, D, mo, mo))
    classes = 10
    logits = dev(rng.standard_normal((B, classes)).astype(np.float32))
    labels = dev(rng.integers(0, classes, B).astype(np.float32))
    prob, loss, sgrad = empty((B, classes)), empty((1,)), empty((B, classes))
    wt0 = rng.standard_normal(5000).astype(np.float32)
    wt, hist, grad = dev(wt0), dev(np.zeros(5000, np.float32)), dev(rng.standard_normal(5000).astype(np.float32))
    grad0 = host(grad).copy()
    pargs = drv.pool_args(3, 2, n, n, D, B, idx)

    def seq():
        drv.maxpool_forward(pooled, x, pargs)
        drv.maxpool_backward(pgrad, pog, pargs, pooled=pooled)
        drv.lrn_forward(y, pooled, mo, mo, D, B, 5, 1e-4, 0.75, den)
        drv.lrn_backward(lgrad, pog, pooled, mo, mo, D, B, 5, 1e-4, 0.75, den)
        drv.softmax_loss_forward(prob, logits, labels, loss, classes, B)
        drv.softmax_loss_backward(sgrad, prob, labels, classes, B)

    with tuning("pool_plane", 1):
        seq()
        graph = _record(seq)
        _check_replays(graph, [pooled, idx, pgrad, y, den, lgrad, prob, loss, sgrad],
                       lambda: drv.relu_forward(empty((B, D, n, n)), x, x.numel()))

    # an update that accumulates state: every replay is one more iteration
    def step():
        drv.sgd_update(5000, wt, grad, hist, 0.01, 0.9, 0.0005, False)
    graph = _record(step)   # applies the update once (the eager warm-up); the capture executes nothing
    eager_w, eager_h, eager_g = dev(wt0), dev(np.zeros(5000, np.float32)), dev(grad0)
    drv.sgd_update(5000, eager_w, eager_g, eager_h, 0.01, 0.9, 0.0005, False)
    for r in range(3):
        graph.replay()
        drv.sgd_update(5000, eager_w, eager_g, eager_h, 0.01, 0.9, 0.0005, False)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host(wt), host(eager_w), err_msg="replay %d" % r)
        np.testing.assert_array_equal(host(hist), host(eager_h), err_msg="replay %d" % r)
        np.testing.assert_array_equal(host(grad), host(eager_g), err_msg="replay %d" % r)
