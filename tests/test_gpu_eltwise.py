"""GPU parity: ReLU, max pooling, LRN, dropout, softmax loss, SGD / BLAS-1 kernels against the CPU
oracle and the reference's golden files."""
import numpy as np
import pytest

from conftest import load_fixture
from gpu_util import dev, driver, empty, host, rel_err, tuning

pytestmark = pytest.mark.gpu


def test_relu_fixture_and_oracle(oracle):
    import torch
    x = load_fixture("input", "relu_forward_in.txt")
    drv = driver()
    y = empty(x.shape)
    drv.relu_forward(y, dev(x), x.size)
    np.testing.assert_array_equal(host(y), load_fixture("output", "relu_forward.txt"))
    og = np.arange(x.size, dtype=np.float32)
    g = empty(x.shape)
    drv.relu_backward(g, dev(og), dev(x), x.size)
    np.testing.assert_array_equal(host(g), load_fixture("output", "relu_backward.txt"))
    rng = np.random.default_rng(1)
    z = rng.standard_normal(100003).astype(np.float32)
    y = empty(z.shape)
    drv.relu_forward(y, dev(z), z.size)
    np.testing.assert_array_equal(host(y), oracle.relu_forward(z))
    # in place, as the reference runs ReLU on shared input/output layers
    dz = dev(z)
    drv.relu_forward(dz, dz, z.size)
    np.testing.assert_array_equal(host(dz), oracle.relu_forward(z))
    assert torch.cuda.is_available()


@pytest.mark.parametrize("cfg", [(5, 3, 10, 4, 2), (2, 4, 13, 3, 2), (3, 2, 24, 2, 2), (2, 3, 55, 3, 2), (1, 2, 7, 3, 1),
                                 # several planes per workgroup with a partial last group; planes too large
                                 # for the LDS-tiled kernels (forward only, both, window wider than 2 strides)
                                 (7, 11, 13, 3, 2), (1, 2, 100, 3, 2), (1, 1, 150, 2, 2), (1, 1, 140, 5, 2),
                                 # rows of 27, 64 and 65 elements: the lanes-over-rows backward kernel and its limit
                                 (3, 5, 27, 3, 2), (2, 3, 64, 3, 2), (2, 3, 65, 2, 2),
                                 # a last row and column that no window covers ((n - k) % s != 0)
                                 (5, 15, 31, 2, 2), (3, 8, 28, 3, 2), (2, 6, 30, 3, 2)])
@pytest.mark.parametrize("plane_tiled", [False, True])
def test_maxpool_bit_exact(oracle, cfg, plane_tiled):
    # small tensors take the one-lane-per-element kernels unless the plane-tiled ones are forced
    with tuning("pool_plane", int(plane_tiled)):
        _maxpool_bit_exact(oracle, cfg)


def _maxpool_bit_exact(oracle, cfg):
    B, D, n, k, s = cfg
    rng = np.random.default_rng(sum(cfg))
    if cfg == (5, 3, 10, 4, 2):
        x = load_fixture("input", "pooling_forward_in.txt").reshape(B, D, n, n)
    else:
        x = rng.integers(0, 5, size=(B, D, n, n)).astype(np.float32)  # ties on purpose
    drv = driver()
    import torch
    oR = (n - k) // s + 1
    idx = empty((B, D, oR, oR), dtype=torch.int32)
    args = drv.pool_args(k, s, n, n, D, B, idx)
    y = empty((B, D, oR, oR))
    drv.maxpool_forward(y, dev(x), args)
    ry, ridx = oracle.maxpool_forward(x, k, s)
    np.testing.assert_array_equal(host(y), ry)
    np.testing.assert_array_equal(host(idx), ridx)
    og = rng.standard_normal(ry.shape).astype(np.float32)
    if cfg == (5, 3, 10, 4, 2):
        og = np.arange(ry.size, dtype=np.float32).reshape(ry.shape)
    g = empty(x.shape)
    drv.maxpool_backward(g, dev(og), args)
    np.testing.assert_array_equal(host(g), oracle.maxpool_backward(og, ridx, n, n))
    # with the backward of an in-place ReLU on the pooled tensor folded in: the same gradient where
    # the tensor is positive, zero elsewhere (x holds zeros, so the mask bites)
    g2 = empty(x.shape)
    drv.maxpool_backward(g2, dev(og), args, relu_data=dev(x))
    np.testing.assert_array_equal(host(g2), oracle.relu_backward(host(g), x))
    assert cfg == (5, 3, 10, 4, 2) or (x <= 0).any()
    # the same mask taken from the pooling output (a window's arg-max holds the window's maximum)
    g3 = empty(x.shape)
    drv.maxpool_backward(g3, dev(og), args, pooled=y)
    np.testing.assert_array_equal(host(g3), host(g2))
    if cfg == (5, 3, 10, 4, 2):
        np.testing.assert_allclose(host(y).reshape(-1), load_fixture("output", "pooling_forward.txt"), atol=1e-3)
        np.testing.assert_allclose(host(g).reshape(-1), load_fixture("output", "pooling_backward.txt"), atol=1e-3)


@pytest.mark.parametrize("cfg", [(6, 3, 10, 3, 1e-4, 0.75), (2, 96, 27, 5, 1e-4, 0.75), (3, 7, 5, 5, 1e-2, 0.75),
                                 # other exponents (exp2/log2 form) with windows of 5 and 3, a strong alpha,
                                 # and a negative alpha (library powf)
                                 (2, 16, 9, 5, 1e-2, 0.5), (2, 16, 9, 3, 2e-2, 1.25), (2, 20, 6, 5, 0.5, 0.75),
                                 (2, 8, 6, 5, -1e-3, 0.75), (2, 8, 6, 3, -1e-3, 0.6)])
def test_lrn(oracle, cfg):
    B, D, n, size, alpha, beta = cfg
    rng = np.random.default_rng(B + D)
    if cfg[0] == 6:
        x = load_fixture("input", "lrn_forward_in.txt").reshape(B, D, n, n)
        og = load_fixture("input", "lrn_backward_in.txt").reshape(B, D, n, n)
    else:
        x = (rng.standard_normal((B, D, n, n)) * 3).astype(np.float32)
        og = rng.standard_normal((B, D, n, n)).astype(np.float32)
    drv = driver()
    y, den = empty(x.shape), empty(x.shape)
    dx = dev(x)
    drv.lrn_forward(y, dx, n, n, D, B, size, alpha, beta, den)
    ry, rden = oracle.lrn_forward(x, size, alpha, beta)
    assert rel_err(host(den), rden) <= 1e-6
    assert rel_err(host(y), ry) <= 1e-5
    g = empty(x.shape)
    drv.lrn_backward(g, dev(og), dx, n, n, D, B, size, alpha, beta, den)
    rg = oracle.lrn_backward(og, x, rden, size, alpha, beta)
    assert rel_err(host(g), rg) <= 1e-5
    if cfg[0] == 6:
        np.testing.assert_allclose(host(y).reshape(-1), load_fixture("output", "lrn_forward.txt"), atol=1e-3)
        np.testing.assert_allclose(host(g).reshape(-1), load_fixture("output", "lrn_backward.txt"), atol=1e-3)


def test_dropout(oracle):
    import torch
    drv = driver()
    x = load_fixture("input", "dropout_forward_in.txt")
    mask01 = load_fixture("input", "dropout_mask.txt").astype(np.uint32)
    # the golden mask is 0/1: with threshold 0 "mask > threshold" keeps exactly the ones
    y = empty(x.shape)
    drv.dropout_forward_train(y, dev(x), dev(mask01.astype(np.int64)).to(torch.int32), 2.0, 0, x.size)
    np.testing.assert_allclose(host(y), load_fixture("output", "dropout_forward.txt"), atol=1e-3)
    # device flavour: uint32 words against threshold UINT_MAX*ratio
    n = 100000
    drv.init_rng(42)
    words = empty((n,), dtype=torch.int32)
    drv.rand_uint_initialize(words, n)
    w_host = host(words).view(np.uint32)
    keep = (w_host > 2147483648).mean()
    assert abs(keep - 0.5) < 0.01                       # Bernoulli(1 - ratio) mean, as test_device_driver_cpu.cpp does
    words2 = empty((n,), dtype=torch.int32)
    drv.rand_uint_initialize(words2, n)
    assert (host(words2).view(np.uint32) != w_host).mean() > 0.99   # a new mask every call
    drv.init_rng(42)
    words3 = empty((n,), dtype=torch.int32)
    drv.rand_uint_initialize(words3, n)
    np.testing.assert_array_equal(host(words3), host(words))  # same seed, same stream
    z = np.random.default_rng(0).standard_normal(n).astype(np.float32)
    dz = dev(z)
    drv.dropout_forward_train(dz, dz, words, 2.0, 2147483648, n)  # in place as the reference does
    np.testing.assert_array_equal(host(dz), oracle.dropout_forward(z, w_host, 0.5, threshold=True))


def test_softmax_loss(oracle):
    drv = driver()
    for (B, D, use_fixture) in ((5, 100, True), (64, 10, False), (16, 1000, False)):
        rng = np.random.default_rng(B)
        if use_fixture:
            x = load_fixture("input", "softmax_forward_in.txt").reshape(B, D, 1, 1)
            labels = load_fixture("input", "softmax_label.txt")
        else:
            x = (rng.standard_normal((B, D, 1, 1)) * 4).astype(np.float32)
            labels = rng.integers(0, D, size=B).astype(np.float32)
        prob, loss = empty(x.shape), empty((1,))
        dl = dev(labels)
        drv.softmax_loss_forward(prob, dev(x), dl, loss, D, B)
        rprob, rloss = oracle.softmax_loss_forward(x, labels)
        assert rel_err(host(prob), rprob) <= 1e-5
        assert abs(float(host(loss)[0]) - rloss) <= 1e-4 * max(1.0, abs(rloss))
        if use_fixture:
            assert abs(float(host(loss)[0]) - 23.4224) < 1e-3
        g = empty(x.shape)
        drv.softmax_loss_backward(g, prob, dl, D, B, 1)
        rg = oracle.softmax_loss_backward(rprob, labels)
        assert rel_err(host(g), rg) <= 1e-5
        # both passes in one launch: the same probabilities, loss and gradient bit for bit, call after call
        # (the launch's arrival counter must come back to zero each time)
        for _ in range(3):
            prob2, loss2, g2 = empty(x.shape), empty((1,)), empty(x.shape)
            drv.softmax_loss_forward_backward(prob2, g2, dev(x), dl, loss2, D, B, 1)
            np.testing.assert_array_equal(host(prob2), host(prob))
            np.testing.assert_array_equal(host(loss2), host(loss))
            np.testing.assert_array_equal(host(g2), host(g))
    # a label that is no class index: that image's loss (and the sum) is NaN, its gradient subtracts no 1
    x = np.zeros((3, 4, 1, 1), np.float32)
    bad = np.array([1.0, 7.0, 2.0], np.float32)
    prob, loss, g = empty(x.shape), empty((1,)), empty(x.shape)
    drv.softmax_loss_forward_backward(prob, g, dev(x), dev(bad), loss, 4, 3, 1)
    assert np.isnan(host(loss)[0])
    np.testing.assert_allclose(host(g).reshape(3, 4)[1], np.full(4, 0.25 / 3, np.float32), rtol=1e-6)
    np.testing.assert_allclose(host(g).reshape(3, 4)[0], np.array([0.25, -0.75, 0.25, 0.25], np.float32) / 3, rtol=1e-6)
    pin = load_fixture("input", "softmax_backward_in.txt")
    labels = load_fixture("input", "softmax_label.txt")
    g = empty(pin.shape)
    drv.softmax_loss_backward(g, dev(pin), dev(labels), 100, 5, 1)
    np.testing.assert_allclose(host(g), load_fixture("output", "softmax_backward.txt"), atol=1e-3)


def test_sgd_and_blas1(oracle):
    drv = driver()
    rng = np.random.default_rng(31)
    n = 614400  # AlexNet conv2 weights
    w = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    h = rng.standard_normal(n).astype(np.float32)
    for lam, l1 in ((0.0, False), (0.0005, False), (0.0005, True)):
        dw, dg, dh = dev(w), dev(g), dev(h)
        drv.sgd_update(n, dw, dg, dh, 0.01, 0.9, lam, l1)
        rw, rg, rh = w.copy(), g.copy(), h.copy()
        oracle.sgd_update(rw, rg, rh, 0.01, 0.9, lam, l1)
        np.testing.assert_array_equal(host(dg), rg)
        np.testing.assert_array_equal(host(dh), rh)
        np.testing.assert_array_equal(host(dw), rw)
    # the three separate driver calls the reference makes give the same bits as the fused kernel
    dw, dg, dh = dev(w), dev(g), dev(h)
    drv.math_saxpy(n, 0.0005, dw, dg)
    drv.math_saxpby(n, 0.01, dg, 0.9, dh)
    drv.math_saxpy(n, -1.0, dh, dw)
    rw, rg, rh = w.copy(), g.copy(), h.copy()
    oracle.sgd_update(rw, rg, rh, 0.01, 0.9, 0.0005, False)
    np.testing.assert_array_equal(host(dw), rw)
    dg = dev(g)
    drv.L1_update(n, dg, 0.25, dev(w))
    np.testing.assert_array_equal(host(dg), g + np.float32(0.25) * np.where(w > 0, 1, -1).astype(np.float32))


def test_sgd_batch_matches_single_updates(oracle):
    """Several tensors in one launch (more than one table of 16, sizes around the 512-element
    chunks, an empty one, every regulariser): the bits of the oracle's update for each."""
    drv = driver()
    rng = np.random.default_rng(77)
    sizes = [1, 10, 256, 511, 512, 513, 2047, 2048, 2049, 0, 4097, 500, 20, 50, 96, 384, 4096, 1000, 34848, 25000, 307200, 7, 800]
    jobs, refs, devs = [], [], []
    for t, n in enumerate(sizes):
        w, g, h = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
        step, mom = np.float32(0.01 * (1 + t % 3)), np.float32(0.9 if t % 2 else 0.0)
        lam, l1 = [(0.0, False), (0.0005, False), (0.001, True)][t % 3]
        rw, rg, rh = w.copy(), g.copy(), h.copy()
        if n:
            oracle.sgd_update(rw, rg, rh, float(step), float(mom), lam, l1)
        dw, dg, dh = (dev(a) if n else empty((1,)) for a in (w, g, h))
        jobs.append((n, dw, dg, dh, float(step), float(mom), lam, l1))
        refs.append((rw, rg, rh))
        devs.append((dw, dg, dh))
    drv.sgd_update_batch(jobs)
    for n, (rw, rg, rh), (dw, dg, dh) in zip(sizes, refs, devs):
        if n == 0:
            continue
        np.testing.assert_array_equal(host(dw), rw)
        np.testing.assert_array_equal(host(dg), rg)
        np.testing.assert_array_equal(host(dh), rh)
    drv.sgd_update_batch([])  # nothing to do


def test_fill_and_memory():
    """tests/test_device_driver_cpu.cpp:22-206 counterparts: constant init, memset, memcpy."""
    import ctypes as C
    drv = driver()
    n = 1000
    buf = empty((n,))
    drv.sconstant_initialize(buf, n, 3.25)
    assert (host(buf) == 3.25).all()
    drv.memset(buf, 0, n * 4)
    assert (host(buf) == 0).all()
    src = np.arange(n, dtype=np.float32)
    drv.memcpy(buf, src.ctypes.data, n * 4, 0)
    back = np.zeros(n, np.float32)
    drv.memcpy(back.ctypes.data, buf, n * 4, 1)
    np.testing.assert_array_equal(back, src)
    p = drv.malloc(4096)
    assert p != 0
    drv.memcpy(p, buf, 4000, 2)
    out = np.zeros(n, np.float32)
    drv.memcpy(out.ctypes.data, p, 4000, 1)
    np.testing.assert_array_equal(out, src)
    drv.free(p)
    assert C.sizeof(C.c_void_p) == 8


def test_fillers_on_the_device_equal_the_host_draws():
    """cct_hip_fill_* = the host draw (pinned in tests/test_fillers.py) copied to the device."""
    import ctypes as C
    from caffecontroll_amd import _lib
    drv = driver()
    lib = _lib.load()
    n = 1200
    want = np.empty(n, np.float32)
    for name, args in (("xavier", (48, 3)), ("bernoulli", (0.3, 5)), ("gaussian", (0.5, 0.01, 7))):
        t = empty((n,))
        getattr(drv, "fill_" + name)(t, n, *args)
        _lib.check(getattr(lib, "cct_filler_draw_" + name)(want.ctypes.data_as(C.c_void_p), n, *args), name)
        np.testing.assert_array_equal(host(t), want)
