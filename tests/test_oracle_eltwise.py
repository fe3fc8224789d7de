"""Pins the oracle's ReLU / max-pool / LRN / dropout / softmax-loss against the reference's golden
files (tests/input/* -> tests/output/*) and against their definitions in numpy."""
import numpy as np

from conftest import load_fixture

EPS = 1e-3  # tests/test_types.h:12


def test_relu_fixture(oracle):
    x = load_fixture("input", "relu_forward_in.txt").reshape(5, 3, 20, 20)
    y = oracle.relu_forward(x)
    np.testing.assert_array_equal(y.reshape(-1), load_fixture("output", "relu_forward.txt"))
    og = np.arange(x.size, dtype=np.float32).reshape(x.shape)
    g = oracle.relu_backward(og, x)
    np.testing.assert_array_equal(g.reshape(-1), load_fixture("output", "relu_backward.txt"))


def test_maxpool_fixture(oracle):
    x = load_fixture("input", "pooling_forward_in.txt").reshape(5, 3, 10, 10)
    y, idx = oracle.maxpool_forward(x, 4, 2)
    assert y.shape == (5, 3, 4, 4)
    np.testing.assert_allclose(y.reshape(-1), load_fixture("output", "pooling_forward.txt"), atol=EPS)
    og = np.arange(y.size, dtype=np.float32).reshape(y.shape)
    g = oracle.maxpool_backward(og, idx, 10, 10)
    np.testing.assert_allclose(g.reshape(-1), load_fixture("output", "pooling_backward.txt"), atol=EPS)


def test_maxpool_definition_and_ties(oracle):
    rng = np.random.default_rng(2)
    x = rng.integers(0, 4, size=(2, 3, 13, 13)).astype(np.float32)  # many ties
    k, s = 3, 2
    y, idx = oracle.maxpool_forward(x, k, s)
    oR = (13 - k) // s + 1
    for ph in range(oR):
        for pw in range(oR):
            win = x[:, :, ph * s:ph * s + k, pw * s:pw * s + k].reshape(2, 3, -1)
            np.testing.assert_array_equal(y[:, :, ph, pw], win.max(axis=2))
            am = win.argmax(axis=2)  # first maximum in row-major order
            np.testing.assert_array_equal(idx[:, :, ph, pw], (ph * s + am // k) * 13 + pw * s + am % k)


def test_lrn_fixture_and_definition(oracle):
    x = load_fixture("input", "lrn_forward_in.txt").reshape(6, 3, 10, 10)
    size, alpha, beta = 3, 1e-4, 0.75
    y, den = oracle.lrn_forward(x, size, alpha, beta)
    np.testing.assert_allclose(y.reshape(-1), load_fixture("output", "lrn_forward.txt"), atol=EPS)
    # definition: scale = 1 + alpha/size * sum_{window} x^2 ; y = x / scale^beta
    x64 = x.astype(np.float64)
    sq = np.zeros_like(x64)
    w = size // 2
    for dd in range(3):
        lo, hi = max(0, dd - w), min(3, dd + w + 1)
        sq[:, dd] = (x64[:, lo:hi] ** 2).sum(axis=1)
    scale = 1 + alpha / size * sq
    np.testing.assert_allclose(den, scale, rtol=1e-5)
    np.testing.assert_allclose(y, x64 / scale ** beta, rtol=1e-5, atol=1e-6)

    og = load_fixture("input", "lrn_backward_in.txt").reshape(x.shape)
    g = oracle.lrn_backward(og, x, den, size, alpha, beta)
    np.testing.assert_allclose(g.reshape(-1), load_fixture("output", "lrn_backward.txt"), atol=EPS)
    # definition of the gradient (Caffe's across-channel LRN), float64
    og64 = og.astype(np.float64)
    yy = x64 / scale ** beta
    ratio = og64 * yy / scale
    acc = np.zeros_like(x64)
    for dd in range(3):
        lo, hi = max(0, dd - w), min(3, dd + w + 1)
        acc[:, dd] = ratio[:, lo:hi].sum(axis=1)
    expect = og64 * scale ** (-beta) - 2.0 * alpha / size * beta * x64 * acc
    np.testing.assert_allclose(g, expect, rtol=1e-4, atol=1e-6)


def test_lrn_running_window_wider_than_depth(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 7, 3, 3)).astype(np.float32)
    size, alpha, beta = 5, 1e-2, 0.75
    y, den = oracle.lrn_forward(x, size, alpha, beta)
    x64 = x.astype(np.float64)
    sq = np.zeros_like(x64)
    for dd in range(7):
        lo, hi = max(0, dd - 2), min(7, dd + 3)
        sq[:, dd] = (x64[:, lo:hi] ** 2).sum(axis=1)
    np.testing.assert_allclose(den, 1 + alpha / size * sq, rtol=1e-5)
    np.testing.assert_allclose(y, x64 / (1 + alpha / size * sq) ** beta, rtol=1e-5, atol=1e-6)


def test_dropout_fixture(oracle):
    x = load_fixture("input", "dropout_forward_in.txt")
    mask = load_fixture("input", "dropout_mask.txt").astype(np.uint32)
    assert set(np.unique(mask)) <= {0, 1}
    y = oracle.dropout_forward(x, mask, 0.5)
    np.testing.assert_allclose(y, load_fixture("output", "dropout_forward.txt"), atol=EPS)
    g = oracle.dropout_forward(load_fixture("input", "dropout_backward_in.txt"), mask, 0.5)
    np.testing.assert_allclose(g, load_fixture("output", "dropout_backward"), atol=EPS)
    # device flavour: keep iff mask word > UINT_MAX*ratio
    rng = np.random.default_rng(9)
    words = rng.integers(0, 2**32, size=x.size, dtype=np.uint64).astype(np.uint32)
    words[:3] = [2147483648, 2147483649, 2147483647]
    yt = oracle.dropout_forward(x, words, 0.5, threshold=True)
    np.testing.assert_array_equal(yt, x * (words > 2147483648) * np.float32(2.0))


def test_softmax_fixture_and_definition(oracle):
    x = load_fixture("input", "softmax_forward_in.txt").reshape(5, 100, 1, 1)
    labels = load_fixture("input", "softmax_label.txt")
    prob, loss = oracle.softmax_loss_forward(x, labels)
    assert abs(loss - float(load_fixture("output", "softmax_forward.txt")[0])) < EPS
    x64 = x.reshape(5, 100).astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    p64 = e / e.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(prob.reshape(5, 100), p64, rtol=1e-5, atol=1e-7)
    assert abs(loss - (-np.log(p64[np.arange(5), labels.astype(int)]).sum())) < 1e-4

    pin = load_fixture("input", "softmax_backward_in.txt").reshape(5, 100, 1, 1)
    g = oracle.softmax_loss_backward(pin, labels)
    np.testing.assert_allclose(g.reshape(-1), load_fixture("output", "softmax_backward.txt"), atol=EPS)
    onehot = np.zeros((5, 100))
    onehot[np.arange(5), labels.astype(int)] = 1
    np.testing.assert_allclose(g.reshape(5, 100), (pin.reshape(5, 100) - onehot) / 5, rtol=1e-6, atol=1e-7)
