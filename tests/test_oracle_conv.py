"""Pins the oracle's GEMM, bias, whole-convolution and SGD steps against the reference's own
golden files (tests/input/conv_* -> tests/output/conv_*), numpy float64 and a direct
convolution written from the definition."""
import numpy as np
import pytest

from conftest import load_fixture

EPS = 1e-3  # the reference's own tolerance, tests/test_types.h:12


def direct_conv(x, w, bias, s, p):
    """Definition of cross-correlation with zero padding, float64."""
    b, d, n, _ = x.shape
    o, _, k, _ = w.shape
    m = (n + 2 * p - k) // s + 1
    xp = np.zeros((b, d, n + 2 * p, n + 2 * p), np.float64)
    xp[:, :, p:p + n, p:p + n] = x
    out = np.zeros((b, o, m, m), np.float64)
    for r in range(m):
        for c in range(m):
            win = xp[:, :, r * s:r * s + k, c * s:c * s + k].reshape(b, -1)
            out[:, :, r, c] = win @ w.reshape(o, -1).astype(np.float64).T
    if bias is not None:
        out += np.asarray(bias, np.float64)[None, :, None, None]
    return out


def direct_conv_grads(x, w, og, s, p):
    """Gradients from the definition, float64: (dx, dw, db)."""
    b, d, n, _ = x.shape
    o, _, k, _ = w.shape
    m = og.shape[2]
    xp = np.zeros((b, d, n + 2 * p, n + 2 * p), np.float64)
    xp[:, :, p:p + n, p:p + n] = x
    dxp = np.zeros_like(xp)
    dw = np.zeros(w.shape, np.float64)
    w64 = w.astype(np.float64)
    og = og.astype(np.float64)
    for r in range(m):
        for c in range(m):
            g = og[:, :, r, c]                                   # [b][o]
            win = xp[:, :, r * s:r * s + k, c * s:c * s + k]    # [b][d][k][k]
            dw += np.einsum("bo,bdij->odij", g, win)
            dxp[:, :, r * s:r * s + k, c * s:c * s + k] += np.einsum("bo,odij->bdij", g, w64)
    return dxp[:, :, p:p + n, p:p + n], dw, og.sum(axis=(0, 2, 3))


CASES = {
    "small": dict(b=4, d=3, n=20, k=5, s=4, p=2, o=10, suffix=""),
    "large": dict(b=4, d=3, n=127, k=11, s=4, p=2, o=8, suffix="_large"),
}


def _load(case):
    c = CASES[case]
    sfx = c["suffix"]
    x = load_fixture("input", f"conv_forward_in{sfx}.txt").reshape(c["b"], c["d"], c["n"], c["n"])
    shape_w = (c["o"], c["d"], c["k"], c["k"])
    w_fwd = load_fixture("input", f"conv_model{sfx}.txt").reshape(shape_w)
    w_bwd = load_fixture("input", f"conv_backward_model{sfx}.txt").reshape(shape_w)
    bias = load_fixture("input", f"conv_bias_in{sfx}.txt")
    return c, x, w_fwd, w_bwd, bias


@pytest.mark.parametrize("case", ["small", "large"])
def test_conv_forward_fixture(oracle, case):
    c, x, w, _, bias = _load(case)
    out, lowered = oracle.conv_forward(x, w, bias, c["k"], c["s"], c["p"])
    expect = load_fixture("output", f"conv_forward{c['suffix']}.txt").reshape(out.shape)
    np.testing.assert_allclose(out, expect, atol=EPS * max(1.0, np.abs(expect).max() * 1e-3), rtol=1e-5)
    # and against the definition
    ref = direct_conv(x, w, bias, c["s"], c["p"])
    np.testing.assert_allclose(out, ref, rtol=2e-6, atol=1e-4)
    if case == "small":
        # integer inputs and weights: every fp32 partial sum is exact before the bias is added
        out_nb, _ = oracle.conv_forward(x, w, None, c["k"], c["s"], c["p"])
        np.testing.assert_array_equal(out_nb, direct_conv(x, w, None, c["s"], c["p"]).astype(np.float32))


@pytest.mark.parametrize("case", ["small", "large"])
def test_conv_backward_and_sgd_fixture(oracle, case):
    """Mirrors tests/test_parallelized_convolution.cpp:184-270: forward, backward with
    out_grad[i] = 0.1*i, then one SGD step with lr 0.01, momentum 0, no weight decay."""
    c, x, _, w, bias = _load(case)
    k, s, p = c["k"], c["s"], c["p"]
    out, lowered = oracle.conv_forward(x, w, bias, k, s, p)
    og = (np.arange(out.size, dtype=np.float64) * 0.1).astype(np.float32).reshape(out.shape)
    dx, dw, db = oracle.conv_backward(x.shape, w, og, lowered, k, s, p)
    sfx = c["suffix"]

    # the large golden file holds only the first 30752 input-gradient values; the reference test
    # (tests/test_parallelized_convolution_large_CPU.cpp:217-223) compares just that prefix
    exp_dx = load_fixture("output", f"conv_backward{sfx}.txt")
    got_dx = dx.reshape(-1)[:exp_dx.size]
    assert exp_dx.size == (dx.size if case == "small" else 30752)
    np.testing.assert_allclose(got_dx, exp_dx, rtol=2e-5, atol=EPS)

    # definition, float64
    rdx, rdw, rdb = direct_conv_grads(x, w, og, s, p)
    assert np.abs(dx - rdx).max() <= 2e-6 * np.abs(rdx).max()
    assert np.abs(dw - rdw).max() <= 2e-6 * np.abs(rdw).max()
    assert np.abs(db - rdb).max() <= 2e-6 * np.abs(rdb).max()

    # SGD step: stepsize = base_lr * gamma^floor(iter/stepsize) with iter=1, stepsize=10000
    lr = oracle.learning_rate("step", 0.01, 0.1, 1, 10000, 0, 0)
    assert lr == np.float32(0.01)
    wm, hist_w = w.copy().reshape(-1), np.zeros(w.size, np.float32)
    oracle.sgd_update(wm, dw.reshape(-1).copy(), hist_w, lr, 0.0)
    bm, hist_b = bias.copy(), np.zeros(bias.size, np.float32)
    oracle.sgd_update(bm, db.copy(), hist_b, lr, 0.0)
    exp_w = load_fixture("output", f"conv_weights{sfx}.txt")
    exp_b = load_fixture("output", f"conv_bias{sfx}.txt")
    # the golden files are printed with 6 significant digits
    np.testing.assert_allclose(wm, exp_w, rtol=2e-5, atol=EPS)
    np.testing.assert_allclose(bm, exp_b, rtol=2e-5, atol=EPS)


def test_bias_fixture_closed_form(oracle):
    """conv_bias.txt: 0.3 - 0.01 * sum of out_grad over (b, m*m) for channel 0 = -38.4."""
    b, o, m = 4, 10, 5
    og = (np.arange(b * o * m * m, dtype=np.float64) * 0.1).astype(np.float32)
    db = oracle.bias_backward(og, m * m, o, b)
    np.testing.assert_allclose(db, og.reshape(b, o, m * m).astype(np.float64).sum(axis=(0, 2)), rtol=1e-6)
    assert abs((0.3 - 0.01 * db[0]) - (-38.4)) < 1e-3
    out = np.zeros((b, o, m * m), np.float32)
    oracle.bias_forward(out, np.arange(o, dtype=np.float32), m * m, o, b)
    np.testing.assert_array_equal(out, np.broadcast_to(np.arange(o, dtype=np.float32)[None, :, None], out.shape))


@pytest.mark.parametrize("order", [101, 102])
@pytest.mark.parametrize("TA", [111, 112])
@pytest.mark.parametrize("TB", [111, 112])
def test_sgemm_all_layouts(oracle, order, TA, TB):
    rng = np.random.default_rng(order * 7 + TA * 3 + TB)
    M, N, K = 7, 11, 13
    alpha, beta = 1.5, -0.5
    opA = rng.standard_normal((M, K)).astype(np.float32)
    opB = rng.standard_normal((K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    expect = alpha * opA.astype(np.float64) @ opB.astype(np.float64) + beta * C0

    def store(mat, trans):
        """Memory image + leading dimension (padded by 2) of op^-1(mat) in the given order."""
        src = mat.T if trans == 112 else mat
        if order == 102:
            src = src.T
        ld = src.shape[1] + 2
        buf = np.full((src.shape[0], ld), np.nan, np.float32)
        buf[:, :src.shape[1]] = src
        return buf, ld

    A, lda = store(opA, TA)
    B, ldb = store(opB, TB)
    Cbuf, ldc = store(C0, 111)
    for f64 in (False, True):
        Cc = Cbuf.copy()
        oracle.sgemm(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, Cc, ldc, f64acc=f64)
        got = Cc[:, :(N if order == 101 else M)]
        got = got if order == 101 else got.T
        np.testing.assert_allclose(got, expect, rtol=1e-5, atol=1e-5)
        assert np.isnan(Cc[:, -2:]).all()  # padding untouched
    # beta == 0 must not read C
    Cn = np.full_like(Cbuf, np.nan)
    oracle.sgemm(order, TA, TB, M, N, K, 1.0, A, lda, B, ldb, 0.0, Cn, ldc)
    got = Cn[:, :(N if order == 101 else M)]
    got = got if order == 101 else got.T
    np.testing.assert_allclose(got, opA.astype(np.float64) @ opB.astype(np.float64), rtol=1e-5, atol=1e-5)


def test_sgemm_new_and_sgemv(oracle):
    rng = np.random.default_rng(11)
    M, N, K = 5, 9, 6
    for TA in (111, 112):
        for TB in (111, 112):
            a = rng.standard_normal((M, K)).astype(np.float32)
            b = rng.standard_normal((K, N)).astype(np.float32)
            A = np.ascontiguousarray(a.T if TA == 112 else a)
            B = np.ascontiguousarray(b.T if TB == 112 else b)
            Cm = np.zeros((M, N), np.float32)
            oracle.sgemm_new(TA, TB, M, N, K, 1.0, A, B, 0.0, Cm)
            np.testing.assert_allclose(Cm, a.astype(np.float64) @ b, rtol=1e-5, atol=1e-5)
    A = rng.standard_normal((M, N)).astype(np.float32)
    x = rng.standard_normal(N).astype(np.float32)
    y = rng.standard_normal(M).astype(np.float32)
    y0 = y.copy()
    oracle.sgemv(111, M, N, 2.0, A, x, 0.5, y)
    np.testing.assert_allclose(y, 2.0 * A @ x + 0.5 * y0, rtol=1e-5, atol=1e-5)
    xt = rng.standard_normal(M).astype(np.float32)
    yt = np.zeros(N, np.float32)
    oracle.sgemv(112, M, N, 1.0, A, xt, 0.0, yt)
    np.testing.assert_allclose(yt, A.T @ xt, rtol=1e-5, atol=1e-5)


def test_openblas_binding_agrees(oracle):
    """The BLAS route used for the CPU baseline computes the same products as the plain loops."""
    if not oracle.bind_openblas(1):
        pytest.skip("no OpenBLAS shared library found")
    try:
        rng = np.random.default_rng(3)
        x = rng.standard_normal((2, 8, 9, 9)).astype(np.float32)
        w = (rng.standard_normal((6, 8, 3, 3)) * 0.1).astype(np.float32)
        out_b, low = oracle.conv_forward(x, w, None, 3, 1, 1)
        og = rng.standard_normal(out_b.shape).astype(np.float32)
        g_b = oracle.conv_backward(x.shape, w, og, low, 3, 1, 1)
    finally:
        oracle.unbind_openblas()
    out_n, low_n = oracle.conv_forward(x, w, None, 3, 1, 1)
    g_n = oracle.conv_backward(x.shape, w, og, low_n, 3, 1, 1)
    np.testing.assert_allclose(out_b, out_n, rtol=1e-4, atol=1e-5)
    for a, b in zip(g_b, g_n):
        np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4)


def test_fc_equals_conv_with_full_kernel(oracle):
    """Invariant used by tests/test_fc_bridge.cpp:153-159,220-233: FC == conv with k=n, p=0, s=1."""
    rng = np.random.default_rng(17)
    b, d, n, o = 3, 4, 5, 6
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = rng.standard_normal((o, d, n, n)).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    out_c, low = oracle.conv_forward(x, w, bias, n, 1, 0)
    out_f = oracle.fc_forward(x.reshape(b, -1), w.reshape(o, -1), bias)
    np.testing.assert_allclose(out_f, out_c.reshape(b, o), rtol=1e-5, atol=1e-5)
    og = rng.standard_normal((b, o)).astype(np.float32)
    dx_c, dw_c, db_c = oracle.conv_backward(x.shape, w, og.reshape(b, o, 1, 1), low, n, 1, 0)
    dx_f, dw_f, db_f = oracle.fc_backward(x.reshape(b, -1), w.reshape(o, -1), og)
    np.testing.assert_allclose(dx_f, dx_c.reshape(b, -1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dw_f, dw_c.reshape(o, -1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db_f, db_c, rtol=1e-5, atol=1e-5)


def test_sgd_recurrence(oracle):
    rng = np.random.default_rng(23)
    n = 1000
    w = rng.standard_normal(n).astype(np.float32)
    h = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    w0, h0, g0 = w.copy(), h.copy(), g.copy()
    oracle.sgd_update(w, g, h, 0.01, 0.9, 0.0005)
    g1 = (g0 + np.float32(0.0005) * w0).astype(np.float32)
    h1 = (np.float32(0.01) * g1 + np.float32(0.9) * h0).astype(np.float32)
    np.testing.assert_allclose(g, g1, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(h, h1, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(w, w0 - h1, rtol=1e-6, atol=1e-7)
    # L1
    w, h, g = w0.copy(), h0.copy(), g0.copy()
    oracle.sgd_update(w, g, h, 0.01, 0.9, 0.0005, l1=True)
    np.testing.assert_allclose(g, g0 + np.float32(0.0005) * np.where(w0 > 0, 1, -1), rtol=1e-6, atol=1e-7)
