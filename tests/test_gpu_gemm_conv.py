"""GPU parity: sgemm / sgemm_new / sgemv and the whole convolution forward+backward (driver-level
call sequence of ConvolutionBridge) against the CPU oracle and the reference's golden files.

fp32 tolerance (the bar this path is held to): max|gpu - ref| / max|ref| <= 1e-4 per tensor, arbitrated
against a float64-accumulating reference."""
import numpy as np
import pytest

from conftest import load_fixture
from gpu_util import dev, driver, empty, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4
RM, CM, N_, T_ = 101, 102, 111, 112


def _store(mat, trans, order, pad):
    src = mat.T if trans == T_ else mat
    if order == CM:
        src = src.T
    ld = src.shape[1] + pad
    buf = np.full((src.shape[0], ld), np.nan, np.float32)
    buf[:, :src.shape[1]] = src
    return buf, ld


GEMM_CASES = [
    # (M, N, K, pad) -- pad != 0 exercises leading dimensions that break 16-byte alignment
    (7, 11, 13, 0), (64, 64, 16, 0), (65, 63, 17, 3), (128, 128, 64, 0), (256, 384, 100, 0),
    (300, 200, 75, 1), (20, 576, 25, 0), (500, 64, 800, 0), (10, 500, 64, 0), (256, 130, 8, 4),
    # row counts for which the 96-row tile pads least (AlexNet conv1 has 96 output maps), with ragged
    # columns, a K tail and unaligned leading dimensions
    (96, 4000, 363, 0), (90, 1100, 50, 1), (192, 3000, 40, 0), (96, 130, 1100, 3),
]


@pytest.mark.parametrize("case", GEMM_CASES, ids=lambda c: "M%d_N%d_K%d_pad%d" % c)
@pytest.mark.parametrize("TA", [N_, T_])
@pytest.mark.parametrize("TB", [N_, T_])
@pytest.mark.parametrize("order", [RM, CM])
def test_sgemm_all_layouts(oracle, case, TA, TB, order):
    M, N, K, pad = case
    rng = np.random.default_rng(M * 3 + N * 5 + K * 7 + TA + TB + order)
    opA = rng.standard_normal((M, K)).astype(np.float32)
    opB = rng.standard_normal((K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    A, lda = _store(opA, TA, order, pad)
    B, ldb = _store(opB, TB, order, pad)
    Cb, ldc = _store(C0, N_, order, pad)
    for alpha, beta in ((1.0, 0.0), (1.5, -0.5)):
        ref64 = alpha * opA.astype(np.float64) @ opB.astype(np.float64) + beta * C0
        if beta == 0.0:
            Cstart = np.full_like(Cb, np.nan)  # beta == 0 must not read C
        else:
            Cstart = Cb.copy()
        dC = dev(Cstart)
        driver().sgemm(order, TA, TB, M, N, K, alpha, dev(A), lda, dev(B), ldb, beta, dC, ldc)
        out = host(dC)
        got = out[:, :N] if order == RM else out[:, :M].T
        assert rel_err(got, ref64) <= TOL
        if pad:
            assert np.isnan(out[:, -pad:]).all()  # padding columns untouched
        Co = Cstart.copy()
        if beta != 0.0:
            oracle.sgemm(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, Co, ldc)
            ref = Co[:, :N] if order == RM else Co[:, :M].T
            assert rel_err(got, ref) <= TOL


# shapes that meet the preconditions of the direct global -> LDS operand transfers (16-byte aligned bases,
# leading dimensions and row-contiguous row counts multiples of 4, K a multiple of 16): every tile shape,
# ragged tile edges, one split-K case
DMA_CASES = [(64, 64, 16), (128, 128, 64), (256, 384, 96), (300, 200, 80), (500, 64, 800), (96, 4000, 368),
             (192, 3004, 48), (256, 1000, 4096), (20, 576, 32), (260, 132, 1024)]


@pytest.mark.parametrize("case", DMA_CASES, ids=lambda c: "M%d_N%d_K%d" % c)
@pytest.mark.parametrize("TA", [N_, T_])
@pytest.mark.parametrize("TB", [N_, T_])
def test_sgemm_direct_transfer_path_matches_register_path(TA, TB, case):
    """Operand tiles moved global -> LDS directly (the default where the operands allow it) against the same
    kernel staging them through registers (tuning knob gemm_nodma): the k order of every accumulator is the same,
    so the results must be identical bit for bit; and both within tolerance of float64."""
    from gpu_util import tuning
    M, N, K = case
    rng = np.random.default_rng(M + 3 * N + 5 * K + TA + 2 * TB)
    opA = rng.standard_normal((M, K)).astype(np.float32)
    opB = rng.standard_normal((K, N)).astype(np.float32)
    A = np.ascontiguousarray(opA.T if TA == T_ else opA)
    B = np.ascontiguousarray(opB.T if TB == T_ else opB)
    drv = driver()
    dA, dB = dev(A), dev(B)
    c_dma, c_reg = empty((M, N)), empty((M, N))
    drv.sgemm_new(TA, TB, M, N, K, 1.0, dA, dB, 0.0, c_dma)
    def flags():  # template arguments after the tile: <A k-contiguous>,<B k-contiguous>[,true for direct transfers]
        name = drv.lib.cct_hip_last_kernel().decode()
        return name[name.index(">,") + 2:name.rindex(">")].split(",")

    assert len(flags()) == 3 and flags()[2] == "true"
    with tuning("gemm_nodma", 1):
        drv.sgemm_new(TA, TB, M, N, K, 1.0, dA, dB, 0.0, c_reg)
        assert len(flags()) == 2
    np.testing.assert_array_equal(host(c_dma), host(c_reg))
    assert rel_err(host(c_dma), opA.astype(np.float64) @ opB.astype(np.float64)) <= TOL


def test_sgemm_split_k_is_deterministic_and_correct(oracle):
    """Tiny output, long K: the weight-gradient shape class (goes through the split-K path)."""
    M, N, K = 40, 75, 40000
    rng = np.random.default_rng(5)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    ref64 = 0.5 * A.astype(np.float64) @ B.astype(np.float64) + 2.0 * C0
    outs = []
    for _ in range(2):
        dC = dev(C0)
        driver().sgemm(RM, N_, N_, M, N, K, 0.5, dev(A), K, dev(B), N, 2.0, dC, N)
        outs.append(host(dC))
    np.testing.assert_array_equal(outs[0], outs[1])
    assert rel_err(outs[0], ref64) <= TOL


FC_SMALL = [(64, 500, 10), (64, 800, 32), (1, 7, 1), (37, 129, 17), (256, 4096, 16), (1024, 33, 3)]


@pytest.mark.parametrize("shape", FC_SMALL, ids=lambda c: "b%d_i%d_o%d" % c)
def test_fc_small_kernels_match_oracle_and_gemm_path(oracle, shape):
    """Inner-product layers of few outputs (LeNet's 500 -> 10): forward and backward as one launch each,
    against the oracle's FullyConnectedBridge and against the library's own three-GEMM path; the ReLU clamp
    (forward) and the ReLU mask on the input gradient (backward) are exactly those of the separate passes."""
    B_, I, O = shape
    rng = np.random.default_rng(B_ + I + O)
    x = rng.standard_normal((B_, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B_, O)).astype(np.float32)
    bias = rng.standard_normal(O).astype(np.float32)
    drv = driver()
    assert drv.fc_small_supported(B_, I, O)
    dx_, dw_, db_ = dev(x), dev(w), dev(bias)
    y = empty((B_, O))
    drv.fc_small_forward(y, dx_, dw_, db_, B_, I, O)
    ref_y = oracle.fc_forward(x, w, bias)
    assert rel_err(host(y), ref_y) <= TOL
    y_nb, y_relu = empty((B_, O)), empty((B_, O))
    drv.fc_small_forward(y_nb, dx_, dw_, None, B_, I, O)
    assert rel_err(host(y_nb), ref_y - bias[None, :]) <= TOL
    drv.fc_small_forward(y_relu, dx_, dw_, db_, B_, I, O, relu=True)
    np.testing.assert_array_equal(host(y_relu), oracle.relu_forward(host(y)))
    y_gemm = empty((B_, O))
    drv.sgemm_new_bias(N_, T_, B_, O, I, 1.0, dx_, dw_, 0.0, y_gemm, db_, False)
    assert rel_err(host(y), host(y_gemm)) <= 1e-5
    # backward
    gx, gw, gb = empty((B_, I)), empty((O, I)), empty((O,))
    drv.fc_small_backward(gx, gw, gb, dev(dy), dx_, dw_, B_, I, O)
    rdx, rdw, rdb = oracle.fc_backward(x, w, dy)
    assert rel_err(host(gx), rdx) <= TOL and rel_err(host(gw), rdw) <= TOL and rel_err(host(gb), rdb) <= TOL
    gx2, gw2 = empty((B_, I)), empty((O, I))
    drv.fc_small_backward(gx2, gw2, None, dev(dy), dx_, dw_, B_, I, O, relu_data=dx_)
    np.testing.assert_array_equal(host(gx2), oracle.relu_backward(host(gx), x))
    np.testing.assert_array_equal(host(gw2), host(gw))       # run-to-run identical
    gw3 = empty((O, I))
    drv.fc_small_backward(None, gw3, None, dev(dy), dx_, dw_, B_, I, O)   # a first layer: no input gradient
    np.testing.assert_array_equal(host(gw3), host(gw))
    assert not drv.fc_small_supported(B_, I, 33) and not drv.fc_small_supported(1025, I, O)
    from caffecontroll_amd import CctHipError
    with pytest.raises(CctHipError):
        drv.fc_small_forward(y, dx_, dw_, db_, B_, I, 33)


def test_sgemm_new_fc_shapes(oracle):
    """The three sgemm_new calls of FullyConnectedBridge (LeNet ip1: 64 x 800 -> 500)."""
    B_, I, O = 64, 800, 500
    rng = np.random.default_rng(6)
    x = rng.standard_normal((B_, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((B_, O)).astype(np.float32)
    bias = rng.standard_normal(O).astype(np.float32)
    drv = driver()
    y = empty((B_, O))
    drv.sgemm_new(N_, T_, B_, O, I, 1.0, dev(x), dev(w), 0.0, y)
    drv.forward_bias(dev(bias), y, 1, O, B_)
    assert rel_err(host(y), oracle.fc_forward(x, w, bias)) <= TOL
    dx, dw, db = empty((B_, I)), empty((O, I)), empty((O,))
    drv.backward_bias_fc(db, dev(dy), O, B_)
    drv.sgemm_new(N_, N_, B_, I, O, 1.0, dev(dy), dev(w), 0.0, dx)
    drv.sgemm_new(T_, N_, O, I, B_, 1.0, dev(dy), dev(x), 0.0, dw)
    rdx, rdw, rdb = oracle.fc_backward(x, w, dy)
    assert rel_err(host(dx), rdx) <= TOL and rel_err(host(dw), rdw) <= TOL and rel_err(host(db), rdb) <= TOL


FC_FWD_SHAPES = [(64, 500, 800), (64, 10, 500), (256, 1000, 4096), (37, 53, 129), (130, 257, 64), (5, 3, 7)]


@pytest.mark.parametrize("shape", FC_FWD_SHAPES)
@pytest.mark.parametrize("bias,relu", [(True, False), (True, True), (False, True)])
def test_sgemm_new_bias_equals_the_separate_calls(shape, bias, relu):
    """The forward pass of FullyConnectedBridge in one call (sgemm_new + forward_bias over a 1x1
    feature map, src/bridges/FullyConnectedBridge_impl.hxx:224-228, + the in-place ReLU that may
    follow): bit-identical to the separate calls, whole tiles and ragged ones, with and without the
    split over the contraction."""
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N)
    drv = driver()
    X = dev(rng.standard_normal((M, K)).astype(np.float32))
    W = dev((rng.standard_normal((N, K)) * 0.1).astype(np.float32))
    b = dev(rng.standard_normal(N).astype(np.float32)) if bias else None
    sep, fused = empty((M, N)), empty((M, N))
    drv.sgemm_new(N_, T_, M, N, K, 1.0, X, W, 0.0, sep)
    if bias:
        drv.forward_bias(b, sep, 1, N, M)
    if relu:
        drv.relu_forward(sep, sep, M * N)
    drv.sgemm_new_bias(N_, T_, M, N, K, 1.0, X, W, 0.0, fused, b, relu)
    np.testing.assert_array_equal(host(fused), host(sep))
    if relu:
        assert (host(fused) >= 0).all() and (M * N < 100 or (host(fused) == 0).any())


def test_sgemv(oracle):
    rng = np.random.default_rng(7)
    M, N = 130, 70
    A = rng.standard_normal((M, N)).astype(np.float32)
    for TA, xl, yl in ((N_, N, M), (T_, M, N)):
        x = rng.standard_normal(xl).astype(np.float32)
        y0 = rng.standard_normal(yl).astype(np.float32)
        dy = dev(y0)
        driver().sgemv(TA, M, N, 2.0, dev(A), dev(x), 0.5, dy)
        ref = oracle.sgemv(TA, M, N, 2.0, A, x, 0.5, y0.copy())
        assert rel_err(host(dy), ref) <= 1e-5


def test_sgemm_rejects_bad_arguments():
    from caffecontroll_amd import CctHipError
    z = empty((16,), fill=0.0)
    with pytest.raises(CctHipError):
        driver().sgemm(RM, N_, N_, 4, 4, 4, 1.0, z, 3, z, 4, 0.0, z, 4)  # lda < K
    with pytest.raises(CctHipError):
        driver().sgemm(99, N_, N_, 4, 4, 4, 1.0, z, 4, z, 4, 0.0, z, 4)


# ---------------------------------------------------------------------------------------------
def conv_forward_gpu(x, w, bias, k, s, p, fused):
    """Driver-level restatement of ConvolutionBridge::forward's call sequence
    (src/bridges/ConvolutionBridge_impl.hxx:323-364); `fused` uses the single-GEMM epilogue."""
    from caffecontroll_amd.driver import conv_pmap, remap_pmap
    drv = driver()
    b, d, n, _ = x.shape
    o = w.shape[0]
    m = (n + 2 * p - k) // s + 1
    kkd, bmm = k * k * d, b * m * m
    dx, dw = dev(x), dev(w)
    dbias = None if bias is None else dev(bias)
    lowered = empty((bmm, kkd))
    drv.lower_cube(lowered, dx, conv_pmap(b, d, n, k, s, p))
    out = empty((b, o, m, m))
    if fused:
        drv.sgemm_conv_forward(o, b, m * m, kkd, dw, lowered, dbias, out)
        # with the ReLU of a following layer folded into the epilogue: max(x, 0) of the same result
        out_relu = empty((b, o, m, m))
        drv.sgemm_conv_forward(o, b, m * m, kkd, dw, lowered, dbias, out_relu, relu=True)
        np.testing.assert_array_equal(host(out_relu), np.maximum(host(out), np.float32(0)))
    else:
        tmp = empty((o, bmm))
        drv.sgemm(RM, N_, T_, o, bmm, kkd, 1.0, dw, kkd, lowered, kkd, 0.0, tmp, bmm)
        drv.remap(out, tmp, remap_pmap(m, m, o, b))
        if dbias is not None:
            drv.forward_bias(dbias, out, m * m, o, b)
    return out, lowered


def conv_backward_gpu(x_shape, w, og, lowered, k, s, p, need_in_grad=True):
    """Driver-level restatement of ConvolutionBridge::backward (…_impl.hxx:575-621) with the
    output-gradient permutation done out of place and the bias gradient fused into the lift."""
    from caffecontroll_amd.driver import lift_args, remap_pmap
    drv = driver()
    b, d, n, _ = x_shape
    o = w.shape[0]
    m = (n + 2 * p - k) // s + 1
    kkd, bmm = k * k * d, b * m * m
    dw_, dog = dev(w), dev(og)
    og_t = empty((o, bmm))
    drv.remap(og_t, dog, remap_pmap(m, m, b, o))
    db = empty((o,))
    dx = None
    if need_in_grad:
        lg = empty((kkd, bmm))
        drv.sgemm(RM, T_, N_, kkd, bmm, o, 1.0, dw_, kkd, og_t, bmm, 0.0, lg, bmm)
        dx = empty((b, d, n, n))
        drv.inverse_lower_cube_bias_backward(dx, lg, lift_args(b, d, n, k, s, p), db, dog, m * m, o, b)
    else:
        drv.backward_bias(db, dog, m * m, o, b)
    dwg = empty((o, kkd))
    drv.sgemm(RM, N_, N_, o, kkd, bmm, 1.0, og_t, bmm, lowered, kkd, 0.0, dwg, kkd)
    return dx, dwg, db


FIX = {
    "small": dict(b=4, d=3, n=20, k=5, s=4, p=2, o=10, sfx=""),
    "large": dict(b=4, d=3, n=127, k=11, s=4, p=2, o=8, sfx="_large"),
}


@pytest.mark.parametrize("case", ["small", "large"])
@pytest.mark.parametrize("fused", [False, True])
def test_conv_reference_fixtures(oracle, case, fused):
    """tests/test_parallelized_convolution.cpp:123-270 and ..._large_CPU.cpp on the GPU path."""
    c = FIX[case]
    sfx, k, s, p = c["sfx"], c["k"], c["s"], c["p"]
    x = load_fixture("input", f"conv_forward_in{sfx}.txt").reshape(c["b"], c["d"], c["n"], c["n"])
    wshape = (c["o"], c["d"], k, k)
    w_f = load_fixture("input", f"conv_model{sfx}.txt").reshape(wshape)
    w_b = load_fixture("input", f"conv_backward_model{sfx}.txt").reshape(wshape)
    bias = load_fixture("input", f"conv_bias_in{sfx}.txt")
    out, _ = conv_forward_gpu(x, w_f, bias, k, s, p, fused)
    exp = load_fixture("output", f"conv_forward{sfx}.txt").reshape(out.shape)
    got = host(out)
    np.testing.assert_allclose(got, exp, rtol=2e-5, atol=1e-3)
    ref, _ = oracle.conv_forward(x, w_f, bias, k, s, p)
    assert rel_err(got, ref) <= TOL
    if case == "small":
        # integer data: all partial sums are exact in fp32, any summation order gives these bits
        np.testing.assert_array_equal(got, ref)

    out2, lowered = conv_forward_gpu(x, w_b, bias, k, s, p, fused)
    og = (np.arange(out2.numel(), dtype=np.float64) * 0.1).astype(np.float32).reshape(out2.shape)
    dx, dw, db = conv_backward_gpu(x.shape, w_b, og, lowered, k, s, p)
    _, rlow = oracle.conv_forward(x, w_b, bias, k, s, p)
    rdx, rdw, rdb = oracle.conv_backward(x.shape, w_b, og, rlow, k, s, p)
    assert rel_err(host(dx), rdx) <= TOL and rel_err(host(dw), rdw) <= TOL and rel_err(host(db), rdb) <= TOL
    exp_dx = load_fixture("output", f"conv_backward{sfx}.txt")
    np.testing.assert_allclose(host(dx).reshape(-1)[:exp_dx.size], exp_dx, rtol=1e-4, atol=1e-3)
    # SGD step on device, then the golden weights / bias
    drv = driver()
    n_w = dw.numel()
    dmodel, hist = dev(w_b.reshape(-1)), empty((n_w,), fill=0.0)
    drv.sgd_update(n_w, dmodel, dw, hist, 0.01, 0.0)
    dbm, hist_b = dev(bias), empty((bias.size,), fill=0.0)
    drv.sgd_update(bias.size, dbm, db, hist_b, 0.01, 0.0)
    np.testing.assert_allclose(host(dmodel), load_fixture("output", f"conv_weights{sfx}.txt"), rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(host(dbm), load_fixture("output", f"conv_bias{sfx}.txt"), rtol=1e-4, atol=1e-3)


CONV_SHAPES = [  # b d n k s p o
    (64, 1, 28, 5, 1, 0, 20),   # benchmark configuration 1 (LeNet conv1), full size
    (8, 96, 27, 5, 1, 2, 256),  # benchmark configuration 2 geometry, batch 8
    (4, 3, 227, 11, 4, 0, 96),  # benchmark configuration 3 geometry, batch 4
    (16, 20, 12, 5, 1, 0, 50),  # LeNet conv2
    (4, 256, 13, 3, 1, 1, 384), # AlexNet conv3 geometry
]


@pytest.mark.parametrize("shape", CONV_SHAPES, ids=lambda s: "b%d_d%d_n%d_k%d_s%d_p%d_o%d" % s)
def test_conv_forward_backward_vs_oracle(oracle, shape):
    b, d, n, k, s, p, o = shape
    rng = np.random.default_rng(1234 + sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.01).astype(np.float32)
    bias = np.full(o, 0.1, np.float32)
    bound = oracle.bind_openblas(8)  # speed only; the naive loops give the same numbers to 1e-6
    try:
        ref, rlow = oracle.conv_forward(x, w, bias, k, s, p)
        og = rng.standard_normal(ref.shape).astype(np.float32)
        rdx, rdw, rdb = oracle.conv_backward(x.shape, w, og, rlow, k, s, p)
    finally:
        if bound:
            oracle.unbind_openblas()
    for fused in (False, True):
        out, lowered = conv_forward_gpu(x, w, bias, k, s, p, fused)
        np.testing.assert_array_equal(host(lowered), rlow)          # index layout: bit-exact
        assert rel_err(host(out), ref) <= TOL
    dx, dw, db = conv_backward_gpu(x.shape, w, og, lowered, k, s, p)
    assert rel_err(host(dx), rdx) <= TOL
    assert rel_err(host(dw), rdw) <= TOL
    assert rel_err(host(db), rdb) <= TOL
    # first layer of a net skips the data gradient (src/DeepNet.h:1108-1110)
    dx2, dw2, db2 = conv_backward_gpu(x.shape, w, og, lowered, k, s, p, need_in_grad=False)
    assert dx2 is None
    np.testing.assert_array_equal(host(dw2), host(dw))
    assert rel_err(host(db2), rdb) <= TOL


@pytest.mark.parametrize("shape", [(256, 96, 27, 5, 1, 2, 256), (256, 3, 227, 11, 4, 0, 96)],
                         ids=["alexnet_conv2", "alexnet_conv1"])
def test_full_size_conv_against_torch_fp64(shape):
    """benchmark configurations 2 and 3 at full size (b=256): forward output and all three gradients agree
    with float64 torch convolutions on the whole tensor (tolerance 1e-4 of the tensor's max)."""
    import torch
    import torch.nn.functional as F
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    g = torch.Generator(device="cuda").manual_seed(1236)
    x = torch.randn((b, d, n, n), device="cuda", generator=g)
    w = torch.randn((o, d, k, k), device="cuda", generator=g) * 0.01
    bias = torch.full((o,), 0.1, device="cuda")
    og = torch.randn((b, o, m, m), device="cuda", generator=g)
    out, lowered = conv_forward_gpu(host(x), host(w), host(bias), k, s, p, fused=True)
    dx, dw, db = conv_backward_gpu(tuple(x.shape), host(w), host(og), lowered, k, s, p)
    torch.cuda.synchronize()
    # float64 reference in image chunks to bound memory
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    b64 = bias.double().requires_grad_(True)
    ref = F.conv2d(x64, w64, b64, stride=s, padding=p)
    ref.backward(og.double())

    def err(a, r):
        return ((a.double() - r).abs().max() / r.abs().max()).item()

    assert err(out, ref.detach()) <= TOL
    assert err(dx, x64.grad) <= TOL
    assert err(dw.reshape(o, d, k, k), w64.grad) <= TOL
    assert err(db, b64.grad) <= TOL


@pytest.mark.parametrize("shape", [(64, 800, 500, 64, 500), (256, 4096, 4096, 256, 4096), (3, 5, 7, 9, 70),
                                   (128, 128, 64, 33, 129), (0, 5, 7, 4, 3)],
                         ids=lambda s: "m%d_n%d_k%d_rows%d_cols%d" % s)
def test_sgemm_new_with_column_sums(shape):
    """The product with the column sums of another matrix beside it (an inner-product layer's data gradient with its
    bias gradient): the product equals sgemm_new's and the sums equal backward_bias_fc's, bit for bit, whether the
    product's launch has a reduction to carry them or not."""
    M, N, K, rows, cols = shape
    drv = driver()
    rng = np.random.default_rng(sum(shape))
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    src = rng.standard_normal((rows, cols)).astype(np.float32)
    da, db, dsrc = dev(a), dev(b), dev(src)
    c0, c1 = empty((M, N), fill=float("nan")), empty((M, N), fill=float("nan"))
    s0, s1 = empty((cols,), fill=float("nan")), empty((cols,), fill=float("nan"))
    if M:
        drv.sgemm_new(111, 111, M, N, K, 1.0, da, db, 0.0, c0)
    drv.backward_bias_fc(s0, dsrc, cols, rows)
    drv.sgemm_new_colsum(111, 111, M, N, K, 1.0, da, db, 0.0, c1, s1, dsrc, rows, cols)
    assert np.array_equal(host(c0), host(c1), equal_nan=True)
    assert np.array_equal(host(s0), host(s1))
    assert rel_err(host(s1), src.astype(np.float64).sum(axis=0)) <= 1e-5
