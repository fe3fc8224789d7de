"""Strided convolution on the matrix cores without the lowered matrix (AlexNet / CaffeNet conv1:
11x11, stride 4; stride-2 layers with 7x7, 5x5 and 3x3 kernels) against the oracle's lowering
pipeline (lower_cube + GEMM + remap + bias, src/bridges/ConvolutionBridge_impl.hxx:316-364), the
reference's "large" golden scenario, and -- at the full size of benchmark configuration 3 -- float64
torch.  The sums run in another order than the lowered GEMM: agreement to 1e-4 of the tensor's
largest magnitude, bit-exact on small-integer tensors."""
import numpy as np
import pytest

from conftest import load_fixture
from gpu_util import dev, driver, empty, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4

# (b, d, n, k, s, p, o)
SHAPES = [
    (4, 3, 127, 11, 4, 2, 8),      # the reference's large fixture
    (3, 3, 227, 11, 4, 0, 96),     # conv1 geometry, small batch: tiles that straddle two images
    (2, 3, 51, 11, 4, 0, 40),      # two map blocks with padding maps
    (5, 2, 35, 11, 4, 5, 33),      # heavy padding, odd sizes
    (2, 4, 30, 7, 2, 3, 20),       # stride 2
    (3, 5, 17, 5, 2, 2, 64),
    (4, 6, 13, 3, 2, 1, 70),
    (1, 1, 11, 11, 4, 0, 1),       # a single output pixel
    (2, 4, 31, 7, 2, 0, 20),       # no padding: the lanes fetch the source themselves
    (3, 5, 17, 5, 2, 0, 64),
    (4, 6, 13, 3, 2, 0, 70),
    (2, 1, 43, 11, 4, 0, 97),      # one channel, four map blocks
]
# long output rows: the weight gradient takes a row in pieces (the data-gradient kernel does not cover these)
LONG_ROWS = [
    (1, 3, 500, 11, 4, 0, 8),
    (2, 2, 300, 7, 2, 0, 12),
    (1, 2, 401, 5, 2, 0, 9),
    (1, 2, 600, 3, 2, 0, 5),
    (1, 2, 300, 7, 2, 3, 12),      # padded
    (1, 1, 2000, 11, 4, 0, 4),     # 498-pixel output rows
]
_ids = lambda s: "b%d_d%d_n%d_k%d_s%d_p%d_o%d" % s


def _forward(drv, x, w, bias, shape, relu=False):
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    slabs = empty((drv.conv_strided_slab_floats(o, d, k, s, p),))
    drv.conv_strided_slabs(slabs, dev(w), o, d, k, s, p)
    out = empty((b, o, m, m))
    drv.conv_strided_forward(out, dev(x), slabs, None if bias is None else dev(bias), b, d, n, k, s, p, o, relu=relu)
    return host(out)


@pytest.mark.parametrize("shape", SHAPES + LONG_ROWS, ids=_ids)
def test_strided_forward_vs_oracle(oracle, shape):
    b, d, n, k, s, p, o = shape
    drv = driver()
    assert drv.conv_strided_supported(*shape)
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    ref, _ = oracle.conv_forward(x, w, bias, k, s, p)
    got = _forward(drv, x, w, bias, shape)
    assert rel_err(got, ref) <= TOL
    # without bias, with the ReLU of a following layer folded in
    ref0, _ = oracle.conv_forward(x, w, None, k, s, p)
    got0 = _forward(drv, x, w, None, shape, relu=True)
    assert rel_err(got0, np.maximum(ref0, 0)) <= TOL
    # small integers: every product and partial sum is exact, whatever the order
    xi = rng.integers(-4, 5, size=x.shape).astype(np.float32)
    wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    bi = rng.integers(-5, 6, size=o).astype(np.float32)
    refi, _ = oracle.conv_forward(xi, wi, bi, k, s, p)
    np.testing.assert_array_equal(_forward(drv, xi, wi, bi, shape), refi)


def test_strided_forward_reference_large_fixture():
    """tests/test_parallelized_convolution_large_CPU.cpp:71-80: b=4 d=3 n=127 k=11 s=4 p=2 o=8."""
    shape = (4, 3, 127, 11, 4, 2, 8)
    b, d, n, k, s, p, o = shape
    x = load_fixture("input", "conv_forward_in_large.txt").reshape(b, d, n, n)
    w = load_fixture("input", "conv_model_large.txt").reshape(o, d, k, k)
    bias = load_fixture("input", "conv_bias_in_large.txt")
    got = _forward(driver(), x, w, bias, shape)
    np.testing.assert_allclose(got.reshape(-1), load_fixture("output", "conv_forward_large.txt"), rtol=2e-5, atol=1e-3)


def test_strided_forward_full_config3_vs_float64():
    """benchmark configuration 3 at full size (batch 256, 3x227x227, 96 filters 11x11, stride 4) against
    torch conv2d in float64."""
    import torch
    shape = (256, 3, 227, 11, 4, 0, 96)
    b, d, n, k, s, p, o = shape
    rng = np.random.default_rng(3)
    x = rng.uniform(0, 255, (b, d, n, n)).astype(np.float32)
    x -= np.array([104, 117, 123], np.float32)[None, :, None, None]
    w = (rng.standard_normal((o, d, k, k)) * 0.01).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    got = _forward(driver(), x, w, bias, shape)
    ref = torch.nn.functional.conv2d(torch.from_numpy(x).cuda().double(), torch.from_numpy(w).cuda().double(),
                                     torch.from_numpy(bias).cuda().double(), stride=s, padding=p).cpu().numpy()
    assert rel_err(got, ref) <= TOL


@pytest.mark.parametrize("shape", SHAPES + LONG_ROWS, ids=_ids)
def test_strided_backward_weights_vs_oracle(oracle, shape):
    """Weight and bias gradient against the oracle's remap + weight-gradient GEMM on the lowered matrix
    (src/bridges/ConvolutionBridge_impl.hxx:575-604, 619-621)."""
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    drv = driver()
    rng = np.random.default_rng(sum(shape) + 1)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    _, lowered = oracle.conv_forward(x, w, None, k, s, p)
    _, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, k, s, p, need_in_grad=False)
    d_x, d_og = dev(x), dev(og)
    dw, db = empty((o, d, k, k)), empty((o,))
    drv.conv_strided_backward_weights(dw, db, d_og, d_x, b, d, n, k, s, p, o)
    assert rel_err(host(dw), ref_dw) <= TOL
    assert rel_err(host(db), ref_db) <= TOL
    assert rel_err(host(db), og.astype(np.float64).sum(axis=(0, 2, 3))) <= TOL
    np.testing.assert_array_equal(host(d_og), og)  # the output gradient is read in place, not permuted
    # partial sums are added in a fixed order: a second run gives the same bits, with or without the bias gradient
    dw2 = empty((o, d, k, k))
    drv.conv_strided_backward_weights(dw2, None, d_og, d_x, b, d, n, k, s, p, o)
    np.testing.assert_array_equal(host(dw2), host(dw))
    # small integers: every product and partial sum is exact, whatever the order
    xi = rng.integers(-4, 5, size=x.shape).astype(np.float32)
    ogi = rng.integers(-3, 4, size=og.shape).astype(np.float32)
    _, lowered_i = oracle.conv_forward(xi, w, None, k, s, p)
    _, refi_dw, refi_db = oracle.conv_backward(x.shape, w, ogi, lowered_i, k, s, p, need_in_grad=False)
    drv.conv_strided_backward_weights(dw, db, dev(ogi), dev(xi), b, d, n, k, s, p, o)
    np.testing.assert_array_equal(host(dw).reshape(-1), np.asarray(refi_dw).reshape(-1))
    np.testing.assert_array_equal(host(db), refi_db)


def test_strided_backward_weights_reference_large_fixture():
    """tests/test_parallelized_convolution_large_CPU.cpp:71-80, backward: weights after one SGD step with
    learning rate 0.01 (W - 0.01 dW, b - 0.01 db), output gradient 0.1 * i."""
    shape = (4, 3, 127, 11, 4, 2, 8)
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    x = load_fixture("input", "conv_forward_in_large.txt").reshape(b, d, n, n)
    w = load_fixture("input", "conv_backward_model_large.txt").reshape(o, d, k, k)
    bias = load_fixture("input", "conv_bias_in_large.txt")
    og = (0.1 * np.arange(b * o * m * m, dtype=np.float64)).astype(np.float32).reshape(b, o, m, m)
    drv = driver()
    dw, db = empty((o, d, k, k)), empty((o,))
    drv.conv_strided_backward_weights(dw, db, dev(og), dev(x), b, d, n, k, s, p, o)
    want_w = load_fixture("output", "conv_weights_large.txt")
    want_b = load_fixture("output", "conv_bias_large.txt")
    got_w = (w - np.float32(0.01) * host(dw)).reshape(-1)
    got_b = bias - np.float32(0.01) * host(db)
    np.testing.assert_allclose(got_w, want_w, rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(got_b, want_b, rtol=1e-4, atol=1e-3)


def test_strided_backward_weights_full_config3_vs_float64():
    """benchmark configuration 3 at full size against float64 torch (weight gradient in chunks of 32 images)."""
    import torch
    shape = (256, 3, 227, 11, 4, 0, 96)
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    g = torch.Generator(device="cuda").manual_seed(1237)
    x = torch.rand((b, d, n, n), device="cuda", generator=g) * 255 - 115
    og = torch.randn((b, o, m, m), device="cuda", generator=g)
    dw, db = empty((o, d, k, k)), empty((o,))
    driver().conv_strided_backward_weights(dw, db, og, x, b, d, n, k, s, p, o)
    torch.cuda.synchronize()
    ref = torch.zeros((o, d, k, k), dtype=torch.float64, device="cuda")
    for i in range(0, b, 32):
        ref += torch.nn.grad.conv2d_weight(x[i:i + 32].double(), (o, d, k, k), og[i:i + 32].double(), stride=s, padding=p)
    assert ((dw.double() - ref).abs().max() / ref.abs().max()).item() <= TOL
    db_ref = og.double().sum(dim=(0, 2, 3))
    assert ((db.double() - db_ref).abs().max() / db_ref.abs().max()).item() <= TOL


# data gradient: depth * stride^2 maps must come as 1, 3 or 5 blocks of 16 (the 16-row kernel)
# (and the output gradient must be large enough that a 128-pixel tile does not span dozens of images)
DGRAD_SHAPES = [s for s in SHAPES if ((s[1] * s[4] * s[4] + 15) // 16) in (1, 3, 5) and (s[2] + 2 * s[5] - s[3]) // s[4] >= 2] + [
    (3, 3, 61, 11, 4, 0, 20),      # 227-style geometry, smaller: rows left over by the floor division (61 = 4*12 + 13)
    (2, 3, 40, 11, 4, 3, 9),       # padding 3
    (2, 1, 29, 5, 2, 0, 7),        # one channel, stride 2
]


@pytest.mark.parametrize("shape", DGRAD_SHAPES, ids=_ids)
def test_strided_backward_data_vs_oracle(oracle, shape):
    """Input gradient against the oracle's remap + data-gradient GEMM + inverse_lower_cube
    (src/bridges/ConvolutionBridge_impl.hxx:604-616)."""
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    drv = driver()
    assert drv.conv_strided_backward_data_supported(*shape)
    rng = np.random.default_rng(sum(shape) + 2)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    _, lowered = oracle.conv_forward(x, w, None, k, s, p)
    ref_dx, _, _ = oracle.conv_backward(x.shape, w, og, lowered, k, s, p)
    slabs = empty((drv.conv_strided_backward_data_slab_floats(o, d, k, s),))
    drv.conv_strided_backward_data_slabs(slabs, dev(w), o, d, k, s)
    d_og = dev(og)
    dx = empty((b, d, n, n))
    drv.conv_strided_backward_data(dx, d_og, slabs, b, d, n, k, s, p, o)
    assert rel_err(host(dx), ref_dx) <= TOL       # every element written (the buffer starts as NaN)
    np.testing.assert_array_equal(host(d_og), og)  # the output gradient is read in place, not permuted
    # small integers: exact in any order
    wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
    ogi = rng.integers(-3, 4, size=og.shape).astype(np.float32)
    refi_dx, _, _ = oracle.conv_backward(x.shape, wi, ogi, lowered, k, s, p)
    drv.conv_strided_backward_data_slabs(slabs, dev(wi), o, d, k, s)
    drv.conv_strided_backward_data(dx, dev(ogi), slabs, b, d, n, k, s, p, o)
    np.testing.assert_array_equal(host(dx), refi_dx)


def test_strided_backward_data_reference_large_fixture():
    """tests/test_parallelized_convolution_large_CPU.cpp:71-80, backward: input gradient for the output gradient 0.1 * i."""
    shape = (4, 3, 127, 11, 4, 2, 8)
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    w = load_fixture("input", "conv_backward_model_large.txt").reshape(o, d, k, k)
    og = (0.1 * np.arange(b * o * m * m, dtype=np.float64)).astype(np.float32).reshape(b, o, m, m)
    drv = driver()
    slabs = empty((drv.conv_strided_backward_data_slab_floats(o, d, k, s),))
    drv.conv_strided_backward_data_slabs(slabs, dev(w), o, d, k, s)
    dx = empty((b, d, n, n))
    drv.conv_strided_backward_data(dx, dev(og), slabs, b, d, n, k, s, p, o)
    want = load_fixture("output", "conv_backward_large.txt")
    np.testing.assert_allclose(host(dx).reshape(-1)[:want.size], want, rtol=1e-4, atol=1e-3)


def test_strided_backward_data_full_config3_vs_float64():
    """benchmark configuration 3 at full size against float64 torch, in chunks of 32 images."""
    import torch
    shape = (256, 3, 227, 11, 4, 0, 96)
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    g = torch.Generator(device="cuda").manual_seed(1238)
    w = torch.randn((o, d, k, k), device="cuda", generator=g) * 0.01
    og = torch.randn((b, o, m, m), device="cuda", generator=g)
    drv = driver()
    slabs = empty((drv.conv_strided_backward_data_slab_floats(o, d, k, s),))
    drv.conv_strided_backward_data_slabs(slabs, w, o, d, k, s)
    dx = empty((b, d, n, n))
    drv.conv_strided_backward_data(dx, og, slabs, b, d, n, k, s, p, o)
    torch.cuda.synchronize()
    worst = scale = 0.0
    for i in range(0, b, 32):
        ref = torch.nn.grad.conv2d_input((min(32, b - i), d, n, n), w.double(), og[i:i + 32].double(), stride=s, padding=p)
        worst = max(worst, (dx[i:i + 32].double() - ref).abs().max().item())
        scale = max(scale, ref.abs().max().item())
    assert worst / scale <= TOL


def test_unsupported_geometries_are_refused():
    from caffecontroll_amd import CctHipError
    drv = driver()
    assert not drv.conv_strided_supported(2, 3, 30, 11, 3, 0, 8)     # stride 3
    assert not drv.conv_strided_supported(2, 3, 30, 9, 4, 0, 8)      # no 9x9 instance
    assert not drv.conv_strided_supported(2, 3, 2000, 11, 4, 2, 8)   # padded rows too long for the LDS patch
    assert drv.conv_strided_supported(2, 3, 9000, 11, 4, 0, 8)       # long rows: the weight gradient takes them in pieces
    assert not drv.conv_strided_supported(2, 3, 12000, 11, 4, 0, 8)  # more than its 64 pieces
    with pytest.raises(CctHipError, match="not covered"):
        drv.conv_strided_forward(empty((4,)), empty((4,)), empty((4,)), None, 2, 3, 30, 11, 3, 0, 8)
