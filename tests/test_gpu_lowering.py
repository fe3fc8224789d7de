"""GPU parity: lowering, lifting, remap and bias kernels against the CPU oracle (bit-exact for the
index/copy work and for the order-preserving lift), plus full-size AlexNet-conv2 properties."""
import numpy as np
import pytest

from gpu_util import dev, driver, empty, host, rel_err

pytestmark = pytest.mark.gpu

# b d n k s p
SHAPES = [
    (64, 1, 28, 5, 1, 0),     # LeNet conv1 (benchmark configuration 1)
    (4, 3, 20, 5, 4, 2),      # reference small fixture shape
    (4, 3, 127, 11, 4, 2),    # reference large fixture shape
    (3, 96, 27, 5, 1, 2),     # AlexNet conv2 geometry, small batch (vector-store path, 2-row bands)
    (2, 3, 227, 11, 4, 0),    # AlexNet conv1 geometry
    (2, 20, 12, 5, 1, 0),     # LeNet conv2
    (2, 256, 13, 3, 1, 1),    # AlexNet conv3 geometry (channel slabs)
    (1, 7, 9, 3, 2, 1), (2, 5, 8, 1, 1, 0), (1, 2, 6, 6, 1, 0), (1, 9, 10, 3, 3, 2), (5, 4, 7, 4, 2, 3),
    (5, 1, 7, 1, 1, 0), (3, 2, 9, 1, 2, 0), (2, 3, 6, 1, 1, 0),   # lowered rows of one, two and three floats
]


def _ids(s):
    return "b%d_d%d_n%d_k%d_s%d_p%d" % s


@pytest.mark.parametrize("shape", SHAPES, ids=_ids)
def test_lower_cube_bit_exact(oracle, shape):
    from caffecontroll_amd.driver import conv_pmap
    b, d, n, k, s, p = shape
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    dst = empty((b * m * m, k * k * d))
    driver().lower_cube(dst, dev(x), conv_pmap(b, d, n, k, s, p))
    np.testing.assert_array_equal(host(dst), oracle.lower_cube(x, k, s, p))


@pytest.mark.parametrize("shape", SHAPES, ids=_ids)
def test_inverse_lower_cube_bit_exact(oracle, shape):
    from caffecontroll_amd.driver import lift_args
    b, d, n, k, s, p = shape
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(sum(shape) + 1)
    y = rng.standard_normal((k * k * d, b * m * m)).astype(np.float32)
    dst = empty((b, d, n, n))
    driver().inverse_lower_cube(dst, dev(y), lift_args(b, d, n, k, s, p))
    np.testing.assert_array_equal(host(dst), oracle.inverse_lower_cube(y, b, d, n, k, s, p))


@pytest.mark.parametrize("shape", [SHAPES[1], SHAPES[3], SHAPES[5]], ids=_ids)
def test_lift_fused_with_bias_gradient(oracle, shape):
    from caffecontroll_amd.driver import lift_args
    b, d, n, k, s, p = shape
    o = 10
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(77)
    y = rng.standard_normal((k * k * d, b * m * m)).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    dst, db = empty((b, d, n, n)), empty((o,))
    driver().inverse_lower_cube_bias_backward(dst, dev(y), lift_args(b, d, n, k, s, p), db, dev(og),
                                              m * m, o, b)
    np.testing.assert_array_equal(host(dst), oracle.inverse_lower_cube(y, b, d, n, k, s, p))
    ref = oracle.bias_backward(og, m * m, o, b)
    exact = og.astype(np.float64).sum(axis=(0, 2, 3))
    # tolerance 1e-4 relative to the largest gradient; both must also agree with float64
    assert rel_err(host(db), ref) <= 1e-4
    assert rel_err(host(db), exact) <= 1e-4
    # standalone entry point gives the same numbers as the fused launch
    db2 = empty((o,))
    driver().backward_bias(db2, dev(og), m * m, o, b)
    np.testing.assert_array_equal(host(db2), host(db))


@pytest.mark.parametrize("dims", [(5, 5, 10, 4), (27, 27, 16, 3), (1, 1, 7, 5), (24, 24, 20, 2), (3, 2, 1, 4)])
def test_remap_bit_exact(oracle, dims):
    from caffecontroll_amd.driver import remap_pmap
    R, Cc, depth, batch = dims
    rng = np.random.default_rng(3)
    x = rng.standard_normal((depth * batch, R, Cc)).astype(np.float32)
    dst = empty(x.shape)
    driver().remap(dst, dev(x), remap_pmap(R, Cc, depth, batch))
    np.testing.assert_array_equal(host(dst), oracle.remap(x, R, Cc, depth, batch))


@pytest.mark.parametrize("dims", [(5, 5, 4, 10), (55, 55, 3, 6), (1, 1, 7, 5), (70, 70, 2, 3), (3, 2, 1, 1)])
def test_remap_with_bias_gradient(oracle, dims):
    """The backward remap of a convolution ([image][map] -> [map][image] slices) that also sums each
    map's slices: the copy is bit-exact, the sums agree with the oracle's bias gradient and with
    float64 within the fp32 tolerance, and a second run gives the same bits."""
    from caffecontroll_amd.driver import remap_pmap
    R, Cc, images, maps = dims
    rng = np.random.default_rng(17 + sum(dims))
    x = rng.standard_normal((images, maps, R, Cc)).astype(np.float32)
    dst, bias = empty(x.shape), empty((maps,))
    driver().remap_bias_backward(dst, dev(x), remap_pmap(R, Cc, images, maps), bias)
    np.testing.assert_array_equal(host(dst).reshape(-1), oracle.remap(x.reshape(images * maps, R, Cc), R, Cc, images, maps).reshape(-1))
    ref = oracle.bias_backward(x, R * Cc, maps, images)
    scale = max(np.abs(ref).max(), 1.0)
    assert np.abs(host(bias) - ref).max() / scale <= 1e-4
    assert np.abs(host(bias) - x.astype(np.float64).sum(axis=(0, 2, 3))).max() / scale <= 1e-4
    bias2 = empty((maps,))
    driver().remap_bias_backward(empty(x.shape), dev(x), remap_pmap(R, Cc, images, maps), bias2)
    np.testing.assert_array_equal(host(bias2), host(bias))


def test_remap_rejects_overlap():
    from caffecontroll_amd import CctHipError
    from caffecontroll_amd.driver import remap_pmap
    buf = empty((4 * 3 * 9,), fill=0.0)
    with pytest.raises(CctHipError):
        driver().remap(buf, buf, remap_pmap(3, 3, 4, 3))


def test_forward_bias(oracle):
    rng = np.random.default_rng(8)
    b, o, fmap = 5, 7, 33
    out = rng.standard_normal((b, o, fmap)).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    d_out = dev(out)
    driver().forward_bias(dev(bias), d_out, fmap, o, b)
    np.testing.assert_array_equal(host(d_out), oracle.bias_forward(out.copy(), bias, fmap, o, b))


def test_lower_rejects_non_square():
    from caffecontroll_amd import CctHipError
    from caffecontroll_amd.driver import conv_pmap
    a = conv_pmap(1, 1, 8, 3, 1, 0)
    a.sC = 9
    with pytest.raises(CctHipError):
        driver().lower_cube(empty((36, 9)), empty((1, 1, 8, 9), fill=0.0), a)


def test_empty_batch_is_a_no_op():
    from caffecontroll_amd.driver import conv_pmap
    driver().lower_cube(empty((1,)), empty((1,)), conv_pmap(0, 3, 8, 3, 1, 0))
    driver().device_sync()


# ---------------------------------------------------------------------------------------------
# Full AlexNet-conv2 size (benchmark configuration 2): properties that do not need the slow CPU oracle.
CFG2 = (256, 96, 27, 5, 1, 2)


CFG3 = (256, 3, 227, 11, 4, 0)


@pytest.mark.parametrize("cfg", [CFG2, CFG3], ids=["alexnet_conv2", "alexnet_conv1"])
def test_full_size_lower_matches_unfold_and_adjoint(cfg):
    """At the full benchmark sizes (config 2: b=256,d=96,n=27,k=5,p=2; config 3: b=256,d=3,n=227,
    k=11,s=4): (i) the lowered matrix equals torch's unfold (an independent im2col) bit for bit;
    (ii) lift(lower(x)) == x * multiplicity; (iii) <lower(x),y> == <x,lift(y)> in float64 within
    rounding."""
    import torch
    import torch.nn.functional as F
    from caffecontroll_amd.driver import conv_pmap, lift_args
    b, d, n, k, s, p = cfg
    m = (n + 2 * p - k) // s + 1
    g = torch.Generator(device="cuda").manual_seed(1235)
    x = torch.randn((b, d, n, n), device="cuda", generator=g)
    low = empty((b * m * m, k * k * d))
    driver().lower_cube(low, x, conv_pmap(b, d, n, k, s, p))
    ref = F.unfold(x, k, padding=p, stride=s)          # [b][d*k*k][m*m]
    ref = ref.transpose(1, 2).reshape(b * m * m, d * k * k)
    assert torch.equal(low, ref)
    del ref
    # (ii) multiplicity: lifting an all-ones lowered matrix counts the windows covering each pixel
    ones_t = torch.ones((k * k * d, b * m * m), device="cuda")
    mult = empty((b, d, n, n))
    driver().inverse_lower_cube(mult, ones_t, lift_args(b, d, n, k, s, p))
    # lowered matrix transposed into the lift's [k*k*d][b*m*m] layout
    low_t = low.t().contiguous()
    back = empty((b, d, n, n))
    driver().inverse_lower_cube(back, low_t, lift_args(b, d, n, k, s, p))
    torch.cuda.synchronize()
    assert torch.allclose(back, x * mult, rtol=1e-5, atol=1e-5)
    if cfg == CFG2:
        assert int(mult.max().item()) == k * k and int(mult.min().item()) == 9  # corners see 3x3 windows
    else:
        # stride 4, kernel 11: a pixel is covered by at most ceil(11/4)^2 = 9 windows, corners by one
        assert int(mult.max().item()) == 9 and int(mult.min().item()) == 1
    # (iii) adjoint identity with a random y
    y = torch.randn((k * k * d, b * m * m), device="cuda", generator=g)
    lift_y = empty((b, d, n, n))
    driver().inverse_lower_cube(lift_y, y, lift_args(b, d, n, k, s, p))
    lhs = (low_t.double() * y.double()).sum().item()
    rhs = (x.double() * lift_y.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-6 * (low_t.double().abs() * y.double().abs()).sum().item()
