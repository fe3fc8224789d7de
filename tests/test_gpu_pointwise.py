"""1 x 1 convolutions (stride 1, no padding) as products on the tensors as they lie -- forward and data
gradient one product per image in one launch, weight gradient one product summed over the images --
against the CPU oracle's lowering pipeline (lower_cube with k = 1 + GEMM + remap + bias,
src/bridges/ConvolutionBridge_impl.hxx:294-373, 551-628), through the C ABI and through the bridge."""
import numpy as np
import pytest

from gpu_util import driver, dev, empty, host, rel_err, tuning

pytestmark = pytest.mark.gpu
TOL = 1e-4

# (b, d, n, o)
SHAPES = [
    (4, 64, 13, 96),      # 169 pixels: not a multiple of four (operands staged through registers)
    (3, 16, 8, 32),       # everything a multiple of 16: operands straight into LDS
    (2, 160, 28, 64),     # 784 pixels
    (5, 3, 7, 5),         # tiny: one partial tile
    (1, 33, 31, 129),     # one image, odd everything
    (64, 32, 4, 48),      # many small images: the weight gradient sums groups of them per slice
    (2, 8, 60, 20),       # 3600 pixels per map
    (7, 130, 6, 70),
]
_ids = lambda s: "b%d_d%d_n%d_o%d" % s


def _tensors(shape, seed):
    b, d, n, o = shape
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, 1, 1)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    og = rng.standard_normal((b, o, n, n)).astype(np.float32)
    return x, w, bias, og


@pytest.mark.parametrize("per_image", [1, 2], ids=["per_image", "across_images"])
@pytest.mark.parametrize("shape", SHAPES + [(3, 5, 1, 7), (9, 16, 2, 32)], ids=_ids)
def test_forward_and_data_gradient_in_both_forms(oracle, shape, per_image):
    """Forward and data gradient as one product per image and as one product whose columns run over the pixels of
    all images (planes that are not a multiple of four floats: vectors that straddle two images; planes shorter than
    a vector keep one product per image whatever the knob says)."""
    b, d, n, o = shape
    x, w, bias, og = _tensors(shape, 7 + sum(shape))
    drv = driver()
    ref_out, lowered = oracle.conv_forward(x, w, bias, 1, 1, 0)
    ref_dx, _, _ = oracle.conv_backward(x.shape, w, og, lowered, 1, 1, 0)
    out, dx = empty((b, o, n, n), fill=float("nan")), empty((b, d, n, n), fill=float("nan"))
    with tuning("conv1x1_per_image", per_image):
        drv.conv1x1_forward(out, dev(x), dev(w), dev(bias), b, d, n * n, o)
        drv.conv1x1_backward_data(dx, dev(og), dev(w), b, d, n * n, o)
    assert rel_err(host(out), ref_out) <= TOL
    assert rel_err(host(dx), ref_dx) <= TOL


@pytest.mark.parametrize("shape", SHAPES, ids=_ids)
def test_pointwise_products_match_oracle(oracle, shape):
    b, d, n, o = shape
    x, w, bias, og = _tensors(shape, 99 + sum(shape))
    drv = driver()
    assert drv.conv1x1_supported(b, d, n, 1, 1, 0, o)
    ref_out, lowered = oracle.conv_forward(x, w, bias, 1, 1, 0)
    ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, 1, 1, 0)
    d_x, d_w, d_og, d_bias = dev(x), dev(w), dev(og), dev(bias)

    out = empty((b, o, n, n))
    drv.conv1x1_forward(out, d_x, d_w, d_bias, b, d, n * n, o)
    assert rel_err(host(out), ref_out) <= TOL
    # without bias, with the ReLU of a following layer folded in
    ref0, _ = oracle.conv_forward(x, w, None, 1, 1, 0)
    out0 = empty((b, o, n, n))
    drv.conv1x1_forward(out0, d_x, d_w, None, b, d, n * n, o, relu=True)
    assert rel_err(host(out0), np.maximum(ref0, 0)) <= TOL
    # against a float64 einsum as well: the oracle's k = 1 lowering is the identity it should be
    want = np.einsum("oc,bcp->bop", w.reshape(o, d).astype(np.float64), x.reshape(b, d, n * n).astype(np.float64))
    assert rel_err(host(out0), np.maximum(want, 0).reshape(b, o, n, n)) <= TOL

    dx = empty((b, d, n, n))
    drv.conv1x1_backward_data(dx, d_og, d_w, b, d, n * n, o)
    assert rel_err(host(dx), ref_dx) <= TOL

    dw, db = empty((o, d, 1, 1)), empty((o,))
    drv.conv1x1_backward_weights(dw, d_og, d_x, b, d, n * n, o, db=db)
    assert rel_err(host(dw), np.asarray(ref_dw).reshape(o, d, 1, 1)) <= TOL
    assert rel_err(host(db), ref_db) <= TOL
    # partial sums are added in a fixed order: a second run gives the same bits, with or without the bias gradient
    dw2 = empty((o, d, 1, 1))
    drv.conv1x1_backward_weights(dw2, d_og, d_x, b, d, n * n, o)
    np.testing.assert_array_equal(host(dw2), host(dw))
    # nothing but the outputs was written
    np.testing.assert_array_equal(host(d_x), x)
    np.testing.assert_array_equal(host(d_og), og)
    np.testing.assert_array_equal(host(d_w), w)


def test_pointwise_small_integers_are_exact():
    """Small integers: every product and partial sum is exact in fp32, whatever the order of the sums."""
    b, d, n, o = 6, 40, 9, 24
    rng = np.random.default_rng(5)
    x = rng.integers(-3, 4, (b, d, n, n)).astype(np.float32)
    w = rng.integers(-3, 4, (o, d)).astype(np.float32)
    og = rng.integers(-3, 4, (b, o, n, n)).astype(np.float32)
    drv = driver()
    out, dx, dw, db = empty((b, o, n, n)), empty((b, d, n, n)), empty((o, d)), empty((o,))
    drv.conv1x1_forward(out, dev(x), dev(w), None, b, d, n * n, o)
    drv.conv1x1_backward_data(dx, dev(og), dev(w), b, d, n * n, o)
    drv.conv1x1_backward_weights(dw, dev(og), dev(x), b, d, n * n, o, db=db)
    x2, og2 = x.reshape(b, d, -1), og.reshape(b, o, -1)
    np.testing.assert_array_equal(host(out).reshape(b, o, -1), np.einsum("oc,bcp->bop", w, x2))
    np.testing.assert_array_equal(host(dx).reshape(b, d, -1), np.einsum("oc,bop->bcp", w, og2))
    np.testing.assert_array_equal(host(dw), np.einsum("bop,bcp->oc", og2, x2))
    np.testing.assert_array_equal(host(db), og2.sum(axis=(0, 2)))


def test_pointwise_full_size_vs_float64():
    """A 256 -> 256 layer on 28 x 28 maps at batch 64 against torch in float64."""
    import torch
    b, d, n, o = 64, 256, 28, 256
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn((b, d, n, n), device="cuda", generator=g)
    w = torch.randn((o, d, 1, 1), device="cuda", generator=g) * 0.05
    bias = torch.randn((o,), device="cuda", generator=g)
    og = torch.randn((b, o, n, n), device="cuda", generator=g)
    drv = driver()
    out, dx, dw, db = empty((b, o, n, n)), empty((b, d, n, n)), empty((o, d, 1, 1)), empty((o,))
    drv.conv1x1_forward(out, x, w, bias, b, d, n * n, o)
    drv.conv1x1_backward_data(dx, og, w, b, d, n * n, o)
    drv.conv1x1_backward_weights(dw, og, x, b, d, n * n, o, db=db)
    torch.cuda.synchronize()
    x64, w64, og64 = x.double(), w.double(), og.double()
    ref = torch.nn.functional.conv2d(x64, w64, bias.double())
    assert ((out.double() - ref).abs().max() / ref.abs().max()).item() <= TOL
    ref = torch.nn.grad.conv2d_input(x.shape, w64, og64)
    assert ((dx.double() - ref).abs().max() / ref.abs().max()).item() <= TOL
    ref = torch.nn.grad.conv2d_weight(x64, w.shape, og64)
    assert ((dw.double() - ref).abs().max() / ref.abs().max()).item() <= TOL
    ref = og64.sum(dim=(0, 2, 3))
    assert ((db.double() - ref).abs().max() / ref.abs().max()).item() <= TOL


def test_pointwise_support_and_errors():
    from caffecontroll_amd import CctHipError
    drv = driver()
    assert drv.conv1x1_supported(4, 3, 20, 1, 1, 0, 10)
    assert not drv.conv1x1_supported(4, 3, 20, 1, 2, 0, 10)   # stride 2
    assert not drv.conv1x1_supported(4, 3, 20, 1, 1, 1, 10)   # padding
    assert not drv.conv1x1_supported(4, 3, 20, 3, 1, 0, 10)   # k = 3
    with pytest.raises(CctHipError):
        drv.conv1x1_forward(empty((4,)), empty((4,)), None, None, 1, 2, 2, 1)
    with pytest.raises(CctHipError):
        drv.conv1x1_backward_data(empty((4,)), empty((4,)), empty((4,)), 1, 0, 2, 1)
    # an empty batch: nothing to do forward, zero gradients backward
    dw, db = empty((6,)), empty((3,))
    drv.conv1x1_forward(empty((4,)), empty((4,)), empty((6,)), None, 0, 2, 4, 3)
    drv.conv1x1_backward_weights(dw, empty((4,)), empty((4,)), 0, 2, 4, 3, db=db)
    assert not host(dw).any() and not host(db).any()
    with pytest.raises(CctHipError):   # an empty batch does not excuse a bad layer shape
        drv.conv1x1_backward_weights(dw, empty((4,)), empty((4,)), 0, -2, 4, 3)


@pytest.mark.parametrize("shape", [(4, 64, 13, 96), (3, 16, 8, 32), (9, 20, 30, 7)], ids=_ids)
def test_bridge_runs_pointwise_layers_without_lowering(oracle, shape):
    """ConvolutionBridge on a 1 x 1 layer: level 3 by default (no lowered matrix is ever allocated), level 1 and 0
    the lowering path; all within 1e-4 of the oracle's ConvolutionBridge."""
    from caffecontroll_amd.bridges import ConvolutionLayer
    b, d, n, o = shape
    x, w, bias, og = _tensors(shape, 31 + sum(shape))
    ref_out, lowered = oracle.conv_forward(x, w, bias, 1, 1, 0)
    ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, 1, 1, 0)
    drv = driver()
    for level in (None, 1, 0):
        in_grad, out_data, out_grad = empty((b, d, n, n)), empty((b, o, n, n)), dev(og)
        layer = ConvolutionLayer(b, d, n, 1, 1, 0, o, dev(x), in_grad, out_data, out_grad)
        assert layer.path() == 3
        if level is not None:
            layer.set_options(fused=level, profile=True)
            assert layer.path() == level
        else:
            layer.set_options(profile=True)
        drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
        drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
        layer.forward()
        layer.backward(with_update=False)
        kernels = layer.stage_kernels()
        if level is None:
            assert kernels["Lower Cube"] == "" and kernels["Inverse Lwr"] == "" and kernels["Bw Remap"] == ""
            assert kernels["GEMM"].startswith("gemm_batched_kernel") and kernels["GEMM Wghts"] != ""
        else:
            assert kernels["Lower Cube"] != ""
        assert rel_err(host(out_data), ref_out) <= TOL, level
        assert rel_err(host(in_grad), ref_dx) <= TOL, level
        dw, db = np.empty((o, d, 1, 1), np.float32), np.empty((o,), np.float32)
        drv.memcpy(dw.ctypes.data, layer.model_grad_ptr(), dw.nbytes, 1)
        drv.memcpy(db.ctypes.data, layer.bias_grad_ptr(), db.nbytes, 1)
        assert rel_err(dw, np.asarray(ref_dw).reshape(dw.shape)) <= TOL, level
        assert rel_err(db, ref_db) <= TOL, level
        np.testing.assert_array_equal(host(out_grad), og)
        layer.close()
