"""GPU parity at operator level: ParallelizedBridge<ConvolutionBridge> on the HIP driver against
the reference's golden files (the same scenario as tests/test_parallelized_convolution.cpp:123-270
and ..._large_CPU.cpp) and against the CPU oracle on seeded tensors."""
import numpy as np
import pytest

from conftest import load_fixture
from gpu_util import dev, driver, empty, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _copy_to(ptr, arr):
    a = np.ascontiguousarray(arr, np.float32)
    driver().memcpy(ptr, a.ctypes.data, a.nbytes, 0)


def _read(ptr, shape):
    out = np.empty(shape, np.float32)
    driver().memcpy(out.ctypes.data, ptr, out.nbytes, 1)
    return out


FIX = {
    "small": dict(b=4, d=3, n=20, k=5, s=4, p=2, o=10, sfx=""),
    "large": dict(b=4, d=3, n=127, k=11, s=4, p=2, o=8, sfx="_large"),
}


@pytest.mark.parametrize("case", ["small", "large"])
@pytest.mark.parametrize("fused", [True, False])
def test_pbridge_reference_scenario(case, fused):
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    c = FIX[case]
    b, d, n, k, s, p, o, sfx = (c[x] for x in ("b", "d", "n", "k", "s", "p", "o", "sfx"))
    m = (n + 2 * p - k) // s + 1
    driver()
    x = load_fixture("input", f"conv_forward_in{sfx}.txt").reshape(b, d, n, n)
    in_data, in_grad = dev(x), empty((b, d, n, n), fill=0.0)
    out_data, out_grad = empty((b, o, m, m), fill=0.0), empty((b, o, m, m), fill=0.0)
    # solver of the reference test: lr 0.01, momentum 0, policy "step" with stepsize 10000
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad,
                             solver=solver_param(base_lr=0.01, momentum=0.0, lr_policy="step", stepsize=10000))
    layer.set_options(fused=fused)
    # TestForward
    _copy_to(layer.model_ptr(), load_fixture("input", f"conv_model{sfx}.txt"))
    _copy_to(layer.bias_ptr(), load_fixture("input", f"conv_bias_in{sfx}.txt"))
    layer.forward()
    exp = load_fixture("output", f"conv_forward{sfx}.txt")
    np.testing.assert_allclose(host(out_data).reshape(-1), exp, rtol=2e-5, atol=1e-3)
    # TestBackward
    _copy_to(layer.model_ptr(), load_fixture("input", f"conv_backward_model{sfx}.txt"))
    og = (np.arange(b * o * m * m, dtype=np.float64) * 0.1).astype(np.float32)
    out_grad.copy_(dev(og).reshape(out_grad.shape))
    og_before = host(out_grad).copy()
    layer.forward()
    layer.backward(with_update=True)
    exp_dx = load_fixture("output", f"conv_backward{sfx}.txt")
    np.testing.assert_allclose(host(in_grad).reshape(-1)[:exp_dx.size], exp_dx, rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(_read(layer.model_ptr(), (o * d * k * k,)),
                               load_fixture("output", f"conv_weights{sfx}.txt"), rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(_read(layer.bias_ptr(), (o,)),
                               load_fixture("output", f"conv_bias{sfx}.txt"), rtol=1e-4, atol=1e-3)
    # the caller's output-gradient cube is left as it was (the HIP bridge permutes into scratch)
    np.testing.assert_array_equal(host(out_grad), og_before)
    layer.close()


@pytest.mark.parametrize("shape", [(8, 96, 27, 5, 1, 2, 256), (64, 1, 28, 5, 1, 0, 20), (4, 3, 227, 11, 4, 0, 96)],
                         ids=lambda s: "b%d_d%d_n%d_k%d_s%d_p%d_o%d" % s)
def test_pbridge_vs_oracle_with_momentum(oracle, shape):
    """Two iterations with momentum and weight decay: gradients, history and weights track the
    oracle's ConvolutionBridge + SGDGradientUpdater restatement."""
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(1234 + sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.01).astype(np.float32)
    bias = np.full(o, 0.1, np.float32)
    driver()
    in_data, in_grad = dev(x), empty((b, d, n, n))
    out_data, out_grad = empty((b, o, m, m)), empty((b, o, m, m), fill=0.0)
    lr, mom, wd = 0.01, 0.9, 0.0005
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad,
                             solver=solver_param(base_lr=lr, momentum=mom, weight_decay=wd),
                             lr_mult=(1.0, 2.0), decay_mult=(1.0, 0.0))
    _copy_to(layer.model_ptr(), w)
    _copy_to(layer.bias_ptr(), bias)
    rw, rb = w.copy(), bias.copy()
    hw, hb = np.zeros(w.size, np.float32), np.zeros(o, np.float32)
    bound = oracle.bind_openblas(8)
    try:
        for it in range(2):
            og = rng.standard_normal((b, o, m, m)).astype(np.float32)
            out_grad.copy_(dev(og))
            layer.forward()
            layer.backward(with_update=True)
            ref_out, rlow = oracle.conv_forward(x, rw, rb, k, s, p)
            rdx, rdw, rdb = oracle.conv_backward(x.shape, rw, og, rlow, k, s, p)
            assert rel_err(host(out_data), ref_out) <= TOL
            assert rel_err(host(in_grad), rdx) <= TOL
            rw_flat = rw.reshape(-1)
            oracle.sgd_update(rw_flat, rdw.reshape(-1), hw, lr * 1.0, mom, wd * 1.0)
            oracle.sgd_update(rb, rdb, hb, lr * 2.0, mom, 0.0)
            rw = rw_flat.reshape(w.shape)
            assert rel_err(_read(layer.model_ptr(), w.shape), rw) <= TOL
            assert rel_err(_read(layer.bias_ptr(), (o,)), rb) <= TOL
            assert rel_err(_read(layer.history_ptr(), (w.size,)), hw) <= TOL
    finally:
        if bound:
            oracle.unbind_openblas()
    layer.close()


def test_stage_profile_and_first_layer_mode():
    from caffecontroll_amd.bridges import STAGE_NAMES, ConvolutionLayer
    b, d, n, k, s, p, o = 4, 8, 12, 3, 1, 1, 16
    driver()
    in_data, in_grad = empty((b, d, n, n), fill=1.0), empty((b, d, n, n), fill=-5.0)
    out_data, out_grad = empty((b, o, n, n)), empty((b, o, n, n), fill=1.0)
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad)
    layer.set_options(fused=False, profile=True, needs_backward_grad=False)
    layer.forward()
    layer.backward()
    ms = layer.stage_ms()
    assert set(ms) == set(STAGE_NAMES)
    assert ms["Lower Cube"] > 0 and ms["GEMM"] > 0 and ms["Remap"] > 0 and ms["Bias"] > 0 and ms["GEMM Wghts"] > 0
    assert ms["GEMM Data"] == 0 and ms["Inverse Lwr"] == 0      # skipped for a first layer
    assert (host(in_grad) == -5.0).all()                          # and the input gradient is untouched
    # bias gradient of an all-ones output gradient = b * m * m
    bg = np.empty(o, np.float32)
    driver().memcpy(bg.ctypes.data, layer.bias_grad_ptr(), bg.nbytes, 1)
    assert (bg == b * n * n).all()
    layer.close()


POLICIES = [
    # (policy, base_lr, gamma, stepsize, power, max_iter)
    ("fixed", 0.05, 0.3, 3, 2.0, 50),
    ("step", 0.02, 0.5, 3, 3.0, 50),
    ("exp", 0.05, 0.9, 3, 3.0, 50),
    ("inv", 0.05, 0.05, 3, 0.75, 50),
    ("poly", 0.05, 0.05, 3, 2.0, 12),
    ("sigmoid", 0.05, -0.7, 4, 2.0, 50),
]


@pytest.mark.parametrize("policy", POLICIES, ids=lambda c: c[0])
@pytest.mark.parametrize("l1", [False, True], ids=["L2", "L1"])
def test_stepped_sgd_follows_the_schedule_bit_for_bit(oracle, policy, l1):
    """SGDGradientUpdater::update with get_stepsize = lr_mult * Util::get_learning_rate(policy, ...,
    iter) (src/algorithms/GradientUpdater.h:42-45, 154-193; src/util.h:76-93) over nine iterations,
    across two `step` boundaries.  Input and output gradient are small integers, so the weight and
    bias gradients are exact and the same in every iteration (they do not depend on the weights):
    the weights on the device must then equal the oracle's updater, driven by the oracle's
    schedule, bit for bit after every iteration."""
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    name, base, gamma, stepsize, power, max_iter = policy
    b, d, n, k, s, p, o = 2, 3, 8, 3, 1, 1, 4
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(31)
    x = rng.integers(-3, 4, size=(b, d, n, n)).astype(np.float32)
    og = rng.integers(-2, 3, size=(b, o, m, m)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    driver()
    in_data, in_grad = dev(x), empty((b, d, n, n))
    out_data, out_grad = empty((b, o, m, m)), dev(og)
    mom, wd, lr_mult, decay_mult = 0.9, 0.0005, (1.0, 2.0), (1.0, 0.5)
    sp = solver_param(base_lr=base, momentum=mom, weight_decay=wd, lr_policy=name, gamma=gamma, stepsize=stepsize,
                      power=power, max_iter=max_iter, regularization_type="L1" if l1 else "L2")
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad, solver=sp,
                             lr_mult=lr_mult, decay_mult=decay_mult)
    _copy_to(layer.model_ptr(), w)
    _copy_to(layer.bias_ptr(), bias)
    _, lowered = oracle.conv_forward(x, w, bias, k, s, p)
    _, dw, db = oracle.conv_backward(x.shape, w, og, lowered, k, s, p)
    rw, rb = w.reshape(-1).copy(), bias.copy()
    hw, hb = np.zeros(w.size, np.float32), np.zeros(o, np.float32)
    f32 = np.float32
    rates = []
    for it in range(1, 10):
        layer.forward()
        layer.backward(with_update=True)
        rate = f32(oracle.learning_rate(name, base, gamma, it, stepsize, power, max_iter))
        rates.append(float(rate))
        oracle.sgd_update(rw, dw.reshape(-1).copy(), hw, f32(lr_mult[0]) * rate, mom, f32(wd) * f32(decay_mult[0]), l1)
        oracle.sgd_update(rb, db.copy(), hb, f32(lr_mult[1]) * rate, mom, f32(wd) * f32(decay_mult[1]), l1)
        np.testing.assert_array_equal(_read(layer.model_ptr(), (w.size,)), rw, err_msg="weights, iteration %d" % it)
        np.testing.assert_array_equal(_read(layer.bias_ptr(), (o,)), rb, err_msg="bias, iteration %d" % it)
        np.testing.assert_array_equal(_read(layer.history_ptr(), (w.size,)), hw, err_msg="momentum, iteration %d" % it)
    if name != "fixed":
        assert len(set(rates)) > 2, rates   # the schedule moved during the run, so it was exercised
    layer.close()


@pytest.mark.parametrize("share", [(False, False), (False, True), (True, False)], ids=["host-host", "host-dev", "dev-host"])
def test_pbridge_on_host_layers_like_the_reference_tests(share):
    """share_pointer_with_prev/next_bridge = false (src/bridges/ParallelizedBridge.h:183-198): the
    layer on that side is host memory and the bridge moves it to and from its own device cubes.  The
    reference's golden scenario (tests/test_parallelized_convolution.cpp:123-270) run on plain host
    arrays, as the reference test itself does, and the mixed placements against it."""
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    share_prev, share_next = share
    c = FIX["small"]
    b, d, n, k, s, p, o = (c[x] for x in ("b", "d", "n", "k", "s", "p", "o"))
    m = (n + 2 * p - k) // s + 1
    driver()
    x = load_fixture("input", "conv_forward_in.txt").reshape(b, d, n, n)
    og = (np.arange(b * o * m * m, dtype=np.float64) * 0.1).astype(np.float32).reshape(b, o, m, m)
    in_data = dev(x) if share_prev else x.copy()
    in_grad = empty((b, d, n, n)) if share_prev else np.full((b, d, n, n), np.nan, np.float32)
    out_data = empty((b, o, m, m)) if share_next else np.full((b, o, m, m), np.nan, np.float32)
    out_grad = dev(og) if share_next else og.copy()
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad,
                             solver=solver_param(base_lr=0.01, momentum=0.0, lr_policy="step", stepsize=10000),
                             share_prev=share_prev, share_next=share_next)
    as_host = lambda t: host(t) if hasattr(t, "data_ptr") else t
    _copy_to(layer.model_ptr(), load_fixture("input", "conv_model.txt"))
    _copy_to(layer.bias_ptr(), load_fixture("input", "conv_bias_in.txt"))
    layer.forward()
    np.testing.assert_allclose(as_host(out_data).reshape(-1), load_fixture("output", "conv_forward.txt"), rtol=2e-5, atol=1e-3)
    _copy_to(layer.model_ptr(), load_fixture("input", "conv_backward_model.txt"))
    layer.forward()
    layer.backward(with_update=True)
    np.testing.assert_allclose(as_host(in_grad).reshape(-1), load_fixture("output", "conv_backward.txt"), rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(_read(layer.model_ptr(), (o * d * k * k,)), load_fixture("output", "conv_weights.txt"),
                               rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(_read(layer.bias_ptr(), (o,)), load_fixture("output", "conv_bias.txt"), rtol=1e-4, atol=1e-3)
    layer.close()


@pytest.mark.parametrize("shape", [(32, 48, 27, 5, 1, 2, 64), (10, 3, 67, 11, 4, 0, 32), (7, 16, 13, 3, 1, 1, 48), (3, 8, 20, 5, 1, 0, 16),
                                   (9, 24, 14, 1, 1, 0, 40), (5, 6, 20, 7, 1, 3, 12), (6, 4, 100, 3, 1, 1, 8)],
                         ids=lambda s: "b%d_d%d_n%d_k%d_s%d_p%d_o%d" % s)
@pytest.mark.parametrize("first_layer", [False, True])
def test_pbridge_overlapped_staging_equals_blocking_copies(shape, first_layer):
    """Host-resident layers on both sides: the batch moved in four pieces through the copy streams (upload of
    piece i+1 and download of piece i-1 beside the kernels of piece i; weight gradient in one call once the whole
    output gradient has arrived) against one blocking copy in, the pass, one blocking copy out
    (src/bridges/ParallelizedBridge_impl.hxx:595-621, 686-705): output, input gradient, weight and bias gradients
    and the updated weights bit for bit, on pinned and on pageable host arrays, two iterations in a row; batches
    that do not divide by four, stride-1 and strided layers, a 1 x 1 layer, a 7 x 7 layer and a 100-wide image."""
    import torch
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    driver()
    results = {}
    for mode in ("blocking", "pieces-pinned", "pieces-pageable"):
        if mode == "pieces-pinned":
            mk = lambda a: torch.from_numpy(a.copy()).pin_memory().numpy()
        else:
            mk = lambda a: a.copy()
        h_in, h_ig = mk(x), mk(np.full(x.shape, np.nan, np.float32))
        h_out, h_og = mk(np.full(og.shape, np.nan, np.float32)), mk(og)
        layer = ConvolutionLayer(b, d, n, k, s, p, o, h_in, h_ig, h_out, h_og, share_prev=False, share_next=False,
                                 solver=solver_param(base_lr=0.01, momentum=0.9, weight_decay=0.0005))
        layer.set_options(fused=3, needs_backward_grad=not first_layer)
        assert layer.path() == 3
        layer.set_staging(mode != "blocking")
        assert layer.staging_overlapped() == (mode != "blocking")
        _copy_to(layer.model_ptr(), w)
        _copy_to(layer.bias_ptr(), bias)
        snap = []
        for it in range(2):
            layer.forward()
            layer.backward(with_update=True)
            snap.append([h_out.copy(), None if first_layer else h_ig.copy(), _read(layer.model_grad_ptr(), (w.size,)),
                         _read(layer.bias_grad_ptr(), (o,)), _read(layer.model_ptr(), (w.size,)), _read(layer.bias_ptr(), (o,))])
        results[mode] = snap
        layer.close()
    assert not np.isnan(results["blocking"][1][0]).any()
    for mode in ("pieces-pinned", "pieces-pageable"):
        for it in range(2):
            for got, want, name in zip(results[mode][it], results["blocking"][it],
                                       ("output", "input gradient", "weight gradient", "bias gradient", "weights", "bias")):
                if want is None:
                    continue
                np.testing.assert_array_equal(got, want, err_msg="%s, iteration %d, %s" % (mode, it, name))


def test_pbridge_share_with_next_can_be_raised_after_construction(oracle):
    """The reference builds a bridge with share_pointer_with_next_bridge false and lets the builder of the next
    bridge raise it (src/DeepNet.h:1116-1120).  Here: a bridge created over a host output layer first copies its
    output to the host; once told to share, it writes into the next bridge's device tensors, reads its output
    gradient from there, and leaves the host arrays alone."""
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    b, d, n, k, s, p, o = 4, 6, 13, 3, 1, 1, 10
    m = n
    rng = np.random.default_rng(3)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    ref_out, low = oracle.conv_forward(x, w, bias, k, s, p)
    ref_dx, _, _ = oracle.conv_backward(x.shape, w, og, low, k, s, p)
    driver()
    in_data, in_grad = dev(x), empty((b, d, n, n))
    h_out, h_og = np.full((b, o, m, m), np.nan, np.float32), np.zeros((b, o, m, m), np.float32)
    layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, h_out, h_og, share_prev=True, share_next=False,
                             solver=solver_param(base_lr=0.0))
    _copy_to(layer.model_ptr(), w)
    _copy_to(layer.bias_ptr(), bias)
    layer.forward()
    assert rel_err(h_out, ref_out) <= 1e-4
    d_out, d_og = empty((b, o, m, m)), dev(og)
    layer.share_with_next(d_out, d_og)
    h_out[...] = np.nan
    layer.forward()
    assert rel_err(host(d_out), ref_out) <= 1e-4
    assert np.isnan(h_out).all()                  # nothing is copied to the host any more
    layer.backward(with_update=True)              # ParallelizedBridge::backward reads the device gradient in place
    assert rel_err(host(in_grad), ref_dx) <= 1e-4
    layer.close()
