"""GPU parity for whole training iterations (benchmark configurations 4 and 5): LeNet at its full batch and
CaffeNet/AlexNet at a small batch, layer chain on the device against the CPU oracle chain."""
import numpy as np
import pytest

from gpu_util import driver, rel_err
from oracle_net import OracleNet

pytestmark = pytest.mark.gpu
TOL = 1e-4
GRAD_TOL = 5e-3


def _up(ptr, arr):
    a = np.ascontiguousarray(arr)
    driver().memcpy(ptr, a.ctypes.data, a.nbytes, 0)


def _down(ptr, n, dtype=np.float32):
    out = np.empty(n, dtype)
    driver().memcpy(out.ctypes.data, ptr, out.nbytes, 1)
    return out


def _init_and_sync_params(net, ref, rng, std_of=None):
    from caffecontroll_amd import nets
    for (li, gi), p in ref.params.items():
        fan_in = p["w"][0].size
        scale = np.sqrt(3.0 / fan_in)
        p["w"][...] = rng.uniform(-scale, scale, p["w"].shape).astype(np.float32)
        p["b"][...] = rng.uniform(0, 0.2, p["b"].shape).astype(np.float32)
        wp, wn = net.tensor(li, nets.MODEL, gi)
        bp, bn = net.tensor(li, nets.BIAS, gi)
        assert wn == p["w"].size and bn == p["b"].size
        _up(wp, p["w"])
        _up(bp, p["b"])


def _compare_params(net, ref, tol):
    from caffecontroll_amd import nets
    worst = 0.0
    for (li, gi), p in sorted(ref.params.items()):
        for which, key in ((nets.MODEL, "w"), (nets.BIAS, "b")):
            ptr, n = net.tensor(li, which, gi)
            e = rel_err(_down(ptr, n), p[key].reshape(-1))
            worst = max(worst, e)
            assert e <= tol, "layer %d group %d %s: %.3g" % (li, gi, key, e)
        for which, k in ((nets.MODEL_GRAD, 0), (nets.BIAS_GRAD, 1)):
            ptr, n = net.tensor(li, which, gi)
            got = _down(ptr, n)
            want = ref.grads[(li, gi)][k].reshape(-1)
            # the device gradient buffer holds g + lambda*w after the update step, as the reference's does
            L = ref.layers[li]
            lam = ref.solver["weight_decay"] * L.decay_mult[k]
            # w before the update = w_after + h_after
            w_before = p["w" if k == 0 else "b"].reshape(-1) + p["hw" if k == 0 else "hb"]
            e = rel_err(got, want + np.float32(lam) * w_before)
            # Looser than the per-operator bar on purpose: when two candidates of a pooling window
            # differ by an ulp between the two sides the argmax flips, the gradient of that window
            # is routed to the neighbouring pixel, and a weight gradient moves by ~1e-3 of its
            # largest entry although every operator is within 1e-6 (bias gradients, which only sum
            # the routed values, stay at 1e-6).
            assert e <= GRAD_TOL, "layer %d group %d grad %d: %.3g" % (li, gi, k, e)
    return worst


def test_lenet_training_iterations(oracle):
    """benchmark configuration 4: batch 64, 1x28x28 uniform[0,1) images, 10 classes, lr 0.01, momentum 0.9."""
    from caffecontroll_amd import nets
    rng = np.random.default_rng(1234 + 4)
    B = 64
    layers = nets.lenet_layers()
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    driver()
    net = nets.Net(B, 1, 28, layers, nets.solver_param(**solver))
    ref = OracleNet(oracle, layers, B, 1, 28, solver)
    _init_and_sync_params(net, ref, rng)
    bound = oracle.bind_openblas(8)
    try:
        for it in range(3):
            x = rng.uniform(0, 1, (B, 1, 28, 28)).astype(np.float32)
            labels = rng.integers(0, 10, B).astype(np.float32)
            _up(net.input_ptr(), x)
            _up(net.labels_ptr(), labels)
            net.forward()
            prob = ref.forward(x, labels)
            ptr, n = net.tensor(len(layers) - 1, nets.OUTPUT)
            assert rel_err(_down(ptr, n), prob.reshape(-1)) <= TOL
            assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
            # pooled conv1 features and their argmax agree exactly in index, to 1e-4 in value
            ptr, n = net.tensor(1, nets.OUTPUT)
            assert rel_err(_down(ptr, n), ref.acts[2].reshape(-1)) <= TOL
            net.backward()
            ref.backward()
            _compare_params(net, ref, TOL)
    finally:
        if bound:
            oracle.unbind_openblas()
    net.close()


@pytest.mark.parametrize("groups", [True, False])
def test_caffenet_training_iteration_small_batch(oracle, groups):
    """benchmark configuration 5 geometry (3x227x227, 1000 classes, grouped conv2/4/5, LRN, dropout) at
    batch 2; dropout masks are injected so both sides drop the same units."""
    from caffecontroll_amd import nets
    rng = np.random.default_rng(1234 + 5)
    B = 2
    layers = nets.caffenet_layers(groups=groups)
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    driver()
    net = nets.Net(B, 3, 227, layers, nets.solver_param(**solver))
    ref = OracleNet(oracle, layers, B, 3, 227, solver)
    _init_and_sync_params(net, ref, rng)
    net.freeze_dropout_masks(True)
    for li, L in enumerate(layers):
        if L.type == nets.DROPOUT:
            ptr, n = net.tensor(li, nets.AUX)
            mask = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
            _up(ptr, mask)
            ref.masks[li] = mask
    x = rng.uniform(0, 255, (B, 3, 227, 227)).astype(np.float32)
    x -= np.array([104, 117, 123], np.float32)[None, :, None, None]
    x *= np.float32(1 / 64.0)  # keep activations in a numerically ordinary range with these random weights
    labels = rng.integers(0, 1000, B).astype(np.float32)
    _up(net.input_ptr(), x)
    _up(net.labels_ptr(), labels)
    bound = oracle.bind_openblas(8)
    try:
        net.forward()
        prob = ref.forward(x, labels)
        # layer by layer (non in-place layers), deepest error first to show
        ai = 1
        for li, L in enumerate(layers):
            if L.type in (nets.RELU, nets.DROPOUT):
                continue
            ptr, n = net.tensor(li, nets.OUTPUT)
            e = rel_err(_down(ptr, n), ref.acts[ai].reshape(-1))
            assert e <= 5 * TOL, "forward layer %d (type %d): %.3g" % (li, L.type, e)
            ai += 1
        assert abs(net.loss() - ref.loss) <= 5 * TOL * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        _compare_params(net, ref, 5 * TOL)
    finally:
        if bound:
            oracle.unbind_openblas()
    net.close()


def test_dropout_masks_change_and_test_phase_is_identity():
    from caffecontroll_amd import nets
    driver()
    layers = [nets.fc(32), nets.dropout(0.5), nets.fc(4), nets.softmax_loss()]
    net = nets.Net(8, 2, 3, layers, nets.solver_param(random_seed=5))
    x = np.ones((8, 2, 3, 3), np.float32)
    _up(net.input_ptr(), x)
    _up(net.labels_ptr(), np.zeros(8, np.float32))
    wp, wn = net.tensor(0, nets.MODEL)
    _up(wp, np.full(wn, 0.1, np.float32))
    net.forward()
    ptr, n = net.tensor(1, nets.AUX)
    m1 = _down(ptr, n, np.uint32).copy()
    out1 = _down(*net.tensor(1, nets.OUTPUT))
    keep = m1 > 2147483648
    np.testing.assert_allclose(out1, np.where(keep, 2 * 1.8, 0).astype(np.float32), rtol=1e-6)
    net.forward()
    m2 = _down(ptr, n, np.uint32)
    assert (m1 != m2).any()
    net.set_train(False)
    net.forward()
    np.testing.assert_allclose(_down(*net.tensor(1, nets.OUTPUT)), np.full(n, 1.8, np.float32), rtol=1e-6)
    net.close()
