"""GPU parity for whole training iterations (benchmark configurations 4 and 5): LeNet at its full batch and
CaffeNet/AlexNet at a small batch, layer chain on the device against the CPU oracle chain."""
import numpy as np
import pytest

from gpu_util import driver, rel_err
from oracle.oracle_net import OracleNet

pytestmark = pytest.mark.gpu
TOL = 1e-4


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


def _check_forward_and_align_switches(net, ref, layers, tol):
    """Every non-in-place layer's output against the oracle's (within `tol` of its largest magnitude),
    then the oracle's activations and max-pool arg-max indices are written into the device's
    buffers, so that both sides read the same ReLU masks and route pooled gradients to the same
    pixels in the backward pass.  Returns (worst forward error, activations, sign disagreements,
    pooling windows, arg-max disagreements)."""
    from caffecontroll_amd import nets
    ai, worst = 1, 0.0
    elements = sign_flips = windows = argmax_flips = 0
    for li, L in enumerate(layers):
        if L.type in (nets.RELU, nets.DROPOUT):
            continue
        ptr, n = net.tensor(li, nets.OUTPUT)
        got, want = _down(ptr, n), ref.acts[ai].reshape(-1)
        e = rel_err(got, want)
        worst = max(worst, e)
        assert e <= tol, "forward layer %d (type %d): %.3g" % (li, L.type, e)
        elements += n
        sign_flips += int(np.count_nonzero((got > 0) != (want > 0)))
        _up(ptr, want)
        if L.type == nets.MAXPOOL:
            ptr, n = net.tensor(li, nets.AUX)
            want = ref.saved[(li, "idx")].reshape(-1).astype(np.int32)
            windows += n
            argmax_flips += int(np.count_nonzero(_down(ptr, n, np.int32) != want))
            _up(ptr, want)
        ai += 1
    return worst, elements, sign_flips, windows, argmax_flips


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
            worst = max(worst, e)
            assert e <= tol, "layer %d group %d grad %d: %.3g" % (li, gi, k, e)
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
    # the tensors `bench.py --workload lenet` times; later iterations draw new images
    import bench
    wl = bench.net_workload("lenet")
    for (li, gi), p in sorted(ref.params.items()):
        w, bias = wl["params"][(li, gi)]
        p["w"][...] = w.reshape(p["w"].shape)
        p["b"][...] = bias
        _up(net.tensor(li, nets.MODEL, gi)[0], p["w"])
        _up(net.tensor(li, nets.BIAS, gi)[0], p["b"])
    bound = oracle.bind_openblas(8)
    try:
        for it in range(3):
            x = wl["x"] if it == 0 else rng.uniform(0, 1, (B, 1, 28, 28)).astype(np.float32)
            labels = wl["labels"] if it == 0 else rng.integers(0, 10, B).astype(np.float32)
            _up(net.input_ptr(), x)
            _up(net.labels_ptr(), labels)
            net.forward()
            prob = ref.forward(x, labels)
            if it == 0:   # the loss bench.py checks its first pass against
                assert abs(ref.loss / B - bench.FIRST_LOSS_PER_IMAGE["lenet"]) <= 1e-4 * ref.loss / B, ref.loss / B
            ptr, n = net.tensor(len(layers) - 1, nets.OUTPUT)
            assert rel_err(_down(ptr, n), prob.reshape(-1)) <= TOL
            assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
            # every layer to 1e-4; ReLU masks and pooling arg-max aligned before the backward pass
            _, elements, sign_flips, windows, argmax_flips = _check_forward_and_align_switches(net, ref, layers, TOL)
            assert sign_flips <= 1e-4 * elements and argmax_flips <= 1e-4 * windows
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
        _, elements, sign_flips, windows, argmax_flips = _check_forward_and_align_switches(net, ref, layers, TOL)
        assert sign_flips <= 1e-4 * elements and argmax_flips <= 1e-4 * windows
        assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        _compare_params(net, ref, TOL)
    finally:
        if bound:
            oracle.unbind_openblas()
    net.close()


@pytest.mark.timeout(900)
def test_caffenet_full_batch_iteration(oracle):
    """benchmark configuration 5 at its full size: batch 256, grouped conv2/4/5, the instances the bench
    times (plane-tiled pooling, run-of-channels LRN, 4/6/8-wavefront weight gradients, deferred batched
    SGD), against the oracle chain run the way the reference runs on a CPU (16 batch partitions).

    Forward: every layer's output within 1e-4 of its largest magnitude, loss within 1e-4.
    The network has two kinds of switches that a rounding difference can flip: the arg-max of a
    pooling window and the sign test of a ReLU.  Both sides may disagree on them only where the
    competing values agree to rounding -- on fewer than 1e-5 of the windows / activations, which is
    asserted.  One flipped switch reroutes a whole gradient value (a single fc6 unit changes 3 % of
    that layer's weight gradient), so before the backward pass the oracle's switches are written
    into the device's buffers -- its arg-max indices and its activations, which the masks are read
    from -- and the backward pass is then held to the per-operator bar of 1e-4: every weight and
    bias gradient and every updated weight."""
    from caffecontroll_amd import nets
    import bench
    wl = bench.net_workload("caffenet")          # the tensors `bench.py --workload caffenet` times
    rng = np.random.default_rng(77)
    B, layers, x, labels = wl["B"], wl["layers"], wl["x"], wl["labels"]
    assert B == 256
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    driver()
    net = nets.Net(B, 3, 227, layers, nets.solver_param(**solver))
    ref = OracleNet(oracle, layers, B, 3, 227, solver, partitions=16)
    for (li, gi), p in sorted(ref.params.items()):
        w, bias = wl["params"][(li, gi)]
        p["w"][...] = w.reshape(p["w"].shape)
        p["b"][...] = bias
        _up(net.tensor(li, nets.MODEL, gi)[0], p["w"])
        _up(net.tensor(li, nets.BIAS, gi)[0], p["b"])
    net.freeze_dropout_masks(True)
    for li, L in enumerate(layers):
        if L.type == nets.DROPOUT:
            ptr, n = net.tensor(li, nets.AUX)
            mask = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
            _up(ptr, mask)
            ref.masks[li] = mask
    _up(net.input_ptr(), x)
    _up(net.labels_ptr(), labels)
    bound = oracle.bind_openblas(1)
    try:
        # TEST phase first (dropout off): the loss bench.py checks its first pass against
        net.set_train(False)
        ref.train = False
        net.forward()
        ref.forward(x, labels)
        assert abs(net.loss() - ref.loss) <= TOL * abs(ref.loss)
        assert abs(ref.loss / B - bench.FIRST_LOSS_PER_IMAGE["caffenet"]) <= 1e-4 * ref.loss / B, ref.loss / B
        net.set_train(True)
        ref.train = True
        net.forward()
        ref.forward(x, labels)
        worst_fwd, elements, sign_flips, windows, argmax_flips = _check_forward_and_align_switches(net, ref, layers, TOL)
        assert abs(net.loss() - ref.loss) <= TOL * abs(ref.loss)
        # N(0, 0.01) weights give nearly uniform class scores: the loss per image sits at ln(1000)
        assert abs(ref.loss / B - np.log(1000.0)) < 0.1
        assert argmax_flips <= 1e-5 * windows, (argmax_flips, windows)
        assert sign_flips <= 1e-5 * elements, (sign_flips, elements)
        net.backward()
        ref.backward()
        worst_bwd = 0.0
        for (li, gi), p in sorted(ref.params.items()):
            for which, k, key, hist in ((nets.MODEL_GRAD, 0, "w", "hw"), (nets.BIAS_GRAD, 1, "b", "hb")):
                ptr, n = net.tensor(li, which, gi)
                lam = np.float32(solver["weight_decay"] * layers[li].decay_mult[k])
                w_before = p[key].reshape(-1) + p[hist]          # w after the update + its momentum step
                want = ref.grads[(li, gi)][k].reshape(-1) + lam * w_before
                e = rel_err(_down(ptr, n), want)
                worst_bwd = max(worst_bwd, e)
                assert e <= TOL, "layer %d group %d gradient %d: %.3g" % (li, gi, k, e)
            for which, key in ((nets.MODEL, "w"), (nets.BIAS, "b")):
                ptr, n = net.tensor(li, which, gi)
                assert rel_err(_down(ptr, n), p[key].reshape(-1)) <= TOL
        print("full-batch CaffeNet: worst forward error %.3g, worst gradient error %.3g, arg-max differing on %d of %d "
              "windows, ReLU sign on %d of %d activations, loss/image %.5f"
              % (worst_fwd, worst_bwd, argmax_flips, windows, sign_flips, elements, ref.loss / B))
    finally:
        if bound:
            oracle.unbind_openblas()
    net.close()


@pytest.mark.timeout(900)
def test_caffenet_full_batch_iteration_untouched(oracle):
    """The iteration bench.py times, end to end with nothing written into the device between the forward and the
    backward pass: the device keeps its own pooling arg-max indices and ReLU signs.  Where those differ from the
    oracle's (a few windows / activations in ten million, on values equal to rounding) a whole gradient value is
    rerouted, so the gradients are held to a looser bar than in the aligned test above -- 2e-2 of each tensor's
    largest magnitude, 1e-2 in the root-mean-square sense (measured: 6e-3 and 2.5e-3 at worst, in the layers
    below the last pooling; 1e-6 above it) -- and the result of the iteration, the updated weights and biases,
    to 1e-4 of theirs (measured 5e-6: one SGD step moves a weight by the learning rate times its gradient)."""
    from caffecontroll_amd import nets
    import bench
    wl = bench.net_workload("caffenet")
    rng = np.random.default_rng(78)
    B, layers, x, labels = wl["B"], wl["layers"], wl["x"], wl["labels"]
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    driver()
    net = nets.Net(B, 3, 227, layers, nets.solver_param(**solver))
    ref = OracleNet(oracle, layers, B, 3, 227, solver, partitions=16)
    for (li, gi), p in sorted(ref.params.items()):
        w, bias = wl["params"][(li, gi)]
        p["w"][...] = w.reshape(p["w"].shape)
        p["b"][...] = bias
        _up(net.tensor(li, nets.MODEL, gi)[0], p["w"])
        _up(net.tensor(li, nets.BIAS, gi)[0], p["b"])
    net.freeze_dropout_masks(True)
    for li, L in enumerate(layers):
        if L.type == nets.DROPOUT:
            ptr, n = net.tensor(li, nets.AUX)
            mask = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
            _up(ptr, mask)
            ref.masks[li] = mask
    _up(net.input_ptr(), x)
    _up(net.labels_ptr(), labels)
    bound = oracle.bind_openblas(1)
    try:
        net.forward()
        net.backward()            # nothing touched in between
        ref.forward(x, labels)
        ref.backward()
        assert abs(net.loss() - ref.loss) <= TOL * abs(ref.loss)
        worst_g = worst_rms = worst_w = 0.0
        for (li, gi), p in sorted(ref.params.items()):
            for which, k, key, hist in ((nets.MODEL_GRAD, 0, "w", "hw"), (nets.BIAS_GRAD, 1, "b", "hb")):
                ptr, n = net.tensor(li, which, gi)
                lam = np.float32(solver["weight_decay"] * layers[li].decay_mult[k])
                w_before = p[key].reshape(-1) + p[hist]
                want = (ref.grads[(li, gi)][k].reshape(-1) + lam * w_before).astype(np.float64)
                got = _down(ptr, n).astype(np.float64)
                e = np.abs(got - want).max() / np.abs(want).max()
                rms = np.sqrt(np.mean((got - want) ** 2)) / np.sqrt(np.mean(want ** 2))
                worst_g, worst_rms = max(worst_g, e), max(worst_rms, rms)
                assert e <= 2e-2 and rms <= 1e-2, "layer %d group %d gradient %d: max %.3g rms %.3g" % (li, gi, k, e, rms)
            for which, key in ((nets.MODEL, "w"), (nets.BIAS, "b")):
                ptr, n = net.tensor(li, which, gi)
                e = rel_err(_down(ptr, n), p[key].reshape(-1))
                worst_w = max(worst_w, e)
                assert e <= TOL, "layer %d group %d updated %s: %.3g" % (li, gi, key, e)
        print("untouched full-batch CaffeNet iteration: worst gradient error %.3g (rms %.3g), worst updated-weight error %.3g"
              % (worst_g, worst_rms, worst_w))
    finally:
        if bound:
            oracle.unbind_openblas()
    net.close()


@pytest.mark.parametrize("level", [3, -1])
def test_wide_network_in_network_style_iterations(oracle, level):
    """A chain with the geometries beyond CaffeNet's and LeNet's: 3x72x72 inputs, a 7 x 7 stride-1 layer (images in
    column bands on the all-direct path), 1 x 1 layers (products on the tensors as they lie at any level), a 3 x 3 layer
    on 36-pixel rows (weight gradient one image per step); two training iterations with momentum and weight decay,
    every layer's output, the loss and every updated parameter against the oracle chain."""
    from caffecontroll_amd import nets
    rng = np.random.default_rng(77 + level)
    B, D, S, classes = 6, 3, 72, 7
    layers = [nets.conv(16, 7, 1, 3), nets.relu(), nets.conv(24, 1), nets.relu(), nets.maxpool(2, 2),
              nets.conv(32, 3, 1, 1), nets.relu(), nets.maxpool(2, 2), nets.conv(16, 1), nets.relu(),
              nets.fc(classes), nets.softmax_loss()]
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    driver()
    net = nets.Net(B, D, S, layers, nets.solver_param(**solver))
    net.set_conv_path(level)
    ref = OracleNet(oracle, layers, B, D, S, solver)
    _init_and_sync_params(net, ref, rng)
    for _ in range(2):
        x = rng.standard_normal((B, D, S, S)).astype(np.float32)
        labels = rng.integers(0, classes, B).astype(np.float32)
        _up(net.input_ptr(), x)
        _up(net.labels_ptr(), labels)
        net.forward()
        ref.forward(x, labels)
        _check_forward_and_align_switches(net, ref, layers, TOL)
        assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        _compare_params(net, ref, TOL)
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
