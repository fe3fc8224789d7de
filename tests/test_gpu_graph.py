"""Networks whose layers name their bottoms: a tensor read by two towers (the reference's Split:
shared data, one gradient per reader, gradients added before the producer's backward step,
src/DeepNet.h:1924-2028) and CONCAT (src/DeepNet.h:1700-1757), on the device against the oracle."""
import numpy as np
import pytest

from gpu_util import driver, rel_err
from oracle.oracle_net import OracleGraph

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _up(ptr, arr):
    a = np.ascontiguousarray(arr)
    driver().memcpy(ptr, a.ctypes.data, a.nbytes, 0)


def _down(ptr, n, dtype=np.float32):
    out = np.empty(n, dtype)
    driver().memcpy(out.ctypes.data, ptr, out.nbytes, 1)
    return out


def two_tower_layers(nets):
    """The shape of benchmark/train_val/caffenet_train_val_8_split.prototxt in small: a stem, two towers
    that both read the stem's LRN output, CONCAT, inner product, loss."""
    return [
        nets.conv(8, 3, pad=1), nets.relu(), nets.maxpool(2, 2), nets.lrn(3, 1e-2, 0.75),      # 0-3: stem
        nets.conv(6, 3, pad=1).read_from(3), nets.relu(), nets.maxpool(2, 2),                   # 4-6: tower A
        nets.conv(10, 3, pad=1, group=2).read_from(3), nets.relu(), nets.maxpool(2, 2),         # 7-9: tower B
        nets.concat(6, 9),                                                                      # 10
        nets.fc(32), nets.relu(), nets.dropout(0.5), nets.fc(5), nets.softmax_loss(),           # 11-15
    ]


def _sync_params(net, ref, rng, nets):
    for (li, gi), p in sorted(ref.params.items()):
        p["w"][...] = (rng.standard_normal(p["w"].shape) * 0.2).astype(np.float32)
        p["b"][...] = rng.uniform(-0.1, 0.2, p["b"].shape).astype(np.float32)
        _up(net.tensor(li, nets.MODEL, gi)[0], p["w"])
        _up(net.tensor(li, nets.BIAS, gi)[0], p["b"])


def test_two_towers_split_and_concat(oracle):
    from caffecontroll_amd import nets
    layers = two_tower_layers(nets)
    B, D, S = 6, 3, 12
    solver = dict(base_lr=0.05, momentum=0.9, weight_decay=0.001)
    driver()
    net = nets.Net(B, D, S, layers, nets.solver_param(**solver))
    ref = OracleGraph(oracle, layers, B, D, S, solver)
    rng = np.random.default_rng(8)
    _sync_params(net, ref, rng, nets)
    net.freeze_dropout_masks(True)
    ptr, n = net.tensor(13, nets.AUX)
    ref.masks[13] = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
    _up(ptr, ref.masks[13])
    for it in range(2):
        x = rng.standard_normal((B, D, S, S)).astype(np.float32)
        labels = rng.integers(0, 5, B).astype(np.float32)
        _up(net.input_ptr(), x)
        _up(net.labels_ptr(), labels)
        net.forward()
        ref.forward(x, labels)
        for li, L in enumerate(layers):
            if L.type in (nets.RELU, nets.DROPOUT):
                continue
            ptr, n = net.tensor(li, nets.OUTPUT)
            want = ref.val[ref.blob[li]] if li != len(layers) - 1 else ref.out[li]
            assert rel_err(_down(ptr, n), want.reshape(-1)) <= TOL, "forward layer %d" % li
            if L.type == nets.MAXPOOL:      # same arg-max on both sides (checked, then aligned for the backward pass)
                ptr, n = net.tensor(li, nets.AUX)
                want = ref.saved[(li, "idx")].reshape(-1).astype(np.int32)
                assert np.count_nonzero(_down(ptr, n, np.int32) != want) <= 1
                _up(ptr, want)
        assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        # the gradient of the shared tensor (the LRN output): tower A's plus tower B's, in that order
        ptr, n = net.tensor(4, nets.INPUT_GRAD)
        assert rel_err(_down(ptr, n), ref.tensor_grads[3].reshape(-1)) <= TOL
        for (li, gi), p in sorted(ref.params.items()):
            for which, k, key, hist in ((nets.MODEL_GRAD, 0, "w", "hw"), (nets.BIAS_GRAD, 1, "b", "hb")):
                ptr, n = net.tensor(li, which, gi)
                lam = np.float32(solver["weight_decay"] * layers[li].decay_mult[k])
                want = ref.grads[(li, gi)][k].reshape(-1) + lam * (p[key].reshape(-1) + p[hist])
                assert rel_err(_down(ptr, n), want) <= TOL, "layer %d group %d gradient %d" % (li, gi, k)
            for which, key in ((nets.MODEL, "w"), (nets.BIAS, "b")):
                ptr, n = net.tensor(li, which, gi)
                assert rel_err(_down(ptr, n), p[key].reshape(-1)) <= TOL
    net.close()


def test_concat_of_two_convolutions_equals_one_with_stacked_filters():
    """conv_a(x) and conv_b(x) stacked by CONCAT hold the very values of one convolution whose
    filters are those of a followed by those of b (every output map is computed on its own); the
    input gradient, a sum over all maps, agrees to rounding (two partial sums instead of one)."""
    from caffecontroll_amd import nets
    B, D, S, oa, ob = 4, 5, 9, 7, 9
    rng = np.random.default_rng(3)
    driver()
    stem = [nets.conv(D, 1)]       # a weight layer in front, so that the towers compute an input gradient
    split = stem + [nets.conv(oa, 3, pad=1).read_from(0), nets.conv(ob, 3, pad=1).read_from(0), nets.concat(1, 2),
                    nets.fc(3), nets.softmax_loss()]
    single = stem + [nets.conv(oa + ob, 3, pad=1), nets.fc(3), nets.softmax_loss()]
    sp = nets.solver_param(base_lr=0.0)
    net_s, net_1 = nets.Net(B, D, S, split, sp), nets.Net(B, D, S, single, sp)
    w0 = rng.standard_normal((D, D, 1, 1)).astype(np.float32)
    wa = rng.standard_normal((oa, D, 3, 3)).astype(np.float32)
    wb = rng.standard_normal((ob, D, 3, 3)).astype(np.float32)
    ba, bb = rng.standard_normal(oa).astype(np.float32), rng.standard_normal(ob).astype(np.float32)
    wf = (rng.standard_normal((3, (oa + ob) * S * S)) * 0.01).astype(np.float32)
    for net in (net_s, net_1):
        _up(net.tensor(0, nets.MODEL)[0], w0)
    _up(net_s.tensor(1, nets.MODEL)[0], wa); _up(net_s.tensor(1, nets.BIAS)[0], ba)
    _up(net_s.tensor(2, nets.MODEL)[0], wb); _up(net_s.tensor(2, nets.BIAS)[0], bb)
    _up(net_s.tensor(4, nets.MODEL)[0], wf)
    _up(net_1.tensor(1, nets.MODEL)[0], np.concatenate([wa, wb])); _up(net_1.tensor(1, nets.BIAS)[0], np.concatenate([ba, bb]))
    _up(net_1.tensor(2, nets.MODEL)[0], wf)
    x = rng.standard_normal((B, D, S, S)).astype(np.float32)
    labels = rng.integers(0, 3, B).astype(np.float32)
    for net in (net_s, net_1):
        _up(net.input_ptr(), x)
        _up(net.labels_ptr(), labels)
        net.forward()
        net.backward()
    cat = _down(*net_s.tensor(3, nets.OUTPUT))
    one = _down(*net_1.tensor(1, nets.OUTPUT))
    np.testing.assert_array_equal(cat, one)
    assert net_s.loss() == net_1.loss()
    # gradient of the shared tensor: conv_a's reader first, conv_b's added to it
    g_split = _down(*net_s.tensor(1, nets.INPUT_GRAD))
    g_one = _down(*net_1.tensor(1, nets.INPUT_GRAD))
    assert rel_err(g_split, g_one) <= 1e-5
    # the stacked filter gradient is the two towers' gradients side by side
    gw = np.concatenate([_down(*net_s.tensor(1, nets.MODEL_GRAD)), _down(*net_s.tensor(2, nets.MODEL_GRAD))])
    assert rel_err(gw, _down(*net_1.tensor(1, nets.MODEL_GRAD))) <= 1e-5
    net_s.close()
    net_1.close()


def test_graph_descriptions_are_checked_on_the_host():
    from caffecontroll_amd import CctHipError, nets
    bad = [
        ([nets.conv(4, 3), nets.conv(4, 3).read_from(1)], "earlier layer"),
        ([nets.conv(4, 3), nets.conv(4, 3), nets.concat(0)], "at least two"),
        ([nets.conv(4, 3), nets.maxpool(2, 2), nets.concat(0, 1)], "differ in height"),
        ([nets.conv(4, 3), nets.conv(4, 3).read_from(0), nets.relu().read_from(0)], "already reads"),
    ]
    for layers, fragment in bad:
        with pytest.raises(CctHipError) as e:
            nets.validate(2, 3, 12, layers + [nets.softmax_loss()])
        assert fragment in str(e.value), str(e.value)
