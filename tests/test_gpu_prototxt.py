"""GPU checks of the configuration front end, the fillers, model files / snapshots and the
training loop: a network built from prototxt text must be the network built from layer records,
files must have the reference's byte layout (src/DeepNet.h:328-422) and a restored snapshot must
continue training bit for bit."""
import os

import numpy as np
import pytest

from gpu_util import driver

pytestmark = pytest.mark.gpu

NET_TEXT = """
name: "small"
layer { name: "data" type: "Data" top: "data" top: "label" include { phase: TRAIN }
        data_param { source: "none" batch_size: 8 } }
layer { name: "conv1" type: "Convolution" bottom: "data" top: "conv1"
        param { lr_mult: 1 } param { lr_mult: 2 }
        convolution_param { num_output: 6 kernel_size: 3 pad: 1
          weight_filler { type: "gaussian" std: 0.05 } bias_filler { type: "constant" value: 0.25 } } }
layer { name: "relu1" type: "ReLU" bottom: "conv1" top: "conv1" }
layer { name: "pool1" type: "Pooling" bottom: "conv1" top: "pool1" pooling_param { pool: MAX kernel_size: 2 stride: 2 } }
layer { name: "conv2" type: "Convolution" bottom: "pool1" top: "conv2"
        blobs_lr: 1 blobs_lr: 2 weight_decay: 1 weight_decay: 0
        convolution_param { num_output: 8 kernel_size: 3 group: 2
          weight_filler { type: "xavier" } bias_filler { type: "constant" value: 0 } } }
layer { name: "ip1" type: "InnerProduct" bottom: "conv2" top: "ip1"
        inner_product_param { num_output: 4 weight_filler { type: "xavier" } } }
layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip1" bottom: "label" top: "loss" }
"""
SOLVER_TEXT = """
base_lr: 0.05  momentum: 0.9  weight_decay: 0.0005  lr_policy: "inv" gamma: 0.01 power: 0.75
max_iter: 12 display: 4 random_seed: 77
"""


def _down(ptr, n):
    out = np.empty(n, np.float32)
    driver().memcpy(out.ctypes.data, ptr, out.nbytes, 1)
    return out


def _blobs(net, which_model, which_bias):
    """Per layer: all group models, then all group biases (the order of the model file)."""
    out = []
    for li, s in enumerate(net.layers):
        g = max(1, s.group)
        for which in (which_model, which_bias):
            for gi in range(g):
                ptr, n = net.tensor(li, which, gi)
                if ptr:
                    out.append(_down(ptr, n))
    return out


def _build():
    from caffecontroll_amd import prototxt as P
    driver()
    sp, ctl = P.solver_from_prototxt(SOLVER_TEXT)
    nd = P.network_from_prototxt(NET_TEXT)
    return sp, ctl, nd, nd.build(depth=2, size=10, solver=sp)


def _batches(n, seed=5):
    """Four separable classes: the class index decides which quadrant of the image is bright."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        y = rng.integers(0, 4, 8)
        x = rng.normal(0, 0.1, (8, 2, 10, 10)).astype(np.float32)
        for i, c in enumerate(y):
            x[i, :, (c // 2) * 5:(c // 2) * 5 + 5, (c % 2) * 5:(c % 2) * 5 + 5] += 1.0
        out.append((x, y.astype(np.float32)))
    return out


def test_prototxt_network_equals_hand_built_network():
    from caffecontroll_amd import nets
    sp, ctl, nd, net = _build()
    f = nets.filler
    layers = [nets.conv(6, 3, pad=1, lr_mult=(1, 2), decay_mult=(1, 1), weight_filler=f("gaussian", std=0.05),
                        bias_filler=f("constant", 0.25)), nets.relu(), nets.maxpool(2, 2),
              nets.conv(8, 3, group=2, lr_mult=(1, 2), decay_mult=(1, 0), weight_filler=f("xavier")),
              nets.fc(4, lr_mult=(1, 1), decay_mult=(1, 1), weight_filler=f("xavier")), nets.softmax_loss()]
    ref = nets.Net(8, 2, 10, layers, sp)
    a, b = _blobs(net, nets.MODEL, nets.BIAS), _blobs(ref, nets.MODEL, nets.BIAS)
    assert len(a) == len(b) == 8
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    assert net.parameter_size() == sum(x.size for x in a) == 6 * 2 * 9 + 6 + 8 * 3 * 9 + 8 + 4 * 8 * 9 + 4
    # fillers: gaussian(0, 0.05), constants, xavier bound sqrt(3 / fan_in) with fan_in = d*k*k
    w1 = a[0]
    assert abs(w1.std() - 0.05) < 0.015 and abs(w1.mean()) < 0.02 and np.unique(w1).size == w1.size
    assert np.all(a[1] == np.float32(0.25)) and np.all(a[4] == 0) and np.all(a[5] == 0)
    for w, fan_in in ((a[2], 3 * 9), (a[3], 3 * 9), (a[6], 8 * 9)):
        bound = np.sqrt(3.0 / fan_in)
        assert np.abs(w).max() <= bound * (1 + 1e-6) and np.abs(w).max() > 0.7 * bound
    # the two networks train identically
    from caffecontroll_amd import solver as S
    for x, y in _batches(3):
        for n_ in (net, ref):
            S.upload_batch(n_, x, y)
            n_.forward()
            n_.backward()
        assert net.loss() == ref.loss()
    for x, y in zip(_blobs(net, nets.MODEL, nets.BIAS), _blobs(ref, nets.MODEL, nets.BIAS)):
        assert np.array_equal(x, y)
    net.close()
    ref.close()


def test_model_file_layout_and_snapshot_resume(tmp_path):
    from caffecontroll_amd import CctHipError, nets
    from caffecontroll_amd import solver as S
    sp, ctl, nd, net = _build()
    data = _batches(6)

    def step(n_, xy):
        S.upload_batch(n_, *xy)
        n_.forward()
        n_.backward()

    for xy in data[:3]:
        step(net, xy)
    stem = net.write_snapshot(str(tmp_path / "solver.prototxt"), 3)
    assert stem.endswith("solver.prototxt.snapshot_iter3")
    model, hist = _blobs(net, nets.MODEL, nets.BIAS), _blobs(net, nets.MODEL_HISTORY, nets.BIAS_HISTORY)
    # byte layout: raw fp32, per layer the model then the bias; one int in the ITER file
    assert np.array_equal(np.fromfile(stem + ".MODEL.bin", np.float32), np.concatenate(model))
    assert np.array_equal(np.fromfile(stem + ".HISTORY.bin", np.float32), np.concatenate(hist))
    assert np.fromfile(stem + ".ITER.bin", np.int32).tolist() == [3]
    assert any(np.abs(h).max() > 0 for h in hist)
    for xy in data[3:]:
        step(net, xy)
    final = _blobs(net, nets.MODEL, nets.BIAS)
    loss_final = net.loss()

    # a fresh network restored from the snapshot continues bit for bit (weights, momentum and
    # the position in the learning-rate schedule)
    sp2, _, nd2, net2 = _build()
    assert net2.read_snapshot(stem) == 3
    for x, y in zip(_blobs(net2, nets.MODEL_HISTORY, nets.BIAS_HISTORY), hist):
        assert np.array_equal(x, y)
    for xy in data[3:]:
        step(net2, xy)
    assert net2.loss() == loss_final
    for x, y in zip(_blobs(net2, nets.MODEL, nets.BIAS), final):
        assert np.array_equal(x, y)
    # without the iteration counter the schedule restarts and the result differs
    sp3, _, nd3, net3 = _build()
    net3.read_snapshot(stem)
    net3.set_iter(0)
    for xy in data[3:]:
        step(net3, xy)
    assert not all(np.array_equal(x, y) for x, y in zip(_blobs(net3, nets.MODEL, nets.BIAS), final))

    # model file alone
    mf = str(tmp_path / "model.bin")
    net.write_model(mf)
    assert os.path.getsize(mf) == 4 * net.parameter_size()
    net3.read_model(mf)
    for x, y in zip(_blobs(net3, nets.MODEL, nets.BIAS), final):
        assert np.array_equal(x, y)
    # errors: missing file, truncated file
    with pytest.raises(CctHipError, match="Error opening"):
        net3.read_model(str(tmp_path / "absent.bin"))
    with open(mf, "rb") as f_:
        head = f_.read(100)
    with open(str(tmp_path / "short.bin"), "wb") as f_:
        f_.write(head)
    with pytest.raises(CctHipError, match="fewer values"):
        net3.read_model(str(tmp_path / "short.bin"))
    with pytest.raises(CctHipError):
        net3.write_model(str(tmp_path / "no_such_dir" / "m.bin"))
    for n_ in (net, net2, net3):
        n_.close()


def test_training_loop_learns_and_reports(tmp_path):
    from caffecontroll_amd import solver as S
    sp, ctl, nd, net = _build()
    lines = []
    out = str(tmp_path / "out.bin")
    ctl = dict(ctl, snapshot=8, snapshot_prefix=str(tmp_path / "snap"), test_interval=12)
    reports = S.train(net, sp, ctl, _batches(5), test_batches=_batches(2, seed=9), output_model_file=out, log=lines.append)
    assert [r[0] for r in reports] == [3, 7, 11]
    assert reports[-1][1] < reports[0][1] and reports[-1][1] < 0.7 and reports[-1][2] > 0.8
    assert sum("Training Status Report" in l for l in lines) == 3
    assert any(l.startswith("Training Status Report (Epoch 1 / Mini-batch iter 7)") for l in lines)
    assert sum("Writing snapshot" in l for l in lines) == 1 and any("Loss = " in l for l in lines)
    assert os.path.getsize(out) == 4 * net.parameter_size()
    assert len([f for f in os.listdir(tmp_path) if f.startswith("snap.")]) == 1
    # LR printed for the report after iteration 3 follows the inv policy at iter 4
    want = 0.05 * (1 + 0.01 * 4) ** -0.75
    assert ("LR = %g" % want) in lines[0]
    loss, acc = S.test(net, _batches(2, seed=11), log=None)
    assert acc > 0.8 and loss < 0.7
    with pytest.raises(ValueError):
        S.upload_batch(net, np.zeros((8, 2, 9, 9), np.float32), np.zeros(8))
    net.close()


TOWER_TEXT = """
name: "towers"
layer { name: "data" type: "Data" top: "data" top: "label" data_param { source: "none" batch_size: 6 } }
layer { name: "conv1" type: "Convolution" bottom: "data" top: "conv1" param { lr_mult: 1 } param { lr_mult: 2 decay_mult: 0 }
        convolution_param { num_output: 8 kernel_size: 3 pad: 1 weight_filler { type: "gaussian" std: 0.2 }
                            bias_filler { type: "constant" value: 0.1 } } }
layer { name: "relu1" type: "ReLU" bottom: "conv1" top: "conv1" }
layer { name: "pool1" type: "Pooling" bottom: "conv1" top: "pool1" pooling_param { pool: MAX kernel_size: 2 stride: 2 } }
layer { name: "norm1" type: "LRN" bottom: "pool1" top: "norm1" lrn_param { local_size: 3 alpha: 0.01 beta: 0.75 } }
layer { name: "conv2" type: "Convolution" bottom: "norm1" top: "conv2"
        convolution_param { num_output: 6 kernel_size: 3 pad: 1 weight_filler { type: "xavier" } } }
layer { name: "relu2" type: "ReLU" bottom: "conv2" top: "conv2" }
layer { name: "pool2" type: "Pooling" bottom: "conv2" top: "pool2" pooling_param { pool: MAX kernel_size: 2 stride: 2 } }
layer { name: "conv2b" type: "Convolution" bottom: "norm1" top: "conv2b"
        convolution_param { num_output: 10 kernel_size: 3 pad: 1 group: 2 weight_filler { type: "xavier" } } }
layer { name: "relu2b" type: "ReLU" bottom: "conv2b" top: "conv2b" }
layer { name: "pool2b" type: "Pooling" bottom: "conv2b" top: "pool2b" pooling_param { pool: MAX kernel_size: 2 stride: 2 } }
layer { name: "concat" type: "Concat" bottom: "pool2" bottom: "pool2b" top: "concat" }
layer { name: "fc6" type: "InnerProduct" bottom: "concat" top: "fc6"
        inner_product_param { num_output: 16 weight_filler { type: "gaussian" std: 0.1 } bias_filler { type: "constant" value: 0.05 } } }
layer { name: "relu6" type: "ReLU" bottom: "fc6" top: "fc6" }
layer { name: "fc8" type: "InnerProduct" bottom: "fc6" top: "fc8" inner_product_param { num_output: 5 weight_filler { type: "xavier" } } }
layer { name: "loss" type: "SoftmaxWithLoss" bottom: "fc8" bottom: "label" top: "loss" }
"""
TOWER_SOLVER = 'base_lr: 0.05 momentum: 0.9 weight_decay: 0.001 lr_policy: "fixed" max_iter: 4 random_seed: 11'


@pytest.mark.parametrize("text, solver_text, depth, size", [(NET_TEXT, 'base_lr: 0.05 momentum: 0.9 weight_decay: 0.0005 lr_policy: "fixed" random_seed: 77', 2, 10),
                                                            (TOWER_TEXT, TOWER_SOLVER, 3, 12)], ids=["chain", "two-towers"])
def test_prototxt_network_trains_like_the_oracle(oracle, text, solver_text, depth, size):
    """From configuration text to trained weights, against the oracle: the network the front end
    builds (fillers, multipliers, groups, a blob read by two towers, Concat) is run for three
    iterations on the device and by the oracle graph on the same filler-drawn weights; every
    layer's output, every gradient and every updated weight agree within 1e-4."""
    from caffecontroll_amd import nets, prototxt as P
    from gpu_util import rel_err
    from oracle.oracle_net import OracleGraph
    sp, _ = P.solver_from_prototxt(solver_text)
    nd = P.network_from_prototxt(text)
    driver()
    net = nd.build(depth=depth, size=size, solver=sp)
    layers, B = nd.layers, nd.batch_size
    solver = dict(base_lr=sp.base_lr, momentum=sp.momentum, weight_decay=sp.weight_decay)
    ref = OracleGraph(oracle, layers, B, depth, size, solver)
    for (li, gi), p in ref.params.items():          # the weights the device drew with the prototxt's fillers
        p["w"][...] = _down(*net.tensor(li, nets.MODEL, gi)).reshape(p["w"].shape)
        p["b"][...] = _down(*net.tensor(li, nets.BIAS, gi))
        assert np.abs(p["w"]).max() > 0
    classes = ref.params[max(ref.params)]["b"].size
    rng = np.random.default_rng(21)
    up = lambda ptr, a: driver().memcpy(ptr, np.ascontiguousarray(a).ctypes.data, a.nbytes, 0)
    for it in range(3):
        x = rng.standard_normal((B, depth, size, size)).astype(np.float32)
        labels = rng.integers(0, classes, B).astype(np.float32)
        up(net.input_ptr(), x)
        up(net.labels_ptr(), labels)
        net.forward()
        ref.forward(x, labels)
        for li, L in enumerate(layers):
            if L.type in (nets.RELU, nets.DROPOUT):
                continue
            want = ref.val[ref.blob[li]] if li != len(layers) - 1 else ref.out[li]
            assert rel_err(_down(*net.tensor(li, nets.OUTPUT)), want.reshape(-1)) <= 1e-4, (it, nd.names[li])
            if L.type == nets.MAXPOOL:
                ptr, n = net.tensor(li, nets.AUX)
                want = ref.saved[(li, "idx")].reshape(-1).astype(np.int32)
                got = np.empty(n, np.int32)
                driver().memcpy(got.ctypes.data, ptr, got.nbytes, 1)
                assert np.count_nonzero(got != want) <= 1
                up(ptr, want)
        assert abs(net.loss() - ref.loss) <= 1e-4 * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        for (li, gi), p in sorted(ref.params.items()):
            for which, key in ((nets.MODEL, "w"), (nets.BIAS, "b")):
                assert rel_err(_down(*net.tensor(li, which, gi)), p[key].reshape(-1)) <= 1e-4, (it, nd.names[li], key)
            for which, hist in ((nets.MODEL_HISTORY, "hw"), (nets.BIAS_HISTORY, "hb")):
                assert rel_err(_down(*net.tensor(li, which, gi)), p[hist]) <= 1e-4, (it, nd.names[li], hist)
    net.close()
