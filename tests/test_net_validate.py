"""Host-side rejection of malformed layer chains, solver fields and labels (no device is touched):
`cct_net_validate` is what `cct_net_create` runs first, `NetworkDef.validate` maps its message to
the prototxt's layer name, `solver.check_labels` guards the index the loss layer reads with."""
import numpy as np
import pytest

from caffecontroll_amd import CctHipError, nets, prototxt
from caffecontroll_amd.bridges import solver_param
from caffecontroll_amd.solver import check_labels


def test_reference_shaped_chains_pass():
    nets.validate(64, 1, 28, nets.lenet_layers())
    nets.validate(256, 3, 227, nets.caffenet_layers())
    nets.validate(2, 3, 227, nets.caffenet_layers(groups=False, num_classes=10))


@pytest.mark.parametrize("layers, fragment", [
    ([nets.conv(8, 3, stride=0)], "stride >= 1"),
    ([nets.conv(8, 0)], "kernel_size >= 1"),
    ([nets.conv(8, 3, pad=-1)], "pad >= 0"),
    ([nets.conv(0, 3)], "num_output >= 1"),
    ([nets.conv(8, 31)], "exceeds the padded input"),
    ([nets.conv(8, 3), nets.maxpool(2, 2), nets.conv(8, 16, pad=1)], "layer 2: kernel_size 16 exceeds the padded input (15)"),
    ([nets.conv(9, 3, group=2)], "group must divide"),
    ([nets.conv(8, 3), nets.conv(8, 3, group=3)], "layer 1: group must divide"),
    ([nets.maxpool(3, 0)], "stride >= 1"),
    ([nets.maxpool(0, 1)], "kernel_size >= 1"),
    ([nets.maxpool(29, 2)], "pooling kernel_size 29 exceeds the input (28)"),
    ([nets.fc(0)], "num_output >= 1"),
    ([nets.lrn(local_size=4)], "odd"),
    ([nets.lrn(local_size=0)], "odd"),
    ([nets.lrn(alpha=float("nan"))], "finite"),
    ([nets.dropout(1.0)], "[0, 1)"),
    ([nets.dropout(-0.1)], "[0, 1)"),
    ([nets.dropout(float("nan"))], "[0, 1)"),
    ([nets._spec(42)], "unknown layer type 42"),
    ([nets.conv(1 << 20, 1)], "2^31 elements"),
])
def test_bad_layers_are_rejected_with_the_layer_named(layers, fragment):
    with pytest.raises(CctHipError) as e:
        nets.validate(4, 2, 28, layers + [nets.softmax_loss()])
    assert fragment in str(e.value), str(e.value)


def test_bad_filler_type():
    c = nets.conv(8, 3)
    c.weight_filler.type = 9
    with pytest.raises(CctHipError, match="unknown filler type"):
        nets.validate(4, 2, 28, [c])


@pytest.mark.parametrize("kw, fragment", [
    (dict(lr_policy="multistep"), "lr_policy"),
    (dict(lr_policy="cosine"), "lr_policy"),
    (dict(lr_policy="step", stepsize=0), "stepsize >= 1"),
    (dict(lr_policy="poly", max_iter=0), "max_iter >= 1"),
    (dict(regularization_type="L3"), "L2 or L1"),
])
def test_bad_solver_fields(kw, fragment):
    with pytest.raises(CctHipError) as e:
        nets.validate(4, 1, 28, nets.lenet_layers(), solver_param(**kw))
    assert fragment in str(e.value)


def test_bad_sizes():
    for b, d, n in ((0, 1, 28), (4, 0, 28), (4, 1, 0), (-1, 1, 28)):
        with pytest.raises(CctHipError, match="positive"):
            nets.validate(b, d, n, nets.lenet_layers())
    with pytest.raises(CctHipError, match="no layers"):
        nets.validate(4, 1, 28, [])


def test_bad_filler_parameters_are_refused_not_fatal():
    """What the filler draws would refuse is said by the validation walk, with the layer's index: a negative or
    non-finite gaussian std, a bernoulli probability outside [0, 1]; std 0 (constant weights in the reference) passes."""
    def chain(**kw):
        return [nets.conv(4, 3, **kw), nets.fc(3), nets.softmax_loss()]
    nets.validate(2, 1, 8, chain(weight_filler=nets.filler("gaussian", std=0.0)))
    for kw, fragment in ((dict(weight_filler=nets.filler("gaussian", std=-1.0)), "layer 0: weight filler: gaussian std"),
                         (dict(bias_filler=nets.filler("gaussian", std=float("nan"))), "layer 0: bias filler: gaussian std"),
                         (dict(weight_filler=nets.filler("bernoulli", value=1.5)), "bernoulli probability"),
                         (dict(bias_filler=nets.filler("constant", value=float("inf"))), "constant value")):
        with pytest.raises(CctHipError) as e:
            nets.validate(2, 1, 8, chain(**kw))
        assert fragment in str(e.value)
    with pytest.raises(CctHipError, match="layer 1: weight filler"):
        nets.validate(2, 1, 8, [nets.conv(4, 3), nets.fc(3, weight_filler=nets.filler("bernoulli", value=-0.1)),
                                nets.softmax_loss()])


def test_net_create_refuses_before_touching_a_device():
    """cct_net_create runs the same check first: on this path nothing device-side is reached, so
    the call is safe (and meaningful) on a machine without a GPU."""
    with pytest.raises(CctHipError, match="exceeds the padded input"):
        nets.Net(4, 1, 28, [nets.conv(8, 40), nets.softmax_loss()])


NET_TEXT = """
name: "t"
layer { name: "data" type: "Data" top: "data" top: "label" data_param { batch_size: 4 } transform_param { crop_size: 20 } }
layer { name: "c1" type: "Convolution" bottom: "data" top: "c1" convolution_param { num_output: 8 kernel_size: %(k)d stride: %(s)d } }
layer { name: "p1" type: "Pooling" bottom: "c1" top: "p1" pooling_param { pool: MAX kernel_size: %(pk)d stride: 2 } }
layer { name: "n1" type: "LRN" bottom: "p1" top: "n1" lrn_param { local_size: %(ls)d } }
layer { name: "d1" type: "Dropout" bottom: "n1" top: "n1" dropout_param { dropout_ratio: %(dr)g } }
layer { name: "ip" type: "InnerProduct" bottom: "n1" top: "ip" inner_product_param { num_output: 10 } }
layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip" bottom: "label" }
"""


def _net(**kw):
    f = dict(k=3, s=1, pk=2, ls=5, dr=0.5)
    f.update(kw)
    return prototxt.network_from_prototxt(NET_TEXT % f)


def test_prototxt_mirror_names_the_layer():
    _net().validate(3)  # the well-formed file passes
    for kw, name in ((dict(s=0), "c1"), (dict(ls=4), "n1"), (dict(dr=1.0), "d1"), (dict(k=0), "c1")):
        with pytest.raises(prototxt.PrototxtError) as e:
            _net(**kw)
        assert repr(name) in str(e.value)
    with pytest.raises(prototxt.PrototxtError) as e:
        _net(k=21).validate(3)       # only the geometry walk can see that 21 > 20
    assert "'c1'" in str(e.value) and "exceeds the padded input" in str(e.value)
    with pytest.raises(prototxt.PrototxtError) as e:
        _net(pk=19).validate(3)
    assert "'p1'" in str(e.value)
    with pytest.raises(prototxt.PrototxtError) as e:
        _net(k=21).build(3)          # build() validates before it creates anything
    assert "'c1'" in str(e.value)


def test_check_labels():
    ok = check_labels([0, 3, 9], 10)
    assert ok.dtype == np.float32 and ok.tolist() == [0.0, 3.0, 9.0]
    for bad in ([0, 10], [-1, 2], [float("nan"), 1], [1e9]):
        with pytest.raises(ValueError, match="outside"):
            check_labels(bad, 10)
