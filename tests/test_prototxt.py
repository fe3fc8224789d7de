"""The text front end (solver / network prototxt -> layer records) without a GPU.

The hand-written texts below use every syntax form the reference's own files use; when the
reference checkout is present its LeNet / AlexNet / CaffeNet definitions are read too and must map
onto the layer chains this package builds by hand for the benchmark configurations."""
import os

import pytest

from caffecontroll_amd import nets
from caffecontroll_amd import prototxt as P

REF = "/root/reference"

NET = """
name: "tiny"   # a comment
layer {
  name: "pix" type: "Data" top: "data" top: "label"
  include { phase: TRAIN }
  transform_param { scale: 0.00390625 crop_size: 12 mirror: true mean_file: "m.binaryproto" }
  data_param { source: "some/lmdb" batch_size: 6 backend: LMDB }
}
layer {
  name: "pix" type: "Data" top: "data" top: "label"
  include: { phase: TEST }
  transform_param { scale: 0.5 }
  data_param { source: "other/lmdb" batch_size: 3 backend: LMDB }
}
layer {
  name: "conv1" type: "Convolution" bottom: "data" top: "conv1"
  param { lr_mult: 1 } param { lr_mult: 2 decay_mult: 0 }
  convolution_param {
    num_output: 8 kernel_size: 3 pad: 1 group: 2
    weight_filler { type: "gaussian" std: 0.01 }
    bias_filler { type: "constant" value: 1 }
  }
}
layer { name: "relu1" type: "ReLU" bottom: "conv1" top: "conv1" }
layer { name: "pool1" type: "POOLING" bottom: "conv1" top: "pool1" pooling_param { pool: MAX kernel_size: 3 stride: 2 } }
layer { name: "norm1" type: "LRN" bottom: "pool1" top: "norm1" lrn_param { local_size: 3 alpha: 0.0001 beta: 0.75 } }
layer {
  name: "ip1" type: "InnerProduct" bottom: "norm1" top: "ip1"
  blobs_lr: 1 blobs_lr: 2 weight_decay: 1 weight_decay: 0
  inner_product_param { num_output: 5 weight_filler { type: "xavier" } }
  gpu_0_batch_proportion: 1.0
}
layer { name: "drop" type: "Dropout" bottom: "ip1" top: "ip1" dropout_param { dropout_ratio: 0.25 } }
layer { name: "accuracy" type: "Accuracy" bottom: "ip1" bottom: "label" top: "accuracy" include { phase: TEST } }
layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip1" bottom: "label" top: "loss" }
"""

SOLVER = """
net: "a/b.prototxt"
test_iter: 100
test_interval: 500
base_lr: 0.005
lr_policy: "step"
gamma: 0.1
stepsize: 100000
display: 1
max_iter: 500
momentum: 0.9
weight_decay: 0.0005
# snapshot: 10000
"""


def _key(s):
    return (s.type, s.num_output, s.kernel_size, s.stride, s.pad, s.group, s.bias_term, s.lrn_local_size,
            round(s.lrn_alpha, 9), round(s.lrn_beta, 9), round(s.dropout_ratio, 9))


def test_text_format_forms():
    m = P.parse('a: 1 a: 2 b { c: "x" "y" d: -1.5e-3 } e: { f: TRAIN } g: [1, 2, 3] h: true s: \'q\\n\' # tail')
    assert m.all("a") == [1, 2] and m.get("a") == 2
    assert m.msg("b").get("c") == "xy" and m.msg("b").get("d") == -1.5e-3
    assert m.msg("e").get("f") == "TRAIN" and m.all("g") == [1, 2, 3] and m.get("h") is True
    assert m.get("s") == "q\n"
    assert m.msg("absent").get("x", 7) == 7
    for bad in ("a {", "a: }", "{", 'a: "unterminated'):
        with pytest.raises(P.PrototxtError):
            P.parse(bad)


def test_network_mapping():
    nd = P.network_from_prototxt(NET)
    assert nd.name == "tiny" and nd.batch_size == 6 and nd.crop_size == 12 and nd.scale == 0.00390625
    assert nd.mirror is True and nd.mean_file == "m.binaryproto" and nd.source == "some/lmdb"
    assert nd.names == ["conv1", "relu1", "pool1", "norm1", "ip1", "drop", "loss"]
    want = [nets.conv(8, 3, pad=1, group=2), nets.relu(), nets.maxpool(3, 2), nets.lrn(3, 1e-4, 0.75), nets.fc(5),
            nets.dropout(0.25), nets.softmax_loss()]
    assert [_key(s) for s in nd.layers] == [_key(s) for s in want]
    c, ip = nd.layers[0], nd.layers[4]
    # new-style multipliers (absent decay_mult = 1) and old-style ones
    assert tuple(c.lr_mult) == (1.0, 2.0) and tuple(c.decay_mult) == (1.0, 0.0)
    assert tuple(ip.lr_mult) == (1.0, 2.0) and tuple(ip.decay_mult) == (1.0, 0.0)
    assert (c.weight_filler.type, round(c.weight_filler.std, 6)) == (nets.FILLER_TYPES["gaussian"], 0.01)
    assert (c.bias_filler.type, c.bias_filler.value) == (nets.FILLER_TYPES["constant"], 1.0)
    assert ip.weight_filler.type == nets.FILLER_TYPES["xavier"] and ip.bias_filler.type == 0
    assert nd.output_shapes(4, 12) == [(8, 12), (8, 12), (8, 5), (8, 5), (5, 1), (5, 1), (5, 1)]
    # the reference's behaviour: group is ignored
    assert P.network_from_prototxt(NET, groups="ignore").layers[0].group == 1
    # the TEST phase picks the other data layer
    t = P.network_from_prototxt(NET, phase="TEST")
    assert t.batch_size == 3 and t.scale == 0.5 and t.crop_size == 0 and t.names == nd.names


def test_graph_mapping():
    """A blob read by two layers (the reference inserts the Split itself), an explicit Split, and
    Concat: every layer names the index of the layer that last wrote its bottom."""
    # ip1 now reads conv1 (after its in-place ReLU) next to pool1
    nd = P.network_from_prototxt(NET.replace('bottom: "norm1" top: "ip1"', 'bottom: "conv1" top: "ip1"'))
    bottoms = [[s.bottoms[j] for j in range(s.n_bottoms)] for s in nd.layers]
    assert bottoms == [[-1], [0], [1], [2], [1], [4], [5]]
    two = """
    layer { name: "data" type: "Data" top: "data" top: "label" data_param { batch_size: 2 } transform_param { crop_size: 12 } }
    layer { name: "c1" type: "Convolution" bottom: "data" top: "c1" convolution_param { num_output: 4 kernel_size: 3 } }
    layer { name: "sp" type: "Split" bottom: "c1" top: "c1_a" top: "c1_b" }
    layer { name: "a" type: "Convolution" bottom: "c1_a" top: "a" convolution_param { num_output: 3 kernel_size: 3 } }
    layer { name: "b" type: "Convolution" bottom: "c1_b" top: "b" convolution_param { num_output: 5 kernel_size: 3 } }
    layer { name: "cat" type: "Concat" bottom: "a" bottom: "b" top: "cat" }
    layer { name: "ip" type: "InnerProduct" bottom: "cat" top: "ip" inner_product_param { num_output: 2 } }
    layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip" bottom: "label" }
    """
    nd = P.network_from_prototxt(two)
    assert nd.names == ["c1", "a", "b", "cat", "ip", "loss"]
    assert [s.type for s in nd.layers] == [nets.CONV, nets.CONV, nets.CONV, nets.CONCAT, nets.FC, nets.SOFTMAXLOSS]
    assert [[s.bottoms[j] for j in range(s.n_bottoms)] for s in nd.layers] == [[-1], [0], [0], [1, 2], [3], [4]]
    assert nd.output_shapes(3, 12) == [(4, 10), (3, 8), (5, 8), (8, 8), (2, 1), (2, 1)]
    nd.validate(3)
    with pytest.raises(P.PrototxtError, match="channel axis"):
        P.network_from_prototxt(two.replace('top: "cat" }', 'top: "cat" concat_param { axis: 2 } }'))
    with pytest.raises(P.PrototxtError, match="'cat'"):
        P.network_from_prototxt(two.replace("num_output: 5 kernel_size: 3", "num_output: 5 kernel_size: 5")).validate(3)


def test_rejected_networks():
    with pytest.raises(P.PrototxtError, match="BatchNorm"):
        P.network_from_prototxt(NET.replace('type: "LRN"', 'type: "BatchNorm"'))
    with pytest.raises(P.PrototxtError, match="no earlier layer produces"):
        P.network_from_prototxt(NET.replace('bottom: "norm1" top: "ip1"', 'bottom: "nowhere" top: "ip1"'))
    with pytest.raises(P.PrototxtError, match="no SoftmaxWithLoss"):
        P.network_from_prototxt(NET[:NET.index('layer { name: "loss"')])
    with pytest.raises(P.PrototxtError, match="Data layer"):
        P.network_from_prototxt('layer { name: "ip" type: "InnerProduct" bottom: "data" top: "ip" }')
    with pytest.raises(P.PrototxtError, match="MAX"):
        P.network_from_prototxt(NET.replace("pool: MAX", "pool: AVE"))
    with pytest.raises(P.PrototxtError, match="filler"):
        P.network_from_prototxt(NET.replace('"xavier"', '"msra"'))


def test_solver_fields_and_defaults():
    sp, ctl = P.solver_from_prototxt(SOLVER)
    assert abs(sp.base_lr - 0.005) < 1e-9 and abs(sp.momentum - 0.9) < 1e-7 and abs(sp.gamma - 0.1) < 1e-8
    assert sp.lr_policy == b"step" and sp.stepsize == 100000 and sp.max_iter == 500
    assert abs(sp.weight_decay - 0.0005) < 1e-9 and sp.regularization_type == b"L2" and sp.random_seed == -1
    assert ctl == {"net": "a/b.prototxt", "max_iter": 500, "display": 1, "snapshot": 0, "snapshot_prefix": None,
                   "test_iter": [100], "test_interval": 500}
    with pytest.raises(P.PrototxtError):
        P.solver_from_prototxt("base_lr: 0.1")


needs_reference = pytest.mark.skipif(not os.path.isdir(REF), reason="reference checkout not present")


@needs_reference
def test_reference_lenet_files():
    sp, ctl, nd = P.load_solver(REF + "/tests/lenet_train/lenet_solver.prototxt", root=REF)
    assert sp.lr_policy == b"inv" and abs(sp.base_lr - 0.01) < 1e-9 and ctl["max_iter"] == 100
    assert nd.batch_size == 64 and nd.scale == 0.00390625
    assert [_key(s) for s in nd.layers] == [_key(s) for s in nets.lenet_layers()]
    assert [(tuple(s.lr_mult), tuple(s.decay_mult)) for s in nd.layers if s.type in (nets.CONV, nets.FC)] == \
        [(tuple(s.lr_mult), tuple(s.decay_mult)) for s in nets.lenet_layers() if s.type in (nets.CONV, nets.FC)]
    assert nd.layers[0].weight_filler.type == nets.FILLER_TYPES["xavier"]
    assert nd.output_shapes(1, 28)[-1] == (10, 1)


@needs_reference
def test_reference_imagenet_files():
    base = REF + "/tests/imagenet_train/solver/"
    for fname, groups in (("alexnet_solver_1GPU.prototxt", False), ("caffenet_solver_1000.prototxt", True)):
        sp, ctl, nd = P.load_solver(base + fname, root=REF)
        assert nd.batch_size == 256 and nd.crop_size == 227 and sp.lr_policy == b"step"
        want = nets.caffenet_layers(groups=groups)
        if groups:
            want[8].group = 2  # this file of the reference also puts `group: 2` on conv3
        assert [_key(s) for s in nd.layers] == [_key(s) for s in want], fname
        convs = [s for s in nd.layers if s.type == nets.CONV]
        assert [(tuple(s.lr_mult), tuple(s.decay_mult)) for s in convs] == [((1.0, 2.0), (1.0, 0.0))] * 5
        assert all(s.weight_filler.type == nets.FILLER_TYPES["gaussian"] for s in convs)
        assert nd.output_shapes(3, 227)[-1] == (1000, 1)
    # the reference's two-tower network (a blob read by two towers, Concat before fc6)
    nd = P.network_from_prototxt(P.parse_file(REF + "/benchmark/train_val/caffenet_train_val_8_split.prototxt"))
    assert [s.type for s in nd.layers].count(nets.CONV) == 9 and nets.CONCAT in [s.type for s in nd.layers]
    norm1 = nd.names.index("norm1")
    readers = [nd.names[i] for i, s in enumerate(nd.layers) if norm1 in [s.bottoms[j] for j in range(s.n_bottoms)]]
    assert readers == ["conv2", "conv2b"]
    nd.validate(3, 227)
    assert nd.output_shapes(3, 227)[nd.names.index("concat")] == (256, 6)
    # every solver file of the reference's tests resolves to a network this front end accepts
    import glob
    for f in glob.glob(base + "*.prototxt") + glob.glob(REF + "/tests/lenet_train/*solver*.prototxt"):
        P.load_solver(f, root=REF)
