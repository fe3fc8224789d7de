"""Layer chains on the device (``cct_net_*`` of ``include/cct_bridge.h``) and the two networks of
the benchmark configurations: LeNet and CaffeNet/AlexNet."""
import ctypes as C
import os

from . import _lib
from ._lib import check
from .bridges import SolverParam, solver_param  # noqa: F401

CONV, FC, RELU, MAXPOOL, LRN, DROPOUT, SOFTMAXLOSS, CONCAT = 1, 2, 3, 4, 5, 6, 7, 8
MAX_BOTTOMS = 4


FILLER_TYPES = {"constant": 0, "xavier": 1, "gaussian": 2, "bernoulli": 3}


class Filler(C.Structure):
    """cnn.proto FillerParameter: type, value (constant / bernoulli p), mean and std (gaussian)."""
    _fields_ = [("type", C.c_int), ("value", C.c_float), ("mean", C.c_float), ("std", C.c_float)]


def filler(type="constant", value=0.0, mean=0.0, std=1.0):
    if type not in FILLER_TYPES:
        raise ValueError("unknown filler type %r" % (type,))
    return Filler(FILLER_TYPES[type], value, mean, std)


class LayerSpec(C.Structure):
    _fields_ = [("type", C.c_int), ("num_output", C.c_int), ("kernel_size", C.c_int), ("stride", C.c_int),
                ("pad", C.c_int), ("group", C.c_int), ("bias_term", C.c_int), ("lrn_local_size", C.c_int),
                ("lrn_alpha", C.c_float), ("lrn_beta", C.c_float), ("dropout_ratio", C.c_float),
                ("lr_mult", C.c_float * 2), ("decay_mult", C.c_float * 2),
                ("weight_filler", Filler), ("bias_filler", Filler),
                ("n_bottoms", C.c_int), ("bottoms", C.c_int * MAX_BOTTOMS)]

    def read_from(self, *layer_indices):
        """The layers whose outputs this layer reads (index in the layer list, -1 = the network
        input); without it a layer reads the one before it.  Returns self."""
        if not 1 <= len(layer_indices) <= MAX_BOTTOMS:
            raise ValueError("a layer has 1..%d bottoms" % MAX_BOTTOMS)
        self.n_bottoms = len(layer_indices)
        for j, b in enumerate(layer_indices):
            self.bottoms[j] = b
        return self


def _spec(t, **kw):
    s = LayerSpec()
    s.type, s.stride, s.group, s.bias_term = t, 1, 1, 1
    s.lr_mult[0], s.lr_mult[1], s.decay_mult[0], s.decay_mult[1] = 1.0, 2.0, 1.0, 0.0
    s.weight_filler, s.bias_filler = filler(), filler()
    for k, v in kw.items():
        if k in ("lr_mult", "decay_mult"):
            getattr(s, k)[0], getattr(s, k)[1] = v
        else:
            setattr(s, k, v)
    return s


def conv(num_output, kernel_size, stride=1, pad=0, group=1, **kw):
    return _spec(CONV, num_output=num_output, kernel_size=kernel_size, stride=stride, pad=pad, group=group, **kw)


def fc(num_output, **kw):
    return _spec(FC, num_output=num_output, **kw)


def relu():
    return _spec(RELU)


def maxpool(kernel_size, stride):
    return _spec(MAXPOOL, kernel_size=kernel_size, stride=stride)


def lrn(local_size=5, alpha=1e-4, beta=0.75):
    return _spec(LRN, lrn_local_size=local_size, lrn_alpha=alpha, lrn_beta=beta)


def dropout(ratio=0.5):
    return _spec(DROPOUT, dropout_ratio=ratio)


def softmax_loss():
    return _spec(SOFTMAXLOSS)


def concat(*layer_indices):
    """Depth-wise concatenation of the outputs of the given layers."""
    return _spec(CONCAT).read_from(*layer_indices)


def lenet_layers():
    """tests/lenet_train/lenet_train_test.prototxt of the reference: conv(20,5)-pool2-conv(50,5)-pool2-
    ip500-relu-ip10-softmax loss; lr_mult 1 (weights) / 2 (bias), decay_mult left at its default 1 for
    both, xavier weights and zero biases."""
    kw = dict(decay_mult=(1.0, 1.0), weight_filler=filler("xavier"))
    return [conv(20, 5, **kw), maxpool(2, 2), conv(50, 5, **kw), maxpool(2, 2), fc(500, **kw), relu(), fc(10, **kw),
            softmax_loss()]


def caffenet_layers(groups=True, num_classes=1000):
    """tests/imagenet_train/train_val/alexnet_train_val_1GPU.prototxt of the reference (layer order
    conv-relu-pool-norm).  ``groups=True`` runs conv2/4/5 as two channel groups, as the original
    network defines them; the reference itself ignores `group` (src/DeepNet.h:1075-1077)."""
    g = 2 if groups else 1
    return [conv(96, 11, stride=4), relu(), maxpool(3, 2), lrn(),
            conv(256, 5, pad=2, group=g), relu(), maxpool(3, 2), lrn(),
            conv(384, 3, pad=1), relu(),
            conv(384, 3, pad=1, group=g), relu(),
            conv(256, 3, pad=1, group=g), relu(), maxpool(3, 2),
            fc(4096), relu(), dropout(0.5), fc(4096), relu(), dropout(0.5), fc(num_classes), softmax_loss()]


_P, _I = C.c_void_p, C.c_int
NET_PROTOTYPES = {
    "cct_net_create": ([C.POINTER(_P), _I, _I, _I, C.POINTER(LayerSpec), _I, C.POINTER(SolverParam)], _I),
    "cct_net_destroy": ([_P], _I),
    "cct_net_input": ([_P], _P),
    "cct_net_labels": ([_P], _P),
    "cct_net_num_layers": ([_P], _I),
    "cct_net_tensor": ([_P, _I, _I, _I, C.POINTER(C.c_size_t)], _P),
    "cct_net_set_train": ([_P, _I], _I),
    "cct_net_freeze_dropout_masks": ([_P, _I], _I),
    "cct_net_set_conv_path": ([_P, _I], _I),
    "cct_net_forward": ([_P], _I),
    "cct_net_backward": ([_P], _I),
    "cct_net_loss": ([_P, C.POINTER(C.c_float)], _I),
    "cct_net_set_profiling": ([_P, _I], _I),
    "cct_net_layer_ms": ([_P, _I, C.POINTER(C.c_float), C.POINTER(C.c_float)], _I),
    "cct_net_update_ms": ([_P, C.POINTER(C.c_float)], _I),
    "cct_net_conv_bridges": ([_P, _I], _I),
    "cct_net_conv_stage_ms": ([_P, _I, _I, C.POINTER(C.c_float)], _I),
    "cct_net_conv_stage_kernel": ([_P, _I, _I, _I], C.c_char_p),
    "cct_net_write_model": ([_P, C.c_char_p], _I),
    "cct_net_read_model": ([_P, C.c_char_p], _I),
    "cct_net_write_snapshot": ([_P, C.c_char_p, _I], _I),
    "cct_net_read_snapshot": ([_P, C.c_char_p, C.POINTER(_I)], _I),
    "cct_net_set_iter": ([_P, _I], _I),
    "cct_net_get_iter": ([_P], _I),
    "cct_net_num_classes": ([_P], _I),
    "cct_net_validate": ([_I, _I, _I, C.POINTER(LayerSpec), _I, C.POINTER(SolverParam)], _I),
    "cct_solver_learning_rate": ([C.POINTER(SolverParam), _I], C.c_float),
    "cct_net_parameter_size": ([_P], C.c_size_t),
}
_bound = False


def _bind():
    global _bound
    lib = _lib.load()
    if not _bound:
        for name, (argtypes, restype) in NET_PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, restype
        _bound = True
    return lib


MODEL, BIAS, MODEL_GRAD, BIAS_GRAD, OUTPUT, INPUT_GRAD, AUX, MODEL_HISTORY, BIAS_HISTORY = range(9)


def solver_learning_rate(solver, iteration):
    """Util::get_learning_rate (src/util.h:76-93) for the solver's policy at `iteration`, from the
    C++ host layer (no device needed); NaN for a policy the reference rejects."""
    return _bind().cct_solver_learning_rate(C.byref(solver), int(iteration))


def validate(batch, depth, size, layers, solver=None):
    """Checks a layer chain the way `Net` does, without touching a device; raises CctHipError with
    the offending layer in the message."""
    lib = _bind()
    layers = list(layers)
    arr = (LayerSpec * len(layers))(*layers)
    sp = solver or solver_param()
    check(lib.cct_net_validate(batch, depth, size, arr, len(layers), C.byref(sp)), "net_validate")


class Net:
    """A chain of layers resident on the device; one ``forward()`` + ``backward()`` is one training
    iteration (gradients and SGD update of every layer)."""

    def __init__(self, batch, depth, size, layers, solver=None):
        self.lib = _bind()
        self.layers = list(layers)
        arr = (LayerSpec * len(self.layers))(*self.layers)
        self._solver = solver or solver_param()
        h = C.c_void_p()
        check(self.lib.cct_net_create(C.byref(h), batch, depth, size, arr, len(self.layers),
                                      C.byref(self._solver)), "net_create")
        self.h = h
        self.batch, self.depth, self.size = batch, depth, size

    def input_ptr(self):
        return self.lib.cct_net_input(self.h)

    def labels_ptr(self):
        return self.lib.cct_net_labels(self.h)

    def tensor(self, layer, which, group=0):
        """(device address, element count) or (None, 0)."""
        n = C.c_size_t()
        p = self.lib.cct_net_tensor(self.h, layer, group, which, C.byref(n))
        return p, n.value

    def set_train(self, train):
        check(self.lib.cct_net_set_train(self.h, int(train)), "net_set_train")

    def set_conv_path(self, level):
        """Path level of every convolution layer: 0 staged .. 3 all direct (where covered), -1 default."""
        check(self.lib.cct_net_set_conv_path(self.h, int(level)), "net_set_conv_path")

    def freeze_dropout_masks(self, freeze=True):
        check(self.lib.cct_net_freeze_dropout_masks(self.h, int(freeze)), "net_freeze_dropout_masks")

    def forward(self):
        check(self.lib.cct_net_forward(self.h), "net_forward")

    def backward(self):
        check(self.lib.cct_net_backward(self.h), "net_backward")

    def loss(self):
        v = C.c_float()
        check(self.lib.cct_net_loss(self.h, C.byref(v)), "net_loss")
        return v.value

    # ---- per-layer device times (the breakdown the reference prints per bridge) ----
    def set_profiling(self, on=True):
        check(self.lib.cct_net_set_profiling(self.h, int(on)), "net_set_profiling")

    def layer_ms(self, layer):
        """(forward ms, backward ms) of the layer's last profiled steps; waits for them."""
        f, b = C.c_float(), C.c_float()
        check(self.lib.cct_net_layer_ms(self.h, layer, C.byref(f), C.byref(b)), "net_layer_ms")
        return f.value, b.value

    def update_ms(self):
        v = C.c_float()
        check(self.lib.cct_net_update_ms(self.h, C.byref(v)), "net_update_ms")
        return v.value

    def conv_stages(self, layer):
        """Per bridge of a convolution layer: {stage label: (ms, kernel instance)} of the last profiled pass."""
        from .bridges import STAGE_NAMES
        out = []
        for bi in range(self.lib.cct_net_conv_bridges(self.h, layer)):
            ms = (C.c_float * len(STAGE_NAMES))()
            check(self.lib.cct_net_conv_stage_ms(self.h, layer, bi, ms), "net_conv_stage_ms")
            ent = {}
            for si, name in enumerate(STAGE_NAMES):
                if ms[si] > 0:
                    key = name if name not in ent else name + " (backward)"
                    ent[key] = (ms[si], self.lib.cct_net_conv_stage_kernel(self.h, layer, bi, si).decode())
            out.append(ent)
        return out

    # ---- model files and snapshots in the reference's format (src/DeepNet.h:268-422) ----
    def write_model(self, path):
        check(self.lib.cct_net_write_model(self.h, os.fsencode(path)), "net_write_model")

    def read_model(self, path):
        check(self.lib.cct_net_read_model(self.h, os.fsencode(path)), "net_read_model")

    def write_snapshot(self, base_filename, iteration):
        """Writes <base>.snapshot_iter<N>.MODEL.bin / .HISTORY.bin / .ITER.bin; returns the common stem."""
        check(self.lib.cct_net_write_snapshot(self.h, os.fsencode(base_filename), iteration), "net_write_snapshot")
        return "%s.snapshot_iter%d" % (base_filename, iteration)

    def read_snapshot(self, stem):
        """Restores weights, momentum and the iteration counter; returns the iteration."""
        it = C.c_int()
        check(self.lib.cct_net_read_snapshot(self.h, os.fsencode(stem), C.byref(it)), "net_read_snapshot")
        return it.value

    def set_iter(self, iteration):
        check(self.lib.cct_net_set_iter(self.h, iteration), "net_set_iter")

    def get_iter(self):
        """Number of updates the gradient updaters have applied (their schedule position)."""
        return self.lib.cct_net_get_iter(self.h)

    def num_classes(self):
        """Scores per image entering the loss layer (0 if the chain has none)."""
        return self.lib.cct_net_num_classes(self.h)

    def parameter_size(self):
        return self.lib.cct_net_parameter_size(self.h)

    def close(self):
        if self.h:
            self.lib.cct_net_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
