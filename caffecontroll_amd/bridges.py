"""Python handles on the C++ operator layer (``include/cct_bridge.h``): a convolution layer run
as ``ParallelizedBridge<ConvolutionBridge>`` with one device partition, the way the reference
builds it for ``gpu_0_batch_proportion: 1.0`` (src/DeepNet.h:1065-1131)."""
import ctypes as C

from . import _lib
from ._lib import check

STAGE_NAMES = ("Lower Cube", "GEMM", "Remap", "Bias",                        # forward
               "Bw Bias", "Bw Remap", "GEMM Data", "Inverse Lwr", "GEMM Wghts")  # backward


class SolverParam(C.Structure):
    _fields_ = [("base_lr", C.c_float), ("momentum", C.c_float), ("gamma", C.c_float), ("power", C.c_float),
                ("weight_decay", C.c_float), ("stepsize", C.c_int), ("max_iter", C.c_int),
                ("random_seed", C.c_int), ("lr_policy", C.c_char_p), ("regularization_type", C.c_char_p)]


class ConvParam(C.Structure):
    _fields_ = [("num_output", C.c_int), ("kernel_size", C.c_int), ("stride", C.c_int), ("pad", C.c_int),
                ("bias_term", C.c_int), ("lr_mult_weights", C.c_float), ("lr_mult_bias", C.c_float),
                ("decay_mult_weights", C.c_float), ("decay_mult_bias", C.c_float)]


_P, _I = C.c_void_p, C.c_int
BRIDGE_PROTOTYPES = {
    "cct_conv_bridge_create": ([C.POINTER(_P), _I, _I, _I, C.POINTER(ConvParam), C.POINTER(SolverParam),
                                _P, _P, _P, _P], _I),
    "cct_conv_bridge_create_shared": ([C.POINTER(_P), _I, _I, _I, C.POINTER(ConvParam), C.POINTER(SolverParam),
                                       _P, _P, _P, _P, _I, _I], _I),
    "cct_conv_bridge_destroy": ([_P], _I),
    "cct_conv_bridge_set_options": ([_P, _I, _I, _I], _I),
    "cct_conv_bridge_path": ([_P], _I),
    "cct_conv_bridge_model": ([_P], _P),
    "cct_conv_bridge_bias": ([_P], _P),
    "cct_conv_bridge_model_grad": ([_P], _P),
    "cct_conv_bridge_bias_grad": ([_P], _P),
    "cct_conv_bridge_lowered": ([_P], _P),
    "cct_conv_bridge_history": ([_P], _P),
    "cct_conv_bridge_forward": ([_P], _I),
    "cct_conv_bridge_backward": ([_P, _I], _I),
    "cct_conv_bridge_set_staging": ([_P, _I], _I),
    "cct_conv_bridge_staging": ([_P], _I),
    "cct_conv_bridge_share_with_next": ([_P, _P, _P], _I),
    "cct_conv_bridge_stage_ms": ([_P, C.POINTER(C.c_float)], _I),
    "cct_conv_bridge_stage_kernel": ([_P, _I], C.c_char_p),
}
_bound = False


def _bind():
    global _bound
    lib = _lib.load()
    if not _bound:
        for name, (argtypes, restype) in BRIDGE_PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, restype
        _bound = True
    return lib


def solver_param(base_lr=0.01, momentum=0.0, weight_decay=0.0, lr_policy="fixed", gamma=0.1, stepsize=100000,
                 power=0.0, max_iter=0, random_seed=-1, regularization_type="L2"):
    s = SolverParam()
    s.base_lr, s.momentum, s.gamma, s.power, s.weight_decay = base_lr, momentum, gamma, power, weight_decay
    s.stepsize, s.max_iter, s.random_seed = stepsize, max_iter, random_seed
    s.lr_policy, s.regularization_type = lr_policy.encode(), regularization_type.encode()
    return s


class ConvolutionLayer:
    """ParallelizedBridge<ConvolutionBridge> over caller-provided device tensors.

    ``in_data``/``in_grad``: [b][d][n][n]; ``out_data``/``out_grad``: [b][o][m][m] (objects with
    ``data_ptr()``; they must stay alive as long as this object)."""

    def __init__(self, b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad, bias_term=True,
                 solver=None, lr_mult=(1.0, 1.0), decay_mult=(1.0, 1.0), share_prev=True, share_next=True):
        """share_prev / share_next = False: the input / output layer is HOST memory (contiguous float32
        numpy arrays); the bridge then copies to and from its own device cubes, as the reference's
        ParallelizedBridge does for a bridge whose neighbour is not on the same device."""
        self.lib = _bind()
        self.shape = (b, d, n, k, s, p, o)
        self.m = (n + 2 * p - k) // s + 1
        cp = ConvParam(o, k, s, p, int(bias_term), lr_mult[0], lr_mult[1], decay_mult[0], decay_mult[1])
        self._solver = solver or solver_param()
        self._keep = (in_data, in_grad, out_data, out_grad)
        h = C.c_void_p()
        ptr = lambda t: None if t is None else (t.data_ptr() if hasattr(t, "data_ptr") else t.ctypes.data)
        check(self.lib.cct_conv_bridge_create_shared(C.byref(h), b, d, n, C.byref(cp), C.byref(self._solver),
                                                     ptr(in_data), ptr(in_grad), ptr(out_data), ptr(out_grad),
                                                     int(share_prev), int(share_next)),
              "conv_bridge_create")
        self.h = h

    def set_options(self, fused=None, profile=False, needs_backward_grad=True):
        """fused: path level 0..3 (0 separate passes, 1 fused epilogues, 2 direct data gradient,
        3 all-direct, no lowered matrix); None keeps the bridge's default (3 where the geometry is
        covered by the direct kernels, else 1).  True/False mean "default" / 0."""
        if fused is None or fused is True:
            level = -1
        elif fused is False:
            level = 0
        else:
            level = int(fused)
        check(self.lib.cct_conv_bridge_set_options(self.h, level, int(profile), int(needs_backward_grad)),
              "conv_bridge_set_options")

    def path(self):
        """Path level in effect (0..3)."""
        return self.lib.cct_conv_bridge_path(self.h)

    def set_staging(self, overlapped=True):
        """Host-resident layers: move the batch in pieces with copies and kernels overlapped (default), or as
        one blocking copy in, the pass, one blocking copy out."""
        check(self.lib.cct_conv_bridge_set_staging(self.h, int(overlapped)), "conv_bridge_set_staging")

    def share_with_next(self, out_data, out_grad):
        """Raise share_pointer_with_next_bridge on a bridge created with a host-resident output layer: its output
        layer becomes these DEVICE tensors ([b][o][m][m]) and the copies to / from the host stop."""
        self._keep = self._keep + (out_data, out_grad)
        check(self.lib.cct_conv_bridge_share_with_next(self.h, out_data.data_ptr(), out_grad.data_ptr()),
              "conv_bridge_share_with_next")

    def staging_overlapped(self):
        return bool(self.lib.cct_conv_bridge_staging(self.h))

    # device addresses of the cubes the reference exposes on the bridge
    def model_ptr(self):
        return self.lib.cct_conv_bridge_model(self.h)

    def bias_ptr(self):
        return self.lib.cct_conv_bridge_bias(self.h)

    def model_grad_ptr(self):
        return self.lib.cct_conv_bridge_model_grad(self.h)

    def bias_grad_ptr(self):
        return self.lib.cct_conv_bridge_bias_grad(self.h)

    def lowered_ptr(self):
        return self.lib.cct_conv_bridge_lowered(self.h)

    def history_ptr(self):
        return self.lib.cct_conv_bridge_history(self.h)

    def forward(self):
        check(self.lib.cct_conv_bridge_forward(self.h), "conv_bridge_forward")

    def backward(self, with_update=False):
        check(self.lib.cct_conv_bridge_backward(self.h, int(with_update)), "conv_bridge_backward")

    def stage_ms(self):
        arr = (C.c_float * len(STAGE_NAMES))()
        check(self.lib.cct_conv_bridge_stage_ms(self.h, arr), "conv_bridge_stage_ms")
        return dict(zip(STAGE_NAMES, list(arr)))

    def stage_kernels(self):
        """Stage name -> kernel instance the library launched for it ("" if the stage did not run)."""
        return {name: (self.lib.cct_conv_bridge_stage_kernel(self.h, i) or b"").decode()
                for i, name in enumerate(STAGE_NAMES)}

    def close(self):
        if self.h:
            self.lib.cct_conv_bridge_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
