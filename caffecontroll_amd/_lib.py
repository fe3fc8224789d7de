"""ctypes loader for ``libcct_hip.so`` with the prototypes of ``include/cct_hip.h``.

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libcct_hip.so")

ROW_MAJOR, COL_MAJOR, NO_TRANS, TRANS = 101, 102, 111, 112


class CctHipError(RuntimeError):
    pass


class PMapHelper(C.Structure):
    """cct_pmap_helper == struct PMapHelper, src/sched/DeviceHeader.h:25-35."""
    _fields_ = [(n, C.c_size_t) for n in (
        "dR", "dC", "dD", "dB", "sR", "sC", "sD", "sB", "dBR", "dBC", "sBR", "sBC",
        "kR", "kC", "kD", "kB", "stride", "padding")]


class InverseLowerCubeArgs(C.Structure):
    """cct_inverse_lower_cube_args == struct _inverse_lower_cube_arg_helper, src/kernels/lowering.h:22-32."""
    _fields_ = [(n, C.c_size_t) for n in (
        "data_output_width", "data_output_height", "kernel_size", "stride", "padding",
        "iR", "iC", "iD", "iB")]


class PoolArgs(C.Structure):
    """cct_pool_args == struct _pool_forward_arg_helper, src/kernels/pool.h:7-17."""
    _fields_ = [(n, C.c_int) for n in ("stride", "kernel_size", "iR", "iC", "oR", "oC", "D", "B")] + \
               [("max_index", C.c_void_p)]


class SgdJob(C.Structure):
    """cct_sgd_job: one tensor of a batched SGD update."""
    _fields_ = [("n", C.c_size_t), ("model", C.c_void_p), ("gradient", C.c_void_p), ("history", C.c_void_p),
                ("stepsize", C.c_float), ("momentum", C.c_float), ("lam", C.c_float), ("l1", C.c_int)]


class LrnForwardArgs(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("iR", "iC", "iD", "iB", "norm_window", "local_size")] + \
               [("denoms", C.c_void_p)]


class LrnForwardNormalizeArgs(C.Structure):
    _fields_ = [("alpha_over_size", C.c_float), ("beta", C.c_float), ("denoms", C.c_void_p)]


class LrnBackwardArgs(C.Structure):
    _fields_ = [("oR", C.c_int), ("oC", C.c_int), ("oD", C.c_int), ("oB", C.c_int),
                ("alpha_over_size", C.c_float), ("beta", C.c_float),
                ("norm_window", C.c_int), ("local_size", C.c_int),
                ("denoms", C.c_void_p), ("input_data", C.c_void_p), ("output_data", C.c_void_p)]


_P, _I, _F, _Z, _U = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint

# name -> argtypes; every function returns int (0 = ok) unless listed in _RESTYPE
PROTOTYPES = {
    "cct_hip_init": [_I],
    "cct_hip_set_stream": [_P],
    "cct_hip_set_tuning": [C.c_char_p, _I],
    "cct_hip_device_sync": [],
    "cct_hip_last_error": [],
    "cct_hip_last_kernel": [],
    "cct_hip_compute_units": [],
    "cct_hip_malloc": [C.POINTER(_P), _Z],
    "cct_hip_free": [_P],
    "cct_hip_memcpy": [_P, _P, _Z, _I],
    "cct_hip_memset": [_P, _I, _Z],
    "cct_hip_pipe_create": [C.POINTER(_P)],
    "cct_hip_pipe_destroy": [_P],
    "cct_hip_pipe_begin": [_P],
    "cct_hip_pipe_upload": [_P, _P, _P, _Z, C.POINTER(_I)],
    "cct_hip_pipe_wait_upload": [_P, _I],
    "cct_hip_pipe_download": [_P, _P, _P, _Z],
    "cct_hip_pipe_finish": [_P],
    "cct_hip_lower_cube": [_P, _P, C.POINTER(PMapHelper)],
    "cct_hip_inverse_lower_cube": [_P, _P, C.POINTER(InverseLowerCubeArgs)],
    "cct_hip_inverse_lower_cube_bias_backward": [_P, _P, C.POINTER(InverseLowerCubeArgs), _P, _P, _I, _I, _I],
    "cct_hip_remap": [_P, _P, C.POINTER(PMapHelper)],
    "cct_hip_remap_bias_backward": [_P, _P, C.POINTER(PMapHelper), _P],
    "cct_hip_copy_depth_slice": [_P, _P, _I, _I, _I, _I, _Z, _I],
    "cct_hip_sgemm": [_I, _I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I],
    "cct_hip_sgemm_new": [_I, _I, _I, _I, _I, _F, _P, _P, _F, _P],
    "cct_hip_sgemm_new_colsum": [_I, _I, _I, _I, _I, _F, _P, _P, _F, _P, _P, _P, _I, _I],
    "cct_hip_sgemm_new_bias": [_I, _I, _I, _I, _I, _F, _P, _P, _F, _P, _P, _I],
    "cct_hip_sgemm_conv_forward": [_I, _I, _I, _I, _P, _P, _P, _P, _I],
    "cct_hip_conv1x1_supported": [_I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv1x1_forward": [_P, _P, _P, _P, _I, _I, _I, _I, _I],
    "cct_hip_conv1x1_backward_data": [_P, _P, _P, _I, _I, _I, _I],
    "cct_hip_conv1x1_backward_weights": [_P, _P, _P, _P, _I, _I, _I, _I],
    "cct_hip_conv_small_supported": [_I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_small_forward": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_small_backward_weights": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I],
    "cct_hip_fc_small_supported": [_I, _I, _I],
    "cct_hip_fc_small_forward": [_P, _P, _P, _P, _I, _I, _I, _I],
    "cct_hip_fc_small_backward": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "cct_hip_conv_direct_supported": [_I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_direct_slab_floats": [_I, _I, _I, _I],
    "cct_hip_conv_direct_slabs": [_P, _P, _I, _I, _I, _I],
    "cct_hip_conv_direct_forward": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z, _I],
    "cct_hip_conv_direct_backward_data": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z],
    "cct_hip_conv_direct_backward_data_relu": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z, _P],
    "cct_hip_conv_direct_backward_weights": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z],
    "cct_hip_conv_direct_supported_grouped": [_I, _I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_direct_slab_floats_grouped": [_I, _I, _I, _I, _I],
    "cct_hip_conv_direct_slabs_grouped": [_P, _P, _I, _I, _I, _I, _I],
    "cct_hip_conv_direct_forward_grouped": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z, _I, _I],
    "cct_hip_conv_direct_backward_data_grouped": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z, _P, _I],
    "cct_hip_conv_direct_backward_weights_grouped": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _Z, _Z, _I],
    "cct_hip_conv_strided_supported": [_I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_strided_slab_floats": [_I, _I, _I, _I, _I],
    "cct_hip_conv_strided_slabs": [_P, _P, _I, _I, _I, _I, _I],
    "cct_hip_conv_strided_forward": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_strided_backward_weights": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_strided_backward_data_supported": [_I, _I, _I, _I, _I, _I, _I],
    "cct_hip_conv_strided_backward_data_slab_floats": [_I, _I, _I, _I],
    "cct_hip_conv_strided_backward_data_slabs": [_P, _P, _I, _I, _I, _I],
    "cct_hip_conv_strided_backward_data": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I],
    "cct_hip_sgemv": [_I, _I, _I, _F, _P, _P, _F, _P],
    "cct_hip_math_saxpy": [_Z, _F, _P, _P],
    "cct_hip_math_saxpby": [_Z, _F, _P, _F, _P],
    "cct_hip_L1_update": [_I, _P, _F, _P],
    "cct_hip_sgd_update": [_Z, _P, _P, _P, _F, _F, _F, _I],
    "cct_hip_sgd_update_batch": [C.POINTER(SgdJob), _I],
    "cct_hip_sconstant_initialize": [_P, _Z, _F],
    "cct_hip_fill_xavier": [_P, _Z, _Z, _I],
    "cct_hip_fill_bernoulli": [_P, _Z, _F, _I],
    "cct_hip_fill_gaussian": [_P, _Z, _F, _F, _I],
    "cct_filler_draw_xavier": [_P, _Z, _Z, _I],
    "cct_filler_draw_bernoulli": [_P, _Z, _F, _I],
    "cct_filler_draw_gaussian": [_P, _Z, _F, _F, _I],
    "cct_hip_init_rng": [_I],
    "cct_hip_rand_uint_initialize": [_P, _I],
    "cct_hip_forward_bias": [_P, _P, _I, _I, _I],
    "cct_hip_backward_bias": [_P, _P, _I, _I, _I],
    "cct_hip_backward_bias_noalloc": [_P, _P, _I, _I, _I],
    "cct_hip_backward_bias_fc": [_P, _P, _I, _I],
    "cct_hip_relu_forward": [_P, _P, _Z],
    "cct_hip_relu_backward": [_P, _P, _P, _Z],
    "cct_hip_maxpool_forward": [_P, _P, C.POINTER(PoolArgs)],
    "cct_hip_maxpool_backward": [_P, _P, C.POINTER(PoolArgs)],
    "cct_hip_maxpool_backward_relu": [_P, _P, C.POINTER(PoolArgs), _P],
    "cct_hip_maxpool_backward_relu_pooled": [_P, _P, C.POINTER(PoolArgs), _P],
    "cct_hip_lrn_forward": [_P, _P, C.POINTER(LrnForwardArgs), C.POINTER(LrnForwardNormalizeArgs)],
    "cct_hip_lrn_backward": [_P, _P, C.POINTER(LrnBackwardArgs)],
    "cct_hip_dropout_forward_train": [_P, _P, _P, _F, _U, _Z],
    "cct_hip_softmax_loss_forward": [_P, _P, _P, _P, _I, _I],
    "cct_hip_softmax_loss_backward": [_P, _P, _P, _I, _I, _I],
    "cct_hip_softmax_loss_forward_backward": [_P, _P, _P, _P, _P, _I, _I, _I],
    "cct_hip_timer_create": [C.POINTER(_P)],
    "cct_hip_timer_destroy": [_P],
    "cct_hip_timer_start": [_P],
    "cct_hip_timer_stop": [_P],
    "cct_hip_timer_elapsed_ms": [_P, C.POINTER(_F)],
}
_RESTYPE = {"cct_hip_last_error": C.c_char_p, "cct_hip_last_kernel": C.c_char_p, "cct_hip_conv_direct_slab_floats": C.c_size_t,
            "cct_hip_conv_direct_slab_floats_grouped": C.c_size_t,
            "cct_hip_conv_strided_slab_floats": C.c_size_t,
            "cct_hip_conv_strided_backward_data_slab_floats": C.c_size_t}

_lib = None


def load():
    """Load the shared library and attach prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CctHipError(
            "%s is missing: build it with `python -m caffecontroll_amd.build` "
            "(there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the ABI symbol is absent
        fn.argtypes = argtypes
        fn.restype = _RESTYPE.get(name, C.c_int)
    _lib = lib
    return lib


def check(rc, what=""):
    if rc != 0:
        msg = load().cct_hip_last_error()
        raise CctHipError("%s failed (code %d): %s" % (what or "cct_hip call", rc,
                                                       msg.decode() if msg else ""))
