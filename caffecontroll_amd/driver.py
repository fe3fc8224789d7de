"""Python view of the C ABI, named after the reference's ``DeviceDriver`` members
(src/sched/DeviceDriver.h:56-274).  Arguments are device addresses (``int``) or objects with a
``data_ptr()`` method (torch tensors); nothing here computes on the host.
"""
import ctypes as C

from . import _lib
from ._lib import (COL_MAJOR, NO_TRANS, ROW_MAJOR, TRANS, InverseLowerCubeArgs, LrnBackwardArgs,
                   LrnForwardArgs, LrnForwardNormalizeArgs, PMapHelper, PoolArgs, check)

__all__ = ["HIPDriver", "conv_pmap", "lift_args", "remap_pmap", "ROW_MAJOR", "COL_MAJOR",
           "NO_TRANS", "TRANS"]


def _p(x):
    if x is None:
        return None
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return int(x)


def conv_pmap(b, d, n, k, s, p):
    """PMapHelper as Connector::lower_cube fills it (src/Connector_impl_Lowering_type1.hxx:65-82)."""
    m = (n + 2 * p - k) // s + 1
    a = PMapHelper()
    a.dR, a.dC, a.dD, a.dB = k * k * d, m * m * b, 1, 1
    a.sR, a.sC, a.sD, a.sB = n, n, d, b
    a.dBR, a.dBC = a.dR, a.dC
    a.sBR, a.sBC = min(16, n), min(16, n)
    a.kR, a.kC, a.kD, a.kB = k, k, d, 1
    a.stride, a.padding = s, p
    return a


def lift_args(b, d, n, k, s, p):
    """_inverse_lower_cube_arg_helper as Connector::inverse_lower_cube fills it
    (src/Connector_impl_Lowering_type1.hxx:158-168)."""
    m = (n + 2 * p - k) // s + 1
    a = InverseLowerCubeArgs()
    a.data_output_width = a.data_output_height = m
    a.kernel_size, a.stride, a.padding = k, s, p
    a.iR, a.iC, a.iD, a.iB = n, n, d, b
    return a


def remap_pmap(R, Cc, depth, batch):
    """PMapHelper as Connector::remap_output fills it (src/Connector_impl_Lowering_type1.hxx:107-121)."""
    a = PMapHelper()
    a.dR, a.dC, a.dD, a.dB = R, Cc, depth, batch
    a.sR, a.sC, a.sD, a.sB = R, Cc, depth, batch
    a.dBR, a.dBC = R, Cc
    a.sBR, a.sBC = min(16, R), min(16, Cc)
    return a


class HIPDriver:
    """One per process; all work goes to one HIP stream (see ``set_stream``)."""

    def __init__(self, device_id=0):
        self.lib = _lib.load()
        check(self.lib.cct_hip_init(device_id), "init")

    # -- state ------------------------------------------------------------------------------
    def set_stream(self, stream_handle):
        check(self.lib.cct_hip_set_stream(stream_handle), "set_stream")

    def set_tuning(self, name, value):
        """Tuning knob (see cct_hip_set_tuning in include/cct_hip.h), e.g. ("direct_tile", 22)."""
        check(self.lib.cct_hip_set_tuning(name.encode(), int(value)), "set_tuning")

    def device_sync(self):
        check(self.lib.cct_hip_device_sync(), "device_sync")

    def compute_units(self):
        return self.lib.cct_hip_compute_units()

    # -- memory -----------------------------------------------------------------------------
    def malloc(self, size_in_byte):
        out = C.c_void_p()
        check(self.lib.cct_hip_malloc(C.byref(out), size_in_byte), "malloc")
        return out.value or 0

    def free(self, ptr):
        check(self.lib.cct_hip_free(_p(ptr)), "free")

    def memcpy(self, dst, src, size_in_byte, kind):
        check(self.lib.cct_hip_memcpy(_p(dst), _p(src), size_in_byte, kind), "memcpy")

    def memset(self, dst, value, size_in_byte):
        check(self.lib.cct_hip_memset(_p(dst), value, size_in_byte), "memset")

    # -- lowering / lifting -----------------------------------------------------------------
    def lower_cube(self, dst, src, args):
        check(self.lib.cct_hip_lower_cube(_p(dst), _p(src), C.byref(args)), "lower_cube")

    def inverse_lower_cube(self, dst, src, args):
        check(self.lib.cct_hip_inverse_lower_cube(_p(dst), _p(src), C.byref(args)), "inverse_lower_cube")

    def inverse_lower_cube_bias_backward(self, dst, src, args, bias_grad, out_grad, fmap, depth, batch):
        check(self.lib.cct_hip_inverse_lower_cube_bias_backward(
            _p(dst), _p(src), C.byref(args), _p(bias_grad), _p(out_grad), fmap, depth, batch),
            "inverse_lower_cube_bias_backward")

    def remap(self, dst, src, args):
        check(self.lib.cct_hip_remap(_p(dst), _p(src), C.byref(args)), "remap")

    def remap_bias_backward(self, dst, src, args, bias_grad):
        """remap plus the bias gradient of the maps (source slice j belongs to map j % sB)."""
        check(self.lib.cct_hip_remap_bias_backward(_p(dst), _p(src), C.byref(args), _p(bias_grad)),
              "remap_bias_backward")

    # -- BLAS-shaped ------------------------------------------------------------------------
    def sgemm(self, order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc):
        check(self.lib.cct_hip_sgemm(order, TA, TB, M, N, K, alpha, _p(A), lda, _p(B), ldb, beta,
                                     _p(Cm), ldc), "sgemm")

    def sgemm_new_bias(self, TA, TB, M, N, K, alpha, A, B, beta, Cm, col_bias=None, relu=False):
        """sgemm_new, then Cm[m][n] += col_bias[n] and, with relu, max(., 0), in the same pass."""
        check(self.lib.cct_hip_sgemm_new_bias(TA, TB, M, N, K, alpha, _p(A), _p(B), beta, _p(Cm), _p(col_bias),
                                              int(relu)), "sgemm_new_bias")

    def sgemm_new_colsum(self, TA, TB, M, N, K, alpha, A, B, beta, Cm, colsum, colsum_src, rows, cols):
        """sgemm_new, and beside it colsum[c] = sum over r of colsum_src[r][c] (rows x cols, dense)."""
        check(self.lib.cct_hip_sgemm_new_colsum(TA, TB, M, N, K, alpha, _p(A), _p(B), beta, _p(Cm), _p(colsum),
                                                _p(colsum_src), rows, cols), "sgemm_new_colsum")

    def sgemm_new(self, TA, TB, M, N, K, alpha, A, B, beta, Cm):
        check(self.lib.cct_hip_sgemm_new(TA, TB, M, N, K, alpha, _p(A), _p(B), beta, _p(Cm)), "sgemm_new")

    def sgemm_conv_forward(self, o, batch, fmap, K, model, lowered, bias, out, relu=False):
        check(self.lib.cct_hip_sgemm_conv_forward(o, batch, fmap, K, _p(model), _p(lowered), _p(bias),
                                                  _p(out), int(relu)), "sgemm_conv_forward")

    # -- inner-product layers with few outputs: one launch per pass -----------------------------
    def fc_small_supported(self, batch, in_features, out_features):
        return bool(self.lib.cct_hip_fc_small_supported(batch, in_features, out_features))

    def fc_small_forward(self, y, x, w, bias, batch, in_features, out_features, relu=False):
        check(self.lib.cct_hip_fc_small_forward(_p(y), _p(x), _p(w), _p(bias), batch, in_features, out_features,
                                                int(relu)), "fc_small_forward")

    def fc_small_backward(self, dx, dw, db, dy, x, w, batch, in_features, out_features, relu_data=None):
        check(self.lib.cct_hip_fc_small_backward(_p(dx), _p(dw), _p(db), _p(dy), _p(x), _p(w), batch, in_features,
                                                 out_features, _p(relu_data)), "fc_small_backward")

    # -- convolutions with a very short contraction and few maps (LeNet conv1) -------------------
    # 1 x 1 convolutions (stride 1, no padding) as products on the tensors as they lie; plane = n * n
    def conv1x1_supported(self, b, d, n, k, s, p, o):
        return bool(self.lib.cct_hip_conv1x1_supported(b, d, n, k, s, p, o))

    def conv1x1_forward(self, out, x, w, bias, b, d, plane, o, relu=False):
        check(self.lib.cct_hip_conv1x1_forward(_p(out), _p(x), _p(w), _p(bias), b, d, plane, o, int(relu)),
              "conv1x1_forward")

    def conv1x1_backward_data(self, dx, dout, w, b, d, plane, o):
        check(self.lib.cct_hip_conv1x1_backward_data(_p(dx), _p(dout), _p(w), b, d, plane, o), "conv1x1_backward_data")

    def conv1x1_backward_weights(self, dw, dout, x, b, d, plane, o, db=None):
        check(self.lib.cct_hip_conv1x1_backward_weights(_p(dw), _p(db), _p(dout), _p(x), b, d, plane, o),
              "conv1x1_backward_weights")

    def conv_small_supported(self, b, d, n, k, s, p, o):
        return bool(self.lib.cct_hip_conv_small_supported(b, d, n, k, s, p, o))

    def conv_small_forward(self, out, x, w, bias, b, d, n, k, p, o, relu=False):
        check(self.lib.cct_hip_conv_small_forward(_p(out), _p(x), _p(w), _p(bias), b, d, n, k, p, o, int(relu)),
              "conv_small_forward")

    def conv_small_backward_weights(self, dw, dout, x, b, d, n, k, p, o, db=None):
        check(self.lib.cct_hip_conv_small_backward_weights(_p(dw), _p(db), _p(dout), _p(x), b, d, n, k, p, o),
              "conv_small_backward_weights")

    # `groups` > 1: a grouped convolution (d and o are the layer's totals), all groups in one launch
    def conv_direct_supported(self, b, d, n, k, s, p, o, groups=1):
        return bool(self.lib.cct_hip_conv_direct_supported_grouped(b, d, n, k, s, p, o, groups))

    def conv_direct_slab_floats(self, o, d, k, for_data_gradient, groups=1):
        return int(self.lib.cct_hip_conv_direct_slab_floats_grouped(o, d, k, int(for_data_gradient), groups))

    def conv_direct_slabs(self, slabs, model, o, d, k, for_data_gradient, groups=1):
        check(self.lib.cct_hip_conv_direct_slabs_grouped(_p(slabs), _p(model), o, d, k, int(for_data_gradient),
                                                         groups), "conv_direct_slabs")

    # -- strided convolution without the lowered matrix ------------------------------------------
    def conv_strided_supported(self, b, d, n, k, s, p, o):
        return bool(self.lib.cct_hip_conv_strided_supported(b, d, n, k, s, p, o))

    def conv_strided_slab_floats(self, o, d, k, s, p):
        return int(self.lib.cct_hip_conv_strided_slab_floats(o, d, k, s, p))

    def conv_strided_slabs(self, slabs, model, o, d, k, s, p):
        check(self.lib.cct_hip_conv_strided_slabs(_p(slabs), _p(model), o, d, k, s, p), "conv_strided_slabs")

    def conv_strided_forward(self, out, inp, slabs, bias, b, d, n, k, s, p, o, relu=False):
        check(self.lib.cct_hip_conv_strided_forward(_p(out), _p(inp), _p(slabs), _p(bias), b, d, n, k, s, p, o,
                                                    int(relu)), "conv_strided_forward")

    def conv_strided_backward_weights(self, model_grad, bias_grad, out_grad, inp, b, d, n, k, s, p, o):
        check(self.lib.cct_hip_conv_strided_backward_weights(_p(model_grad), _p(bias_grad), _p(out_grad), _p(inp),
                                                             b, d, n, k, s, p, o), "conv_strided_backward_weights")

    def conv_strided_backward_data_supported(self, b, d, n, k, s, p, o):
        return bool(self.lib.cct_hip_conv_strided_backward_data_supported(b, d, n, k, s, p, o))

    def conv_strided_backward_data_slab_floats(self, o, d, k, s):
        return int(self.lib.cct_hip_conv_strided_backward_data_slab_floats(o, d, k, s))

    def conv_strided_backward_data_slabs(self, slabs, model, o, d, k, s):
        check(self.lib.cct_hip_conv_strided_backward_data_slabs(_p(slabs), _p(model), o, d, k, s),
              "conv_strided_backward_data_slabs")

    def conv_strided_backward_data(self, in_grad, out_grad, slabs, b, d, n, k, s, p, o):
        check(self.lib.cct_hip_conv_strided_backward_data(_p(in_grad), _p(out_grad), _p(slabs), b, d, n, k, s, p, o),
              "conv_strided_backward_data")

    def conv_direct_forward(self, out, inp, slabs, bias, b, d, n, k, p, o, in_stride=0, out_stride=0, relu=False,
                            groups=1):
        check(self.lib.cct_hip_conv_direct_forward_grouped(_p(out), _p(inp), _p(slabs), _p(bias), b, d, n, k, p, o,
                                                           in_stride, out_stride, int(relu), groups),
              "conv_direct_forward")

    def conv_direct_backward_data(self, din, dout, slabs, b, d, n, k, p, o, in_stride=0, out_stride=0,
                                  relu_data=None, groups=1):
        """relu_data: the layer's input tensor when it is the output of an in-place ReLU; the gradient
        is then stored already masked with (relu_data > 0)."""
        check(self.lib.cct_hip_conv_direct_backward_data_grouped(_p(din), _p(dout), _p(slabs), b, d, n, k, p, o,
                                                                 in_stride, out_stride, _p(relu_data), groups),
              "conv_direct_backward_data")

    def conv_direct_backward_weights(self, dw, dout, inp, b, d, n, k, p, o, db=None, in_stride=0, out_stride=0,
                                     groups=1):
        check(self.lib.cct_hip_conv_direct_backward_weights_grouped(_p(dw), _p(db), _p(dout), _p(inp), b, d, n, k,
                                                                    p, o, in_stride, out_stride, groups),
              "conv_direct_backward_weights")

    def sgemv(self, TA, M, N, alpha, A, x, beta, y):
        check(self.lib.cct_hip_sgemv(TA, M, N, alpha, _p(A), _p(x), beta, _p(y)), "sgemv")

    def math_saxpy(self, n, alpha, x, y):
        check(self.lib.cct_hip_math_saxpy(n, alpha, _p(x), _p(y)), "math_saxpy")

    def math_saxpby(self, n, alpha, x, beta, y):
        check(self.lib.cct_hip_math_saxpby(n, alpha, _p(x), beta, _p(y)), "math_saxpby")

    def L1_update(self, n, gradient, lam, model):
        check(self.lib.cct_hip_L1_update(n, _p(gradient), lam, _p(model)), "L1_update")

    def sgd_update(self, n, model, gradient, history, stepsize, momentum, lam=0.0, l1=False):
        check(self.lib.cct_hip_sgd_update(n, _p(model), _p(gradient), _p(history), stepsize, momentum,
                                          lam, int(l1)), "sgd_update")

    def sgd_update_batch(self, jobs):
        """jobs: sequence of (n, model, gradient, history, stepsize, momentum, lam, l1); one launch
        per 16 tensors, the arithmetic of `sgd_update` on every element."""
        from ._lib import SgdJob
        table = (SgdJob * len(jobs))()
        for t, (n, model, gradient, history, stepsize, momentum, lam, l1) in zip(table, jobs):
            t.n, t.model, t.gradient, t.history = n, _p(model), _p(gradient), _p(history)
            t.stepsize, t.momentum, t.lam, t.l1 = stepsize, momentum, lam, int(l1)
        check(self.lib.cct_hip_sgd_update_batch(table, len(jobs)), "sgd_update_batch")

    def sconstant_initialize(self, arr, n, value):
        check(self.lib.cct_hip_sconstant_initialize(_p(arr), n, value), "sconstant_initialize")

    def fill_xavier(self, arr, n, n_batch, seed):
        check(self.lib.cct_hip_fill_xavier(_p(arr), n, n_batch, seed), "fill_xavier")

    def fill_bernoulli(self, arr, n, p, seed):
        check(self.lib.cct_hip_fill_bernoulli(_p(arr), n, p, seed), "fill_bernoulli")

    def fill_gaussian(self, arr, n, mean, std, seed):
        check(self.lib.cct_hip_fill_gaussian(_p(arr), n, mean, std, seed), "fill_gaussian")

    def init_rng(self, seed):
        check(self.lib.cct_hip_init_rng(seed), "init_rng")

    def rand_uint_initialize(self, buf, n):
        check(self.lib.cct_hip_rand_uint_initialize(_p(buf), n), "rand_uint_initialize")

    # -- bias -------------------------------------------------------------------------------
    def forward_bias(self, bias, out, fmap, depth, batch):
        check(self.lib.cct_hip_forward_bias(_p(bias), _p(out), fmap, depth, batch), "forward_bias")

    def backward_bias(self, bias_grad, out_grad, fmap, depth, batch):
        check(self.lib.cct_hip_backward_bias(_p(bias_grad), _p(out_grad), fmap, depth, batch),
              "backward_bias")

    def backward_bias_noalloc(self, bias_grad, out_grad, fmap, depth, batch):
        check(self.lib.cct_hip_backward_bias_noalloc(_p(bias_grad), _p(out_grad), fmap, depth, batch),
              "backward_bias_noalloc")

    def backward_bias_fc(self, bias_grad, out_grad, D, B):
        check(self.lib.cct_hip_backward_bias_fc(_p(bias_grad), _p(out_grad), D, B), "backward_bias_fc")

    # -- elementwise / pooling / loss -------------------------------------------------------
    def relu_forward(self, out, inp, n):
        check(self.lib.cct_hip_relu_forward(_p(out), _p(inp), n), "relu_forward")

    def relu_backward(self, in_grad, out_grad, in_data, n):
        check(self.lib.cct_hip_relu_backward(_p(in_grad), _p(out_grad), _p(in_data), n), "relu_backward")

    @staticmethod
    def pool_args(k, s, iR, iC, D, B, max_index):
        a = PoolArgs()
        a.stride, a.kernel_size, a.iR, a.iC = s, k, iR, iC
        a.oR, a.oC, a.D, a.B = (iR - k) // s + 1, (iC - k) // s + 1, D, B
        a.max_index = _p(max_index)
        return a

    def maxpool_forward(self, out, inp, args):
        check(self.lib.cct_hip_maxpool_forward(_p(out), _p(inp), C.byref(args)), "maxpool_forward")

    def maxpool_backward(self, in_grad, out_grad, args, relu_data=None, pooled=None):
        """relu_data: the pooled tensor when it is the output of an in-place ReLU; the gradient then
        comes out already masked with (relu_data > 0).  pooled: the same result from the pooling
        layer's output tensor instead (cct_hip_maxpool_backward_relu_pooled)."""
        if pooled is not None:
            check(self.lib.cct_hip_maxpool_backward_relu_pooled(_p(in_grad), _p(out_grad), C.byref(args), _p(pooled)),
                  "maxpool_backward_relu_pooled")
            return
        if relu_data is not None:
            check(self.lib.cct_hip_maxpool_backward_relu(_p(in_grad), _p(out_grad), C.byref(args), _p(relu_data)),
                  "maxpool_backward_relu")
            return
        check(self.lib.cct_hip_maxpool_backward(_p(in_grad), _p(out_grad), C.byref(args)), "maxpool_backward")

    def lrn_forward(self, out, inp, R, Cc, D, B, local_size, alpha, beta, denoms):
        a = LrnForwardArgs()
        a.iR, a.iC, a.iD, a.iB = R, Cc, D, B
        a.norm_window, a.local_size, a.denoms = local_size // 2, local_size, _p(denoms)
        a2 = LrnForwardNormalizeArgs()
        a2.alpha_over_size, a2.beta, a2.denoms = alpha / local_size, beta, _p(denoms)
        check(self.lib.cct_hip_lrn_forward(_p(out), _p(inp), C.byref(a), C.byref(a2)), "lrn_forward")

    def lrn_backward(self, in_grad, out_grad, in_data, R, Cc, D, B, local_size, alpha, beta, denoms):
        a = LrnBackwardArgs()
        a.oR, a.oC, a.oD, a.oB = R, Cc, D, B
        a.alpha_over_size, a.beta = alpha / local_size, beta
        a.norm_window, a.local_size = local_size // 2, local_size
        a.denoms, a.input_data, a.output_data = _p(denoms), _p(in_data), _p(in_data)
        check(self.lib.cct_hip_lrn_backward(_p(in_grad), _p(out_grad), C.byref(a)), "lrn_backward")

    def dropout_forward_train(self, out, inp, mask, scale, threshold, n):
        check(self.lib.cct_hip_dropout_forward_train(_p(out), _p(inp), _p(mask), scale, threshold, n),
              "dropout_forward_train")

    def softmax_loss_forward(self, prob, inp, labels, loss_sum, len_per_image, batch):
        check(self.lib.cct_hip_softmax_loss_forward(_p(prob), _p(inp), _p(labels), _p(loss_sum),
                                                    len_per_image, batch), "softmax_loss_forward")

    def softmax_loss_forward_backward(self, prob, in_grad, inp, labels, loss_sum, len_per_image, batch, spatial=1):
        """The forward pass and the gradient of the backward pass in one launch."""
        check(self.lib.cct_hip_softmax_loss_forward_backward(_p(prob), _p(in_grad), _p(inp), _p(labels), _p(loss_sum),
                                                             len_per_image, batch, spatial),
              "softmax_loss_forward_backward")

    def softmax_loss_backward(self, in_grad, prob, labels, len_per_image, batch, spatial=1):
        check(self.lib.cct_hip_softmax_loss_backward(_p(in_grad), _p(prob), _p(labels), len_per_image,
                                                     batch, spatial), "softmax_loss_backward")

    # -- timing -----------------------------------------------------------------------------
    def timer(self):
        return _Timer(self.lib)


class _Timer:
    """hipEvent pair recorded on the library's stream."""

    def __init__(self, lib):
        self.lib = lib
        h = C.c_void_p()
        check(lib.cct_hip_timer_create(C.byref(h)), "timer_create")
        self.h = h

    def start(self):
        check(self.lib.cct_hip_timer_start(self.h), "timer_start")

    def stop(self):
        check(self.lib.cct_hip_timer_stop(self.h), "timer_stop")

    def elapsed_ms(self):
        ms = C.c_float()
        check(self.lib.cct_hip_timer_elapsed_ms(self.h, C.byref(ms)), "timer_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            self.lib.cct_hip_timer_destroy(self.h)
        except Exception:
            pass
