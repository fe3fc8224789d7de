"""ctypes binding of the CPU oracle (``libcct_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

All functions take and return C-contiguous ``numpy`` float32 arrays.  Reference citations
live next to the C implementations in ``cct_oracle.c``.
"""
import ctypes as C
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcct_oracle.so")

ROW_MAJOR, COL_MAJOR, NO_TRANS, TRANS = 101, 102, 111, 112


class PMap(C.Structure):
    """struct PMapHelper, src/sched/DeviceHeader.h:25-35 (same field order)."""
    _fields_ = [(n, C.c_size_t) for n in (
        "dR", "dC", "dD", "dB", "sR", "sC", "sD", "sB", "dBR", "dBC", "sBR", "sBC",
        "kR", "kC", "kD", "kB", "stride", "padding")]


class LiftArgs(C.Structure):
    """struct _inverse_lower_cube_arg_helper, src/kernels/lowering.h:22-32."""
    _fields_ = [(n, C.c_size_t) for n in (
        "data_output_width", "data_output_height", "kernel_size", "stride", "padding",
        "iR", "iC", "iD", "iB")]


class ConvShape(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("b", "d", "n", "k", "s", "p", "o")]

    @property
    def m(self):
        return (self.n + 2 * self.p - self.k) // self.s + 1


def build(force=False):
    """Compile the oracle with gcc if the shared library is missing (or ``force``)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


def lib():
    global _lib
    if _lib is not None:
        return _lib
    L = C.CDLL(build())
    sz, i, f = C.c_size_t, C.c_int, C.c_float
    L.cct_oracle_lower_cube.argtypes = [_f32p, _f32p, C.POINTER(PMap)]
    L.cct_oracle_inverse_lower_cube.argtypes = [_f32p, _f32p, C.POINTER(LiftArgs)]
    L.cct_oracle_remap.argtypes = [_f32p, _f32p, C.POINTER(PMap)]
    gemm_args = [i, i, i, i, i, i, f, _f32p, i, _f32p, i, f, _f32p, i]
    L.cct_oracle_sgemm.argtypes = gemm_args
    L.cct_oracle_sgemm_f64acc.argtypes = gemm_args
    L.cct_oracle_sgemm_new.argtypes = [i, i, i, i, i, f, _f32p, _f32p, f, _f32p]
    L.cct_oracle_sgemv.argtypes = [i, i, i, f, _f32p, _f32p, f, _f32p]
    L.cct_oracle_saxpy.argtypes = [sz, f, _f32p, _f32p]
    L.cct_oracle_saxpby.argtypes = [sz, f, _f32p, f, _f32p]
    L.cct_oracle_bind_openblas.argtypes = [C.c_char_p, i]
    L.cct_oracle_bind_openblas.restype = i
    L.cct_oracle_blas_is_bound.restype = i
    L.cct_oracle_bias_forward.argtypes = [_f32p, _f32p, sz, sz, sz]
    L.cct_oracle_bias_backward.argtypes = [_f32p, _f32p, sz, sz, sz]
    L.cct_oracle_conv_forward.argtypes = [C.POINTER(ConvShape), _f32p, _f32p, C.c_void_p, _f32p, _f32p]
    L.cct_oracle_conv_backward.argtypes = [C.POINTER(ConvShape), _f32p, _f32p, _f32p, _f32p,
                                           C.c_void_p, _f32p, C.c_void_p, i]
    L.cct_oracle_sgd_update.argtypes = [sz, _f32p, _f32p, _f32p, f, f, f, i]
    L.cct_oracle_learning_rate.argtypes = [C.c_char_p, f, f, f, f, f, f]
    L.cct_oracle_learning_rate.restype = f
    L.cct_oracle_relu_forward.argtypes = [_f32p, _f32p, sz]
    L.cct_oracle_relu_backward.argtypes = [_f32p, _f32p, _f32p, sz]
    L.cct_oracle_maxpool_forward.argtypes = [_f32p, _i32p, _f32p] + [i] * 8
    L.cct_oracle_maxpool_backward.argtypes = [_f32p, _f32p, _i32p] + [i] * 6
    L.cct_oracle_lrn_forward.argtypes = [_f32p, _f32p, _f32p, i, i, i, i, i, f, f]
    L.cct_oracle_lrn_backward.argtypes = [_f32p, _f32p, _f32p, _f32p, i, i, i, i, i, f, f]
    L.cct_oracle_dropout_forward.argtypes = [_f32p, _f32p, _u32p, f, sz]
    L.cct_oracle_dropout_forward_threshold.argtypes = [_f32p, _f32p, _u32p, f, sz]
    L.cct_oracle_softmax_loss_forward.argtypes = [_f32p, _f32p, _f32p, sz, sz, sz, sz]
    L.cct_oracle_softmax_loss_forward.restype = f
    L.cct_oracle_softmax_loss_backward.argtypes = [_f32p, _f32p, _f32p, sz, sz, sz, sz]
    L.cct_oracle_fc_forward.argtypes = [_f32p, _f32p, _f32p, C.c_void_p, i, i, i]
    L.cct_oracle_fc_backward.argtypes = [C.c_void_p, _f32p, C.c_void_p, _f32p, _f32p, _f32p,
                                         i, i, i, i]
    L.cct_oracle_process_image.argtypes = [_f32p, np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS"),
                                           C.c_void_p, i, i, i, i, i, i, i, f]
    _lib = L
    return L


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _vp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# ---------------------------------------------------------------------------------------
def conv_pmap(b, d, n, k, s, p):
    """PMapHelper exactly as Connector::lower_cube fills it
    (src/Connector_impl_Lowering_type1.hxx:65-82)."""
    m = (n + 2 * p - k) // s + 1
    a = PMap()
    a.dR, a.dC, a.dD, a.dB = k * k * d, m * m * b, 1, 1
    a.sR, a.sC, a.sD, a.sB = n, n, d, b
    a.dBR, a.dBC = a.dR, a.dC
    a.sBR, a.sBC = min(16, n), min(16, n)
    a.kR, a.kC, a.kD, a.kB = k, k, d, 1
    a.stride, a.padding = s, p
    return a


def lift_args(b, d, n, k, s, p):
    m = (n + 2 * p - k) // s + 1
    a = LiftArgs()
    a.data_output_width = a.data_output_height = m
    a.kernel_size, a.stride, a.padding = k, s, p
    a.iR, a.iC, a.iD, a.iB = n, n, d, b
    return a


def remap_pmap(R, Cc, depth, batch):
    a = PMap()
    a.dR, a.dC, a.dD, a.dB = R, Cc, depth, batch
    a.sR, a.sC, a.sD, a.sB = R, Cc, depth, batch
    a.dBR, a.dBC, a.sBR, a.sBC = R, Cc, R, Cc
    return a


def lower_cube(x, k, s, p):
    """x: [b][d][n][n] -> lowered [b*m*m][k*k*d]."""
    x = _f32(x)
    b, d, n, _ = x.shape
    m = (n + 2 * p - k) // s + 1
    out = np.empty((b * m * m, k * k * d), np.float32)
    lib().cct_oracle_lower_cube(out, x, C.byref(conv_pmap(b, d, n, k, s, p)))
    return out


def inverse_lower_cube(y, b, d, n, k, s, p):
    """y: [k*k*d][b*m*m] -> input gradient [b][d][n][n] (destination cleared first)."""
    y = _f32(y)
    out = np.zeros((b, d, n, n), np.float32)
    lib().cct_oracle_inverse_lower_cube(out, y, C.byref(lift_args(b, d, n, k, s, p)))
    return out


def remap(x, R, Cc, depth, batch):
    x = _f32(x)
    out = np.empty_like(x)
    lib().cct_oracle_remap(out, x, C.byref(remap_pmap(R, Cc, depth, batch)))
    return out


def sgemm(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc, f64acc=False):
    fn = lib().cct_oracle_sgemm_f64acc if f64acc else lib().cct_oracle_sgemm
    fn(order, TA, TB, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc)
    return Cm


def sgemm_new(TA, TB, M, N, K, alpha, A, B, beta, Cm):
    lib().cct_oracle_sgemm_new(TA, TB, M, N, K, alpha, A, B, beta, Cm)
    return Cm


def sgemv(TA, M, N, alpha, A, x, beta, y):
    lib().cct_oracle_sgemv(TA, M, N, alpha, A, x, beta, y)
    return y


def find_openblas():
    """Path of an OpenBLAS exporting (scipy_)cblas_sgemm, or None."""
    try:
        import scipy
        root = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs")
        hits = sorted(glob.glob(os.path.join(root, "libscipy_openblas*.so")))
        if hits:
            return hits[0]
    except Exception:
        pass
    return None


def bind_openblas(nthreads=1):
    path = find_openblas()
    if path is None:
        return False
    return bool(lib().cct_oracle_bind_openblas(path.encode(), nthreads))


def unbind_openblas():
    lib().cct_oracle_bind_openblas(None, 0)


def blas_is_bound():
    return bool(lib().cct_oracle_blas_is_bound())


def bias_forward(out, bias, fmap, depth, batch):
    lib().cct_oracle_bias_forward(out, _f32(bias), fmap, depth, batch)
    return out


def bias_backward(out_grad, fmap, depth, batch):
    g = np.empty(depth, np.float32)
    lib().cct_oracle_bias_backward(g, _f32(out_grad), fmap, depth, batch)
    return g


def conv_forward(x, model, bias, k, s, p):
    """x [b][d][n][n], model [o][d][k][k], bias [o] or None -> (out [b][o][m][m], lowered)."""
    x, model = _f32(x), _f32(model)
    b, d, n, _ = x.shape
    o = model.shape[0]
    sh = ConvShape(b, d, n, k, s, p, o)
    m = sh.m
    lowered = np.empty((b * m * m, k * k * d), np.float32)
    out = np.empty((b, o, m, m), np.float32)
    bias = None if bias is None else _f32(bias)
    lib().cct_oracle_conv_forward(C.byref(sh), x, model, _vp(bias), lowered, out)
    return out, lowered


def conv_backward(x_shape, model, out_grad, lowered, k, s, p, need_in_grad=True, bias_term=True):
    """Returns (in_grad or None, model_grad, bias_grad or None).  ``out_grad`` is copied first:
    the reference permutes the caller's cube in place, callers of this wrapper keep theirs."""
    b, d, n, _ = x_shape
    model = _f32(model)
    o = model.shape[0]
    sh = ConvShape(b, d, n, k, s, p, o)
    og = np.array(out_grad, dtype=np.float32, order="C", copy=True)
    lowered = _f32(lowered)
    lowered_grad = np.empty(lowered.size, np.float32)
    in_grad = np.empty((b, d, n, n), np.float32) if need_in_grad else None
    model_grad = np.empty_like(model)
    bias_grad = np.empty(o, np.float32) if bias_term else None
    lib().cct_oracle_conv_backward(C.byref(sh), model, og, lowered, lowered_grad, _vp(in_grad),
                                   model_grad, _vp(bias_grad), int(need_in_grad))
    return in_grad, model_grad, bias_grad


def sgd_update(model, grad, history, stepsize, momentum, lam=0.0, l1=False):
    lib().cct_oracle_sgd_update(model.size, model, grad, history, stepsize, momentum, lam, int(l1))


def learning_rate(policy, base_lr, gamma, it, stepsize, power, max_iter):
    return lib().cct_oracle_learning_rate(policy.encode(), base_lr, gamma, it, stepsize, power, max_iter)


def relu_forward(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().cct_oracle_relu_forward(out, x, x.size)
    return out


def relu_backward(out_grad, in_data):
    out_grad, in_data = _f32(out_grad), _f32(in_data)
    g = np.empty_like(out_grad)
    lib().cct_oracle_relu_backward(g, out_grad, in_data, g.size)
    return g


def maxpool_forward(x, k, s):
    x = _f32(x)
    B, D, iR, iC = x.shape
    oR, oC = (iR - k) // s + 1, (iC - k) // s + 1
    out = np.empty((B, D, oR, oC), np.float32)
    idx = np.zeros((B, D, oR, oC), np.int32)
    lib().cct_oracle_maxpool_forward(out, idx, x, k, s, iR, iC, oR, oC, D, B)
    return out, idx


def maxpool_backward(out_grad, idx, iR, iC):
    out_grad = _f32(out_grad)
    B, D, oR, oC = out_grad.shape
    g = np.empty((B, D, iR, iC), np.float32)
    lib().cct_oracle_maxpool_backward(g, out_grad, np.ascontiguousarray(idx, np.int32), iR, iC, oR, oC, D, B)
    return g


def lrn_forward(x, local_size, alpha, beta):
    x = _f32(x)
    B, D, R, Cc = x.shape
    out, den = np.empty_like(x), np.empty_like(x)
    lib().cct_oracle_lrn_forward(out, den, x, R, Cc, D, B, local_size, alpha, beta)
    return out, den


def lrn_backward(out_grad, in_data, denoms, local_size, alpha, beta):
    out_grad, in_data, denoms = _f32(out_grad), _f32(in_data), _f32(denoms)
    B, D, R, Cc = in_data.shape
    g = np.empty_like(in_data)
    lib().cct_oracle_lrn_backward(g, out_grad, in_data, denoms, R, Cc, D, B, local_size, alpha, beta)
    return g


def dropout_forward(x, mask, ratio, threshold=False):
    x = _f32(x)
    mask = np.ascontiguousarray(mask, np.uint32)
    out = np.empty_like(x)
    fn = lib().cct_oracle_dropout_forward_threshold if threshold else lib().cct_oracle_dropout_forward
    fn(out, x, mask, ratio, x.size)
    return out


def softmax_loss_forward(x, labels):
    """x [B][D][R][C] -> (prob, summed loss)."""
    x, labels = _f32(x), _f32(labels)
    B, D, R, Cc = x.shape
    prob = np.empty_like(x)
    loss = lib().cct_oracle_softmax_loss_forward(prob, x, labels, R, Cc, D, B)
    return prob, loss


def softmax_loss_backward(prob, labels):
    prob, labels = _f32(prob), _f32(labels)
    B, D, R, Cc = prob.shape
    g = np.empty_like(prob)
    lib().cct_oracle_softmax_loss_backward(g, prob, labels, R, Cc, D, B)
    return g


def fc_forward(x, model, bias):
    x, model = _f32(x), _f32(model)
    B, I = x.shape
    O = model.shape[0]
    out = np.empty((B, O), np.float32)
    bias = None if bias is None else _f32(bias)
    lib().cct_oracle_fc_forward(out, x, model, _vp(bias), B, I, O)
    return out


def fc_backward(x, model, out_grad, need_in_grad=True, bias_term=True):
    x, model, out_grad = _f32(x), _f32(model), _f32(out_grad)
    B, I = x.shape
    O = model.shape[0]
    in_grad = np.empty((B, I), np.float32) if need_in_grad else None
    model_grad = np.empty((O, I), np.float32)
    bias_grad = np.empty(O, np.float32) if bias_term else None
    lib().cct_oracle_fc_backward(_vp(in_grad), model_grad, _vp(bias_grad), x, model, out_grad,
                                 B, I, O, int(need_in_grad))
    return in_grad, model_grad, bias_grad


def transform_batch(raw, mean, crop_size, params, scale):
    """Corpus::process_image over a batch: raw uint8 [b][c][h][w], mean [c][h][w] or None,
    params int [b][3] = (h_off, w_off, mirror)."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    b, c, h, w = raw.shape
    rows, cols = (crop_size, crop_size) if crop_size else (h, w)
    out = np.empty((b, c, rows, cols), np.float32)
    mean = None if mean is None else _f32(mean)
    for i_ in range(b):
        ho, wo, mi = (int(v) for v in params[i_]) if crop_size else (0, 0, 0)
        lib().cct_oracle_process_image(out[i_], raw[i_], _vp(mean), c, h, w, crop_size, ho, wo, mi, scale)
    return out
