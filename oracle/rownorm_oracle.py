"""ctypes front end of librownorm_oracle.so (see rownorm_oracle.c).

TEST INFRASTRUCTURE ONLY.  Every function takes float32 numpy arrays (low
precision inputs are widened first, which is exact) and returns float32
arrays computed with double accumulators.  Shapes follow the operator
contracts of src/ATen/native/xpu/LayerNorm.cpp:35-305 and
src/ATen/native/xpu/SoftMax.cpp:22-100 in the reference: inputs are viewed
as [M, N] with N the product of the normalized dimensions.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librownorm_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i64 = ctypes.c_int64


def build(force=False):
    """Compile the checker with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "rownorm_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "librownorm_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_welford_moments.argtypes = [_f32p, _i64, _f64p, _f64p]
        L.oracle_layer_norm_fwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64,
                                            ctypes.c_double]
        L.oracle_rms_norm_fwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _i64, _i64, ctypes.c_double]
        L.oracle_layer_norm_bwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                            _f64p, _i64, _i64]
        L.oracle_rms_norm_bwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f64p, _i64, _i64]
        L.oracle_softmax_fwd.argtypes = [_f32p, _f32p, _i64, _i64, ctypes.c_int]
        L.oracle_softmax_bwd.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, ctypes.c_int]
        L.oracle_group_norm_fwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64,
                                            _i64, _i64, ctypes.c_double]
        L.oracle_group_norm_bwd.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                                            _i64, _i64, _i64, _i64]
        L.oracle_group_norm_fwd.restype = None
        L.oracle_group_norm_bwd.restype = None
        _u8p = ctypes.POINTER(ctypes.c_uint8)
        L.oracle_safe_softmax_fwd.argtypes = [_f32p, _f32p, _i64, _i64]
        L.oracle_masked_softmax_fwd.argtypes = [_f32p, _u8p, _f32p, _i64, _i64]
        L.oracle_masked_softmax_bwd.argtypes = [_f32p, _f32p, _u8p, _f32p, _i64, _i64]
        for f in ("oracle_safe_softmax_fwd", "oracle_masked_softmax_fwd",
                  "oracle_masked_softmax_bwd"):
            getattr(L, f).restype = None
        for f in ("oracle_welford_moments", "oracle_layer_norm_fwd", "oracle_rms_norm_fwd",
                  "oracle_layer_norm_bwd", "oracle_rms_norm_bwd", "oracle_softmax_fwd",
                  "oracle_softmax_bwd"):
            getattr(L, f).restype = None
        _lib = L
    return _lib


def _c(a):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _mn(x, n_norm_dims):
    shape = x.shape
    axis = len(shape) - n_norm_dims
    M = int(np.prod(shape[:axis], dtype=np.int64)) if axis > 0 else 1
    N = int(np.prod(shape[axis:], dtype=np.int64))
    stat_shape = tuple(shape[:axis]) + (1,) * n_norm_dims
    return M, N, stat_shape


def welford_moments(x):
    x = _c(x).reshape(-1)
    m = ctypes.c_double()
    v = ctypes.c_double()
    lib().oracle_welford_moments(_p(x), x.size, ctypes.byref(m), ctypes.byref(v))
    return m.value, v.value


def layer_norm_fwd(x, normalized_shape, gamma=None, beta=None, eps=1e-5):
    """native_layer_norm -> (y, mean, rstd); mean/rstd shaped input.shape[:axis] + [1]*k."""
    x = _c(x)
    M, N, stat_shape = _mn(x, len(normalized_shape))
    gamma, beta = _c(gamma), _c(beta)
    y = np.empty_like(x)
    mean = np.empty(M, np.float32)
    rstd = np.empty(M, np.float32)
    if M > 0 and N > 0:
        lib().oracle_layer_norm_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(mean), _p(rstd), M, N,
                                    float(eps))
    return y, mean.reshape(stat_shape), rstd.reshape(stat_shape)


def rms_norm_fwd(x, normalized_shape, gamma=None, eps=None):
    """_fused_rms_norm -> (y, rstd); eps=None means FLT_EPSILON (LayerNorm.cpp:218-224)."""
    x = _c(x)
    M, N, stat_shape = _mn(x, len(normalized_shape))
    if eps is None:
        eps = float(np.finfo(np.float32).eps)
    gamma = _c(gamma)
    y = np.empty_like(x)
    rstd = np.empty(M, np.float32)
    if M > 0 and N > 0:
        lib().oracle_rms_norm_fwd(_p(x), _p(gamma), _p(y), _p(rstd), M, N, float(eps))
    return y, rstd.reshape(stat_shape)


def layer_norm_bwd(dy, x, normalized_shape, mean, rstd, gamma=None, mask=(True, True, True)):
    """native_layer_norm_backward -> (dx, dgamma, dbeta), None where the mask is False."""
    x, dy = _c(x), _c(dy)
    M, N, _ = _mn(x, len(normalized_shape))
    mean = _c(mean).reshape(-1)
    rstd = _c(rstd).reshape(-1)
    gamma = _c(gamma)
    dx = np.empty_like(x) if mask[0] else None
    dg = np.zeros(N, np.float32) if mask[1] else None
    db = np.zeros(N, np.float32) if mask[2] else None
    if M > 0 and N > 0:
        scratch = np.zeros(2 * N, np.float64)
        lib().oracle_layer_norm_bwd(_p(dy), _p(x), _p(mean), _p(rstd), _p(gamma), _p(dx), _p(dg),
                                    _p(db), scratch.ctypes.data_as(_f64p), M, N)
    wshape = tuple(normalized_shape)
    return (dx, None if dg is None else dg.reshape(wshape),
            None if db is None else db.reshape(wshape))


def rms_norm_bwd(dy, x, normalized_shape, rstd, gamma=None, mask=(True, True)):
    """_fused_rms_norm_backward -> (dx, dgamma)."""
    x, dy = _c(x), _c(dy)
    M, N, _ = _mn(x, len(normalized_shape))
    rstd = _c(rstd).reshape(-1)
    gamma = _c(gamma)
    dx = np.empty_like(x) if mask[0] else None
    dg = np.zeros(N, np.float32) if mask[1] else None
    if M > 0 and N > 0:
        scratch = np.zeros(N, np.float64)
        lib().oracle_rms_norm_bwd(_p(dy), _p(x), _p(rstd), _p(gamma), _p(dx), _p(dg),
                                  scratch.ctypes.data_as(_f64p), M, N)
    return dx, None if dg is None else dg.reshape(tuple(normalized_shape))


def round_to(a, dtype):
    """float32 values rounded to the storage format `dtype` ("f32", "f16" or "bf16") with round to
    nearest even, returned as float32: what a store of the accumulate type into a tensor of that
    dtype does.  bfloat16 keeps the top 16 bits of the float32 pattern; NaN stays NaN."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if dtype == "f32":
        return a.copy()
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    if dtype != "bf16":
        raise ValueError("dtype must be f32, f16 or bf16, got %r" % (dtype,))
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = rounded.view(np.float32).copy()
    out[np.isnan(a)] = np.nan
    return out


def residual_sum(x, residual, dtype):
    """h = x + residual as the fused add -> norm operators form it: the float32 sum of the two
    rows rounded once to the row dtype (an elementwise add of two tensors of that dtype)."""
    return round_to(_c(x) + _c(residual), dtype)


def add_layer_norm_fwd(x, residual, normalized_shape, gamma=None, beta=None, eps=1e-5, dtype="f32"):
    """Fused residual add -> LayerNorm: the pinned layer_norm_fwd applied to residual_sum().
    -> (y, h, mean, rstd).  The reference has no fused operator; its forward starts from the
    summed row (VectorizedLayerNormKernelFunctor, LayerNormKernels.cpp:469-586)."""
    h = residual_sum(x, residual, dtype)
    y, mean, rstd = layer_norm_fwd(h, normalized_shape, gamma, beta, eps)
    return y, h, mean, rstd


def add_rms_norm_fwd(x, residual, normalized_shape, gamma=None, eps=None, dtype="f32"):
    """Fused residual add -> RMSNorm -> (y, h, rstd)."""
    h = residual_sum(x, residual, dtype)
    y, rstd = rms_norm_fwd(h, normalized_shape, gamma, eps)
    return y, h, rstd


def add_layer_norm_bwd(dy, dh_in, h, normalized_shape, mean, rstd, gamma=None,
                       mask=(True, True, True)):
    """Backward of the fused add -> LayerNorm: the norm's input gradient plus the gradient that
    reaches h by the residual path (None: none), summed in float64.  -> (dh, dgamma, dbeta)."""
    dx, dg, db = layer_norm_bwd(dy, h, normalized_shape, mean, rstd, gamma, mask)
    if dx is not None and dh_in is not None:
        dx = (dx.astype(np.float64) + _c(dh_in).astype(np.float64)).astype(np.float32)
    return dx, dg, db


def add_rms_norm_bwd(dy, dh_in, h, normalized_shape, rstd, gamma=None, mask=(True, True)):
    dx, dg = rms_norm_bwd(dy, h, normalized_shape, rstd, gamma, mask)
    if dx is not None and dh_in is not None:
        dx = (dx.astype(np.float64) + _c(dh_in).astype(np.float64)).astype(np.float32)
    return dx, dg


def softmax_fwd(x, is_log=False):
    """_softmax / _log_softmax over the last dimension."""
    x = _c(x)
    y = np.empty_like(x)
    if x.size:
        N = x.shape[-1] if x.ndim else 1
        lib().oracle_softmax_fwd(_p(x), _p(y), x.size // N, N, int(is_log))
    return y


def softmax_bwd(grad, y, is_log=False):
    """_softmax_backward_data / _log_softmax_backward_data over the last dimension."""
    grad, y = _c(grad), _c(y)
    gi = np.empty_like(y)
    if y.size:
        N = y.shape[-1] if y.ndim else 1
        lib().oracle_softmax_bwd(_p(grad), _p(y), _p(gi), y.size // N, N, int(is_log))
    return gi


def safe_softmax_fwd(x):
    """_safe_softmax over the last dimension (rows of -inf give zeros)."""
    x = _c(x)
    y = np.empty_like(x)
    if x.size:
        N = x.shape[-1] if x.ndim else 1
        lib().oracle_safe_softmax_fwd(_p(x), _p(y), x.size // N, N)
    return y


def _mask_bytes(mask, shape):
    m = np.ascontiguousarray(np.broadcast_to(np.asarray(mask).astype(bool), shape), dtype=np.uint8)
    return m, m.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))


def masked_softmax_fwd(x, mask):
    """_masked_softmax over the last dimension; mask (True = leave out) broadcasts to x."""
    x = _c(x)
    y = np.empty_like(x)
    if x.size:
        N = x.shape[-1] if x.ndim else 1
        m, mp = _mask_bytes(mask, x.shape)
        lib().oracle_masked_softmax_fwd(_p(x), mp, _p(y), x.size // N, N)
    return y


def masked_softmax_bwd(grad, y, mask):
    """_masked_softmax_backward over the last dimension."""
    grad, y = _c(grad), _c(y)
    gi = np.empty_like(y)
    if y.size:
        N = y.shape[-1] if y.ndim else 1
        m, mp = _mask_bytes(mask, y.shape)
        lib().oracle_masked_softmax_bwd(_p(grad), _p(y), mp, _p(gi), y.size // N, N)
    return gi


def _nchw(x):
    N, C = x.shape[0], x.shape[1]
    HxW = int(np.prod(x.shape[2:], dtype=np.int64)) if x.ndim > 2 else 1
    return N, C, HxW


def group_norm_fwd(x, groups, gamma=None, beta=None, eps=1e-5):
    """native_group_norm on [N, C, *] -> (y, mean[N, groups], rstd[N, groups])."""
    x = _c(x)
    N, C, HxW = _nchw(x)
    gamma, beta = _c(gamma), _c(beta)
    y = np.empty_like(x)
    mean = np.zeros((N, groups), np.float32)
    rstd = np.zeros((N, groups), np.float32)
    if x.size:
        lib().oracle_group_norm_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(mean), _p(rstd), N, C, HxW,
                                    groups, float(eps))
    return y, mean, rstd


def group_norm_bwd(dy, x, groups, mean, rstd, gamma=None, mask=(True, True, True)):
    """native_group_norm_backward -> (dx, dgamma, dbeta), None where the mask is False."""
    x, dy = _c(x), _c(dy)
    N, C, HxW = _nchw(x)
    mean, rstd, gamma = _c(mean).reshape(-1), _c(rstd).reshape(-1), _c(gamma)
    dx = np.empty_like(x) if mask[0] else None
    dg = np.zeros(C, np.float32) if mask[1] else None
    db = np.zeros(C, np.float32) if mask[2] else None
    lib().oracle_group_norm_bwd(_p(dy), _p(x), _p(mean), _p(rstd), _p(gamma), _p(dx), _p(dg), _p(db),
                                N, C, HxW, groups)
    return dx, dg, db
