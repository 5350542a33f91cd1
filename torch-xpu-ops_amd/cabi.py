"""ctypes bindings of the extern "C" launcher ABI declared in include/mi355x_rownorm.h.

The functions here take torch tensors purely as device memory (``data_ptr()``) plus the current
HIP stream; shapes are [M, N] views of contiguous tensors.  They allocate outputs and the
backward workspace with torch, call the ABI, and raise ``RuntimeError`` on a non-zero status.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_KERNEL_LIB = os.path.join(_HERE, "lib", "libmi355x_rownorm.so")

F32, F16, BF16 = 0, 1, 2
OP_LAYER_NORM_FWD, OP_LAYER_NORM_BWD, OP_RMS_NORM_FWD, OP_RMS_NORM_BWD = 0, 1, 2, 3
OP_SOFTMAX_FWD, OP_SOFTMAX_BWD = 4, 5
OP_SOFTMAX_STRIDED_FWD, OP_SOFTMAX_STRIDED_BWD = 6, 7
OP_GROUP_NORM_FWD, OP_GROUP_NORM_BWD = 8, 9
SOFTMAX, LOG_SOFTMAX, SAFE_SOFTMAX = 0, 1, 2

EXPORTED_SYMBOLS = (
    "mi355x_rownorm_error_string", "mi355x_rownorm_abi_version", "mi355x_layer_norm_fwd",
    "mi355x_layer_norm_bwd_workspace_bytes", "mi355x_layer_norm_bwd", "mi355x_rms_norm_fwd",
    "mi355x_rms_norm_bwd_workspace_bytes", "mi355x_rms_norm_bwd",
    "mi355x_rms_norm_bwd_static_limit_bytes", "mi355x_rms_norm_bwd_static",
    "mi355x_add_layer_norm_fwd", "mi355x_add_rms_norm_fwd", "mi355x_add_layer_norm_bwd",
    "mi355x_add_rms_norm_bwd", "mi355x_softmax_fwd",
    "mi355x_softmax_bwd", "mi355x_safe_softmax_fwd", "mi355x_masked_softmax_fwd",
    "mi355x_masked_softmax_bwd", "mi355x_softmax_strided_fwd", "mi355x_softmax_strided_bwd",
    "mi355x_softmax_strided_plan", "mi355x_group_norm_fwd",
    "mi355x_group_norm_bwd_workspace_bytes", "mi355x_group_norm_bwd", "mi355x_group_norm_plan",
    "mi355x_rownorm_plan", "mi355x_rownorm_plan_at", "mi355x_rownorm_set_override",
    "mi355x_rownorm_stream_probe", "mi355x_rownorm_set_team_wait_us",
)


class Plan(ctypes.Structure):
    _fields_ = [("resident", ctypes.c_int32), ("lanes_per_row", ctypes.c_int32),
                ("packs_per_lane", ctypes.c_int32), ("block_threads", ctypes.c_int32),
                ("rows_per_block", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("grid_blocks", ctypes.c_int64), ("partial_rows", ctypes.c_int64)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_ if k != "reserved"}


_lib = None
_vp, _i64, _int, _f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float


def lib():
    """The kernel library; raises if it has not been built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_KERNEL_LIB):
            raise RuntimeError("%s is missing: run build.py next to this file" % _KERNEL_LIB)
        L = ctypes.CDLL(_KERNEL_LIB)
        L.mi355x_rownorm_error_string.restype = ctypes.c_char_p
        L.mi355x_rownorm_error_string.argtypes = [_int]
        L.mi355x_rownorm_abi_version.restype = _int
        L.mi355x_layer_norm_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int,
                                            _int, _vp]
        L.mi355x_rms_norm_fwd.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _f, _int, _int, _vp]
        L.mi355x_layer_norm_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.mi355x_layer_norm_bwd_workspace_bytes.argtypes = [_i64, _i64, _int, _int, _int, _int]
        L.mi355x_rms_norm_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.mi355x_rms_norm_bwd_workspace_bytes.argtypes = [_i64, _i64, _int, _int, _int]
        L.mi355x_layer_norm_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                            ctypes.c_size_t, _i64, _i64, _int, _int, _vp]
        L.mi355x_rms_norm_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t,
                                          _i64, _i64, _int, _int, _vp]
        L.mi355x_rms_norm_bwd_static_limit_bytes.restype = ctypes.c_size_t
        L.mi355x_rms_norm_bwd_static_limit_bytes.argtypes = []
        L.mi355x_rms_norm_bwd_static.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int,
                                                 _int, _vp]
        L.mi355x_add_layer_norm_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64,
                                                _f, _int, _int, _int, _vp]
        L.mi355x_add_rms_norm_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int,
                                              _int, _int, _vp]
        L.mi355x_add_layer_norm_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                                ctypes.c_size_t, _i64, _i64, _int, _int, _vp]
        L.mi355x_add_rms_norm_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                              ctypes.c_size_t, _i64, _i64, _int, _int, _vp]
        L.mi355x_softmax_fwd.argtypes = [_vp, _vp, _i64, _i64, _int, _int, _int, _vp]
        L.mi355x_softmax_bwd.argtypes = [_vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp]
        L.mi355x_safe_softmax_fwd.argtypes = [_vp, _vp, _i64, _i64, _int, _int, _vp]
        L.mi355x_masked_softmax_fwd.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                                _int, _vp]
        L.mi355x_masked_softmax_bwd.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                                _i64, _int, _vp]
        L.mi355x_softmax_strided_fwd.argtypes = [_vp, _vp, _i64, _i64, _i64, _int, _int, _int, _vp]
        L.mi355x_softmax_strided_bwd.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _int,
                                                 _vp]
        L.mi355x_softmax_strided_plan.argtypes = [_int, _i64, _i64, _i64, _int,
                                                  ctypes.POINTER(Plan)]
        L.mi355x_group_norm_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f,
                                            _int, _int, _vp]
        L.mi355x_group_norm_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.mi355x_group_norm_bwd_workspace_bytes.argtypes = [_i64, _i64, _i64, _i64, _int, _int,
                                                            _int, _int]
        L.mi355x_group_norm_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                            ctypes.c_size_t, _i64, _i64, _i64, _i64, _int, _int,
                                            _vp]
        L.mi355x_group_norm_plan.argtypes = [_int, _i64, _i64, _i64, _i64, _int,
                                             ctypes.POINTER(Plan)]
        L.mi355x_rownorm_plan.argtypes = [_int, _i64, _i64, _int, _int, ctypes.POINTER(Plan)]
        L.mi355x_rownorm_plan_at.argtypes = [_int, _i64, _i64, _int, _int, _int,
                                             ctypes.POINTER(Plan)]
        L.mi355x_rownorm_set_override.argtypes = [_int, _int, _int, _int, _int]
        L.mi355x_rownorm_stream_probe.argtypes = [_vp, _vp, _vp, ctypes.c_size_t, _int, _vp]
        L.mi355x_rownorm_stream_probe.restype = _int
        L.mi355x_rownorm_set_team_wait_us.argtypes = [ctypes.c_uint]
        L.mi355x_rownorm_set_team_wait_us.restype = _int
        for name in ("mi355x_layer_norm_fwd", "mi355x_rms_norm_fwd", "mi355x_layer_norm_bwd",
                     "mi355x_rms_norm_bwd", "mi355x_rms_norm_bwd_static",
                     "mi355x_add_layer_norm_fwd", "mi355x_add_rms_norm_fwd",
                     "mi355x_add_layer_norm_bwd", "mi355x_add_rms_norm_bwd", "mi355x_softmax_fwd",
                     "mi355x_softmax_bwd",
                     "mi355x_safe_softmax_fwd", "mi355x_masked_softmax_fwd",
                     "mi355x_masked_softmax_bwd", "mi355x_softmax_strided_fwd",
                     "mi355x_softmax_strided_bwd", "mi355x_softmax_strided_plan",
                     "mi355x_group_norm_fwd", "mi355x_group_norm_bwd", "mi355x_group_norm_plan",
                     "mi355x_rownorm_plan", "mi355x_rownorm_plan_at",
                     "mi355x_rownorm_set_override"):
            getattr(L, name).restype = _int
        _lib = L
    return _lib


def error_string(code):
    return lib().mi355x_rownorm_error_string(code).decode()


def _check(code, what):
    if code != 0:
        raise RuntimeError("%s failed: %s (code %d)" % (what, error_string(code), code))


def dtype_code(dt):
    import torch
    try:
        return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[dt]
    except KeyError:
        raise RuntimeError("dtype %s is not implemented by the MI355X kernels" % dt)


def plan(op, M, N, x_dtype=F32, w_dtype=F32, off_line=False):
    """The launch layout of a call; off_line: its tensors do not all start on a 128-byte line."""
    p = Plan()
    _check(lib().mi355x_rownorm_plan_at(op, M, N, x_dtype, w_dtype, int(off_line),
                                        ctypes.byref(p)), "plan")
    d = p.as_dict()
    d["row_chunks"] = p.reserved  # workgroups a row is split over (0: not split)
    return d


def set_override(op, lanes_per_row=0, packs_per_lane=0, block_threads=0, blocks_per_cu=0):
    _check(lib().mi355x_rownorm_set_override(op, lanes_per_row, packs_per_lane, block_threads,
                                             blocks_per_cu), "set_override")


def strided_plan(backward, outer, dim_size, inner, dtype=F32):
    p = Plan()
    _check(lib().mi355x_softmax_strided_plan(int(backward), outer, dim_size, inner, dtype,
                                             ctypes.byref(p)), "strided_plan")
    d = p.as_dict()
    d["dim_chunks"] = p.reserved  # workgroups the dim_size rows of a tile are split over (0: not split)
    return d


def group_norm_plan(backward, N, C, HxW, groups, dtype=F32):
    p = Plan()
    _check(lib().mi355x_group_norm_plan(int(backward), N, C, HxW, groups, dtype, ctypes.byref(p)),
           "group_norm_plan")
    d = p.as_dict()
    d["uniform"] = p.reserved  # 1: every pack in one channel, 2: packs may straddle two, 0: general kernels
    return d


def set_team_wait_us(microseconds=0xffffffff):
    """Bound of a workgroup's wait in the team kernels (norm forward rows beyond one workgroup's
    registers, softmax forward / backward of few very long rows); 0: every wait gives up at once
    and each workgroup sums its rows itself."""
    _check(lib().mi355x_rownorm_set_team_wait_us(ctypes.c_uint(microseconds)), "set_team_wait_us")


def clear_overrides():
    for op in range(10):
        set_override(op)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("expected a HIP GPU tensor, got device %s (no CPU path)" % t.device)


def _rows(x, n_norm_dims):
    axis = x.dim() - n_norm_dims
    M = 1
    for s in x.shape[:axis]:
        M *= s
    N = 1
    for s in x.shape[axis:]:
        N *= s
    return M, N


def _wd(x, *ws):
    for w in ws:
        if w is not None:
            return dtype_code(w.dtype)
    return dtype_code(x.dtype)


def layer_norm_fwd(x, gamma, beta, eps, n_norm_dims=1, y=None, mean=None, rstd=None):
    """-> (y, mean[M], rstd[M]); x is viewed as [M, N] (must be dense)."""
    import torch
    _gpu(x, gamma, beta)
    M, N = _rows(x, n_norm_dims)
    y = torch.empty_like(x) if y is None else y
    mean = torch.empty(M, dtype=torch.float32, device=x.device) if mean is None else mean
    rstd = torch.empty(M, dtype=torch.float32, device=x.device) if rstd is None else rstd
    _check(lib().mi355x_layer_norm_fwd(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(mean),
                                       _ptr(rstd), M, N, eps, dtype_code(x.dtype),
                                       _wd(x, gamma, beta), _stream()), "layer_norm_fwd")
    return y, mean, rstd


def rms_norm_fwd(x, gamma, eps, n_norm_dims=1, y=None, rstd=None):
    import torch
    _gpu(x, gamma)
    M, N = _rows(x, n_norm_dims)
    y = torch.empty_like(x) if y is None else y
    rstd = torch.empty(M, dtype=torch.float32, device=x.device) if rstd is None else rstd
    _check(lib().mi355x_rms_norm_fwd(_ptr(x), _ptr(gamma), _ptr(y), _ptr(rstd), M, N, eps,
                                     dtype_code(x.dtype), _wd(x, gamma), _stream()),
           "rms_norm_fwd")
    return y, rstd


def layer_norm_bwd(dy, x, mean, rstd, gamma, n_norm_dims=1, want=(True, True, True),
                   w_dtype=None, dx=None, dgamma=None, dbeta=None, workspace=None):
    import torch
    _gpu(dy, x, mean, rstd, gamma)
    M, N = _rows(x, n_norm_dims)
    wdt = w_dtype if w_dtype is not None else (gamma.dtype if gamma is not None else x.dtype)
    if want[0] and dx is None:
        dx = torch.empty_like(x)
    if want[1] and dgamma is None:
        dgamma = torch.empty(N, dtype=wdt, device=x.device)
    if want[2] and dbeta is None:
        dbeta = torch.empty(N, dtype=wdt, device=x.device)
    xd, wd = dtype_code(x.dtype), dtype_code(wdt)
    nbytes = lib().mi355x_layer_norm_bwd_workspace_bytes(M, N, xd, wd, int(dgamma is not None),
                                                         int(dbeta is not None))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _check(lib().mi355x_layer_norm_bwd(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma),
                                       _ptr(dx), _ptr(dgamma), _ptr(dbeta), _ptr(workspace),
                                       0 if workspace is None else workspace.numel(), M, N, xd, wd,
                                       _stream()), "layer_norm_bwd")
    return dx, dgamma, dbeta


def rms_norm_bwd(dy, x, rstd, gamma, n_norm_dims=1, want=(True, True), w_dtype=None, dx=None,
                 dgamma=None, workspace=None):
    import torch
    _gpu(dy, x, rstd, gamma)
    M, N = _rows(x, n_norm_dims)
    wdt = w_dtype if w_dtype is not None else (gamma.dtype if gamma is not None else x.dtype)
    if want[0] and dx is None:
        dx = torch.empty_like(x)
    if want[1] and dgamma is None:
        dgamma = torch.empty(N, dtype=wdt, device=x.device)
    xd, wd = dtype_code(x.dtype), dtype_code(wdt)
    nbytes = lib().mi355x_rms_norm_bwd_workspace_bytes(M, N, xd, wd, int(dgamma is not None))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _check(lib().mi355x_rms_norm_bwd(_ptr(dy), _ptr(x), _ptr(rstd), _ptr(gamma), _ptr(dx),
                                     _ptr(dgamma), _ptr(workspace),
                                     0 if workspace is None else workspace.numel(), M, N, xd, wd,
                                     _stream()), "rms_norm_bwd")
    return dx, dgamma


def rms_norm_bwd_static(dy, x, rstd, gamma, dx, dgamma, n_norm_dims=1, w_dtype=None):
    """mi355x_rms_norm_bwd_static: the caller brings every output (either may be None = not
    wanted); the scratch is the library's own static device array, nothing is allocated."""
    _gpu(dy, x, rstd, gamma, dx, dgamma)
    M, N = _rows(x, n_norm_dims)
    wdt = w_dtype if w_dtype is not None else (
        dgamma.dtype if dgamma is not None else (gamma.dtype if gamma is not None else x.dtype))
    _check(lib().mi355x_rms_norm_bwd_static(_ptr(dy), _ptr(x), _ptr(rstd), _ptr(gamma), _ptr(dx),
                                            _ptr(dgamma), M, N, dtype_code(x.dtype),
                                            dtype_code(wdt), _stream()), "rms_norm_bwd_static")
    return dx, dgamma


def add_layer_norm_fwd(x, residual, gamma, beta, eps, n_norm_dims=1, y_dtype=None, h=None, y=None,
                       mean=None, rstd=None):
    """Fused residual add -> LayerNorm (-> cast): -> (y, h, mean[M], rstd[M]) with h = x + residual
    (pass h=residual to update the residual stream in place).  residual=None: the plain norm with
    the output cast (h comes back None)."""
    import torch
    _gpu(x, residual, gamma, beta, h, y)
    M, N = _rows(x, n_norm_dims)
    if residual is not None and h is None:
        h = torch.empty_like(x)
    y = torch.empty(x.shape, dtype=y_dtype or x.dtype, device=x.device) if y is None else y
    mean = torch.empty(M, dtype=torch.float32, device=x.device) if mean is None else mean
    rstd = torch.empty(M, dtype=torch.float32, device=x.device) if rstd is None else rstd
    _check(lib().mi355x_add_layer_norm_fwd(_ptr(x), _ptr(residual), _ptr(gamma), _ptr(beta),
                                           _ptr(h), _ptr(y), _ptr(mean), _ptr(rstd), M, N, eps,
                                           dtype_code(x.dtype), _wd(x, gamma, beta),
                                           dtype_code(y.dtype), _stream()), "add_layer_norm_fwd")
    return y, h, mean, rstd


def add_rms_norm_fwd(x, residual, gamma, eps, n_norm_dims=1, y_dtype=None, h=None, y=None,
                     rstd=None):
    """Fused residual add -> RMSNorm (-> cast): -> (y, h, rstd[M])."""
    import torch
    _gpu(x, residual, gamma, h, y)
    M, N = _rows(x, n_norm_dims)
    if residual is not None and h is None:
        h = torch.empty_like(x)
    y = torch.empty(x.shape, dtype=y_dtype or x.dtype, device=x.device) if y is None else y
    rstd = torch.empty(M, dtype=torch.float32, device=x.device) if rstd is None else rstd
    _check(lib().mi355x_add_rms_norm_fwd(_ptr(x), _ptr(residual), _ptr(gamma), _ptr(h), _ptr(y),
                                         _ptr(rstd), M, N, eps, dtype_code(x.dtype), _wd(x, gamma),
                                         dtype_code(y.dtype), _stream()), "add_rms_norm_fwd")
    return y, h, rstd


def add_layer_norm_bwd(dy, dh_in, h, mean, rstd, gamma, n_norm_dims=1, want=(True, True, True),
                       w_dtype=None, dh=None, dgamma=None, dbeta=None, workspace=None):
    """Backward of the fused add -> LayerNorm: -> (dh, dgamma, dbeta); dh = the norm's input
    gradient + dh_in (None: nothing to add) is the gradient of both x and residual."""
    import torch
    _gpu(dy, dh_in, h, mean, rstd, gamma)
    M, N = _rows(h, n_norm_dims)
    wdt = w_dtype if w_dtype is not None else (gamma.dtype if gamma is not None else h.dtype)
    if want[0] and dh is None:
        dh = torch.empty_like(h)
    if want[1] and dgamma is None:
        dgamma = torch.empty(N, dtype=wdt, device=h.device)
    if want[2] and dbeta is None:
        dbeta = torch.empty(N, dtype=wdt, device=h.device)
    xd, wd = dtype_code(h.dtype), dtype_code(wdt)
    nbytes = lib().mi355x_layer_norm_bwd_workspace_bytes(M, N, xd, wd, int(dgamma is not None),
                                                         int(dbeta is not None))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=h.device)
    _check(lib().mi355x_add_layer_norm_bwd(_ptr(dy), _ptr(dh_in), _ptr(h), _ptr(mean), _ptr(rstd),
                                           _ptr(gamma), _ptr(dh), _ptr(dgamma), _ptr(dbeta),
                                           _ptr(workspace),
                                           0 if workspace is None else workspace.numel(), M, N, xd,
                                           wd, _stream()), "add_layer_norm_bwd")
    return dh, dgamma, dbeta


def add_rms_norm_bwd(dy, dh_in, h, rstd, gamma, n_norm_dims=1, want=(True, True), w_dtype=None,
                     dh=None, dgamma=None, workspace=None):
    import torch
    _gpu(dy, dh_in, h, rstd, gamma)
    M, N = _rows(h, n_norm_dims)
    wdt = w_dtype if w_dtype is not None else (gamma.dtype if gamma is not None else h.dtype)
    if want[0] and dh is None:
        dh = torch.empty_like(h)
    if want[1] and dgamma is None:
        dgamma = torch.empty(N, dtype=wdt, device=h.device)
    xd, wd = dtype_code(h.dtype), dtype_code(wdt)
    nbytes = lib().mi355x_rms_norm_bwd_workspace_bytes(M, N, xd, wd, int(dgamma is not None))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=h.device)
    _check(lib().mi355x_add_rms_norm_bwd(_ptr(dy), _ptr(dh_in), _ptr(h), _ptr(rstd), _ptr(gamma),
                                         _ptr(dh), _ptr(dgamma), _ptr(workspace),
                                         0 if workspace is None else workspace.numel(), M, N, xd, wd,
                                         _stream()), "add_rms_norm_bwd")
    return dh, dgamma


def softmax_fwd(x, is_log=False, out_dtype=None, y=None):
    import torch
    _gpu(x)
    N = x.shape[-1] if x.dim() else 1
    rows = x.numel() // N if N else 0
    od = x.dtype if out_dtype is None else out_dtype
    y = torch.empty(x.shape, dtype=od, device=x.device) if y is None else y
    _check(lib().mi355x_softmax_fwd(_ptr(x), _ptr(y), rows, N, dtype_code(x.dtype),
                                    dtype_code(y.dtype), int(is_log), _stream()), "softmax_fwd")
    return y


def softmax_bwd(grad, y, is_log=False, gi_dtype=None, gi=None):
    import torch
    _gpu(grad, y)
    N = y.shape[-1] if y.dim() else 1
    rows = y.numel() // N if N else 0
    od = grad.dtype if gi_dtype is None else gi_dtype
    gi = torch.empty(y.shape, dtype=od, device=y.device) if gi is None else gi
    _check(lib().mi355x_softmax_bwd(_ptr(grad), _ptr(y), _ptr(gi), rows, N,
                                    dtype_code(grad.dtype), dtype_code(gi.dtype), int(is_log),
                                    _stream()), "softmax_bwd")
    return gi


def safe_softmax_fwd(x, out_dtype=None, y=None):
    """softmax over the last dim; rows that are all -inf give zeros."""
    import torch
    _gpu(x)
    N = x.shape[-1] if x.dim() else 1
    rows = x.numel() // N if N else 0
    od = x.dtype if out_dtype is None else out_dtype
    y = torch.empty(x.shape, dtype=od, device=x.device) if y is None else y
    _check(lib().mi355x_safe_softmax_fwd(_ptr(x), _ptr(y), rows, N, dtype_code(x.dtype),
                                         dtype_code(y.dtype), _stream()), "safe_softmax_fwd")
    return y


def mask_row_map(shape, mask_shape):
    """(mask_rows, div, stride, mod) for a bool mask of ``mask_shape`` under last-dim softmax of a
    dense tensor of ``shape``: the mask's own shape, [B, T] or [T, T] or [B, 1, T, T] under
    [B, H, T, T]."""
    shape, mask_shape = tuple(shape), tuple(mask_shape)
    N = shape[-1]
    rows = 1
    for s in shape[:-1]:
        rows *= s
    if mask_shape == shape:
        return rows, 1, 1, 1
    if len(shape) == 4:
        B, H, T, _ = shape
        if mask_shape == (B, N) and T == N:
            return B, H * T, 1, 1
        if mask_shape == (T, N) and T == N:
            return T, 1, 0, T
        if mask_shape == (B, 1, T, N):
            return B * T, H * T, T, T
    raise RuntimeError("mask shape %s does not fit input %s" % (mask_shape, shape))


def masked_softmax_fwd(x, mask, y=None, row_map=None):
    """mask: torch.bool, True = leave the element out."""
    import torch
    _gpu(x, mask)
    if mask.dtype != torch.bool:
        raise RuntimeError("Mask should be a boolean tensor")
    N = x.shape[-1] if x.dim() else 1
    rows = x.numel() // N if N else 0
    mrows, div, stride, mod = row_map or mask_row_map(x.shape, mask.shape)
    y = torch.empty_like(x) if y is None else y
    _check(lib().mi355x_masked_softmax_fwd(_ptr(x), _ptr(mask), _ptr(y), rows, N, mrows, div,
                                           stride, mod, dtype_code(x.dtype), _stream()),
           "masked_softmax_fwd")
    return y


def masked_softmax_bwd(grad, y, mask, gi=None, row_map=None):
    import torch
    _gpu(grad, y, mask)
    if mask.dtype != torch.bool:
        raise RuntimeError("Mask should be a boolean tensor")
    N = y.shape[-1] if y.dim() else 1
    rows = y.numel() // N if N else 0
    mrows, div, stride, mod = row_map or mask_row_map(y.shape, mask.shape)
    gi = torch.empty_like(grad) if gi is None else gi
    _check(lib().mi355x_masked_softmax_bwd(_ptr(grad), _ptr(y), _ptr(mask), _ptr(gi), rows, N,
                                           mrows, div, stride, mod, dtype_code(grad.dtype),
                                           _stream()), "masked_softmax_bwd")
    return gi


def _outer_dim_inner(shape, dim):
    dim = dim % len(shape)
    outer = inner = 1
    for s in shape[:dim]:
        outer *= s
    for s in shape[dim + 1:]:
        inner *= s
    return outer, shape[dim], inner


def softmax_strided_fwd(x, dim, mode=SOFTMAX, out_dtype=None, y=None):
    """softmax (mode SOFTMAX / LOG_SOFTMAX / SAFE_SOFTMAX) over any dim of a dense tensor."""
    import torch
    _gpu(x)
    outer, D, inner = _outer_dim_inner(x.shape, dim)
    od = x.dtype if out_dtype is None else out_dtype
    y = torch.empty(x.shape, dtype=od, device=x.device) if y is None else y
    _check(lib().mi355x_softmax_strided_fwd(_ptr(x), _ptr(y), outer, D, inner, dtype_code(x.dtype),
                                            dtype_code(y.dtype), mode, _stream()),
           "softmax_strided_fwd")
    return y


def softmax_strided_bwd(grad, y, dim, mode=SOFTMAX, gi_dtype=None, gi=None):
    import torch
    _gpu(grad, y)
    outer, D, inner = _outer_dim_inner(y.shape, dim)
    od = grad.dtype if gi_dtype is None else gi_dtype
    gi = torch.empty(y.shape, dtype=od, device=y.device) if gi is None else gi
    _check(lib().mi355x_softmax_strided_bwd(_ptr(grad), _ptr(y), _ptr(gi), outer, D, inner,
                                            dtype_code(grad.dtype), dtype_code(gi.dtype), mode,
                                            _stream()), "softmax_strided_bwd")
    return gi


def _nchw(x):
    N, C = x.shape[0], x.shape[1]
    HxW = 1
    for s in x.shape[2:]:
        HxW *= s
    return N, C, HxW


def group_norm_fwd(x, gamma, beta, groups, eps, y=None, mean=None, rstd=None):
    """-> (y, mean[N, groups], rstd[N, groups]); x is a dense [N, C, *]; the statistics come in
    the weight dtype (the input dtype when there are no weights)."""
    import torch
    _gpu(x, gamma, beta)
    N, C, HxW = _nchw(x)
    sdt = gamma.dtype if gamma is not None else (beta.dtype if beta is not None else x.dtype)
    y = torch.empty_like(x) if y is None else y
    mean = torch.empty(N, groups, dtype=sdt, device=x.device) if mean is None else mean
    rstd = torch.empty(N, groups, dtype=sdt, device=x.device) if rstd is None else rstd
    _check(lib().mi355x_group_norm_fwd(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(mean),
                                       _ptr(rstd), N, C, HxW, groups, eps, dtype_code(x.dtype),
                                       dtype_code(sdt), _stream()), "group_norm_fwd")
    return y, mean, rstd


def group_norm_bwd(dy, x, mean, rstd, gamma, groups, want=(True, True, True), dx=None,
                   dgamma=None, dbeta=None, workspace=None):
    import torch
    _gpu(dy, x, mean, rstd, gamma)
    N, C, HxW = _nchw(x)
    wdt = mean.dtype
    if want[0] and dx is None:
        dx = torch.empty_like(x)
    if want[1] and dgamma is None:
        dgamma = torch.empty(C, dtype=wdt, device=x.device)
    if want[2] and dbeta is None:
        dbeta = torch.empty(C, dtype=wdt, device=x.device)
    xd, wd = dtype_code(x.dtype), dtype_code(wdt)
    nbytes = lib().mi355x_group_norm_bwd_workspace_bytes(N, C, HxW, groups, xd, wd,
                                                         int(dgamma is not None),
                                                         int(dbeta is not None))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _check(lib().mi355x_group_norm_bwd(_ptr(dy), _ptr(x), _ptr(mean), _ptr(rstd), _ptr(gamma),
                                       _ptr(dx), _ptr(dgamma), _ptr(dbeta), _ptr(workspace),
                                       0 if workspace is None else workspace.numel(), N, C, HxW,
                                       groups, xd, wd, _stream()), "group_norm_bwd")
    return dx, dgamma, dbeta
