"""MI355X-native LayerNorm / RMSNorm / softmax operators (the row-wise reduce-then-normalize
family of intel/torch-xpu-ops, rebuilt for gfx950).

The directory name is not a Python identifier; load the package with ``importlib`` under the
name ``torch_xpu_ops_amd`` (see ``load_package`` in ``tests/conftest.py``) or put its parent on
``sys.path`` and use ``importlib.import_module("torch-xpu-ops_amd")``.

Two layers are exposed:
  * ``ops``   -- ``torch.ops.mi355x.*``: the C++ host layer with the ATen operator signatures
                 (native_layer_norm, native_layer_norm_backward, _fused_rms_norm,
                 _fused_rms_norm_backward, _softmax, _log_softmax and their backward ops).
  * ``fused`` -- ``add_rms_norm`` / ``add_layer_norm``: the residual add fused into the norm, with
                 autograd (``torch.ops.mi355x.add_rms_norm`` & co. underneath).
  * ``cabi``  -- ctypes bindings of the ``extern "C"`` launcher ABI (include/mi355x_rownorm.h),
                 taking torch tensors only as device memory.
There is no CPU path and no fallback: if the compiled libraries are missing the import raises.
(float64 GPU tensors, which these float32-accumulating kernels do not compute, are passed on by
the host layer to the kernels PyTorch-ROCm ships.)
"""
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libmi355x_rownorm.so")
HOST_LIB = os.path.join(LIB_DIR, "libmi355x_rownorm_aten.so")

_state = {"host_loaded": False, "aten_lib": None}


def _require(path):
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `python %s` (hipcc --offload-arch=gfx950). "
            "This package has no fallback path." % (path, os.path.join(_HERE, "build.py")))
    return path


def load_host_library():
    """Loads the C++ host layer and returns ``torch.ops.mi355x``."""
    import torch
    if not _state["host_loaded"]:
        _require(KERNEL_LIB)
        torch.ops.load_library(_require(HOST_LIB))
        _state["host_loaded"] = True
    return torch.ops.mi355x


class _LazyOps(object):
    def __getattr__(self, name):
        return getattr(load_host_library(), name)


ops = _LazyOps()

from . import cabi  # noqa: E402  (ctypes layer; loads the kernel library on first use)
from . import fused  # noqa: E402  (fused residual add -> norm with autograd)


def override_aten_ops():
    """Explicit opt-in: route the aten ops of this family to the MI355X kernels for GPU tensors,
    so ``F.layer_norm`` / ``F.rms_norm`` / ``F.group_norm`` / ``F.softmax`` / ``F.log_softmax``,
    ``torch._masked_softmax`` / ``torch._safe_softmax`` and their autograd formulas run them.
    PyTorch warns about overriding existing kernels; that is why this is never done at import.
    float64 GPU tensors are handed on to the kernels PyTorch-ROCm itself ships (one warning per
    process), so code that worked before the override keeps working.  ``restore_aten_ops()``
    undoes the override."""
    import torch
    if _state["aten_lib"] is not None:
        return _state["aten_lib"]
    m = load_host_library()
    lib = torch.library.Library("aten", "IMPL")
    lib.impl("native_layer_norm", m.native_layer_norm.default, "CUDA")
    lib.impl("native_layer_norm_backward", m.native_layer_norm_backward.default, "CUDA")
    lib.impl("_fused_rms_norm", m._fused_rms_norm.default, "CUDA")
    lib.impl("_fused_rms_norm_backward", m._fused_rms_norm_backward.default, "CUDA")
    lib.impl("_softmax", m._softmax.default, "CUDA")
    lib.impl("_log_softmax", m._log_softmax.default, "CUDA")
    lib.impl("_softmax_backward_data", m._softmax_backward_data.default, "CUDA")
    lib.impl("_log_softmax_backward_data", m._log_softmax_backward_data.default, "CUDA")
    # the structured `.out` kernels the reference implements (src/ATen/native/xpu/SoftMax.cpp:
    # 22-100): torch.softmax(x, dim, out=o) and the backward `.out` forms
    lib.impl("_softmax.out", m._softmax.out, "CUDA")
    lib.impl("_log_softmax.out", m._log_softmax.out, "CUDA")
    lib.impl("_softmax_backward_data.out", m._softmax_backward_data.out, "CUDA")
    lib.impl("_log_softmax_backward_data.out", m._log_softmax_backward_data.out, "CUDA")
    lib.impl("native_group_norm", m.native_group_norm.default, "CUDA")
    lib.impl("native_group_norm_backward", m.native_group_norm_backward.default, "CUDA")
    lib.impl("_safe_softmax", m._safe_softmax.default, "CUDA")
    lib.impl("_masked_softmax", m._masked_softmax.default, "CUDA")
    lib.impl("_masked_softmax_backward", m._masked_softmax_backward.default, "CUDA")
    _state["aten_lib"] = lib
    return lib


def restore_aten_ops():
    """Drops the registrations made by ``override_aten_ops()``: the aten ops go back to the kernels
    PyTorch-ROCm ships.  A no-op when nothing is overridden."""
    lib = _state["aten_lib"]
    if lib is not None:
        lib._destroy()
        _state["aten_lib"] = None
