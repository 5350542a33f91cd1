"""CPU-only checks of the ATen-facing host layer (torch.ops.mi355x.*): the operators are
registered with the reference's schemas, raise the same argument errors as ATen before any
launch, and refuse tensors that are not on a GPU (there is no CPU path to fall back to)."""
import pytest
import torch


def _aten_message(fn):
    with pytest.raises(RuntimeError) as e:
        fn()
    return str(e.value).split("\n")[0]


def test_ops_are_registered_with_the_reference_schemas(ops):
    expect = {
        "native_layer_norm": "(Tensor input, int[] normalized_shape, Tensor? weight, Tensor? bias, float eps) -> (Tensor, Tensor, Tensor)",
        "native_layer_norm_backward": "(Tensor grad_out, Tensor input, int[] normalized_shape, Tensor mean, Tensor rstd, Tensor? weight, Tensor? bias, bool[3] output_mask) -> (Tensor, Tensor, Tensor)",
        "_fused_rms_norm": "(Tensor input, int[] normalized_shape, Tensor? weight, float? eps) -> (Tensor, Tensor)",
        "_fused_rms_norm_backward": "(Tensor grad_out, Tensor input, int[] normalized_shape, Tensor rstd, Tensor? weight, bool[2] output_mask) -> (Tensor, Tensor)",
        "_softmax": "(Tensor self, int dim, bool half_to_float) -> Tensor",
        "_log_softmax": "(Tensor self, int dim, bool half_to_float) -> Tensor",
        "_softmax_backward_data": "(Tensor grad_output, Tensor output, int dim, ScalarType input_dtype) -> Tensor",
        "_log_softmax_backward_data": "(Tensor grad_output, Tensor output, int dim, ScalarType input_dtype) -> Tensor",
        "native_group_norm": "(Tensor input, Tensor? weight, Tensor? bias, int N, int C, int HxW, int group, float eps) -> (Tensor, Tensor, Tensor)",
        "native_group_norm_backward": "(Tensor grad_out, Tensor input, Tensor mean, Tensor rstd, Tensor? weight, int N, int C, int HxW, int group, bool[3] output_mask) -> (Tensor, Tensor, Tensor)",
        "_safe_softmax": "(Tensor self, int dim, ScalarType? dtype=None) -> Tensor",
        "_masked_softmax": "(Tensor self, Tensor mask, int? dim=None, int? mask_type=None) -> Tensor",
        "_masked_softmax_backward": "(Tensor grad_output, Tensor output, Tensor mask, int? dim=None) -> Tensor",
    }
    for name, sig in expect.items():
        schema = str(getattr(ops, name).default._schema)
        assert schema == "mi355x::" + name + sig, schema
    for name in ("_softmax", "_log_softmax", "_softmax_backward_data", "_log_softmax_backward_data"):
        assert hasattr(getattr(ops, name), "out")


def test_shape_errors_match_aten(ops):
    x = torch.randn(4, 8)
    cases = [
        lambda m: m.native_layer_norm(x, [7], None, None, 1e-5),
        lambda m: m.native_layer_norm(x, [], None, None, 1e-5),
        lambda m: m.native_layer_norm(x, [8], torch.randn(7), None, 1e-5),
        lambda m: m.native_layer_norm(x, [8], None, torch.randn(9), 1e-5),
        lambda m: m.native_layer_norm(x, [2, 4, 8], None, None, 1e-5),
    ]
    for fn in cases:
        assert _aten_message(lambda: fn(ops)) == _aten_message(lambda: fn(torch.ops.aten))
    with pytest.raises(RuntimeError, match="Expected weight to be of same shape"):
        ops._fused_rms_norm(x, [8], torch.randn(4), None)
    with pytest.raises(RuntimeError, match="Given normalized_shape="):
        ops._fused_rms_norm_backward(x, x, [5], torch.randn(4, 1), None, [True, False])


def test_cpu_tensors_are_rejected_loudly(ops):
    x = torch.randn(4, 8)
    m, r = torch.zeros(4, 1), torch.ones(4, 1)
    calls = [
        lambda: ops.native_layer_norm(x, [8], None, None, 1e-5),
        lambda: ops.native_layer_norm_backward(x, x, [8], m, r, None, None, [True, False, False]),
        lambda: ops._fused_rms_norm(x, [8], None, None),
        lambda: ops._fused_rms_norm_backward(x, x, [8], r, None, [True, False]),
        lambda: ops._softmax(x, -1, False),
        lambda: ops._log_softmax(x, -1, False),
        lambda: ops._softmax_backward_data(x, x, -1, torch.float32),
        lambda: ops._log_softmax_backward_data(x, x, -1, torch.float32),
        lambda: ops._safe_softmax(x, -1),
        lambda: ops.native_group_norm(x, None, None, 4, 8, 1, 2, 1e-5),
        lambda: ops.native_group_norm_backward(x, x, m[:, :1].expand(4, 2), r.expand(4, 2), None, 4, 8, 1, 2,
                                               [True, False, False]),
        lambda: ops._masked_softmax(x, x > 0, -1, 2),
        lambda: ops._masked_softmax_backward(x, x, x > 0, -1),
    ]
    for fn in calls:
        with pytest.raises(RuntimeError, match="no CPU path"):
            fn()


def test_softmax_backward_dtype_rule(ops):
    # SoftMax.cpp:49-55 in the reference: grad dtype != input dtype is legal only for
    # (Float grad, Half input)
    g = torch.randn(2, 4)
    with pytest.raises(RuntimeError, match="expected input and grad types to match"):
        ops._softmax_backward_data(g, g, -1, torch.bfloat16)
    with pytest.raises(RuntimeError, match="expected input and grad types to match"):
        ops._log_softmax_backward_data(g.half(), g.half(), -1, torch.float32)


def test_ctypes_layer_rejects_cpu_tensors(cabi):
    x = torch.randn(4, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        cabi.rms_norm_fwd(x, None, 1e-6)
    with pytest.raises(RuntimeError, match="not implemented"):
        cabi.dtype_code(torch.float64)


def test_masked_softmax_argument_errors(ops):
    # the checks and messages of masked_softmax_kernel / masked_softmax_backward_kernel
    # (SoftMaxKernels.cpp:2308-2338 and 2382-2390 in the reference); CPU ATen words the shape
    # errors differently and accepts a missing mask type, the reference does not
    x = torch.randn(2, 3, 4, 4)
    ok = torch.zeros(2, 3, 4, 4, dtype=torch.bool)
    assert _aten_message(lambda: ops._masked_softmax(x, ok.float(), -1, 2)) == \
        _aten_message(lambda: torch.ops.aten._masked_softmax(x, ok.float(), -1, 2))
    with pytest.raises(RuntimeError, match="Mask Type should be defined"):
        ops._masked_softmax(x, ok, -1, None)
    with pytest.raises(RuntimeError, match="Mask Type should be 0 .src_mask., 1 .src_key_padding"):
        ops._masked_softmax(x, ok, -1, 3)
    with pytest.raises(RuntimeError, match="Mask shape should match input. mask: .2, 2, 4, 4."):
        ops._masked_softmax(x, ok[:, :2], -1, 2)
    with pytest.raises(RuntimeError, match="Mask shape should match input"):
        ops._masked_softmax(x, ok[0, 0], -1, 1)  # [T, T] is not a key-padding mask
    with pytest.raises(RuntimeError, match="Mask shape should match input"):
        ops._masked_softmax(x, ok[:, 0, 0], -1, 0)  # [B, T] is not a src mask


def test_group_norm_argument_errors_match_aten(ops):
    x = torch.randn(2, 6, 4)
    cases = [
        lambda m: m.native_group_norm(x, None, None, 2, 6, 4, 4, 1e-5),              # C % groups
        lambda m: m.native_group_norm(x, torch.randn(5), None, 2, 6, 4, 3, 1e-5),     # weight size
        lambda m: m.native_group_norm(x, None, None, 2, 6, 4, 0, 1e-5),              # no groups
        lambda m: m.native_group_norm_backward(x.half(), x, torch.zeros(2, 3), torch.ones(2, 3), None, 2, 6, 4,
                                               3, [True, False, False]),              # dY dtype
    ]
    for fn in cases:
        assert _aten_message(lambda: fn(ops)) == _aten_message(lambda: fn(torch.ops.aten))
    with pytest.raises(RuntimeError, match="Expected bias to be a vector of size equal to the number of channels"):
        ops.native_group_norm(x, None, torch.randn(7), 2, 6, 4, 3, 1e-5)
