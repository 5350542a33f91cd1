"""Fused residual add -> LayerNorm / RMSNorm with autograd, on top of ``torch.ops.mi355x``.

The step either side of the norm in a transformer block::

    h = x + residual            # the residual stream
    y = rms_norm(h) * weight    # input of the next projection

runs as one kernel that reads x and residual once and writes h and y once (an add followed by a
norm reads three tensors and writes two).  ``y`` can be written in 16 bits from float32 rows
(``out_dtype``), fusing the cast in front of a 16-bit matrix multiply as well.  The backward adds
the gradient that reaches ``h`` through the residual stream to the norm's input gradient in the
same kernel.  The reference (intel/torch-xpu-ops) has no fused operator: the results equal its
LayerNorm / RMSNorm applied to ``x + residual`` rounded to the row dtype.
"""
import torch


def _ops():
    from . import load_host_library
    return load_host_library()


class _AddRMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, residual, weight, eps, normalized_shape):
        y, h, rstd = _ops().add_rms_norm(x, residual, normalized_shape, weight, eps, None)
        ctx.save_for_backward(h, rstd, weight)
        ctx.normalized_shape = normalized_shape
        # an output the loss does not use arrives as None in backward, not as a tensor of
        # zeros that would be allocated, written and read for nothing
        ctx.set_materialize_grads(False)
        return y, h

    @staticmethod
    def backward(ctx, grad_y, grad_h):
        h, rstd, weight = ctx.saved_tensors
        if grad_y is None:  # only h feeds the loss: its gradient passes through
            return grad_h, grad_h, None, None, None
        want_w = weight is not None and ctx.needs_input_grad[2]
        dh, dw = _ops().add_rms_norm_backward(
            grad_y.contiguous(), None if grad_h is None else grad_h.contiguous(), h,
            ctx.normalized_shape, rstd, weight, [True, want_w])
        # h = x + residual: both get the gradient of h
        return dh, dh, dw, None, None


class _AddLayerNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, residual, weight, bias, eps, normalized_shape):
        y, h, mean, rstd = _ops().add_layer_norm(x, residual, normalized_shape, weight, bias, eps,
                                                 None)
        ctx.save_for_backward(h, mean, rstd, weight, bias)
        ctx.normalized_shape = normalized_shape
        ctx.set_materialize_grads(False)
        return y, h

    @staticmethod
    def backward(ctx, grad_y, grad_h):
        h, mean, rstd, weight, bias = ctx.saved_tensors
        if grad_y is None:
            return grad_h, grad_h, None, None, None, None
        mask = [True, weight is not None and ctx.needs_input_grad[2],
                bias is not None and ctx.needs_input_grad[3]]
        dh, dw, db = _ops().add_layer_norm_backward(
            grad_y.contiguous(), None if grad_h is None else grad_h.contiguous(), h,
            ctx.normalized_shape, mean, rstd, weight, bias, mask)
        return dh, dh, dw, db, None, None


def add_rms_norm(x, residual, weight=None, eps=None, normalized_shape=None):
    """-> (y, h) with h = x + residual and y = rms_norm(h) * weight; differentiable."""
    shape = list(normalized_shape) if normalized_shape is not None else [x.shape[-1]]
    return _AddRMSNorm.apply(x, residual, weight, eps, shape)


def add_layer_norm(x, residual, weight=None, bias=None, eps=1e-5, normalized_shape=None):
    """-> (y, h) with h = x + residual and y = layer_norm(h); differentiable."""
    shape = list(normalized_shape) if normalized_shape is not None else [x.shape[-1]]
    return _AddLayerNorm.apply(x, residual, weight, bias, eps, shape)
