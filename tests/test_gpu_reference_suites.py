"""Two of the reference's own device-vs-CPU suites, run against these kernels through the opt-in
aten override (nn.LayerNorm / F.softmax on GPU tensors, autograd included), with the reference's
sizes and tolerances:

  test/xpu/test_nn_xpu.py:9669-9727   test_layer_norm_backwards_eps: weight/bias gradients for
      (m, n) from (3, 3) to (128*1024, 32) and (32, 128*1024), every affine/bias combination;
  test/xpu/test_nn_xpu.py:14056-14106 test_softmax_results: softmax and log_softmax with
      dtype=float, odd sizes, inputs sliced by (1, 1) so rows start misaligned, dim 0 and 1,
      forward, backward and double backward.
"""
import itertools

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from helpers import gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def overridden(pkg):
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    return pkg


def test_layer_norm_backwards_eps(overridden, gpu):
    sizes = [(3, 3), (5, 5), (11, 11), (55, 55), (32, 32), (1024, 32), (1024, 1024), (33, 33), (1025, 33),
             (1025, 1025), (128 * 1024, 32), (32, 128 * 1024)]
    g = gen(81)
    for affine, bias in itertools.product([True, False], repeat=2):
        for m, n in sizes:
            print("case layer_norm_backwards_eps", affine, bias, m, n, flush=True)
            x = torch.randn(m, n, generator=g, requires_grad=True)
            go = torch.rand(m, n, generator=g)
            xg = x.clone().detach().to(gpu).requires_grad_()
            ln = nn.LayerNorm(n, elementwise_affine=affine, bias=bias)
            lng = nn.LayerNorm(n, elementwise_affine=affine, bias=bias, device=gpu)
            ln(x).backward(go)
            lng(xg).backward(go.to(gpu))
            atol, rtol = (1e-3, 1e-3) if m > 64 * 1024 else (1e-4, 1e-5)
            if affine:
                torch.testing.assert_close(lng.weight.grad.cpu(), ln.weight.grad, rtol=rtol, atol=atol,
                                           msg=lambda s: "weight grad failed: m=%d n=%d\n%s" % (m, n, s))
            if bias and affine:
                torch.testing.assert_close(lng.bias.grad.cpu(), ln.bias.grad, rtol=rtol, atol=atol,
                                           msg=lambda s: "bias grad failed: m=%d n=%d\n%s" % (m, n, s))
            torch.testing.assert_close(xg.grad.cpu(), x.grad, rtol=1e-4, atol=1e-5,
                                       msg=lambda s: "input grad failed: m=%d n=%d\n%s" % (m, n, s))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
def test_softmax_results(overridden, gpu, dtype):
    sizes = [(0, 10), (32, 20), (10, 0), (31, 20), (32, 21), (31, 23), (32, 1536), (31, 2048), (33, 2049),
             (16, 30576)]
    shifts = [(0, 0), (1, 0), (0, 1), (1, 1)]
    g = gen(82)
    for fn in (F.softmax, F.log_softmax):
        for size in sizes:
            for shift in shifts:
                print("case softmax_results", fn.__name__, dtype, size, shift, flush=True)
                base = torch.rand(size, generator=g).to(dtype)
                if dtype == torch.float16:
                    base = base / 100.0
                go_base = torch.rand(size, generator=g).to(dtype)
                inp = base.to(gpu)[shift[0]:, shift[1]:].detach().requires_grad_(True)
                ref_inp = base[shift[0]:, shift[1]:].clone().detach().requires_grad_(True)
                grad_out = go_base.to(gpu)[shift[0]:, shift[1]:]
                ref_grad_out = go_base[shift[0]:, shift[1]:].clone()
                for dim in (0, 1):
                    out = fn(inp, dtype=torch.float, dim=dim)
                    ref_out = fn(ref_inp, dtype=torch.float, dim=dim)
                    (gi,) = torch.autograd.grad(out, inp, grad_outputs=grad_out, create_graph=True)
                    (ref_gi,) = torch.autograd.grad(ref_out, ref_inp, grad_outputs=ref_grad_out,
                                                    create_graph=True)
                    gi.sum().backward()
                    ref_gi.sum().backward()
                    assert out.dtype == torch.float32 and gi.dtype == dtype
                    # default assertEqual tolerances of the reference's TestCase for these dtypes
                    tol = dict(rtol=1.3e-6, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-3, atol=1e-5)
                    torch.testing.assert_close(out.cpu(), ref_out, rtol=1.3e-6, atol=1e-5)
                    torch.testing.assert_close(gi.cpu(), ref_gi, **tol)
                    torch.testing.assert_close(inp.grad.cpu(), ref_inp.grad, **tol)
