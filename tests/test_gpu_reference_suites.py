"""The reference's own device-vs-CPU and closed-form tests for this path, run against these
kernels through the opt-in aten override (nn.LayerNorm / F.rms_norm / F.softmax on GPU tensors,
autograd included), with the reference's sizes and tolerances.  The two big suites:

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


# ---------------------------------------------------------------------------------------------
# The smaller tests of test/xpu/test_nn_xpu.py that pin this path, with the reference's shapes
# and tolerances (assertEqual's defaults are torch.testing.assert_close's).

def test_layer_norm_numeric(overridden, gpu):
    """test_nn_xpu.py:11544-11572: closed form on [2, 256, 256, 144] normalized over the last
    three dimensions (rows of 9.4 M elements: the multi-pass kernel), atol 1e-5."""
    shape = [256, 256, 144]
    ln = nn.LayerNorm(shape).float().to(gpu)
    x = torch.rand(2, *shape, generator=gen(91)).to(gpu)
    y = ln(x)
    xv = x.view(2, -1)
    ref = ((xv - xv.mean(-1, keepdim=True)) / torch.sqrt(xv.var(-1, unbiased=False, keepdim=True) + ln.eps))
    ref = (ref * ln.weight.view(-1) + ln.bias.view(-1)).view_as(x)
    torch.testing.assert_close(y, ref, rtol=0, atol=1e-5)
    torch.testing.assert_close(y.cpu(), ln.cpu()(x.cpu()), rtol=0, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_layer_norm_general(overridden, gpu, dtype):
    """test_nn_xpu.py:10602-10644: output mean 0 / variance 1, weight and bias applied, bad
    normalized shapes rejected."""
    g = gen(92)
    delta = 1e-1 if dtype != torch.float32 else 1e-5
    for i in range(2, 6):
        shape = torch.randint(3, 6, (i,), generator=g).tolist()
        x = (torch.rand(*shape, generator=g) * 10).to(gpu, dtype)
        nd = int(torch.randint(1, i, (1,), generator=g))
        lead = shape[:-nd]
        ln = nn.LayerNorm(shape[-nd:], eps=0).to(gpu, dtype)
        out = ln(x).detach().float().view(*(lead + [-1]))
        assert abs(float(out.mean(-1).abs().mean())) <= delta
        assert abs(float(out.var(-1, unbiased=False).abs().mean()) - 1) <= delta
        scale, bias = (0.2 + 1.8 * torch.rand(2, generator=g)).tolist()
        ln.weight.data.fill_(scale)
        ln.bias.data.fill_(bias)
        out = ln(x).detach().float().view(*(lead + [-1]))
        assert abs(float(out.mean(-1).abs().mean()) - bias) <= delta
        assert abs(float(out.var(-1, unbiased=False).abs().mean()) - scale ** 2) <= delta * max(1.0, scale ** 2)
    for norm_shape, input_shape in (((), ()), ((2, 3), (3,)), ((2,), (1, 2, 3)), ((10,), (2, 3)), (10, (2, 3))):
        ln = nn.LayerNorm(norm_shape).to(gpu, dtype)
        with pytest.raises(RuntimeError):
            ln(torch.rand(input_shape).to(gpu, dtype))


def test_layer_norm_eps_constant_rows(overridden, gpu):
    """test_nn_xpu.py:9657-9661: constant rows without affine parameters come out as zeros."""
    x = torch.tensor([[[2.0, 2.0], [14.0, 14.0]], [[2.0, 2.0], [14.0, 14.0]]], device=gpu)
    ln = nn.LayerNorm(2, eps=1e-6, elementwise_affine=False)
    assert torch.equal(ln(x), torch.zeros_like(x))


def test_layernorm_half_precision_and_weight_bias(overridden, gpu):
    """test_nn_xpu.py:15076-15104: the fp16 result is the fp32 result rounded, bit for bit; an
    absent weight is ones, an absent bias zeros."""
    width = 128
    g = gen(93)
    x = (torch.rand(1, 5, width, generator=g) * 0.1).half().to(gpu)
    w = torch.ones(width, device=gpu, dtype=torch.half)
    b = torch.zeros(width, device=gpu, dtype=torch.half)
    y16 = torch.layer_norm(x, (width,), w, b, 1e-5)
    y32 = torch.layer_norm(x.float(), (width,), w.float(), b.float(), 1e-5).half()
    torch.testing.assert_close(y16, y32, rtol=0, atol=0)
    x = (torch.rand(1, 5, width, generator=g) * 0.1).to(gpu)
    data = torch.randn(width, generator=g).to(gpu)
    ones, zeros = torch.ones(width, device=gpu), torch.zeros(width, device=gpu)
    assert torch.equal(torch.layer_norm(x, (width,), None, data, 1e-5),
                       torch.layer_norm(x, (width,), ones, data, 1e-5))
    assert torch.equal(torch.layer_norm(x, (width,), data, None, 1e-5),
                       torch.layer_norm(x, (width,), data, zeros, 1e-5))


def _rms_ref(x, shape, weight=None, eps=None):
    eps = torch.finfo(x.dtype).eps if eps is None else eps
    dims = [x.ndim - i - 1 for i in range(len(shape))]
    up = x.float()
    r = up * torch.rsqrt(up.pow(2).mean(dim=dims, keepdim=True) + eps)
    if weight is not None:
        r = r * weight
    return r.type_as(x)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
def test_rmsnorm_numeric_and_epsilon(overridden, gpu, dtype):
    """test_nn_xpu.py:11575-11621: closed form in fp32 then cast; the default eps is the input
    dtype's machine epsilon (inputs of +-1e-12)."""
    g = gen(94)
    if dtype != torch.float32:
        shape = (1, 2, 3)
        x = torch.rand(*shape, generator=g).to(gpu, dtype)
        w = torch.rand(*shape, generator=g).to(gpu, dtype)
        torch.testing.assert_close(F.rms_norm(x, shape, w, 0.5), _rms_ref(x, shape, w, 0.5))
    x = torch.tensor([[1e-12, -1e-12], [1e-12, -1e-12]], dtype=dtype, device=gpu)
    torch.testing.assert_close(F.rms_norm(x, (2, 2)), _rms_ref(x, (2, 2)))


def test_log_softmax_sums_to_one_and_backward(overridden, gpu):
    """test_nn_xpu.py:14141-14159 (test_softmax_double, in fp32: the kernels take no float64)."""
    g = gen(95)
    logits = torch.randn(5, 513, generator=g).to(gpu)
    ones = F.log_softmax(logits, dim=1).exp().sum(dim=1)
    torch.testing.assert_close(ones, torch.ones_like(ones))
    logits.requires_grad_()
    out = F.log_softmax(logits, dim=1)
    grad = torch.randn(5, 513, generator=g).to(gpu)
    out.backward(grad)
    lc = logits.detach().cpu().requires_grad_()
    F.log_softmax(lc, dim=1).backward(grad.cpu())
    torch.testing.assert_close(logits.grad.cpu(), lc.grad)


def test_log_softmax_big(overridden, gpu):
    """test_nn_xpu.py:14177-14190: log_softmax of half values and of the same values + 1.5e3
    (exactly representable) are equal."""
    g = gen(96)
    for shape in ((16, 4), (4, 1536)):
        small = torch.randint(100, shape, generator=g).half().to(gpu)
        big = small + 1.5e3
        torch.testing.assert_close(F.log_softmax(small, -1), F.log_softmax(big, -1))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=str)
def test_softmax_backward_data_aligned_and_unaligned(overridden, gpu, dtype):
    """test_nn_xpu.py:17922-17998: _softmax_backward_data on 2048 and 2049 elements and on
    operands that start one element into a buffer, against the CPU."""
    g = gen(97)

    def check(grad_output, output):
        r = torch._softmax_backward_data(grad_output, output, 0, output.dtype)
        e = torch._softmax_backward_data(grad_output.cpu(), output.cpu(), 0, dtype)
        torch.testing.assert_close(r.cpu(), e)

    def unaligned(t):
        buf = torch.ones(t.numel() + 1, device=gpu, dtype=dtype)
        v = buf[1:]
        v.copy_(t)
        assert v.data_ptr() % 16 != 0
        return v

    check(torch.rand(2048, generator=g).to(gpu, dtype), torch.rand(2048, generator=g).to(gpu, dtype))
    check((torch.rand(2049, generator=g) / 2049).to(gpu, dtype), torch.rand(2049, generator=g).to(gpu, dtype))
    check((torch.rand(2048, generator=g) / 2048).to(gpu, dtype), unaligned(torch.ones(2048)))
    check(unaligned(torch.ones(2048) / 2048), torch.rand(2048, generator=g).to(gpu, dtype))


def test_softmax_bfloat16(overridden, gpu):
    """test_nn_xpu.py:15824-15841: bf16 softmax over every dim of [16, 33, 15, 16] against fp32,
    to 1e-2, and to 0.05 with inputs scaled by 1000 (exp must not overflow); forward and the
    gradient of the input."""
    g = gen(98)
    for dim in range(4):
        for prec, scale in ((1e-2, 1.0), (0.05, 1000.0)):
            x1 = (torch.randn(16, 33, 15, 16, generator=g) * scale).to(gpu).requires_grad_()
            x2 = x1.detach().bfloat16().requires_grad_()
            go1 = torch.randn(16, 33, 15, 16, generator=g).to(gpu)
            o1 = torch.softmax(x1, dim)
            o2 = torch.softmax(x2, dim)
            o1.backward(go1)
            o2.backward(go1.bfloat16())
            assert o2.dtype == torch.bfloat16 and x2.grad.dtype == torch.bfloat16
            torch.testing.assert_close(o2.float(), torch.softmax(x2.detach().float(), dim), atol=prec, rtol=prec)
            if scale == 1.0:
                torch.testing.assert_close(o1, o2.float(), atol=prec, rtol=0)
            xr = x2.detach().float().requires_grad_()
            torch.softmax(xr, dim).backward(go1.bfloat16().float())
            torch.testing.assert_close(x2.grad.float(), xr.grad, atol=prec, rtol=prec)
