"""The ATen-signature host layer (torch.ops.mi355x.*) on the GPU against PyTorch's CPU ATen ops:
shapes and dtypes of the saved tensors, output masks, empty inputs, non-contiguous inputs,
softmax over any dimension, out= forms, half_to_float, and the opt-in aten override with
autograd end to end.  Mirrors test/regressions/test_softmax.py:18-46,
test/regressions/test_rms_norm.py:52-160 and test/repro/test_layer_norm_group_norm_align.py:25-78
of the reference ("compute on CPU, compute on the device, compare")."""
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, gen

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_native_layer_norm_contract(ops, gpu, dtype):
    x = torch.randn(2, 3, 4, 5, generator=gen(1)).to(dtype)
    w = torch.randn(4, 5, generator=gen(2)).to(dtype)
    b = torch.randn(4, 5, generator=gen(3)).to(dtype)
    y, mean, rstd = ops.native_layer_norm(x.to(gpu), [4, 5], w.to(gpu), b.to(gpu), 1e-5)
    # statistics are float32 whatever the input dtype (LayerNorm.cpp:72-75 in the reference),
    # shaped input.shape[:axis] + [1] * k (:82-94)
    assert y.shape == x.shape and y.dtype == dtype and y.is_contiguous()
    assert mean.shape == (2, 3, 1, 1) and rstd.shape == (2, 3, 1, 1)
    assert mean.dtype == torch.float32 and rstd.dtype == torch.float32
    cy, cm, cr = torch.ops.aten.native_layer_norm(x.float(), [4, 5], w.float(), b.float(), 1e-5)
    assert_close(y, cy, dtype, "y")
    assert_close(mean, cm, dtype, "mean")
    assert_close(rstd, cr, dtype, "rstd")
    dy = torch.randn(2, 3, 4, 5, generator=gen(4)).to(dtype)
    dx, dg, db = ops.native_layer_norm_backward(dy.to(gpu), x.to(gpu), [4, 5], mean, rstd, w.to(gpu),
                                                b.to(gpu), [True, True, True])
    cdx, cdg, cdb = torch.ops.aten.native_layer_norm_backward(
        dy.float(), x.float(), [4, 5], cm, cr, w.float(), b.float(), [True, True, True])
    assert dx.shape == x.shape and dg.shape == (4, 5) and db.shape == (4, 5)
    assert dx.dtype == dtype and dg.dtype == dtype and db.dtype == dtype
    assert_close(dx, cdx, dtype, "dx")
    assert_close(dg, cdg, dtype, "dgamma")
    assert_close(db, cdb, dtype, "dbeta")
    # output masks: undefined tensors come back as None
    a, bb, c = ops.native_layer_norm_backward(dy.to(gpu), x.to(gpu), [4, 5], mean, rstd, w.to(gpu),
                                              b.to(gpu), [True, False, False])
    assert bb is None and c is None and torch.equal(a, dx)
    a, bb, c = ops.native_layer_norm_backward(dy.to(gpu), x.to(gpu), [4, 5], mean, rstd, w.to(gpu),
                                              b.to(gpu), [False, True, True])
    assert a is None and torch.equal(bb, dg) and torch.equal(c, db)


def test_layer_norm_mixed_precision_and_noncontiguous(ops, gpu):
    # bf16 rows with float32 gamma/beta: a CPU-ATen feature the reference's kernels lack
    x = torch.randn(33, 48, 96, generator=gen(5)).bfloat16()
    xt = x.transpose(0, 1)  # non-contiguous input
    w = torch.randn(96, generator=gen(6))
    b = torch.randn(96, generator=gen(7))
    y, mean, rstd = ops.native_layer_norm(xt.to(gpu), [96], w.to(gpu), b.to(gpu), 1e-5)
    cy, cm, cr = torch.ops.aten.native_layer_norm(xt.float(), [96], w, b, 1e-5)
    assert y.dtype == torch.bfloat16 and mean.shape == (48, 33, 1)
    assert_close(y, cy, torch.bfloat16, "y")
    dy = torch.randn(48, 33, 96, generator=gen(8)).bfloat16()
    dx, dg, db = ops.native_layer_norm_backward(dy.to(gpu), xt.to(gpu), [96], mean, rstd, w.to(gpu),
                                                b.to(gpu), [True, True, True])
    cdx, cdg, cdb = torch.ops.aten.native_layer_norm_backward(dy.float(), xt.float(), [96], cm, cr, w,
                                                              b, [True, True, True])
    assert dx.dtype == torch.bfloat16 and dg.dtype == torch.float32 and db.dtype == torch.float32
    assert_close(dx, cdx, torch.bfloat16, "dx")
    assert_close(dg, cdg, torch.bfloat16, "dgamma")
    assert_close(db, cdb, torch.bfloat16, "dbeta")


def test_empty_batches(ops, gpu):
    # LayerNorm.cpp:77,150-181 in the reference: M == 0 launches nothing; dgamma/dbeta are zeros
    x = torch.empty(0, 16, device=gpu)
    w = torch.ones(16, device=gpu)
    y, mean, rstd = ops.native_layer_norm(x, [16], w, w, 1e-5)
    assert y.shape == (0, 16) and mean.shape == (0, 1) and rstd.shape == (0, 1)
    dx, dg, db = ops.native_layer_norm_backward(x, x, [16], mean, rstd, w, w, [True, True, True])
    assert dx.shape == (0, 16) and bool((dg == 0).all()) and bool((db == 0).all())
    y, rstd = ops._fused_rms_norm(x, [16], w, None)
    assert y.shape == (0, 16) and rstd.shape == (0, 1)
    dx, dg = ops._fused_rms_norm_backward(x, x, [16], rstd, w, [True, True])
    assert dx.shape == (0, 16) and bool((dg == 0).all())
    assert ops._softmax(x, -1, False).shape == (0, 16)
    assert ops._softmax(torch.empty(4, 0, device=gpu), -1, False).shape == (4, 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_fused_rms_norm_contract(ops, gpu, dtype):
    x = torch.randn(2, 3, 4, 5, generator=gen(9)).to(dtype)
    w = torch.randn(4, 5, generator=gen(10)).to(dtype)
    for eps in (1e-6, None):
        y, rstd = ops._fused_rms_norm(x.to(gpu), [4, 5], w.to(gpu), eps)
        cy, crstd = torch.ops.aten._fused_rms_norm(x.float(), [4, 5], w.float(), eps)
        assert y.dtype == dtype and rstd.dtype == torch.float32 and rstd.shape == (2, 3, 1, 1)
        assert_close(y, cy, dtype, "y")
        assert_close(rstd, crstd, dtype, "rstd")
    # eps=None means FLT_EPSILON for every supported dtype (LayerNorm.cpp:218-224): closed form
    x32 = x.float()
    closed = x32 * torch.rsqrt(x32.pow(2).mean((-2, -1), keepdim=True) + torch.finfo(torch.float32).eps) * w.float()
    assert_close(y, closed, dtype, "y vs closed form")
    dy = torch.randn(2, 3, 4, 5, generator=gen(11)).to(dtype)
    dx, dg = ops._fused_rms_norm_backward(dy.to(gpu), x.to(gpu), [4, 5], rstd, w.to(gpu), [True, True])
    xr, wr = x.float().requires_grad_(), w.float().requires_grad_()
    F.rms_norm(xr, (4, 5), wr, torch.finfo(torch.float32).eps).backward(dy.float())
    assert_close(dx, xr.grad, dtype, "dx", scale=2.0)
    assert_close(dg, wr.grad, dtype, "dgamma", scale=2.0)
    a, b = ops._fused_rms_norm_backward(dy.to(gpu), x.to(gpu), [4, 5], rstd, w.to(gpu), [True, False])
    assert b is None and torch.equal(a, dx)


SOFTMAX_SHAPES = [(), (7,), (31, 23), (32, 1536), (33, 2049), (4, 5, 600), (2, 3, 4, 5)]


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES, ids=str)
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_softmax_every_dim(ops, gpu, shape, dtype):
    # test/regressions/test_softmax.py:18-46 and test/xpu/test_nn_xpu.py:14056-14106: every dim,
    # forward and backward, against the CPU
    x = (2 * torch.randn(shape, generator=gen(12))).to(dtype)
    g = torch.randn(shape, generator=gen(13)).to(dtype)
    for dim in range(-1, max(len(shape), 1) - 1):
        for is_log in (False, True):
            fwd = ops._log_softmax if is_log else ops._softmax
            bwd = ops._log_softmax_backward_data if is_log else ops._softmax_backward_data
            cfwd = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
            cbwd = (torch.ops.aten._log_softmax_backward_data if is_log
                    else torch.ops.aten._softmax_backward_data)
            y = fwd(x.to(gpu), dim, False)
            assert y.shape == x.shape and y.dtype == dtype
            cy = cfwd(x.float(), dim, False)
            assert_close(y, cy, dtype, "y dim=%d" % dim)
            gi = bwd(g.to(gpu), y, dim, dtype)
            cgi = cbwd(g.float(), y.cpu().float(), dim, torch.float32)
            assert gi.shape == x.shape and gi.dtype == dtype
            assert_close(gi, cgi, dtype, "grad_input dim=%d" % dim, scale=2.0)


def test_softmax_sliced_rows_and_out_variants(ops, gpu):
    # rows of a (1,1)-sliced tensor start at arbitrary alignments (test_nn_xpu.py:14071-14078)
    base = torch.randn(34, 2050, generator=gen(14))
    xs = base.to(gpu)[1:, 1:]
    y = ops._softmax(xs, 1, False)
    assert_close(y, torch.ops.aten._softmax(base[1:, 1:], 1, False), torch.float32, "sliced y")
    y0 = ops._softmax(xs, 0, False)
    assert_close(y0, torch.ops.aten._softmax(base[1:, 1:], 0, False), torch.float32, "sliced y dim 0")
    out = torch.empty(33, 2049, device=gpu)
    r = ops._softmax.out(xs, 1, False, out=out)
    assert r.data_ptr() == out.data_ptr() and torch.equal(out, y)
    g = torch.randn(33, 2049, generator=gen(15)).to(gpu)
    gi = ops._softmax_backward_data(g, y, 1, torch.float32)
    gout = torch.empty(33, 2049, device=gpu)
    ops._softmax_backward_data.out(g, y, 1, torch.float32, grad_input=gout)
    assert torch.equal(gi, gout)
    lout = torch.empty(33, 2049, device=gpu)
    ops._log_softmax.out(xs, 1, False, out=lout)
    assert torch.equal(lout, ops._log_softmax(xs, 1, False))


def test_softmax_half_to_float(ops, gpu):
    # test/xpu/test_nn_xpu.py:15036-15047: softmax(half, dtype=float) == softmax(float(half))
    x = torch.randn(32, 100, generator=gen(16)).half().to(gpu)
    y = ops._softmax(x, -1, True)
    assert y.dtype == torch.float32
    assert_close(y, ops._softmax(x.float(), -1, False), torch.float32, "half_to_float y")
    g = torch.randn(32, 100, generator=gen(17)).to(gpu)
    gi = ops._softmax_backward_data(g, y, -1, torch.float16)
    assert gi.dtype == torch.float16
    assert_close(gi, ops._softmax_backward_data(g, y, -1, torch.float32), torch.float16, "grad_input")
    with pytest.raises(RuntimeError, match="Half type only"):
        ops._softmax(x.bfloat16(), -1, True)


def test_unsupported_dtype_is_an_error_not_a_fallback(ops, gpu):
    x = torch.randint(0, 5, (4, 8), dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError, match="not implemented by the MI355X kernels"):
        ops._softmax(x, -1, False)
    xc = torch.randn(4, 8, dtype=torch.complex64, device=gpu)
    with pytest.raises(RuntimeError, match="not implemented by the MI355X kernels"):
        ops._softmax(xc, -1, False)


def test_zero_width_rows_have_defined_statistics(ops, gpu):
    """M > 0 rows of no elements: nothing is launched, and the saved statistics are what the CPU
    kernel's formulas give on an empty row (mean 0, rstd NaN), not uninitialised memory."""
    x = torch.empty(3, 0, device=gpu)
    y, mean, rstd = ops.native_layer_norm(x, [0], None, None, 1e-5)
    cy, cm, cr = torch.ops.aten.native_layer_norm(x.cpu(), [0], None, None, 1e-5)
    assert y.shape == (3, 0) and mean.shape == cm.shape and rstd.shape == cr.shape
    assert torch.equal(mean.cpu(), cm) and bool(torch.isnan(rstd).all()) and bool(torch.isnan(cr).all())
    y, rstd = ops._fused_rms_norm(x, [0], None, 1e-5)
    _, cr = torch.ops.aten._fused_rms_norm(x.cpu(), [0], None, 1e-5)
    assert y.shape == (3, 0) and rstd.shape == cr.shape
    assert bool(torch.isnan(rstd).all()) and bool(torch.isnan(cr).all())
    xg = torch.empty(2, 4, 0, device=gpu)
    y, mean, rstd = ops.native_group_norm(xg, None, None, 2, 4, 0, 2, 1e-5)
    _, cm, cr = torch.ops.aten.native_group_norm(xg.cpu(), None, None, 2, 4, 0, 2, 1e-5)
    assert y.shape == (2, 4, 0) and mean.shape == (2, 2)
    assert torch.equal(mean.cpu(), cm) and bool(torch.isnan(rstd).all()) and bool(torch.isnan(cr).all())


def test_float64_is_delegated_to_the_stock_kernels(pkg, ops, gpu):
    """The kernels accumulate in float32 and do not take float64; the reference computes float64
    in double (sycl/LayerNormKernels.cpp:1418-1438, sycl/SoftMaxKernels.cpp:2125-2178).  The host
    layer hands float64 GPU tensors to the kernels PyTorch-ROCm ships (the idea of
    src/ATen/native/xpu/XPUFallback.cpp:59-69), so that after the aten override everything that
    worked before still works and gives the same bits."""
    import warnings
    g = gen(60)
    x = torch.randn(6, 5, 64, generator=g, dtype=torch.float64).to(gpu)
    w = torch.randn(64, generator=g, dtype=torch.float64).to(gpu)
    b = torch.randn(64, generator=g, dtype=torch.float64).to(gpu)
    dy = torch.randn(6, 5, 64, generator=g, dtype=torch.float64).to(gpu)
    xn = torch.randn(4, 8, 6, 6, generator=g, dtype=torch.float64).to(gpu)
    wn = torch.randn(8, generator=g, dtype=torch.float64).to(gpu)
    mask = (torch.rand(6, 5, 64, generator=g) < 0.3).to(gpu)

    def everything():
        out = []
        for fn in (lambda t: F.layer_norm(t, (64,), w, b, 1e-5),
                   lambda t: F.rms_norm(t, (64,), w, 1e-6),
                   lambda t: F.softmax(t, -1), lambda t: F.softmax(t, 1),
                   lambda t: F.log_softmax(t, -1), lambda t: F.log_softmax(t, 0),
                   lambda t: torch._masked_softmax(t, mask, -1, 2),
                   lambda t: torch.ops.aten._safe_softmax(t, -1)):
            xs = x.detach().clone().requires_grad_()
            y = fn(xs)
            y.backward(dy)
            out += [y.detach(), xs.grad]
        xs = xn.detach().clone().requires_grad_()
        y = F.group_norm(xs, 2, wn, wn, 1e-5)
        y.backward(torch.ones_like(y))
        out += [y.detach(), xs.grad]
        o = torch.empty_like(x)
        torch.softmax(x, -1, out=o)
        out.append(o)
        return out

    pkg.restore_aten_ops()
    stock = everything()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
        ours = everything()
    assert len(stock) == len(ours)
    for a, r in zip(ours, stock):
        assert a.dtype == torch.float64 and torch.equal(a, r)
    # and the operators called directly
    y, mean, rstd = ops.native_layer_norm(x, [64], w, b, 1e-5)
    sy, sm, sr = torch.ops.aten.native_layer_norm.default(x, [64], w, b, 1e-5)
    assert y.dtype == torch.float64 and torch.equal(y, sy) and torch.equal(rstd, sr)
    ref = F.layer_norm(x.cpu(), (64,), w.cpu(), b.cpu(), 1e-5)
    assert float((y.cpu() - ref).abs().max()) < 1e-12  # float64 accuracy, not float32
    # restore really restores: float32 goes back to the stock kernels, and forth again
    x32 = x.float()
    over = F.softmax(x32, -1)
    pkg.restore_aten_ops()
    stock32 = F.softmax(x32, -1)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    assert torch.equal(F.softmax(x32, -1), over)
    assert_close(over, stock32, torch.float32, "override vs stock softmax")


def test_aten_override_runs_autograd_end_to_end(pkg, gpu):
    """Explicit opt-in routing of the aten ops to these kernels: F.layer_norm / F.rms_norm /
    F.softmax / F.log_softmax with autograd on the GPU against the same on the CPU."""
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.randn(6, 40, 256, generator=gen(20)).to(dtype)
        w = torch.randn(256, generator=gen(21)).to(dtype)
        b = torch.randn(256, generator=gen(22)).to(dtype)
        dy = torch.randn(6, 40, 256, generator=gen(23)).to(dtype)
        # one op at a time (a chain of bfloat16 ops rounds between the ops, which a float32
        # reference chain does not), plus the whole chain in float32
        stages = {
            "layer_norm": lambda xs, ws, bs: F.layer_norm(xs, (256,), ws, bs, 1e-5),
            "rms_norm": lambda xs, ws, bs: F.rms_norm(xs, (256,), ws, 1e-6),
            "softmax": lambda xs, ws, bs: F.softmax(xs, -1),
            "log_softmax": lambda xs, ws, bs: F.log_softmax(xs, -1),
        }
        if dtype == torch.float32:
            stages["chain"] = lambda xs, ws, bs: (
                F.softmax(F.rms_norm(F.layer_norm(xs, (256,), ws, bs, 1e-5), (256,), ws, 1e-6), -1)
                + F.log_softmax(F.layer_norm(xs, (256,), ws, bs, 1e-5), -1))

        for name, fn in stages.items():
            def run(dev, upcast):
                cast = (lambda t: t.float()) if upcast else (lambda t: t)
                xs, ws, bs = (cast(t).detach().clone().to(dev).requires_grad_() for t in (x, w, b))
                out = fn(xs, ws, bs)
                out.backward(cast(dy).to(dev))
                return out, xs.grad, ws.grad, bs.grad

            got = run(gpu, False)
            ref = run("cpu", True)
            for a, r, nm in zip(got, ref, ("out", "dx", "dw", "db")):
                if r is None:  # a stage that does not use this parameter
                    assert a is None
                    continue
                assert a is not None, "%s: %s is missing on the GPU" % (name, nm)
                assert a.dtype == dtype
                assert_close(a, r, dtype, "%s %s" % (name, nm), scale=4.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_aten_override_routes_the_out_overloads(pkg, cabi, gpu, dtype):
    """The reference's softmax ops are structured `.out` kernels (src/ATen/native/xpu/SoftMax.cpp:
    22-100).  After the opt-in, torch.softmax(x, dim, out=o) / torch.log_softmax(..., out=o) and
    the backward `.out` forms run the MI355X kernels: bit-equal to the C ABI called directly.  The
    stock kernels' results differ from these in the last bits on this input, which is how the test
    knows the call was routed."""
    import warnings
    x = (3 * torch.randn(64, 3000, generator=gen(30))).to(dtype).to(gpu)
    g = torch.randn(64, 3000, generator=gen(31)).to(dtype).to(gpu)
    pkg.restore_aten_ops()
    stock = torch.empty_like(x)
    torch.log_softmax(x, -1, out=stock)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    try:
        for is_log, fn, bwd in ((False, torch.softmax, torch.ops.aten._softmax_backward_data),
                                (True, torch.log_softmax, torch.ops.aten._log_softmax_backward_data)):
            want = cabi.softmax_fwd(x, is_log)
            o = torch.full_like(x, 7.0)
            r = fn(x, -1, out=o)
            assert r.data_ptr() == o.data_ptr() and torch.equal(o, want)
            want_gi = cabi.softmax_bwd(g, want, is_log)
            gi = torch.full_like(x, 7.0)
            kw = {"out": gi} if is_log else {"grad_input": gi}
            bwd.out(g, want, -1, dtype, **kw)
            assert torch.equal(gi, want_gi)
            # over a non-innermost dimension too
            o0 = torch.empty_like(x)
            fn(x, 0, out=o0)
            assert torch.equal(o0, getattr(pkg.ops, "_log_softmax" if is_log else "_softmax")(x, 0, False))
        mine = torch.empty_like(x)
        torch.log_softmax(x, -1, out=mine)
        assert_close(mine, stock, dtype, "routed vs stock log_softmax")
    finally:
        pkg.restore_aten_ops()
    again = torch.empty_like(x)
    torch.log_softmax(x, -1, out=again)
    assert torch.equal(again, stock)  # the stock kernel is back


def test_aten_override_masked_and_safe_softmax_autograd(pkg, gpu):
    """torch._masked_softmax / torch._safe_softmax on GPU tensors after the opt-in, forward and
    through autograd, against the CPU: the sizes, dims and mask types of
    test/xpu/test_nn_xpu.py:13744-13965 (test_masked_softmax_mask_types, _lowp, _grad) and
    test/regressions/test_safe_softmax.py:18-52 in the reference."""
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    g = gen(50)
    for (B, H, L) in ((1, 1, 32), (3, 4, 310), (2, 2, 1200)):
        src = torch.randint(0, 2, (L, L), generator=g).bool()
        pad = torch.randint(0, 2, (B, L), generator=g).bool()
        generic = torch.randint(0, 2, (B, H, L, L), generator=g).bool()
        expanded = {0: src.reshape(1, 1, L, L).expand(B, H, L, L),
                    1: pad.reshape(B, 1, 1, L).expand(B, H, L, L), 2: generic}
        for dtype in (torch.float32, torch.bfloat16):
            x = torch.randn(B, H, L, L, generator=g).to(dtype)
            dy = torch.randn(B, H, L, L, generator=g).to(dtype)
            for dim in (0, 3):
                for mask, mtype in ((src, 0), (pad, 1), (generic, 2)):
                    print("case override masked", (B, H, L), dtype, dim, mtype, flush=True)
                    dead = expanded[mtype].all(dim, keepdim=True).expand(B, H, L, L)
                    # forward with the mask in its own layout
                    out = torch._masked_softmax(x.to(gpu), mask.to(gpu), dim, mtype)
                    ref = torch._masked_softmax(x.float(), mask, dim, mtype)
                    assert out.dtype == dtype
                    # fully masked slices are unspecified in the reference's tests (NaN or 0)
                    assert_close(out.cpu().masked_fill(dead, 0), ref.masked_fill(dead, 0), dtype,
                                 "masked out")
                    if mtype == 0:
                        continue
                    # autograd hands the forward's mask to _masked_softmax_backward, which wants
                    # it in the gradient's shape: expanded masks, as test_masked_softmax_lowp uses
                    full = expanded[mtype]
                    xs = x.detach().clone().to(gpu).requires_grad_()
                    out = torch._masked_softmax(xs, full.to(gpu), dim, mtype)
                    out.backward(dy.to(gpu))
                    xr = x.float().detach().clone().requires_grad_()
                    torch._masked_softmax(xr, full, dim, mtype).backward(dy.float())
                    assert xs.grad.dtype == dtype
                    assert_close(out.detach().cpu().masked_fill(dead, 0), ref.masked_fill(dead, 0),
                                 dtype, "masked out (expanded mask)")
                    assert_close(xs.grad.cpu().masked_fill(dead, 0), xr.grad.masked_fill(dead, 0), dtype,
                                 "masked dx", scale=2.0)
                    assert bool((xs.grad.cpu()[full & ~dead] == 0).all())
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        x = torch.randn(32, 48, 64, generator=g).to(dtype)
        dy = torch.randn(32, 48, 64, generator=g).to(dtype)
        for dim, sl in ((-1, (0, 0, slice(None))), (1, (0, slice(None), 0)), (0, (slice(None), 0, 0))):
            for poison in (False, True):
                xc = x.clone()
                if poison:
                    xc[sl] = float("-inf")
                xs = xc.detach().clone().to(gpu).requires_grad_()
                out = torch.ops.aten._safe_softmax(xs, dim)
                out.backward(dy.to(gpu))
                xr = xc.float().detach().clone().requires_grad_()
                ref = torch.ops.aten._safe_softmax(xr, dim)
                ref.backward(dy.float())
                assert_close(out, ref, dtype, "safe out dim=%d" % dim)
                assert_close(xs.grad, xr.grad, dtype, "safe dx dim=%d" % dim, scale=2.0)
                if poison:
                    assert bool((out.detach()[sl] == 0).all())
