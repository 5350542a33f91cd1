"""The five benchmark configurations at their full sizes, HIP kernels (through the C ABI) against
PyTorch's CPU ATen ops and the CPU oracle on the same seeded inputs.

Inputs follow the stated recipe: torch.Generator().manual_seed(1234 + cfg), made on the CPU in
float32, cast, copied to the GPU.  Tolerances (helpers.TOL): float32 rtol = atol = 1e-5;
bfloat16/float16 atol 1e-2, rtol 1.6e-2 against a reference accumulated in float32 or better
(the CPU op evaluated on float32-upcast inputs, and the float64 oracle), saved mean/rstd included.
"""
import pytest
import torch

from helpers import (abs_err, assert_close, colsum_slack, gen, offset_view, rowsum_slack,
                     stress_rows, to_np32)

pytestmark = pytest.mark.gpu


def test_config1_layer_norm_fwd_fp32(cabi, oracle, gpu):
    M, N = 4096, 1024
    g = gen(1234 + 1)
    x = torch.randn(M, N, generator=g)
    gamma = 1 + 0.1 * torch.randn(N, generator=g)
    beta = 0.1 * torch.randn(N, generator=g)
    y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-5)
    cy, cm, cr = torch.ops.aten.native_layer_norm(x, [N], gamma, beta, 1e-5)
    assert_close(y, cy, torch.float32, "y vs ATen CPU")
    assert_close(mean, cm.reshape(-1), torch.float32, "mean vs ATen CPU")
    assert_close(rstd, cr.reshape(-1), torch.float32, "rstd vs ATen CPU")
    oy, om, orr = oracle.layer_norm_fwd(x.numpy(), (N,), gamma.numpy(), beta.numpy(), 1e-5)
    assert_close(y, oy, torch.float32, "y vs oracle")
    assert_close(mean, om.reshape(-1), torch.float32, "mean vs oracle")
    assert_close(rstd, orr.reshape(-1), torch.float32, "rstd vs oracle")


def test_config2_rms_norm_fwd_bwd_bf16(cabi, oracle, gpu):
    M, N, eps = 16384, 4096, 1e-6
    g = gen(1234 + 2)
    x = torch.randn(M, N, generator=g).bfloat16()
    w = (1 + 0.02 * torch.randn(N, generator=g)).bfloat16()
    dy = torch.randn(M, N, generator=g).bfloat16()
    xg, wg, dyg = x.to(gpu), w.to(gpu), dy.to(gpu)
    y, rstd = cabi.rms_norm_fwd(xg, wg, eps)
    dx, dw = cabi.rms_norm_bwd(dyg, xg, rstd, wg)
    assert y.dtype == torch.bfloat16 and rstd.dtype == torch.float32
    assert dx.dtype == torch.bfloat16 and dw.dtype == torch.bfloat16
    # CPU ATen on float32-upcast inputs (forward op; backward by autograd: no CPU backward kernel)
    xr, wr = x.float().requires_grad_(), w.float().requires_grad_()
    cy, crstd = torch.ops.aten._fused_rms_norm(xr, [N], wr, eps)
    cy.backward(dy.float())
    assert_close(y, cy, torch.bfloat16, "y vs ATen CPU")
    assert_close(rstd, crstd.reshape(-1), torch.bfloat16, "rstd vs ATen CPU")
    assert_close(dx, xr.grad, torch.bfloat16, "dx vs ATen CPU")
    assert_close(dw, wr.grad, torch.bfloat16, "dweight vs ATen CPU")
    # float64 oracle from the device's own saved rstd
    oy, orstd = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(w), eps)
    odx, odw = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rstd), to_np32(w))
    assert_close(y, oy, torch.bfloat16, "y vs oracle")
    assert_close(rstd, orstd.reshape(-1), torch.float32, "rstd vs oracle (fp32 bar)")
    assert_close(dx, odx, torch.bfloat16, "dx vs oracle")
    assert_close(dw, odw, torch.bfloat16, "dweight vs oracle")
    # closed form of the reference's own regression test (test/regressions/test_rms_norm.py:82-83)
    closed = (dy.float() * x.float() * crstd.detach()).sum(0)
    assert_close(dw, closed, torch.bfloat16, "dweight vs sum(dY * x * rstd)")
    # run-to-run determinism of the two-stage column reduction
    dx2, dw2 = cabi.rms_norm_bwd(dyg, xg, rstd, wg)
    assert torch.equal(dw, dw2) and torch.equal(dx, dx2)


def test_config3_softmax_log_softmax_fwd_bwd_bf16_causal(cabi, oracle, gpu):
    B, H, T = 4, 32, 2048
    s = torch.empty(B, H, T, T, dtype=torch.bfloat16, device=gpu)
    grad = torch.empty(B, H, T, T, dtype=torch.bfloat16, device=gpu)
    g = gen(1234 + 3)
    tri = torch.triu(torch.ones(T, T), 1).bool()
    host = {}
    for b in range(B):
        sb = 3.0 * torch.randn(H, T, T, generator=g)
        sb.masked_fill_(tri, float("-inf"))
        gb = torch.randn(H, T, T, generator=g)
        s[b].copy_(sb.bfloat16())
        grad[b].copy_(gb.bfloat16())
        if b in (0, B - 1):  # parity per [32, 2048, 2048] slice bounds host memory
            host[b] = (sb.bfloat16(), gb.bfloat16())
    del sb, gb
    trig = tri.to(gpu)
    for is_log in (False, True):
        name = "log_softmax" if is_log else "softmax"
        y = cabi.softmax_fwd(s, is_log)
        gi = cabi.softmax_bwd(grad, y, is_log)
        # size-independent properties on the full tensor
        if is_log:
            assert bool(torch.isneginf(y[..., trig]).all())
            rowsum = torch.exp(y.float()).sum(-1)
        else:
            assert bool((y[..., trig] == 0).all())
            rowsum = y.float().sum(-1)
            # softmax backward rows sum to zero (up to the bf16 rounding of T outputs)
            assert float(gi.float().sum(-1).abs().max()) < 0.05
        assert float((rowsum - 1).abs().max()) < 2e-2, name + ": rows must sum to one"
        assert bool(torch.isfinite(gi).all())
        fwd = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
        bwd = (torch.ops.aten._log_softmax_backward_data if is_log
               else torch.ops.aten._softmax_backward_data)
        for b, (sb, gb) in host.items():
            cy = fwd(sb.float(), -1, False)
            assert_close(y[b], cy, torch.bfloat16, "%s y[%d] vs ATen CPU" % (name, b))
            yb = y[b].cpu()
            cgi = bwd(gb.float(), yb.float(), -1, torch.float32)
            assert_close(gi[b], cgi, torch.bfloat16, "%s grad_input[%d] vs ATen CPU" % (name, b))
        # float64 oracle on four heads of the first slice
        sb, gb = host[0]
        oy = oracle.softmax_fwd(to_np32(sb[:4]), is_log)
        assert_close(y[0, :4], oy, torch.bfloat16, name + " y vs oracle")
        ogi = oracle.softmax_bwd(to_np32(gb[:4]), to_np32(y[0, :4]), is_log)
        assert_close(gi[0, :4], ogi, torch.bfloat16, name + " grad_input vs oracle")
        del y, gi


def test_config4_layer_norm_fwd_bwd_bf16_fp32_weights(cabi, oracle, gpu):
    M, N, eps = 16384, 8192, 1e-5
    g = gen(1234 + 4)
    x = torch.randn(M, N, generator=g).bfloat16()
    gamma = 1 + 0.1 * torch.randn(N, generator=g)
    beta = 0.1 * torch.randn(N, generator=g)
    dy = torch.randn(M, N, generator=g).bfloat16()
    xg, dyg, gg, bg = x.to(gpu), dy.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, eps)
    dx, dgm, dbt = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
    assert y.dtype == torch.bfloat16 and dx.dtype == torch.bfloat16
    assert mean.dtype == rstd.dtype == dgm.dtype == dbt.dtype == torch.float32
    # fp32-accumulated reference: the CPU op on float32-upcast inputs
    x32, dy32 = x.float(), dy.float()
    cy, cm, cr = torch.ops.aten.native_layer_norm(x32, [N], gamma, beta, eps)
    cdx, cdg, cdb = torch.ops.aten.native_layer_norm_backward(dy32, x32, [N], cm, cr, gamma, beta,
                                                              [True, True, True])
    assert_close(y, cy, torch.bfloat16, "y vs ATen CPU")
    assert_close(mean, cm.reshape(-1), torch.bfloat16, "mean vs ATen CPU")
    assert_close(rstd, cr.reshape(-1), torch.bfloat16, "rstd vs ATen CPU")
    assert_close(dx, cdx, torch.bfloat16, "dx vs ATen CPU")
    assert_close(dgm, cdg, torch.bfloat16, "dgamma vs ATen CPU")
    assert_close(dbt, cdb, torch.bfloat16, "dbeta vs ATen CPU")
    # the saved statistics and the column sums are float32 results: hold them to the fp32 bar
    # against the float64 oracle (column reduction over all 16384 rows)
    _, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, eps)
    assert_close(mean, om.reshape(-1), torch.float32, "mean vs oracle (fp32 bar)")
    assert_close(rstd, orr.reshape(-1), torch.float32, "rstd vs oracle (fp32 bar)")
    _, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean), to_np32(rstd),
                                        to_np32(gamma), mask=(False, True, True))
    xhat = (x32 - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
    assert_close(dgm, odg, torch.float32, "dgamma vs oracle (fp32 bar)", slack=colsum_slack(dy32 * xhat))
    assert_close(dbt, odb, torch.float32, "dbeta vs oracle (fp32 bar)", slack=colsum_slack(dy32))
    del xhat
    rows = slice(0, 512)
    oy, _, _ = oracle.layer_norm_fwd(to_np32(x[rows]), (N,), to_np32(gamma), to_np32(beta), eps)
    assert_close(y[rows], oy, torch.bfloat16, "y vs oracle")
    odx, _, _ = oracle.layer_norm_bwd(to_np32(dy[rows]), to_np32(x[rows]), (N,), to_np32(mean[rows]),
                                      to_np32(rstd[rows]), to_np32(gamma), mask=(True, False, False))
    assert_close(dx[rows], odx, torch.bfloat16, "dx vs oracle")
    # dbeta of a sum() loss is the row count (test/regressions/test_rms_norm.py:152-160)
    _, _, db1 = cabi.layer_norm_bwd(torch.ones_like(dyg), xg, mean, rstd, gg, want=(False, True, True))
    assert bool((db1 == float(M)).all())


STRESS = [(1 << 20, 64), (8192, 127), (8192, 4097), (8192, 5120), (8192, 16384)]
ORACLE_ROWS = None  # every row is checked against the float64 oracle (row 0 is the constant row)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
@pytest.mark.parametrize("shape", STRESS, ids=str)
def test_config5_stress_norms(cabi, oracle, gpu, dtype, shape):
    """LayerNorm and RMSNorm forward+backward on irregular shapes: 0.1% +-1e4 outliers, one
    constant row, every tensor 2 elements into its buffer (8-byte / 4-byte aligned only)."""
    M, N = shape
    print("case stress norms", dtype, shape, flush=True)
    x = stress_rows(M, N, 1234 + 5, dtype)
    g = gen(77)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
    xg, dyg = offset_view(x.to(gpu)), offset_view(dy.to(gpu))
    gg, bg = offset_view(gamma.to(gpu)), offset_view(beta.to(gpu))
    out = lambda like: offset_view(torch.empty_like(like))  # noqa: E731
    stat = lambda: offset_view(torch.empty(M, device=gpu))  # noqa: E731
    wout = lambda: offset_view(torch.empty(N, dtype=dtype, device=gpu))  # noqa: E731
    R = slice(0, ORACLE_ROWS)
    x32, dy32, g32, b32 = x.float(), dy.float(), gamma.float(), beta.float()
    # fp32: the CPU kernel sums rows holding +-1e4 in float32; the comparison against it carries
    # that kernel's own measured distance from the float64 oracle, element by element, as slack
    # (every row has an oracle value).  16-bit results are compared at the stated tolerance.
    own = (lambda cpu, exact: abs_err(cpu, exact)) if dtype == torch.float32 else (lambda cpu, exact: None)

    # ---- LayerNorm
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5, y=out(xg), mean=stat(), rstd=stat())
    cy, cm, cr = torch.ops.aten.native_layer_norm(x32, [N], g32, b32, 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x[R]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y[R], oy, dtype, "LN y vs oracle")
    # the statistics of every row against the float64 closed form at the stated tolerance, and
    # against ATen CPU with that kernel's own distance from the closed form as slack
    x64 = x.double()
    m64 = x64.mean(1)
    r64 = 1.0 / torch.sqrt(x64.var(1, unbiased=False) + 1e-5)
    # a row that holds +1e4 and -1e4 has a mean near zero made of float32 partial sums near
    # 1e4: the mean gets four float32 roundings of the row's mean magnitude on top
    cancel = 4.0 * 2.0 ** -23 * x64.abs().mean(1)
    del x64
    assert_close(mean[R], om.reshape(-1), dtype, "LN mean vs oracle", slack=cancel[R])
    assert_close(rstd[R], orr.reshape(-1), dtype, "LN rstd vs oracle")
    assert_close(y, cy, dtype, "LN y vs ATen CPU", slack=own(cy, oy))
    assert_close(mean, m64, dtype, "LN mean vs float64", slack=cancel)
    assert_close(rstd, r64, dtype, "LN rstd vs float64")
    assert_close(mean, cm.reshape(-1), dtype, "LN mean vs ATen CPU",
                 slack=(cm.reshape(-1).double() - m64).abs() + cancel)
    assert_close(rstd, cr.reshape(-1), dtype, "LN rstd vs ATen CPU",
                 slack=(cr.reshape(-1).double() - r64).abs())
    # the constant row: mean exact, y == beta exactly (CPU ATen gives the same)
    assert float(mean[0]) == 1.5
    assert torch.equal(y[0].cpu(), beta) and torch.equal(cy[0].to(dtype), beta)
    dx, dgm, dbt = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, dx=out(xg), dgamma=wout(),
                                       dbeta=wout())
    odx, _, _ = oracle.layer_norm_bwd(to_np32(dy[R]), to_np32(x[R]), (N,), to_np32(mean[R]),
                                      to_np32(rstd[R]), to_np32(gamma), mask=(True, False, False))
    assert_close(dx[R], odx, dtype, "LN dx vs oracle")
    _, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean), to_np32(rstd),
                                        to_np32(gamma), mask=(False, True, True))
    # float32 column sums over all M rows: allow the summation's own rounding (helpers.colsum_slack)
    sl_g = sl_b = None
    if dtype == torch.float32:
        xhat = (x32 - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
        sl_g, sl_b = colsum_slack(dy32 * xhat), colsum_slack(dy32)
        del xhat
    assert_close(dgm, odg, dtype, "LN dgamma vs oracle", slack=sl_g)
    assert_close(dbt, odb, dtype, "LN dbeta vs oracle", slack=sl_b)
    cdx, cdg, cdb = torch.ops.aten.native_layer_norm_backward(
        dy32, x32, [N], mean.cpu().reshape(M, 1), rstd.cpu().reshape(M, 1), g32, b32,
        [True, True, True])
    assert_close(dx, cdx, dtype, "LN dx vs ATen CPU", slack=own(cdx, odx))
    assert_close(dgm, cdg, dtype, "LN dgamma vs ATen CPU",
                 slack=abs_err(cdg, odg) + sl_g if dtype == torch.float32 else None)
    assert_close(dbt, cdb, dtype, "LN dbeta vs ATen CPU",
                 slack=abs_err(cdb, odb) + sl_b if dtype == torch.float32 else None)
    del y, dx, cy, cdx

    # ---- RMSNorm
    y, rstd = cabi.rms_norm_fwd(xg, gg, 1e-6, y=out(xg), rstd=stat())
    oy, orr = oracle.rms_norm_fwd(to_np32(x[R]), (N,), to_np32(gamma), 1e-6)
    assert_close(y[R], oy, dtype, "RMS y vs oracle")
    assert_close(rstd[R], orr.reshape(-1), dtype, "RMS rstd vs oracle")
    cy, crs = torch.ops.aten._fused_rms_norm(x32, [N], g32, 1e-6)
    assert_close(y, cy, dtype, "RMS y vs ATen CPU", slack=own(cy, oy))
    assert_close(rstd, crs.reshape(-1), dtype, "RMS rstd vs ATen CPU",
                 slack=own(crs.reshape(-1), orr.reshape(-1)))
    dx, dgm = cabi.rms_norm_bwd(dyg, xg, rstd, gg, dx=out(xg), dgamma=wout())
    odx, _ = oracle.rms_norm_bwd(to_np32(dy[R]), to_np32(x[R]), (N,), to_np32(rstd[R]),
                                 to_np32(gamma), mask=(True, False))
    assert_close(dx[R], odx, dtype, "RMS dx vs oracle")
    _, odg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rstd), to_np32(gamma),
                                 mask=(False, True))
    sl_g = colsum_slack(dy32 * x32 * rstd.cpu().reshape(M, 1)) if dtype == torch.float32 else None
    assert_close(dgm, odg, dtype, "RMS dgamma vs oracle", slack=sl_g)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
@pytest.mark.parametrize("shape", STRESS, ids=str)
def test_config5_stress_softmax(cabi, oracle, gpu, dtype, shape):
    M, N = shape
    print("case stress softmax", dtype, shape, flush=True)
    x = stress_rows(M, N, 1234 + 5, dtype)
    grad = torch.randn(M, N, generator=gen(78)).to(dtype)
    xg, gg = offset_view(x.to(gpu)), offset_view(grad.to(gpu))
    R = slice(0, ORACLE_ROWS)
    x32, g32 = x.float(), grad.float()
    for is_log in (False, True):
        nm = "log_softmax" if is_log else "softmax"
        y = cabi.softmax_fwd(xg, is_log, y=offset_view(torch.empty_like(xg)))
        gi = cabi.softmax_bwd(gg, y, is_log, gi=offset_view(torch.empty_like(xg)))
        oy = oracle.softmax_fwd(to_np32(x[R]), is_log)
        assert_close(y[R], oy, dtype, nm + " y vs oracle")
        ogi = oracle.softmax_bwd(to_np32(grad[R]), to_np32(y[R]), is_log)
        # gi = g - exp(y) * sum(g)  /  y * (g - sum(y*g)): a float32 row sum of up to 16384 terms
        # cannot be better than its own rounding (helpers.rowsum_slack)
        yc = y.cpu().float()
        sl = None
        if dtype == torch.float32:
            sl = rowsum_slack(g32, torch.exp(yc)) if is_log else rowsum_slack(yc * g32, yc)
        assert_close(gi[R], ogi, dtype, nm + " grad_input vs oracle",
                     slack=None if sl is None else sl[R])
        fwd = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
        bwd = (torch.ops.aten._log_softmax_backward_data if is_log
               else torch.ops.aten._softmax_backward_data)
        cy = fwd(x32, -1, False)
        assert_close(y, cy, dtype, nm + " y vs ATen CPU")
        cgi = bwd(g32, yc, -1, torch.float32)
        # the CPU backward sums the same row in float32 too: twice the allowance
        assert_close(gi, cgi, dtype, nm + " grad_input vs ATen CPU",
                     slack=None if sl is None else 2 * sl)
        del y, gi, cy, cgi, yc, sl
