"""Tensors of more than 2^31 elements: row offsets beyond the 32-bit range.

The reference keeps separate 64-bit-index instantiations for such tensors (canUse32BitIndexMath,
src/ATen/native/xpu/sycl/LayerNormKernels.cpp:1147, SoftMaxKernels.cpp:1594, 1668-1720); the HIP
kernels form every row offset in 64 bits.  bf16 [2^19 + 3, 4104] is 2 151 690 264 elements (4.3 GB a
tensor; generated on the GPU); the first, middle and last 64 rows are compared with the float64
oracle and every row with a property that needs no reference: softmax rows sum to one, their
gradients to zero; a normalized row has mean(xhat^2) = 1 (RMSNorm) or mean 0 and variance 1
(LayerNorm); sum_j dx_j * x_j = 0 for the RMSNorm backward; dgamma against the closed form
sum_i dy * x * rstd (test/regressions/test_rms_norm.py:82-83 in the reference) in float64 on the
GPU.  A second shape, [2^19 + 64, 4096], takes the backward kernels for rows that fill their
layout exactly.
"""
import pytest
import torch

from helpers import assert_close, to_np32

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
CHUNK = 32768  # rows per step of the all-rows checks (a float32 copy of a chunk is 0.5 GB)


def _sample_rows(M):
    return [slice(0, 64), slice(M // 2, M // 2 + 64), slice(M - 64, M)]


def _chunks(M):
    for r0 in range(0, M, CHUNK):
        yield slice(r0, min(M, r0 + CHUNK))


def _randn(M, N, gpu, seed):
    g = torch.Generator(device=gpu).manual_seed(seed)
    t = torch.empty(M, N, dtype=BF, device=gpu)
    for r in _chunks(M):
        t[r] = torch.randn(r.stop - r.start, N, generator=g, device=gpu).to(BF)
    return t


@pytest.mark.parametrize("shape", [((1 << 19) + 3, 4104), ((1 << 19) + 64, 4096)], ids=str)
def test_rms_norm_fwd_bwd_beyond_2_31_elements(cabi, oracle, gpu, shape):
    M, N = shape
    assert M * N > (1 << 31)
    print("case large rms", shape, flush=True)
    x, dy = _randn(M, N, gpu, 11), _randn(M, N, gpu, 12)
    w = (1 + 0.1 * torch.randn(N, device=gpu)).to(BF)
    y, rstd = cabi.rms_norm_fwd(x, w, 1e-6)
    dx, dw = cabi.rms_norm_bwd(dy, x, rstd, w)
    for r in _sample_rows(M):
        oy, orstd = oracle.rms_norm_fwd(to_np32(x[r]), (N,), to_np32(w), 1e-6)
        assert_close(y[r], oy, BF, "y rows %d.." % r.start)
        assert_close(rstd[r], orstd.reshape(-1), torch.float32, "rstd rows %d.." % r.start)
        odx, _ = oracle.rms_norm_bwd(to_np32(dy[r]), to_np32(x[r]), (N,), to_np32(rstd[r]),
                                     to_np32(w), mask=(True, False))
        assert_close(dx[r], odx, BF, "dx rows %d.." % r.start)
    # every row: mean((y / w)^2) = 1 up to the bf16 rounding of y; sum_j dx_j x_j = 0 against
    # sum_j |dx_j x_j|; dweight = sum_i dy * x * rstd, summed in float64 on the GPU
    w32 = w.float()
    closed = torch.zeros(N, dtype=torch.float64, device=gpu)
    for r in _chunks(M):
        x32 = x[r].float()
        ms = (y[r].float() / w32).pow(2).mean(1)
        assert float((ms - 1).abs().max()) < 2e-2, "rows %d..: mean((y/w)^2) != 1" % r.start
        p = dx[r].float() * x32
        assert float((p.sum(1).abs() / p.abs().sum(1)).max()) < 2e-2, "rows %d..: sum dx*x" % r.start
        closed += (dy[r].double() * x32.double() * rstd[r].double().reshape(-1, 1)).sum(0)
        del x32, p
    assert_close(dw, closed, BF, "dweight vs sum(dY * x * rstd)")
    # bit-reproducible
    dx2, dw2 = cabi.rms_norm_bwd(dy, x, rstd, w)
    assert torch.equal(dw, dw2) and torch.equal(dx[M - 64:], dx2[M - 64:])


@pytest.mark.parametrize("shape", [((1 << 19) + 3, 4104), ((1 << 19) + 64, 4096)], ids=str)
def test_layer_norm_fwd_bwd_beyond_2_31_elements(cabi, oracle, gpu, shape):
    M, N = shape
    print("case large layer_norm", shape, flush=True)
    x, dy = _randn(M, N, gpu, 21), _randn(M, N, gpu, 22)
    gamma = (1 + 0.1 * torch.randn(N, device=gpu)).to(BF)
    beta = (0.1 * torch.randn(N, device=gpu)).to(BF)
    y, mean, rstd = cabi.layer_norm_fwd(x, gamma, beta, 1e-5)
    dx, dg, db = cabi.layer_norm_bwd(dy, x, mean, rstd, gamma)
    for r in _sample_rows(M):
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x[r]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y[r], oy, BF, "y rows %d.." % r.start)
        assert_close(mean[r], om.reshape(-1), BF, "mean rows %d.." % r.start)
        assert_close(rstd[r], orr.reshape(-1), BF, "rstd rows %d.." % r.start)
        odx, _, _ = oracle.layer_norm_bwd(to_np32(dy[r]), to_np32(x[r]), (N,), to_np32(mean[r]),
                                          to_np32(rstd[r]), to_np32(gamma), mask=(True, False, False))
        assert_close(dx[r], odx, BF, "dx rows %d.." % r.start)
    g32, b32 = gamma.float(), beta.float()
    cg = torch.zeros(N, dtype=torch.float64, device=gpu)
    cb = torch.zeros(N, dtype=torch.float64, device=gpu)
    for r in _chunks(M):
        xh = (y[r].float() - b32) / g32
        assert float(xh.mean(1).abs().max()) < 2e-2, "rows %d..: mean(xhat) != 0" % r.start
        assert float((xh.var(1, unbiased=False) - 1).abs().max()) < 3e-2, "rows %d..: var" % r.start
        # sum_j dx_j = 0 for every LayerNorm row
        d32 = dx[r].float()
        assert float((d32.sum(1).abs() / d32.abs().sum(1)).max()) < 2e-2, "rows %d..: sum dx" % r.start
        xhat = (x[r].double() - mean[r].double().reshape(-1, 1)) * rstd[r].double().reshape(-1, 1)
        cg += (dy[r].double() * xhat).sum(0)
        cb += dy[r].double().sum(0)
        del xh, d32, xhat
    assert_close(dg, cg, BF, "dgamma vs sum(dY * xhat)")
    assert_close(db, cb, BF, "dbeta vs sum(dY)")


def test_softmax_fwd_bwd_beyond_2_31_elements(cabi, oracle, gpu):
    M, N = (1 << 19) + 3, 4104
    print("case large softmax", (M, N), flush=True)
    x, grad = _randn(M, N, gpu, 31), _randn(M, N, gpu, 32)
    x.mul_(3)
    for is_log in (False, True):
        nm = "log_softmax" if is_log else "softmax"
        y = cabi.softmax_fwd(x, is_log)
        gi = cabi.softmax_bwd(grad, y, is_log)
        for r in _sample_rows(M):
            oy = oracle.softmax_fwd(to_np32(x[r]), is_log)
            assert_close(y[r], oy, BF, "%s y rows %d.." % (nm, r.start))
            ogi = oracle.softmax_bwd(to_np32(grad[r]), to_np32(y[r]), is_log)
            assert_close(gi[r], ogi, BF, "%s grad_input rows %d.." % (nm, r.start))
        for r in _chunks(M):
            y32 = y[r].float()
            rowsum = torch.exp(y32).sum(1) if is_log else y32.sum(1)
            assert float((rowsum - 1).abs().max()) < 2e-2, "%s rows %d..: sum != 1" % (nm, r.start)
            if not is_log:
                g32 = gi[r].float()
                assert float(g32.sum(1).abs().max()) < 0.05, "rows %d..: sum grad_input" % r.start
                del g32
            del y32
        del y, gi


def test_long_rows_held_by_teams_beyond_2_31_elements(cabi, oracle, gpu):
    """bf16 [32771, 65544] (2 147 942 424 elements, 4.3 GB a tensor): rows beyond one workgroup's
    registers, whose backward teams of workgroups hold four rows at a time (norm_bwd_team_kernel)
    and whose last groups of rows lie beyond the 32-bit offsets.  RMSNorm forward and backward:
    the first, middle and last rows against the oracle; every row against sum_j dx_j x_j = 0;
    dweight against the closed form in float64 on the GPU."""
    M, N = 32771, 65544
    assert M * N > (1 << 31)
    p = cabi.plan(cabi.OP_RMS_NORM_BWD, M, N, cabi.BF16, cabi.BF16)
    assert p["resident"] == 0 and p["block_threads"] == 512 and p["packs_per_lane"] == 2, p
    print("case large long rows", (M, N), flush=True)
    rows = 2048  # rows per step of the all-rows checks
    g = torch.Generator(device=gpu).manual_seed(21)
    x = torch.empty(M, N, dtype=BF, device=gpu)
    dy = torch.empty(M, N, dtype=BF, device=gpu)
    for r0 in range(0, M, rows):
        r = slice(r0, min(M, r0 + rows))
        x[r] = torch.randn(r.stop - r.start, N, generator=g, device=gpu).to(BF)
        dy[r] = torch.randn(r.stop - r.start, N, generator=g, device=gpu).to(BF)
    w = (1 + 0.1 * torch.randn(N, device=gpu)).to(BF)
    y, rstd = cabi.rms_norm_fwd(x, w, 1e-6)
    del y
    dx, dw = cabi.rms_norm_bwd(dy, x, rstd, w)
    for r in (slice(0, 8), slice(M // 2, M // 2 + 8), slice(M - 8, M)):
        odx, _ = oracle.rms_norm_bwd(to_np32(dy[r]), to_np32(x[r]), (N,), to_np32(rstd[r]),
                                     to_np32(w), mask=(True, False))
        assert_close(dx[r], odx, BF, "dx rows %d.." % r.start)
    ref_dw = torch.zeros(N, dtype=torch.float64, device=gpu)
    mag_dw = torch.zeros(N, dtype=torch.float64, device=gpu)
    for r0 in range(0, M, rows):
        r = slice(r0, min(M, r0 + rows))
        dxr, xr = dx[r].double(), x[r].double()
        dot = (dxr * xr).sum(1)
        mag = (dxr * xr).abs().sum(1)
        # (dx is rounded to bf16: each term carries up to 2^-9 of relative error)
        assert bool((dot.abs() <= mag * 2.0 ** -7 + 1e-6).all()), "sum_j dx_j x_j, rows %d.." % r0
        t = dy[r].double() * xr * rstd[r].double().reshape(-1, 1)
        ref_dw += t.sum(0)
        mag_dw += t.abs().sum(0)
        del dxr, xr, t
    err = (dw.double() - ref_dw).abs()
    # bf16 rounding of dweight plus the float32 partial sums of the kernel
    assert bool((err <= 1e-2 + 1.6e-2 * ref_dw.abs() + mag_dw * 2.0 ** -20).all()), float(err.max())
