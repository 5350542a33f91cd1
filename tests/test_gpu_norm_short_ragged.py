"""LayerNorm / RMSNorm forward and backward of short ragged rows (N % 8 != 0 in 16 bits, N % 4 != 0
in fp32, up to 2048 / 1024 elements) on 16-byte aligned tensors: a run of consecutive rows is staged
through LDS with whole aligned accesses and worked there (norm_fwd_flat_kernel,
norm_bwd_flat_kernel), the counterpart of the reference's unvectorized paths for such rows
(can_vectorize() false, src/ATen/native/xpu/sycl/LayerNormKernels.cpp:1121-1163; the backward's
layer_norm_grad_input_kernel and the column sums behind it, :1218-1326).  Through the extern "C" ABI against the float64 oracle (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2): row counts that are not multiples of 8 (a last
piece with a ragged end), in place, without weights, float32 weights beside 16-bit rows, constant
and non-finite rows, and the same rows one element into their buffers (which the general kernels
serve) for comparison."""
import pytest
import torch

from helpers import assert_close, colsum_slack, gen, offset_view, to_np32, xhat_slack

pytestmark = pytest.mark.gpu

NS = [1, 3, 17, 100, 127, 257, 777, 1001, 2047]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_short_ragged_rows_against_oracle(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    wdtype = torch.float32 if mixed else dtype
    E = 4 if dtype == torch.float32 else 8
    for i, N in enumerate(NS):
        if N % E == 0 or (dtype == torch.float32 and N > 1024):
            continue
        for M in (1, 13, 1003):
            print("case short ragged norm rows", dtype, mixed, (M, N), flush=True)
            g = gen(1900 + i)
            x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
            x[M // 2] = -2.5  # a constant row
            gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
            beta = (0.1 * torch.randn(N, generator=g)).to(wdtype)
            xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
            what = "[%d, %d] %s" % (M, N, dtype)
            y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
            oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
            assert_close(y, oy, dtype, "layer_norm y " + what)
            assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
            assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
            assert torch.equal(y[M // 2].cpu(), beta.to(dtype)), "a constant row gives beta " + what
            ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
            roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
            assert_close(ry, roy, dtype, "rms_norm y " + what)
            assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
            # one element into their buffers: the general kernels, the same results to the tolerance
            yo, mo, ro = cabi.layer_norm_fwd(offset_view(xg, 1), gg, bg, 1e-5,
                                             y=offset_view(torch.empty_like(xg), 1))
            assert_close(yo, oy, dtype, "layer_norm y, off the pack " + what)
            assert_close(ro, to_np32(rstd), torch.float32, "rstd, off the pack " + what)
            if M == 13:
                y0, _, _ = cabi.layer_norm_fwd(xg, None, None, 1e-5)
                oy0, _, _ = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, 1e-5)
                assert_close(y0, oy0, dtype, "layer_norm without weights " + what)
                xc = xg.clone()
                yi, mi, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)
                assert yi.data_ptr() == xc.data_ptr()
                assert torch.equal(yi, y) and torch.equal(mi, mean) and torch.equal(ri, rstd)


def test_non_finite_rows_and_many_pieces(cabi, oracle, gpu):
    M, N = 70001, 100  # 875 pieces of 80 rows and one of 1
    g = gen(1950)
    x = (0.25 + torch.randn(M, N, generator=g)).bfloat16()
    x[5, 99] = float("inf")
    x[70000, 0] = float("nan")
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16()
    beta = (0.1 * torch.randn(N, generator=g)).bfloat16()
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    for r in (5, 70000):
        assert bool(torch.isnan(mean[r])) and bool(torch.isnan(y[r]).all())
    fin = torch.ones(M, dtype=torch.bool)
    fin[5] = fin[70000] = False
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x[fin]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y[fin.to(gpu)], oy, torch.bfloat16, "finite rows beside non-finite ones")
    assert_close(rstd[fin.to(gpu)], orr.reshape(-1), torch.float32, "rstd of the finite rows")
    ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    assert float(rr[5]) == 0.0 and bool(torch.isnan(rr[70000]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_short_ragged_rows_backward_against_oracle(cabi, oracle, gpu, dtype, mixed):
    """dX, dgamma, dbeta of LayerNorm and dX, dgamma of RMSNorm: one piece, a ragged last piece,
    more pieces than the launch has workgroups (70001 rows of 17: a workgroup walks several);
    dX alone, the column sums alone, no gamma, dX over dY in place, and the same rows one element
    into their buffers (the general kernels) beside them."""
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    wdtype = torch.float32 if mixed else dtype
    E = 4 if dtype == torch.float32 else 8
    for i, N in enumerate(NS):
        if N % E == 0 or (dtype == torch.float32 and N > 1024):
            continue
        for M in (1, 13, 1003) + ((70001,) if N == 17 else ()):
            print("case short ragged norm rows backward", dtype, mixed, (M, N), flush=True)
            g = gen(1960 + i)
            x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
            dy = torch.randn(M, N, generator=g).to(dtype)
            x[M // 2] = -2.5  # a constant row
            gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
            xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
            what = "[%d, %d] %s" % (M, N, dtype)
            _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
            dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
            odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                                  to_np32(rstd), to_np32(gamma))
            xhat = (x.float() - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
            sl_g = colsum_slack(dy.float() * xhat) + xhat_slack(dy, mean, rstd)
            sl_b = colsum_slack(dy.float())
            assert_close(dx, odx, dtype, "layer_norm dx " + what)
            assert_close(dg, odg, wdtype, "dgamma " + what, slack=sl_g)
            assert_close(db, odb, wdtype, "dbeta " + what, slack=sl_b)
            _, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
            rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
            rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
            sl_r = colsum_slack(dy.float() * x.float() * rr.cpu().reshape(M, 1))
            assert_close(rdx, rodx, dtype, "rms_norm dx " + what)
            assert_close(rdg, rodg, wdtype, "rms dgamma " + what, slack=sl_r)
            # one element into their buffers: the general kernels, the same results to the tolerance
            dxo, dgo, dbo = cabi.layer_norm_bwd(offset_view(dyg, 1), offset_view(xg, 1), mean, rstd, gg,
                                                dx=offset_view(torch.empty_like(xg), 1))
            assert_close(dxo, odx, dtype, "layer_norm dx, off the pack " + what)
            assert_close(dgo, odg, wdtype, "dgamma, off the pack " + what, slack=sl_g)
            assert_close(dbo, odb, wdtype, "dbeta, off the pack " + what, slack=sl_b)
            if M in (13, 70001):
                dx1, n1, n2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(True, False, False))
                assert n1 is None and n2 is None and torch.equal(dx1, dx), "dX alone " + what
                n0, dg1, db1 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(False, True, True))
                assert n0 is None and torch.equal(dg1, dg) and torch.equal(db1, db), "sums alone " + what
                rdx1, rn = cabi.rms_norm_bwd(dyg, xg, rr, gg, want=(True, False))
                assert rn is None and torch.equal(rdx1, rdx), "rms dX alone " + what
                dx0, dg0, db0 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, None, w_dtype=wdtype)
                odx0, odg0, odb0 = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                                         to_np32(rstd), None)
                assert_close(dx0, odx0, dtype, "dx without gamma " + what)
                assert_close(dg0, odg0, wdtype, "dgamma without gamma " + what, slack=sl_g)
                dyc = dyg.clone()
                dxi, dgi, dbi = cabi.layer_norm_bwd(dyc, xg, mean, rstd, gg, dx=dyc)
                assert dxi.data_ptr() == dyc.data_ptr()
                assert torch.equal(dxi, dx) and torch.equal(dgi, dg) and torch.equal(dbi, db)
                # twice the same bits (the order of every sum is fixed)
                dx2, dg2, db2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
                assert torch.equal(dx2, dx) and torch.equal(dg2, dg) and torch.equal(db2, db)


def test_backward_non_finite_rows_stay_in_their_rows(cabi, oracle, gpu):
    M, N = 2000, 100
    g = gen(1990)
    x = (0.25 + torch.randn(M, N, generator=g)).bfloat16()
    dy = torch.randn(M, N, generator=g).bfloat16()
    dy[7, 3] = float("inf")
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16()
    xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
    _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
    dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
    assert not bool(torch.isfinite(dx[7]).any()), "the row of the infinite dy element"
    fin = torch.ones(M, dtype=torch.bool)
    fin[7] = False
    odx, _, _ = oracle.layer_norm_bwd(to_np32(dy[fin]), to_np32(x[fin]), (N,), to_np32(mean.cpu()[fin]),
                                      to_np32(rstd.cpu()[fin]), to_np32(gamma))
    assert_close(dx[fin.to(gpu)], odx, torch.bfloat16, "rows beside the non-finite one")
    assert not bool(torch.isfinite(db[3])) and bool(torch.isfinite(db[:3]).all())
    assert bool(torch.isfinite(db[4:]).all())
