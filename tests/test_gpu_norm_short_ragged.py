"""LayerNorm / RMSNorm forward of short ragged rows (N % 8 != 0 in 16 bits, N % 4 != 0 in fp32, up to
2048 / 1024 elements) on 16-byte aligned tensors: a run of consecutive rows is staged through LDS
with whole aligned accesses and normalized there (norm_fwd_flat_kernel), the counterpart of the
reference's unvectorized path for such rows (can_vectorize() false, src/ATen/native/xpu/sycl/
LayerNormKernels.cpp:1121-1163).  Through the extern "C" ABI against the float64 oracle (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2): row counts that are not multiples of 8 (a last
piece with a ragged end), in place, without weights, float32 weights beside 16-bit rows, constant
and non-finite rows, and the same rows one element into their buffers (which the general kernels
serve) for comparison."""
import pytest
import torch

from helpers import assert_close, gen, offset_view, to_np32

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
