"""GPU parity of the HIP kernels, called through the extern "C" ABI, against the CPU oracle and
against PyTorch's CPU ATen ops on the same seeded inputs.

Mirrors the reference's own harness for this path, "compute on CPU, compute on the device,
assertEqual" (test/xpu/extended/test_ops_xpu.py:124-145, test/repro/
test_layer_norm_group_norm_align.py:25-78 in intel/torch-xpu-ops).

Tolerances (written out in helpers.TOL): float32 rtol = atol = 1e-5; float16/bfloat16 atol 1e-2,
rtol 1.6e-2 against a reference accumulated in float32 or better, saved mean/rstd included.
"""
import pytest
import torch

from helpers import assert_close, gen, rowsum_slack, to_np32, xhat_slack

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# rows x normalized size: tiny, odd, power-of-two, wider than one wavefront / one workgroup
SHAPES = [(1, 1), (3, 8), (7, 64), (5, 127), (64, 256), (33, 1024), (17, 2048), (9, 4097),
          (12, 4096), (4, 5120), (6, 8192), (3, 16384), (2, 40000),
          # hidden sizes that are not powers of two: 3 or 5 packs a lane, 512 lanes beyond 8192
          (10, 1536), (5, 2560), (7, 3072), (6, 6144), (5, 7168), (4, 10240), (5, 12288),
          (3, 14336), (3, 20480)]


def _mk(M, N, dtype, seed, wdtype=None):
    g = gen(seed)
    x = torch.randn(M, N, generator=g).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    wdt = dtype if wdtype is None else wdtype
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdt)
    beta = (0.1 * torch.randn(N, generator=g)).to(wdt)
    return x, dy, gamma, beta


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_layer_norm_fwd_bwd(cabi, oracle, gpu, dtype, shape, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    M, N = shape
    print("case layer_norm", dtype, shape, mixed, flush=True)
    x, dy, gamma, beta = _mk(M, N, dtype, 11, torch.float32 if mixed else None)
    y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert y.dtype == dtype and mean.dtype == torch.float32 and rstd.dtype == torch.float32
    assert_close(y, oy, dtype, "y")
    assert_close(mean, om.reshape(-1), dtype, "mean")
    assert_close(rstd, orr.reshape(-1), dtype, "rstd")
    if dtype == torch.float32:
        cy, cm, cr = torch.ops.aten.native_layer_norm(x, [N], gamma, beta, 1e-5)
        assert_close(y, cy, dtype, "y vs ATen CPU")
        assert_close(mean, cm.reshape(-1), dtype, "mean vs ATen CPU")
        assert_close(rstd, cr.reshape(-1), dtype, "rstd vs ATen CPU")
    # backward consumes the device's own saved statistics
    dx, dg, db = cabi.layer_norm_bwd(dy.to(gpu), x.to(gpu), mean, rstd, gamma.to(gpu))
    odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                          to_np32(rstd), to_np32(gamma))
    assert dx.dtype == dtype and dg.dtype == gamma.dtype and db.dtype == gamma.dtype
    assert_close(dx, odx, dtype, "dx")
    assert_close(dg, odg, gamma.dtype, "dgamma",
                 slack=xhat_slack(dy, mean, rstd) if mixed else None)
    assert_close(db, odb, gamma.dtype, "dbeta")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_rms_norm_fwd_bwd(cabi, oracle, gpu, dtype, shape):
    M, N = shape
    print("case rms_norm", dtype, shape, flush=True)
    x, dy, gamma, _ = _mk(M, N, dtype, 12)
    y, rstd = cabi.rms_norm_fwd(x.to(gpu), gamma.to(gpu), 1e-6)
    oy, orr = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
    assert_close(y, oy, dtype, "y")
    assert_close(rstd, orr.reshape(-1), dtype, "rstd")
    # closed form of the reference's own numeric test (test/xpu/test_nn_xpu.py:11576-11588)
    x32, g32 = x.float(), gamma.float()
    closed = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + 1e-6) * g32
    assert_close(y, closed, dtype, "y vs closed form")
    dx, dg = cabi.rms_norm_bwd(dy.to(gpu), x.to(gpu), rstd, gamma.to(gpu))
    odx, odg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rstd), to_np32(gamma))
    assert_close(dx, odx, dtype, "dx")
    assert_close(dg, odg, dtype, "dgamma")
    if dtype == torch.float32:
        # ATen has no CPU _fused_rms_norm_backward: autograd through F.rms_norm on CPU instead
        xr, gr = x.clone().requires_grad_(), gamma.clone().requires_grad_()
        torch.nn.functional.rms_norm(xr, (N,), gr, 1e-6).backward(dy)
        assert_close(dx, xr.grad, dtype, "dx vs CPU autograd", scale=2.0)
        assert_close(dg, gr.grad, dtype, "dgamma vs CPU autograd", scale=2.0)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("is_log", [False, True], ids=["softmax", "log_softmax"])
def test_softmax_fwd_bwd(cabi, oracle, gpu, dtype, shape, is_log):
    M, N = shape
    print("case softmax", dtype, shape, is_log, flush=True)
    g = gen(13)
    x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
    if N > 4:
        x[0, N // 2:] = float("-inf")  # a masked tail, as a causal row has
    grad = torch.randn(M, N, generator=g).to(dtype)
    y = cabi.softmax_fwd(x.to(gpu), is_log)
    oy = oracle.softmax_fwd(to_np32(x), is_log)
    assert y.dtype == dtype
    assert_close(y, oy, dtype, "y")
    fn = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
    if dtype == torch.float32:
        assert_close(y, fn(x, -1, False), dtype, "y vs ATen CPU")
    else:
        assert_close(y, fn(x.float(), -1, False), dtype, "y vs ATen CPU on upcast input")
    gi = cabi.softmax_bwd(grad.to(gpu), y, is_log)
    ogi = oracle.softmax_bwd(to_np32(grad), to_np32(y), is_log)
    # a float32 row sum cannot be better than its own rounding (helpers.rowsum_slack)
    yc, g32 = y.cpu().float(), grad.float()
    sl = None
    if dtype == torch.float32:
        sl = rowsum_slack(g32, torch.exp(yc)) if is_log else rowsum_slack(yc * g32, yc)
    assert_close(gi, ogi, dtype, "grad_input", slack=sl)
    bfn = (torch.ops.aten._log_softmax_backward_data if is_log
           else torch.ops.aten._softmax_backward_data)
    cgi = bfn(g32, yc, -1, torch.float32)
    # the CPU kernel sums the same row in float32 too: twice the allowance
    assert_close(gi, cgi, dtype, "grad_input vs ATen CPU", slack=None if sl is None else 2 * sl)


def test_softmax_half_to_float(cabi, oracle, gpu):
    # softmax(half, dtype=float) must equal softmax(float(half)), forward and backward (the
    # identity test/xpu/test_nn_xpu.py:15036-15047 checks on the reference's device).  The two
    # calls pack 8 resp. 4 elements per lane, so row sums may differ in the last float32 bits.
    g = gen(14)
    for N in (37, 1024, 4097):
        for is_log in (False, True):
            x = torch.randn(19, N, generator=g).half().to(gpu)
            grad = torch.randn(19, N, generator=g).to(gpu)
            y_h2f = cabi.softmax_fwd(x, is_log, out_dtype=torch.float32)
            y_f = cabi.softmax_fwd(x.float(), is_log)
            assert y_h2f.dtype == torch.float32
            assert_close(y_h2f, y_f, torch.float32, "half_to_float y")
            gi_h = cabi.softmax_bwd(grad, y_h2f, is_log, gi_dtype=torch.float16)
            gi_f = cabi.softmax_bwd(grad, y_f, is_log)
            assert gi_h.dtype == torch.float16
            assert_close(gi_h, gi_f, torch.float16, "half_to_float grad_input")
