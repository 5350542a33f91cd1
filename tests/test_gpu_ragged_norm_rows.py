"""LayerNorm / RMSNorm forward of ragged 16-bit rows on 256 lanes or more (N % 8 != 0, N from about
3060 elements): every row sits at another 2-byte alignment, and the kernel addresses it through
the 16-byte aligned window that holds it, with gamma / beta held shifted by the window's head
(the reference's unaligned path: can_vectorize() false, src/ATen/native/xpu/sycl/
LayerNormKernels.cpp:1121-1163, and test/xpu/test_nn_xpu.py:17922-17998 for tensors that start one
element into their buffers).  Through the extern "C" ABI against the float64 oracle (16-bit atol
1e-2, rtol 1.6e-2; statistics float32 rtol = atol = 1e-5), with inputs, weights and outputs at
different offsets into their buffers, the bytes around every output checked untouched."""
import pytest
import torch

from helpers import assert_close, gen, to_np32

pytestmark = pytest.mark.gpu

GUARD = 64  # elements either side of a view that must keep their fill


def _view(t, off, fill=-77.0):
    """A copy of `t` that starts GUARD + off elements into a buffer filled with `fill`."""
    buf = torch.full((t.numel() + 2 * GUARD + 16,), fill, dtype=t.dtype, device=t.device)
    v = buf[GUARD + off:GUARD + off + t.numel()].view(t.shape)
    v.copy_(t)
    return buf, v


def _untouched(buf, off, numel, fill=-77.0):
    head, tail = buf[:GUARD + off], buf[GUARD + off + numel:]
    return bool((head == fill).all()) and bool((tail == fill).all())


# (rows, N): one row block a workgroup (grid = rows); three row blocks a workgroup at a stride of
# 1024 rows; 512 and 1024 lanes; a row whose window holds one pack more than the row itself
SHAPES = [(37, 4097), (3000, 4097), (1100, 5121), (600, 8193), (300, 12289), (520, 3071), (64, 4103)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("offs", [(0, 0, 0), (2, 2, 2), (1, 5, 3), (7, 0, 6)], ids=str)
def test_windowed_forward_against_oracle(cabi, oracle, gpu, dtype, offs):
    ox, oy, ow = offs
    code = cabi.dtype_code(dtype)
    for i, (M, N) in enumerate(SHAPES):
        print("case ragged norm rows", dtype, offs, (M, N), flush=True)
        p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)
        nrb = -(-M // p["rows_per_block"])
        assert p["resident"] == 1 and p["lanes_per_row"] >= 256, p
        assert p["lanes_per_row"] * p["packs_per_lane"] * 8 >= N + 7, p  # (holds the window)
        assert p["grid_blocks"] % 8 == 0 or p["grid_blocks"] >= nrb, p   # (one head a workgroup)
        g = gen(1700 + i)
        x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
        x[0] = 1.25        # a constant row
        x[M - 1, :3] = 0.0  # the head of a row is not representative of it
        gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
        beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
        _, xg = _view(x.to(gpu), ox)
        _, gg = _view(gamma.to(gpu), ow)
        _, bg = _view(beta.to(gpu), (ow + 3) % 8)
        ybuf, yv = _view(torch.zeros(M, N, dtype=dtype, device=gpu), oy)
        what = "[%d, %d] %s offsets %s" % (M, N, dtype, offs)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5, y=yv)
        oyy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oyy, dtype, "layer_norm y " + what)
        assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
        assert torch.equal(y[0].cpu(), beta), "a constant row gives beta bit for bit"
        assert _untouched(ybuf, oy, M * N), "layer_norm wrote outside y " + what
        ybuf2, yv2 = _view(torch.zeros(M, N, dtype=dtype, device=gpu), oy)
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6, y=yv2)
        roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "rms_norm y " + what)
        assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
        assert _untouched(ybuf2, oy, M * N), "rms_norm wrote outside y " + what
        if i % 3 == 0:
            # no weights; in place
            y0, _, _ = cabi.layer_norm_fwd(xg, None, None, 1e-5)
            oy0, _, _ = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, 1e-5)
            assert_close(y0, oy0, dtype, "layer_norm without weights " + what)
            xbuf, xc = _view(x.to(gpu), ox)
            yi, mi, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)
            assert yi.data_ptr() == xc.data_ptr()
            assert torch.equal(yi, y) and torch.equal(mi, mean) and torch.equal(ri, rstd)
            assert _untouched(xbuf, ox, M * N), "in-place layer_norm wrote outside x " + what


def test_windowed_forward_with_fp32_weights_and_special_rows(cabi, oracle, gpu):
    M, N = 700, 4097
    g = gen(1750)
    x = (0.25 + torch.randn(M, N, generator=g)).bfloat16()
    x[3, 4096] = float("inf")   # the last element of a row: the window's ragged end pack
    x[5, 0] = float("nan")      # the first: its ragged head pack
    gamma = 1 + 0.1 * torch.randn(N, generator=g)
    beta = 0.1 * torch.randn(N, generator=g)
    _, xg = _view(x.to(gpu), 3)
    _, gg = _view(gamma.to(gpu), 1)
    _, bg = _view(beta.to(gpu), 2)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    assert bool(torch.isnan(mean[3])) and bool(torch.isnan(y[3]).all())
    assert bool(torch.isnan(mean[5])) and bool(torch.isnan(y[5]).all())
    fin = [r for r in range(M) if r not in (3, 5)]
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x[fin]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y[fin], oy, torch.bfloat16, "finite rows beside non-finite ones")
    assert_close(mean[fin], om.reshape(-1), torch.float32, "mean of the finite rows")
    assert_close(rstd[fin], orr.reshape(-1), torch.float32, "rstd of the finite rows")
    ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    assert float(rr[3]) == 0.0 and bool(torch.isnan(rr[5]))
    roy, ror = oracle.rms_norm_fwd(to_np32(x[fin]), (N,), to_np32(gamma), 1e-6)
    assert_close(ry[fin], roy, torch.bfloat16, "rms_norm, finite rows")


def test_fused_add_and_forced_layouts_on_windowed_rows(cabi, oracle, gpu):
    """The residual add in front of the norm reads two tensors and writes two through the same
    window; a forced 512-lane layout and a forced grid keep the window, a forced 128-lane layout
    gives the row-start addressing: all within the tolerance of the oracle."""
    M, N = 900, 4099
    dtype = torch.float16
    g = gen(1760)
    x = (0.5 * torch.randn(M, N, generator=g)).to(dtype)
    res = (0.5 * torch.randn(M, N, generator=g)).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
    _, xg = _view(x.to(gpu), 5)
    _, rg = _view(res.to(gpu), 2)
    _, gg = _view(gamma.to(gpu), 7)
    _, bg = _view(beta.to(gpu), 4)
    hbuf, hv = _view(torch.zeros(M, N, dtype=dtype, device=gpu), 6)
    ybuf, yv = _view(torch.zeros(M, N, dtype=dtype, device=gpu), 1)
    y, h, _, _ = cabi.add_layer_norm_fwd(xg, rg, gg, bg, 1e-5, h=hv, y=yv)
    hs = (x.float() + res.float()).to(dtype)
    assert torch.equal(h.cpu(), hs), "h = x + residual, rounded once"
    oy, om, orr = oracle.layer_norm_fwd(to_np32(hs), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y, oy, dtype, "add + layer_norm y")
    assert _untouched(hbuf, 6, M * N) and _untouched(ybuf, 1, M * N)
    code = cabi.dtype_code(dtype)
    for forced in ((512, 2, 0, 0), (0, 0, 0, 3), (128, 0, 0, 0)):
        try:
            cabi.set_override(cabi.OP_LAYER_NORM_FWD, *forced)
            if forced[0] == 128:
                # (a row of 4099 elements does not fit 128 lanes: a shorter one does)
                Ns = 2045
                xs = x[:, :Ns].contiguous()
                _, xsg = _view(xs.to(gpu), 5)
                _, gs = _view(gamma[:Ns].contiguous().to(gpu), 7)
                _, bs = _view(beta[:Ns].contiguous().to(gpu), 4)
                ys, _, _ = cabi.layer_norm_fwd(xsg, gs, bs, 1e-5)
                oys, _, _ = oracle.layer_norm_fwd(to_np32(xs), (Ns,), to_np32(gamma[:Ns]),
                                                  to_np32(beta[:Ns]), 1e-5)
                assert_close(ys, oys, dtype, "forced 128 lanes")
            else:
                yf, mf, rf = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
                oyf, _, orf = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
                assert_close(yf, oyf, dtype, "forced %s" % (forced,))
                assert_close(rf, orf.reshape(-1), torch.float32, "rstd, forced %s" % (forced,))
        finally:
            cabi.clear_overrides()
    assert cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)["lanes_per_row"] == 256
