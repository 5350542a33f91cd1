"""GroupNorm forward on feature maps beyond one workgroup's registers (a VAE decoder's 128x128 to
512x512 maps: slabs of 0.25 to 1 M elements), channels of whole 16-byte packs: a slab is held in
the registers of a team of workgroups (norm_fwd_team_kernel in its GroupNorm mode), X is read once.
It serves the regime of the reference's multi-pass kernels (src/ATen/native/xpu/sycl/
GroupNormKernels.cpp:364-530).  Through the extern "C" ABI against the float64 oracle (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2), against the path a workgroup takes when its
wait gives up (forced from the host by a wait of zero: no kernel hangs), with and without weights,
with float32 weights beside 16-bit rows, and in place (which the multi-pass kernel serves)."""
import pytest
import torch

from helpers import assert_close, gen, to_np32

pytestmark = pytest.mark.gpu

# (N, C, HxW, groups): 64 slabs of 131072 elements (2 workgroups a slab); 32 slabs of 262144 with a
# ragged last chunk; 9 slabs of 81920 + 8 (a slab that is one pack longer than 20 strides);
# 16 slabs of 1 M elements (16 workgroups a slab); 2 slabs of 4 M elements (fewer slabs than the
# 8 teams a launch otherwise asks for: all at once, 256 workgroups a slab)
SHAPES = [(2, 256, 16384, 32), (4, 64, 32776, 8), (3, 6, 40964 * 8 // 2, 3), (1, 128, 131072, 16),
          (2, 8, 524288, 1)]


def _with_wait(cabi, us, fn):
    try:
        cabi.set_team_wait_us(us)
        return fn()
    finally:
        cabi.set_team_wait_us()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_team_forward_against_oracle_and_the_give_up_path(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    wdtype = torch.float32 if mixed else dtype
    code = cabi.dtype_code(dtype)
    E = 4 if dtype == torch.float32 else 8
    for i, (N, C, HxW, groups) in enumerate(SHAPES):
        if HxW % E:
            continue
        print("case group norm large maps", dtype, mixed, (N, C, HxW, groups), flush=True)
        p = cabi.group_norm_plan(0, N, C, HxW, groups, code)
        rows = N * groups
        assert p["resident"] == 0 and 8 <= p["grid_blocks"] <= 512, p
        g = gen(1800 + i)
        x = (0.5 + torch.randn(N, C, HxW, generator=g)).to(dtype)
        x[0, 0, :3] = 0.0   # the head of a slab is not representative of it
        x[N - 1, C - 1] = 1.25
        gamma = (1 + 0.1 * torch.randn(C, generator=g)).to(wdtype)
        beta = (0.1 * torch.randn(C, generator=g)).to(wdtype)
        xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
        what = "[%d, %d, %d] in %d groups %s" % (N, C, HxW, groups, dtype)
        y, mean, rstd = cabi.group_norm_fwd(xg, gg, bg, groups, 1e-5)
        oy, om, orr = oracle.group_norm_fwd(to_np32(x), groups, to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "group_norm y " + what)
        assert_close(mean.float(), om.reshape(-1), wdtype, "mean " + what)
        assert_close(rstd.float(), orr.reshape(-1), wdtype, "rstd " + what)
        assert mean.dtype == wdtype and mean.numel() == rows
        # a second run gives the same bits; every wait giving up at once gives the same result
        # to rounding
        y2, mean2, rstd2 = cabi.group_norm_fwd(xg, gg, bg, groups, 1e-5)
        assert torch.equal(y.view(torch.uint8), y2.view(torch.uint8))
        assert torch.equal(rstd.view(torch.uint8), rstd2.view(torch.uint8))
        fy, fm, fr = _with_wait(cabi, 0, lambda: cabi.group_norm_fwd(xg, gg, bg, groups, 1e-5))
        assert_close(fy, oy, dtype, "y, every wait given up " + what)
        assert_close(fr.float(), orr.reshape(-1), wdtype, "rstd, every wait given up " + what)
        if i % 2 == 0:
            # without weights; in place (the multi-pass kernel)
            y0, _, _ = cabi.group_norm_fwd(xg, None, None, groups, 1e-5)
            oy0, _, _ = oracle.group_norm_fwd(to_np32(x), groups, None, None, 1e-5)
            assert_close(y0, oy0, dtype, "group_norm without weights " + what)
            xc = xg.clone()
            yi, mi, ri = cabi.group_norm_fwd(xc, gg, bg, groups, 1e-5, y=xc)
            assert yi.data_ptr() == xc.data_ptr()
            assert_close(yi, oy, dtype, "in place y " + what)


def test_special_slabs_and_channels_that_are_not_whole_packs(cabi, oracle, gpu):
    """A slab with an inf or a NaN has NaN statistics and output and leaves its neighbours alone;
    channels that are not whole packs keep the multi-pass kernel."""
    N, C, HxW, groups = 2, 64, 16384, 8
    g = gen(1850)
    x = (0.25 + torch.randn(N, C, HxW, generator=g)).bfloat16()
    x[0, 9, 777] = float("inf")    # slab (0, 1)
    x[1, 63, HxW - 1] = float("nan")  # slab (1, 7), its last element
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).bfloat16()
    beta = (0.1 * torch.randn(C, generator=g)).bfloat16()
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.group_norm_fwd(xg, gg, bg, groups, 1e-5)
    D = C // groups
    bad = {(0, 1), (1, 7)}
    for n in range(N):
        for gr in range(groups):
            slab = y[n, gr * D:(gr + 1) * D]
            if (n, gr) in bad:
                assert bool(torch.isnan(slab).all()) and bool(torch.isnan(mean.reshape(-1)[n * groups + gr]))
            else:
                assert bool(torch.isfinite(slab).all())
    good = torch.tensor([[0 if (n, gr) in bad else 1 for gr in range(groups)] for n in range(N)],
                        dtype=torch.bool)
    xs = x.clone()
    xs[0, 9, 777] = 0.0
    xs[1, 63, HxW - 1] = 0.0
    oy, om, orr = oracle.group_norm_fwd(to_np32(xs), groups, to_np32(gamma), to_np32(beta), 1e-5)
    for n in range(N):
        for gr in range(groups):
            if good[n, gr]:
                assert_close(y[n, gr * D:(gr + 1) * D], oy[n, gr * D:(gr + 1) * D], torch.bfloat16,
                             "slab (%d, %d) beside non-finite ones" % (n, gr))
    # HxW = 16388 elements: 2048.5 packs of bf16 a channel
    N, C, HxW, groups = 1, 64, 16388, 8
    x = torch.randn(N, C, HxW, generator=g).bfloat16()
    p = cabi.group_norm_plan(0, N, C, HxW, groups, cabi.BF16)
    assert p["resident"] == 0 and p["grid_blocks"] <= N * groups, p
    y, mean, rstd = cabi.group_norm_fwd(x.to(gpu), gg, bg, groups, 1e-5)
    oy, om, orr = oracle.group_norm_fwd(to_np32(x), groups, to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y, oy, torch.bfloat16, "channels of 2048.5 packs")


# (N, C, HxW, groups) for the backward: 64 slabs of 8 channels of 2048 packs (bf16: four packs a
# lane, a workgroup a channel); slabs of 8 channels of 4097 packs (two workgroups a channel, the
# second nearly empty: the multi-launch kernels keep them) and of 6000 packs (two workgroups a
# channel, the second ragged); 16 slabs of 8 channels of 16384 packs (four workgroups a channel,
# 32 a slab); one group of 3 channels of 300 to 600 packs (short channels keep the multi-launch
# kernels)
BWD_SHAPES = [(2, 256, 16384, 32), (2, 16, 4097 * 8, 2), (3, 16, 6000 * 8, 2), (1, 128, 131072, 16),
              (5, 3, 2400, 1)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_team_backward_against_oracle_and_the_give_up_path(cabi, oracle, gpu, dtype, mixed):
    """native_group_norm_backward on slabs beyond one workgroup's registers whose channels are
    whole packs: gn_bwd_team_kernel holds a slab in the registers of a team of workgroups, one or
    several a channel, the channel sums cross the team once, dY and X are read once (the
    reference: two kernels over the slab, GroupNormKernels.cpp:1088-1165 and 1353-1589).
    Against the oracle, with every wait given up (a workgroup then sums the slab itself), in
    place and with dX over X (the multi-launch kernels), without gamma, dX alone, twice the
    same bits."""
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    wdtype = torch.float32 if mixed else dtype
    E = 4 if dtype == torch.float32 else 8
    for i, (N, C, HxW, groups) in enumerate(BWD_SHAPES):
        if HxW % E:
            continue
        print("case group norm large maps backward", dtype, mixed, (N, C, HxW, groups), flush=True)
        g = gen(1860 + i)
        x = (0.5 + torch.randn(N, C, HxW, generator=g)).to(dtype)
        dy = torch.randn(N, C, HxW, generator=g).to(dtype)
        x[N - 1, C - 1] = 1.25  # a constant channel
        gamma = (1 + 0.1 * torch.randn(C, generator=g)).to(wdtype)
        xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
        what = "[%d, %d, %d] in %d groups %s" % (N, C, HxW, groups, dtype)
        _, mean, rstd = cabi.group_norm_fwd(xg, gg, None, groups, 1e-5)
        dx, dg, db = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, groups)
        odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), groups, to_np32(mean.float()),
                                              to_np32(rstd.float()), to_np32(gamma))
        D = C // groups
        mu = mean.float().cpu().reshape(N, groups, 1, 1)
        rs = rstd.float().cpu().reshape(N, groups, 1, 1)
        xhat = ((x.float().reshape(N, groups, D, HxW) - mu) * rs).reshape(N, C, HxW)
        # (float32 partial sums: a few ulps of the sum of the magnitudes, per channel)
        sl_g = (dy.float() * xhat).abs().sum(dim=(0, 2)) * 2.0 ** -22
        sl_b = dy.float().abs().sum(dim=(0, 2)) * 2.0 ** -22
        assert_close(dx, odx, dtype, "group_norm dx " + what)
        assert_close(dg.float(), odg, wdtype, "dgamma " + what, slack=sl_g)
        assert_close(db.float(), odb, wdtype, "dbeta " + what, slack=sl_b)
        dx2, dg2, db2 = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, groups)
        for a, b in ((dx, dx2), (dg, dg2), (db, db2)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "twice the same bits " + what
        fdx, fdg, fdb = _with_wait(cabi, 0, lambda: cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, groups))
        assert_close(fdx, odx, dtype, "dx, every wait given up " + what)
        assert_close(fdg.float(), odg, wdtype, "dgamma, every wait given up " + what, slack=sl_g)
        assert_close(fdb.float(), odb, wdtype, "dbeta, every wait given up " + what, slack=sl_b)
        # in place over dY and over X: the multi-launch kernels
        for over in ("dy", "x"):
            dyc, xc = dyg.clone(), xg.clone()
            target = dyc if over == "dy" else xc
            idx, idg, idb = cabi.group_norm_bwd(dyc, xc, mean, rstd, gg, groups, dx=target)
            assert idx.data_ptr() == target.data_ptr()
            assert_close(idx, odx, dtype, "dx over %s %s" % (over, what))
            assert_close(idg.float(), odg, wdtype, "dgamma, dx over %s %s" % (over, what), slack=sl_g)
        if i % 2 == 0:
            dx1, n1, n2 = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, groups, want=(True, False, False))
            assert n1 is None and n2 is None and torch.equal(dx1, dx), "dX alone " + what
            dx0, dg0, db0 = cabi.group_norm_bwd(dyg, xg, mean, rstd, None, groups)
            odx0, odg0, odb0 = oracle.group_norm_bwd(to_np32(dy), to_np32(x), groups,
                                                     to_np32(mean.float()), to_np32(rstd.float()), None)
            assert_close(dx0, odx0, dtype, "dx without gamma " + what)
            assert_close(dg0.float(), odg0, wdtype, "dgamma without gamma " + what, slack=sl_g)
