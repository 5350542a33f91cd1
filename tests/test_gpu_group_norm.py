"""GPU parity of native_group_norm / native_group_norm_backward, through the C ABI and through
the host operators, against the CPU oracle, the committed golden vectors and PyTorch's CPU ATen
ops on the same seeded inputs.

Mirrors test/repro/test_layer_norm_group_norm_align.py:81-154 (1-d and 2-d inputs, small and
large batch, float32/float16/bfloat16, forward + all three gradients against the CPU),
test/regressions/test_group_norm.py:24-60 (the native_group_norm sample inputs: eps 0.5 and -0.5,
absent weight/bias, an empty batch) and test/xpu/test_nn_xpu.py:10833-10890, 11657-11790
(GroupNorm general, empty, numeric) in intel/torch-xpu-ops.
Tolerances: float32 rtol = atol = 1e-5; float16/bfloat16 atol 1e-2, rtol 1.6e-2, statistics
included (compared in float32 where the op returns them in 16 bits).
"""
import pytest
import torch
import torch.nn.functional as F

from helpers import GOLDEN_DTYPES, assert_close, colsum_slack, gen, load_golden, offset_view, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (N, C, spatial, groups)
SHAPES = [(2, 4, (), 2), (64, 32, (), 4), (256, 32, (), 4), (64, 32, (16,), 4), (256, 32, (4, 4), 4),
          (3, 6, (5,), 3), (2, 6, (7, 3), 2), (4, 64, (32, 32), 32), (2, 320, (16, 16), 32),
          (1, 8, (127,), 1), (3, 10, (4097,), 5), (2, 8, (64, 129), 2), (1, 4, (1 << 17,), 2),
          (2, 6, (1,), 6), (5, 5, (5,), 1),
          # rows of 6..10 packs a lane on 512 lanes (16-bit: L = 24576 .. 40960; fp32: 12288 ..
          # 20480) and an fp32 row of 11 packs a lane on 1024 lanes
          (2, 12, (64, 64), 2), (2, 14, (64, 64), 2), (2, 18, (64, 64), 2), (1, 20, (64, 64), 2),
          (2, 12, (2048,), 2), (2, 14, (2048,), 2), (1, 20, (2048,), 2), (1, 22, (64, 64), 2),
          # channels of 1, 3, 5, 125 and 1025 packs (the pack -> channel lookup multiplies by a
          # rounded-up reciprocal of the packs per channel instead of dividing)
          (4, 12, (8,), 3), (4, 12, (4,), 3), (3, 10, (24,), 5), (2, 6, (5, 8), 2), (2, 9, (1000,), 3),
          (1, 6, (8200,), 2),
          # rows of whole packs whose channels are not (packs straddle two channels): 7x7, 14x14
          # and 27x27 maps, a channel barely longer than a pack, 64, 65 and 512 channels a group (the most the
          # straddling kernels take) and 520 (general kernels)
          (4, 64, (7, 7), 8), (2, 64, (14, 14), 2), (2, 128, (7, 7), 2), (2, 130, (7, 7), 2),
          (1, 16, (27, 27), 1), (3, 8, (9,), 1), (2, 24, (3, 4), 3), (70, 32, (7, 7), 4),
          (2, 512, (7, 7), 1), (1, 1040, (7, 7), 2),
          # 16-bit rows that fill an exact layout, channels of whole runs of 64 packs (32x32 and
          # 64x64 maps with 10, 20, 30 and 60 channels a group; 10 at 64x64 is above): 256 x 5
          # (backward), 512 x 5, 768 x 5, 960 x 8
          (3, 10, (32, 32), 1), (2, 40, (32, 32), 2), (2, 60, (32, 32), 2), (2, 120, (32, 32), 2),
          # from 8192 samples under few channels the backward's second stage first folds its
          # partial rows (one a sample) in place, 512 at a time: 16 folds and a ragged 17th
          (8269, 24, (), 4), (8200, 16, (3,), 2)]
CASES = load_golden("aten_cpu_group_norm.npz")


def _mk(N, C, sp, dtype, seed, wdtype=None):
    g = gen(seed)
    x = (0.5 + torch.randn((N, C) + tuple(sp), generator=g)).to(dtype)
    dy = torch.randn((N, C) + tuple(sp), generator=g).to(dtype)
    wdt = dtype if wdtype is None else wdtype
    gamma = (1 + 0.1 * torch.randn(C, generator=g)).to(wdt)
    beta = (0.1 * torch.randn(C, generator=g)).to(wdt)
    return x, dy, gamma, beta


def _hxw(sp):
    n = 1
    for s in sp:
        n *= s
    return n


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_group_norm_fwd_bwd(cabi, oracle, gpu, dtype, shape, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    N, C, sp, G = shape
    HxW = _hxw(sp)
    print("case group_norm", dtype, shape, mixed, flush=True)
    x, dy, gamma, beta = _mk(N, C, sp, dtype, 71, torch.float32 if mixed else None)
    y, mean, rstd = cabi.group_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), G, 1e-5)
    oy, om, orr = oracle.group_norm_fwd(to_np32(x), G, to_np32(gamma), to_np32(beta), 1e-5)
    assert y.dtype == dtype and mean.dtype == gamma.dtype and rstd.dtype == gamma.dtype
    assert mean.shape == (N, G) and rstd.shape == (N, G)
    assert_close(y, oy, dtype, "y")
    assert_close(mean, om, gamma.dtype, "mean")
    assert_close(rstd, orr, gamma.dtype, "rstd")
    cy, cm, cr = torch.ops.aten.native_group_norm(x.float(), gamma.float(), beta.float(), N, C, HxW, G, 1e-5)
    # the CPU kernel evaluates y = x*a + (beta - a*mean), a = rstd*gamma: two products of size
    # |x*a| that cancel, each rounded to float32 (it shows when a group's variance is ~0)
    a_abs = (cr.reshape(N, G, 1, 1) * gamma.float().reshape(1, G, C // G, 1)).abs()
    cpu_slack = (4 * 2.0 ** -24 * a_abs * x.float().reshape(N, G, C // G, HxW).abs()).reshape(x.shape)
    assert_close(y, cy, dtype, "y vs ATen CPU", slack=cpu_slack)
    assert_close(mean, cm, gamma.dtype, "mean vs ATen CPU")
    assert_close(rstd, cr, gamma.dtype, "rstd vs ATen CPU")
    # backward consumes the device's own saved statistics (16-bit when the op returns them so)
    dx, dg, db = cabi.group_norm_bwd(dy.to(gpu), x.to(gpu), mean, rstd, gamma.to(gpu), G)
    odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), G, to_np32(mean), to_np32(rstd),
                                          to_np32(gamma))
    assert dx.dtype == dtype and dg.dtype == gamma.dtype and db.dtype == gamma.dtype
    assert_close(dx, odx, dtype, "dx")
    # dgamma/dbeta are float32 sums over N*HxW terms: allow the sum's own rounding
    D = C // G
    xh = (x.float().reshape(N, G, D, HxW) - mean.cpu().float().reshape(N, G, 1, 1)) * \
        rstd.cpu().float().reshape(N, G, 1, 1)
    dyf = dy.float().reshape(N, G, D, HxW)
    sl_g = colsum_slack((dyf * xh).permute(0, 3, 1, 2).reshape(N * HxW, C))
    sl_b = colsum_slack(dyf.permute(0, 3, 1, 2).reshape(N * HxW, C))
    assert_close(dg, odg, gamma.dtype, "dgamma", slack=sl_g)
    assert_close(db, odb, gamma.dtype, "dbeta", slack=sl_b)
    # (one value per group: every CPU gradient is rounding noise of terms that cancel, times
    # rstd = 1/sqrt(eps); the exact answers, which the oracle gives, are 0)
    if dtype == torch.float32 and (C // G) * HxW > 1:
        cdx, cdg, cdb = torch.ops.aten.native_group_norm_backward(
            dy, x, mean.cpu(), rstd.cpu(), gamma, N, C, HxW, G, [True, True, True])
        # the CPU kernel's dx = c1*dy + c2*x + c3 cancels terms of size |rstd*gamma*dy|
        dx_slack = (8 * 2.0 ** -24 * a_abs * dy.float().reshape(N, G, C // G, HxW).abs()).reshape(x.shape)
        assert_close(dx, cdx, dtype, "dx vs ATen CPU", slack=dx_slack, scale=2.0)
        assert_close(dg, cdg, dtype, "dgamma vs ATen CPU", slack=2 * sl_g, scale=2.0)
        assert_close(db, cdb, dtype, "dbeta vs ATen CPU", slack=2 * sl_b, scale=2.0)


@pytest.mark.parametrize("case", sorted(CASES))
def test_golden_vectors(cabi, gpu, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    G = int(case.split("g")[-1])
    variants = [("gn", c["gamma"], c["beta"])]
    if dt != torch.float32:
        variants.append(("gnmix", c["gamma"].float(), c["beta"].float()))
    for pre, gk, bk in variants:
        y, mean, rstd = cabi.group_norm_fwd(c["x"].to(gpu), gk.to(gpu), bk.to(gpu), G, 1e-5)
        assert mean.dtype == c[pre + "_mean"].dtype
        assert_close(y, c[pre + "_y"], dt, case + " y")
        assert_close(mean, c[pre + "_mean"], mean.dtype, case + " mean")
        assert_close(rstd, c[pre + "_rstd"], mean.dtype, case + " rstd")
        dx, dg, db = cabi.group_norm_bwd(c["dy"].to(gpu), c["x"].to(gpu), c[pre + "_mean"].to(gpu),
                                         c[pre + "_rstd"].to(gpu), gk.to(gpu), G)
        assert_close(dx, c[pre + "_dx"], dt, case + " dx", scale=2.0)
        assert_close(dg, c[pre + "_dgamma"], dt, case + " dgamma", scale=4.0)
        assert_close(db, c[pre + "_dbeta"], dt, case + " dbeta", scale=4.0)


def test_edge_cases(cabi, oracle, gpu):
    # constant slabs give beta bit for bit, mean the constant, rstd 1/sqrt(eps)
    for dtype in DTYPES:
        for (C, G, sp) in ((8, 2, (16,)), (6, 3, (5,)), (4, 4, (1024,)), (2, 1, (100000,))):
            cval = torch.tensor(-3.3333).to(dtype)
            x = torch.full((3, C) + sp, float(cval)).to(dtype).to(gpu)
            gamma = (1 + 0.1 * torch.randn(C, generator=gen(1))).to(dtype).to(gpu)
            beta = (0.1 * torch.randn(C, generator=gen(2))).to(dtype).to(gpu)
            y, mean, rstd = cabi.group_norm_fwd(x, gamma, beta, G, 1e-5)
            assert torch.equal(mean.cpu().float(), torch.full((3, G), float(cval)))
            assert torch.equal(y, beta.view(1, C, 1).expand_as(y)), (dtype, C, G, sp)
    # absent weight / bias == ones / zeros; output masks
    x = torch.randn(4, 12, 9, 5, generator=gen(3)).to(gpu)
    dy = torch.randn(4, 12, 9, 5, generator=gen(4)).to(gpu)
    ones, zeros = torch.ones(12, device=gpu), torch.zeros(12, device=gpu)
    y0, m0, r0 = cabi.group_norm_fwd(x, None, None, 3, 1e-5)
    y1, m1, r1 = cabi.group_norm_fwd(x, ones, zeros, 3, 1e-5)
    y2, _, _ = cabi.group_norm_fwd(x, ones, None, 3, 1e-5)
    assert torch.equal(y0, y1) and torch.equal(y0, y2) and torch.equal(m0, m1) and torch.equal(r0, r1)
    dx, dg, db = cabi.group_norm_bwd(dy, x, m0, r0, ones, 3)
    dx0, _, _ = cabi.group_norm_bwd(dy, x, m0, r0, None, 3, want=(True, False, False))
    assert torch.equal(dx, dx0)
    for want in [(False, True, True), (False, True, False), (False, False, True), (True, True, False)]:
        a, b, c = cabi.group_norm_bwd(dy, x, m0, r0, ones, 3, want=want)
        assert (a is None) == (not want[0]) and (b is None) == (not want[1]) and (c is None) == (not want[2])
        assert (a is None or torch.equal(a, dx)) and (b is None or torch.equal(b, dg)) and \
            (c is None or torch.equal(c, db))
    # run-to-run determinism of the channel sums
    for _ in range(3):
        _, dg2, db2 = cabi.group_norm_bwd(dy, x, m0, r0, ones, 3)
        assert torch.equal(dg2, dg) and torch.equal(db2, db)
    # eps 0.5 and -0.5 (test/regressions/test_group_norm.py:27-28), empty batch
    xs = torch.randn(2, 6, 3, generator=gen(5)).half()
    for eps in (0.5, -0.5):
        y, mean, rstd = cabi.group_norm_fwd(xs.to(gpu), None, None, 2, eps)
        cy, cm, cr = torch.ops.aten.native_group_norm(xs.float(), None, None, 2, 6, 3, 2, eps)
        ok = torch.isfinite(cy)
        assert torch.equal(torch.isfinite(y.cpu().float()), ok)
        assert_close(torch.where(ok, y.cpu().float(), 0), torch.where(ok, cy, 0), torch.float16, "y eps=%g" % eps)
    e = torch.empty(0, 2, device=gpu)
    y, mean, rstd = cabi.group_norm_fwd(e, None, None, 1, 1e-5)
    assert y.shape == (0, 2) and mean.shape == (0, 1)


def test_exact_layouts_many_rows_absent_weights_and_special_rows(cabi, oracle, gpu):
    """The 16-bit kernels for rows that fill a layout of whole wavefronts exactly, channels of whole
    runs of 64 packs (gn_fwd_exact_kernel / gn_bwd_exact_kernel): more rows than the resident grid
    has workgroups, weights absent, misaligned weight pointers (a scalar load takes the aligned word
    around a 16-bit weight), constant and non-finite rows, dX alone and the channel sums alone (the
    latter is the general kernel's: the two must agree), run-to-run determinism."""
    bf = torch.bfloat16
    # [25, 640, 32, 32] / 32: 800 rows of 512 x 5 packs (forward grid 768, backward 512);
    # [66, 320, 32, 32] / 32: 2112 rows of 256 x 5 packs (backward grid 2048; general forward)
    for (N, C, sp, G, lay) in ((25, 640, (32, 32), 32, (512, 5)), (66, 320, (32, 32), 32, (256, 5))):
        HxW = _hxw(sp)
        for bwd in (0, 1):
            p = cabi.group_norm_plan(bwd, N, C, HxW, G, cabi.BF16)
            if bwd or lay != (256, 5):
                assert (p["lanes_per_row"], p["packs_per_lane"]) == lay and p["grid_blocks"] < N * G, p
        print("case group_norm exact layouts, many rows", (N, C, sp, G), flush=True)
        x, dy, gamma, beta = _mk(N, C, sp, bf, 75)
        x[1, :C // G] = 2.5                      # a constant row
        x[2, C // G, 3, 3] = float("inf")        # a row with an inf: NaN statistics
        x[3, 2 * (C // G), 0, 1] = float("nan")
        xg, dyg, gg, bg = x.to(gpu), dy.to(gpu), gamma.to(gpu), beta.to(gpu)
        y, mean, rstd = cabi.group_norm_fwd(xg, gg, bg, G, 1e-5)
        oy, om, orr = oracle.group_norm_fwd(to_np32(x), G, to_np32(gamma), to_np32(beta), 1e-5)
        oy = torch.as_tensor(oy).float().reshape(x.shape)
        orr = torch.as_tensor(orr).float().reshape(N, G)
        fin = torch.isfinite(oy)
        assert torch.equal(torch.isfinite(y.cpu().float()), fin)
        assert_close(torch.where(fin, y.cpu().float(), 0), torch.where(fin, oy, 0), bf, "y")
        assert torch.equal(y[1, :C // G].cpu(), beta[:C // G].view(-1, 1, 1).expand(C // G, *sp))
        assert bool(torch.isnan(mean[2, 1])) and bool(torch.isnan(rstd[2, 1])) and bool(torch.isnan(mean[3, 2]))
        okr = torch.isfinite(rstd.cpu().float())
        assert torch.equal(okr, torch.isfinite(orr))
        assert_close(torch.where(okr, rstd.cpu().float(), 0), torch.where(okr, orr, 0), bf, "rstd")
        # backward on finite inputs
        x[2, C // G, 3, 3] = 1.0
        x[3, 2 * (C // G), 0, 1] = -1.0
        xg = x.to(gpu)
        y, mean, rstd = cabi.group_norm_fwd(xg, gg, bg, G, 1e-5)
        dx, dg, db = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, G)
        odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), G, to_np32(mean), to_np32(rstd),
                                              to_np32(gamma))
        assert_close(dx, odx, bf, "dx")
        assert_close(dg, odg, bf, "dgamma")
        assert_close(db, odb, bf, "dbeta")
        dx1, none1, none2 = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, G, want=(True, False, False))
        assert none1 is None and none2 is None and torch.equal(dx1, dx)
        none0, dg1, db1 = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, G, want=(False, True, True))
        assert none0 is None
        assert_close(dg1, odg, bf, "dgamma alone")
        assert_close(db1, odb, bf, "dbeta alone")
        dx2, dg2, db2 = cabi.group_norm_bwd(dyg, xg, mean, rstd, gg, G)
        assert torch.equal(dx2, dx) and torch.equal(dg2, dg) and torch.equal(db2, db)
    # absent weights == ones / zeros, and weights that start on an odd 16-bit element
    for wdt in (bf, torch.float32):
        N, C, sp, G = 3, 40, (32, 32), 2
        x, dy, gamma, beta = _mk(N, C, sp, bf, 76, wdt)
        xg, dyg = x.to(gpu), dy.to(gpu)
        ones, zeros = torch.ones(C, device=gpu, dtype=wdt), torch.zeros(C, device=gpu, dtype=wdt)
        y1, m1, r1 = cabi.group_norm_fwd(xg, ones, zeros, G, 1e-5)
        y2, m2, _ = cabi.group_norm_fwd(xg, ones, None, G, 1e-5)
        assert torch.equal(y1, y2) and torch.equal(m1, m2)
        if wdt == bf:
            y0, m0, r0 = cabi.group_norm_fwd(xg, None, None, G, 1e-5)
            assert torch.equal(y0, y1) and torch.equal(m0, m1) and torch.equal(r0, r1)
        dx0, _, _ = cabi.group_norm_bwd(dyg, xg, m1, r1, None, G, want=(True, False, False))
        dx1, _, _ = cabi.group_norm_bwd(dyg, xg, m1, r1, ones, G)
        assert torch.equal(dx0, dx1)
        go, bo = offset_view(gamma.to(gpu), 1), offset_view(beta.to(gpu), 1)
        ya, ma, ra = cabi.group_norm_fwd(xg, gamma.to(gpu), beta.to(gpu), G, 1e-5)
        yb, mb, rb = cabi.group_norm_fwd(xg, go, bo, G, 1e-5)
        assert torch.equal(ya, yb) and torch.equal(ma, mb)
        # statistics that start on an odd element as well
        da = cabi.group_norm_bwd(dyg, xg, ma, ra, gamma.to(gpu), G)
        dbb = cabi.group_norm_bwd(dyg, xg, offset_view(ma.reshape(-1), 1).reshape(ma.shape),
                                  offset_view(ra.reshape(-1), 1).reshape(ra.shape), go, G)
        for u, v in zip(da, dbb):
            assert torch.equal(u, v)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_forced_variants_multipass_and_misaligned(cabi, oracle, gpu, dtype):
    dt = cabi.dtype_code(dtype)
    for (N, C, sp, G) in ((3, 8, (32,), 2), (2, 6, (25,), 3), (2, 16, (256,), 4), (1, 4, (2500,), 2)):
        HxW = _hxw(sp)
        x, dy, gamma, beta = _mk(N, C, sp, dtype, 72)
        oy, om, orr = oracle.group_norm_fwd(to_np32(x), G, to_np32(gamma), to_np32(beta), 1e-5)
        odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), G, om, orr, to_np32(gamma))
        xg, dyg, gg, bg = (offset_view(t.to(gpu), 1) for t in (x, dy, gamma, beta))
        mean_g = offset_view(torch.from_numpy(om).to(dtype).to(gpu), 1)
        rstd_g = offset_view(torch.from_numpy(orr).to(dtype).to(gpu), 1)
        odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), G, to_np32(mean_g), to_np32(rstd_g),
                                              to_np32(gamma))
        tried = 0
        for op, bwd in ((cabi.OP_GROUP_NORM_FWD, False), (cabi.OP_GROUP_NORM_BWD, True)):
            layouts = [(-1, 0)]
            for Gl in (8, 16, 32, 64, 128, 256, 512, 1024):
                for V in (1, 2, 4, 8, 16):
                    cabi.set_override(op, Gl, V)
                    try:
                        cabi.group_norm_plan(bwd, N, C, HxW, G, dt)
                        layouts.append((Gl, V))
                    except RuntimeError:
                        pass
            for (Gl, V) in layouts:
                print("forced group_norm", dtype, (N, C, sp, G), "bwd" if bwd else "fwd", Gl, V, flush=True)
                cabi.set_override(op, Gl, V)
                if not bwd:
                    y, mean, rstd = cabi.group_norm_fwd(xg, gg, bg, G, 1e-5, y=offset_view(torch.empty_like(xg), 3))
                    assert_close(y, oy, dtype, "y G=%d V=%d" % (Gl, V))
                    assert_close(mean, om, dtype, "mean")
                    assert_close(rstd, orr, dtype, "rstd")
                else:
                    dx, dg, db = cabi.group_norm_bwd(dyg, xg, mean_g, rstd_g, gg, G,
                                                     dx=offset_view(torch.empty_like(xg), 3))
                    assert_close(dx, odx, dtype, "dx G=%d V=%d" % (Gl, V))
                    assert_close(dg, odg, dtype, "dgamma G=%d V=%d" % (Gl, V), scale=2.0)
                    assert_close(db, odb, dtype, "dbeta G=%d V=%d" % (Gl, V), scale=2.0)
                tried += 1
            cabi.set_override(op)
        assert tried >= 4


def test_host_ops_and_aten_override(pkg, ops, gpu):
    """torch.ops.mi355x.native_group_norm(_backward) with ATen's schemas, then F.group_norm with
    autograd after the explicit opt-in, against the CPU (test_layer_norm_group_norm_align.py:81-154
    in the reference: 1-d / 2-d inputs, small and large batch)."""
    for dtype in DTYPES:
        x, dy, gamma, beta = _mk(3, 12, (6, 5), dtype, 73)
        y, mean, rstd = ops.native_group_norm(x.to(gpu), gamma.to(gpu), beta.to(gpu), 3, 12, 30, 4, 1e-5)
        cy, cm, cr = torch.ops.aten.native_group_norm(x.float(), gamma.float(), beta.float(), 3, 12, 30, 4, 1e-5)
        assert y.dtype == dtype and mean.dtype == dtype and mean.shape == (3, 4)
        assert_close(y, cy, dtype, "y")
        assert_close(mean, cm, dtype, "mean")
        assert_close(rstd, cr, dtype, "rstd")
        dx, dg, db = ops.native_group_norm_backward(dy.to(gpu), x.to(gpu), mean, rstd, gamma.to(gpu), 3, 12,
                                                    30, 4, [True, True, True])
        cdx, cdg, cdb = torch.ops.aten.native_group_norm_backward(
            dy.float(), x.float(), mean.cpu().float(), rstd.cpu().float(), gamma.float(), 3, 12, 30, 4,
            [True, True, True])
        assert_close(dx, cdx, dtype, "dx", scale=2.0)
        assert_close(dg, cdg, dtype, "dgamma", scale=4.0)
        assert_close(db, cdb, dtype, "dbeta", scale=4.0)
        a, b, c = ops.native_group_norm_backward(dy.to(gpu), x.to(gpu), mean, rstd, None, 3, 12, 30, 4,
                                                 [True, False, False])
        assert b is None and c is None
    # mixed: bfloat16 rows with float32 weights -> float32 statistics
    x, dy, gamma, beta = _mk(2, 8, (16,), torch.bfloat16, 74, torch.float32)
    y, mean, rstd = ops.native_group_norm(x.to(gpu), gamma.to(gpu), beta.to(gpu), 2, 8, 16, 2, 1e-5)
    assert y.dtype == torch.bfloat16 and mean.dtype == torch.float32
    # empty batch (test/xpu/test_nn_xpu.py:11662-11667)
    e = torch.empty(0, 4, 3, device=gpu)
    y, mean, rstd = ops.native_group_norm(e, None, None, 0, 4, 3, 2, 1e-5)
    assert y.shape == (0, 4, 3) and mean.shape == (0, 2)
    dx, dg, db = ops.native_group_norm_backward(e, e, mean, rstd, torch.ones(4, device=gpu), 0, 4, 3, 2,
                                                [True, True, True])
    assert dx.shape == (0, 4, 3) and bool((dg == 0).all()) and bool((db == 0).all())
    # non-contiguous (channels-last) input is accepted and gives a contiguous result
    xc = torch.randn(2, 8, 6, 6, generator=gen(75)).to(gpu).contiguous(memory_format=torch.channels_last)
    y, _, _ = ops.native_group_norm(xc, None, None, 2, 8, 36, 4, 1e-5)
    assert y.is_contiguous()
    assert_close(y, torch.ops.aten.native_group_norm(xc.cpu().contiguous(), None, None, 2, 8, 36, 4, 1e-5)[0],
                 torch.float32, "channels-last input")

    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        pkg.override_aten_ops()
    for dtype, N, C, G, sp in ((torch.float32, 64, 32, 4, ()), (torch.float32, 256, 32, 4, ()),
                               (torch.float16, 256, 32, 4, ()), (torch.bfloat16, 256, 32, 4, ()),
                               (torch.float32, 64, 32, 4, (16,)), (torch.float32, 256, 32, 4, (16,)),
                               (torch.float16, 256, 32, 4, (16,)), (torch.float32, 4, 64, 32, (24, 24))):
        print("case F.group_norm", dtype, N, C, G, sp, flush=True)
        x, dy, gamma, beta = _mk(N, C, sp, dtype, 76)

        def run(dev, upcast):
            cast = (lambda t: t.float()) if upcast else (lambda t: t)
            xs, ws, bs = (cast(t).detach().clone().to(dev).requires_grad_() for t in (x, gamma, beta))
            out = F.group_norm(xs, G, ws, bs, 1e-5)
            out.backward(cast(dy).to(dev))
            return out, xs.grad, ws.grad, bs.grad

        got, ref = run(gpu, False), run("cpu", True)
        for a, r, nm in zip(got, ref, ("out", "dx", "dw", "db")):
            assert a.dtype == dtype
            assert_close(a, r, dtype, "F.group_norm %s" % nm, scale=4.0)
