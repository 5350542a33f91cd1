"""LayerNorm / RMSNorm forward rows of 5 to 16 packs a lane on 1024 lanes (16-bit rows of 32776 to
131072 elements, float32 rows of 16388 to 65536): the register-resident kernel
(norm_fwd_resident_kernel) with gamma / beta held in registers where they fit and loaded per pack
of the output where they do not.  The reference serves such rows with its one-work-group-per-row
forward (RowwiseMomentsFunctor + LayerNormForwardKernelFunctor,
src/ATen/native/xpu/sycl/LayerNormKernels.cpp:197-260, 590-660 behind the dispatch at :1121-1163).
Checked through the extern "C" ABI against the CPU oracle at the family's tolerances (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2), against the multi-pass kernel forced on the
same inputs, with and without weights, with float32 weights beside 16-bit rows, with the residual
add and the output cast fused in, and for run-to-run determinism."""
import pytest
import torch

from helpers import assert_close, colsum_slack, gen, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
NAME = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}
# packs a lane -> row length in packs of 1024 lanes (the last two leave lanes without a pack, or
# with packs outside the row)
PACKS = [(5, 5 * 1024), (6, 6 * 1024), (6, 5 * 1024 + 1), (8, 7 * 1024), (8, 8 * 1024),
         (10, 9 * 1024 + 512), (12, 12 * 1024), (16, 12 * 1024 + 4), (16, 16 * 1024)]


def _mk(M, N, dtype, wdtype, seed, shift=0.5):
    g = gen(seed)
    x = (shift + torch.randn(M, N, generator=g)).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
    beta = (0.1 * torch.randn(N, generator=g)).to(wdtype)
    return x, gamma, beta


def _multi_pass(cabi, op, fn):
    try:
        cabi.set_override(op, -1, 1)
        return fn()
    finally:
        cabi.clear_overrides()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_forward_against_oracle_and_multi_pass_kernel(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    E = 4 if dtype == torch.float32 else 8
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (V, packs) in enumerate(PACKS):
        # (from 10 packs a lane, fewer rows than half the compute units are split over workgroups)
        M, N = (5 if V < 10 else 128) + i, packs * E
        print("case long rows", dtype, mixed, (M, N), flush=True)
        for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD):
            p = cabi.plan(op, M, N, code, wcode)
            assert (p["resident"], p["lanes_per_row"], p["packs_per_lane"]) == (1, 1024, V), p
        x, gamma, beta = _mk(M, N, dtype, wdtype, 1400 + i)
        xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
        what = "[%d, %d] %s" % (M, N, dtype)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "layer_norm y " + what)
        assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
        sy, sm, sr = _multi_pass(cabi, cabi.OP_LAYER_NORM_FWD,
                                 lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
        assert_close(y, to_np32(sy), dtype, "layer_norm y against the multi-pass kernel " + what)
        assert_close(rstd, to_np32(sr), torch.float32, "rstd against the multi-pass kernel " + what)
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
        roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "rms_norm y " + what)
        assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
        # a second run gives the same bits
        y2, mean2, rstd2 = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        ry2, rr2 = cabi.rms_norm_fwd(xg, gg, 1e-6)
        for a, b in ((y, y2), (mean, mean2), (rstd, rstd2), (ry, ry2), (rr, rr2)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
        if i % 3 == 0:
            # no weights
            y0, _, _ = cabi.layer_norm_fwd(xg, None, None, 1e-5)
            oy0, _, _ = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, 1e-5)
            assert_close(y0, oy0, dtype, "layer_norm without weights " + what)
            ry0, _ = cabi.rms_norm_fwd(xg, None, 1e-6)
            roy0, _ = oracle.rms_norm_fwd(to_np32(x), (N,), None, 1e-6)
            assert_close(ry0, roy0, dtype, "rms_norm without weights " + what)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_constant_and_shifted_rows(cabi, oracle, gpu, dtype):
    """A constant row gives beta bit for bit; rows far from zero keep their statistics."""
    E = 4 if dtype == torch.float32 else 8
    N = 6 * 1024 * E
    x, gamma, beta = _mk(6, N, dtype, dtype, 1450, shift=100.0)
    x[1] = 3.0
    x[2, :3] = 0.0  # the head of the row is not representative of it
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    assert torch.equal(y[1].cpu(), beta)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    ok = [0, 2, 3, 4, 5]
    assert_close(y[ok], oy[ok], dtype, "shifted rows y")
    assert_close(mean[ok], om.reshape(-1)[ok], torch.float32, "shifted rows mean")
    assert_close(rstd[ok], orr.reshape(-1)[ok], dtype, "shifted rows rstd")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_fused_add_and_cast(cabi, oracle, gpu, dtype):
    """Residual add -> norm on rows of 5 to 12 packs a lane (float32 LayerNorm: to 10), and
    float32 rows written out in bf16; rows beyond that take the multi-pass kernel and agree."""
    E = 4 if dtype == torch.float32 else 8
    for i, packs in enumerate((5 * 1024, 8 * 1024, 10 * 1024, 12 * 1024, 16 * 1024)):
        M, N = (4 if packs < 10 * 1024 else 128) + i, packs * E
        print("case long rows fused add", dtype, (M, N), flush=True)
        g = gen(1460 + i)
        x = torch.randn(M, N, generator=g).to(dtype)
        res = (2 * torch.randn(M, N, generator=g)).to(dtype)
        gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
        beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
        xg, rg, gg, bg = x.to(gpu), res.to(gpu), gamma.to(gpu), beta.to(gpu)
        h_cpu = x + res
        y, h, mean, rstd = cabi.add_layer_norm_fwd(xg, rg, gg, bg, 1e-5)
        assert torch.equal(h.cpu(), h_cpu)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(h_cpu), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "add_layer_norm y")
        assert_close(rstd, orr.reshape(-1), torch.float32, "add_layer_norm rstd")
        ry, rh, rr = cabi.add_rms_norm_fwd(xg, rg, gg, 1e-6)
        assert torch.equal(rh.cpu(), h_cpu)
        roy, ror = oracle.rms_norm_fwd(to_np32(h_cpu), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "add_rms_norm y")
        assert_close(rr, ror.reshape(-1), torch.float32, "add_rms_norm rstd")
        if dtype == torch.float32:
            cy, _, _, crstd = cabi.add_layer_norm_fwd(xg, None, gg, bg, 1e-5, y_dtype=torch.bfloat16)
            oy0, _, orr0 = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
            assert_close(cy, oy0, torch.bfloat16, "layer_norm with bf16 output")
            assert_close(crstd, orr0.reshape(-1), torch.float32, "rstd with bf16 output")
            ay, ah, arr = cabi.add_rms_norm_fwd(xg, rg, gg, 1e-6, y_dtype=torch.bfloat16)
            assert torch.equal(ah.cpu(), h_cpu)
            assert_close(ay, roy, torch.bfloat16, "add_rms_norm with bf16 output")


def test_host_op_on_a_long_hidden_size(ops, gpu):
    """aten-signature native_layer_norm on [2, 3, 49152] bf16 (6 packs a lane)."""
    x = (0.3 + torch.randn(2, 3, 49152, generator=gen(1470))).bfloat16()
    w = (1 + 0.1 * torch.randn(49152, generator=gen(1471))).bfloat16()
    b = (0.1 * torch.randn(49152, generator=gen(1472))).bfloat16()
    y, mean, rstd = ops.native_layer_norm(x.to(gpu), [49152], w.to(gpu), b.to(gpu), 1e-5)
    ref = torch.nn.functional.layer_norm(x.float(), [49152], w.float(), b.float(), 1e-5)
    assert_close(y, to_np32(ref), torch.bfloat16, "native_layer_norm long rows")
    assert mean.shape == (2, 3, 1) and rstd.shape == (2, 3, 1)


# ---- backward: 16-bit rows of 16392 .. 32768 elements, dgamma sums in LDS ------------------

BWD_N = [(3, 16392), (3, 18432), (3, 20480), (3, 24576), (4, 24584), (4, 28672), (4, 32768)]


def _bwd_case(cabi, oracle, gpu, M, N, dtype, wdtype, seed, rms):
    g = gen(seed)
    x = (0.3 + torch.randn(M, N, generator=g)).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
    xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
    what = "[%d, %d] %s / %s" % (M, N, dtype, wdtype)
    # float32 column sums: the summation's own rounding is allowed for (helpers.colsum_slack)
    wide = wdtype == torch.float32
    if rms:
        _, rstd = cabi.rms_norm_fwd(xg, gg, 1e-6)
        sl = colsum_slack(dy.double() * x.double() * rstd.cpu().double().reshape(M, 1)) if wide else None
        dx, dg = cabi.rms_norm_bwd(dyg, xg, rstd, gg)
        odx, odg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rstd), to_np32(gamma))
        assert_close(dx, odx, dtype, "rms_norm dx " + what)
        assert_close(dg, odg, wdtype, "rms_norm dgamma " + what, slack=sl)
        try:
            cabi.set_override(cabi.OP_RMS_NORM_BWD, -1, 1)
            mdx, mdg = cabi.rms_norm_bwd(dyg, xg, rstd, gg)
        finally:
            cabi.clear_overrides()
        assert_close(dx, to_np32(mdx), dtype, "rms_norm dx against the multi-pass kernels " + what)
        # the same bits on a second run, and with only one of the two results asked for
        dx2, dg2 = cabi.rms_norm_bwd(dyg, xg, rstd, gg)
        assert torch.equal(dx2.view(torch.uint8), dx.view(torch.uint8))
        assert torch.equal(dg2.view(torch.uint8), dg.view(torch.uint8))
        dx3, none = cabi.rms_norm_bwd(dyg, xg, rstd, gg, want=(True, False))
        assert none is None and torch.equal(dx3.view(torch.uint8), dx.view(torch.uint8))
        none, dg3 = cabi.rms_norm_bwd(dyg, xg, rstd, gg, want=(False, True))
        assert none is None and torch.equal(dg3.view(torch.uint8), dg.view(torch.uint8))
    else:
        beta = (0.1 * torch.randn(N, generator=g)).to(wdtype)
        _, mean, rstd = cabi.layer_norm_fwd(xg, gg, beta.to(gpu), 1e-5)
        xhat = (x.double() - mean.cpu().double().reshape(M, 1)) * rstd.cpu().double().reshape(M, 1)
        sl = colsum_slack(dy.double() * xhat) if wide else None
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                              to_np32(rstd), to_np32(gamma))
        assert_close(dx, odx, dtype, "layer_norm dx " + what)
        assert_close(dg, odg, wdtype, "layer_norm dgamma " + what, slack=sl)
        assert_close(db, odb, wdtype, "layer_norm dbeta " + what,
                     slack=colsum_slack(dy.double()) if wide else None)
        dx2, dg2, db2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
        for a, b in ((dx, dx2), (dg, dg2), (db, db2)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_backward_with_dgamma_sums_in_lds(cabi, oracle, gpu, dtype, mixed):
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (V, N) in enumerate(BWD_N):
        # one row, fewer rows than workgroups, and more rows than the 256 workgroups of the grid
        for M in ((1, 37, 300) if i in (1, 6) else (5 + i,)):
            print("case long rows backward", dtype, mixed, (M, N), flush=True)
            p = cabi.plan(cabi.OP_RMS_NORM_BWD, M, N, code, wcode)
            # (the RMSNorm with 16-bit weights holds rows of up to 2560 packs in registers alone,
            # on 512 lanes x 5 packs)
            want = (1, 512, 5) if (N <= 20480 and not mixed) else (1, 1024, V)
            # with fp32 weights, rows that fill a layout of whole wavefronts exactly take it
            if mixed:
                want = {18432: (1, 768, 3), 20480: (1, 640, 4)}.get(N, want)
            assert (p["resident"], p["lanes_per_row"], p["packs_per_lane"]) == want, p
            p = cabi.plan(cabi.OP_LAYER_NORM_BWD, M, N, code, wcode)
            # the LayerNorm backward with four packs a lane keeps the multi-pass kernels
            assert p["resident"] == (1 if V == 3 else 0), p
            _bwd_case(cabi, oracle, gpu, M, N, dtype, wdtype, 1480 + i, True)
            _bwd_case(cabi, oracle, gpu, M, N, dtype, wdtype, 1490 + i, False)


def test_fused_add_backward_on_long_rows(cabi, oracle, gpu):
    """The residual path's gradient added to dx, bf16 rows of 20480 and 32768 elements."""
    for i, N in enumerate((20480, 32768)):
        M = 9 + i
        g = gen(1495 + i)
        h = torch.randn(M, N, generator=g).bfloat16()
        dy = torch.randn(M, N, generator=g).bfloat16()
        dh_in = torch.randn(M, N, generator=g).bfloat16()
        gamma = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16()
        hg, dyg, dhg, gg = h.to(gpu), dy.to(gpu), dh_in.to(gpu), gamma.to(gpu)
        _, rstd = cabi.rms_norm_fwd(hg, gg, 1e-6)
        dh, dg = cabi.add_rms_norm_bwd(dyg, dhg, hg, rstd, gg)
        odh, odg = oracle.add_rms_norm_bwd(to_np32(dy), to_np32(dh_in), to_np32(h), (N,),
                                           to_np32(rstd), to_np32(gamma))
        assert_close(dh, odh, torch.bfloat16, "add_rms_norm dh [%d, %d]" % (M, N))
        assert_close(dg, odg, torch.bfloat16, "add_rms_norm dgamma [%d, %d]" % (M, N))
        _, mean, rstd = cabi.layer_norm_fwd(hg, gg, gg, 1e-5)
        dh, dg, db = cabi.add_layer_norm_bwd(dyg, dhg, hg, mean, rstd, gg)
        odh, odg, odb = oracle.add_layer_norm_bwd(to_np32(dy), to_np32(dh_in), to_np32(h), (N,),
                                                  to_np32(mean), to_np32(rstd), to_np32(gamma))
        assert_close(dh, odh, torch.bfloat16, "add_layer_norm dh [%d, %d]" % (M, N))
        assert_close(dg, odg, torch.bfloat16, "add_layer_norm dgamma [%d, %d]" % (M, N))
        assert_close(db, odb, torch.bfloat16, "add_layer_norm dbeta [%d, %d]" % (M, N))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_forward_rows_of_5_and_6_packs_on_512_lanes(cabi, oracle, gpu, dtype, mixed):
    """16-bit forward rows of 16392 .. 24576 elements (hidden 18432, 20480, 24576)."""
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (V, N) in enumerate(((5, 16392), (5, 18432), (5, 20480), (6, 20488), (6, 24576))):
        M = 7 + i
        print("case 512-lane long rows", dtype, mixed, (M, N), flush=True)
        p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, wcode)
        assert (p["resident"], p["lanes_per_row"], p["packs_per_lane"]) == (1, 512, V), p
        x, gamma, beta = _mk(M, N, dtype, wdtype, 1520 + i)
        xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        what = "[%d, %d] %s" % (M, N, dtype)
        assert_close(y, oy, dtype, "layer_norm y " + what)
        assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
        roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "rms_norm y " + what)
        assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
        y2, _, _ = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        assert torch.equal(y2.view(torch.uint8), y.view(torch.uint8))
