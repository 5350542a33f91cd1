"""Short LayerNorm / RMSNorm rows (at most one wavefront of 16-byte packs): the one-pack-a-lane
layouts on 8..64 lanes that the backward always takes and the forward takes for tensors that do
not start on a 128-byte line, through the extern "C" ABI against the CPU oracle.  Tolerances as
everywhere: float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2."""
import pytest
import torch

from helpers import assert_close, colsum_slack, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# whole packs only (the ragged-row kernels keep their own layout): 4 fp32 / 8 16-bit elements
LENGTHS = [8, 16, 24, 32, 64, 96, 128, 200, 256, 264, 384, 512]


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("offset", [0, 2, 8, 32], ids=lambda o: "off%d" % o)
def test_short_rows_match_the_oracle(cabi, oracle, gpu, dtype, offset):
    code = cabi.dtype_code(dtype)
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    for N in LENGTHS:
        if N % E:
            continue
        M = 1031  # not a multiple of any rows-per-workgroup count
        print("case short rows", dtype, offset, (M, N), flush=True)
        packs = N // E
        pb = cabi.plan(cabi.OP_LAYER_NORM_BWD, M, N, code, code)
        if packs <= 64:
            assert pb["packs_per_lane"] == 1 and pb["lanes_per_row"] >= packs, pb
            # the forward looks at its pointers: off a 128-byte line it takes the same layout,
            # and the plan query reports that when told so
            off_line = (offset * (16 // E)) % 128 != 0
            pf = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code, off_line=off_line)
            assert (pf["packs_per_lane"] == 1 and pf["lanes_per_row"] >= packs) == (
                off_line or packs <= 8), (offset, pf)
        g = gen(900 + N)
        x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
        x[3] = 1.5  # a constant row
        dy = torch.randn(M, N, generator=g).to(dtype)
        gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
        beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
        place = (lambda t: offset_view(t.to(gpu), offset)) if offset else (lambda t: t.to(gpu))
        xg, dyg, gg, bg = place(x), place(dy), place(gamma), place(beta)
        out = lambda: place(torch.empty(M, N, dtype=dtype))  # noqa: E731
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5, y=out())
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "layer_norm y N=%d" % N)
        assert_close(mean, om.reshape(-1), dtype, "mean N=%d" % N)
        assert_close(rstd, orr.reshape(-1), dtype, "rstd N=%d" % N)
        assert torch.equal(y[3].cpu(), beta)
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, dx=out())
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                              to_np32(rstd), to_np32(gamma))
        xhat = (x.float() - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
        sl_g, sl_b = colsum_slack(dy.float() * xhat), colsum_slack(dy.float())
        assert_close(dx, odx, dtype, "layer_norm dx N=%d" % N)
        assert_close(dg, odg, dtype, "dgamma N=%d" % N, slack=sl_g)
        assert_close(db, odb, dtype, "dbeta N=%d" % N, slack=sl_b)
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6, y=out())
        roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "rms_norm y N=%d" % N)
        assert_close(rr, ror.reshape(-1), dtype, "rms rstd N=%d" % N)
        rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg, dx=out())
        rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
        assert_close(rdx, rodx, dtype, "rms_norm dx N=%d" % N)
        assert_close(rdg, rodg, dtype, "rms dgamma N=%d" % N,
                     slack=colsum_slack(dy.float() * x.float() * rr.cpu().reshape(M, 1)))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("offset", [0, 2, 8, 32], ids=lambda o: "off%d" % o)
def test_short_softmax_rows_match_the_oracle(cabi, oracle, gpu, dtype, offset):
    """softmax / log_softmax forward and backward take the same layout for tensors off a line;
    masked entries (-inf), a fully masked row and the float16 -> float32 output included."""
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    for N in LENGTHS:
        if N % E:
            continue
        M = 1031
        print("case short softmax rows", dtype, offset, (M, N), flush=True)
        g = gen(950 + N)
        x = (3 * torch.randn(M, N, generator=g)).to(dtype)
        x[5, N // 2:] = float("-inf")
        x[7] = float("-inf")
        grad = torch.randn(M, N, generator=g).to(dtype)
        place = (lambda t: offset_view(t.to(gpu), offset)) if offset else (lambda t: t.to(gpu))
        xg, gg = place(x), place(grad)
        for is_log in (False, True):
            y = cabi.softmax_fwd(xg, is_log, y=place(torch.empty(M, N, dtype=dtype)))
            assert_close(y, oracle.softmax_fwd(to_np32(x), is_log), dtype,
                         "softmax y N=%d log=%d" % (N, is_log))
            gi = cabi.softmax_bwd(gg, y, is_log, gi=place(torch.empty(M, N, dtype=dtype)))
            assert_close(gi, oracle.softmax_bwd(to_np32(grad), to_np32(y), is_log), dtype,
                         "softmax grad_input N=%d log=%d" % (N, is_log))
            if dtype == torch.float16:
                y32 = cabi.softmax_fwd(xg, is_log, y=place(torch.empty(M, N)))
                assert_close(y32, oracle.softmax_fwd(to_np32(x), is_log), torch.float32,
                             "softmax float16 -> float32 N=%d log=%d" % (N, is_log))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_rows_of_one_to_four_packs_over_many_rows(cabi, oracle, gpu, dtype):
    """Rows of 16 to 64 bytes (one, two or four whole packs) in tensors on a 16-byte boundary are
    staged through LDS on one, two or four lanes a row: more rows than one launch of workgroups
    holds at a time (each walks several pieces), a ragged last piece, the forward in place, dX
    alone and the column sums alone, twice the same bits."""
    E = 16 // torch.empty(0, dtype=dtype).element_size()
    for packs in (1, 2, 3, 4):
        N = packs * E
        for M in (5, 300007):
            print("case rows of few packs", dtype, (M, N), flush=True)
            g = gen(990 + packs)
            x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
            x[M // 2] = -2.5  # a constant row
            dy = torch.randn(M, N, generator=g).to(dtype)
            gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
            beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
            xg, dyg, gg, bg = x.to(gpu), dy.to(gpu), gamma.to(gpu), beta.to(gpu)
            what = "[%d, %d] %s" % (M, N, dtype)
            y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
            oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
            assert_close(y, oy, dtype, "layer_norm y " + what)
            assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
            assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
            assert torch.equal(y[M // 2].cpu(), beta), "a constant row gives beta " + what
            xc = xg.clone()
            yi, mi, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)
            assert torch.equal(yi, y) and torch.equal(mi, mean) and torch.equal(ri, rstd)
            ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
            roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
            assert_close(ry, roy, dtype, "rms_norm y " + what)
            assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
            dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
            odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                                  to_np32(rstd), to_np32(gamma))
            xhat = (x.float() - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
            assert_close(dx, odx, dtype, "layer_norm dx " + what)
            assert_close(dg, odg, dtype, "dgamma " + what, slack=colsum_slack(dy.float() * xhat))
            assert_close(db, odb, dtype, "dbeta " + what, slack=colsum_slack(dy.float()))
            dx1, n1, n2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(True, False, False))
            assert n1 is None and n2 is None and torch.equal(dx1, dx), "dX alone " + what
            n0, dg1, db1 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(False, True, True))
            assert n0 is None and torch.equal(dg1, dg) and torch.equal(db1, db), "sums alone " + what
            rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
            rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
            assert_close(rdx, rodx, dtype, "rms_norm dx " + what)
            assert_close(rdg, rodg, dtype, "rms dgamma " + what,
                         slack=colsum_slack(dy.float() * x.float() * rr.cpu().reshape(M, 1)))
