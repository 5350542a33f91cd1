"""LayerNorm / RMSNorm backward of rows beyond one workgroup's registers, whole 16-byte packs on
16-byte aligned tensors, dX apart from dY and X: norm_bwd_team_kernel, where a team of workgroups
holds four rows at a time (two packs of dY and of X a lane and row), the rows' partial sums cross the
team through library-owned device memory with a bounded wait, the next four rows are already on
their way during the exchange, every lane keeps the column sums of its own columns, and dY and X
are read once (a workgroup whose wait runs out sums its rows itself).  It serves the regime of the
reference's backward for rows that do not fit a workgroup (src/ATen/native/xpu/sycl/
LayerNormKernels.cpp:1218-1406 over Norm.h:632-812) and the long-row shapes of its micro-benchmark
(test/microbench/layer_norm.py:17-22).  Through the extern "C" ABI, against the float64 oracle
(float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2; column sums with the slack of their
float32 partial sums), against the path a workgroup takes when its wait gives up (forced from the
host by a wait of zero: no kernel hangs), against the multi-launch kernels (in place, which they
serve; forced by override), and for run-to-run determinism.  The plan sends a call to teams from
the second round of four rows a team on; the shapes here also ask for it by override, whatever the
rounds, the last test goes through the plan alone."""
import pytest
import torch

from helpers import assert_close, colsum_slack, gen, to_np32, xhat_slack

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (rows, packs a row): five workgroups a row (the last holds 104 packs), 51 teams, 76 groups of 4
# rows the last of which holds 1; 17 workgroups a row whose last holds one pack, 15 teams, a last
# group of 3 rows; five workgroups a row the last of which has idle upper packs, and fewer groups
# of rows (8) than teams there could be; 49 workgroups a row, 5 teams, one round and a part of one
SHAPES = [(301, 4200), (103, 16385), (30, 4608), (26, 50176)]


def _mk(M, N, dtype, wdtype, seed):
    g = gen(seed)
    x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
    return x, dy, gamma


def _with_wait(cabi, us, fn):
    try:
        cabi.set_team_wait_us(us)
        return fn()
    finally:
        cabi.set_team_wait_us()


def _force_teams(cabi):
    for op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD):
        cabi.set_override(op, -1, 0, 1)


def _forced(cabi, op, chunks, fn):
    """fn() on the multi-launch kernels with every row split into `chunks`; the team override
    is back in place afterwards."""
    try:
        cabi.set_override(op, -1, chunks)
        return fn()
    finally:
        cabi.clear_overrides()
        _force_teams(cabi)


def _team_planned(cabi, op, M, N, code, wcode):
    p = cabi.plan(op, M, N, code, wcode)
    return p["resident"] == 0 and p["row_chunks"] >= 2 and p["block_threads"] == 512 \
        and p["packs_per_lane"] == 2 and p["grid_blocks"] % p["row_chunks"] == 0 \
        and p["grid_blocks"] <= 256 and p["partial_rows"] >= p["grid_blocks"] // p["row_chunks"]


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_team_backward_against_oracle_fallback_and_multi_launch_kernels(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    try:
        _force_teams(cabi)
        _team_backward_cases(cabi, oracle, gpu, dtype, mixed)
    finally:
        cabi.clear_overrides()


def _team_backward_cases(cabi, oracle, gpu, dtype, mixed):
    E = 4 if dtype == torch.float32 else 8
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (M, packs) in enumerate(SHAPES):
        N = packs * E
        print("case team rows backward", dtype, mixed, (M, N), flush=True)
        planned = [_team_planned(cabi, op, M, N, code, wcode)
                   for op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD)]
        assert all(planned), (M, N, planned)
        x, dy, gamma = _mk(M, N, dtype, wdtype, 1700 + i)
        x[M // 2] = -2.5  # a constant row
        xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
        what = "[%d, %d] %s" % (M, N, dtype)
        _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
        _, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
        rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                              to_np32(rstd), to_np32(gamma))
        rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
        xhat = (x.float() - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
        sl_g = colsum_slack(dy.float() * xhat) + xhat_slack(dy, mean, rstd)
        sl_b = colsum_slack(dy.float())
        sl_r = colsum_slack(dy.float() * x.float() * rr.cpu().reshape(M, 1))
        assert_close(dx, odx, dtype, "layer_norm dx " + what)
        assert_close(dg, odg, wdtype, "dgamma " + what, slack=sl_g)
        assert_close(db, odb, wdtype, "dbeta " + what, slack=sl_b)
        assert_close(rdx, rodx, dtype, "rms_norm dx " + what)
        assert_close(rdg, rodg, wdtype, "rms dgamma " + what, slack=sl_r)
        # a second run gives the same bits (another call id, another slot)
        dx2, dg2, db2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
        rdx2, rdg2 = cabi.rms_norm_bwd(dyg, xg, rr, gg)
        for a, b in ((dx, dx2), (dg, dg2), (db, db2), (rdx, rdx2), (rdg, rdg2)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "twice the same bits " + what
        # every wait gives up at once: each workgroup sums its rows itself
        fdx, fdg, fdb = _with_wait(cabi, 0, lambda: cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg))
        assert_close(fdx, odx, dtype, "fallback dx " + what)
        assert_close(fdg, odg, wdtype, "fallback dgamma " + what, slack=sl_g)
        assert_close(fdb, odb, wdtype, "fallback dbeta " + what, slack=sl_b)
        if all(planned):
            # (the column sums do not depend on the rows' sums: the same bits either way)
            assert torch.equal(fdg, dg) and torch.equal(fdb, db), "column sums, fallback " + what
        frdx, frdg = _with_wait(cabi, 0, lambda: cabi.rms_norm_bwd(dyg, xg, rr, gg))
        assert_close(frdx, rodx, dtype, "fallback rms dx " + what)
        assert_close(frdg, rodg, wdtype, "fallback rms dgamma " + what, slack=sl_r)
        # the multi-launch kernels: forced by override, and in place (dX over dY)
        sdx, sdg, sdb = _forced(cabi, cabi.OP_LAYER_NORM_BWD, 3,
                                lambda: cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg))
        assert_close(dx, to_np32(sdx), dtype, "dx, team against split rows " + what)
        assert_close(sdg, odg, wdtype, "split rows dgamma " + what, slack=sl_g)
        dyc = dyg.clone()
        idx, idg, idb = cabi.layer_norm_bwd(dyc, xg, mean, rstd, gg, dx=dyc)
        assert idx.data_ptr() == dyc.data_ptr()
        assert_close(idx, odx, dtype, "in place dx " + what)
        assert_close(idg, odg, wdtype, "in place dgamma " + what, slack=sl_g)
        assert_close(idb, odb, wdtype, "in place dbeta " + what, slack=sl_b)
        if i % 2 == 0:
            # dX alone (no workspace), the column sums alone, no gamma
            dx1, n1, n2 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(True, False, False))
            assert n1 is None and n2 is None and torch.equal(dx1, dx), "dX alone " + what
            n0, dg1, db1 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(False, True, True))
            assert n0 is None
            assert_close(dg1, odg, wdtype, "dgamma alone " + what, slack=sl_g)
            assert_close(db1, odb, wdtype, "dbeta alone " + what, slack=sl_b)
            rdx1, rn = cabi.rms_norm_bwd(dyg, xg, rr, gg, want=(True, False))
            assert rn is None and torch.equal(rdx1, rdx), "rms dX alone " + what
            dx0, dg0, db0 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, None, w_dtype=wdtype)
            odx0, odg0, odb0 = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                                     to_np32(rstd), None)
            assert_close(dx0, odx0, dtype, "dx without gamma " + what)
            assert_close(dg0, odg0, wdtype, "dgamma without gamma " + what, slack=sl_g)


def test_team_backward_plans_and_workspace(cabi):
    """The plan of a team backward: whole teams of row_chunks workgroups, at most 256 workgroups,
    and a workspace that holds one partial row a team of each column sum wanted; a single round
    (and, for a LayerNorm on teams of more than 64 workgroups, fewer than four) keeps the
    multi-launch kernels."""
    for (M, N, ln_team, rms_team) in ((512, 401408, True, True), (4096, 65536, True, True),
                                      (100, 401408, True, True), (8192, 24584, True, None),
                                      (16, 1048576, False, True), (16, 401408, False, False)):
        for op, nparts in ((cabi.OP_LAYER_NORM_BWD, 2), (cabi.OP_RMS_NORM_BWD, 1)):
            p = cabi.plan(op, M, N, cabi.BF16, cabi.BF16)
            team = ln_team if op == cabi.OP_LAYER_NORM_BWD else rms_team
            if p["resident"] or team is None:
                continue
            assert _team_planned(cabi, op, M, N, cabi.BF16, cabi.BF16) == team, (M, N, op, p)
            if not team:
                continue
            teams = p["grid_blocks"] // p["row_chunks"]
            assert p["grid_blocks"] == teams * p["row_chunks"] <= 256, p
            assert p["row_chunks"] == (N // 8 + 1023) // 1024, p
            assert 1 <= teams <= (M + 3) // 4 and p["partial_rows"] >= teams, p
            if op == cabi.OP_LAYER_NORM_BWD:
                nbytes = cabi.lib().mi355x_layer_norm_bwd_workspace_bytes(M, N, cabi.BF16, cabi.BF16, 1, 1)
            else:
                nbytes = cabi.lib().mi355x_rms_norm_bwd_workspace_bytes(M, N, cabi.BF16, cabi.BF16, 1)
            assert nbytes >= p["partial_rows"] * N * 4 * nparts, (p, nbytes)


def test_team_backward_non_finite_rows_stay_in_their_rows(cabi, oracle, gpu):
    M, N = 41, 4200 * 8
    x, dy, gamma = _mk(M, N, torch.bfloat16, torch.bfloat16, 1750)
    dy[7, 12345] = float("inf")
    xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
    _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
    try:
        _force_teams(cabi)
        assert _team_planned(cabi, cabi.OP_LAYER_NORM_BWD, M, N, cabi.BF16, cabi.BF16)
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
    finally:
        cabi.clear_overrides()
    assert not bool(torch.isfinite(dx[7]).any()), "the row of the infinite dy element"
    fin = torch.ones(M, dtype=torch.bool)
    fin[7] = False
    odx, _, _ = oracle.layer_norm_bwd(to_np32(dy[fin]), to_np32(x[fin]), (N,), to_np32(mean.cpu()[fin]),
                                      to_np32(rstd.cpu()[fin]), to_np32(gamma))
    assert_close(dx[fin.to(gpu)], odx, torch.bfloat16, "rows beside the non-finite one")
    assert not bool(torch.isfinite(db[12345]))
    assert bool(torch.isfinite(db[:12345]).all()) and bool(torch.isfinite(db[12346:]).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_team_backward_chosen_by_the_plan(cabi, oracle, gpu, dtype):
    """No override: 1640 rows of 5120 packs make 51 teams of 5 workgroups and 9 rounds (the last
    with 2 groups of rows), which the plan sends to the teams."""
    E = 4 if dtype == torch.float32 else 8
    M, N = 1640, 5120 * E
    code = cabi.dtype_code(dtype)
    for op in (cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_BWD):
        assert _team_planned(cabi, op, M, N, code, code), cabi.plan(op, M, N, code, code)
    print("case team rows backward by the plan", dtype, (M, N), flush=True)
    x, dy, gamma = _mk(M, N, dtype, dtype, 1790)
    xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
    _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
    _, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
    rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
    odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                          to_np32(rstd), to_np32(gamma))
    xhat = (x.float() - mean.cpu().reshape(M, 1)) * rstd.cpu().reshape(M, 1)
    assert_close(dx, odx, dtype, "layer_norm dx")
    assert_close(dg, odg, dtype, "dgamma", slack=colsum_slack(dy.float() * xhat) + xhat_slack(dy, mean, rstd))
    assert_close(db, odb, dtype, "dbeta", slack=colsum_slack(dy.float()))
    del odx, xhat
    rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
    assert_close(rdx, rodx, dtype, "rms_norm dx")
    assert_close(rdg, rodg, dtype, "rms dgamma",
                 slack=colsum_slack(dy.float() * x.float() * rr.cpu().reshape(M, 1)))
