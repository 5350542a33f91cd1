"""LayerNorm / RMSNorm forward of many rows too long for eight teams of workgroups at a time (the
9.8 M-element rows of the reference's micro-benchmark): norm_fwd_rows_team_kernel spreads a row
over one team of up to 256 workgroups, ten packs a lane, keeps the gamma / beta of a lane's columns
for the whole call, and has three rows in flight a workgroup -- one being requested, one summed and
published, one gathered and written -- so that neither loads nor the exchange are waited for.  X is
read once and the weights once a call.  The regime of the reference's split-row kernels
(src/ATen/native/xpu/sycl/Norm.h:632-812 behind LayerNormKernels.cpp:1121-1163) at the long-row
shapes of its micro-benchmark (test/microbench/layer_norm.py:17-22).  Through the extern "C" ABI
against the float64 oracle (float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2), against
the path a workgroup takes when its wait gives up (forced from the host by a wait of zero: no
kernel hangs), against the multi-launch kernels, and for run-to-run determinism.  The plan sends
a call there from 16 rounds on when fewer than eight of the other teams would exist; the small
shapes here reach the kernel through the override that asks for it whatever the rounds."""
import pytest
import torch

from helpers import assert_close, gen, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (rows, packs a row, rows at a time, packs a lane): 4 workgroups a row (the last holds 1640
# packs: idle upper packs), a team a row, one round; 7 workgroups a row, 36 teams, two rounds;
# 52 workgroups a row (the last holds 1030 packs), 4 teams, 14 rows: three rounds and a part
SHAPES = [(37, 17000, 1, 10), (71, 33000, 1, 10), (14, 262150, 1, 10)]


def _mk(M, N, dtype, wdtype, seed):
    g = gen(seed)
    x = (0.5 + torch.randn(M, N, generator=g)).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
    beta = (0.1 * torch.randn(N, generator=g)).to(wdtype)
    return x, gamma, beta


def _with_wait(cabi, us, fn):
    try:
        cabi.set_team_wait_us(us)
        return fn()
    finally:
        cabi.set_team_wait_us()


def _force_groups(cabi):
    for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD):
        cabi.set_override(op, -1, 0, 1)


def _split(cabi, op, chunks, fn):
    try:
        cabi.set_override(op, -1, chunks)
        return fn()
    finally:
        cabi.clear_overrides()
        _force_groups(cabi)


def _groups_planned(p, R, V):
    return p["resident"] == 0 and p["row_chunks"] >= 2 and p["block_threads"] == 512 \
        and p["packs_per_lane"] == V and p["rows_per_block"] == R \
        and p["grid_blocks"] % p["row_chunks"] == 0 and p["grid_blocks"] <= 256


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_groups_of_rows_against_oracle_fallback_and_split_kernels(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    try:
        _force_groups(cabi)
        _cases(cabi, oracle, gpu, dtype, mixed)
    finally:
        cabi.clear_overrides()


def _cases(cabi, oracle, gpu, dtype, mixed):
    E = 4 if dtype == torch.float32 else 8
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (M, packs, R, V) in enumerate(SHAPES):
        if mixed and V == 10:
            continue  # (one row at a time holds weights no wider than the rows)
        N = packs * E
        print("case groups of rows", dtype, mixed, (M, N), flush=True)
        for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD):
            p = cabi.plan(op, M, N, code, wcode)
            assert _groups_planned(p, R, V), p
            assert p["row_chunks"] == (packs + V * 512 - 1) // (V * 512), p
        x, gamma, beta = _mk(M, N, dtype, wdtype, 1800 + i)
        x[0, :3] = 0.0  # the head of a row is not representative of it
        x[2] = 1.25  # a constant row
        xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
        what = "[%d, %d] %s" % (M, N, dtype)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "layer_norm y " + what)
        assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
        assert torch.equal(y[2].cpu(), beta.to(dtype)), "a constant row gives beta bit for bit"
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
        roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
        assert_close(ry, roy, dtype, "rms_norm y " + what)
        assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd " + what)
        # a second run gives the same bits (another call id, another slot)
        y2, mean2, rstd2 = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        ry2, rr2 = cabi.rms_norm_fwd(xg, gg, 1e-6)
        for a, b in ((y, y2), (mean, mean2), (rstd, rstd2), (ry, ry2), (rr, rr2)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
        # every wait gives up at once (each workgroup then sums its rows itself), and the
        # split-row kernels: same statistics to float32 rounding, same y to the tolerance
        fy, fm, fr = _with_wait(cabi, 0, lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
        assert_close(fy, oy, dtype, "fallback y " + what)
        assert_close(fr, orr.reshape(-1), torch.float32, "fallback rstd " + what)
        assert_close(fm, om.reshape(-1), torch.float32, "fallback mean " + what)
        fry, frr = _with_wait(cabi, 0, lambda: cabi.rms_norm_fwd(xg, gg, 1e-6))
        assert_close(fry, roy, dtype, "fallback rms y " + what)
        assert_close(rr, to_np32(frr), torch.float32, "rms rstd, teams against fallback " + what)
        sy, sm, sr = _split(cabi, cabi.OP_LAYER_NORM_FWD, 5,
                            lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
        assert_close(y, to_np32(sy), dtype, "y, teams against split rows " + what)
        assert_close(mean, to_np32(sm), torch.float32, "mean, teams against split rows " + what)
        assert_close(rstd, to_np32(sr), torch.float32, "rstd, teams against split rows " + what)
        if i != 1:
            # no weights; in place (which the multi-launch kernels serve)
            y0, _, _ = cabi.layer_norm_fwd(xg, None, None, 1e-5)
            oy0, _, _ = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, 1e-5)
            assert_close(y0, oy0, dtype, "layer_norm without weights " + what)
            xc = xg.clone()
            yi, mi, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)
            assert yi.data_ptr() == xc.data_ptr()
            assert_close(yi, oy, dtype, "in place y " + what)
            assert_close(ri, orr.reshape(-1), torch.float32, "in place rstd " + what)


def test_groups_of_rows_non_finite_rows_stay_in_their_rows(cabi, oracle, gpu):
    M, N = 9, 17000 * 8
    x, gamma, beta = _mk(M, N, torch.bfloat16, torch.bfloat16, 1850)
    x[1, 70000] = float("inf")
    x[6, N - 1] = float("nan")
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    try:
        _force_groups(cabi)
        assert _groups_planned(cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, cabi.BF16, cabi.BF16), 1, 10)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    finally:
        cabi.clear_overrides()
    assert bool(torch.isnan(mean[1])) and bool(torch.isnan(rstd[1])) and bool(torch.isnan(y[1]).all())
    assert bool(torch.isnan(mean[6])) and bool(torch.isnan(y[6]).all())
    fin = [0, 2, 3, 4, 5, 7, 8]
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x[fin]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y[fin], oy, torch.bfloat16, "finite rows beside non-finite ones")
    assert_close(rstd[fin], orr.reshape(-1), torch.float32, "rstd of the finite rows")
    assert float(rr[1]) == 0.0 and bool(torch.isnan(rr[6]))
