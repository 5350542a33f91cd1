"""LayerNorm / RMSNorm forward of rows beyond one workgroup's registers (more than 16384 packs:
131072 16-bit or 65536 float32 elements), whole 16-byte packs: norm_fwd_team_kernel, where a team of
workgroups holds a row in registers, exchanges partial sums through library-owned device memory
with a bounded wait, and X is read once (a workgroup whose wait runs out sums the whole row itself).  It serves the regime of the reference's split-row kernels
(src/ATen/native/xpu/sycl/Norm.h:632-812 behind LayerNormKernels.cpp:1121-1163) and the shapes of
its micro-benchmark (test/microbench/layer_norm.py:17-22).  Through the extern "C" ABI, against the
float64 oracle (float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2), against the path a
workgroup takes when its wait gives up (forced from the host by a wait of zero: no kernel hangs),
against the multi-launch split-row kernels, in place (which those kernels serve), and for
run-to-run determinism."""
import pytest
import torch

from helpers import assert_close, gen, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (rows, packs a row): nine teams of 33 workgroups (one stride of 512 packs each, the last chunk a
# single pack); twelve teams of 25 (two strides each, the last chunk ragged); three workgroups a row
# and two rounds of 170 teams; eight teams of 64 with five packs a lane
SHAPES = [(9, 16385), (12, 25000), (300, 17500), (8, 163840)]


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


def _split(cabi, op, chunks, fn):
    try:
        cabi.set_override(op, -1, chunks)
        return fn()
    finally:
        cabi.clear_overrides()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_team_forward_against_oracle_fallback_and_split_kernels(cabi, oracle, gpu, dtype, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    E = 4 if dtype == torch.float32 else 8
    wdtype = torch.float32 if mixed else dtype
    code, wcode = cabi.dtype_code(dtype), cabi.dtype_code(wdtype)
    for i, (M, packs) in enumerate(SHAPES):
        N = packs * E
        print("case team rows", dtype, mixed, (M, N), flush=True)
        for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_RMS_NORM_FWD):
            p = cabi.plan(op, M, N, code, wcode)
            # (the plan of a team launch: workgroups a row, and a grid of whole teams, 8 at least)
            assert p["resident"] == 0 and p["row_chunks"] >= 2 and p["grid_blocks"] <= 512, p
            assert p["grid_blocks"] % p["row_chunks"] == 0, p
            assert 8 <= p["grid_blocks"] // p["row_chunks"] <= M, p
        x, gamma, beta = _mk(M, N, dtype, wdtype, 1600 + i)
        x[0, :3] = 0.0  # the head of a row is not representative of it
        if M > 2:
            x[2] = 1.25  # a constant row
        xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
        what = "[%d, %d] %s" % (M, N, dtype)
        y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, dtype, "layer_norm y " + what)
        assert_close(mean, om.reshape(-1), torch.float32, "mean " + what)
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd " + what)
        if M > 2:
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
        # every wait gives up at once (each workgroup then sums the whole row itself) and the
        # split-row kernels: same statistics to float32 rounding, same y to the family's tolerance
        fy, fm, fr = _with_wait(cabi, 0, lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
        assert_close(fy, oy, dtype, "fallback y " + what)
        assert_close(fr, orr.reshape(-1), torch.float32, "fallback rstd " + what)
        assert_close(rstd, to_np32(fr), torch.float32, "rstd, team against fallback " + what)
        fry, frr = _with_wait(cabi, 0, lambda: cabi.rms_norm_fwd(xg, gg, 1e-6))
        assert_close(fry, roy, dtype, "fallback rms y " + what)
        assert_close(rr, to_np32(frr), torch.float32, "rms rstd, team against fallback " + what)
        sy, sm, sr = _split(cabi, cabi.OP_LAYER_NORM_FWD, 5,
                            lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
        assert_close(y, to_np32(sy), dtype, "y, team against split rows " + what)
        assert_close(mean, to_np32(sm), torch.float32, "mean, team against split rows " + what)
        assert_close(rstd, to_np32(sr), torch.float32, "rstd, team against split rows " + what)
        if i % 2 == 0:
            # no weights; in place
            y0, _, _ = cabi.layer_norm_fwd(xg, None, None, 1e-5)
            oy0, _, _ = oracle.layer_norm_fwd(to_np32(x), (N,), None, None, 1e-5)
            assert_close(y0, oy0, dtype, "layer_norm without weights " + what)
            xc = xg.clone()
            yi, mi, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)
            assert yi.data_ptr() == xc.data_ptr()
            assert_close(yi, oy, dtype, "in place y " + what)
            assert_close(ri, orr.reshape(-1), torch.float32, "in place rstd " + what)
            assert_close(mi, om.reshape(-1), torch.float32, "in place mean " + what)


def test_fewer_than_eight_teams_keep_the_multi_launch_kernels(cabi, oracle, gpu):
    """Rows that would make fewer than 8 teams (their phases run in step and nothing hides the
    wait) keep the split-row / two-pass kernels; the result is the same to the tolerance."""
    for (M, N) in ((3, 16385 * 8), (2, 1310720)):
        p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, cabi.BF16, cabi.BF16)
        assert p["resident"] == 0 and p["grid_blocks"] <= M, p
        x, gamma, beta = _mk(M, N, torch.bfloat16, torch.bfloat16, 1640)
        y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-5)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
        assert_close(y, oy, torch.bfloat16, "y [%d, %d]" % (M, N))
        assert_close(rstd, orr.reshape(-1), torch.float32, "rstd [%d, %d]" % (M, N))


def test_team_forward_non_finite_rows_and_missing_statistics(cabi, oracle, gpu):
    M, N = 9, 20000 * 8
    x, gamma, beta = _mk(M, N, torch.bfloat16, torch.bfloat16, 1650)
    x[1, 70000] = float("inf")
    x[3, N - 1] = float("nan")
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    assert bool(torch.isnan(mean[1])) and bool(torch.isnan(rstd[1])) and bool(torch.isnan(y[1]).all())
    assert bool(torch.isnan(mean[3])) and bool(torch.isnan(y[3]).all())
    p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, cabi.BF16, cabi.BF16)
    assert p["grid_blocks"] // max(p["row_chunks"], 1) >= 8, p  # (a team launch)
    fin = [0, 2, 4, 5, 6, 7, 8]
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x[fin]), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y[fin], oy, torch.bfloat16, "finite rows beside non-finite ones")
    assert_close(rstd[fin], orr.reshape(-1), torch.float32, "rstd of the finite rows")
    ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    assert float(rr[1]) == 0.0 and bool(torch.isnan(rr[3]))


def test_microbench_shape_of_the_reference(cabi, oracle, gpu):
    """bf16 [8, 4194304] (64 workgroups a row, every compute unit two) and [512, 401408] (eight a
    row, eight rounds): every row's moments and every element against float64 arithmetic."""
    for (M, N) in ((8, 4194304), (512, 3136 * 128)):
        print("case team rows", (M, N), flush=True)
        g = torch.Generator(device=gpu).manual_seed(1660)
        x = (0.25 + torch.randn(M, N, generator=g, device=gpu)).bfloat16()
        gamma = (1 + 0.1 * torch.randn(N, generator=g, device=gpu)).bfloat16()
        beta = (0.1 * torch.randn(N, generator=g, device=gpu)).bfloat16()
        y, mean, rstd = cabi.layer_norm_fwd(x, gamma, beta, 1e-5)
        xd = x.double()
        mu = xd.mean(1)
        rs = 1.0 / torch.sqrt(xd.var(1, unbiased=False) + 1e-5)
        assert_close(mean, mu, torch.float32, "mean [%d, %d]" % (M, N))
        assert_close(rstd, rs, torch.float32, "rstd [%d, %d]" % (M, N))
        ref = ((xd - mu[:, None]) * rs[:, None] * gamma.double() + beta.double())
        assert_close(y, ref, torch.bfloat16, "y [%d, %d]" % (M, N))
        del xd, ref
        fy, fm, fr = _with_wait(cabi, 0, lambda: cabi.layer_norm_fwd(x, gamma, beta, 1e-5))
        assert_close(rstd, to_np32(fr), torch.float32, "rstd, team against fallback")
        assert_close(y, to_np32(fy), torch.bfloat16, "y, team against fallback")
        del fy
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_few_rows_that_one_workgroup_would_hold(cabi, oracle, gpu, dtype):
    """Rows of exactly 16384 packs (16 a lane on 1024 lanes: the longest one workgroup holds), too
    few of them for the compute units: the teams take them as well; with one row more than half
    the compute units the register-resident kernel keeps them."""
    E = 4 if dtype == torch.float32 else 8
    N = 16384 * E
    code = cabi.dtype_code(dtype)
    for M in (100, 128):
        p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)
        assert p["row_chunks"] >= 2 and p["grid_blocks"] % p["row_chunks"] == 0, p
        assert p["grid_blocks"] // p["row_chunks"] == M and p["grid_blocks"] <= 512, p
    p = cabi.plan(cabi.OP_LAYER_NORM_FWD, 129, N, code, code)
    assert p["resident"] == 1 and p["grid_blocks"] <= 129, p
    M = 100
    x, gamma, beta = _mk(M, N, dtype, dtype, 1680)
    x[7] = 1.25
    xg, gg, bg = x.to(gpu), gamma.to(gpu), beta.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y, oy, dtype, "layer_norm y")
    assert_close(mean, om.reshape(-1), torch.float32, "mean")
    assert_close(rstd, orr.reshape(-1), torch.float32, "rstd")
    assert torch.equal(y[7].cpu(), beta), "a constant row gives beta bit for bit"
    fy, fm, fr = _with_wait(cabi, 0, lambda: cabi.layer_norm_fwd(xg, gg, bg, 1e-5))
    assert_close(fy, oy, dtype, "fallback y")
    assert_close(rstd, to_np32(fr), torch.float32, "rstd, team against fallback")
    ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
    assert_close(ry, roy, dtype, "rms_norm y")
    assert_close(rr, ror.reshape(-1), torch.float32, "rms rstd")
    xc = xg.clone()
    yi, _, ri = cabi.layer_norm_fwd(xc, gg, bg, 1e-5, y=xc)  # in place: the resident kernel
    assert_close(yi, oy, dtype, "in place y")
