"""softmax / log_softmax forward and backward of few, very long rows (fewer rows than half the
compute units, 32768 16-bit or 16384 float32 elements and more, whole 16-byte packs):
softmax_fwd_team_kernel / softmax_bwd_team_kernel, where a team of workgroups holds a row in
registers and exchanges (maximum, sum) pairs -- the backward: sums -- through library-owned device
memory with a bounded wait.  It serves the rows the reference gives one
work-group each (SoftmaxForwardKernelFunctor / SoftmaxBackwardKernelFunctor, src/ATen/native/xpu/sycl/
SoftMaxKernels.cpp:546-684, 952-1080).
Through the extern "C" ABI, against the float64 oracle (float32 rtol = atol = 1e-5; 16-bit atol 1e-2,
rtol 1.6e-2), against the path a workgroup takes when its wait gives up (forced from the host by a
wait of zero: no kernel hangs), against the one-workgroup-a-row kernels, and for run-to-run
determinism; masked (-inf) entries, rows without a finite element, NaN, the float16 -> float32
output, in place (which the one-workgroup-a-row kernels serve)."""
import pytest
import torch

from helpers import assert_close, gen, rowsum_slack, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (rows, packs a row): one team of 8; five teams whose last chunk is ragged; 40 teams of 9 with
# one pack in the last chunk; 100 teams of 5 with four packs a lane; two rounds of 56 teams of 9
# with 16 packs a lane
SHAPES = [(1, 4096), (5, 5000), (40, 4097), (100, 9000), (100, 70000)]


def _with_wait(cabi, us, fn):
    try:
        cabi.set_team_wait_us(us)
        return fn()
    finally:
        cabi.set_team_wait_us()


def _one_workgroup_a_row(cabi, fn, op=None):
    try:
        cabi.set_override(cabi.OP_SOFTMAX_FWD if op is None else op, 0, 0, 0, 2)  # (any override: no team)
        return fn()
    finally:
        cabi.clear_overrides()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_team_softmax_against_oracle_fallback_and_row_kernels(cabi, oracle, gpu, dtype):
    E = 4 if dtype == torch.float32 else 8
    code = cabi.dtype_code(dtype)
    for i, (M, packs) in enumerate(SHAPES):
        N = packs * E
        print("case softmax team rows", dtype, (M, N), flush=True)
        p = cabi.plan(cabi.OP_SOFTMAX_FWD, M, N, code, code)
        assert p["row_chunks"] >= 2 and p["grid_blocks"] <= 512, p
        assert p["grid_blocks"] % p["row_chunks"] == 0, p
        teams = p["grid_blocks"] // p["row_chunks"]
        assert teams == M or 8 <= teams < M, p
        g = gen(2100 + i)
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        x[0, :5] = float("-inf")
        if M > 2:
            x[1, N // 2:] = float("-inf")   # whole chunks without a finite element
            x[2] = float("-inf")            # a row without one
        if M > 4:
            x[3, N - 1] = float("nan")
            x[4, 7] = 80.0                  # a maximum far above the rest
        xg = x.to(gpu)
        for is_log in (False, True):
            what = "%s [%d, %d] %s" % ("log_softmax" if is_log else "softmax", M, N, dtype)
            y = cabi.softmax_fwd(xg, is_log)
            oy = oracle.softmax_fwd(to_np32(x), is_log)
            assert_close(y, oy, dtype, what)
            if M > 2:
                assert bool(torch.isnan(y[2]).all()), what + ": a row without a finite element"
            if not is_log:
                fin = [r for r in range(M) if r not in (2, 3)]
                s = y[fin].float().sum(-1).cpu()
                assert float((s - 1).abs().max()) < (1e-4 if dtype == torch.float32 else 2e-2), what
            y2 = cabi.softmax_fwd(xg, is_log)
            assert torch.equal(y.view(torch.uint8), y2.view(torch.uint8)), what + ": run to run"
            fy = _with_wait(cabi, 0, lambda: cabi.softmax_fwd(xg, is_log))
            assert_close(fy, oy, dtype, what + ", every wait given up")
            ry = _one_workgroup_a_row(cabi, lambda: cabi.softmax_fwd(xg, is_log))
            assert_close(ry, oy, dtype, what + ", one workgroup a row")
            xc = xg.clone()
            yi = cabi.softmax_fwd(xc, is_log, y=xc)
            assert yi.data_ptr() == xc.data_ptr()
            assert_close(yi, oy, dtype, what + ", in place")
        if not M > 2:
            continue
        sy = cabi.safe_softmax_fwd(xg)
        assert bool((sy[2] == 0).all()), "safe softmax: zeros for a row without a finite element"
        fin = [r for r in range(M) if r != 2]
        assert_close(sy[fin], oracle.softmax_fwd(to_np32(x[fin]), False), dtype, "safe softmax")


def test_team_softmax_float16_rows_to_float32(cabi, oracle, gpu):
    M, N = 6, 50000 * 8
    x = (2.0 * torch.randn(M, N, generator=gen(2150))).half()
    xg = x.to(gpu)
    p = cabi.plan(cabi.OP_SOFTMAX_FWD, M, N, cabi.F16, cabi.F16)
    assert p["row_chunks"] >= 2, p
    for is_log in (False, True):
        y = cabi.softmax_fwd(xg, is_log, out_dtype=torch.float32)
        assert y.dtype == torch.float32
        assert_close(y, oracle.softmax_fwd(to_np32(x), is_log), torch.float32, "half to float, log %s" % is_log)
        fy = _with_wait(cabi, 0, lambda: cabi.softmax_fwd(xg, is_log, out_dtype=torch.float32))
        assert_close(fy, to_np32(y), torch.float32, "half to float, every wait given up")


def test_shapes_the_team_does_not_take(cabi, oracle, gpu):
    """Ragged rows, rows off a 16-byte boundary, more rows than half the compute units and rows
    under 4096 packs keep the one-workgroup-a-row kernels (the plan says which)."""
    for (M, N) in ((4, 8 * 4096 + 3), (200, 8 * 4096), (4, 8 * 4000)):
        p = cabi.plan(cabi.OP_SOFTMAX_FWD, M, N, cabi.BF16, cabi.BF16)
        assert p["row_chunks"] == 0 and p["grid_blocks"] <= M, p
    M, N = 4, 8 * 4096
    x = torch.randn(M, N + 8, generator=gen(2160)).bfloat16().to(gpu)
    xo = x.reshape(-1)[1:1 + M * N].view(M, N)  # 2-byte aligned rows
    y = cabi.softmax_fwd(xo)
    assert_close(y, oracle.softmax_fwd(to_np32(xo), False), torch.bfloat16, "rows off a 16-byte boundary")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_team_softmax_backward_against_oracle_fallback_and_row_kernels(cabi, oracle, gpu, dtype):
    E = 4 if dtype == torch.float32 else 8
    code = cabi.dtype_code(dtype)
    for i, (M, packs) in enumerate(SHAPES):
        N = packs * E
        print("case softmax team rows backward", dtype, (M, N), flush=True)
        p = cabi.plan(cabi.OP_SOFTMAX_BWD, M, N, code, code)
        assert p["row_chunks"] >= 2 and p["grid_blocks"] <= 512, p
        assert p["grid_blocks"] % p["row_chunks"] == 0, p
        g = gen(2200 + i)
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        x[0, :5] = float("-inf")
        grad = torch.randn(M, N, generator=g).to(dtype)
        xg, gg = x.to(gpu), grad.to(gpu)
        for is_log in (False, True):
            what = "%s backward [%d, %d] %s" % ("log_softmax" if is_log else "softmax", M, N, dtype)
            y = cabi.softmax_fwd(xg, is_log)
            gi = cabi.softmax_bwd(gg, y, is_log)
            ogi = oracle.softmax_bwd(to_np32(grad), to_np32(y), is_log)
            # (a float32 sum over up to 560000 products: the tolerance of the family plus the
            # sum's own rounding, which y or exp(y) carries into every element)
            yy = y.float().cpu()
            w = torch.exp(yy) if is_log else yy
            terms = grad.float() if is_log else grad.float() * yy
            assert_close(gi, ogi, dtype, what, slack=rowsum_slack(terms, w))
            gi2 = cabi.softmax_bwd(gg, y, is_log)
            assert torch.equal(gi.view(torch.uint8), gi2.view(torch.uint8)), what + ": run to run"
            fgi = _with_wait(cabi, 0, lambda: cabi.softmax_bwd(gg, y, is_log))
            assert_close(fgi, ogi, dtype, what + ", every wait given up", slack=rowsum_slack(terms, w))
            rgi = _one_workgroup_a_row(cabi, lambda: cabi.softmax_bwd(gg, y, is_log), cabi.OP_SOFTMAX_BWD)
            assert_close(rgi, ogi, dtype, what + ", one workgroup a row", slack=rowsum_slack(terms, w))
            gc = gg.clone()
            gii = cabi.softmax_bwd(gc, y, is_log, gi=gc)  # in place on grad: the row kernels
            assert gii.data_ptr() == gc.data_ptr()
            assert_close(gii, ogi, dtype, what + ", in place", slack=rowsum_slack(terms, w))


def test_team_softmax_backward_float32_to_float16(cabi, oracle, gpu):
    """The backward of the float16 -> float32 forward: float32 grad and y, float16 gradient."""
    M, N = 6, 50000 * 4
    g = gen(2250)
    x = (2.0 * torch.randn(M, N, generator=g))
    grad = torch.randn(M, N, generator=g)
    y = torch.softmax(x, -1)
    p = cabi.plan(cabi.OP_SOFTMAX_BWD, M, N, cabi.F32, cabi.F32)
    assert p["row_chunks"] >= 2, p
    gi = cabi.softmax_bwd(grad.to(gpu), y.to(gpu), False, gi_dtype=torch.float16)
    assert gi.dtype == torch.float16
    assert_close(gi, oracle.softmax_bwd(to_np32(grad), to_np32(y), False), torch.float16, "float to half")
