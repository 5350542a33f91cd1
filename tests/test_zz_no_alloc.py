"""mi355x_rms_norm_bwd_static -- the entry point for callers that cannot allocate device memory
(HIP graph capture, serving loops): the RMSNorm backward with its scratch in a static device array
of the library.  Through the extern "C" ABI, against mi355x_rms_norm_bwd given the full workspace
(bit for bit: same kernels, same fixed summation order) and against the CPU oracle (16-bit: atol
1e-2, rtol 1.6e-2; float32: rtol = atol = 1e-5), on two calls in a row, the second one smaller so
that it finds the first call's partial rows in the scratch."""
import ctypes

import pytest
import torch

from helpers import assert_close, colsum_slack, gen, to_np32

pytestmark = pytest.mark.gpu


def _inputs(M, N, dtype, wdtype, seed, gpu):
    g = gen(seed)
    x = torch.randn(M, N, generator=g).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    w = (1 + 0.02 * torch.randn(N, generator=g)).to(wdtype)
    return x.to(gpu), dy.to(gpu), w.to(gpu)


def _both(cabi, x, dy, w, want_dx=True, want_dw=True):
    """-> ((dx, dw) of the static entry point, (dx, dw) of the allocating one), each on its own
    pre-filled output buffers."""
    M, N = x.shape
    _, rstd = cabi.rms_norm_fwd(x, w, 1e-6)
    dx_s = torch.full_like(x, 7.0) if want_dx else None
    dw_s = torch.full_like(w, 7.0) if want_dw else None
    # the first launch of a kernel loads its code object (and with it the static array) into
    # device memory; after that a call must leave the free device memory exactly as it found it
    cabi.rms_norm_bwd_static(dy, x, rstd, w, dx_s, dw_s, w_dtype=w.dtype)
    for t in (dx_s, dw_s):
        if t is not None:
            t.fill_(7.0)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    cabi.rms_norm_bwd_static(dy, x, rstd, w, dx_s, dw_s, w_dtype=w.dtype)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # no device memory was taken
    dx_r, dw_r = cabi.rms_norm_bwd(dy, x, rstd, w, want=(want_dx, want_dw), w_dtype=w.dtype)
    return rstd, (dx_s, dw_s), (dx_r, dw_r)


def _check_oracle(oracle, x, dy, w, rstd, got, dtype):
    N = x.shape[1]
    odx, odw = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rstd), to_np32(w))
    if got[0] is not None:
        assert_close(got[0], odx, dtype, "static dx")
    if got[1] is not None:
        # a float32 column sum over all rows carries its own rounding (helpers.colsum_slack)
        sl = None
        if got[1].dtype == torch.float32:
            sl = colsum_slack(dy.cpu().double() * x.cpu().double() * rstd.cpu().double().reshape(-1, 1))
        assert_close(got[1], odw, got[1].dtype, "static dweight", slack=sl)


@pytest.mark.parametrize("dtype,wdtype", [(torch.bfloat16, torch.bfloat16),
                                          (torch.float16, torch.float32),
                                          (torch.float32, torch.float32)], ids=str)
def test_two_calls_in_a_row_second_smaller(cabi, oracle, gpu, dtype, wdtype):
    for (M, N, seed) in ((2048, 4096, 91), (300, 1000, 92)):
        print("case static scratch", dtype, wdtype, (M, N), flush=True)
        x, dy, w = _inputs(M, N, dtype, wdtype, seed, gpu)
        rstd, got, ref = _both(cabi, x, dy, w)
        assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
        _check_oracle(oracle, x, dy, w, rstd, got, dtype)


def test_split_rows_and_partial_requests(cabi, oracle, gpu):
    # a few very long rows: the split-row partial sums sit behind the column sums in the scratch
    print("case static scratch split rows", flush=True)
    x, dy, w = _inputs(2, 300000, torch.bfloat16, torch.bfloat16, 93, gpu)
    p = cabi.plan(cabi.OP_RMS_NORM_BWD, 2, 300000, cabi.BF16, cabi.BF16)
    assert p["row_chunks"] > 1
    rstd, got, ref = _both(cabi, x, dy, w)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    _check_oracle(oracle, x, dy, w, rstd, got, torch.bfloat16)
    # then a smaller resident call, dX only and dweight only
    x, dy, w = _inputs(512, 2048, torch.bfloat16, torch.bfloat16, 94, gpu)
    for want in ((True, False), (False, True)):
        rstd, got, ref = _both(cabi, x, dy, w, *want)
        for a, b in zip(got, ref):
            assert (a is None and b is None) or torch.equal(a, b)
        _check_oracle(oracle, x, dy, w, rstd, got, torch.bfloat16)


def test_rows_of_three_packs_a_lane_on_1024_lanes(cabi, oracle, gpu):
    # hidden 18432: 256 partial rows of 18432 floats (18 MiB of the scratch), then a smaller call
    for (M, N, seed) in ((300, 18432, 95), (64, 4096, 96)):
        print("case static scratch", (M, N), flush=True)
        x, dy, w = _inputs(M, N, torch.bfloat16, torch.bfloat16, seed, gpu)
        rstd, got, ref = _both(cabi, x, dy, w)
        assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
        _check_oracle(oracle, x, dy, w, rstd, got, torch.bfloat16)


def test_limit_is_an_error_before_any_launch(cabi, gpu):
    L = cabi.lib()
    limit = L.mi355x_rms_norm_bwd_static_limit_bytes()
    assert limit == 32 << 20
    # the launch plans of this build stay within the limit (at most 512 partial rows of 8192
    # floats, or 256 of up to 32768: 32 MiB); a forced grid of eight workgroups a compute unit
    # does not
    for (m, n) in ((16384, 8192), (16384, 16384), (4096, 18432), (4096, 32768), (4096, 65536)):
        assert L.mi355x_rms_norm_bwd_workspace_bytes(m, n, cabi.BF16, cabi.BF16, 1) <= limit
    for (m, n) in ((16384, 4096), (4096, 16384), (16384, 8192), (2048, 32768), (64, 1 << 20)):
        assert L.mi355x_rms_norm_bwd_workspace_bytes(m, n, cabi.F32, cabi.F32, 1) <= limit
        assert L.mi355x_rms_norm_bwd_workspace_bytes(m, n, cabi.F16, cabi.F32, 1) <= limit
    M, N = 16384, 8192
    # real device memory behind every pointer: should a validation regression ever let one of
    # these calls launch, it reads and writes memory it owns instead of faulting the GPU
    bufs = [torch.zeros(M * N, dtype=torch.bfloat16, device=gpu) for _ in range(3)]
    stat = torch.ones(M, device=gpu)
    wt = [torch.ones(N, dtype=torch.bfloat16, device=gpu) for _ in range(2)]
    P = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    try:
        cabi.set_override(cabi.OP_RMS_NORM_BWD, 0, 0, 0, 8)
        need = L.mi355x_rms_norm_bwd_workspace_bytes(M, N, cabi.BF16, cabi.BF16, 1)
        assert need > limit
        assert L.mi355x_rms_norm_bwd_static(P(bufs[0]), P(bufs[1]), P(stat), P(wt[0]), P(bufs[2]),
                                            P(wt[1]), M, N, cabi.BF16, cabi.BF16, stream) == -6
    finally:
        cabi.clear_overrides()
    torch.cuda.synchronize()
    assert float(bufs[2].float().abs().max()) == 0.0 and float(wt[1].float().min()) == 1.0  # untouched
    assert "static" in cabi.error_string(-6)
    # dX alone needs no scratch at that size: accepted (nothing launched here: empty problem)
    assert L.mi355x_rms_norm_bwd_static(P(bufs[0]), P(bufs[1]), P(stat), P(wt[0]), P(bufs[2]), None,
                                        0, N, cabi.BF16, cabi.BF16, stream) == 0
