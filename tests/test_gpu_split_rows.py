"""Few rows, each far too long for the registers: the split-row LayerNorm / RMSNorm kernels (the
regime of Norm.h:632-812 in intel/torch-xpu-ops, where one row spans several work-groups), through
the extern "C" ABI against the CPU oracle, against the one-workgroup-per-row kernels, and for
run-to-run determinism.  Tolerances as everywhere: float32 rtol = atol = 1e-5; 16-bit atol 1e-2,
rtol 1.6e-2."""
import ctypes

import pytest
import torch

from helpers import assert_close, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _mk(M, N, dtype, seed, shift=0.0):
    g = gen(seed)
    x = (shift + torch.randn(M, N, generator=g)).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(N, generator=g)).to(dtype)
    return x, dy, gamma, beta


def _check_all(cabi, oracle, gpu, x, dy, gamma, beta, dtype, what):
    M, N = x.shape
    xg, dyg, gg, bg = (offset_view(t.to(gpu), 1) for t in (x, dy, gamma, beta))
    y, mean, rstd = cabi.layer_norm_fwd(xg, gg, bg, 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    assert_close(y, oy, dtype, "layer_norm y " + what)
    assert_close(mean, om.reshape(-1), dtype, "mean " + what)
    assert_close(rstd, orr.reshape(-1), dtype, "rstd " + what)
    dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
    odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                          to_np32(rstd), to_np32(gamma))
    assert_close(dx, odx, dtype, "layer_norm dx " + what)
    assert_close(dg, odg, dtype, "dgamma " + what)
    assert_close(db, odb, dtype, "dbeta " + what)
    ry, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
    roy, ror = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(gamma), 1e-6)
    assert_close(ry, roy, dtype, "rms_norm y " + what)
    assert_close(rr, ror.reshape(-1), dtype, "rms rstd " + what)
    rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
    rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
    assert_close(rdx, rodx, dtype, "rms_norm dx " + what)
    assert_close(rdg, rodg, dtype, "rms dgamma " + what)
    return (y, mean, rstd, dx, dg, db, ry, rr, rdx, rdg)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", [(1, 300000), (3, 150001), (2, 1 << 18)], ids=str)
def test_few_long_rows_are_split_and_match_the_oracle(cabi, oracle, gpu, dtype, shape):
    M, N = shape
    print("case split rows", dtype, shape, flush=True)
    code = cabi.dtype_code(dtype)
    for op in (cabi.OP_LAYER_NORM_FWD, cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_FWD,
               cabi.OP_RMS_NORM_BWD):
        p = cabi.plan(op, M, N, code, code)
        assert p["resident"] == 0 and p["row_chunks"] > 1, p
    x, dy, gamma, beta = _mk(M, N, dtype, 81)
    first = _check_all(cabi, oracle, gpu, x, dy, gamma, beta, dtype, "split")
    # partial sums are added in a fixed order: a second run gives the same bits
    again = _check_all(cabi, oracle, gpu, x, dy, gamma, beta, dtype, "split, second run")
    for a, b in zip(first, again):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_forced_chunk_counts_against_one_workgroup_per_row(cabi, oracle, gpu, dtype):
    """G = -1 forces the streaming kernels; V = 1 keeps a row on one workgroup, V > 1 cuts it into
    that many chunks.  Ragged row lengths, rows with a large mean, a short last chunk."""
    ops = (cabi.OP_LAYER_NORM_FWD, cabi.OP_LAYER_NORM_BWD, cabi.OP_RMS_NORM_FWD, cabi.OP_RMS_NORM_BWD)
    code = cabi.dtype_code(dtype)
    try:
        for (M, N, shift) in ((5, 40000, 0.0), (3, 33333, 3.0), (4, 8192 * 3 + 1, -2.0)):
            x, dy, gamma, beta = _mk(M, N, dtype, 82, shift)
            results = {}
            for chunks in (1, 2, 3, 7):
                for op in ops:
                    cabi.set_override(op, -1, chunks)
                p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)
                assert p["resident"] == 0
                assert (p["row_chunks"] > 1) == (chunks > 1), (chunks, p)
                print("forced chunks", dtype, (M, N), chunks, p["row_chunks"], flush=True)
                results[chunks] = _check_all(cabi, oracle, gpu, x, dy, gamma, beta, dtype,
                                             "chunks=%d" % chunks)
            # dbeta = sum dy does not depend on how the rows were cut (dgamma does, through the
            # last bits of the mean / rstd each forward produced)
            for chunks in (2, 3, 7):
                assert torch.equal(results[chunks][5], results[1][5])
    finally:
        cabi.clear_overrides()


def test_constant_rows_give_beta_bit_for_bit(cabi, gpu):
    """x - mean is exactly zero on a constant row (a mean error would be amplified by rstd = 316),
    also when the row's sums come from several workgroups."""
    for dtype in DTYPES:
        M, N = 2, 200000
        x = torch.full((M, N), 1.5, dtype=dtype, device=gpu)
        g = gen(83)
        gamma = torch.randn(N, generator=g).to(dtype).to(gpu)
        beta = torch.randn(N, generator=g).to(dtype).to(gpu)
        y, mean, rstd = cabi.layer_norm_fwd(x, gamma, beta, 1e-5)
        assert torch.equal(y, beta.expand(M, N))
        assert torch.equal(mean, torch.full((M,), 1.5, device=gpu))
        assert_close(rstd, torch.full((M,), 316.227783203125), torch.float32, "rstd")


def test_fallbacks_keep_a_row_on_one_workgroup(cabi, oracle, gpu):
    """Without mean / rstd outputs, with Y on top of X, or with a workspace that only holds the
    column sums, the call still succeeds: the row is not split."""
    L = cabi.lib()
    P = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    M, N = 2, 150000
    x, dy, gamma, beta = _mk(M, N, torch.float32, 84)
    xg, dyg, gg, bg = (t.to(gpu) for t in (x, dy, gamma, beta))
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    F32 = cabi.F32
    # no statistics wanted
    y = torch.empty_like(xg)
    assert L.mi355x_layer_norm_fwd(P(xg), P(gg), P(bg), P(y), None, None, M, N, 1e-5, F32, F32,
                                   stream) == 0
    assert_close(y, oy, torch.float32, "y without statistics")
    # in place
    xin = xg.clone()
    mean = torch.empty(M, device=gpu)
    rstd = torch.empty(M, device=gpu)
    assert L.mi355x_layer_norm_fwd(P(xin), P(gg), P(bg), P(xin), P(mean), P(rstd), M, N, 1e-5, F32,
                                   F32, stream) == 0
    assert_close(xin, oy, torch.float32, "y in place")
    assert_close(mean, om.reshape(-1), torch.float32, "mean in place")
    # backward with the column-sum workspace only, and dX only with no workspace at all
    odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), om.reshape(-1),
                                          orr.reshape(-1), to_np32(gamma))
    mean_g = torch.from_numpy(om.reshape(-1).copy()).to(gpu)
    rstd_g = torch.from_numpy(orr.reshape(-1).copy()).to(gpu)
    full = L.mi355x_layer_norm_bwd_workspace_bytes(M, N, F32, F32, 1, 1)
    dx_only = L.mi355x_layer_norm_bwd_workspace_bytes(M, N, F32, F32, 0, 0)
    assert 0 < dx_only < full
    cols = full - dx_only
    ws = torch.empty(cols, dtype=torch.uint8, device=gpu)
    dx = torch.empty_like(xg)
    dg = torch.empty_like(gg)
    db = torch.empty_like(gg)
    assert L.mi355x_layer_norm_bwd(P(dyg), P(xg), P(mean_g), P(rstd_g), P(gg), P(dx), P(dg), P(db),
                                   P(ws), cols, M, N, F32, F32, stream) == 0
    assert_close(dx, odx, torch.float32, "dx, short workspace")
    assert_close(dg, odg, torch.float32, "dgamma, short workspace")
    assert L.mi355x_layer_norm_bwd(P(dyg), P(xg), P(mean_g), P(rstd_g), P(gg), P(dx), P(dg), P(db),
                                   P(ws), cols - 1, M, N, F32, F32, stream) == -4  # ROWNORM_ERR_WORKSPACE
    dx2 = torch.empty_like(xg)
    assert L.mi355x_layer_norm_bwd(P(dyg), P(xg), P(mean_g), P(rstd_g), P(gg), P(dx2), None, None,
                                   None, 0, M, N, F32, F32, stream) == 0
    assert_close(dx2, odx, torch.float32, "dx, no workspace")


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32], ids=str)
def test_one_partial_row_writes_the_column_sums_itself(cabi, oracle, gpu, wdtype):
    """Rows so long that the columns alone fill the machine (bf16 from 1048576 elements) take one
    partial row, and the column-sum kernels then write dgamma / dbeta themselves, rounded once
    from the fp32 sums, without a second stage (the reference's second stage is the at::sum over
    its block buffers, LayerNormKernels.cpp:1312-1314): each wanted alone, both with dX (the fused
    dX + column-sum kernel), a ragged row end, and RMSNorm."""
    for (M, N) in ((3, 1048576 + 24), (5, 1048576 + 3)):
        p = cabi.plan(cabi.OP_LAYER_NORM_BWD, M, N, cabi.BF16, cabi.dtype_code(wdtype))
        assert p["resident"] == 0 and p["partial_rows"] == 1, p
        g = gen(1700 + M)
        x = (0.5 + torch.randn(M, N, generator=g)).bfloat16()
        dy = torch.randn(M, N, generator=g).bfloat16()
        gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdtype)
        xg, dyg, gg = x.to(gpu), dy.to(gpu), gamma.to(gpu)
        what = "[%d, %d] weights %s" % (M, N, wdtype)
        _, mean, rstd = cabi.layer_norm_fwd(xg, gg, None, 1e-5)
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean),
                                              to_np32(rstd), to_np32(gamma))
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg)
        assert_close(dx, odx, torch.bfloat16, "dx " + what)
        assert_close(dg, odg, wdtype, "dgamma " + what)
        assert_close(db, odb, wdtype, "dbeta " + what)
        _, dg1, n1 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(False, True, False))
        _, n2, db1 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(False, False, True))
        assert n1 is None and n2 is None
        assert_close(dg1, odg, wdtype, "dgamma alone " + what)
        assert_close(db1, odb, wdtype, "dbeta alone " + what)
        dx2, dg2, n3 = cabi.layer_norm_bwd(dyg, xg, mean, rstd, gg, want=(True, True, False))
        assert n3 is None and torch.equal(dx2, dx) and torch.equal(dg2, dg)
        _, rr = cabi.rms_norm_fwd(xg, gg, 1e-6)
        rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rr, gg)
        rodx, rodg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(rr), to_np32(gamma))
        assert_close(rdx, rodx, torch.bfloat16, "rms dx " + what)
        assert_close(rdg, rodg, wdtype, "rms dgamma " + what)
