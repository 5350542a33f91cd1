"""Rows built to defeat a badly centred variance: the statistics of LayerNorm (and GroupNorm, whose
forward shares the scheme) on rows whose head lies far from the rest of the row.

The 16-bit resident kernels centre their one-round sums on the median of the row's first three
elements; the few-long-rows kernels centre float64 sums on it; the float32 resident and multi-pass
kernels take a true mean first.  Two heads are fed to every one of those kernels: `x[0:3] = 0`
before a row of `offset + N(0, 1)` (a padded / BOS-like head: the centre is `offset` standard
deviations away), and `x[0:2] = +1e4` (6e4 in float16) before a row of N(0, 1) (two of the three
centre candidates are outliers).  Everything is compared with the float64 CPU oracle at the
family's tolerances -- float32 rtol = atol = 1e-5, 16-bit atol 1e-2 / rtol 1.6e-2 -- mean and rstd
included.  Non-finite rows (a NaN or an inf element) must give the statistics CPU ATen gives.

The Welford merge these kernels stand in for: WelfordOps::combine,
src/ATen/native/xpu/sycl/SharedReduceOps.h:71-88 of intel/torch-xpu-ops."""
import pytest
import torch

from helpers import assert_close, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu


def _weights(N, dtype, seed):
    g = gen(seed)
    return ((1 + 0.1 * torch.randn(N, generator=g)).to(dtype),
            (0.1 * torch.randn(N, generator=g)).to(dtype))


def _zero_head(M, N, offset, dtype, seed):
    x = offset + torch.randn(M, N, generator=gen(seed))
    x[:, 0:3] = 0.0
    return x.to(dtype)


def _outlier_head(M, N, dtype, seed):
    x = torch.randn(M, N, generator=gen(seed))
    x[:, 0:2] = 6e4 if dtype == torch.float16 else 1e4
    return x.to(dtype)


def _check_layer_norm(cabi, oracle, gpu, x, dtype, what, off=0):
    M, N = x.shape
    gamma, beta = _weights(N, dtype, 5)
    put = (lambda t: offset_view(t.to(gpu), off)) if off else (lambda t: t.to(gpu))
    y, mean, rstd = cabi.layer_norm_fwd(put(x), put(gamma), put(beta), 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(gamma), to_np32(beta), 1e-5)
    ex = (assert_close(mean, om.reshape(-1), dtype, "mean, " + what),
          assert_close(rstd, orr.reshape(-1), dtype, "rstd, " + what),
          assert_close(y, oy, dtype, "y, " + what))
    print("  %-58s mean %.3f rstd %.3f y %.3f of the tolerance" % ((what,) + ex), flush=True)


# (rows, N): resident on few lanes, on 512 lanes, the float32 / 16-bit resident maxima, and rows
# beyond the registers (few rows: split over workgroups)
RESIDENT = {torch.float32: [(9, 4096), (5, 16384), (3, 32768)],
            torch.float16: [(9, 4096), (5, 16384), (3, 32768)],
            torch.bfloat16: [(9, 4096), (5, 16384), (3, 32768)]}
LONG = [(2, 131072), (2, 300000), (1, 300001)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_layer_norm_resident_kernels(cabi, oracle, gpu, dtype):
    code = cabi.dtype_code(dtype)
    for (M, N) in RESIDENT[dtype]:
        assert cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)["resident"] == 1
        for offset in (100.0, 1000.0):
            _check_layer_norm(cabi, oracle, gpu, _zero_head(M, N, offset, dtype, 31), dtype,
                              "resident %s [%d, %d] zero head, offset %g" % (dtype, M, N, offset))
        _check_layer_norm(cabi, oracle, gpu, _outlier_head(M, N, dtype, 32), dtype,
                          "resident %s [%d, %d] outlier head" % (dtype, M, N))
    # ragged rows and pointers off 16-byte alignment take the general kernels
    for (M, N) in ((7, 4097), (3, 16383)):
        _check_layer_norm(cabi, oracle, gpu, _zero_head(M, N, 1000.0, dtype, 33), dtype,
                          "general %s [%d, %d] zero head, offset 1000" % (dtype, M, N), off=1)
        _check_layer_norm(cabi, oracle, gpu, _outlier_head(M, N, dtype, 34), dtype,
                          "general %s [%d, %d] outlier head" % (dtype, M, N), off=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("chunks", [0, 1, 5], ids=["planned_split", "one_workgroup_per_row",
                                                    "five_chunks"])
def test_layer_norm_long_rows(cabi, oracle, gpu, dtype, chunks):
    """chunks = 0: the planner's own split over workgroups; 1: the multi-pass kernel, one
    workgroup a row; 5: a forced split with a short last chunk."""
    code = cabi.dtype_code(dtype)
    try:
        if chunks:
            cabi.set_override(cabi.OP_LAYER_NORM_FWD, -1, chunks)
        for (M, N) in LONG:
            p = cabi.plan(cabi.OP_LAYER_NORM_FWD, M, N, code, code)
            assert p["resident"] == 0 and (p["row_chunks"] > 1) == (chunks != 1), p
            for offset in (100.0, 1000.0):
                _check_layer_norm(cabi, oracle, gpu, _zero_head(M, N, offset, dtype, 35), dtype,
                                  "%d chunks %s [%d, %d] zero head, offset %g" % (
                                      p["row_chunks"], dtype, M, N, offset), off=1)
            _check_layer_norm(cabi, oracle, gpu, _outlier_head(M, N, dtype, 36), dtype,
                              "%d chunks %s [%d, %d] outlier head" % (p["row_chunks"], dtype, M, N),
                              off=1)
    finally:
        cabi.clear_overrides()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_group_norm(cabi, oracle, gpu, dtype):
    """(sample, group) slabs of 4096 and 16384 elements (registers) and 131072 (two-pass kernel)."""
    for (N, C, H, W, groups) in ((3, 8, 32, 32, 2), (2, 32, 32, 32, 2), (2, 4, 256, 256, 2)):
        L = C // groups * H * W
        plan = cabi.group_norm_plan(False, N, C, H * W, groups, cabi.dtype_code(dtype))
        assert plan["resident"] == (1 if L <= 16384 else 0), plan
        gamma, beta = _weights(C, dtype, 6)
        for kind in ("zero head, offset 100", "zero head, offset 1000", "outlier head"):
            if kind == "outlier head":
                rows = _outlier_head(N * groups, L, dtype, 37)
            else:
                rows = _zero_head(N * groups, L, float(kind.split()[-1]), dtype, 38)
            x = rows.reshape(N, C, H, W)
            y, mean, rstd = cabi.group_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), groups, 1e-5)
            oy, om, orr = oracle.group_norm_fwd(to_np32(x), groups, to_np32(gamma), to_np32(beta),
                                                1e-5)
            what = "group_norm %s L=%d %s" % (dtype, L, kind)
            # the statistics come back in the weight dtype: one rounding to 16 bits on top
            ex = (assert_close(mean, om, dtype, "mean, " + what),
                  assert_close(rstd, orr, dtype, "rstd, " + what),
                  assert_close(y, oy, dtype, "y, " + what))
            print("  %-58s mean %.3f rstd %.3f y %.3f of the tolerance" % ((what,) + ex), flush=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_non_finite_rows_give_what_cpu_aten_gives(cabi, gpu, dtype):
    """A NaN or an inf element makes mean, rstd and the whole row of y NaN (inf - inf in the CPU
    kernel's Welford recurrence).  The variance clamp must not turn that into a finite rstd."""
    try:
        for (N, force) in ((64, None), (4096, None), (4097, None), (40000, None), (40000, (-1, 1)),
                           (300000, None)):
            if force:
                cabi.set_override(cabi.OP_LAYER_NORM_FWD, *force)
            x = torch.randn(4, N, generator=gen(39)).to(dtype)
            x[1, N // 3] = float("nan")
            x[2, N // 2] = float("inf")
            gamma, beta = _weights(N, dtype, 7)
            y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), gamma.to(gpu), beta.to(gpu), 1e-5)
            cy, cm, cr = torch.ops.aten.native_layer_norm(x.float(), [N], gamma.float(),
                                                          beta.float(), 1e-5)
            assert bool(torch.isnan(cr[1]).all()) and bool(torch.isnan(cr[2]).all())  # CPU ATen
            for r in (1, 2):
                assert bool(torch.isnan(y[r]).all()), (dtype, N, r)
                assert bool(torch.isnan(rstd[r])), (dtype, N, r)
            assert bool(torch.isnan(cm[1]).all()) and bool(torch.isnan(cm[2]).all())  # CPU ATen
            assert bool(torch.isnan(mean[1])) and bool(torch.isnan(mean[2]))
            for r in (0, 3):  # the finite rows are untouched
                assert_close(y[r], cy[r], dtype, "finite row %d beside non-finite ones" % r)
            cabi.clear_overrides()
        # GroupNorm: resident and two-pass
        for (C, H) in ((8, 16), (4, 256)):
            x = torch.randn(2, C, H, H, generator=gen(40)).to(dtype)
            x[0, 0, 1, 1] = float("nan")
            x[1, C - 1, 2, 3] = float("inf")
            y, mean, rstd = cabi.group_norm_fwd(x.to(gpu), None, None, 2, 1e-5)
            assert bool(torch.isnan(rstd[0, 0])) and bool(torch.isnan(rstd[1, 1]))
            assert bool(torch.isnan(mean[0, 0])) and bool(torch.isnan(mean[1, 1]))
            assert bool(torch.isnan(y[0, :C // 2]).all()) and bool(torch.isnan(y[1, C // 2:]).all())
            assert bool(torch.isfinite(y[0, C // 2:]).all()) and bool(torch.isfinite(y[1, :C // 2]).all())
    finally:
        cabi.clear_overrides()
