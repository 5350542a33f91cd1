"""The CPU oracle against the committed PyTorch-CPU-ATen golden vectors (tests/golden/).

The vectors were produced by the installed torch wheel, not by the reference repository (which
holds no golden files for this path and cannot be run here).  This is the check that ties the
oracle to the parity target named for the path: fp32 within rtol = atol = 1e-5, 16-bit outputs
within atol 1e-2 / rtol 1.6e-2.  Where the fp32 CPU kernel itself sums a long row in float32
(dgamma/dbeta over rows with +-1e4 outliers, log_softmax backward) the bound is widened by a
stated factor; those are the CPU kernel's rounding, not the oracle's.
"""
import numpy as np
import pytest
import torch

from helpers import GOLDEN_DTYPES, assert_close, load_golden, to_np32

CASES = load_golden()
NAMES = sorted(CASES)


@pytest.mark.parametrize("case", NAMES)
def test_layer_norm_matches_golden(oracle, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    N = c["x"].shape[1]
    for pre, gk, bk in (("ln", c["gamma"], c["beta"]),) + (
            (("lnmix", c["gamma"].float(), c["beta"].float()),) if dt != torch.float32 else ()):
        y, mean, rstd = oracle.layer_norm_fwd(to_np32(c["x"]), (N,), to_np32(gk), to_np32(bk), 1e-5)
        assert_close(y, c[pre + "_y"], dt, case + " y")
        assert_close(mean.reshape(-1), c[pre + "_mean"], dt, case + " mean")
        assert_close(rstd.reshape(-1), c[pre + "_rstd"], dt, case + " rstd")
        # backward from the golden (possibly 16-bit) statistics, as the CPU op consumed them
        dx, dg, db = oracle.layer_norm_bwd(to_np32(c["dy"]), to_np32(c["x"]), (N,),
                                           to_np32(c[pre + "_mean"]), to_np32(c[pre + "_rstd"]),
                                           to_np32(gk))
        # fp32 CPU dX uses ds/db sums of dy*gamma*x, which cancel badly on the +-1e4 rows
        assert_close(dx, c[pre + "_dx"], dt, case + " dx", scale=4.0 if dt == torch.float32 else 1.0)
        # (the CPU kernel's mixed-precision dgamma/dbeta are float32 tensors holding values
        # rounded to the 16-bit row dtype, so the row dtype's tolerance applies)
        assert_close(dg, c[pre + "_dgamma"], dt, case + " dgamma", scale=4.0)
        assert_close(db, c[pre + "_dbeta"], dt, case + " dbeta", scale=4.0)
    # the all-constant row: y is beta bit for bit, mean the constant, rstd 1/sqrt(eps)
    y, mean, rstd = oracle.layer_norm_fwd(to_np32(c["x"]), (N,), to_np32(c["gamma"]),
                                          to_np32(c["beta"]), 1e-5)
    assert np.array_equal(y[0], to_np32(c["beta"]))
    assert mean[0, 0] == np.float32(1.5)
    assert rstd[0, 0] == pytest.approx(316.227783203125, rel=1e-7)


@pytest.mark.parametrize("case", NAMES)
def test_rms_norm_matches_golden(oracle, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    N = c["x"].shape[1]
    y, rstd = oracle.rms_norm_fwd(to_np32(c["x"]), (N,), to_np32(c["gamma"]), 1e-6)
    assert_close(y, c["rms_y"], dt, case + " y")
    assert_close(rstd.reshape(-1), c["rms_rstd"], torch.float32, case + " rstd", scale=2.0)
    dx, dg = oracle.rms_norm_bwd(to_np32(c["dy"]), to_np32(c["x"]), (N,), to_np32(c["rms_rstd"]),
                                 to_np32(c["gamma"]))
    # golden backward is autograd through the composite: 16-bit intermediates round more often
    assert_close(dx, c["rms_dx"], dt, case + " dx", scale=4.0)
    assert_close(dg, c["rms_dgamma"], dt, case + " dgamma", scale=4.0)


@pytest.mark.parametrize("case", NAMES)
def test_softmax_matches_golden(oracle, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    for is_log, nm in ((False, "sm"), (True, "lsm")):
        y = oracle.softmax_fwd(to_np32(c["sm_x"]), is_log)
        assert_close(y, c[nm + "_y"], dt, case + " " + nm + " y")
        assert np.all(np.isnan(y[2]))  # the fully masked row
        gi = oracle.softmax_bwd(to_np32(c["dy"]), to_np32(c[nm + "_y"]), is_log)
        # log_softmax backward subtracts exp(y) * sum(g); the fp32 CPU kernel's row sum of 4097
        # terms is only good to a few 1e-5
        assert_close(gi, c[nm + "_gi"], dt, case + " " + nm + " grad_input",
                     scale=8.0 if (is_log and dt == torch.float32) else 1.0)


@pytest.mark.parametrize("case", NAMES)
def test_safe_and_masked_softmax_match_golden(oracle, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    y = oracle.safe_softmax_fwd(to_np32(c["sm_x"]))
    assert_close(y, c["ssm_y"], dt, case + " safe y")
    assert np.all(y[2] == 0)  # the all -inf row
    mask = c["msk"].numpy().astype(bool)
    y = oracle.masked_softmax_fwd(to_np32(c["msm_x"]), mask)
    assert_close(y, c["msm_y"], dt, case + " masked y")
    if mask.shape[0] > 4:
        assert np.all(np.isnan(y[4]))  # every element masked
    assert np.all(y[mask & ~np.isnan(y)] == 0)
    gi = oracle.masked_softmax_bwd(to_np32(c["dy"]), to_np32(c["msm_y"]), mask)
    assert_close(gi, c["msm_gi"], dt, case + " masked grad_input")
    assert np.all(gi[mask] == 0)
