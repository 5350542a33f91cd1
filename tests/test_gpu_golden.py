"""The HIP kernels, through the extern "C" ABI, against the committed PyTorch-CPU-ATen golden
vectors of the main family (tests/golden/aten_cpu_golden.npz: ln_*, lnmix_*, rms_*, sm_*, lsm_* --
the inputs with +-1e4 outliers, a constant row, a fully masked row, and the CPU ops' own outputs in
the inputs' dtype, 16-bit outputs included).  Same bounds as tests/test_oracle_golden.py holds the
oracle to: float32 rtol = atol = 1e-5, 16-bit atol 1e-2 / rtol 1.6e-2.  Where a result is a sum
(the backward, rstd) the stored CPU value is itself a float32 (or rounded 16-bit) evaluation that
sits some distance from the float64 oracle on these +-1e4 inputs; the comparison against it
carries exactly that measured distance, |CPU golden - oracle| per element, as slack, so a HIP
result may be as far from the golden value as the tolerance plus the golden value's own error and
no farther (no blanket factors).  The saved statistics
follow the GPU contract (float32, src/ATen/native/xpu/LayerNorm.cpp:72-75 in the reference) and are
compared with the CPU op's 16-bit ones at the 16-bit tolerance."""
import pytest
import torch

from helpers import GOLDEN_DTYPES, abs_err, assert_close, load_golden, offset_view, to_np32

pytestmark = pytest.mark.gpu

CASES = load_golden()
NAMES = sorted(CASES)


@pytest.mark.parametrize("case", NAMES)
@pytest.mark.parametrize("offset", [0, 1], ids=["aligned", "off1"])
def test_layer_norm_and_rms_norm_against_golden(cabi, oracle, gpu, case, offset):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    N = c["x"].shape[1]
    put = (lambda t: offset_view(t.to(gpu), offset)) if offset else (lambda t: t.to(gpu))
    x, dy = put(c["x"]), put(c["dy"])
    own = lambda golden, exact: abs_err(golden, exact)  # noqa: E731  (the golden value's own error)
    variants = (("ln", c["gamma"], c["beta"]),)
    if dt != torch.float32:
        variants += (("lnmix", c["gamma"].float(), c["beta"].float()),)
    for pre, gamma, beta in variants:
        y, mean, rstd = cabi.layer_norm_fwd(x, put(gamma), put(beta), 1e-5)
        assert y.dtype == dt and mean.dtype == torch.float32
        assert_close(y, c[pre + "_y"], dt, case + " " + pre + " y")
        assert_close(mean, c[pre + "_mean"], dt, case + " " + pre + " mean")
        assert_close(rstd, c[pre + "_rstd"], dt, case + " " + pre + " rstd")
        assert torch.equal(y[0].cpu(), beta.to(dt))  # the constant row: beta bit for bit
        # backward from the golden statistics, as the CPU op consumed them
        dx, dg, db = cabi.layer_norm_bwd(dy, x, put(c[pre + "_mean"].float()),
                                         put(c[pre + "_rstd"].float()), put(gamma))
        assert dg.dtype == gamma.dtype and db.dtype == gamma.dtype
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(c["dy"]), to_np32(c["x"]), (N,),
                                              to_np32(c[pre + "_mean"]), to_np32(c[pre + "_rstd"]),
                                              to_np32(gamma))
        assert_close(dx, odx, dt, case + " " + pre + " dx vs oracle")
        assert_close(dx, c[pre + "_dx"], dt, case + " " + pre + " dx",
                     slack=own(c[pre + "_dx"], odx))
        assert_close(dg, c[pre + "_dgamma"], dt, case + " " + pre + " dgamma",
                     slack=own(c[pre + "_dgamma"], odg))
        assert_close(db, c[pre + "_dbeta"], dt, case + " " + pre + " dbeta",
                     slack=own(c[pre + "_dbeta"], odb))
    y, rstd = cabi.rms_norm_fwd(x, put(c["gamma"]), 1e-6)
    assert_close(y, c["rms_y"], dt, case + " rms y")
    _, orstd = oracle.rms_norm_fwd(to_np32(c["x"]), (N,), to_np32(c["gamma"]), 1e-6)
    assert_close(rstd, orstd.reshape(-1), torch.float32, case + " rms rstd vs oracle")
    assert_close(rstd, c["rms_rstd"], torch.float32, case + " rms rstd",
                 slack=own(c["rms_rstd"], orstd.reshape(-1)))
    dx, dg = cabi.rms_norm_bwd(dy, x, put(c["rms_rstd"]), put(c["gamma"]))
    odx, odg = oracle.rms_norm_bwd(to_np32(c["dy"]), to_np32(c["x"]), (N,), to_np32(c["rms_rstd"]),
                                   to_np32(c["gamma"]))
    assert_close(dx, odx, dt, case + " rms dx vs oracle")
    assert_close(dx, c["rms_dx"], dt, case + " rms dx", slack=own(c["rms_dx"], odx))
    assert_close(dg, c["rms_dgamma"], dt, case + " rms dgamma", slack=own(c["rms_dgamma"], odg))


@pytest.mark.parametrize("case", NAMES)
@pytest.mark.parametrize("offset", [0, 1], ids=["aligned", "off1"])
def test_softmax_against_golden(cabi, oracle, gpu, case, offset):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    put = (lambda t: offset_view(t.to(gpu), offset)) if offset else (lambda t: t.to(gpu))
    x, dy = put(c["sm_x"]), put(c["dy"])
    for is_log, nm in ((False, "sm"), (True, "lsm")):
        y = cabi.softmax_fwd(x, is_log)
        assert y.dtype == dt
        assert_close(y, c[nm + "_y"], dt, case + " " + nm + " y")
        assert bool(torch.isnan(y[2]).all())  # the fully masked row
        gi = cabi.softmax_bwd(dy, put(c[nm + "_y"]), is_log)
        ogi = oracle.softmax_bwd(to_np32(c["dy"]), to_np32(c[nm + "_y"]), is_log)
        assert_close(gi, c[nm + "_gi"], dt, case + " " + nm + " grad_input",
                     slack=abs_err(c[nm + "_gi"], ogi))
