"""Shared input generators, tolerances and comparison helpers for the test suite."""
import numpy as np
import torch

# Tolerances stated for this operator family: float32 results within rtol = atol = 1e-5 of the
# CPU result; float16 / bfloat16 results within atol 1e-2, rtol 1.6e-2 of a reference that
# accumulates in float32 or better (saved mean / rstd included).
TOL = {torch.float32: (1e-5, 1e-5), torch.float16: (1.6e-2, 1e-2), torch.bfloat16: (1.6e-2, 1e-2)}


def tol_for(dtype):
    return TOL[dtype]


def to_np32(t):
    if t is None:
        return None
    return t.detach().to("cpu", torch.float32).contiguous().numpy()


def excess(actual, expected, rtol, atol, slack=None):
    """max over elements of |a - e| / (atol + rtol * |e| [+ slack]); <= 1 passes.
    NaN/inf positions must agree exactly."""
    a = torch.as_tensor(actual).detach().to("cpu", torch.float64).reshape(-1)
    e = torch.as_tensor(expected).detach().to("cpu", torch.float64).reshape(-1)
    assert a.shape == e.shape, (a.shape, e.shape)
    if a.numel() == 0:
        return 0.0
    fin = torch.isfinite(e)
    same_special = torch.equal(torch.isnan(a), torch.isnan(e)) and torch.equal(
        a[~fin & ~torch.isnan(e)], e[~fin & ~torch.isnan(e)])
    if not same_special:
        return float("inf")
    if not bool(fin.any()):
        return 0.0
    d = (a[fin] - e[fin]).abs()
    bound = atol + rtol * e[fin].abs()
    if slack is not None:
        bound = bound + torch.as_tensor(slack).detach().to("cpu", torch.float64).reshape(-1)[fin]
    return float((d / bound).max())


def assert_close(actual, expected, dtype, what, slack=None, scale=1.0):
    rtol, atol = tol_for(dtype)
    ex = excess(actual, expected, rtol * scale, atol * scale, slack)
    assert ex <= 1.0, "%s: error is %.3g x the tolerance (rtol %g, atol %g)" % (
        what, ex, rtol * scale, atol * scale)
    return ex


def abs_err(a, b):
    a = torch.as_tensor(a).detach().to("cpu", torch.float64)
    b = torch.as_tensor(b).detach().to("cpu", torch.float64)
    d = (a - b).abs()
    d = torch.where(torch.isfinite(d), d, torch.zeros_like(d))
    return d


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def offset_view(t, offset=2):
    """A copy of `t` living `offset` elements into a fresh 256-byte aligned buffer, so its data
    pointer is only offset*itemsize aligned."""
    buf = torch.empty(t.numel() + offset + 64, dtype=t.dtype, device=t.device)
    v = buf[offset:offset + t.numel()].view(t.shape)
    v.copy_(t)
    assert v.data_ptr() % 16 == (offset * t.element_size()) % 16
    return v


def stress_rows(M, N, seed, dtype=torch.float32):
    """N(0,1) rows with 0.1% of entries replaced by +-1e4 and row 0 constant (1.5)."""
    g = gen(seed)
    x = torch.randn(M, N, generator=g)
    mask = torch.rand(M, N, generator=g) < 0.001
    sign = torch.where(torch.rand(M, N, generator=g) < 0.5, -1.0, 1.0)
    x = torch.where(mask, 1e4 * sign, x)
    x[0] = 1.5
    return x.to(dtype)


def causal_scores(B, H, T, seed, dtype=torch.bfloat16):
    g = gen(seed)
    s = 3.0 * torch.randn(B, H, T, T, generator=g)
    s.masked_fill_(torch.triu(torch.ones(T, T), 1).bool(), float("-inf"))
    return s.to(dtype)


def load_golden(name="aten_cpu_golden.npz"):
    """tests/golden/<name> as {case: {name: torch tensor}} with the stored dtypes."""
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)
    z = np.load(path, allow_pickle=False)
    cases = {}
    for key in z.files:
        case, name = key.split("/", 1)
        if case == "meta":
            continue
        arr = z[key]
        if name.endswith(":bf16"):
            t = torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)
            name = name[:-5]
        elif name.endswith(":f16"):
            t = torch.from_numpy(arr.view(np.int16).copy()).view(torch.float16)
            name = name[:-4]
        else:
            t = torch.from_numpy(arr.copy())
        cases.setdefault(case, {})[name] = t
    return cases


GOLDEN_DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


EPS32 = 2.0 ** -24


def colsum_slack(terms):
    """Allowance for a float32 column sum over many rows: 16 * 2^-24 * ||terms||_2 per column.
    A sum of M float32 products carries a rounding error that grows like eps * sqrt(M) * rms(term)
    whatever the order of summation, while rtol * |result| shrinks to nothing on the columns whose
    terms cancel; the CPU kernel's float32 sums show the same behaviour."""
    t = torch.as_tensor(terms).to(torch.float64)
    return 16.0 * EPS32 * t.pow(2).sum(0).sqrt()


def xhat_slack(dy, mean, rstd):
    """Allowance for a float32 dgamma beside 16-bit rows.  The 16-bit backward kernels form the
    normalized element as fma(x, rstd, -mean * rstd) (one instruction an element less than
    (x - mean) * rstd): each term of the column sum then carries the float32 rounding of
    mean * rstd, 2^-24 * |mean * rstd|, times |dy|.  That is far below a 16-bit unit of x itself,
    and only shows against the float32 tolerance where a column's terms cancel or the row has no
    spread at all (N = 1: rstd = 1 / sqrt(eps))."""
    mr = (torch.as_tensor(mean).double().cpu() * torch.as_tensor(rstd).double().cpu()).abs()
    return 2.0 * EPS32 * (torch.as_tensor(dy).double().cpu().abs() * mr.reshape(-1, 1)).sum(0)


def rowsum_slack(terms, weight):
    """Allowance for an output of the form weight * (float32 sum of `terms` over a row): the sum's
    rounding, 16 * 2^-24 * ||terms||_2 per row, times |weight| per element."""
    t = torch.as_tensor(terms).to(torch.float64)
    w = torch.as_tensor(weight).to(torch.float64).abs()
    w = torch.where(torch.isfinite(w), w, torch.zeros_like(w))
    return w * (16.0 * EPS32 * t.pow(2).sum(-1, keepdim=True).sqrt())


def assert_same_arithmetic(a, b, what, max_fraction=1e-3):
    """Two kernel instances that evaluate the same formulas on the same values: the results are
    equal except where the compiler contracted a multiply-add in one instance and not in the other,
    which moves a result by at most one unit in the last place of its dtype.  Asserts that every
    element is equal or adjacent and that at most `max_fraction` of them (or two) differ; NaN / inf
    positions must agree."""
    assert a.dtype == b.dtype and a.shape == b.shape, (what, a.dtype, b.dtype, a.shape, b.shape)
    if torch.equal(a, b):
        return
    af, bf = a.detach().double().cpu().reshape(-1), b.detach().double().cpu().reshape(-1)
    fin = torch.isfinite(af) & torch.isfinite(bf)
    assert torch.equal(torch.isnan(af), torch.isnan(bf)) and torch.equal(af[~fin & ~torch.isnan(af)],
                                                                         bf[~fin & ~torch.isnan(bf)]), what
    d = (af[fin] - bf[fin]).abs()
    ulp = torch.finfo(a.dtype).eps * torch.maximum(af[fin].abs(), bf[fin].abs()).clamp_min(
        torch.finfo(a.dtype).tiny)
    assert bool((d <= ulp).all()), "%s: results more than one ulp apart (max %.3g ulp)" % (
        what, float((d / ulp).max()))
    ndiff = int((d > 0).sum())
    assert ndiff <= max(2, max_fraction * d.numel()), "%s: %d of %d elements differ" % (
        what, ndiff, d.numel())
