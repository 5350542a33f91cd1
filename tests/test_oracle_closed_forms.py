"""Pins the CPU oracle (oracle/rownorm_oracle.c) without importing anything from the reference:
numpy / scipy closed forms, central finite differences for every backward function, brute force
on tiny inputs, and the invariants the reference's own tests use (cited per test).  Each check
is chosen so that a dropped term, a wrong sign or a transposed operand fails it.
"""
import numpy as np
import pytest
import scipy.special

RNG = np.random.default_rng(1234)


def _rand(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


# ---------------------------------------------------------------- Welford ----
@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 127, 1000, 4097])
def test_welford_matches_numpy_moments(oracle, n):
    x = (_rand(n) * 3 + 7).astype(np.float32)
    mean, var = oracle.welford_moments(x)
    assert mean == pytest.approx(np.mean(x.astype(np.float64)), rel=1e-13, abs=1e-13)
    assert var == pytest.approx(np.var(x.astype(np.float64)), rel=1e-11, abs=1e-13)


def test_welford_catastrophic_cancellation(oracle):
    # test/regressions/test_layer_norm.py:20-30 in the reference: x = 1e15 + {0..4}.  In float32
    # all five values round to the same number, so the row is constant: variance exactly 0.
    x = (np.float32(1e15) + np.arange(5, dtype=np.float32)).astype(np.float32)
    mean, var = oracle.welford_moments(x)
    assert var == 0.0 and mean == float(x[0])
    # and in a case where a sum-of-squares formula loses everything
    x = (1e4 + np.array([0.0, 1.0, 2.0, 3.0, 4.0])).astype(np.float32)
    mean, var = oracle.welford_moments(x)
    assert mean == pytest.approx(10002.0, abs=1e-9) and var == pytest.approx(2.0, rel=1e-12)


# ------------------------------------------------------------- LayerNorm ----
@pytest.mark.parametrize("shape,nd", [((5, 7), 1), ((3, 4, 16), 1), ((2, 3, 4, 5), 2), ((6, 129), 1)])
def test_layer_norm_fwd_closed_form(oracle, shape, nd):
    # closed form of test/xpu/test_nn_xpu.py:11544-11572 (test_LayerNorm_numeric)
    x = _rand(*shape) * 2 + 0.5
    ns = shape[-nd:]
    gamma, beta = _rand(*ns), _rand(*ns)
    y, mean, rstd = oracle.layer_norm_fwd(x, ns, gamma, beta, 1e-5)
    xd = x.astype(np.float64).reshape(-1, int(np.prod(ns)))
    mu = xd.mean(1, keepdims=True)
    var = xd.var(1, keepdims=True)
    ref = ((xd - mu) / np.sqrt(var + 1e-5)) * gamma.reshape(1, -1) + beta.reshape(1, -1)
    np.testing.assert_allclose(y.reshape(xd.shape), ref, rtol=2e-6, atol=2e-6)
    stat_shape = shape[:-nd] + (1,) * nd
    assert mean.shape == stat_shape and rstd.shape == stat_shape
    np.testing.assert_allclose(mean.reshape(-1), mu.reshape(-1), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(rstd.reshape(-1), 1 / np.sqrt(var.reshape(-1) + 1e-5), rtol=1e-6)


def test_layer_norm_fwd_no_affine_and_constant_rows(oracle):
    # weight=None == ones, bias=None == zeros (test_nn_xpu.py:15076-15104); constant rows give
    # exactly beta / zeros (test_nn_xpu.py:9657-9661, test_layer_norm_eps)
    x = _rand(4, 33)
    y0, _, _ = oracle.layer_norm_fwd(x, (33,), None, None, 1e-5)
    y1, _, _ = oracle.layer_norm_fwd(x, (33,), np.ones(33, np.float32), np.zeros(33, np.float32), 1e-5)
    assert np.array_equal(y0, y1)
    assert abs(y0.mean(1)).max() < 1e-6 and abs(y0.var(1) - 1).max() < 1e-4
    for c in (1.5, 0.1, -3.3333):
        xc = np.full((2, 14), c, np.float32)
        beta = _rand(14)
        y, mean, rstd = oracle.layer_norm_fwd(xc, (14,), _rand(14), beta, 1e-6)
        assert np.array_equal(y, np.broadcast_to(beta, y.shape))
        assert np.all(mean == np.float32(c))
        np.testing.assert_allclose(rstd, 1000.0, rtol=1e-6)


def _ln_loss(oracle, x, gamma, beta, w, eps):
    y, _, _ = oracle.layer_norm_fwd(x, (x.shape[-1],), gamma, beta, eps)
    return float((y.astype(np.float64) * w).sum())


def test_layer_norm_bwd_finite_differences(oracle):
    # d/dx, d/dgamma, d/dbeta of sum(w * layer_norm(x)) by central differences in float32 inputs /
    # float64 arithmetic; a wrong sign or dropped s1/s2 term is off by O(1), far above the bound.
    M, N, eps = 3, 9, 1e-3
    x, gamma, beta, w = _rand(M, N), _rand(N) + 1.5, _rand(N), _rand(M, N)
    y, mean, rstd = oracle.layer_norm_fwd(x, (N,), gamma, beta, eps)
    dx, dg, db = oracle.layer_norm_bwd(w, x, (N,), mean, rstd, gamma)
    h = 1e-2
    for (r, c) in [(0, 0), (1, 4), (2, 8)]:
        xp, xm = x.copy(), x.copy()
        xp[r, c] += h
        xm[r, c] -= h
        fd = (_ln_loss(oracle, xp, gamma, beta, w, eps) - _ln_loss(oracle, xm, gamma, beta, w, eps)) / (
            float(xp[r, c]) - float(xm[r, c]))
        assert dx[r, c] == pytest.approx(fd, rel=2e-3, abs=2e-3)
    for c in (0, 5):
        gp, gm = gamma.copy(), gamma.copy()
        gp[c] += h
        gm[c] -= h
        fd = (_ln_loss(oracle, x, gp, beta, w, eps) - _ln_loss(oracle, x, gm, beta, w, eps)) / (
            float(gp[c]) - float(gm[c]))
        assert dg[c] == pytest.approx(fd, rel=1e-3, abs=1e-3)
        bp, bm = beta.copy(), beta.copy()
        bp[c] += h
        bm[c] -= h
        fd = (_ln_loss(oracle, x, gamma, bp, w, eps) - _ln_loss(oracle, x, gamma, bm, w, eps)) / (
            float(bp[c]) - float(bm[c]))
        assert db[c] == pytest.approx(fd, rel=1e-3, abs=1e-3)


def test_layer_norm_bwd_invariants_and_masks(oracle):
    M, N = 11, 40
    x, dy, gamma = _rand(M, N), _rand(M, N), _rand(N)
    _, mean, rstd = oracle.layer_norm_fwd(x, (N,), gamma, None, 1e-5)
    dx, dg, db = oracle.layer_norm_bwd(dy, x, (N,), mean, rstd, gamma)
    # each row of dx is orthogonal to the constant vector and to xhat
    xhat = (x - mean) * rstd
    assert abs(dx.sum(1)).max() < 1e-5
    assert abs((dx.astype(np.float64) * xhat).sum(1)).max() < 5e-4
    # dbeta of a sum() loss is the row count (test/regressions/test_rms_norm.py:152-160)
    _, _, db1 = oracle.layer_norm_bwd(np.ones((M, N), np.float32), x, (N,), mean, rstd, gamma)
    assert np.array_equal(db1, np.full(N, M, np.float32))
    np.testing.assert_allclose(dg, (dy.astype(np.float64) * xhat).sum(0), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, dy.astype(np.float64).sum(0), rtol=1e-6, atol=1e-6)
    a, b, c = oracle.layer_norm_bwd(dy, x, (N,), mean, rstd, gamma, mask=(True, False, False))
    assert b is None and c is None and np.array_equal(a, dx)
    a, b, c = oracle.layer_norm_bwd(dy, x, (N,), mean, rstd, gamma, mask=(False, True, True))
    assert a is None and np.array_equal(b, dg) and np.array_equal(c, db)
    # gamma=None behaves as ones
    d0 = oracle.layer_norm_bwd(dy, x, (N,), mean, rstd, None)[0]
    d1 = oracle.layer_norm_bwd(dy, x, (N,), mean, rstd, np.ones(N, np.float32))[0]
    assert np.array_equal(d0, d1)


# --------------------------------------------------------------- RMSNorm ----
def test_rms_norm_fwd_closed_form(oracle):
    # x * rsqrt(mean(x^2) + eps) * w, test/xpu/test_nn_xpu.py:11575-11621
    for shape, nd in (((6, 31), 1), ((2, 3, 4, 5), 2)):
        x = _rand(*shape)
        ns = shape[-nd:]
        w = _rand(*ns)
        for eps in (1e-6, None):
            y, rstd = oracle.rms_norm_fwd(x, ns, w, eps)
            e = np.finfo(np.float32).eps if eps is None else eps
            xd = x.astype(np.float64).reshape(-1, int(np.prod(ns)))
            r = 1 / np.sqrt((xd ** 2).mean(1, keepdims=True) + e)
            np.testing.assert_allclose(y.reshape(xd.shape), xd * r * w.reshape(1, -1), rtol=2e-6, atol=1e-7)
            assert rstd.shape == shape[:-nd] + (1,) * nd
            np.testing.assert_allclose(rstd.reshape(-1), r.reshape(-1), rtol=1e-6)
    tiny = np.full((2, 8), 1e-12, np.float32)  # the reference's epsilon test uses +-1e-12 inputs
    y, rstd = oracle.rms_norm_fwd(tiny, (8,), None, None)
    np.testing.assert_allclose(rstd, 1 / np.sqrt(1e-24 + np.finfo(np.float32).eps), rtol=1e-6)


def test_rms_norm_bwd_closed_form_and_finite_differences(oracle):
    M, N, eps = 4, 10, 1e-3
    x, w, dy = _rand(M, N), _rand(N) + 1.2, _rand(M, N)
    _, rstd = oracle.rms_norm_fwd(x, (N,), w, eps)
    dx, dg = oracle.rms_norm_bwd(dy, x, (N,), rstd, w)
    # dgamma = sum_rows dY * x * rstd (test/regressions/test_rms_norm.py:82-83)
    np.testing.assert_allclose(dg, (dy.astype(np.float64) * x * rstd).sum(0), rtol=1e-6, atol=1e-6)

    def loss(xx, ww):
        y, _ = oracle.rms_norm_fwd(xx, (N,), ww, eps)
        return float((y.astype(np.float64) * dy).sum())

    h = 1e-2
    for (r, c) in [(0, 0), (2, 7), (3, 9)]:
        xp, xm = x.copy(), x.copy()
        xp[r, c] += h
        xm[r, c] -= h
        fd = (loss(xp, w) - loss(xm, w)) / (float(xp[r, c]) - float(xm[r, c]))
        assert dx[r, c] == pytest.approx(fd, rel=2e-3, abs=2e-3)
    a, b = oracle.rms_norm_bwd(dy, x, (N,), rstd, w, mask=(True, False))
    assert b is None and np.array_equal(a, dx)


# --------------------------------------------------------------- softmax ----
@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (7, 64), (2, 3, 129), (4, 2049)])
def test_softmax_fwd_matches_scipy(oracle, shape):
    x = _rand(*shape) * 3
    np.testing.assert_allclose(oracle.softmax_fwd(x), scipy.special.softmax(x.astype(np.float64), -1),
                               rtol=2e-7, atol=1e-12)
    np.testing.assert_allclose(oracle.softmax_fwd(x, True),
                               scipy.special.log_softmax(x.astype(np.float64), -1), rtol=2e-7, atol=2e-7)


def test_softmax_fwd_invariants_and_specials(oracle):
    x = _rand(9, 513) * 4
    s, ls = oracle.softmax_fwd(x), oracle.softmax_fwd(x, True)
    # exp(log_softmax).sum() == 1 (test/xpu/test_nn_xpu.py:14141-14145)
    np.testing.assert_allclose(s.sum(-1), 1, rtol=1e-6)
    np.testing.assert_allclose(np.exp(ls.astype(np.float64)).sum(-1), 1, rtol=1e-6)
    # shift invariance (test_nn_xpu.py:14177-14190, test_log_softmax_big)
    np.testing.assert_allclose(oracle.softmax_fwd(x + np.float32(1.5e3), True), ls, rtol=0, atol=2e-3)
    # masked entries: -inf -> 0 / -inf; a fully masked row -> NaN (SoftMaxKernels.cpp:331-332)
    xm = x.copy()
    xm[0, 100:] = -np.inf
    xm[1, :] = -np.inf
    s, ls = oracle.softmax_fwd(xm), oracle.softmax_fwd(xm, True)
    assert np.all(s[0, 100:] == 0) and np.all(np.isneginf(ls[0, 100:]))
    np.testing.assert_allclose(s[0, :100].sum(), 1, rtol=1e-6)
    assert np.all(np.isnan(s[1])) and np.all(np.isnan(ls[1]))
    # overflow guard: inputs scaled by 1000 stay finite (test_nn_xpu.py:15824-15841)
    assert np.all(np.isfinite(oracle.softmax_fwd(x * 1000)))


def test_softmax_bwd_closed_form_and_finite_differences(oracle):
    M, N = 3, 12
    x, g = _rand(M, N) * 2, _rand(M, N)
    for is_log in (False, True):
        y = oracle.softmax_fwd(x, is_log)
        gi = oracle.softmax_bwd(g, y, is_log)
        yd, gd = y.astype(np.float64), g.astype(np.float64)
        if is_log:
            ref = gd - np.exp(yd) * gd.sum(-1, keepdims=True)
        else:
            ref = yd * (gd - (yd * gd).sum(-1, keepdims=True))
        np.testing.assert_allclose(gi, ref, rtol=1e-6, atol=1e-7)
        h = 1e-2
        for (r, c) in [(0, 0), (1, 5), (2, 11)]:
            xp, xm = x.copy(), x.copy()
            xp[r, c] += h
            xm[r, c] -= h
            lp = float((oracle.softmax_fwd(xp, is_log).astype(np.float64) * g).sum())
            lm = float((oracle.softmax_fwd(xm, is_log).astype(np.float64) * g).sum())
            fd = (lp - lm) / (float(xp[r, c]) - float(xm[r, c]))
            assert gi[r, c] == pytest.approx(fd, rel=2e-3, abs=2e-3)
    # softmax backward rows sum to zero
    y = oracle.softmax_fwd(x)
    assert abs(oracle.softmax_bwd(g, y).sum(-1)).max() < 1e-6
    # masked entries: y = 0 -> gradient 0; log: y = -inf -> gradient g (exp(-inf) = 0)
    y0 = y.copy()
    y0[0, 3] = 0
    assert oracle.softmax_bwd(g, y0)[0, 3] == 0
    ly = oracle.softmax_fwd(x, True)
    ly[0, 3] = -np.inf
    assert oracle.softmax_bwd(g, ly, True)[0, 3] == g[0, 3]


# ---------------------------------------------- masked and safe softmax ----
def test_masked_softmax_is_softmax_of_the_unmasked_elements(oracle):
    rng = np.random.default_rng(7)
    M, N = 6, 37
    x, g = _rand(M, N) * 3, _rand(M, N)
    mask = rng.random((M, N)) < 0.4
    mask[0] = False
    mask[1, 1:] = True  # a single survivor
    mask[1, 0] = False
    y = oracle.masked_softmax_fwd(x, mask)
    gi = oracle.masked_softmax_bwd(g, y, mask)
    for r in range(M):
        keep = ~mask[r]
        ref = scipy.special.softmax(x[r, keep].astype(np.float64))
        np.testing.assert_allclose(y[r, keep], ref, rtol=2e-7, atol=1e-12)
        assert np.all(y[r, mask[r]] == 0) and np.all(gi[r, mask[r]] == 0)
        # backward of the compacted row with the plain formula
        yd, gd = y[r, keep].astype(np.float64), g[r, keep].astype(np.float64)
        np.testing.assert_allclose(gi[r, keep], yd * (gd - (yd * gd).sum()), rtol=1e-6, atol=1e-7)
    assert y[1, 0] == 1.0
    # broadcasting: a [N] mask applies to every row
    yb = oracle.masked_softmax_fwd(x, mask[2])
    assert np.array_equal(yb[5], oracle.masked_softmax_fwd(x[5:6], mask[2:3])[0])
    # every element masked -> NaN row, zero gradient
    full = np.ones((M, N), bool)
    assert np.all(np.isnan(oracle.masked_softmax_fwd(x, full)))
    assert np.all(oracle.masked_softmax_bwd(g, y, full) == 0)
    # a saved output that holds NaN (every unmasked input was -inf) poisons its whole row, the
    # masked positions too: 0 * (g - NaN), as SoftMaxKernels.cpp:991-1047 evaluates it
    xn = x.copy()
    xn[3, ~mask[3]] = -np.inf
    yn = oracle.masked_softmax_fwd(xn, mask)
    assert np.all(np.isnan(yn[3]))
    gn = oracle.masked_softmax_bwd(g, yn, mask)
    assert np.all(np.isnan(gn[3])) and np.array_equal(gn[[0, 1, 2]], gi[[0, 1, 2]])
    # masking with the mask equals feeding -inf to the plain softmax
    xm = np.where(mask, -np.inf, x).astype(np.float32)
    np.testing.assert_array_equal(y, oracle.softmax_fwd(xm))


def test_safe_softmax_differs_from_softmax_only_on_all_neg_inf_rows(oracle):
    x = _rand(5, 33) * 3
    x[1, 10:] = -np.inf
    x[3, :] = -np.inf
    s, ss = oracle.softmax_fwd(x), oracle.safe_softmax_fwd(x)
    keep = [0, 1, 2, 4]
    np.testing.assert_array_equal(ss[keep], s[keep])
    assert np.all(np.isnan(s[3])) and np.all(ss[3] == 0)
    # a NaN input still poisons its row
    x[0, 5] = np.nan
    assert np.all(np.isnan(oracle.safe_softmax_fwd(x)[0]))
