"""The CPU oracle's GroupNorm functions: pinned by the LayerNorm functions (already pinned
elsewhere) applied to each (sample, group) slab, by finite differences, by invariants, and by the
committed PyTorch-CPU-ATen golden vectors (tests/golden/aten_cpu_group_norm.npz)."""
import numpy as np
import pytest
import torch

from helpers import GOLDEN_DTYPES, assert_close, load_golden, to_np32

CASES = load_golden("aten_cpu_group_norm.npz")


def _rand(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("N,C,sp,G", [(3, 8, (4, 8), 2), (2, 6, (5,), 3), (5, 12, (), 4), (2, 4, (3, 3), 1),
                                      (2, 6, (7,), 6)])
def test_group_norm_is_layer_norm_per_group_with_channel_affine(oracle, N, C, sp, G):
    x, dy = _rand(N, C, *sp, seed=1) + 0.5, _rand(N, C, *sp, seed=2)
    gamma, beta = 1 + 0.3 * _rand(C, seed=3), 0.2 * _rand(C, seed=4)
    HxW = int(np.prod(sp)) if sp else 1
    D, L = C // G, (C // G) * HxW
    y, mean, rstd = oracle.group_norm_fwd(x, G, gamma, beta, 1e-5)
    # forward: LayerNorm over each [D*HxW] slab with the weights expanded per element
    ge = np.repeat(gamma.reshape(G, D), HxW, axis=1)           # [G, L]
    be = np.repeat(beta.reshape(G, D), HxW, axis=1)
    xr = x.reshape(N, G, L)
    for g in range(G):
        ly, lm, lr = oracle.layer_norm_fwd(xr[:, g], (L,), ge[g], be[g], 1e-5)
        np.testing.assert_allclose(y.reshape(N, G, L)[:, g], ly, rtol=2e-6, atol=2e-6)
        np.testing.assert_allclose(mean[:, g], lm.reshape(-1), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(rstd[:, g], lr.reshape(-1), rtol=1e-6)
    # numpy closed form
    mu = xr.astype(np.float64).mean(-1)
    var = xr.astype(np.float64).var(-1)
    np.testing.assert_allclose(mean, mu, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(rstd, 1 / np.sqrt(var + 1e-5), rtol=1e-6)
    # backward: dx equals LayerNorm's with the expanded weights; dgamma/dbeta are the per-element
    # LayerNorm column sums folded over HxW
    dx, dg, db = oracle.group_norm_bwd(dy, x, G, mean, rstd, gamma)
    dyr = dy.reshape(N, G, L)
    for g in range(G):
        ldx, ldg, ldb = oracle.layer_norm_bwd(dyr[:, g], xr[:, g], (L,), mean[:, g], rstd[:, g], ge[g])
        np.testing.assert_allclose(dx.reshape(N, G, L)[:, g], ldx, rtol=2e-5, atol=2e-6)
        np.testing.assert_allclose(dg.reshape(G, D)[g], ldg.reshape(D, HxW).sum(-1), rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(db.reshape(G, D)[g], ldb.reshape(D, HxW).sum(-1), rtol=2e-5, atol=2e-5)
    # dbeta of a sum() loss counts the elements per channel
    _, _, db1 = oracle.group_norm_bwd(np.ones_like(x), x, G, mean, rstd, gamma)
    np.testing.assert_allclose(db1, N * HxW)
    # masks and absent weights
    a, b, c = oracle.group_norm_bwd(dy, x, G, mean, rstd, gamma, mask=(True, False, False))
    assert b is None and c is None and np.array_equal(a, dx)
    y1, _, _ = oracle.group_norm_fwd(x, G, None, None, 1e-5)
    y2, _, _ = oracle.group_norm_fwd(x, G, np.ones(C, np.float32), np.zeros(C, np.float32), 1e-5)
    np.testing.assert_array_equal(y1, y2)


def test_group_norm_bwd_finite_differences(oracle):
    N, C, HxW, G = 2, 6, 4, 3
    x, w = _rand(N, C, HxW, seed=5), _rand(N, C, HxW, seed=6)
    gamma, beta = 1 + 0.3 * _rand(C, seed=7), 0.2 * _rand(C, seed=8)

    def loss(xx, gg, bb):
        y, _, _ = oracle.group_norm_fwd(xx, G, gg, bb, 1e-3)
        return float((y.astype(np.float64) * w).sum())

    _, mean, rstd = oracle.group_norm_fwd(x, G, gamma, beta, 1e-3)
    dx, dg, db = oracle.group_norm_bwd(w, x, G, mean, rstd, gamma)
    h = 1e-2
    for idx in [(0, 0, 0), (1, 3, 2), (1, 5, 3)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        fd = (loss(xp, gamma, beta) - loss(xm, gamma, beta)) / (float(xp[idx]) - float(xm[idx]))
        assert dx[idx] == pytest.approx(fd, rel=2e-3, abs=2e-3)
    for c in (0, 4):
        gp, gm = gamma.copy(), gamma.copy()
        gp[c] += h
        gm[c] -= h
        assert dg[c] == pytest.approx((loss(x, gp, beta) - loss(x, gm, beta)) / (float(gp[c]) - float(gm[c])),
                                      rel=2e-3, abs=2e-3)
        bp, bm = beta.copy(), beta.copy()
        bp[c] += h
        bm[c] -= h
        assert db[c] == pytest.approx((loss(x, gamma, bp) - loss(x, gamma, bm)) / (float(bp[c]) - float(bm[c])),
                                      rel=2e-3, abs=2e-3)


@pytest.mark.parametrize("case", sorted(CASES))
def test_group_norm_matches_golden(oracle, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    G = int(case.split("g")[-1])
    x = to_np32(c["x"])
    variants = [("gn", c["gamma"], c["beta"])]
    if dt != torch.float32:
        variants.append(("gnmix", c["gamma"].float(), c["beta"].float()))
    for pre, gk, bk in variants:
        y, mean, rstd = oracle.group_norm_fwd(x, G, to_np32(gk), to_np32(bk), 1e-5)
        sdt = c[pre + "_mean"].dtype
        assert_close(y, c[pre + "_y"], dt, case + " y")
        assert_close(mean, c[pre + "_mean"], sdt, case + " mean")
        assert_close(rstd, c[pre + "_rstd"], sdt, case + " rstd")
        # backward from the golden statistics, as the CPU op consumed them
        dx, dg, db = oracle.group_norm_bwd(to_np32(c["dy"]), x, G, to_np32(c[pre + "_mean"]),
                                           to_np32(c[pre + "_rstd"]), to_np32(gk))
        assert_close(dx, c[pre + "_dx"], dt, case + " dx", scale=2.0)
        assert_close(dg, c[pre + "_dgamma"], dt, case + " dgamma", scale=4.0)
        assert_close(db, c[pre + "_dbeta"], dt, case + " dbeta", scale=4.0)
