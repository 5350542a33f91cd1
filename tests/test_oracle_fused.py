"""Pins the oracle's functions for the fused residual add -> norm operators (no GPU):

  * round_to: against torch's own float32 -> float16 / bfloat16 conversion, bit for bit, on random
    values, ties, subnormals, overflow, infinities and NaN;
  * residual_sum: against an elementwise torch add of two tensors of the row dtype, bit for bit;
  * add_*_fwd: the identity that defines the operator -- the already pinned norm applied to that
    sum (the reference has no fused operator: its forward, LayerNormKernels.cpp:469-586, starts
    from the summed row);
  * add_*_bwd: central finite differences of sum(dy * norm(x + r)) + sum(g * (x + r)) in float64,
    and additivity in the residual-path gradient.
"""
import numpy as np
import pytest
import torch

import oracle

TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def test_round_to_matches_torch_bit_for_bit():
    g = torch.Generator().manual_seed(3)
    vals = [torch.randn(20000, generator=g) * s for s in (1.0, 1e-3, 1e3, 1e-30, 6e4, 3e38)]
    # exact ties of the bfloat16 grid (bit 15 set, lower bits clear) with even and odd keepers,
    # values one ulp either side of them, float16 ties, subnormals, the extremes
    base = torch.tensor([0x3F800000, 0x3F810000, 0x40490000, 0x7F7F0000, 0x00010000],
                        dtype=torch.int64)
    ties = torch.cat([base + 0x8000, base + 0x7FFF, base + 0x8001, base | 0x80008000])
    vals.append(ties.to(torch.int32).view(torch.float32))
    vals.append(torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 65504.0, 65519.9,
                              65520.0, 1e-8, 5.96e-8, 2.98e-8, 3.0e-8, 1 + 2.0 ** -11,
                              1 + 3 * 2.0 ** -11, 3.4028235e38, 3.39e38]))
    a = torch.cat(vals)
    for name in ("f16", "bf16", "f32"):
        want = a.to(TORCH[name]).float().numpy()
        got = oracle.round_to(a.numpy(), name)
        assert got.dtype == np.float32
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert bool(same.all()), (name, a.numpy()[~same][:5], got[~same][:5], want[~same][:5])


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_residual_sum_is_an_elementwise_add_in_the_row_dtype(name):
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(64, 257, generator=g) * 3).to(TORCH[name])
    r = (torch.randn(64, 257, generator=g) * 50).to(TORCH[name])
    x[0, :4] = torch.tensor([1e4, -1e4, 6e4, 1e-4]).to(TORCH[name])
    r[0, :4] = torch.tensor([1e-3, 1e4, 6e4, 1e-4]).to(TORCH[name])   # float16: 6e4 + 6e4 = inf
    want = (x + r).float().numpy()
    got = oracle.residual_sum(x.float().numpy(), r.float().numpy(), name)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("name", ["f32", "bf16"])
def test_fused_forward_is_the_norm_of_the_sum(name):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(9, 130, generator=g).to(TORCH[name])
    r = torch.randn(9, 130, generator=g).to(TORCH[name])
    w = (1 + 0.1 * torch.randn(130, generator=g)).numpy()
    b = (0.1 * torch.randn(130, generator=g)).numpy()
    h = (x + r).float().numpy()
    y, hh, mean, rstd = oracle.add_layer_norm_fwd(x.float().numpy(), r.float().numpy(), (130,), w,
                                                  b, 1e-5, name)
    ry, rm, rr = oracle.layer_norm_fwd(h, (130,), w, b, 1e-5)
    assert np.array_equal(hh, h) and np.array_equal(y, ry)
    assert np.array_equal(mean, rm) and np.array_equal(rstd, rr)
    y, hh, rstd = oracle.add_rms_norm_fwd(x.float().numpy(), r.float().numpy(), (130,), w, 1e-6,
                                          name)
    ry, rr = oracle.rms_norm_fwd(h, (130,), w, 1e-6)
    assert np.array_equal(hh, h) and np.array_equal(y, ry) and np.array_equal(rstd, rr)
    # and against torch's own composition on the CPU
    ty = torch.nn.functional.layer_norm((x + r).float(), (130,), torch.from_numpy(w),
                                        torch.from_numpy(b), 1e-5)
    yl = oracle.add_layer_norm_fwd(x.float().numpy(), r.float().numpy(), (130,), w, b, 1e-5, name)[0]
    assert np.allclose(yl, ty.numpy(), rtol=1e-5, atol=1e-5)


def _ln64(h, w, b, eps):
    mu = h.mean(-1, keepdims=True)
    var = h.var(-1, keepdims=True)
    return (h - mu) / np.sqrt(var + eps) * w + b


def _rms64(h, w, eps):
    return h / np.sqrt((h * h).mean(-1, keepdims=True) + eps) * w


@pytest.mark.parametrize("rms", [False, True], ids=["layer_norm", "rms_norm"])
def test_fused_backward_by_finite_differences(rms):
    rng = np.random.default_rng(6)
    M, N = 3, 7
    x, r = rng.standard_normal((M, N)), rng.standard_normal((M, N))
    dy, gh = rng.standard_normal((M, N)), rng.standard_normal((M, N))
    w, b = 1 + 0.1 * rng.standard_normal(N), 0.1 * rng.standard_normal(N)
    eps = 1e-5

    def loss(xx):
        h = xx + r
        y = _rms64(h, w, eps) if rms else _ln64(h, w, b, eps)
        return float((dy * y).sum() + (gh * h).sum())

    fd = np.zeros((M, N))
    for i in range(M):
        for j in range(N):
            d = np.zeros((M, N))
            d[i, j] = 1e-6
            fd[i, j] = (loss(x + d) - loss(x - d)) / 2e-6
    h32 = (x + r).astype(np.float32)
    f32 = lambda a: a.astype(np.float32)  # noqa: E731
    if rms:
        _, rstd = oracle.rms_norm_fwd(h32, (N,), f32(w), eps)
        dh, dw = oracle.add_rms_norm_bwd(f32(dy), f32(gh), h32, (N,), rstd, f32(w))
        plain, pw = oracle.rms_norm_bwd(f32(dy), h32, (N,), rstd, f32(w))
        none, _ = oracle.add_rms_norm_bwd(f32(dy), None, h32, (N,), rstd, f32(w))
    else:
        _, mean, rstd = oracle.layer_norm_fwd(h32, (N,), f32(w), f32(b), eps)
        dh, dw, db = oracle.add_layer_norm_bwd(f32(dy), f32(gh), h32, (N,), mean, rstd, f32(w))
        plain, pw, pb = oracle.layer_norm_bwd(f32(dy), h32, (N,), mean, rstd, f32(w))
        none, _, _ = oracle.add_layer_norm_bwd(f32(dy), None, h32, (N,), mean, rstd, f32(w))
        assert np.array_equal(db, pb)
    assert np.allclose(dh, fd, rtol=2e-4, atol=2e-5)           # float32 inputs to the oracle
    assert np.array_equal(none, plain) and np.array_equal(dw, pw)
    assert np.allclose(dh - plain, gh, rtol=0, atol=1e-6)       # additive in the residual path
