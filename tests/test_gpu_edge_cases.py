"""Edge cases of the operator contracts on the GPU, through the C ABI: constant rows, masked and
fully masked softmax rows, empty and single-element problems, output masks, absent gamma/beta,
misaligned pointers, every compiled kernel variant (forced), the multi-pass kernels (forced), and
run-to-run determinism.  Each case names the reference test it mirrors."""
import pytest
import torch

from helpers import assert_close, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_constant_rows_give_beta_exactly(cabi, gpu, dtype):
    # test/xpu/test_nn_xpu.py:9657-9661 (test_layer_norm_eps) and the CPU kernel's behaviour:
    # mean is the constant, rstd = 1/sqrt(eps), y == beta bit for bit
    for N in (2, 14, 64, 127, 1024, 4097, 16384):
        for cval in (1.5, 0.1, -3.3333):
            c = torch.tensor(cval).to(dtype)
            x = torch.full((3, N), float(c)).to(dtype).to(gpu)
            g = gen(5)
            gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype).to(gpu)
            beta = (0.1 * torch.randn(N, generator=g)).to(dtype).to(gpu)
            y, mean, rstd = cabi.layer_norm_fwd(x, gamma, beta, 1e-5)
            assert torch.equal(mean.cpu(), torch.full((3,), float(c))), (N, cval)
            assert_close(rstd, torch.full((3,), 316.227783203125), torch.float32, "rstd")
            assert torch.equal(y, beta.expand_as(y)), (N, cval)
    # no affine: exactly zeros
    x = torch.full((2, 14), 0.7, device=gpu)
    y, _, _ = cabi.layer_norm_fwd(x, None, None, 1e-6)
    assert bool((y == 0).all())


def test_layer_norm_large_offset_rows(cabi, oracle, gpu):
    # test/regressions/test_layer_norm.py:20-30: x = 1e15 + {0..4} must not give NaN; plus a row
    # whose mean dwarfs its spread, where a sum-of-squares variance would cancel to garbage
    x = (torch.tensor(1e15) + torch.arange(5.0)).reshape(1, 5)
    y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), None, None, 1e-5)
    cy, cm, cr = torch.ops.aten.native_layer_norm(x, [5], None, None, 1e-5)
    assert bool(torch.isfinite(y).all())
    assert_close(y, cy, torch.float32, "y")
    assert_close(mean, cm.reshape(-1), torch.float32, "mean")
    x = 1e4 + torch.randn(7, 300, generator=gen(3))
    y, mean, rstd = cabi.layer_norm_fwd(x.to(gpu), None, None, 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(x.numpy(), (300,), None, None, 1e-5)
    assert_close(y, oy, torch.float32, "y")
    assert_close(rstd, orr.reshape(-1), torch.float32, "rstd")
    assert_close(mean, om.reshape(-1), torch.float32, "mean")


def test_absent_gamma_beta_mean_ones_zeros(cabi, gpu):
    # test/xpu/test_nn_xpu.py:15076-15104: weight=None == ones, bias=None == zeros
    x = torch.randn(9, 777, generator=gen(1)).to(gpu)
    dy = torch.randn(9, 777, generator=gen(2)).to(gpu)
    ones, zeros = torch.ones(777, device=gpu), torch.zeros(777, device=gpu)
    y0, m0, r0 = cabi.layer_norm_fwd(x, None, None, 1e-5)
    y1, m1, r1 = cabi.layer_norm_fwd(x, ones, zeros, 1e-5)
    assert torch.equal(y0, y1) and torch.equal(m0, m1) and torch.equal(r0, r1)
    y2, _, _ = cabi.layer_norm_fwd(x, ones, None, 1e-5)
    assert torch.equal(y0, y2)
    dx0, _, _ = cabi.layer_norm_bwd(dy, x, m0, r0, None, want=(True, False, False))
    dx1, _, _ = cabi.layer_norm_bwd(dy, x, m0, r0, ones, want=(True, False, False))
    assert torch.equal(dx0, dx1)
    ry0, rr0 = cabi.rms_norm_fwd(x, None, 1e-6)
    ry1, rr1 = cabi.rms_norm_fwd(x, ones, 1e-6)
    assert torch.equal(ry0, ry1) and torch.equal(rr0, rr1)


def test_output_masks(cabi, gpu):
    # LayerNorm.cpp:137-181 / 276-300 in the reference: only the requested gradients are produced
    M, N = 37, 1536
    x = torch.randn(M, N, generator=gen(4)).to(gpu)
    dy = torch.randn(M, N, generator=gen(5)).to(gpu)
    gamma = torch.randn(N, generator=gen(6)).to(gpu)
    _, mean, rstd = cabi.layer_norm_fwd(x, gamma, None, 1e-5)
    dx, dg, db = cabi.layer_norm_bwd(dy, x, mean, rstd, gamma)
    for want in [(True, False, False), (False, True, True), (False, True, False),
                 (False, False, True), (True, True, False)]:
        a, b, c = cabi.layer_norm_bwd(dy, x, mean, rstd, gamma, want=want)
        assert (a is None) == (not want[0]) and (b is None) == (not want[1]) and (c is None) == (not want[2])
        if want[0]:
            assert torch.equal(a, dx)
        if want[1]:
            assert torch.equal(b, dg)
        if want[2]:
            assert torch.equal(c, db)
    _, rr = cabi.rms_norm_fwd(x, gamma, 1e-6)
    rdx, rdg = cabi.rms_norm_bwd(dy, x, rr, gamma)
    a, b = cabi.rms_norm_bwd(dy, x, rr, gamma, want=(True, False))
    assert b is None and torch.equal(a, rdx)
    a, b = cabi.rms_norm_bwd(dy, x, rr, gamma, want=(False, True))
    assert a is None and torch.equal(b, rdg)


def test_empty_and_single_element(cabi, gpu):
    for M, N in ((0, 16), (5, 0)):
        x = torch.empty(M, N, device=gpu)
        y, mean, rstd = cabi.layer_norm_fwd(x, None, None, 1e-5)
        assert y.shape == (M, N) and mean.shape == (M,)
        assert cabi.softmax_fwd(x).shape == (M, N)
        assert cabi.softmax_bwd(x, x).shape == (M, N)
    x = torch.tensor([[3.0]], device=gpu)
    assert float(cabi.softmax_fwd(x)) == 1.0 and float(cabi.softmax_fwd(x, True)) == 0.0
    y, mean, rstd = cabi.layer_norm_fwd(x, None, None, 1e-5)
    assert float(y) == 0.0 and float(mean) == 3.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_softmax_masked_rows(cabi, gpu, dtype):
    # -inf entries give 0 / -inf, a fully masked row gives NaN (SoftMaxKernels.cpp:331-332 in the
    # reference; CPU ATen gives NaN too); backward: y = 0 -> +-0, log: y = -inf -> grad unchanged
    N = 2048
    x = (3 * torch.randn(6, N, generator=gen(8))).to(dtype)
    x[0, 1000:] = float("-inf")
    x[1, :] = float("-inf")
    x[2, 5] = float("inf")
    x[3, 17] = float("nan")
    g = torch.randn(6, N, generator=gen(9)).to(dtype)
    for is_log in (False, True):
        y = cabi.softmax_fwd(x.to(gpu), is_log)
        ref = (torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax)(x.float(), -1, False)
        assert_close(y, ref, dtype, "masked rows y")
        yc = y.cpu()
        assert bool(torch.isnan(yc[1]).all()) and bool(torch.isnan(yc[2]).all()) and bool(torch.isnan(yc[3]).all())
        if is_log:
            assert bool(torch.isneginf(yc[0, 1000:]).all())
        else:
            assert bool((yc[0, 1000:] == 0).all())
        gi = cabi.softmax_bwd(g.to(gpu), y, is_log).cpu()
        if is_log:
            assert torch.equal(gi[0, 1000:], g[0, 1000:])
        else:
            assert bool((gi[0, 1000:] == 0).all())
        assert bool(torch.isfinite(gi[0]).all()) and bool(torch.isfinite(gi[4:]).all())


def test_log_softmax_shift_invariance_and_overflow_guard(cabi, gpu):
    # test/xpu/test_nn_xpu.py:14177-14190 (test_log_softmax_big) and :15824-15841 (x1000 inputs)
    x = torch.randn(16, 1000, generator=gen(10)).half().to(gpu)
    a = cabi.softmax_fwd(x, True)
    b = cabi.softmax_fwd(x + 1.5e3, True)
    assert float((a.float() - b.float()).abs().max()) < 1.0  # x + 1500 in half is coarse
    xf = torch.randn(16, 1000, generator=gen(11)).to(gpu)
    assert_close(cabi.softmax_fwd(xf + 1.5e3, True), cabi.softmax_fwd(xf, True), torch.float32,
                 "shift invariance", scale=30.0)  # x + 1500 rounds x to 1.2e-4
    xb = (1000 * torch.randn(16, 1000, generator=gen(12))).bfloat16()
    y = cabi.softmax_fwd(xb.to(gpu))
    assert bool(torch.isfinite(y).all())
    assert_close(y, torch.ops.aten._softmax(xb.float(), -1, False), torch.bfloat16, "scaled inputs",
                 scale=5.0)  # the reference's own test allows 0.05


@pytest.mark.parametrize("off", [1, 2, 3, 5])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
def test_misaligned_pointers(cabi, oracle, gpu, dtype, off):
    # test/xpu/test_nn_xpu.py:17922-17998 (tensors whose data pointer is offset by one element) and
    # :14056-14106 (rows of a sliced tensor start at arbitrary alignments)
    for N in (2048, 2049, 127):
        M = 9
        x = torch.randn(M, N, generator=gen(20)).to(dtype)
        dy = torch.randn(M, N, generator=gen(21)).to(dtype)
        w = torch.randn(N, generator=gen(22)).to(dtype)
        xg, dyg, wg = (offset_view(t.to(gpu), off) for t in (x, dy, w))
        y = cabi.softmax_fwd(xg, y=offset_view(torch.empty_like(xg), off))
        assert_close(y, oracle.softmax_fwd(to_np32(x)), dtype, "softmax y")
        gi = cabi.softmax_bwd(dyg, y, gi=offset_view(torch.empty_like(xg), off))
        assert_close(gi, oracle.softmax_bwd(to_np32(dy), to_np32(y)), dtype, "softmax grad_input")
        ly, mean, rstd = cabi.layer_norm_fwd(xg, wg, None, 1e-5, y=offset_view(torch.empty_like(xg), off),
                                             mean=offset_view(torch.empty(M, device=gpu), 1),
                                             rstd=offset_view(torch.empty(M, device=gpu), 3))
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(w), None, 1e-5)
        assert_close(ly, oy, dtype, "layer_norm y")
        dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, wg, dx=offset_view(torch.empty_like(xg), off),
                                         dgamma=offset_view(torch.empty_like(wg), off),
                                         dbeta=offset_view(torch.empty_like(wg), off))
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(mean), to_np32(rstd),
                                              to_np32(w))
        assert_close(dx, odx, dtype, "layer_norm dx")
        assert_close(dg, odg, dtype, "layer_norm dgamma")
        assert_close(db, odb, dtype, "layer_norm dbeta")


def _variants(cabi, op, N, dt):
    """Every (lanes, packs) the library accepts for rows of N elements of dtype code dt."""
    found = []
    for G in (8, 16, 32, 64, 128, 256, 512, 1024):
        for V in (1, 2, 4, 8, 16):
            cabi.set_override(op, G, V)
            try:
                p = cabi.plan(op, 100, N, dt, dt)
                found.append((G, V, p["block_threads"]))
            except RuntimeError:
                pass
    cabi.set_override(op)
    return found


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_every_compiled_variant_and_the_multipass_kernels(cabi, oracle, gpu, dtype):
    """Forces each (lanes per row, packs per lane) kernel that exists for a shape, and the
    multi-pass kernels, and checks them all against the oracle; they must also agree with the
    automatic choice to the stated tolerance."""
    dt = cabi.dtype_code(dtype)
    total = 0
    for N in (64, 200, 1001, 1024, 4096, 5000):
        M = 21
        x = torch.randn(M, N, generator=gen(30)).to(dtype)
        dy = torch.randn(M, N, generator=gen(31)).to(dtype)
        w = (1 + 0.1 * torch.randn(N, generator=gen(32))).to(dtype)
        b = (0.1 * torch.randn(N, generator=gen(33))).to(dtype)
        xg, dyg, wg, bg = x.to(gpu), dy.to(gpu), w.to(gpu), b.to(gpu)
        oy, om, orr = oracle.layer_norm_fwd(to_np32(x), (N,), to_np32(w), to_np32(b), 1e-5)
        odx, odg, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(x), (N,), om, orr, to_np32(w))
        ory, orr2 = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(w), 1e-6)
        ordx, ordg = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), orr2, to_np32(w))
        mean_g = torch.from_numpy(om.reshape(-1)).to(gpu)
        rstd_g = torch.from_numpy(orr.reshape(-1)).to(gpu)
        rstd2_g = torch.from_numpy(orr2.reshape(-1)).to(gpu)
        for stream_only in (False, True):
            fwd_v = [(-1, 0, 0)] if stream_only else _variants(cabi, cabi.OP_LAYER_NORM_FWD, N, dt)
            bwd_v = [(-1, 0, 0)] if stream_only else _variants(cabi, cabi.OP_LAYER_NORM_BWD, N, dt)
            assert fwd_v and bwd_v
            for (G, V, _) in fwd_v:
                print("forced fwd", dtype, N, G, V, flush=True)
                cabi.set_override(cabi.OP_LAYER_NORM_FWD, G, V)
                cabi.set_override(cabi.OP_RMS_NORM_FWD, G, V)
                y, mean, rstd = cabi.layer_norm_fwd(xg, wg, bg, 1e-5)
                assert_close(y, oy, dtype, "LN y G=%d V=%d" % (G, V))
                assert_close(mean, om.reshape(-1), dtype, "LN mean")
                assert_close(rstd, orr.reshape(-1), dtype, "LN rstd")
                ry, rr = cabi.rms_norm_fwd(xg, wg, 1e-6)
                assert_close(ry, ory, dtype, "RMS y G=%d V=%d" % (G, V))
                assert_close(rr, orr2.reshape(-1), dtype, "RMS rstd")
                total += 1
            for (G, V, _) in bwd_v:
                print("forced bwd", dtype, N, G, V, flush=True)
                cabi.set_override(cabi.OP_LAYER_NORM_BWD, G, V)
                cabi.set_override(cabi.OP_RMS_NORM_BWD, G, V)
                dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean_g, rstd_g, wg)
                assert_close(dx, odx, dtype, "LN dx G=%d V=%d" % (G, V))
                assert_close(dg, odg, dtype, "LN dgamma G=%d V=%d" % (G, V))
                assert_close(db, odb, dtype, "LN dbeta G=%d V=%d" % (G, V))
                rdx, rdg = cabi.rms_norm_bwd(dyg, xg, rstd2_g, wg)
                assert_close(rdx, ordx, dtype, "RMS dx G=%d V=%d" % (G, V))
                assert_close(rdg, ordg, dtype, "RMS dgamma G=%d V=%d" % (G, V))
                total += 1
        cabi.clear_overrides()
        sx = (3 * torch.randn(M, N, generator=gen(34))).to(dtype)
        sxg = sx.to(gpu)
        for is_log in (False, True):
            osy = oracle.softmax_fwd(to_np32(sx), is_log)
            for (G, V, _) in _variants(cabi, cabi.OP_SOFTMAX_FWD, N, dt) + [(-1, 0, 0)]:
                cabi.set_override(cabi.OP_SOFTMAX_FWD, G, V)
                y = cabi.softmax_fwd(sxg, is_log)
                assert_close(y, osy, dtype, "softmax y G=%d V=%d" % (G, V))
                total += 1
            cabi.set_override(cabi.OP_SOFTMAX_FWD)
            y = cabi.softmax_fwd(sxg, is_log)
            osg = oracle.softmax_bwd(to_np32(dy), to_np32(y), is_log)
            for (G, V, _) in _variants(cabi, cabi.OP_SOFTMAX_BWD, N, dt) + [(-1, 0, 0)]:
                cabi.set_override(cabi.OP_SOFTMAX_BWD, G, V)
                gi = cabi.softmax_bwd(dyg, y, is_log)
                assert_close(gi, osg, dtype, "softmax grad_input G=%d V=%d" % (G, V))
                total += 1
            cabi.set_override(cabi.OP_SOFTMAX_BWD)
    assert total > 40


def test_rows_wider_than_the_register_file(cabi, oracle, gpu):
    # rows that only the multi-pass kernels can take (the role of SoftmaxForwardKernelFunctor and
    # the K5/K6 split path in the reference), without forcing
    N, M = 300001, 3
    x = torch.randn(M, N, generator=gen(40))
    dy = torch.randn(M, N, generator=gen(41))
    w = 1 + 0.1 * torch.randn(N, generator=gen(42))
    assert cabi.plan(cabi.OP_LAYER_NORM_BWD, M, N)["resident"] == 0
    xg, dyg, wg = x.to(gpu), dy.to(gpu), w.to(gpu)
    y, mean, rstd = cabi.layer_norm_fwd(xg, wg, wg, 1e-5)
    oy, om, orr = oracle.layer_norm_fwd(x.numpy(), (N,), w.numpy(), w.numpy(), 1e-5)
    assert_close(y, oy, torch.float32, "y")
    assert_close(mean, om.reshape(-1), torch.float32, "mean")
    dx, dg, db = cabi.layer_norm_bwd(dyg, xg, mean, rstd, wg)
    odx, odg, odb = oracle.layer_norm_bwd(dy.numpy(), x.numpy(), (N,), to_np32(mean), to_np32(rstd), w.numpy())
    assert_close(dx, odx, torch.float32, "dx")
    assert_close(dg, odg, torch.float32, "dgamma")
    assert_close(db, odb, torch.float32, "dbeta")
    for is_log in (False, True):
        sy = cabi.softmax_fwd(xg, is_log)
        assert_close(sy, oracle.softmax_fwd(x.numpy(), is_log), torch.float32, "softmax y")
        gi = cabi.softmax_bwd(dyg, sy, is_log)
        assert_close(gi, oracle.softmax_bwd(dy.numpy(), to_np32(sy), is_log), torch.float32, "grad_input")


def test_backward_is_deterministic(cabi, gpu):
    M, N = 5000, 3072
    x = torch.randn(M, N, generator=gen(50)).bfloat16().to(gpu)
    dy = torch.randn(M, N, generator=gen(51)).bfloat16().to(gpu)
    w = torch.randn(N, generator=gen(52)).to(gpu)
    _, mean, rstd = cabi.layer_norm_fwd(x, w, w, 1e-5)
    first = cabi.layer_norm_bwd(dy, x, mean, rstd, w)
    for _ in range(3):
        again = cabi.layer_norm_bwd(dy, x, mean, rstd, w)
        assert all(torch.equal(a, b) for a, b in zip(first, again))
