"""The fused residual add -> LayerNorm / RMSNorm (-> output cast) operators on the GPU, through the
extern "C" ABI (mi355x_add_layer_norm_fwd / _bwd, mi355x_add_rms_norm_fwd / _bwd), the host
operators (torch.ops.mi355x.add_rms_norm & co.) and the autograd wrappers.

The reference has no fused operator; its forward (VectorizedLayerNormKernelFunctor,
src/ATen/native/xpu/sycl/LayerNormKernels.cpp:469-586) starts from the summed row.  So the checks
are: h equals an elementwise add of the two tensors in the row dtype bit for bit (computed by
PyTorch on the CPU); y, mean, rstd and the gradients match the CPU oracle's norm of that h at the
family's tolerances (float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2); and the fused
kernels agree with the unfused kernels run on h, forward and backward -- statistics bit for bit,
element results equal or adjacent (helpers.assert_same_arithmetic: the two template instances may
contract a multiply-add differently) -- because they share their arithmetic.  Every kernel family is reached: rows in registers (whole packs and
ragged), rows beyond the registers on one workgroup, and few very long rows split over
workgroups."""
import ctypes

import pytest
import torch

from helpers import assert_close, assert_same_arithmetic, colsum_slack, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
NAME = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16"}
# (rows, N): registers / ragged / 512 lanes / beyond the registers, one workgroup a row (M >= 512)
# / split over workgroups
SHAPES = [(7, 64), (5, 127), (33, 1024), (9, 4097), (12, 4096), (4, 5120), (6, 8192), (3, 16384),
          (520, 40000), (2, 300000)]


def _staged(dtype, N):
    """Short ragged rows: the plain kernels (no add, no cast) stage them through LDS and sum a row
    in another order than the kernels with the add or the cast, which take the general layout."""
    E = 4 if dtype == torch.float32 else 8
    return N % E != 0 and N <= 256 * E


def _mk(M, N, dtype, seed, wdtype=None):
    g = gen(seed)
    x = torch.randn(M, N, generator=g).to(dtype)
    res = (2 * torch.randn(M, N, generator=g)).to(dtype)
    dy = torch.randn(M, N, generator=g).to(dtype)
    gh = torch.randn(M, N, generator=g).to(dtype)
    wdt = dtype if wdtype is None else wdtype
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(wdt)
    beta = (0.1 * torch.randn(N, generator=g)).to(wdt)
    return x, res, dy, gh, gamma, beta


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("mixed", [False, True], ids=["w_same", "w_fp32"])
def test_add_norm_forward_and_backward(cabi, oracle, gpu, dtype, shape, mixed):
    if mixed and dtype == torch.float32:
        pytest.skip("mixed precision means float32 weights beside 16-bit rows")
    M, N = shape
    print("case fused add norm", dtype, shape, mixed, flush=True)
    x, res, dy, gh, gamma, beta = _mk(M, N, dtype, 21, torch.float32 if mixed else None)
    xg, rg, dyg, ghg, gg, bg = (t.to(gpu) for t in (x, res, dy, gh, gamma, beta))
    h_cpu = x + res  # an elementwise add in the row dtype: one rounding of the float32 sum
    wtol = gamma.dtype
    # 16-bit rows of 4096 / 5120 elements: the plain forward takes an exact two-pack layout
    # (5120: 320 lanes x 2 packs) that the fused add does not have (256 lanes x 3 packs there)
    same_layout = not (dtype != torch.float32 and N == 5120) and not _staged(dtype, N)
    for rms in (False, True):
        what = "rms_norm" if rms else "layer_norm"
        if rms:
            y, h, rstd = cabi.add_rms_norm_fwd(xg, rg, gg, 1e-6)
            uy, urstd = cabi.rms_norm_fwd(h, gg, 1e-6)
            oy, oh, orr = oracle.add_rms_norm_fwd(to_np32(x), to_np32(res), (N,), to_np32(gamma),
                                                  1e-6, NAME[dtype])
        else:
            y, h, mean, rstd = cabi.add_layer_norm_fwd(xg, rg, gg, bg, 1e-5)
            uy, umean, urstd = cabi.layer_norm_fwd(h, gg, bg, 1e-5)
            oy, oh, om, orr = oracle.add_layer_norm_fwd(to_np32(x), to_np32(res), (N,),
                                                        to_np32(gamma), to_np32(beta), 1e-5,
                                                        NAME[dtype])
            if same_layout:
                assert torch.equal(mean, umean)
            else:
                assert_close(mean, umean, torch.float32, what + " mean, fused against plain on h")
            assert_close(mean, om.reshape(-1), dtype, what + " mean")
        assert torch.equal(h.cpu(), h_cpu), what + ": h is not the elementwise sum"
        assert torch.equal(torch.from_numpy(oh), h_cpu.float())
        # the fused kernel and the plain kernel on h share their arithmetic (and, on the same
        # lane layout, the order of their sums: bit-equal statistics)
        if same_layout:
            assert torch.equal(rstd, urstd), what
        else:
            assert_close(rstd, urstd, torch.float32, what + " rstd, fused against plain on h")
        if not _staged(dtype, N):
            assert_same_arithmetic(y, uy, what + " y, fused against plain on h")
        assert_close(uy, oy, dtype, what + " y, plain on h")
        assert_close(y, oy, dtype, what + " y")
        assert_close(rstd, orr.reshape(-1), dtype, what + " rstd")
        # in place on the residual stream (h written over res) and over x
        for over in ("res", "x"):
            xx, rr = xg.clone(), rg.clone()
            target = rr if over == "res" else xx
            if rms:
                y2, h2, rstd2 = cabi.add_rms_norm_fwd(xx, rr, gg, 1e-6, h=target)
            else:
                y2, h2, _, rstd2 = cabi.add_layer_norm_fwd(xx, rr, gg, bg, 1e-5, h=target)
            assert h2.data_ptr() == target.data_ptr()
            assert torch.equal(h2, h) and torch.equal(y2, y) and torch.equal(rstd2, rstd), (what, over)
        # backward: dh = norm backward at h + the gradient of the residual path.  (16-bit rows of
        # 5120 and 6144 elements, and LayerNorm rows of 4096, take another lane layout -- another
        # order of the column sums -- with the residual gradient than without: there the two
        # are each held to the oracle, below, and not to each other)
        same_bwd_layout = not (dtype != torch.float32 and (N in (5120, 6144) or (N == 4096 and not rms)))
        same_bwd_layout = same_bwd_layout and not _staged(dtype, N)
        # (and long rows whose plain backward goes to teams of workgroups, which the backward
        # with a residual gradient does not)
        pb = cabi.plan(cabi.OP_RMS_NORM_BWD if rms else cabi.OP_LAYER_NORM_BWD, M, N,
                       cabi.dtype_code(dtype), cabi.dtype_code(gamma.dtype))
        same_bwd_layout = same_bwd_layout and not (pb["resident"] == 0 and pb["block_threads"] == 512
                                                   and pb["packs_per_lane"] == 2)
        if rms:
            dh, dg = cabi.add_rms_norm_bwd(dyg, ghg, h, rstd, gg)
            udx, udg = cabi.rms_norm_bwd(dyg, h, rstd, gg)
            nh, _ = cabi.add_rms_norm_bwd(dyg, None, h, rstd, gg)
            odh, odg = oracle.add_rms_norm_bwd(to_np32(dy), to_np32(gh), to_np32(h), (N,),
                                               to_np32(rstd), to_np32(gamma))
            xhat = h.cpu().double() * rstd.cpu().double().reshape(M, 1)
        else:
            dh, dg, db = cabi.add_layer_norm_bwd(dyg, ghg, h, mean, rstd, gg)
            udx, udg, udb = cabi.layer_norm_bwd(dyg, h, mean, rstd, gg)
            nh, _, _ = cabi.add_layer_norm_bwd(dyg, None, h, mean, rstd, gg)
            odh, odg, odb = oracle.add_layer_norm_bwd(to_np32(dy), to_np32(gh), to_np32(h), (N,),
                                                      to_np32(mean), to_np32(rstd), to_np32(gamma))
            xhat = (h.cpu().double() - mean.cpu().double().reshape(M, 1)) * \
                rstd.cpu().double().reshape(M, 1)
            if same_bwd_layout:
                assert_same_arithmetic(db, udb, what + " dbeta, fused against plain")
            sl = colsum_slack(dy.double()) if wtol == torch.float32 else None
            assert_close(db, odb, wtol, what + " dbeta", slack=sl)
        if _staged(dtype, N):
            pdx = (oracle.rms_norm_bwd(to_np32(dy), to_np32(h), (N,), to_np32(rstd), to_np32(gamma))
                   if rms else oracle.layer_norm_bwd(to_np32(dy), to_np32(h), (N,), to_np32(mean),
                                                     to_np32(rstd), to_np32(gamma)))[0]
            assert_close(udx, pdx, dtype, what + " plain dx")
            assert_close(udg, odg, wtol, what + " plain dgamma",
                         slack=colsum_slack(dy.double() * xhat) if wtol == torch.float32 else None)
        assert torch.equal(nh, udx), what + ": no residual gradient must be the plain backward"
        if same_bwd_layout:
            assert_same_arithmetic(dg, udg, what + " dgamma, fused against plain", max_fraction=0.05)
        assert_close(dh, odh, dtype, what + " dh")
        sl = colsum_slack(dy.double() * xhat) if wtol == torch.float32 else None
        assert_close(dg, odg, wtol, what + " dgamma", slack=sl)
        # in place on the incoming gradient
        ghc = ghg.clone()
        if rms:
            dh2, _ = cabi.add_rms_norm_bwd(dyg, ghc, h, rstd, gg, dh=ghc)
        else:
            dh2, _, _ = cabi.add_layer_norm_bwd(dyg, ghc, h, mean, rstd, gg, dh=ghc)
        assert torch.equal(dh2, dh), what + ": dh written over grad_h"


@pytest.mark.parametrize("ydtype", [torch.bfloat16, torch.float16], ids=str)
def test_output_cast_of_float32_rows(cabi, oracle, gpu, ydtype):
    """y written in 16 bits from float32 rows: one rounding of the float32 result, so it equals the
    plain float32 kernel's y converted afterwards, bit for bit; with and without the add."""
    for (M, N) in ((7, 64), (5, 127), (12, 4096), (9, 4097), (4, 5120), (3, 16384), (520, 40000),
                   (2, 300000)):
        print("case output cast", ydtype, (M, N), flush=True)
        x, res, _, _, gamma, beta = _mk(M, N, torch.float32, 22)
        xg, rg, gg, bg = (t.to(gpu) for t in (x, res, gamma, beta))
        for rms in (False, True):
            for add in (False, True):
                r = rg if add else None
                if rms:
                    y, h, rstd = cabi.add_rms_norm_fwd(xg, r, gg, 1e-6, y_dtype=ydtype)
                    y32, h32, rstd32 = cabi.add_rms_norm_fwd(xg, r, gg, 1e-6)
                else:
                    y, h, mean, rstd = cabi.add_layer_norm_fwd(xg, r, gg, bg, 1e-5, y_dtype=ydtype)
                    y32, h32, mean32, rstd32 = cabi.add_layer_norm_fwd(xg, r, gg, bg, 1e-5)
                    if _staged(torch.float32, N) and not add:
                        assert_close(mean, to_np32(mean32), torch.float32, "mean, cast against plain")
                    else:
                        assert torch.equal(mean, mean32)
                assert y.dtype == ydtype
                if _staged(torch.float32, N) and not add:
                    # (the float32 y comes from the LDS-staged kernel, the cast one does not)
                    assert_close(y, to_np32(y32), ydtype, "cast y against the float32 y")
                    assert_close(rstd, to_np32(rstd32), torch.float32, "rstd, cast against plain")
                else:
                    assert_same_arithmetic(y, y32.to(ydtype), "cast y against the float32 y converted")
                    assert torch.equal(rstd, rstd32)
                if add:
                    assert torch.equal(h, h32) and torch.equal(h.cpu(), x + res)
                else:
                    assert h is None
                    # no add, no cast: the plain operator
                    plain = (cabi.rms_norm_fwd(xg, gg, 1e-6)[0] if rms
                             else cabi.layer_norm_fwd(xg, gg, bg, 1e-5)[0])
                    assert torch.equal(y32, plain)  # the very same kernel
                hsrc = to_np32(x + res) if add else to_np32(x)
                oy = (oracle.rms_norm_fwd(hsrc, (N,), to_np32(gamma), 1e-6)[0] if rms
                      else oracle.layer_norm_fwd(hsrc, (N,), to_np32(gamma), to_np32(beta), 1e-5)[0])
                assert_close(y, oy, ydtype, "cast y")


def test_misaligned_pointers_and_argument_checks(cabi, oracle, gpu):
    x, res, dy, gh, gamma, beta = _mk(37, 520, torch.bfloat16, 23)
    put = lambda t, o: offset_view(t.to(gpu), o)  # noqa: E731
    y, h, rstd = cabi.add_rms_norm_fwd(put(x, 1), put(res, 3), put(gamma, 1), 1e-6,
                                       h=put(torch.empty_like(x), 5), y=put(torch.empty_like(x), 7))
    assert torch.equal(h.cpu(), x + res)
    oy, _, orr = oracle.add_rms_norm_fwd(to_np32(x), to_np32(res), (520,), to_np32(gamma), 1e-6, "bf16")
    assert_close(y, oy, torch.bfloat16, "misaligned y")
    L = cabi.lib()
    one = ctypes.c_void_p(256)  # never dereferenced: every call below is rejected before a launch
    BF, F16, F32 = cabi.BF16, cabi.F16, cabi.F32
    # y_dtype: the row dtype, or a 16-bit type for float32 rows only
    assert L.mi355x_add_rms_norm_fwd(one, one, one, one, one, one, 4, 8, 1e-6, BF, BF, F32, None) == -1
    assert L.mi355x_add_rms_norm_fwd(one, one, one, one, one, one, 4, 8, 1e-6, BF, BF, F16, None) == -1
    assert L.mi355x_add_rms_norm_fwd(one, one, one, one, one, one, 4, 8, 1e-6, F32, F32, 7, None) == -1
    # a residual needs somewhere to put h
    assert L.mi355x_add_rms_norm_fwd(one, one, one, None, one, one, 4, 8, 1e-6, BF, BF, BF, None) == -3
    assert L.mi355x_add_layer_norm_fwd(one, one, one, one, None, one, one, one, 4, 8, 1e-5, BF, BF,
                                       BF, None) == -3
    # empty problems are no-ops
    assert L.mi355x_add_rms_norm_fwd(None, None, None, None, None, None, 0, 8, 1e-6, BF, BF, BF, None) == 0
    assert L.mi355x_add_rms_norm_bwd(None, None, None, None, None, None, None, None, 0, 0, 8, BF, BF,
                                     None) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_host_operators_and_autograd(pkg, ops, gpu, dtype):
    """torch.ops.mi355x.add_rms_norm / add_layer_norm (+ the in-place forms and the backward ops)
    and pkg.fused with autograd, against the unfused composition run by PyTorch on the CPU in
    float32."""
    B, T, D = 3, 17, 384
    g = gen(24)
    x = torch.randn(B, T, D, generator=g).to(dtype)
    res = torch.randn(B, T, D, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    b = (0.1 * torch.randn(D, generator=g)).to(dtype)
    xg, rg, wg, bg = (t.to(gpu) for t in (x, res, w, b))
    y, h, mean, rstd = ops.add_layer_norm(xg, rg, [D], wg, bg, 1e-5)
    assert y.shape == x.shape and mean.shape == (B, T, 1) and mean.dtype == torch.float32
    assert torch.equal(h.cpu(), x + res)
    ref = torch.nn.functional.layer_norm((x + res).float(), (D,), w.float(), b.float(), 1e-5)
    assert_close(y, ref, dtype, "add_layer_norm y")
    rr = rg.clone()
    y2, mean2, rstd2 = ops.add_layer_norm_(xg, rr, [D], wg, bg, 1e-5)
    assert torch.equal(rr, h) and torch.equal(y2, y) and torch.equal(rstd2, rstd)
    y, h, rstd = ops.add_rms_norm(xg, rg, [D], wg, None)
    ref = torch.nn.functional.rms_norm((x + res).float(), (D,), w.float(), None)
    assert rstd.shape == (B, T, 1)
    assert_close(y, ref, dtype, "add_rms_norm y")
    rr = rg.clone()
    y2, rstd2 = ops.add_rms_norm_(xg, rr, [D], wg, None)
    assert torch.equal(rr, h) and torch.equal(y2, y) and torch.equal(rstd2, rstd)
    if dtype == torch.float32:
        yb, _, _ = ops.add_rms_norm(xg, rg, [D], wg, None, torch.bfloat16)
        assert yb.dtype == torch.bfloat16
        assert_same_arithmetic(yb, y.bfloat16(), "out_dtype bfloat16")
        with pytest.raises(RuntimeError, match="out_dtype"):
            ops.add_rms_norm(xg, rg, [D], wg, None, torch.float64)
    else:
        with pytest.raises(RuntimeError, match="out_dtype"):
            ops.add_rms_norm(xg, rg, [D], wg, None, torch.float32)
    with pytest.raises(RuntimeError, match="residual must have the shape"):
        ops.add_rms_norm(xg, rg[:, :5], [D], wg, None)
    # autograd: two blocks chained through the residual stream, so that h of the first block
    # gets a gradient from both of its uses
    def chain(xs, rs, ws, bs, fused):
        if fused:
            y1, h1 = pkg.fused.add_rms_norm(xs, rs, ws, 1e-6)
            y2, h2 = pkg.fused.add_layer_norm(y1, h1, ws, bs, 1e-5)
        else:
            h1 = xs + rs
            y1 = torch.nn.functional.rms_norm(h1, (D,), ws, 1e-6)
            h2 = y1 + h1
            y2 = torch.nn.functional.layer_norm(h2, (D,), ws, bs, 1e-5)
        return y2, h2
    gy = torch.randn(B, T, D, generator=g).to(dtype)
    gh2 = torch.randn(B, T, D, generator=g).to(dtype)
    leaves = [t.detach().clone().requires_grad_() for t in (xg, rg, wg, bg)]
    y2, h2 = chain(*leaves, True)
    torch.autograd.backward([y2, h2], [gy.to(gpu), gh2.to(gpu)])
    cl = [t.float().detach().clone().requires_grad_() for t in (x, res, w, b)]
    cy2, ch2 = chain(*cl, False)
    torch.autograd.backward([cy2, ch2], [gy.float(), gh2.float()])
    assert_close(y2, cy2, dtype, "chain y", scale=4.0)
    for a, c, nm in zip(leaves, cl, ("dx", "dresidual", "dweight", "dbias")):
        assert a.grad is not None and a.grad.dtype == dtype
        assert_close(a.grad, c.grad, dtype, "chain " + nm, scale=8.0)
    assert torch.equal(leaves[0].grad, leaves[1].grad)  # x and residual share the gradient of h


def test_unused_outputs_are_not_materialized_and_direct_ops_refuse_grad(pkg, ops, gpu):
    """Only y, or only h, feeds the loss: the unused output's gradient reaches backward as None
    (no tensor of zeros is made for it) and the results equal the unfused composition; the direct
    operators, which record no autograd graph, refuse tensors that require a gradient."""
    B, D = 37, 512
    g = gen(25)
    dtype = torch.bfloat16
    x = torch.randn(B, D, generator=g).to(dtype)
    res = torch.randn(B, D, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    b = (0.1 * torch.randn(D, generator=g)).to(dtype)
    gy = torch.randn(B, D, generator=g).to(dtype)
    for norm in ("rms", "ln"):
        for use in ("y", "h"):
            leaves = [t.to(gpu).requires_grad_() for t in (x, res, w, b)]
            if norm == "rms":
                y, h = pkg.fused.add_rms_norm(leaves[0], leaves[1], leaves[2], 1e-6)
            else:
                y, h = pkg.fused.add_layer_norm(leaves[0], leaves[1], leaves[2], leaves[3], 1e-5)
            (y if use == "y" else h).backward(gy.to(gpu))
            cl = [t.float().requires_grad_() for t in (x, res, w, b)]
            ch = cl[0] + cl[1]
            cy = (torch.nn.functional.rms_norm(ch, (D,), cl[2], 1e-6) if norm == "rms"
                  else torch.nn.functional.layer_norm(ch, (D,), cl[2], cl[3], 1e-5))
            (cy if use == "y" else ch).backward(gy.float())
            if use == "h":
                # the gradient of h passes through to x and residual, the weights get none
                assert torch.equal(leaves[0].grad.cpu(), gy) and torch.equal(leaves[1].grad.cpu(), gy)
                assert leaves[2].grad is None and leaves[3].grad is None
            else:
                assert_close(leaves[0].grad, cl[0].grad, dtype, norm + " dx, only y used", scale=2.0)
                assert torch.equal(leaves[0].grad, leaves[1].grad)
                assert_close(leaves[2].grad, cl[2].grad, dtype, norm + " dweight, only y used",
                             scale=2.0)
    xg = x.to(gpu).requires_grad_()
    with pytest.raises(RuntimeError, match="records no autograd graph"):
        ops.add_rms_norm(xg, res.to(gpu), [D], w.to(gpu), None)
    with pytest.raises(RuntimeError, match="records no autograd graph"):
        ops.add_layer_norm(x.to(gpu), res.to(gpu), [D], w.to(gpu).requires_grad_(), b.to(gpu), 1e-5)
    with torch.no_grad():
        ops.add_rms_norm(xg, res.to(gpu), [D], w.to(gpu), None)  # fine: nothing is recorded
