"""GPU parity of _safe_softmax, _masked_softmax and _masked_softmax_backward, through the C ABI
and through the host operators, against the CPU oracle, the committed golden vectors and PyTorch's
CPU ATen ops on the same seeded inputs.

The reference tests these ops by "same op on CPU, assertEqual" (test/xpu/test_transformers_xpu.py
and test/xpu/test_nn_xpu.py masked-softmax cases in intel/torch-xpu-ops: mask types 0/1/2, fully
masked rows, [B, T] key padding and [T, T] source masks under [B, H, T, T] scores).

Tolerances as for softmax: float32 rtol = atol = 1e-5; float16/bfloat16 atol 1e-2, rtol 1.6e-2.
"""
import pytest
import torch

from helpers import GOLDEN_DTYPES, assert_close, gen, load_golden, offset_view, rowsum_slack, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
SHAPES = [(1, 1), (3, 8), (7, 64), (5, 127), (64, 256), (33, 1024), (9, 4097), (12, 4096),
          (6, 8192), (3, 16384), (2, 40000)]
CASES = load_golden()


def _mask(M, N, g, p=0.3):
    mask = torch.rand(M, N, generator=g) < p
    if M > 1:
        mask[1] = False          # an untouched row
    if M > 2:
        mask[2] = True           # every element masked
    if M > 3 and N > 1:
        mask[3] = True
        mask[3, N // 3] = False  # a single survivor
    return mask


def _check_masked(cabi, oracle, gpu, x, grad, mask, dtype, tag):
    xg, gg, mg = x.to(gpu), grad.to(gpu), mask.to(gpu)
    y = cabi.masked_softmax_fwd(xg, mg)
    assert y.dtype == dtype and y.shape == x.shape
    oy = oracle.masked_softmax_fwd(to_np32(x), mask.numpy())
    assert_close(y, oy, dtype, tag + " y")
    full = mask.expand(x.shape)
    yc = y.cpu()
    dead = full.all(-1, keepdim=True).expand(x.shape)
    assert bool(torch.isnan(yc[dead]).all()), tag + ": fully masked rows are NaN"
    assert bool((yc[full & ~dead] == 0).all()), tag + ": masked elements are exactly 0"
    cy = torch.ops.aten._masked_softmax(x.float(), full.contiguous(), -1, 2)
    assert_close(y, cy, dtype, tag + " y vs ATen CPU")
    # backward consumes the device's own output and the full-shape mask
    fg = full.contiguous().to(gpu)
    gi = cabi.masked_softmax_bwd(gg, y, fg)
    ogi = oracle.masked_softmax_bwd(to_np32(grad), to_np32(y), full.numpy())
    ok = ~torch.isnan(torch.from_numpy(ogi))
    y0 = torch.where(full, torch.zeros(()), yc.float())
    sl = rowsum_slack(y0 * grad.float(), y0) if dtype == torch.float32 else None
    assert_close(gi, ogi, dtype, tag + " grad_input", slack=sl)
    gic = gi.cpu()
    assert bool((gic[full & ok] == 0).all()), tag + ": masked elements get a zero gradient"
    cgi = torch.ops.aten._masked_softmax_backward(grad.float(), yc.float(), full.contiguous(), -1)
    assert_close(gi, cgi, dtype, tag + " grad_input vs ATen CPU", slack=None if sl is None else 2 * sl)
    return y, gi


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_masked_softmax_fwd_bwd(cabi, oracle, gpu, dtype, shape):
    M, N = shape
    print("case masked_softmax", dtype, shape, flush=True)
    g = gen(41)
    x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
    grad = torch.randn(M, N, generator=g).to(dtype)
    _check_masked(cabi, oracle, gpu, x, grad, _mask(M, N, g), dtype, "full mask")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_nan_output_poisons_its_backward_row(cabi, oracle, gpu, dtype):
    """A row whose unmasked inputs are all -inf comes out NaN, and its backward is NaN at the
    masked positions too: 0 * (g - NaN), as SoftMaxKernels.cpp:991-1047 evaluates it."""
    g = gen(43)
    for (M, N) in ((6, 40), (5, 127), (4, 2048), (3, 4097)):
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        grad = torch.randn(M, N, generator=g).to(dtype)
        mask = torch.rand(M, N, generator=g) < 0.4
        x[1] = torch.where(mask[1], x[1], torch.full_like(x[1], float("-inf")))
        y = cabi.masked_softmax_fwd(x.to(gpu), mask.to(gpu))
        assert_close(y, oracle.masked_softmax_fwd(to_np32(x), mask.numpy()), dtype, "y")
        assert bool(torch.isnan(y[1]).all())
        gi = cabi.masked_softmax_bwd(grad.to(gpu), y, mask.to(gpu))
        ogi = oracle.masked_softmax_bwd(to_np32(grad), to_np32(y), mask.numpy())
        assert_close(gi, ogi, dtype, "grad_input")
        nan = torch.isnan(gi.cpu())
        assert bool(nan[1].all()) and not bool(nan[[0] + list(range(2, M))].any())
        assert bool(torch.equal(nan, torch.isnan(torch.from_numpy(ogi))))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
@pytest.mark.parametrize("T", [8, 33, 128, 257])
def test_mask_layouts_under_attention_scores(cabi, oracle, gpu, dtype, T):
    # [B, T] key padding (mask_type 1), [T, T] source mask (mask_type 0) and [B, 1, T, T] read in
    # place must give what the mask expanded to the scores' shape gives
    B, H = 3, 5
    g = gen(42)
    x = (3.0 * torch.randn(B, H, T, T, generator=g)).to(dtype)
    grad = torch.randn(B, H, T, T, generator=g).to(dtype)
    causal = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    pad = torch.arange(T)[None, :] >= torch.tensor([T, T // 2, 1])[:, None]          # [B, T]
    both = causal[None, None] | pad[:, None, None, :]                                 # [B, 1, T, T]
    for name, small, view in (("BxT", pad, pad[:, None, None, :]), ("TxT", causal, causal[None, None]),
                              ("Bx1xTxT", both, both)):
        print("case mask layout", name, dtype, T, flush=True)
        full = view.expand(B, H, T, T).contiguous()
        y_small = cabi.masked_softmax_fwd(x.to(gpu), small.contiguous().to(gpu))
        y_full = cabi.masked_softmax_fwd(x.to(gpu), full.to(gpu))
        assert torch.equal(y_small, y_full), name
        assert_close(y_small, oracle.masked_softmax_fwd(to_np32(x), view.numpy()), dtype, name + " y")
        gi_small = cabi.masked_softmax_bwd(grad.to(gpu), y_small, small.contiguous().to(gpu))
        gi_full = cabi.masked_softmax_bwd(grad.to(gpu), y_small, full.to(gpu))
        assert torch.equal(gi_small, gi_full), name


@pytest.mark.parametrize("case", sorted(CASES))
def test_golden_vectors(cabi, gpu, case):
    c = CASES[case]
    dt = GOLDEN_DTYPES[case.split("_")[0]]
    mask = c["msk"].bool()
    y = cabi.masked_softmax_fwd(c["msm_x"].to(gpu), mask.to(gpu))
    assert_close(y, c["msm_y"], dt, case + " masked y")
    gi = cabi.masked_softmax_bwd(c["dy"].to(gpu), c["msm_y"].to(gpu), mask.to(gpu))
    assert_close(gi, c["msm_gi"], dt, case + " masked grad_input")
    ys = cabi.safe_softmax_fwd(c["sm_x"].to(gpu))
    assert_close(ys, c["ssm_y"], dt, case + " safe y")
    assert bool((ys[2] == 0).all())


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_safe_softmax(cabi, oracle, gpu, dtype):
    g = gen(43)
    for (M, N) in ((1, 1), (7, 64), (5, 127), (9, 2048), (4, 4097), (3, 16384), (2, 40000)):
        print("case safe_softmax", dtype, M, N, flush=True)
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        x[0] = float("-inf")
        if M > 1:
            x[1, N // 2:] = float("-inf")
        if M > 2:
            x[2, N // 3] = float("nan")
        y = cabi.safe_softmax_fwd(x.to(gpu))
        assert_close(y, oracle.safe_softmax_fwd(to_np32(x)), dtype, "safe y")
        assert_close(y, torch.ops.aten._safe_softmax(x.float(), -1), dtype, "safe y vs ATen CPU")
        yc = y.cpu()
        assert bool((yc[0] == 0).all())
        if M > 2:
            assert bool(torch.isnan(yc[2]).all())
        # every other row is plain softmax: NaN rows are NaN in both, and the values agree to
        # one unit in the last place (the two code paths may round the last multiply and the
        # conversion to 16 bits in one step or in two)
        plain = cabi.softmax_fwd(x.to(gpu)).cpu()
        assert torch.equal(torch.isnan(yc[1:]), torch.isnan(plain[1:]))
        if M > 1:
            ibits = torch.int32 if dtype == torch.float32 else torch.int16
            ulps = (yc[1:].nan_to_num(nan=0.0).view(ibits).to(torch.int64) -
                    plain[1:].nan_to_num(nan=0.0).view(ibits).to(torch.int64)).abs().max()
            assert int(ulps) <= (0 if dtype == torch.float32 else 1), (dtype, M, N, int(ulps))
    # half input with a float result
    x = torch.randn(5, 300, generator=g).half()
    x[4] = float("-inf")
    y = cabi.safe_softmax_fwd(x.to(gpu), out_dtype=torch.float32)
    assert y.dtype == torch.float32
    assert_close(y, oracle.safe_softmax_fwd(to_np32(x)), torch.float32, "half_to_float safe y")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_forced_variants_multipass_and_misaligned(cabi, oracle, gpu, dtype):
    """Every compiled (lanes, packs) variant and the multi-pass kernels, forced, with the mask
    pointer and the data pointers offset from their allocations."""
    dt = cabi.dtype_code(dtype)
    g = gen(44)
    for N in (64, 200, 1001, 1024, 4096, 5000):
        M = 21
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        grad = torch.randn(M, N, generator=g).to(dtype)
        mask = _mask(M, N, g)
        oy = oracle.masked_softmax_fwd(to_np32(x), mask.numpy())
        xs = x.clone()
        xs[0] = float("-inf")
        osafe = oracle.safe_softmax_fwd(to_np32(xs))
        xg, gg, xsg = (offset_view(t.to(gpu), 1) for t in (x, grad, xs))
        mg = offset_view(mask.to(gpu), 3)
        variants = {}
        for op in (cabi.OP_SOFTMAX_FWD, cabi.OP_SOFTMAX_BWD):
            found = [(-1, 0)]
            for G in (8, 16, 32, 64, 128, 256, 512, 1024):
                for V in (1, 2, 4, 8, 16):
                    cabi.set_override(op, G, V)
                    try:
                        cabi.plan(op, M, N, dt, dt)
                        found.append((G, V))
                    except RuntimeError:
                        pass
            cabi.set_override(op)
            variants[op] = found
        E = 4 if dtype == torch.float32 else 8
        # the masked kernels exist up to 32 elements a lane on 1024 lanes; a forced layout
        # beyond that is refused for a masked call
        has_masked = lambda G, V: not (G == 1024 and V * E > 32)
        for (G, V) in variants[cabi.OP_SOFTMAX_FWD]:
            print("forced masked fwd", dtype, N, G, V, flush=True)
            cabi.set_override(cabi.OP_SOFTMAX_FWD, G, V)
            if has_masked(G, V):
                y = cabi.masked_softmax_fwd(xg, mg)
                assert_close(y, oy, dtype, "masked y G=%d V=%d" % (G, V))
            else:
                with pytest.raises(RuntimeError):
                    cabi.masked_softmax_fwd(xg, mg)
            assert_close(cabi.safe_softmax_fwd(xsg), osafe, dtype, "safe y G=%d V=%d" % (G, V))
        cabi.set_override(cabi.OP_SOFTMAX_FWD)
        y = cabi.masked_softmax_fwd(xg, mg)
        ogi = oracle.masked_softmax_bwd(to_np32(grad), to_np32(y), mask.numpy())
        for (G, V) in variants[cabi.OP_SOFTMAX_BWD]:
            print("forced masked bwd", dtype, N, G, V, flush=True)
            cabi.set_override(cabi.OP_SOFTMAX_BWD, G, V)
            if has_masked(G, V):
                gi = cabi.masked_softmax_bwd(gg, y, mg)
                assert_close(gi, ogi, dtype, "masked grad_input G=%d V=%d" % (G, V))
            else:
                with pytest.raises(RuntimeError):
                    cabi.masked_softmax_bwd(gg, y, mg)
        cabi.set_override(cabi.OP_SOFTMAX_BWD)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_host_ops_match_aten_cpu(ops, gpu, dtype):
    """torch.ops.mi355x._masked_softmax / _masked_softmax_backward / _safe_softmax with the
    reference's schemas: every mask type, every dim, dtype conversion of _safe_softmax."""
    g = gen(45)
    B, H, T = 2, 3, 16
    x = (3.0 * torch.randn(B, H, T, T, generator=g)).to(dtype)
    grad = torch.randn(B, H, T, T, generator=g).to(dtype)
    full = torch.rand(B, H, T, T, generator=g) < 0.3
    pad = torch.arange(T)[None, :] >= torch.tensor([T - 3, 5])[:, None]
    causal = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    for mask, mtype, dims in ((full, 2, (-1, 0, 1, 2, 3, None)), (pad, 1, (-1, None, 1)),
                              (causal, 0, (-1, 3, 2))):
        for dim in dims:
            print("case host masked", dtype, mtype, dim, flush=True)
            y = ops._masked_softmax(x.to(gpu), mask.to(gpu), dim, mtype)
            cy = torch.ops.aten._masked_softmax(x.float(), mask, dim, mtype)
            assert y.dtype == dtype and y.shape == x.shape
            assert_close(y, cy, dtype, "y mask_type=%d dim=%s" % (mtype, dim))
    for dim in (-1, 1, None):
        gi = ops._masked_softmax_backward(grad.to(gpu), x.to(gpu).abs().clamp(max=1), full.to(gpu), dim)
        cgi = torch.ops.aten._masked_softmax_backward(grad.float(), x.float().abs().clamp(max=1), full, dim)
        assert gi.dtype == dtype
        assert_close(gi, cgi, dtype, "grad_input dim=%s" % dim, scale=2.0)
    with pytest.raises(RuntimeError, match="Mask shape should match grad shape"):
        ops._masked_softmax_backward(grad.to(gpu), grad.to(gpu), pad.to(gpu), -1)
    # 0-dim and empty inputs
    s = ops._masked_softmax(torch.tensor(2.0, device=gpu), torch.tensor(False, device=gpu), None, 2)
    assert s.shape == () and float(s) == 1.0
    e = ops._masked_softmax(torch.empty(0, 4, device=gpu), torch.empty(0, 4, dtype=torch.bool, device=gpu), -1, 2)
    assert e.shape == (0, 4)
    # _safe_softmax: dims, all -inf slices, dtype argument
    xs = x.clone()
    xs[0, 1] = float("-inf")
    for dim in (-1, 0, 2):
        y = ops._safe_softmax(xs.to(gpu), dim)
        assert_close(y, torch.ops.aten._safe_softmax(xs.float(), dim), dtype, "safe dim=%d" % dim)
    assert bool((ops._safe_softmax(xs.to(gpu), -1)[0, 1] == 0).all())
    y = ops._safe_softmax(xs.to(gpu), -1, dtype=torch.float32)
    assert y.dtype == torch.float32
    assert_close(y, torch.ops.aten._safe_softmax(xs.float(), -1), dtype, "safe with dtype=float")
