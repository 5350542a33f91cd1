"""GPU parity of softmax / log_softmax / _safe_softmax over a dimension that is not innermost
(the [outer, dim, inner] kernels), through the C ABI, against the CPU oracle applied along the
same axis and against PyTorch's CPU ATen ops.

Mirrors test/regressions/test_softmax.py:18-46 and test/xpu/test_nn_xpu.py:14056-14106
(test_softmax_results: every dim of 4-d inputs, sliced/offset tensors) in intel/torch-xpu-ops.
Tolerances: float32 rtol = atol = 1e-5; float16/bfloat16 atol 1e-2, rtol 1.6e-2.
"""
import numpy as np
import pytest
import torch

from helpers import assert_close, gen, offset_view, rowsum_slack, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (outer, D, inner): small and ragged inner, inner a whole number of packs, inner wider than a
# wavefront of packs, D beyond what the registers hold (multi-pass), D = 1, outer = 1
SHAPES = [(3, 5, 2), (2, 7, 3), (4, 16, 8), (5, 33, 24), (2, 64, 127), (3, 21, 1024), (2, 4, 4100),
          (1, 256, 64), (2, 300, 40), (1, 1000, 16), (2, 3000, 9), (7, 1, 33), (1, 2, 100000)]


def _along(fn, a, axis):
    """Applies a last-dim oracle function along `axis`."""
    return np.moveaxis(fn(np.ascontiguousarray(np.moveaxis(a, axis, -1))), -1, axis)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("is_log", [False, True], ids=["softmax", "log_softmax"])
def test_strided_softmax_fwd_bwd(cabi, oracle, gpu, dtype, shape, is_log):
    print("case strided softmax", dtype, shape, is_log, flush=True)
    g = gen(61)
    x = (3.0 * torch.randn(shape, generator=g)).to(dtype)
    if shape[1] > 4:
        x[0, shape[1] // 2:, 0] = float("-inf")  # a masked tail in one column
    grad = torch.randn(shape, generator=g).to(dtype)
    mode = cabi.LOG_SOFTMAX if is_log else cabi.SOFTMAX
    y = cabi.softmax_strided_fwd(x.to(gpu), 1, mode)
    oy = _along(lambda a: oracle.softmax_fwd(a, is_log), to_np32(x), 1)
    assert y.dtype == dtype and y.shape == x.shape
    assert_close(y, oy, dtype, "y")
    fn = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
    assert_close(y, fn(x.float(), 1, False), dtype, "y vs ATen CPU")
    gi = cabi.softmax_strided_bwd(grad.to(gpu), y, 1, mode)
    ogi = _along(lambda a: a, to_np32(grad), 1)  # keep shapes explicit below
    ogi = np.moveaxis(oracle.softmax_bwd(np.ascontiguousarray(np.moveaxis(to_np32(grad), 1, -1)),
                                         np.ascontiguousarray(np.moveaxis(to_np32(y), 1, -1)), is_log),
                      -1, 1)
    yc, g32 = y.cpu().float().movedim(1, -1), grad.float().movedim(1, -1)
    sl = None
    if dtype == torch.float32:
        sl = rowsum_slack(g32, torch.exp(yc)) if is_log else rowsum_slack(yc * g32, yc)
        sl = sl.movedim(-1, 1)
    assert_close(gi, ogi, dtype, "grad_input", slack=sl)
    bfn = (torch.ops.aten._log_softmax_backward_data if is_log
           else torch.ops.aten._softmax_backward_data)
    cgi = bfn(grad.float(), y.cpu().float(), 1, torch.float32)
    assert_close(gi, cgi, dtype, "grad_input vs ATen CPU", slack=None if sl is None else 2 * sl)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_every_dim_of_a_4d_tensor_and_safe_mode(cabi, oracle, gpu, dtype):
    g = gen(62)
    x = (3.0 * torch.randn(6, 5, 12, 20, generator=g)).to(dtype)
    x[1, :, 3, 4] = float("-inf")
    x[:, 2, 0, 1] = float("-inf")
    for dim in (0, 1, 2, 3, -2):
        y = cabi.softmax_strided_fwd(x.to(gpu), dim, cabi.SAFE_SOFTMAX)
        oy = _along(oracle.safe_softmax_fwd, to_np32(x), dim)
        assert_close(y, oy, dtype, "safe y dim=%d" % dim)
        assert_close(y, torch.ops.aten._safe_softmax(x.float(), dim), dtype, "safe vs ATen dim=%d" % dim)
        p = cabi.softmax_strided_fwd(x.to(gpu), dim, cabi.SOFTMAX)
        assert_close(p, torch.ops.aten._softmax(x.float(), dim, False), dtype, "y dim=%d" % dim)
    assert bool((cabi.softmax_strided_fwd(x.to(gpu), 1, cabi.SAFE_SOFTMAX)[1, :, 3, 4] == 0).all())
    assert bool(torch.isnan(cabi.softmax_strided_fwd(x.to(gpu), 1, cabi.SOFTMAX)[1, :, 3, 4]).all())
    with pytest.raises(RuntimeError, match="invalid shape"):
        cabi.softmax_strided_bwd(x.to(gpu), x.to(gpu), 1, cabi.SAFE_SOFTMAX)


def test_half_to_float(cabi, gpu):
    g = gen(63)
    x = torch.randn(3, 37, 50, generator=g).half().to(gpu)
    grad = torch.randn(3, 37, 50, generator=g).to(gpu)
    for mode in (cabi.SOFTMAX, cabi.LOG_SOFTMAX):
        y = cabi.softmax_strided_fwd(x, 1, mode, out_dtype=torch.float32)
        yf = cabi.softmax_strided_fwd(x.float(), 1, mode)
        assert y.dtype == torch.float32
        assert_close(y, yf, torch.float32, "half_to_float y")
        gi = cabi.softmax_strided_bwd(grad, y, 1, mode, gi_dtype=torch.float16)
        assert gi.dtype == torch.float16
        assert_close(gi, cabi.softmax_strided_bwd(grad, yf, 1, mode), torch.float16, "half_to_float gi")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
def test_forced_variants_multipass_and_misaligned(cabi, oracle, gpu, dtype):
    """Every lanes-along-inner x rows-per-lane layout that can hold the shape, and the multi-pass
    kernels, forced, on tensors whose data pointers are offset from their allocations."""
    dt = cabi.dtype_code(dtype)
    g = gen(64)
    for shape in ((3, 24, 40), (2, 9, 1030), (2, 130, 16), (5, 2, 7)):
        outer, D, inner = shape
        x = (3.0 * torch.randn(shape, generator=g)).to(dtype)
        grad = torch.randn(shape, generator=g).to(dtype)
        xg, gg = offset_view(x.to(gpu), 1), offset_view(grad.to(gpu), 3)
        oy = _along(oracle.softmax_fwd, to_np32(x), 1)
        tried = 0
        for op, bwd in ((cabi.OP_SOFTMAX_STRIDED_FWD, False), (cabi.OP_SOFTMAX_STRIDED_BWD, True)):
            layouts = [(-1, 0)]
            for TX in (1, 2, 4, 8, 16, 32, 64):
                for V in (1, 2, 4, 8):
                    cabi.set_override(op, TX, V)
                    try:
                        p = cabi.strided_plan(bwd, outer, D, inner, dt)
                        assert p["resident"] == 1 and p["lanes_per_row"] == TX and p["packs_per_lane"] == V
                        layouts.append((TX, V))
                    except RuntimeError:
                        pass
            for (TX, V) in layouts:
                print("forced strided", dtype, shape, "bwd" if bwd else "fwd", TX, V, flush=True)
                cabi.set_override(op, TX, V)
                if not bwd:
                    y = cabi.softmax_strided_fwd(xg, 1, y=offset_view(torch.empty_like(xg), 2))
                    assert_close(y, oy, dtype, "y TX=%d V=%d" % (TX, V))
                else:
                    yg = offset_view(torch.from_numpy(oy).to(dtype).to(gpu), 1)
                    gi = cabi.softmax_strided_bwd(gg, yg, 1, gi=offset_view(torch.empty_like(gg), 2))
                    ogi = np.moveaxis(oracle.softmax_bwd(
                        np.ascontiguousarray(np.moveaxis(to_np32(grad), 1, -1)),
                        np.ascontiguousarray(np.moveaxis(to_np32(yg), 1, -1))), -1, 1)
                    assert_close(gi, ogi, dtype, "gi TX=%d V=%d" % (TX, V))
                tried += 1
            cabi.set_override(op)
        assert tried >= 4


def test_host_ops_use_the_strided_kernels_for_every_dim(ops, gpu):
    # test/regressions/test_softmax.py:18-46: every dim, forward and backward, against the CPU
    g = gen(65)
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.randn(4, 6, 10, 18, generator=g).to(dtype)
        dy = torch.randn(4, 6, 10, 18, generator=g).to(dtype)
        for dim in range(-4, 4):
            for is_log in (False, True):
                fwd = ops._log_softmax if is_log else ops._softmax
                bwd = ops._log_softmax_backward_data if is_log else ops._softmax_backward_data
                cf = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
                cb = (torch.ops.aten._log_softmax_backward_data if is_log
                      else torch.ops.aten._softmax_backward_data)
                y = fwd(x.to(gpu), dim, False)
                cy = cf(x.float(), dim, False)
                assert_close(y, cy, dtype, "y dim=%d" % dim)
                gi = bwd(dy.to(gpu), y, dim, dtype)
                assert_close(gi, cb(dy.float(), y.cpu().float(), dim, torch.float32), dtype,
                             "gi dim=%d" % dim, scale=2.0)
        # a non-contiguous input and a non-contiguous out=
        xt = x.to(gpu).transpose(1, 3)
        out = torch.empty(4, 18, 10, 6, dtype=dtype, device=gpu).transpose(0, 1).contiguous().transpose(0, 1)
        ops._softmax.out(xt, 1, False, out=out)
        assert_close(out, torch.ops.aten._softmax(x.float().transpose(1, 3), 1, False), dtype, "out=")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_many_rows_few_columns_are_split_over_workgroups(cabi, oracle, gpu, dtype):
    """D in the thousands under too few columns to fill the machine (the reference's own
    micro-benchmark, test/microbench/softmax.py:17: softmax over dim 0 of [8192, 64] and
    [8192, 8192]): the D rows of a tile are cut into chunks, one workgroup each, and the per-column
    maxima and sums cross three launches inside the output tensor.  Forced chunk counts, a ragged
    inner size, misaligned tensors, masked and NaN columns, the float16 -> float32 output; the
    in-place call falls back to one workgroup a tile."""
    dt = cabi.dtype_code(dtype)
    g = gen(66)
    ops = (cabi.OP_SOFTMAX_STRIDED_FWD, cabi.OP_SOFTMAX_STRIDED_BWD)
    try:
        for shape in ((1, 8192, 64), (2, 2500, 37), (1, 1100, 520), (3, 2300, 8)):
            outer, D, inner = shape
            x = (3.0 * torch.randn(shape, generator=g)).to(dtype)
            x[0, D // 3:, 0] = float("-inf")      # a masked tail
            x[0, :, 1] = float("-inf")            # a fully masked column
            x[0, D // 2, 2] = float("nan")        # a NaN poisons its column
            grad = torch.randn(shape, generator=g).to(dtype)
            xg, gg = offset_view(x.to(gpu), 1), offset_view(grad.to(gpu), 3)
            for chunks in (0, 1, 2, 5):
                for op in ops:
                    cabi.set_override(op, -1 if chunks else 0, chunks)
                p = cabi.strided_plan(False, outer, D, inner, dt)
                assert p["resident"] == 0
                if chunks:
                    assert (p["dim_chunks"] > 1) == (chunks > 1), (chunks, p)
                else:
                    assert p["dim_chunks"] > 1, p  # the planner's own choice for these shapes
                print("case split strided", dtype, shape, chunks, p["dim_chunks"], flush=True)
                for mode, is_log in ((cabi.SOFTMAX, False), (cabi.LOG_SOFTMAX, True)):
                    y = cabi.softmax_strided_fwd(xg, 1, mode, y=offset_view(torch.empty_like(xg), 2))
                    oy = _along(lambda a: oracle.softmax_fwd(a, is_log), to_np32(x), 1)
                    assert_close(y, oy, dtype, "split y chunks=%d log=%d" % (chunks, is_log))
                    gi = cabi.softmax_strided_bwd(gg, y, 1, mode,
                                                  gi=offset_view(torch.empty_like(gg), 2))
                    ogi = np.moveaxis(oracle.softmax_bwd(
                        np.ascontiguousarray(np.moveaxis(to_np32(grad), 1, -1)),
                        np.ascontiguousarray(np.moveaxis(to_np32(y), 1, -1)), is_log), -1, 1)
                    yc, g32 = y.cpu().float().movedim(1, -1), grad.float().movedim(1, -1)
                    sl = None
                    if dtype == torch.float32:
                        sl = (rowsum_slack(g32, torch.exp(yc)) if is_log
                              else rowsum_slack(yc * g32, yc)).movedim(-1, 1)
                    assert_close(gi, ogi, dtype, "split gi chunks=%d log=%d" % (chunks, is_log),
                                 slack=sl)
                ys = cabi.softmax_strided_fwd(xg, 1, cabi.SAFE_SOFTMAX)
                assert_close(ys, _along(oracle.safe_softmax_fwd, to_np32(x), 1), dtype, "split safe y")
                assert bool((ys[0, :, 1] == 0).all())
                if dtype == torch.float16:
                    y32 = cabi.softmax_strided_fwd(xg, 1, cabi.SOFTMAX, out_dtype=torch.float32)
                    assert_close(y32, _along(oracle.softmax_fwd, to_np32(x), 1), torch.float32,
                                 "split float16 -> float32 y")
                    g32g = grad.float().to(gpu)
                    gi16 = cabi.softmax_strided_bwd(g32g, y32, 1, cabi.SOFTMAX,
                                                    gi_dtype=torch.float16)
                    assert_close(gi16, cabi.softmax_strided_bwd(g32g, y32, 1, cabi.SOFTMAX),
                                 torch.float16, "split float32 -> float16 gi")
            cabi.clear_overrides()
            # in place: the output is the input, so the values cannot travel in it
            xin = x.to(gpu).clone()
            cabi.softmax_strided_fwd(xin, 1, cabi.SOFTMAX, y=xin)
            assert_close(xin, _along(oracle.softmax_fwd, to_np32(x), 1), dtype, "in place y")
    finally:
        cabi.clear_overrides()


def test_dim0_of_a_square_matrix_against_the_last_dim_kernels(cabi, gpu):
    """softmax over dim 0 of [8192, 8192] bf16 (test/microbench/softmax.py:17 in the reference)
    equals softmax over the last dim of the transpose, computed by the innermost-dimension kernels,
    within the 16-bit tolerance; forward and backward."""
    H = W = 8192
    g = gen(67)
    x = (2.0 * torch.randn(H, W, generator=g)).bfloat16().to(gpu)
    grad = torch.randn(H, W, generator=g).bfloat16().to(gpu)
    p = cabi.strided_plan(False, 1, H, W, cabi.BF16)
    assert p["resident"] == 0 and p["dim_chunks"] > 1, p
    y = cabi.softmax_strided_fwd(x, 0)
    yt = cabi.softmax_fwd(x.t().contiguous())
    assert_close(y, yt.t(), torch.bfloat16, "dim 0 y vs last-dim kernel")
    gi = cabi.softmax_strided_bwd(grad, y, 0)
    git = cabi.softmax_bwd(grad.t().contiguous(), y.t().contiguous())
    assert_close(gi, git.t(), torch.bfloat16, "dim 0 gi vs last-dim kernel")
    colsum = y.float().sum(0)
    assert_close(colsum, torch.ones_like(colsum), torch.bfloat16, "columns sum to 1")
