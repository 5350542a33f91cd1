"""Short ragged softmax rows (N % pack != 0, N <= 2048 16-bit / 1024 float32: attention scores of
ViT / CLIP / Whisper are rows of 197, 577, 77, 1500 elements) through the LDS-staged kernels
(softmax_fwd_flat_kernel / softmax_bwd_flat_kernel): a workgroup copies a run of whole rows to
LDS with aligned 128-bit accesses and its lane groups work on the rows there.  The reference
takes its general (unvectorized) forward for such rows (SoftMaxKernels.cpp:546-684 behind the
dispatch at :1621-1718).  Checked against the CPU oracle at the family's tolerances (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2) and against the general kernels forced on the
same inputs: every lanes-per-row and packs-per-lane class, row counts that end inside a workgroup's run of rows and
inside a pack, -inf / NaN rows, safe softmax, and tensors off 16-byte alignment (which keep the
general kernels)."""
import pytest
import torch

from helpers import assert_close, gen, offset_view, to_np32

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
# (rows, N): N picks the lanes per row (8 / 16 / 32 / 64), rows end inside a run and inside a pack
SHAPES = [(1, 3), (7, 5), (1001, 33), (333, 77), (64, 129), (515, 197), (9, 255), (40, 257),
          (123, 511), (17, 513), (61, 577), (10, 1001), (24, 1023),
          # 3 and 4 packs a lane, 4 lanes a row, and rows beyond 1024 elements (32 KB of LDS)
          (50, 21), (300, 45), (77, 93), (19, 750), (33, 1500), (9, 2047), (5, 1025),
          # very short rows of whole packs whose pack count fits the resident layouts badly
          (1000, 24), (333, 72), (129, 80), (77, 88)]


def _general(cabi, op, M, N, dtype, fn):
    """Runs fn with the planner's own layout forced, which keeps the general kernel."""
    code = cabi.dtype_code(dtype)
    p = cabi.plan(op, M, N, code, code)
    try:
        if p["resident"]:
            cabi.set_override(op, p["lanes_per_row"], p["packs_per_lane"])
        else:
            cabi.set_override(op, -1, 1)
        return fn()
    finally:
        cabi.clear_overrides()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("is_log", [False, True], ids=["softmax", "log_softmax"])
def test_forward_and_backward_against_oracle(cabi, oracle, gpu, dtype, is_log):
    for i, (M, N) in enumerate(SHAPES):
        g = gen(1200 + i)
        x = (3.0 * torch.randn(M, N, generator=g)).to(dtype)
        if N > 2:
            x[0, N // 2:] = float("-inf")
        grad = torch.randn(M, N, generator=g).to(dtype)
        xg, gg = x.to(gpu), grad.to(gpu)
        assert xg.data_ptr() % 16 == 0 and gg.data_ptr() % 16 == 0
        what = "[%d, %d] %s" % (M, N, dtype)
        y = cabi.softmax_fwd(xg, is_log)
        oy = oracle.softmax_fwd(to_np32(x), is_log)
        assert_close(y, oy, dtype, "forward " + what)
        yref = _general(cabi, cabi.OP_SOFTMAX_FWD, M, N, dtype, lambda: cabi.softmax_fwd(xg, is_log))
        assert_close(yref, oy, dtype, "general forward " + what)
        assert_close(y, to_np32(yref), dtype, "LDS-staged vs general forward " + what)
        # backward on the saved output as the dtype holds it (finite entries: softmax of -inf is 0,
        # log_softmax of -inf is -inf, whose exp is 0)
        ys = y.clone()
        gi = cabi.softmax_bwd(gg, ys, is_log)
        ogi = oracle.softmax_bwd(to_np32(grad), to_np32(ys), is_log)
        assert_close(gi, ogi, dtype, "backward " + what)
        giref = _general(cabi, cabi.OP_SOFTMAX_BWD, M, N, dtype, lambda: cabi.softmax_bwd(gg, ys, is_log))
        assert_close(giref, ogi, dtype, "general backward " + what)
        # the same result on a second run (fixed summation order)
        assert torch.equal(cabi.softmax_fwd(xg, is_log).view(torch.uint8), y.view(torch.uint8))
        assert torch.equal(cabi.softmax_bwd(gg, ys, is_log).view(torch.uint8), gi.view(torch.uint8))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_neighbours_stay_untouched_and_off_alignment_agrees(cabi, oracle, gpu, dtype):
    """The run of rows leaves LDS in whole packs: nothing before the tensor or behind its last
    (partial) pack may change.  A tensor 2 elements off 16-byte alignment takes the general kernel
    and gives the same values."""
    M, N = 77, 197
    x = torch.randn(M, N, generator=gen(1300)).to(dtype)
    oy = oracle.softmax_fwd(to_np32(x), False)
    big = torch.full((M * N + 64,), 7.0, dtype=dtype, device=gpu)
    yv = big[32:32 + M * N].view(M, N)
    assert yv.data_ptr() % 16 == 0
    cabi.softmax_fwd(x.to(gpu), False, y=yv)
    assert_close(yv, oy, dtype, "forward into a view")
    assert bool((big[:32] == 7.0).all()) and bool((big[32 + M * N:] == 7.0).all())
    xo = offset_view(x.to(gpu), 2)
    assert xo.data_ptr() % 16 != 0
    assert_close(cabi.softmax_fwd(xo, False), oy, dtype, "forward off alignment")


def test_special_rows(cabi, oracle, gpu):
    """All -inf rows are NaN (softmax) or zeros (safe softmax); NaN poisons its row only."""
    M, N = 40, 197
    x = torch.randn(M, N, generator=gen(1310))
    x[3] = float("-inf")
    x[5, 17] = float("nan")
    x[7, :100] = float("-inf")
    for dtype in (torch.float32, torch.bfloat16):
        xg = x.to(dtype).to(gpu)
        y = cabi.softmax_fwd(xg, False)
        assert bool(torch.isnan(y[3]).all()) and bool(torch.isnan(y[5]).all())
        ok = [r for r in range(M) if r not in (3, 5)]
        assert_close(y[ok], oracle.softmax_fwd(to_np32(x.to(dtype)[ok]), False), dtype, "finite rows")
        assert bool((y[7, :100] == 0).all())
        ys = cabi.safe_softmax_fwd(xg)
        assert bool((ys[3] == 0).all()) and bool(torch.isnan(ys[5]).all())
        assert_close(ys[ok], oracle.softmax_fwd(to_np32(x.to(dtype)[ok]), False), dtype, "safe softmax")
        ly = cabi.softmax_fwd(xg, True)
        assert bool(torch.isnan(ly[3]).all()) and bool((ly[7, :100] == float("-inf")).all())


def test_vit_attention_shape_through_the_host_op(ops, gpu):
    """aten-signature op on [B, H, T, T] scores with T = 197 (ViT-B/16 at 224 x 224), bf16."""
    x = torch.randn(2, 12, 197, 197, generator=gen(1320)).bfloat16()
    y = ops._softmax(x.to(gpu), -1, False)
    ref = torch.softmax(x.float(), -1)
    assert_close(y, to_np32(ref), torch.bfloat16, "ViT attention softmax")
    g = torch.randn(x.shape, generator=gen(1321)).bfloat16()
    gi = ops._softmax_backward_data(g.to(gpu), y, -1, torch.bfloat16)
    yd = y.cpu().double()
    refg = yd * (g.double() - (yd * g.double()).sum(-1, keepdim=True))
    assert_close(gi, to_np32(refg), torch.bfloat16, "ViT attention softmax backward")
