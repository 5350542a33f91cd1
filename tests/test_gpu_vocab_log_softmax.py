"""log_softmax backward on vocabulary-sized rows (the cross_entropy case): rows too long for both
tensors in registers keep grad resident and stream y past it (log_softmax_bwd_grad_resident_kernel;
the reference walks the row twice in LogSoftmaxBackward, src/ATen/native/xpu/sycl/
SoftMaxKernels.cpp:991-1150).  Every packs-per-lane count of the kernel (9..20; 16-bit rows of
5..8 packs a lane hold both tensors in registers), with the row end inside and at the end of a
lane's last pack, misaligned
tensors and -inf / NaN entries, against the CPU oracle at the family's tolerances (float32
rtol = atol = 1e-5; 16-bit atol 1e-2, rtol 1.6e-2) and against the multi-pass kernel forced on
the same inputs.  The 16-bit forward holds rows of 17..20 packs a lane (the 151936 / 152064-entry
vocabularies) in registers as well: checked against the oracle and the multi-pass kernel."""
import pytest
import torch

from helpers import assert_close, gen, offset_view, rowsum_slack, to_np32

pytestmark = pytest.mark.gpu


def _case(cabi, oracle, gpu, M, N, dtype, off, seed, gi_dtype=None):
    g = gen(seed)
    x = 2.0 * torch.randn(M, N, generator=g)
    x[0, N // 3] = float("-inf")          # y = -inf, exp(y) = 0: the gradient passes through
    grad = torch.randn(M, N, generator=g).to(dtype)
    y = torch.log_softmax(x, -1).to(dtype)
    put = (lambda t: offset_view(t.to(gpu), off)) if off else (lambda t: t.to(gpu))
    yg, gg = put(y), put(grad)
    p = cabi.plan(cabi.OP_SOFTMAX_BWD, M, N, cabi.dtype_code(dtype), cabi.dtype_code(dtype))
    # 16-bit rows up to 65536 elements hold both tensors in registers (storage format); beyond
    # that, and for float32 rows beyond 32768, grad alone stays resident
    assert p["resident"] == (1 if dtype != torch.float32 and N <= 65536 else 0), p
    gi = cabi.softmax_bwd(gg, yg, True, gi_dtype=gi_dtype)
    try:
        cabi.set_override(cabi.OP_SOFTMAX_BWD, -1, 1)     # the multi-pass kernel
        ref = cabi.softmax_bwd(gg, yg, True, gi_dtype=gi_dtype)
    finally:
        cabi.clear_overrides()
    od = dtype if gi_dtype is None else gi_dtype
    ogi = oracle.softmax_bwd(to_np32(grad), to_np32(y), True)
    # float32: exp(y) * (a float32 sum over N terms) carries the sum's rounding (helpers.rowsum_slack)
    sl = rowsum_slack(to_np32(grad), torch.exp(y.double())) if od == torch.float32 else None
    what = "[%d, %d] %s off %d" % (M, N, dtype, off)
    assert_close(gi, ogi, od, "grad-resident log_softmax backward " + what, slack=sl)
    assert_close(ref, ogi, od, "multi-pass log_softmax backward " + what, slack=sl)
    assert_close(gi, to_np32(ref), od, "grad-resident vs multi-pass " + what, slack=sl)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
def test_every_pack_count_16bit(cabi, oracle, gpu, dtype):
    # packs a lane = ceil(N / 8192): 5 (one pack into the fifth round), 5 exactly, 6 .. 16
    for i, N in enumerate((32776, 40960, 49144, 50304, 65536, 73728, 81912, 90112, 100000, 106496,
                           114688, 122880, 128256, 131072,
                           # 17 .. 20: one pack into the round, Qwen's vocabularies, the maximum
                           131080, 140000, 151936, 152064, 163840)):
        _case(cabi, oracle, gpu, 3, N, dtype, 0, 900 + i)
    _case(cabi, oracle, gpu, 2, 50304, dtype, 3, 950)     # 6 bytes off 16-byte alignment
    _case(cabi, oracle, gpu, 2, 128256, dtype, 1, 951)


def test_every_pack_count_float32(cabi, oracle, gpu):
    # float32 rows: 4 elements a pack, the two-tensor kernels end at 32768 elements
    for i, N in enumerate((32772, 36864, 40000, 45056, 50304, 53248, 57344, 61440, 65536,
                           65540, 70000, 75968, 81920)):
        _case(cabi, oracle, gpu, 2, N, torch.float32, 0, 960 + i)
    _case(cabi, oracle, gpu, 2, 50304, torch.float32, 1, 970)


def test_float32_grad_to_float16_gradient(cabi, oracle, gpu):
    """half_to_float: float32 grad and y, float16 grad_input (SoftMax.cpp:72-100)."""
    _case(cabi, oracle, gpu, 2, 50304, torch.float32, 0, 980, gi_dtype=torch.float16)


def test_nan_poisons_its_row_only(cabi, gpu):
    M, N = 3, 50304
    y = torch.log_softmax(torch.randn(M, N, generator=gen(990)), -1).bfloat16()
    grad = torch.randn(M, N, generator=gen(991)).bfloat16()
    grad[1, 777] = float("nan")
    gi = cabi.softmax_bwd(grad.to(gpu), y.to(gpu), True)
    assert bool(torch.isnan(gi[1]).all())
    assert bool(torch.isfinite(gi[0]).all()) and bool(torch.isfinite(gi[2]).all())


def test_softmax_and_ragged_rows_keep_the_multi_pass_kernel(cabi, oracle, gpu):
    """The kernel serves log_softmax on whole packs only; softmax and ragged rows of that length
    still go through the multi-pass kernel and agree with the oracle."""
    M = 2
    for N, is_log in ((50304, False), (50257, True)):
        g = gen(995)
        x = torch.randn(M, N, generator=g)
        grad = torch.randn(M, N, generator=g).bfloat16()
        y = (torch.log_softmax(x, -1) if is_log else torch.softmax(x, -1)).bfloat16()
        gi = cabi.softmax_bwd(grad.to(gpu), y.to(gpu), is_log)
        assert_close(gi, oracle.softmax_bwd(to_np32(grad), to_np32(y), is_log), torch.bfloat16,
                     "N=%d log=%d" % (N, is_log))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("is_log", [False, True], ids=["softmax", "log_softmax"])
def test_forward_rows_of_17_to_20_packs_a_lane(cabi, oracle, gpu, dtype, is_log):
    code = cabi.dtype_code(dtype)
    for i, (V, N) in enumerate(((17, 131080), (18, 140000), (19, 151936), (19, 152064),
                                (20, 163840))):
        M = 3
        print("case vocabulary forward", dtype, is_log, (M, N), flush=True)
        p = cabi.plan(cabi.OP_SOFTMAX_FWD, M, N, code, code)
        assert (p["resident"], p["lanes_per_row"], p["packs_per_lane"]) == (1, 1024, V), p
        x = (3.0 * torch.randn(M, N, generator=gen(1500 + i))).to(dtype)
        x[0, N // 2:] = float("-inf")
        x[1, -1] = 30.0  # the maximum in the last pack of the row
        xg = x.to(gpu)
        y = cabi.softmax_fwd(xg, is_log)
        oy = oracle.softmax_fwd(to_np32(x), is_log)
        assert_close(y, oy, dtype, "forward [%d, %d] %s" % (M, N, dtype))
        try:
            cabi.set_override(cabi.OP_SOFTMAX_FWD, -1, 1)  # the multi-pass kernel
            ref = cabi.softmax_fwd(xg, is_log)
        finally:
            cabi.clear_overrides()
        assert_close(y, to_np32(ref), dtype, "register-resident vs multi-pass forward %d" % N)
        assert torch.equal(cabi.softmax_fwd(xg, is_log).view(torch.uint8), y.view(torch.uint8))
    # float32 output from float16 input (half_to_float, SoftMax.cpp:49-55) on the same kernels
    if dtype == torch.float16:
        x = (3.0 * torch.randn(2, 151936, generator=gen(1510))).to(dtype)
        y32 = cabi.softmax_fwd(x.to(gpu), is_log, out_dtype=torch.float32)
        assert_close(y32, oracle.softmax_fwd(to_np32(x), is_log), torch.float32,
                     "half_to_float 151936")
    # one row more than the registers hold: the multi-pass kernel
    assert cabi.plan(cabi.OP_SOFTMAX_FWD, 3, 163848, code, code)["resident"] == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("is_log", [False, True], ids=["softmax", "log_softmax"])
def test_backward_rows_of_5_to_8_packs_a_lane_in_storage_format(cabi, oracle, gpu, dtype, is_log):
    """16-bit rows of 32776 .. 65536 elements: both tensors in registers, kept packed."""
    code = cabi.dtype_code(dtype)
    for i, (V, N) in enumerate(((5, 32776), (5, 40960), (6, 49152), (7, 50304), (7, 57344),
                                (8, 65528), (8, 65536))):
        M = 3
        print("case packed softmax backward", dtype, is_log, (M, N), flush=True)
        p = cabi.plan(cabi.OP_SOFTMAX_BWD, M, N, code, code)
        assert (p["resident"], p["lanes_per_row"], p["packs_per_lane"]) == (1, 1024, V), p
        g = gen(1600 + i)
        x = 2.0 * torch.randn(M, N, generator=g)
        x[0, N // 3] = float("-inf")
        y = (torch.log_softmax(x, -1) if is_log else torch.softmax(x, -1)).to(dtype)
        grad = torch.randn(M, N, generator=g).to(dtype)
        yg, gg = y.to(gpu), grad.to(gpu)
        gi = cabi.softmax_bwd(gg, yg, is_log)
        ogi = oracle.softmax_bwd(to_np32(grad), to_np32(y), is_log)
        what = "[%d, %d] %s" % (M, N, dtype)
        assert_close(gi, ogi, dtype, "backward " + what)
        try:
            cabi.set_override(cabi.OP_SOFTMAX_BWD, -1, 1)  # the multi-pass kernel
            ref = cabi.softmax_bwd(gg, yg, is_log)
        finally:
            cabi.clear_overrides()
        assert_close(gi, to_np32(ref), dtype, "register-resident vs multi-pass backward " + what)
        assert torch.equal(cabi.softmax_bwd(gg, yg, is_log).view(torch.uint8), gi.view(torch.uint8))


def test_masked_backward_beyond_4_packs_a_lane_keeps_the_multi_pass_kernel(cabi, oracle, gpu):
    """The masked backward widens both tensors to float32 registers; rows of 40960 bf16 elements
    with a mask take the multi-pass kernel and still agree with the oracle."""
    M, N = 4, 40960
    g = gen(1650)
    x = torch.randn(M, N, generator=g)
    mask = torch.rand(M, N, generator=g) < 0.3
    mask[:, 0] = False
    y = torch.softmax(x.masked_fill(mask, float("-inf")), -1).bfloat16()
    grad = torch.randn(M, N, generator=g).bfloat16()
    gi = cabi.masked_softmax_bwd(grad.to(gpu), y.to(gpu), mask.to(gpu))
    ogi = oracle.masked_softmax_bwd(to_np32(grad), to_np32(y), mask.numpy())
    assert_close(gi, ogi, torch.bfloat16, "masked softmax backward [4, 40960]")
