"""ATen's DispatchStub slots for this family (LayerNormKernel / LayerNormBackwardKernel,
GroupNormKernel / GroupNormBackwardKernel) pointed at the MI355X kernels -- what
REGISTER_XPU_DISPATCH does in src/ATen/native/xpu/LayerNorm.cpp:198-201 and GroupNorm.cpp:19-23 of
intel/torch-xpu-ops -- exercised through ATen callers that go through the stubs, with no aten
override in place:

  * aten::native_group_norm / native_group_norm_backward: ATen's own host function allocates the
    outputs and calls GroupNormKernel(device_type, ...);
  * layer_norm on a nested tensor: NestedTensor_layer_norm calls LayerNormKernel on the packed
    [sum of lengths, D] buffer, and its autograd formula calls LayerNormBackwardKernel.

Each result is compared with the CPU oracle (float32 rtol = atol = 1e-5; 16-bit atol 1e-2, rtol
1.6e-2) and, bit for bit, with the same kernels called through the C ABI, which shows that the stub
and not the stock kernel ran.  uninstall_* must put the stock kernels back."""
import warnings

import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close, colsum_slack, gen, to_np32

pytestmark = pytest.mark.gpu


@pytest.fixture()
def stock_aten(pkg):
    """No aten override while these tests run (they test the stub route); put it back afterwards
    if another test had installed it."""
    had = pkg._state["aten_lib"] is not None
    pkg.restore_aten_ops()
    yield
    if had:
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            pkg.override_aten_ops()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_group_norm_stubs(pkg, ops, cabi, oracle, gpu, stock_aten, dtype):
    N, C, H, W, groups = 3, 12, 10, 8, 4
    g = gen(70)
    x = torch.randn(N, C, H, W, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(C, generator=g)).to(dtype)
    b = (0.1 * torch.randn(C, generator=g)).to(dtype)
    dy = torch.randn(N, C, H, W, generator=g).to(dtype)
    xg, wg, bg, dyg = (t.to(gpu) for t in (x, w, b, dy))
    stock = torch.ops.aten.native_group_norm(xg, wg, bg, N, C, H * W, groups, 1e-5)
    ops.install_group_norm_dispatch_stubs()
    try:
        ops.install_group_norm_dispatch_stubs()  # a second install keeps the saved stock kernels
        y, mean, rstd = torch.ops.aten.native_group_norm(xg, wg, bg, N, C, H * W, groups, 1e-5)
        dx, dg, db = torch.ops.aten.native_group_norm_backward(dyg, xg, mean, rstd, wg, N, C, H * W,
                                                               groups, [True, True, True])
        # through autograd as well: F.group_norm -> native_group_norm -> the stub
        xs = xg.detach().clone().requires_grad_()
        F.group_norm(xs, groups, wg, bg, 1e-5).backward(dyg)
        # float64 goes on to the kernels that were registered before
        y64 = torch.ops.aten.native_group_norm(xg.double(), wg.double(), bg.double(), N, C, H * W,
                                               groups, 1e-5)[0]
    finally:
        ops.uninstall_group_norm_dispatch_stubs()
    after = torch.ops.aten.native_group_norm(xg, wg, bg, N, C, H * W, groups, 1e-5)
    for a, s in zip(after, stock):
        assert torch.equal(a, s)  # the stock kernels are back
    # the same kernels through the C ABI: same bits
    cy, cm, cr = cabi.group_norm_fwd(xg, wg, bg, groups, 1e-5)
    assert torch.equal(y, cy) and torch.equal(mean, cm) and torch.equal(rstd, cr)
    cdx, cdg, cdb = cabi.group_norm_bwd(dyg, xg, cm, cr, wg, groups)
    assert torch.equal(dx, cdx) and torch.equal(dg, cdg) and torch.equal(db, cdb)
    assert torch.equal(xs.grad, cdx)
    # and the oracle
    oy, om, orr = oracle.group_norm_fwd(to_np32(x), groups, to_np32(w), to_np32(b), 1e-5)
    assert_close(y, oy, dtype, "y")
    assert_close(mean, om, dtype, "mean")
    assert_close(rstd, orr, dtype, "rstd")
    odx, odg, odb = oracle.group_norm_bwd(to_np32(dy), to_np32(x), groups, to_np32(mean),
                                          to_np32(rstd), to_np32(w))
    assert_close(dx, odx, dtype, "dx")
    assert_close(dg, odg, dtype, "dgamma")
    assert_close(db, odb, dtype, "dbeta")
    ref64 = F.group_norm(x.double(), groups, w.double(), b.double(), 1e-5)
    assert y64.dtype == torch.float64
    assert float((y64.cpu() - ref64).abs().max()) < 1e-10


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_layer_norm_stubs_through_nested_tensors(pkg, ops, cabi, oracle, gpu, stock_aten, dtype):
    D = 192
    lengths = (5, 17, 1, 40)
    g = gen(71)
    parts = [torch.randn(L, D, generator=g).to(dtype) for L in lengths]
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    b = (0.1 * torch.randn(D, generator=g)).to(dtype)
    packed = torch.cat(parts)                     # the [sum of lengths, D] buffer ATen normalizes
    dy = torch.randn(packed.shape, generator=g).to(dtype)
    wg, bg = w.to(gpu), b.to(gpu)

    def run():
        nt = torch.nested.nested_tensor([p.to(gpu) for p in parts]).requires_grad_()
        ws, bs = wg.detach().clone().requires_grad_(), bg.detach().clone().requires_grad_()
        out = F.layer_norm(nt, (D,), ws, bs, 1e-5)
        grads = torch.nested.nested_tensor(list(dy.to(gpu).split(lengths)))
        out.backward(grads)
        return (torch.cat(out.detach().unbind()), torch.cat(nt.grad.unbind()), ws.grad, bs.grad)

    stock = run()
    ops.install_layer_norm_dispatch_stubs()
    try:
        y, dx, dw, db = run()
    finally:
        ops.uninstall_layer_norm_dispatch_stubs()
    after = run()
    for a, s in zip(after, stock):
        assert torch.equal(a, s)  # the stock kernels are back
    M = packed.shape[0]
    cy, cm, cr = cabi.layer_norm_fwd(packed.to(gpu), wg, bg, 1e-5)
    assert torch.equal(y, cy)  # the stub ran these kernels
    cdx, cdw, cdb = cabi.layer_norm_bwd(dy.to(gpu), packed.to(gpu), cm, cr, wg)
    assert torch.equal(dx, cdx) and torch.equal(dw, cdw) and torch.equal(db, cdb)
    oy, om, orr = oracle.layer_norm_fwd(to_np32(packed), (D,), to_np32(w), to_np32(b), 1e-5)
    assert_close(y, oy, dtype, "nested layer_norm y")
    odx, odw, odb = oracle.layer_norm_bwd(to_np32(dy), to_np32(packed), (D,), to_np32(cm),
                                          to_np32(cr), to_np32(w))
    assert_close(dx, odx, dtype, "nested layer_norm dx")
    xh = (packed.double() - torch.from_numpy(om).double().reshape(M, 1)) * \
        torch.from_numpy(orr).double().reshape(M, 1)
    sl = (colsum_slack(dy.double() * xh), colsum_slack(dy.double())) if dtype == torch.float32 \
        else (None, None)
    assert_close(dw, odw, dtype, "nested layer_norm dgamma", slack=sl[0])
    assert_close(db, odb, dtype, "nested layer_norm dbeta", slack=sl[1])
