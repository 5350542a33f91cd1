"""The C-ABI entry points under HIP graph capture: kernels only, launched on the stream they are
given, no allocation and no memset when the caller brings the outputs (and, for the RMSNorm
backward, the entry point whose scratch is the library's static device array).  A graph with the
RMSNorm forward, its backward and a log_softmax is replayed several times on fresh inputs, with
eager work and synchronizations between the replays, and every replay is compared bit for bit
with the same calls made eagerly (the allocating backward included) and with the CPU oracle at
the family's tolerances (16-bit atol 1e-2, rtol 1.6e-2)."""
import pytest
import torch

from helpers import assert_close, colsum_slack, gen, to_np32

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(512, 4096), (96, 18432)], ids=str)
def test_forward_backward_and_log_softmax_replay(cabi, oracle, gpu, shape):
    M, N = shape
    dt = torch.bfloat16
    g = gen(1700)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dt).to(gpu)
    x = torch.empty(M, N, dtype=dt, device=gpu)
    dy = torch.empty_like(x)
    y, dx, lsm = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    rstd = torch.empty(M, dtype=torch.float32, device=gpu)
    dw = torch.empty_like(w)

    def calls():
        cabi.rms_norm_fwd(x, w, 1e-6, y=y, rstd=rstd)
        cabi.rms_norm_bwd_static(dy, x, rstd, w, dx, dw)
        cabi.softmax_fwd(y, True, y=lsm)

    def fill(seed):
        gg = gen(seed)
        x.copy_(torch.randn(M, N, generator=gg).to(dt))
        dy.copy_(torch.randn(M, N, generator=gg).to(dt))

    fill(1701)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls()  # first calls outside the capture (per-device set-up of the static scratch)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()

    for rep in range(3):
        print("case graph replay", shape, rep, flush=True)
        fill(1710 + rep)
        for t in (y, dx, lsm, rstd, dw):
            t.fill_(7)  # a small fill kernel: the replay has to write every output again
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (y, rstd, dx, dw, lsm)]
        # the same calls made eagerly, the backward through the allocating entry point
        ey, erstd = cabi.rms_norm_fwd(x, w, 1e-6)
        edx, edw = cabi.rms_norm_bwd(dy, x, erstd, w)
        elsm = cabi.softmax_fwd(ey, True)
        torch.cuda.synchronize()
        for a, b, what in zip(got, (ey, erstd, edx, edw, elsm), ("y", "rstd", "dx", "dweight", "log_softmax")):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), (what, rep)
        oy, orstd = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(w), 1e-6)
        assert_close(got[0], oy, dt, "replayed forward")
        odx, odw = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(got[1]), to_np32(w))
        assert_close(got[2], odx, dt, "replayed dx")
        assert_close(got[3], odw, dt, "replayed dweight")
        assert_close(got[4], oracle.softmax_fwd(to_np32(got[0]), True), dt, "replayed log_softmax")


def test_long_rows_under_capture_keep_the_multi_launch_kernels(cabi, oracle, gpu):
    """Rows beyond one workgroup's registers, which eager calls give to teams of workgroups
    (forward and backward): a call on a capturing stream takes no bookkeeping slot (a replay
    would run with the id of the capture) and keeps the multi-launch kernels.  Every replay
    against the oracle, and against the eager team kernels at the family's tolerance."""
    M, N = 200, 65536
    dt = torch.bfloat16
    code = cabi.dtype_code(dt)
    p = cabi.plan(cabi.OP_RMS_NORM_BWD, M, N, code, code)
    assert p["resident"] == 0 and p["block_threads"] == 512 and p["packs_per_lane"] == 2, p
    g = gen(1760)
    w = (1 + 0.1 * torch.randn(N, generator=g)).to(dt).to(gpu)
    x = torch.empty(M, N, dtype=dt, device=gpu)
    dy = torch.empty_like(x)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    rstd = torch.empty(M, dtype=torch.float32, device=gpu)
    dw = torch.empty_like(w)
    nbytes = cabi.lib().mi355x_rms_norm_bwd_workspace_bytes(M, N, code, code, 1)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)

    def calls():
        cabi.rms_norm_fwd(x, w, 1e-6, y=y, rstd=rstd)
        cabi.rms_norm_bwd(dy, x, rstd, w, dx=dx, dgamma=dw, workspace=ws)

    def fill(seed):
        gg = gen(seed)
        x.copy_(torch.randn(M, N, generator=gg).to(dt))
        dy.copy_(torch.randn(M, N, generator=gg).to(dt))

    fill(1761)
    calls()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()
    for rep in range(3):
        print("case graph replay of long rows", rep, flush=True)
        fill(1770 + rep)
        for t in (y, dx, rstd, dw):
            t.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (y, rstd, dx, dw)]
        ey, erstd = cabi.rms_norm_fwd(x, w, 1e-6)
        edx, edw = cabi.rms_norm_bwd(dy, x, erstd, w)
        torch.cuda.synchronize()
        oy, orstd = oracle.rms_norm_fwd(to_np32(x), (N,), to_np32(w), 1e-6)
        assert_close(got[0], oy, dt, "replayed forward")
        assert_close(got[1], orstd.reshape(-1), torch.float32, "replayed rstd")
        odx, odw = oracle.rms_norm_bwd(to_np32(dy), to_np32(x), (N,), to_np32(got[1]), to_np32(w))
        sl = colsum_slack(dy.float().cpu() * x.float().cpu() * got[1].cpu().reshape(M, 1))
        assert_close(got[2], odx, dt, "replayed dx")
        assert_close(got[3], odw, dt, "replayed dweight", slack=sl)
        assert_close(edx, odx, dt, "eager dx (teams)")
        assert_close(edw, odw, dt, "eager dweight (teams)", slack=sl)
