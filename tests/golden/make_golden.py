"""Writes tests/golden/aten_cpu_golden.npz: input/output vectors of PyTorch's CPU ATen
implementation of the operator family (the arithmetic parity target named for this path).

Nothing from the reference repository is imported or run: the vectors come from the installed
torch wheel (torch 2.10.0 when this file was last run; the version is stored in the archive).
They pin what no closed form pins: where low-precision outputs are rounded, bit-exact beta on
constant rows, -inf / NaN propagation, and the +-1e4 outlier behaviour.

    python tests/golden/make_golden.py            # rewrites the .npz next to this file

Layout of the archive: "<case>/<tensor>" arrays.  16-bit tensors are stored as uint16 bit
patterns ("...:bf16" / "...:f16" suffix in the key) so numpy needs no bfloat16 support.
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
SHAPES = [(7, 64), (5, 127), (3, 4097)]
DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def put(store, key, t):
    t = t.detach().contiguous()
    if t.dtype == torch.float32:
        store[key] = t.numpy()
    elif t.dtype == torch.float16:
        store[key + ":f16"] = t.view(torch.int16).numpy().view(np.uint16)
    elif t.dtype == torch.bfloat16:
        store[key + ":bf16"] = t.view(torch.int16).numpy().view(np.uint16)
    elif t.dtype == torch.bool:
        store[key] = t.numpy().astype(np.uint8)
    else:
        raise TypeError(t.dtype)


def stress_rows(M, N, g):
    x = torch.randn(M, N, generator=g)
    mask = torch.rand(M, N, generator=g) < 0.002
    sign = torch.where(torch.rand(M, N, generator=g) < 0.5, -1.0, 1.0)
    x = torch.where(mask, 1e4 * sign, x)
    x[0] = 1.5  # one all-constant row
    return x


def main():
    torch.manual_seed(0)
    torch.set_num_threads(1)
    store = {"meta/torch_version": np.frombuffer(torch.__version__.encode(), dtype=np.uint8)}
    for dname, dt in DTYPES.items():
        for (M, N) in SHAPES:
            g = torch.Generator().manual_seed(1000 + N)
            case = "%s_%dx%d" % (dname, M, N)
            x = stress_rows(M, N, g).to(dt)
            dy = torch.randn(M, N, generator=g).to(dt)
            gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dt)
            beta = (0.1 * torch.randn(N, generator=g)).to(dt)
            for k, v in (("x", x), ("dy", dy), ("gamma", gamma), ("beta", beta)):
                put(store, case + "/" + k, v)
            # LayerNorm, eps 1e-5.  CPU ATen returns mean/rstd in the input dtype for unmixed
            # 16-bit inputs; they are stored as returned.
            y, mean, rstd = torch.ops.aten.native_layer_norm(x, [N], gamma, beta, 1e-5)
            put(store, case + "/ln_y", y)
            put(store, case + "/ln_mean", mean.reshape(-1))
            put(store, case + "/ln_rstd", rstd.reshape(-1))
            dx, dg, db = torch.ops.aten.native_layer_norm_backward(
                dy, x, [N], mean, rstd, gamma, beta, [True, True, True])
            put(store, case + "/ln_dx", dx)
            put(store, case + "/ln_dgamma", dg)
            put(store, case + "/ln_dbeta", db)
            # mixed precision: 16-bit rows with float32 gamma/beta (fp32 statistics)
            if dt != torch.float32:
                g32, b32 = gamma.float(), beta.float()
                y, mean, rstd = torch.ops.aten.native_layer_norm(x, [N], g32, b32, 1e-5)
                put(store, case + "/lnmix_y", y)
                put(store, case + "/lnmix_mean", mean.reshape(-1))
                put(store, case + "/lnmix_rstd", rstd.reshape(-1))
                dx, dg, db = torch.ops.aten.native_layer_norm_backward(
                    dy, x, [N], mean, rstd, g32, b32, [True, True, True])
                put(store, case + "/lnmix_dx", dx)
                put(store, case + "/lnmix_dgamma", dg)
                put(store, case + "/lnmix_dbeta", db)
            # RMSNorm, eps 1e-6 (forward op; backward through autograd: ATen has no CPU
            # _fused_rms_norm_backward kernel)
            xr, gr = x.clone().requires_grad_(), gamma.clone().requires_grad_()
            y, rstd = torch.ops.aten._fused_rms_norm(xr, [N], gr, 1e-6)
            put(store, case + "/rms_y", y)
            put(store, case + "/rms_rstd", rstd.reshape(-1).float())
            y.backward(dy)
            put(store, case + "/rms_dx", xr.grad)
            put(store, case + "/rms_dgamma", gr.grad)
            # softmax / log_softmax on scores with a masked tail and one fully masked row
            s = (3.0 * torch.randn(M, N, generator=g))
            s[1, N // 2:] = float("-inf")
            s[2, :] = float("-inf")
            s = s.to(dt)
            put(store, case + "/sm_x", s)
            for is_log, nm in ((False, "sm"), (True, "lsm")):
                fwd = torch.ops.aten._log_softmax if is_log else torch.ops.aten._softmax
                bwd = (torch.ops.aten._log_softmax_backward_data if is_log
                       else torch.ops.aten._softmax_backward_data)
                out = fwd(s, -1, False)
                put(store, case + "/%s_y" % nm, out)
                put(store, case + "/%s_gi" % nm, bwd(dy, out, -1, dt))
            # _safe_softmax on the same scores (row 2 is all -inf -> zeros), and
            # _masked_softmax / _masked_softmax_backward with ~30% of the elements masked,
            # row 3 untouched and row 4 fully masked
            put(store, case + "/ssm_y", torch.ops.aten._safe_softmax(s, -1))
            mask = torch.rand(M, N, generator=g) < 0.3
            if M > 3:
                mask[3] = False
            if M > 4:
                mask[4] = True
            put(store, case + "/msk", mask)
            finite = (3.0 * torch.randn(M, N, generator=g)).to(dt)
            put(store, case + "/msm_x", finite)
            out = torch.ops.aten._masked_softmax(finite, mask, -1, 2)
            put(store, case + "/msm_y", out)
            put(store, case + "/msm_gi",
                torch.ops.aten._masked_softmax_backward(dy, out, mask, -1))
    path = os.path.join(HERE, "aten_cpu_golden.npz")
    np.savez_compressed(path, **store)
    print("wrote", path, os.path.getsize(path), "bytes,", len(store), "arrays")
    group_norm_vectors()


# (N, C, spatial shape, groups): channel size a whole number of 16-byte packs, a ragged one,
# the 2-d input (one element per channel), one group, one channel per group
GN_SHAPES = [(3, 8, (4, 8), 2), (2, 6, (5,), 3), (5, 12, (), 4), (2, 4, (3, 3), 1), (2, 6, (16,), 6)]


def group_norm_vectors():
    """tests/golden/aten_cpu_group_norm.npz: native_group_norm / native_group_norm_backward of
    the CPU kernels, unmixed and (16-bit rows, float32 weights) mixed, eps 1e-5."""
    torch.manual_seed(0)
    store = {"meta/torch_version": np.frombuffer(torch.__version__.encode(), dtype=np.uint8)}
    for dname, dt in DTYPES.items():
        for (N, C, sp, G) in GN_SHAPES:
            g = torch.Generator().manual_seed(2000 + C)
            HxW = int(np.prod(sp)) if sp else 1
            case = "%s_%dx%dx%dg%d" % (dname, N, C, HxW, G)
            x = (0.5 + torch.randn((N, C) + sp, generator=g)).to(dt)
            dy = torch.randn((N, C) + sp, generator=g).to(dt)
            gamma = (1 + 0.1 * torch.randn(C, generator=g)).to(dt)
            beta = (0.1 * torch.randn(C, generator=g)).to(dt)
            for k, v in (("x", x), ("dy", dy), ("gamma", gamma), ("beta", beta)):
                put(store, case + "/" + k, v)
            variants = [("gn", gamma, beta)]
            if dt != torch.float32:
                variants.append(("gnmix", gamma.float(), beta.float()))
            for pre, gk, bk in variants:
                y, mean, rstd = torch.ops.aten.native_group_norm(x, gk, bk, N, C, HxW, G, 1e-5)
                put(store, case + "/%s_y" % pre, y)
                put(store, case + "/%s_mean" % pre, mean)
                put(store, case + "/%s_rstd" % pre, rstd)
                dx, dg, db = torch.ops.aten.native_group_norm_backward(
                    dy, x, mean, rstd, gk, N, C, HxW, G, [True, True, True])
                put(store, case + "/%s_dx" % pre, dx)
                put(store, case + "/%s_dgamma" % pre, dg)
                put(store, case + "/%s_dbeta" % pre, db)
    path = os.path.join(HERE, "aten_cpu_group_norm.npz")
    np.savez_compressed(path, **store)
    print("wrote", path, os.path.getsize(path), "bytes,", len(store), "arrays")


if __name__ == "__main__":
    main()
