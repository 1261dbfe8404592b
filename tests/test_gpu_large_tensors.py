"""Tensors beyond 2^30 elements (byte offsets beyond 4 GiB) through the convolution entry points.

The CPU oracle cannot finish these sizes, so the check is by samples: a few thousand output elements, the highest
addresses among them, are recomputed in float64 from the operands' patches (gathered on the device); the weight gradient is
checked through the adjoint identity <W', wgrad(dY, X)> = <conv(W', X), dY> against the forward pass checked just before.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _sample_coords(rng, N, C, H, W, count):
    n = rng.integers(0, N, count)
    c = rng.integers(0, C, count)
    y = rng.integers(0, H, count)
    x = rng.integers(0, W, count)
    n[:64], c[:64], y[:64], x[:64] = N - 1, C - 1, H - 1 - rng.integers(0, 2, 64), W - 1 - rng.integers(0, 4, 64)  # the far end
    n[64:96], c[64:96], y[64:96], x[64:96] = 0, 0, rng.integers(0, 2, 32), rng.integers(0, 4, 32)  # and the near one
    return n, c, y, x


@pytest.mark.parametrize("N,C,H", [(70000, 16, 32), (1100, 64, 128)])
def test_conv3x3_beyond_4_gib(dev, N, C, H):
    import torch
    from crusaderbackend_amd import capi
    assert N * C * H * H > 2 ** 30
    g = capi.ConvGeom.make(N, C, H, H, C, 3, 3, 1, 1, 1, 1)
    gen = torch.Generator(device=dev).manual_seed(5)
    X = torch.randn(N, C, H, H, device=dev, generator=gen)
    Wt = torch.randn(C, C, 3, 3, device=dev, generator=gen) * (2.0 / (C * 9)) ** 0.5
    Y = torch.empty(N, C, H, H, device=dev)
    capi.conv_fwd(Wt, X, Y, None, g)
    rng = np.random.default_rng(1)
    n, c, y, x = _sample_coords(rng, N, C, H, H, 3000)
    Xp = torch.nn.functional.pad(X[torch.from_numpy(np.unique(n)).to(dev)], (1, 1, 1, 1)).double().cpu().numpy()  # sampled images, padded
    slot = {v: i for i, v in enumerate(np.unique(n))}
    Wn = Wt.double().cpu().numpy()
    Yn = Y[torch.from_numpy(n).to(dev), torch.from_numpy(c).to(dev), torch.from_numpy(y).to(dev), torch.from_numpy(x).to(dev)].cpu().numpy()
    ref = np.array([(Xp[slot[n[i]], :, y[i]:y[i] + 3, x[i]:x[i] + 3] * Wn[c[i]]).sum() for i in range(len(n))])
    tol = 1e-5 * np.sqrt(C * 9) * max(np.sqrt(np.mean(ref ** 2)), 1e-6)
    assert np.all(np.abs(Yn - ref) <= np.maximum(tol, 1e-5 * np.sqrt(C * 9) * np.abs(ref))), np.abs(Yn - ref).max()

    # data gradient with dY := Y (any tensor does): dX[n,ic,y,x] = sum_{oc,fh,fw} W[oc,ic,fh,fw] * dY[n,oc,y+1-fh,x+1-fw]
    dX = torch.empty_like(X)
    capi.conv_dgrad(Wt, Y, dX, g)
    Yp = torch.nn.functional.pad(Y[torch.from_numpy(np.unique(n)).to(dev)], (1, 1, 1, 1)).double().cpu().numpy()
    dXn = dX[torch.from_numpy(n).to(dev), torch.from_numpy(c).to(dev), torch.from_numpy(y).to(dev), torch.from_numpy(x).to(dev)].cpu().numpy()
    Wflip = Wn[:, :, ::-1, ::-1]
    refd = np.array([(Yp[slot[n[i]], :, y[i]:y[i] + 3, x[i]:x[i] + 3] * Wflip[:, c[i]]).sum() for i in range(len(n))])
    told = 1e-5 * np.sqrt(C * 9) * max(np.sqrt(np.mean(refd ** 2)), 1e-6)
    assert np.all(np.abs(dXn - refd) <= np.maximum(told, 1e-5 * np.sqrt(C * 9) * np.abs(refd))), np.abs(dXn - refd).max()
    del dX

    # weight gradient through the adjoint identity, inner products accumulated in float64 on the device, image block by block
    dW = torch.zeros_like(Wt)
    capi.conv_wgrad(Y, X, dW, g)  # dY := Y
    Wq = torch.randn(C, C, 3, 3, device=dev, generator=gen)
    Z = torch.empty_like(Y)
    capi.conv_fwd(Wq, X, Z, None, g)
    lhs = float((dW.double() * Wq.double()).sum())
    rhs, scale, step = 0.0, 0.0, max(1, N // 64)
    for i in range(0, N, step):
        zb, yb = Z[i:i + step].double(), Y[i:i + step].double()
        rhs += float((zb * yb).sum())
        scale += float((zb.abs() * yb.abs()).sum())
    assert abs(lhs - rhs) <= 1e-5 * scale, (lhs, rhs, scale)


def test_gemm_operand_beyond_4_gib(dev):
    """One operand of 1.2e9 elements in each of the NN, NT and TN forms; sampled rows / columns against float64 products."""
    import torch
    from crusaderbackend_amd import capi
    big, K, small = 40000, 30000, 64
    assert big * K > 2 ** 30
    gen = torch.Generator(device=dev).manual_seed(9)
    L = torch.rand(big, K, device=dev, generator=gen) * 2 - 1   # the large operand, 4.8 GB
    S = torch.rand(K, small, device=dev, generator=gen) * 2 - 1
    rows = torch.cat([torch.arange(0, 16), torch.randint(0, big, (96,)), torch.arange(big - 16, big)]).to(dev)
    tol = 1e-5 * K ** 0.5

    def check(got, ref, what):
        scale = float(ref.abs().square().mean().sqrt())
        err = (got.double() - ref).abs()
        assert bool((err <= tol * torch.maximum(ref.abs(), torch.tensor(scale, device=dev, dtype=torch.float64))).all()), (what, float(err.max()))

    C = torch.empty(big, small, device=dev)
    capi.sgemm_nn(L, S, C, big, small, K)                       # C = L * S
    check(C[rows], L[rows].double() @ S.double(), "nn")
    St = S.t().contiguous()                                      # small x K
    C2 = torch.empty(small, big, device=dev)
    capi.sgemm_nt(St, L, C2, small, big, K)                      # C2 = St * L^T
    check(C2[:, rows], St.double() @ L[rows].double().t(), "nt")
    S2 = torch.rand(big, small, device=dev, generator=gen) * 2 - 1
    C3 = torch.empty(K, small, device=dev)
    capi.sgemm_tn(L, S2, C3, K, small, big)                      # C3 = L^T * S2, contraction over the 40000 rows
    cols = torch.cat([torch.arange(0, 16), torch.randint(0, K, (96,)), torch.arange(K - 16, K)]).to(dev)
    ref3 = torch.zeros(len(cols), small, device=dev, dtype=torch.float64)
    for i in range(0, big, 4000):
        ref3 += L[i:i + 4000][:, cols].double().t() @ S2[i:i + 4000].double()
    tol = 1e-5 * big ** 0.5
    check(C3[cols], ref3, "tn")
