"""Pins the CPU oracle's convolution functions (no GPU).

conv forward: torch-CPU conv2d (a textbook cross-correlation, not the reference), committed fixtures made from
it, delta-filter / all-ones closed forms and a pure-Python brute force. dgrad / wgrad: adjoint identities
against the pinned forward for every stride/pad, torch autograd, and central finite differences.
"""
import itertools
import os

import numpy as np
import pytest

from oracle import seblas_oracle as orc
from tests.util import assert_close, normal

# (N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW)
GRID = [
    (1, 1, 4, 4, 1, 1, 1, 1, 1, 0, 0),
    (2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1),
    (2, 3, 9, 7, 5, 3, 3, 2, 2, 1, 1),
    (3, 5, 11, 13, 7, 2, 4, 1, 2, 0, 1),
    (2, 4, 16, 16, 6, 5, 5, 2, 1, 2, 2),
    (2, 2, 5, 6, 3, 3, 3, 3, 3, 2, 2),
    (1, 2, 8, 8, 3, 4, 4, 1, 1, 0, 0),
    (2, 6, 12, 12, 12, 1, 1, 2, 2, 0, 0),
]


def _data(shape, seed=0):
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    OH, OW = orc.out_hw(IH, IW, FH, FW, sH, sW, pH, pW)
    return normal(seed + 1, N, IC, IH, IW), normal(seed + 2, OC, IC, FH, FW), normal(seed + 3, N, OC, OH, OW), normal(seed + 4, OC)


@pytest.mark.parametrize("shape", GRID)
def test_forward_vs_torch_conv2d(shape):
    import torch
    import torch.nn.functional as F
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, _, b = _data(shape)
    ref = F.conv2d(torch.from_numpy(X).double(), torch.from_numpy(W).double(), torch.from_numpy(b).double(),
                   stride=(sH, sW), padding=(pH, pW)).numpy()
    assert_close(orc.conv(W, X, b, sH, sW, pH, pW), ref, IC * FH * FW, "oracle conv+bias")
    ref0 = F.conv2d(torch.from_numpy(X).double(), torch.from_numpy(W).double(), None, stride=(sH, sW),
                    padding=(pH, pW)).numpy()
    assert_close(orc.conv(W, X, None, sH, sW, pH, pW), ref0, IC * FH * FW, "oracle conv, bias=nullptr")


@pytest.mark.parametrize("shape", GRID)
def test_backward_vs_torch_autograd(shape):
    import torch
    import torch.nn.functional as F
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, dY, _ = _data(shape)
    Xt = torch.from_numpy(X).double().requires_grad_()
    Wt = torch.from_numpy(W).double().requires_grad_()
    F.conv2d(Xt, Wt, None, stride=(sH, sW), padding=(pH, pW)).backward(torch.from_numpy(dY).double())
    assert_close(orc.convDerive(W, dY, (IH, IW), sH, sW, pH, pW), Xt.grad.numpy(), OC * FH * FW, "oracle dgrad")
    dW0 = normal(9, OC, IC, FH, FW)
    OH, OW = dY.shape[2:]
    assert_close(orc.convError(dY, X, dW0, sH, sW, pH, pW), dW0 + Wt.grad.numpy(), N * OH * OW, "oracle wgrad")


def _brute_forward(W, X, b, sH, sW, pH, pW):
    OC, IC, FH, FW = W.shape
    N, _, IH, IW = X.shape
    OH, OW = orc.out_hw(IH, IW, FH, FW, sH, sW, pH, pW)
    Y = np.zeros((N, OC, OH, OW))
    for n, oc, oh, ow in itertools.product(range(N), range(OC), range(OH), range(OW)):
        s = 0.0
        for ic, fh, fw in itertools.product(range(IC), range(FH), range(FW)):
            ih, iw = oh * sH - pH + fh, ow * sW - pW + fw
            if 0 <= ih < IH and 0 <= iw < IW:
                s += float(W[oc, ic, fh, fw]) * float(X[n, ic, ih, iw])
        Y[n, oc, oh, ow] = s + (float(b[oc]) if b is not None else 0.0)
    return Y


@pytest.mark.parametrize("shape", [(1, 2, 5, 4, 2, 3, 2, 2, 1, 1, 0), (2, 1, 4, 4, 2, 3, 3, 1, 1, 1, 1)])
def test_forward_vs_pure_python_brute_force(shape):
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, _, b = _data(shape, seed=20)
    assert_close(orc.conv(W, X, b, sH, sW, pH, pW), _brute_forward(W, X, b, sH, sW, pH, pW), IC * FH * FW, "brute")


def test_delta_filter_is_a_shifted_copy():
    """A filter that is 1 at tap (fh,fw) of channel c copies X[:, c] shifted by (fh-pH, fw-pW), zero outside:
    exact, and a wrong pad/stride/tap index moves the copy."""
    N, IC, H, Wd = 2, 3, 6, 7
    X = normal(30, N, IC, H, Wd)
    for (fh, fw, c, pH, pW, s) in [(0, 0, 1, 1, 1, 1), (2, 1, 0, 1, 1, 1), (1, 2, 2, 0, 0, 1), (0, 2, 1, 1, 1, 2)]:
        Wt = np.zeros((1, IC, 3, 3), np.float32)
        Wt[0, c, fh, fw] = 1.0
        Y = orc.conv(Wt, X, None, s, s, pH, pW)
        OH, OW = Y.shape[2:]
        exp = np.zeros_like(Y)
        for oh in range(OH):
            for ow in range(OW):
                ih, iw = oh * s - pH + fh, ow * s - pW + fw
                if 0 <= ih < H and 0 <= iw < Wd:
                    exp[:, 0, oh, ow] = X[:, c, ih, iw]
        assert np.array_equal(Y, exp)


def test_all_ones_gives_tap_counts():
    """All-ones filter on all-ones input: each output is IC * (number of in-image taps), a closed form in pad/stride."""
    IC, H = 3, 8
    X, Wt = np.ones((1, IC, H, H), np.float32), np.ones((2, IC, 3, 3), np.float32)
    Y = orc.conv(Wt, X, None, 1, 1, 1, 1)
    cnt = np.full((H, H), 9.0)
    cnt[0, :] = cnt[-1, :] = cnt[:, 0] = cnt[:, -1] = 6.0
    cnt[0, 0] = cnt[0, -1] = cnt[-1, 0] = cnt[-1, -1] = 4.0
    assert np.array_equal(Y[0, 0], IC * cnt) and np.array_equal(Y[0, 1], IC * cnt)
    Y2 = orc.conv(Wt, X, None, 2, 2, 1, 1)  # stride 2: outputs at even input positions
    assert np.array_equal(Y2[0, 0], IC * cnt[::2, ::2])


def test_one_by_one_is_per_pixel_gemm():
    N, IC, OC, H = 2, 5, 4, 6
    X, Wt = normal(40, N, IC, H, H), normal(41, OC, IC, 1, 1)
    Y = orc.conv(Wt, X, None, 1, 1, 0, 0)
    ref = np.einsum("oi,nihw->nohw", Wt[:, :, 0, 0].astype(np.float64), X.astype(np.float64))
    assert_close(Y, ref, IC, "1x1 conv")


@pytest.mark.parametrize("shape", GRID)
def test_adjoint_identities(shape):
    """<conv(W,X), dY> = <X, convDerive(W,dY)> = <W, convError(dY,X)> pins dgrad and wgrad to the forward."""
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, dY, _ = _data(shape, seed=50)
    a = np.vdot(orc.conv(W, X, None, sH, sW, pH, pW).astype(np.float64), dY)
    b = np.vdot(orc.convDerive(W, dY, (IH, IW), sH, sW, pH, pW).astype(np.float64), X)
    c = np.vdot(orc.convError(dY, X, np.zeros_like(W), sH, sW, pH, pW).astype(np.float64), W)
    scale = np.linalg.norm(dY) * np.linalg.norm(orc.conv(W, X, None, sH, sW, pH, pW))
    assert abs(a - b) <= 1e-5 * scale and abs(a - c) <= 1e-5 * scale


def test_finite_differences_small():
    """Central differences of L = <conv(W,X), dY> on a 4x4 input reproduce dgrad and wgrad."""
    shape = (1, 2, 4, 4, 2, 3, 3, 2, 2, 1, 1)
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, dY, _ = _data(shape, seed=60)
    loss = lambda W_, X_: float(np.vdot(_brute_forward(W_, X_, None, sH, sW, pH, pW), dY.astype(np.float64)))
    eps = 1e-2
    dX = orc.convDerive(W, dY, (IH, IW), sH, sW, pH, pW)
    dW = orc.convError(dY, X, np.zeros_like(W), sH, sW, pH, pW)
    for idx in [(0, 0, 0, 0), (0, 1, 2, 3), (0, 0, 3, 1)]:
        Xp, Xm = X.astype(np.float64).copy(), X.astype(np.float64).copy()
        Xp[idx] += eps
        Xm[idx] -= eps
        assert abs((loss(W, Xp) - loss(W, Xm)) / (2 * eps) - dX[idx]) < 1e-4
    for idx in [(0, 0, 0, 0), (1, 1, 2, 1), (0, 1, 1, 2)]:
        Wp, Wm = W.astype(np.float64).copy(), W.astype(np.float64).copy()
        Wp[idx] += eps
        Wm[idx] -= eps
        assert abs((loss(Wp, X) - loss(Wm, X)) / (2 * eps) - dW[idx]) < 1e-4


def test_wgrad_accumulates_and_conv_bias():
    shape = GRID[1]
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    X, W, dY, b = _data(shape, seed=70)
    once = orc.convError(dY, X, np.zeros_like(W), sH, sW, pH, pW)
    assert np.array_equal(orc.convError(dY, X, once, sH, sW, pH, pW), 2 * once)
    Y = orc.conv(W, X, None, sH, sW, pH, pW)
    assert np.array_equal(orc.convBias(Y, b), Y + b[None, :, None, None])
    assert np.array_equal(orc.conv(W, X, np.zeros(OC, np.float32), sH, sW, pH, pW), Y)  # zero bias == nullptr


def test_committed_golden_fixtures():
    """Small input/output vectors written by tests/golden/make_conv_fixtures.py from torch-CPU float64 conv2d."""
    path = os.path.join(os.path.dirname(__file__), "golden", "conv_fixtures.npz")
    z = np.load(path)
    for i in range(int(z["count"])):
        sH, sW, pH, pW = (int(v) for v in z[f"{i}_geom"])
        X, W, b, dY = z[f"{i}_X"], z[f"{i}_W"], z[f"{i}_b"], z[f"{i}_dY"]
        IC, FH, FW = W.shape[1:]
        OC = W.shape[0]
        N, _, OH, OW = dY.shape
        assert_close(orc.conv(W, X, b, sH, sW, pH, pW), z[f"{i}_Y"], IC * FH * FW, f"fixture {i} fwd")
        assert_close(orc.convDerive(W, dY, X.shape[2:], sH, sW, pH, pW), z[f"{i}_dX"], OC * FH * FW, f"fixture {i} dgrad")
        assert_close(orc.convError(dY, X, np.zeros_like(W), sH, sW, pH, pW), z[f"{i}_dW"], N * OH * OW, f"fixture {i} wgrad")
