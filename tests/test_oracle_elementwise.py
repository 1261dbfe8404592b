"""Pins the CPU oracle of the elementwise / reduction operators (oracle/seblas_oracle_ew.c) by checks that do not
restate its loops: numpy / torch-CPU library routines, closed forms, finite differences and hand-written cases."""
import numpy as np
import pytest

from oracle import seblas_oracle as orc


def rnd(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def test_relu_and_gradient():
    x = rnd(1, 3, 5, 7, 9)
    x.flat[::11] = 0.0  # exact zeros: relu(0) = 0 and the gradient there is 0 (strict '>')
    dy = rnd(2, *x.shape)
    assert np.array_equal(orc.relu(x), np.maximum(x, 0))
    assert np.array_equal(orc.reluGradFast(x, dy), np.where(x > 0, dy, 0).astype(np.float32))
    # derivative of the forward away from the kink
    xs = x[np.abs(x) > 1e-2]
    h = 1e-3
    fd = (orc.relu(xs + h) - orc.relu(xs - h)) / (2 * h)
    np.testing.assert_allclose(orc.reluGradFast(xs, np.ones_like(xs)), fd, atol=1e-3)


@pytest.mark.parametrize("shape,r", [((2, 3, 8, 8), 2), ((1, 4, 6, 9), 3), ((3, 2, 4, 4), 4), ((2, 2, 7, 5), 2)])
def test_maxpool_against_torch(shape, r):
    import torch
    import torch.nn.functional as F

    x = rnd(3, *shape)  # continuous values: no ties
    Y, rec = orc.maxPool(x, r, r)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = F.max_pool2d(xt, kernel_size=r, stride=r)
    assert np.array_equal(Y, yt.detach().numpy().astype(np.float32))
    N, C, IH, IW = shape
    OH, OW = IH // r, IW // r
    assert rec.shape == (N, C, OH * r, OW * r)
    # exactly one 1 per window, at the maximum
    win = rec.reshape(N, C, OH, r, OW, r)
    assert np.array_equal(win.sum(axis=(3, 5)), np.ones((N, C, OH, OW), np.float32))
    assert np.array_equal((x[:, :, :OH * r, :OW * r] * rec).reshape(N, C, OH, r, OW, r).sum(axis=(3, 5)), Y)
    dy = rnd(4, N, C, OH, OW)
    dX, rec_after = orc.maxPoolBack(dy, rec, (IH, IW), r, r)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    assert np.array_equal(dX, xt.grad.numpy().astype(np.float32))
    assert not rec_after.any()  # the pass clears the entries it used


def test_maxpool_tie_rule_and_all_negative():
    # first maximum in row-major window order wins; values below zero are still maxima (start value is -1e15)
    x = np.array([[5, 5, -3, -1],
                  [5, 5, -2, -1],
                  [0, 1, -7, -7],
                  [1, 1, -7, -7]], np.float32).reshape(1, 1, 4, 4)
    Y, rec = orc.maxPool(x, 2, 2)
    assert np.array_equal(Y.reshape(2, 2), np.array([[5, -1], [1, -7]], np.float32))
    expect = np.zeros((4, 4), np.float32)
    expect[0, 0] = expect[0, 3] = expect[2, 1] = expect[2, 2] = 1
    assert np.array_equal(rec.reshape(4, 4), expect)
    dX, _ = orc.maxPoolBack(np.array([[10, 20], [30, 40]], np.float32).reshape(1, 1, 2, 2), rec, (4, 4), 2, 2)
    g = np.zeros((4, 4), np.float32)
    g[0, 0], g[0, 3], g[2, 1], g[2, 2] = 10, 20, 30, 40
    assert np.array_equal(dX.reshape(4, 4), g)
    # a window without a recorded maximum routes the gradient to its first element
    dX0, _ = orc.maxPoolBack(np.ones((1, 1, 2, 2), np.float32), np.zeros((1, 1, 4, 4), np.float32), (4, 4), 2, 2)
    assert np.array_equal(np.argwhere(dX0.reshape(4, 4) == 1), np.array([[0, 0], [0, 2], [2, 0], [2, 2]]))


@pytest.mark.parametrize("rows,step", [(7, 10), (128, 10), (3, 1), (5, 1000), (2, 1500)])
def test_softmax_against_float64(rows, step):
    a = rnd(5, rows, step) * 4
    out = orc.softmax(a, step)
    a64 = a.astype(np.float64)
    e = np.exp(a64 - a64.max(axis=1, keepdims=True))
    ref = e / (e.sum(axis=1, keepdims=True) + 1e-10)
    np.testing.assert_allclose(out, ref, rtol=5e-6, atol=1e-12)  # float exp of arguments down to -30: |x| * 2^-24
    # shift invariance: the row maximum is subtracted before exp
    np.testing.assert_allclose(orc.softmax(a + 50.0, step), out, rtol=1e-4, atol=1e-9)
    assert np.isfinite(orc.softmax(a * 1e4, step)).all()  # no overflow for large logits


def test_cross_entropy_value_and_gradient():
    rows, classes = 16, 10
    z = rnd(6, rows, classes).astype(np.float64)
    labels = np.eye(classes, dtype=np.float32)[np.random.default_rng(7).integers(0, classes, rows)]
    y = orc.softmax(z.astype(np.float32), classes)
    ref = -(labels * np.log(y.astype(np.float64) + 1e-10)).sum()
    assert abs(orc.crossEntropyCalc(y, labels) - ref) <= 1e-5 * abs(ref)
    assert np.array_equal(orc.crossEntropyLoss(y, labels), y - labels)

    # Y - labels is the derivative of the loss with respect to the softmax input (float64 finite differences)
    def loss(zz):
        e = np.exp(zz - zz.max(axis=1, keepdims=True))
        return -(labels * np.log(e / e.sum(axis=1, keepdims=True))).sum()

    g = np.zeros_like(z)
    h = 1e-6
    for i in range(rows):
        for j in range(classes):
            zp, zm = z.copy(), z.copy()
            zp[i, j] += h
            zm[i, j] -= h
            g[i, j] = (loss(zp) - loss(zm)) / (2 * h)
    np.testing.assert_allclose(orc.crossEntropyLoss(y, labels), g, atol=2e-6)
    # a label-free element contributes nothing; a certain, correct prediction costs ~0
    assert orc.crossEntropyCalc(np.array([1.0, 0.0], np.float32), np.array([1.0, 0.0], np.float32)) == pytest.approx(0.0, abs=1e-6)


def test_tensor_arithmetic():
    a, b = rnd(8, 1001), rnd(9, 1001)
    assert np.array_equal(orc.tensorAdd(a, b), a + b)
    assert np.array_equal(orc.tensorSub(a, b), a - b)
    assert np.array_equal(orc.tensorScale(a, np.float32(0.9995)), a * np.float32(0.9995))
    assert np.array_equal(orc.constFill(a, 2.5), np.full_like(a, 2.5))


def test_momentum_closed_form_and_recurrence():
    n, lr, beta = 257, 0.01, 0.9
    x0, g = rnd(10, n), rnd(11, n)
    # constant gradient, no decay: m_k = (1 - beta^k) g, x_k = x0 - lr * sum_{j<=k} m_j
    x, m = x0.copy(), np.zeros(n, np.float32)
    for _ in range(5):
        x, gz, m = orc.momentumApply(x, g, m, lr, beta)
        assert not gz.any()  # the gradient is cleared by the step
    k = np.arange(1, 6)
    np.testing.assert_allclose(m, (1 - beta ** 5) * g.astype(np.float64), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(x, x0 - lr * (1 - beta ** k).sum() * g.astype(np.float64), rtol=1e-5, atol=1e-6)
    # with decay, against a float64 recurrence with changing gradients
    x, m = x0.copy(), rnd(12, n)
    x64, m64 = x.astype(np.float64), m.astype(np.float64)
    for s in range(4):
        gs = rnd(20 + s, n)
        x, _, m = orc.momentumApply(x, gs, m, lr, beta, decay=1 - 5e-4)
        m64 = beta * m64 + (1 - beta) * gs
        x64 = x64 * (1 - 5e-4) - lr * m64
    np.testing.assert_allclose(m, m64, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(x, x64, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape", [(8, 3, 4, 4), (64, 2, 3, 5), (2, 7, 1, 1), (130, 1, 2, 2)])
def test_batchnorm_against_torch(shape):
    import torch
    import torch.nn.functional as F

    N, feat = shape[0], int(np.prod(shape[1:]))
    x = rnd(30, *shape) * 2 + 0.5
    gamma, beta = rnd(31, feat) + 1.0, rnd(32, feat)
    dy = rnd(33, *shape)
    Y, xHat, mean, var = orc.batchNorm(x, beta, gamma)
    xt = torch.tensor(x.reshape(N, feat), dtype=torch.float64, requires_grad=True)
    gt = torch.tensor(gamma, dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(beta, dtype=torch.float64, requires_grad=True)
    yt = F.batch_norm(xt, None, None, weight=gt, bias=bt, training=True, eps=1e-8)
    np.testing.assert_allclose(Y.reshape(N, feat), yt.detach().numpy(), rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(mean, x.reshape(N, feat).astype(np.float64).mean(axis=0), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var, x.reshape(N, feat).astype(np.float64).var(axis=0), rtol=1e-4, atol=1e-7)  # biased
    # xHat: zero mean, unit (biased) variance per feature
    np.testing.assert_allclose(xHat.reshape(N, feat).mean(axis=0), 0, atol=1e-5)
    np.testing.assert_allclose(xHat.reshape(N, feat).astype(np.float64).var(axis=0), 1, rtol=1e-4)
    yt.backward(torch.tensor(dy.reshape(N, feat), dtype=torch.float64))
    dX = orc.batchNormGrad(dy, gamma, x)
    scale = np.abs(xt.grad.numpy()).max()
    np.testing.assert_allclose(dX.reshape(N, feat), xt.grad.numpy(), rtol=1e-3, atol=2e-5 * max(scale, 1))
    dG, dB = orc.batchNormParamGrads(dy, xHat)
    np.testing.assert_allclose(dG, gt.grad.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dB, bt.grad.numpy(), rtol=1e-5, atol=1e-5)


def test_batchnorm_gradient_finite_differences():
    N, feat = 5, 3
    x = rnd(34, N, feat).astype(np.float64)
    gamma, beta, dy = rnd(35, feat) + 1.0, rnd(36, feat), rnd(37, N, feat)

    def f(xx):  # scalar objective <Y, dy> in float64
        m, v = xx.mean(axis=0), xx.var(axis=0)
        return float((((xx - m) / np.sqrt(v + 1e-8) * gamma + beta) * dy).sum())

    g = np.zeros_like(x)
    h = 1e-5
    for i in range(N):
        for j in range(feat):
            xp, xm = x.copy(), x.copy()
            xp[i, j] += h
            xm[i, j] -= h
            g[i, j] = (f(xp) - f(xm)) / (2 * h)
    np.testing.assert_allclose(orc.batchNormGrad(dy, gamma, x.astype(np.float32)), g, rtol=2e-3, atol=2e-4)
