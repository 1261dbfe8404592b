"""GPU parity of the elementwise / reduction operators (through the C ABI) against the CPU oracle.

Bit-exact where the operator only selects, copies or performs individually rounded float operations (ReLU, pooling,
subtract, scale, fill, momentum); within stated tolerances where device exp/log and the summation order differ
(softmax: 1e-5 relative; cross-entropy value: 1e-5*sqrt(count) relative).
"""
import numpy as np
import pytest

from tests.util import normal, to_dev, to_np

pytestmark = pytest.mark.gpu


def _capi():
    from crusaderbackend_amd import capi
    return capi


def _oracle():
    from oracle import seblas_oracle
    return seblas_oracle


def _nan(dev, *shape):
    import torch
    return torch.full(shape, float("nan"), dtype=torch.float32, device=dev)


SIZES = [1, 3, 4, 255, 1024, 4099, 128 * 64 * 32 * 32]


@pytest.mark.parametrize("n", SIZES)
def test_relu_forward_and_gradient(dev, n):
    capi, orc = _capi(), _oracle()
    x, dy = normal(1, n), normal(2, n)
    x[::7] = 0.0
    X, dY = to_dev(x, dev), to_dev(dy, dev)
    Y, dX = _nan(dev, n), _nan(dev, n)
    capi.relu_fwd(X, Y, n)
    capi.relu_bwd(X, dY, dX, n)
    assert np.array_equal(to_np(Y), orc.relu(x))
    assert np.array_equal(to_np(dX), orc.reluGradFast(x, dy))


def test_relu_unaligned_views(dev):
    capi, orc = _capi(), _oracle()
    n = 1001
    x, dy = normal(3, n + 1), normal(4, n + 1)
    X, dY, Y = to_dev(x, dev)[1:], to_dev(dy, dev)[1:], _nan(dev, n + 1)[1:]  # 4-byte aligned only
    capi.relu_fwd(X, Y, n)
    assert np.array_equal(to_np(Y), orc.relu(x[1:]))
    capi.relu_bwd(X, dY, Y, n)
    assert np.array_equal(to_np(Y), orc.reluGradFast(x[1:], dy[1:]))


# (N, C, IH, IW, r): the VGG pooling stages (2x2 on 32/16/8/4/2) at reduced batch, the full first stage, windows
# other than 2x2, extents the window does not divide, rows whose length defeats the 16-byte path
POOL = [(4, 64, 32, 32, 2), (4, 128, 16, 16, 2), (4, 256, 8, 8, 2), (4, 512, 4, 4, 2), (4, 512, 2, 2, 2),
        (128, 64, 32, 32, 2), (2, 3, 9, 9, 3), (2, 5, 7, 5, 2), (3, 2, 6, 6, 2), (1, 1, 4, 8, 4), (2, 3, 8, 10, 2)]


@pytest.mark.parametrize("N,C,IH,IW,r", POOL)
def test_maxpool_forward_and_gradient(dev, N, C, IH, IW, r):
    capi, orc = _capi(), _oracle()
    x = normal(5, N, C, IH, IW)
    x[0, 0, :r, :r] = 1.5  # a window of ties: the first element must win
    OH, OW = IH // r, IW // r
    Yr, rec_r = orc.maxPool(x, r, r)
    X, Y, rec = to_dev(x, dev), _nan(dev, N, C, OH, OW), _nan(dev, N, C, OH * r, OW * r)
    capi.maxpool_fwd(X, Y, rec, N * C, IH, IW, r, r, r, r)
    assert np.array_equal(to_np(Y), Yr)
    assert np.array_equal(to_np(rec), rec_r)
    dy = normal(6, N, C, OH, OW)
    dXr, rec_after = orc.maxPoolBack(dy, rec_r, (IH, IW), r, r)
    dX = _nan(dev, N, C, IH, IW)
    capi.maxpool_bwd(dX, to_dev(dy, dev), rec, N * C, IH, IW, r, r, r, r)
    assert np.array_equal(to_np(dX), dXr)
    assert np.array_equal(to_np(rec), rec_after)


def test_maxpool_rejects_overlapping_windows(dev):
    capi = _capi()
    X, Y, rec = _nan(dev, 1, 1, 8, 8), _nan(dev, 1, 1, 3, 3), _nan(dev, 1, 1, 9, 9)
    with pytest.raises(capi.CrbError, match="non-overlapping"):
        capi.maxpool_fwd(X, Y, rec, 1, 8, 8, 2, 2, 3, 3)
    with pytest.raises(capi.CrbError, match="zero"):
        capi.maxpool_fwd(X, Y, rec, 0, 8, 8, 2, 2, 2, 2)


@pytest.mark.parametrize("rows,step", [(128, 10), (1, 1), (7, 64), (5, 65), (33, 1000), (3, 1025), (2, 5000), (4096, 10)])
def test_softmax(dev, rows, step):
    capi, orc = _capi(), _oracle()
    a = normal(7, rows, step) * 3
    out = _nan(dev, rows, step)
    capi.softmax(to_dev(a, dev), out, rows, step)
    ref = orc.softmax(a, step)
    got = to_np(out)
    assert np.all(np.isfinite(got))
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-12)
    np.testing.assert_allclose(got.sum(axis=1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("rows,classes", [(128, 10), (1, 1), (37, 1000), (2048, 100)])
def test_cross_entropy_value_and_gradient(dev, rows, classes):
    import torch
    capi, orc = _capi(), _oracle()
    n = rows * classes
    y = orc.softmax(normal(8, rows, classes), classes)
    labels = np.eye(classes, dtype=np.float32)[np.random.default_rng(9).integers(0, classes, rows)]
    Y, L = to_dev(y, dev), to_dev(labels, dev)
    dY = _nan(dev, rows, classes)
    capi.cross_entropy_grad(Y, L, dY, n)
    assert np.array_equal(to_np(dY), orc.crossEntropyLoss(y, labels))
    need = capi.cross_entropy_scratch_floats(n)
    scratch = torch.empty(max(need, 1), dtype=torch.float32, device=dev)
    loss = _nan(dev, 1)
    capi.cross_entropy_loss(Y, L, scratch, loss, n)
    ref = orc.crossEntropyCalc(y, labels)
    assert abs(float(to_np(loss)[0]) - ref) <= 1e-5 * np.sqrt(n) * abs(ref) + 1e-6
    again = _nan(dev, 1)
    capi.cross_entropy_loss(Y, L, scratch, again, n)
    assert to_np(again)[0] == to_np(loss)[0]  # fixed summation order
    if need > 1:
        with pytest.raises(capi.CrbError, match="scratch"):
            capi.cross_entropy_loss(Y, L, scratch[:1], loss, n)


@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 512 * 512 * 9])
def test_sub_scale_and_momentum(dev, n):
    capi, orc = _capi(), _oracle()
    a, b = normal(10, n), normal(11, n)
    A = to_dev(a, dev)
    capi.tensor_sub_inplace(A, to_dev(b, dev), n)
    assert np.array_equal(to_np(A), orc.tensorSub(a, b))
    A = to_dev(a, dev)
    capi.tensor_scale_inplace(A, 0.9995, n)
    assert np.array_equal(to_np(A), orc.tensorScale(a, np.float32(0.9995)))

    x, g, m = normal(12, n), normal(13, n), normal(14, n)
    for decay in (1.0, 1.0 - 5e-4):
        X, G, M = to_dev(x, dev), to_dev(g, dev), to_dev(m, dev)
        capi.momentum_apply(X, G, M, n, 0.01, 0.9, decay)
        xr, gr, mr = orc.momentumApply(x, g, m, 0.01, 0.9, decay)
        assert np.array_equal(to_np(M), mr)
        assert np.array_equal(to_np(X), xr)
        assert not to_np(G).any() and not gr.any()


def test_null_and_zero_arguments(dev):
    capi = _capi()
    X = _nan(dev, 8)
    with pytest.raises(capi.CrbError):
        capi.relu_fwd(X, None, 8)
    with pytest.raises(capi.CrbError):
        capi.relu_fwd(X, X, 0)
    with pytest.raises(capi.CrbError):
        capi.softmax(X, X, 0, 8)
    with pytest.raises(capi.CrbError):
        capi.momentum_apply(X, None, X, 8, 0.1, 0.9)


# (N, C, H, W): the ResNet-56 stages at its archived batch of 64, batches beyond the register cache (N > 128), a batch of
# one, feature counts that are not multiples of 64
@pytest.mark.parametrize("N,C,H,W", [(64, 16, 32, 32), (64, 32, 16, 16), (64, 64, 8, 8), (128, 8, 4, 4), (200, 3, 5, 5),
                                     (1, 4, 3, 3), (7, 1, 1, 1), (96, 5, 7, 3), (129, 2, 8, 8), (300, 2, 3, 3), (4, 32, 32, 32),
                                     (70, 32, 32, 32)])
def test_batchnorm(dev, N, C, H, W):
    capi, orc = _capi(), _oracle()
    F = C * H * W
    x = normal(20, N, C, H, W) * 1.5 + 0.3
    gamma, beta, dy = normal(21, F) + 1.0, normal(22, F), normal(23, N, C, H, W)
    Yr, xhr, mr, vr = orc.batchNorm(x, beta, gamma)
    X, G, B = to_dev(x, dev), to_dev(gamma, dev), to_dev(beta, dev)
    Y, xh, m, v = _nan(dev, N, C, H, W), _nan(dev, N, C, H, W), _nan(dev, F), _nan(dev, F)
    capi.batchnorm_fwd(X, B, G, m, v, Y, xh, N, F)
    # tolerance: sums over N samples in a different order; values are O(1)
    tol = 1e-5 * np.sqrt(max(N, 1))
    np.testing.assert_allclose(to_np(m), mr, rtol=0, atol=tol * 2)
    np.testing.assert_allclose(to_np(v), vr, rtol=tol * 4, atol=tol)
    if N > 1:  # with one sample var = 0 and xHat = 0/sqrt(1e-8) amplifies rounding of x - mean = 0 exactly: still 0
        np.testing.assert_allclose(to_np(xh), xhr, rtol=0, atol=tol * 8)
        np.testing.assert_allclose(to_np(Y), Yr, rtol=0, atol=tol * 16)
    else:
        assert not to_np(xh).any() and np.array_equal(to_np(Y).ravel(), np.tile(beta, N))
    dXr = orc.batchNormGrad(dy, gamma, x)
    dX = _nan(dev, N, C, H, W)
    dY = to_dev(dy, dev)
    capi.batchnorm_bwd(dY, G, X, dX, N, F)
    scale = max(float(np.abs(dXr).max()), 1.0)
    np.testing.assert_allclose(to_np(dX), dXr, rtol=0, atol=tol * 32 * scale if N > 1 else 1e30)
    dGr, dBr = orc.batchNormParamGrads(dy, xhr)
    dG, dB = _nan(dev, F), _nan(dev, F)
    capi.batchnorm_param_grads(dY, to_dev(xhr, dev), dG, dB, N, F)
    np.testing.assert_allclose(to_np(dB), dBr, rtol=0, atol=tol * 8)
    np.testing.assert_allclose(to_np(dG), dGr, rtol=0, atol=tol * 16)
    again, dG2, dB2 = _nan(dev, N, C, H, W), _nan(dev, F), _nan(dev, F)
    capi.batchnorm_bwd(dY, G, X, again, N, F, dGamma=dG2, dBeta=dB2)  # parameter gradients as by-products
    assert np.array_equal(to_np(again), to_np(dX))  # fixed summation order
    np.testing.assert_allclose(to_np(dB2), dBr, rtol=0, atol=tol * 8)
    if N > 1:
        np.testing.assert_allclose(to_np(dG2), dGr, rtol=0, atol=tol * 32 * max(float(np.abs(dGr).max()), 1.0) / 8)


def test_momentum_multi_matches_single(dev):
    import torch
    capi, orc = _capi(), _oracle()
    sizes = [1, 16, 144, 2304, 4099, 36864, 65]
    host = [(normal(50 + i, n), normal(60 + i, n), normal(70 + i, n)) for i, n in enumerate(sizes)]
    tens = [tuple(to_dev(a, dev) for a in h) for h in host]
    # one unaligned view in the table
    base = [to_dev(np.concatenate([[0], a]).astype(np.float32), dev) for a in host[-1]]
    tens[-1] = tuple(b[1:] for b in base)
    entries = [(X, G, M, 0.01 * (i + 1), 0.9, 1.0 - 5e-4 * (i % 2)) for i, (X, G, M) in enumerate(tens)]
    table, n, mx = capi.momentum_table(torch, dev, entries)
    capi.momentum_apply_multi(table, n, mx)
    for i, ((x, g, m), (X, G, M)) in enumerate(zip(host, tens)):
        xr, gr, mr = orc.momentumApply(x, g, m, np.float32(0.01 * (i + 1)), 0.9, np.float32(1.0 - 5e-4 * (i % 2)))
        assert np.array_equal(to_np(X), xr) and np.array_equal(to_np(M), mr) and not to_np(G).any()


@pytest.mark.parametrize("N,C,H,W", [(128, 16, 32, 32), (64, 32, 16, 16), (128, 64, 8, 8), (37, 3, 5, 7), (300, 2, 3, 3), (1, 4, 3, 3)])
def test_batchnorm_relu_fused_equals_separate_calls(dev, N, C, H, W):
    """Normalisation + the ReLU behind it in one pass each way: same bits as crb_batchnorm_* followed by / preceded by
    crb_relu_*; optional outputs are left untouched when not asked for."""
    capi = _capi()
    F = C * H * W
    x = normal(40, N, C, H, W) * 1.5 + 0.3
    gamma, beta, dy = normal(41, F) + 1.0, normal(42, F), normal(43, N, C, H, W)
    X, G, B, dY = to_dev(x, dev), to_dev(gamma, dev), to_dev(beta, dev), to_dev(dy, dev)
    # separate
    Y, xh, m, v, R = _nan(dev, N, F), _nan(dev, N, F), _nan(dev, F), _nan(dev, F), _nan(dev, N, F)
    capi.batchnorm_fwd(X, B, G, m, v, Y, xh, N, F)
    capi.relu_fwd(Y, R, N * F)
    dZ, dX, dG, dB = _nan(dev, N, F), _nan(dev, N, F), _nan(dev, F), _nan(dev, F)
    capi.relu_bwd(Y, dY, dZ, N * F)
    capi.batchnorm_bwd(dZ, G, X, dX, N, F, dGamma=dG, dBeta=dB)
    # fused, every optional output asked for
    Y2, xh2, m2, v2, R2 = _nan(dev, N, F), _nan(dev, N, F), _nan(dev, F), _nan(dev, F), _nan(dev, N, F)
    capi.batchnorm_relu_fwd(X, B, G, m2, v2, R2, N, F, Y=Y2, xHat=xh2)
    for a, b in ((Y, Y2), (xh, xh2), (m, m2), (v, v2), (R, R2)):
        assert np.array_equal(to_np(a), to_np(b), equal_nan=True)
    dX2, dG2, dB2 = _nan(dev, N, F), _nan(dev, F), _nan(dev, F)
    capi.batchnorm_relu_bwd(dY, R2, G, X, dX2, N, F, dGamma=dG2, dBeta=dB2)
    for a, b in ((dX, dX2), (dG, dG2), (dB, dB2)):
        assert np.array_equal(to_np(a), to_np(b), equal_nan=True)
    # fused, only the ReLU output
    m3, v3, R3 = _nan(dev, F), _nan(dev, F), _nan(dev, N, F)
    capi.batchnorm_relu_fwd(X, B, G, m3, v3, R3, N, F)
    assert np.array_equal(to_np(R3), to_np(R), equal_nan=True) and np.array_equal(to_np(m3), to_np(m))
    dX3 = _nan(dev, N, F)
    capi.batchnorm_relu_bwd(dY, R3, G, X, dX3, N, F)
    assert np.array_equal(to_np(dX3), to_np(dX), equal_nan=True)


@pytest.mark.parametrize("n", [1, 5, 4096, 128 * 16 * 32 * 32, 1000003])
def test_add_relu_and_relu_grad_copy2(dev, n):
    capi, orc = _capi(), _oracle()
    a, b, dy = normal(50, n), normal(51, n), normal(52, n)
    a[::7] = -b[::7]  # exact zeros in the sum: relu(0) = 0 and no gradient there
    A, Bt, dY = to_dev(a, dev), to_dev(b, dev), to_dev(dy, dev)
    R = _nan(dev, n)
    capi.tensor_add_relu(R, A, Bt, n)
    ref = orc.relu(orc.tensorAdd(a, b))
    assert np.array_equal(to_np(R), ref)
    d1, d2 = _nan(dev, n), _nan(dev, n)
    capi.tensor_relu_grad_copy2(d1, d2, R, dY, n)
    g = orc.reluGradFast(orc.tensorAdd(a, b), dy)
    assert np.array_equal(to_np(d1), g) and np.array_equal(to_np(d2), g)


@pytest.mark.parametrize("N,C,H,W", [(128, 16, 32, 32), (128, 64, 8, 8), (37, 3, 5, 7), (300, 2, 3, 3)])
def test_batchnorm_relu_with_residual_parts_equals_separate_calls(dev, N, C, H, W):
    """The forms used when a residual connection closes between the normalisation and the ReLU (forward: + addend) and
    another one opens right behind the ReLU (backward: gradient in two parts, masked copy for the shortcut)."""
    capi = _capi()
    F = C * H * W
    x, add = normal(60, N, C, H, W) * 1.5 + 0.3, normal(61, N, C, H, W)
    gamma, beta, dy, dy2 = normal(62, F) + 1.0, normal(63, F), normal(64, N, C, H, W), normal(65, N, C, H, W)
    X, A, G, B, dY, dY2 = (to_dev(v, dev) for v in (x, add, gamma, beta, dy, dy2))
    Y, xh, m, v, Z, R = _nan(dev, N, F), _nan(dev, N, F), _nan(dev, F), _nan(dev, F), _nan(dev, N, F), _nan(dev, N, F)
    capi.batchnorm_fwd(X, B, G, m, v, Y, xh, N, F)
    capi.tensor_add(Z, Y, A, N * F)
    capi.relu_fwd(Z, R, N * F)
    g, dZ, dX, dG, dB = _nan(dev, N, F), _nan(dev, N, F), _nan(dev, N, F), _nan(dev, F), _nan(dev, F)
    capi.tensor_add(g, dY, dY2, N * F)
    capi.relu_bwd(Z, g, dZ, N * F)
    capi.batchnorm_bwd(dZ, G, X, dX, N, F, dGamma=dG, dBeta=dB)
    m2, v2, R2 = _nan(dev, F), _nan(dev, F), _nan(dev, N, F)
    capi.batchnorm_relu_fwd(X, B, G, m2, v2, R2, N, F, addend=A)
    assert np.array_equal(to_np(R), to_np(R2)) and np.array_equal(to_np(m), to_np(m2)) and np.array_equal(to_np(v), to_np(v2))
    dX2, dG2, dB2, dM = _nan(dev, N, F), _nan(dev, F), _nan(dev, F), _nan(dev, N, F)
    capi.batchnorm_relu_bwd(dY, R2, G, X, dX2, N, F, dGamma=dG2, dBeta=dB2, dY2=dY2, dYmasked=dM)
    for a, b in ((dX, dX2), (dG, dG2), (dB, dB2), (dZ, dM)):
        assert np.array_equal(to_np(a), to_np(b), equal_nan=True)
    # two-part gradient without a mask copy, and through the shortcut form
    d1, d2 = _nan(dev, N * F), _nan(dev, N * F)
    capi.tensor_relu_grad_copy2(d1, d2, R, dY, N * F, dY2=dY2)
    assert np.array_equal(to_np(d1).ravel(), to_np(dZ).ravel()) and np.array_equal(to_np(d2).ravel(), to_np(dZ).ravel())


def test_prepared_and_frozen_calls_match_the_plain_wrapper(dev):
    import torch
    capi = _capi()
    n = 4099
    x = normal(11, n)
    X = to_dev(x, dev)
    want = np.maximum(x, 0)
    for make in (lambda Y: capi.prepared("crb_relu_fwd", X, Y, n, None), lambda Y: capi.frozen(lambda: capi.relu_fwd(X, Y, n))):
        Y = _nan(dev, n)
        call = make(Y)
        Y.fill_(float("nan"))
        call()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(Y), want)
