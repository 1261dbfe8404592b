"""GPU parity of the convolution entry points (through the C ABI) against the CPU oracle.

The reference only ever tested dgrad with stride 1 / pad 0 (validation/UnitTestTools.cu:172-300);
this grid keeps that family and adds strides, padding, forward, wgrad, bias and the benchmark configurations' layer shapes.
"""
import numpy as np
import pytest

from tests.util import assert_close, he_normal, normal, to_dev, to_np

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


def run_layer(dev, N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW, bias=False, seed=0, ws=False):
    import torch
    capi, orc = _capi(), _oracle()
    g = capi.ConvGeom.make(N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW)
    X = normal(seed + 10, N, IC, IH, IW)
    W = he_normal(seed + 20, OC, IC, FH, FW)
    dY = normal(seed + 30, N, OC, g.OH, g.OW)
    b = normal(seed + 40, OC) if bias else None
    tag = f"N{N} {IC}->{OC} {IH}x{IW} f{FH}x{FW} s{sH}{sW} p{pH}{pW}"
    dX_, dW_, dYd = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev)

    Y = _nan(dev, N, OC, g.OH, g.OW)
    capi.conv_fwd(dW_, dX_, Y, None if b is None else to_dev(b, dev), g)
    assert_close(to_np(Y), orc.conv(W, X, b, sH, sW, pH, pW, threads=8), IC * FH * FW, "conv fwd " + tag)

    dX = _nan(dev, N, IC, IH, IW)
    capi.conv_dgrad(dW_, dYd, dX, g)
    assert_close(to_np(dX), orc.convDerive(W, dY, (IH, IW), sH, sW, pH, pW, threads=8), OC * FH * FW,
                 "conv dgrad " + tag)

    dW0 = normal(seed + 50, OC, IC, FH, FW)
    dWt = to_dev(dW0, dev)
    wsbuf = None
    if ws:
        nbytes = capi.conv_wgrad_workspace_bytes(g)
        wsbuf = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=dev)
    capi.conv_wgrad(dYd, dX_, dWt, g, workspace=wsbuf)
    assert_close(to_np(dWt), orc.convError(dY, X, dW0, sH, sW, pH, pW, threads=8), N * g.OH * g.OW,
                 "conv wgrad " + tag)


# (N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW)
SMALL = [
    (1, 1, 4, 4, 1, 1, 1, 1, 1, 0, 0),
    (2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1),
    (2, 3, 9, 7, 5, 3, 3, 2, 2, 1, 1),
    (3, 5, 11, 13, 7, 2, 4, 1, 2, 0, 1),
    (2, 4, 16, 16, 6, 5, 5, 2, 1, 2, 2),
    (1, 8, 10, 10, 130, 3, 3, 1, 1, 1, 1),
    (2, 130, 6, 6, 9, 1, 1, 1, 1, 0, 0),
    (4, 6, 12, 12, 12, 1, 1, 2, 2, 0, 0),
    (2, 2, 7, 7, 3, 7, 7, 1, 1, 0, 0),
    (2, 2, 5, 6, 3, 3, 3, 3, 3, 2, 2),
]


@pytest.mark.parametrize("shape", SMALL)
def test_conv_small_grid(dev, shape):
    run_layer(dev, *shape, bias=False, seed=1)
    run_layer(dev, *shape, bias=True, seed=2, ws=True)


@pytest.mark.parametrize("feature,filt,C1,C2,N", [(8, 2, 4, 8, 2), (16, 4, 16, 3, 4), (32, 8, 2, 5, 1), (4, 1, 64, 32, 8)])
def test_conv_reference_unit_grid(dev, feature, filt, C1, C2, N):
    """Shape family of the reference's convUnitTest: square features/filters, stride 1, pad 0."""
    run_layer(dev, N, C1, feature, feature, C2, filt, filt, 1, 1, 0, 0, seed=3)


RESNET = [
    (16, 32, 16, 1),  # 16->16 @32x32
    (32, 16, 32, 1),  # 32->32 @16x16
    (64, 8, 64, 1),   # 64->64 @8x8
    (16, 32, 32, 2),  # 16->32 stride 2
    (32, 16, 64, 2),  # 32->64 stride 2
]


@pytest.mark.parametrize("IC,H,OC,s", RESNET)
def test_conv_resnet56_layers(dev, IC, H, OC, s):
    """ResNet-56 layer shapes (benchmark configuration 2) (3x3, pad 1) at batch 16; the full batch-128 shapes are covered by the
    adjoint property test below."""
    run_layer(dev, 16, IC, H, H, OC, 3, 3, s, s, 1, 1, seed=4)


@pytest.mark.parametrize("IC,H", [(24, 32), (108, 16), (330, 8)])
def test_conv_densenet_layers(dev, IC, H):
    """benchmark configuration 4 (DenseNet-BC bottleneck): 1x1 IC->48 bottleneck then 3x3 48->12, with bias, batch 8."""
    run_layer(dev, 8, IC, H, H, 48, 1, 1, 1, 1, 0, 0, bias=True, seed=5)
    run_layer(dev, 8, 48, H, H, 12, 3, 3, 1, 1, 1, 1, bias=True, seed=6)


@pytest.mark.parametrize("IC,H,OC,s", RESNET)
def test_conv_resnet56_layers_full_batch(dev, IC, H, OC, s):
    """benchmark configuration 2 at its own batch (128): forward and both gradients against the oracle, workspace from the caller."""
    run_layer(dev, 128, IC, H, H, OC, 3, 3, s, s, 1, 1, seed=14, ws=True)


@pytest.mark.parametrize("IC,H", [(24, 32), (168, 32), (108, 16), (228, 16), (150, 8), (342, 8)])
def test_conv_densenet_layers_full_batch(dev, IC, H):
    """benchmark configuration 4 at its own batch (64): first and last bottleneck of each stage, then the 3x3 48 -> 12 layer."""
    run_layer(dev, 64, IC, H, H, 48, 1, 1, 1, 1, 0, 0, seed=15)
    run_layer(dev, 64, 48, H, H, 12, 3, 3, 1, 1, 1, 1, seed=16)


@pytest.mark.parametrize("H,base", [(32, 24), (16, 108), (8, 150)])
def test_conv_densenet_every_bottleneck_width_full_batch(dev, H, base):
    """benchmark configuration 4, every one of its 48 bottleneck layers at its own batch (64) and with the bias the dense block
    gives them (seann/operands/prefabs/DenseBlock.cuh:53): IC = base + 12 i, i = 0..15, per stage."""
    for i in range(16):
        run_layer(dev, 64, base + 12 * i, H, H, 48, 1, 1, 1, 1, 0, 0, bias=True, seed=200 + i, ws=bool(i & 1))
    run_layer(dev, 64, 48, H, H, 12, 3, 3, 1, 1, 1, 1, bias=True, seed=17, ws=True)


def test_conv_vgg_stem_and_wide(dev):
    run_layer(dev, 4, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1, bias=True, seed=7)
    run_layer(dev, 2, 256, 4, 4, 512, 3, 3, 1, 1, 1, 1, bias=True, seed=8)


# image layers (at most 3 input channels, 32 wide): the weight gradient with (channel, tap) pairs on the MFMA columns;
# ragged output-channel blocks, 1-3 input channels, slices of one and of several tiles, a ragged last slice
@pytest.mark.parametrize("N,IC,H,OC", [(128, 3, 32, 16), (128, 3, 32, 64), (5, 1, 8, 5), (7, 2, 16, 20), (200, 3, 32, 33), (1, 3, 8, 130)])
def test_conv_image_layers(dev, N, IC, H, OC):
    run_layer(dev, N, IC, H, 32, OC, 3, 3, 1, 1, 1, 1, bias=True, seed=19)
    run_layer(dev, N, IC, H, 32, OC, 3, 3, 1, 1, 1, 1, bias=False, seed=20, ws=True)


@pytest.mark.parametrize("IC,H,OC,s", RESNET)
def test_conv_full_batch_adjoint(dev, IC, H, OC, s):
    """Size-independent property at the full benchmark batch (128): <conv(W,X), dY> = <X, dgrad(W,dY)> =
    <W, wgrad(dY,X)>, inner products accumulated in float64 on the device results."""
    import torch
    capi = _capi()
    N = 128
    g = capi.ConvGeom.make(N, IC, H, H, OC, 3, 3, s, s, 1, 1)
    X, W, dY = normal(10, N, IC, H, H), he_normal(20, OC, IC, 3, 3), normal(30, N, OC, g.OH, g.OW)
    Xd, Wd, dYd = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev)
    Y = _nan(dev, N, OC, g.OH, g.OW)
    dX = _nan(dev, N, IC, H, H)
    dW = torch.zeros(OC, IC, 3, 3, device=dev)
    capi.conv_fwd(Wd, Xd, Y, None, g)
    capi.conv_dgrad(Wd, dYd, dX, g)
    capi.conv_wgrad(dYd, Xd, dW, g)
    a = float(np.vdot(to_np(Y).astype(np.float64), dY.astype(np.float64)))
    b = float(np.vdot(to_np(dX).astype(np.float64), X.astype(np.float64)))
    c = float(np.vdot(to_np(dW).astype(np.float64), W.astype(np.float64)))
    scale = float(np.linalg.norm(to_np(Y).astype(np.float64)) * np.linalg.norm(dY.astype(np.float64)))
    assert abs(a - b) <= 1e-5 * scale and abs(a - c) <= 1e-5 * scale, (a, b, c, scale)


def test_conv_wgrad_accumulates_and_is_deterministic(dev):
    import torch
    capi = _capi()
    g = capi.ConvGeom.make(32, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1)
    X, dY = normal(1, 32, 16, 32, 32), normal(2, 32, 16, 32, 32)
    Xd, dYd = to_dev(X, dev), to_dev(dY, dev)
    dW = torch.zeros(16, 16, 3, 3, device=dev)
    capi.conv_wgrad(dYd, Xd, dW, g)
    once = to_np(dW).copy()
    capi.conv_wgrad(dYd, Xd, dW, g)
    np.testing.assert_allclose(to_np(dW), 2 * once, rtol=1e-6, atol=0)
    dW2 = torch.zeros(16, 16, 3, 3, device=dev)
    capi.conv_wgrad(dYd, Xd, dW2, g)
    assert np.array_equal(to_np(dW2), once), "split-K reduction must be bit-reproducible"


def test_conv_bias_entry(dev):
    capi, orc = _capi(), _oracle()
    Y0, b = normal(1, 5, 7, 6, 3), normal(2, 7)
    Y = to_dev(Y0, dev)
    capi.conv_bias(Y, to_dev(b, dev), 5, 7, 18)
    assert np.array_equal(to_np(Y), orc.convBias(Y0, b))


def test_conv_bias_null_equals_zero_bias(dev):
    import torch
    capi = _capi()
    g = capi.ConvGeom.make(2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1)
    X, W = to_dev(normal(1, 2, 3, 8, 8), dev), to_dev(he_normal(2, 4, 3, 3, 3), dev)
    Y1, Y2 = _nan(dev, 2, 4, 8, 8), _nan(dev, 2, 4, 8, 8)
    capi.conv_fwd(W, X, Y1, None, g)
    capi.conv_fwd(W, X, Y2, torch.zeros(4, device=dev), g)
    assert np.array_equal(to_np(Y1), to_np(Y2))


def test_conv_shape_errors(dev):
    import ctypes
    import torch
    capi = _capi()
    lib = capi.load()
    t = torch.zeros(4096, device=dev)
    g = capi.ConvGeom.make(1, 2, 8, 8, 2, 3, 3, 1, 1, 1, 1, OH=7, OW=8)
    st = lib.crb_conv_fwd(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, ctypes.byref(g), 0, None)
    assert st == capi.CRB_EINVAL_SHAPE and b"rows (h) relationship" in lib.crb_last_error_string()
    g = capi.ConvGeom.make(1, 2, 8, 8, 2, 3, 3, 1, 1, 1, 1, OH=8, OW=9)
    st = lib.crb_conv_dgrad(t.data_ptr(), t.data_ptr(), t.data_ptr(), ctypes.byref(g), None)
    assert st == capi.CRB_EINVAL_SHAPE and b"cols (w) relationship" in lib.crb_last_error_string()
    g = capi.ConvGeom.make(64, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1)
    need = capi.conv_wgrad_workspace_bytes(g)
    assert need > 0
    st = lib.crb_conv_wgrad(t.data_ptr(), t.data_ptr(), t.data_ptr(), ctypes.byref(g), t.data_ptr(), 16, None)
    assert st == capi.CRB_EWORKSPACE


# (N, C, H, W): the VGG stages at reduced / full batch, shapes with C*H*W not a multiple of 4, one row, many rows
@pytest.mark.parametrize("N,C,H,W", [(128, 64, 32, 32), (128, 512, 2, 2), (128, 512, 1, 1), (37, 5, 7, 9), (1, 3, 5, 5),
                                     (300, 2, 3, 3), (16, 48, 8, 8), (2, 1, 1, 1), (64, 12, 16, 16)])
def test_conv_bias_grad(dev, N, C, H, W):
    capi = _capi()
    dY0, dB0 = normal(1, N, C, H, W), normal(2, C)
    dB, dY = to_dev(dB0, dev), to_dev(dY0, dev)
    capi.conv_bias_grad(dY, dB, N, C, H * W)
    assert_close(to_np(dB), dB0 + dY0.astype(np.float64).sum(axis=(0, 2, 3)), N * H * W, "conv bias grad")
    again = to_dev(dB0, dev)
    capi.conv_bias_grad(dY, again, N, C, H * W)
    assert np.array_equal(to_np(again), to_np(dB))  # fixed summation order


def test_bias_grad_and_tensor_helpers(dev):
    import torch
    capi = _capi()
    dY0, dB0 = normal(1, 6, 5, 7, 9), normal(2, 5)
    dB = to_dev(dB0, dev)
    capi.conv_bias_grad(to_dev(dY0, dev), dB, 6, 5, 63)
    assert_close(to_np(dB), dB0 + dY0.astype(np.float64).sum(axis=(0, 2, 3)), 6 * 63, "conv bias grad")
    for count in (1, 3, 4, 1027, 65536 + 5):
        a0, b0 = normal(3, count), normal(4, count)
        a = to_dev(a0, dev)
        capi.tensor_add_inplace(a, to_dev(b0, dev), count)
        assert np.array_equal(to_np(a), a0 + b0)
        capi.tensor_fill(a, 1.5, count)
        assert np.array_equal(to_np(a), np.full(count, 1.5, np.float32))
    # unaligned views take the scalar path
    base = torch.zeros(130, device=dev)
    capi.tensor_fill(base[1:], 2.0, 129)
    assert float(base[0]) == 0.0 and bool((base[1:] == 2.0).all())


# 3x3 / stride 1 / pad 1 shapes chosen so that every configuration of the direct (LDS-staged) path is exercised,
# plus neighbours that must fall back to the implicit-GEMM engine (odd height, channel counts not divisible by 8/16).
# (N, IC, H, W, OC)
DIRECT = [
    (3, 16, 32, 32, 16), (2, 16, 32, 32, 64), (2, 64, 32, 32, 64), (2, 8, 32, 32, 32), (2, 24, 32, 32, 48),
    (2, 8, 36, 32, 16), (2, 8, 12, 32, 16),
    (3, 32, 16, 16, 32), (2, 64, 16, 16, 128), (2, 24, 16, 16, 32), (2, 8, 16, 16, 16), (2, 16, 8, 16, 48),
    (2, 16, 12, 16, 16),
    (3, 64, 8, 8, 64), (2, 128, 8, 8, 256), (2, 32, 8, 8, 128), (2, 8, 8, 8, 16), (2, 24, 8, 8, 32), (2, 8, 4, 8, 32),
    (2, 16, 30, 32, 16), (2, 12, 16, 16, 16), (2, 16, 8, 8, 24), (2, 16, 6, 8, 16),
    (4, 64, 8, 8, 64), (8, 32, 8, 8, 16), (5, 16, 16, 16, 32), (1, 16, 32, 32, 16), (6, 48, 8, 8, 32),
    # channel counts that divide neither the channel chunk nor the channel tile (zero-filled tails)
    (2, 3, 32, 32, 16), (2, 48, 32, 32, 12), (2, 5, 16, 16, 7), (4, 13, 8, 8, 19), (2, 3, 32, 32, 64), (2, 17, 16, 16, 33),
    (4, 1, 8, 8, 1), (2, 9, 32, 32, 70),
    # 33..48 output channels at width 32: 48-wide tiles, 8 rows with enough tiles for the chip, else 4 rows
    (128, 8, 32, 32, 40), (6, 20, 32, 32, 48),
    # 4x4 images (four stacked per tile; batch sizes that leave a partial stack)
    (8, 64, 4, 4, 64), (5, 20, 4, 4, 70), (3, 7, 4, 4, 5), (6, 40, 4, 4, 33), (1, 16, 4, 4, 16), (13, 96, 4, 4, 128),
    (16, 48, 4, 4, 40), (24, 17, 4, 4, 16), (12, 16, 4, 4, 20), (128, 256, 4, 4, 80),
]


@pytest.mark.parametrize("N,IC,H,W,OC", DIRECT)
def test_conv3x3_direct_configs(dev, N, IC, H, W, OC):
    run_layer(dev, N, IC, H, W, OC, 3, 3, 1, 1, 1, 1, bias=True, seed=11)


# 3x3 / pad 1 / stride 1 on 2x2 images: dense products over (channel, pixel) pairs. (N, IC, OC)
TINY2 = [(3, 5, 7), (128, 64, 48), (2, 1, 1), (7, 33, 130), (130, 20, 16), (64, 128, 96)]


@pytest.mark.parametrize("N,IC,OC", TINY2)
def test_conv3x3_on_2x2_images(dev, N, IC, OC):
    run_layer(dev, N, IC, 2, 2, OC, 3, 3, 1, 1, 1, 1, bias=True, seed=41)
    run_layer(dev, N, IC, 2, 2, OC, 3, 3, 1, 1, 1, 1, bias=False, seed=42, ws=True)


def test_conv_relu_flag(dev):
    capi, orc = _capi(), _oracle()
    for (N, IC, H, OC) in [(2, 16, 32, 16), (2, 5, 9, 7), (9, 6, 2, 5)]:  # direct, implicit-GEMM and 2x2-image paths
        g = capi.ConvGeom.make(N, IC, H, H, OC, 3, 3, 1, 1, 1, 1)
        X, W, b = normal(1, N, IC, H, H), he_normal(2, OC, IC, 3, 3), normal(3, OC)
        Y = _nan(dev, N, OC, H, H)
        capi.conv_fwd(to_dev(W, dev), to_dev(X, dev), Y, to_dev(b, dev), g, flags=capi.CRB_FLAG_RELU)
        assert_close(to_np(Y), np.maximum(orc.conv(W, X, b, 1, 1, 1, 1), 0), IC * 9, "conv+bias+relu")


# 3x3 / stride 2 / pad 1 with even input extents: direct forward (input stride 2) and direct data gradient (parity classes).
# (N, IC, IH, IW, OC); output is IH/2 x IW/2. Widths 64/32/16 hit the grid widths 32/16/8; the others fall back.
STRIDE2 = [
    (3, 16, 32, 32, 32), (2, 32, 16, 16, 64), (2, 8, 64, 64, 16), (2, 24, 32, 32, 48), (2, 5, 16, 16, 7), (2, 16, 16, 32, 20),
    (2, 3, 32, 32, 16), (4, 40, 16, 16, 33), (2, 16, 8, 16, 16), (2, 6, 24, 16, 9), (2, 4, 12, 12, 5), (2, 4, 16, 8, 5),
]


@pytest.mark.parametrize("N,IC,IH,IW,OC", STRIDE2)
def test_conv3x3_stride2_direct(dev, N, IC, IH, IW, OC):
    run_layer(dev, N, IC, IH, IW, OC, 3, 3, 2, 2, 1, 1, bias=True, seed=21)


# 1x1 / stride 1 / no padding: direct staged kernel for widths 32/16/8 with rows divisible by 8, batched GEMM forms otherwise
POINTWISE = [(3, 24, 32, 32, 48), (2, 204, 32, 32, 48), (2, 108, 16, 16, 48), (4, 330, 8, 8, 48), (2, 7, 16, 16, 5),
             (2, 64, 32, 32, 64), (2, 17, 8, 8, 33), (2, 16, 12, 16, 16), (2, 16, 8, 12, 16), (1, 40, 24, 32, 70),
             # batches large enough to pass the workgroup-count gate of the staged 1x1 kernel
             (64, 204, 32, 32, 48), (64, 24, 32, 32, 48), (64, 108, 16, 16, 48), (96, 70, 16, 16, 130), (64, 150, 8, 8, 48),
             (128, 37, 8, 8, 64), (48, 80, 32, 32, 20),
             # pixel-contraction weight gradient: ragged last slice, 49..64 output channels, one 64-pixel run per image
             (40, 50, 32, 32, 50), (3, 16, 8, 8, 64), (72, 342, 8, 8, 48),
             # streamed forward / data gradient: 16-byte pixel vectors (131072 pixels), two filter staging passes (IC > 256)
             (128, 20, 32, 32, 24), (32, 300, 32, 32, 40),
             # forward in chunks of 48 channels (contractions of 192 channels and more on 16x16 and 8x8 images)
             (64, 288, 16, 16, 48), (72, 198, 8, 8, 40)]


@pytest.mark.parametrize("N,IC,H,W,OC", POINTWISE)
def test_conv1x1_paths(dev, N, IC, H, W, OC):
    run_layer(dev, N, IC, H, W, OC, 1, 1, 1, 1, 0, 0, bias=True, seed=31)


# Both gradients in one call. Fused shapes (the five layer shapes of CIFAR residual networks, at a small and at the full
# batch), neighbours that must take the two-call route (other channel counts, widths, filter, an odd batch for the 8x8
# tile of 4 images, 1x1, 2x2 images), with and without a caller workspace.
BWD_CASES = [(8, 16, 32, 16, 3, 1, 1), (128, 16, 32, 16, 3, 1, 1), (8, 32, 16, 32, 3, 1, 1), (128, 32, 16, 32, 3, 1, 1),
             (8, 64, 8, 64, 3, 1, 1), (128, 64, 8, 64, 3, 1, 1), (8, 16, 32, 32, 3, 2, 1), (128, 16, 32, 32, 3, 2, 1),
             (8, 32, 16, 64, 3, 2, 1), (128, 32, 16, 64, 3, 2, 1),
             (6, 12, 32, 14, 3, 1, 1), (6, 24, 16, 40, 3, 1, 1), (6, 64, 8, 48, 3, 1, 1), (3, 64, 8, 64, 3, 1, 1),
             (4, 3, 32, 16, 3, 1, 1), (4, 64, 32, 64, 3, 1, 1), (4, 128, 8, 128, 3, 1, 1), (4, 8, 12, 8, 3, 1, 1),
             (4, 16, 16, 8, 5, 1, 2), (4, 24, 8, 12, 1, 1, 0), (4, 32, 2, 32, 3, 1, 1), (4, 32, 4, 32, 3, 1, 1),
             # growth-12 dense layers: both gradients in one launch at the three image sizes (and sizes off the tile grid)
             (8, 48, 32, 12, 3, 1, 1), (64, 48, 32, 12, 3, 1, 1), (8, 48, 16, 12, 3, 1, 1), (64, 48, 16, 12, 3, 1, 1),
             (8, 48, 8, 12, 3, 1, 1), (64, 48, 8, 12, 3, 1, 1), (6, 40, 8, 10, 3, 1, 1), (3, 48, 24, 12, 3, 1, 1), (5, 36, 16, 9, 3, 1, 1)]


@pytest.mark.parametrize("N,IC,H,OC,F,s,p", BWD_CASES)
@pytest.mark.parametrize("own_ws", [False, True])
def test_conv_bwd_equals_separate_calls(dev, N, IC, H, OC, F, s, p, own_ws):
    import torch
    capi, orc = _capi(), _oracle()
    g = capi.ConvGeom.make(N, IC, H, H, OC, F, F, s, s, p, p)
    X, W, dY = normal(1, N, IC, H, H), he_normal(2, OC, IC, F, F), normal(3, N, OC, g.OH, g.OW)
    dW0 = normal(4, OC, IC, F, F)
    Xd, Wd, dYd = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev)
    ws = None
    if own_ws:
        nbytes = capi.conv_wgrad_workspace_bytes(g)
        ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=dev)
    dX1, dW1 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
    capi.conv_dgrad(Wd, dYd, dX1, g)
    capi.conv_wgrad(dYd, Xd, dW1, g, workspace=ws)
    dX2, dW2 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
    capi.conv_bwd(Wd, dYd, Xd, dX2, dW2, g, workspace=ws)
    assert np.array_equal(to_np(dX1), to_np(dX2)) and np.array_equal(to_np(dW1), to_np(dW2))
    if N <= 8:  # and both are the layer's gradients
        assert_close(to_np(dX2), orc.convDerive(W, dY, (H, H), s, s, p, p, threads=8), OC * F * F, "conv bwd dX")
        assert_close(to_np(dW2), orc.convError(dY, X, dW0, s, s, p, p, threads=8), N * g.OH * g.OW, "conv bwd dW")


def test_conv_bwd_errors(dev):
    import ctypes
    import torch
    capi = _capi()
    lib = capi.load()
    t = torch.zeros(1 << 16, device=dev)
    g = capi.ConvGeom.make(64, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1)
    p = t.data_ptr()
    assert lib.crb_conv_bwd(p, p, p, p, p, ctypes.byref(g), p, 16, None) == capi.CRB_EWORKSPACE
    assert lib.crb_conv_bwd(p, p, p, None, p, ctypes.byref(g), None, 0, None) == capi.CRB_ENULL
    assert lib.crb_conv_bwd(p, p, p, p, p, ctypes.byref(g), p + 4, 1 << 17, None) == capi.CRB_EWORKSPACE  # 4-byte aligned workspace
    assert lib.crb_conv_wgrad(p, p, p, ctypes.byref(g), p + 4, 1 << 17, None) == capi.CRB_EWORKSPACE
    assert b"16-byte aligned" in lib.crb_last_error_string()
    g = capi.ConvGeom.make(1, 2, 8, 8, 2, 3, 3, 1, 1, 1, 1, OH=7, OW=8)
    assert lib.crb_conv_bwd(p, p, p, p, p, ctypes.byref(g), None, 0, None) == capi.CRB_EINVAL_SHAPE


def test_conv_bwd_sliced_then_one_sum_equals_bwd(dev):
    """Several layers' backward calls with the slice summation postponed, completed by ONE crb_sum_slices_multi launch:
    bit-identical to crb_conv_bwd layer by layer (fused shapes, a direct-kernel shape outside the fused pairs, both strides)."""
    import torch
    capi = _capi()
    specs = [(128, 16, 32, 16, 1), (128, 32, 16, 32, 1), (128, 64, 8, 64, 1), (128, 16, 32, 32, 2), (128, 32, 16, 64, 2),
             (16, 64, 32, 64, 1), (32, 128, 8, 128, 1), (8, 16, 32, 16, 1), (64, 48, 16, 12, 1), (64, 48, 32, 12, 1), (64, 48, 8, 12, 1),
             (6, 40, 8, 10, 1)]
    layers, entries = [], []
    for i, (N, IC, H, OC, s) in enumerate(specs):
        g = capi.ConvGeom.make(N, IC, H, H, OC, 3, 3, s, s, 1, 1)
        n_slices = capi.conv_bwd_slices(g)
        assert n_slices > 1, specs[i]
        X, W = to_dev(normal(10 + i, N, IC, H, H), dev), to_dev(he_normal(30 + i, OC, IC, 3, 3), dev)
        dY, dW0 = to_dev(normal(50 + i, N, OC, g.OH, g.OW), dev), normal(70 + i, OC, IC, 3, 3)
        ws = torch.empty(capi.conv_wgrad_workspace_bytes(g) // 4, dtype=torch.float32, device=dev)
        assert ws.numel() == n_slices * OC * IC * 9
        dX1, dW1 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd(W, dY, X, dX1, dW1, g)
        dX2, dW2 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd_sliced(W, dY, X, dX2, g, ws)
        layers.append((dX1, dW1, dX2, dW2, dW0))
        entries.append((ws, dW2, n_slices))
    torch.cuda.synchronize()
    for (dX1, dW1, dX2, dW2, dW0) in layers:  # before the sum: dX complete, dW untouched
        assert np.array_equal(to_np(dX1), to_np(dX2)) and np.array_equal(to_np(dW2), dW0)
    table = capi.slice_sum_table(entries)
    capi.sum_slices_multi(table)
    torch.cuda.synchronize()
    for k, (dX1, dW1, dX2, dW2, dW0) in enumerate(layers):
        assert np.array_equal(to_np(dW1), to_np(dW2)), specs[k]


def test_conv_bwd_sliced_many_items_and_errors(dev):
    import ctypes
    import torch
    capi = _capi()
    lib = capi.load()
    # more items than one launch carries (96), of mixed sizes, against a plain sum
    rng = np.random.default_rng(3)
    entries, refs = [], []
    for i in range(130):
        count, n = int(rng.choice([2304, 9216, 36864, 432, 100, 6])), int(rng.choice([2, 7, 16, 33, 64, 256]))
        sl = rng.standard_normal((n, count)).astype(np.float32)
        d0 = rng.standard_normal(count).astype(np.float32)
        ws, dst = to_dev(sl, dev), to_dev(d0, dev)
        entries.append((ws, dst, n))
        refs.append(d0 + sl.astype(np.float64).sum(axis=0))
    capi.sum_slices_multi(capi.slice_sum_table(entries))
    torch.cuda.synchronize()
    for (ws, dst, n), ref in zip(entries, refs):
        assert_close(to_np(dst), ref, n, "slice sum")
    # geometries without a sliced form
    assert capi.conv_bwd_slices(capi.ConvGeom.make(4, 8, 8, 8, 12, 1, 1, 1, 1, 0, 0)) == 0
    assert capi.conv_bwd_slices(capi.ConvGeom.make(4, 16, 12, 12, 8, 3, 3, 1, 1, 1, 1)) == 0
    t = torch.zeros(1 << 16, device=dev)
    p = t.data_ptr()
    g = capi.ConvGeom.make(4, 16, 12, 12, 8, 3, 3, 1, 1, 1, 1)
    assert lib.crb_conv_bwd_sliced(p, p, p, p, ctypes.byref(g), p, 1 << 18, None) == capi.CRB_EINVAL_SHAPE
    g = capi.ConvGeom.make(64, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1)
    assert lib.crb_conv_bwd_sliced(p, p, p, p, ctypes.byref(g), p, 64, None) == capi.CRB_EWORKSPACE
    assert lib.crb_conv_bwd_sliced(p, p, p, p, ctypes.byref(g), None, 0, None) == capi.CRB_ENULL
    bad = (capi.SliceSumItem * 1)(capi.SliceSumItem(p, None, 16, 2))
    assert lib.crb_sum_slices_multi(ctypes.cast(bad, ctypes.c_void_p), 1, None) == capi.CRB_ENULL
    assert lib.crb_sum_slices_multi(None, 0, None) == 0


@pytest.mark.parametrize("shape", [(4, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1), (4, 32, 16, 16, 64, 3, 3, 2, 2, 1, 1),
                                   (4, 24, 16, 16, 48, 1, 1, 1, 1, 0, 0), (3, 8, 2, 2, 8, 3, 3, 1, 1, 1, 1),
                                   (2, 5, 9, 7, 6, 3, 2, 2, 1, 1, 0)])
def test_conv_operands_aligned_to_4_bytes_only(dev, shape):
    """Every operand one float past a 16-byte boundary: the 16-byte-load kernels must not be chosen (or must cope), results as usual."""
    import torch
    capi, orc = _capi(), _oracle()
    N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
    g = capi.ConvGeom.make(*shape)

    def shifted(a):  # device copy whose first element sits 4 bytes past an allocation (allocations are 256-byte aligned)
        buf = torch.empty(a.size + 1, dtype=torch.float32, device=dev)
        v = buf[1:].view(*a.shape)
        v.copy_(to_dev(a, dev))
        assert v.data_ptr() % 16 == 4
        return v

    X, W, dY = normal(1, N, IC, IH, IW), he_normal(2, OC, IC, FH, FW), normal(3, N, OC, g.OH, g.OW)
    b, dW0 = normal(4, OC), normal(5, OC, IC, FH, FW)
    Xd, Wd, dYd, bd = shifted(X), shifted(W), shifted(dY), shifted(b)
    Y = shifted(np.full((N, OC, g.OH, g.OW), np.nan, np.float32))
    capi.conv_fwd(Wd, Xd, Y, bd, g)
    assert_close(to_np(Y), orc.conv(W, X, b, sH, sW, pH, pW, threads=8), IC * FH * FW, "fwd, 4-byte aligned")
    dX = shifted(np.full((N, IC, IH, IW), np.nan, np.float32))
    capi.conv_dgrad(Wd, dYd, dX, g)
    assert_close(to_np(dX), orc.convDerive(W, dY, (IH, IW), sH, sW, pH, pW, threads=8), OC * FH * FW, "dgrad, 4-byte aligned")
    dW = shifted(dW0)
    capi.conv_wgrad(dYd, Xd, dW, g)
    assert_close(to_np(dW), orc.convError(dY, X, dW0, sH, sW, pH, pW, threads=8), N * g.OH * g.OW, "wgrad, 4-byte aligned")
    dX2, dW2 = shifted(np.full((N, IC, IH, IW), np.nan, np.float32)), shifted(dW0)
    capi.conv_bwd(Wd, dYd, Xd, dX2, dW2, g)
    assert np.array_equal(to_np(dX2), to_np(dX)) and np.array_equal(to_np(dW2), to_np(dW))


SHORTCUTS = [(128, 16, 32, 32, 32), (128, 32, 16, 16, 64), (3, 4, 8, 8, 4), (2, 12, 6, 10, 7), (5, 64, 4, 4, 64), (2, 8, 16, 12, 40),
             (4, 36, 8, 8, 9), (7, 40, 2, 2, 5), (1, 4, 2, 2, 1), (33, 16, 32, 32, 32),
             (2, 8, 7, 9, 4), (2, 6, 8, 8, 4), (2, 68, 8, 8, 4)]  # the last three: odd image / channel counts outside the streaming kernels


@pytest.mark.parametrize("N,IC,H,W,OC", SHORTCUTS)
def test_conv1x1_stride2_shortcuts(dev, N, IC, H, W, OC):
    """Projection shortcuts of residual networks (1x1, stride 2, no padding), with the caller's workspace and the library's."""
    run_layer(dev, N, IC, H, W, OC, 1, 1, 2, 2, 0, 0, bias=False, seed=21)
    run_layer(dev, N, IC, H, W, OC, 1, 1, 2, 2, 0, 0, bias=True, seed=22, ws=True)


def test_shortcut_weight_gradients_join_the_postponed_sum(dev):
    """1x1 stride-2 shortcuts have a sliced form too: dX at once, dW after crb_sum_slices_multi, both as crb_conv_bwd gives them."""
    import torch
    capi = _capi()
    layers, entries = [], []
    for i, (N, IC, H, OC) in enumerate([(128, 16, 32, 32), (128, 32, 16, 64), (6, 12, 8, 20)]):
        g = capi.ConvGeom.make(N, IC, H, H, OC, 1, 1, 2, 2, 0, 0)
        n_slices = capi.conv_bwd_slices(g)
        assert n_slices > 1
        X, W = to_dev(normal(10 + i, N, IC, H, H), dev), to_dev(he_normal(30 + i, OC, IC, 1, 1), dev)
        dY, dW0 = to_dev(normal(50 + i, N, OC, g.OH, g.OW), dev), normal(70 + i, OC, IC, 1, 1)
        ws = torch.empty(capi.conv_wgrad_workspace_bytes(g) // 4, dtype=torch.float32, device=dev)
        assert ws.numel() == n_slices * OC * IC
        dX1, dW1 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd(W, dY, X, dX1, dW1, g)
        dX2, dW2 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd_sliced(W, dY, X, dX2, g, ws)
        layers.append((dX1, dW1, dX2, dW2))
        entries.append((ws, dW2, n_slices))
    capi.sum_slices_multi(capi.slice_sum_table(entries))
    torch.cuda.synchronize()
    for dX1, dW1, dX2, dW2 in layers:
        assert np.array_equal(to_np(dX1), to_np(dX2)) and np.array_equal(to_np(dW1), to_np(dW2))


def test_pointwise_weight_gradients_join_the_postponed_sum(dev):
    """1x1 stride-1 layers (dense-network bottlenecks) have a sliced form too: dX at once, dW after crb_sum_slices_multi, both
    exactly as crb_conv_bwd gives them; the growth-12 3x3 layers behind them run both gradients in one launch."""
    import torch
    capi = _capi()
    layers, entries = [], []
    for i, (N, IC, H, OC) in enumerate([(64, 24, 32, 48), (64, 204, 32, 48), (64, 108, 16, 48), (64, 150, 8, 48), (8, 40, 8, 20), (3, 330, 8, 48)]):
        g = capi.ConvGeom.make(N, IC, H, H, OC, 1, 1)
        n_slices = capi.conv_bwd_slices(g)
        assert n_slices > 1, (N, IC, H, OC)
        X, W = to_dev(normal(10 + i, N, IC, H, H), dev), to_dev(he_normal(30 + i, OC, IC, 1, 1), dev)
        dY, dW0 = to_dev(normal(50 + i, N, OC, H, H), dev), normal(70 + i, OC, IC, 1, 1)
        ws = torch.empty(capi.conv_wgrad_workspace_bytes(g) // 4, dtype=torch.float32, device=dev)
        assert ws.numel() >= n_slices * OC * IC
        dX1, dW1 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd(W, dY, X, dX1, dW1, g)
        dX2, dW2 = _nan(dev, N, IC, H, H), to_dev(dW0, dev)
        capi.conv_bwd_sliced(W, dY, X, dX2, g, ws)
        layers.append((dX1, dW1, dX2, dW2))
        entries.append((ws, dW2, n_slices))
    capi.sum_slices_multi(capi.slice_sum_table(entries))
    torch.cuda.synchronize()
    for dX1, dW1, dX2, dW2 in layers:
        assert np.array_equal(to_np(dX1), to_np(dX2)) and np.array_equal(to_np(dW1), to_np(dW2))
    with pytest.raises(capi.CrbError) as ei:  # too small a workspace is refused before anything is launched
        capi.conv_bwd_sliced(W, dY, X, dX2, g, ws[:16])
    assert ei.value.status == capi.CRB_EWORKSPACE


# 32-wide forward with 9..16 input and at most 16 output channels: the contraction in two halves (the second half of the rows
# is committed to LDS behind the first half's MFMAs), rows requested unconditionally — ragged channel counts on both sides,
# image heights that are and are not a whole number of 8-row tiles (the latter take another configuration), odd batches.
@pytest.mark.parametrize("N,IC,H,OC", [(3, 12, 32, 10), (5, 16, 32, 16), (2, 9, 8, 1), (1, 13, 16, 16), (2, 16, 24, 7), (2, 12, 12, 12)])
def test_conv_forward_two_half_contraction(dev, N, IC, H, OC):
    run_layer(dev, N, IC, H, 32, OC, 3, 3, 1, 1, 1, 1, bias=True, seed=61)
