"""Seeded random sweep of convolution and GEMM shapes through the C ABI against the CPU oracle.

The hand-picked grids of the other parity tests follow the tile sizes; this one draws geometries the kernel-selection rules
were not written around (ragged channel counts, non-square images and filters, strides 1-3, padding 0-2, batched GEMMs),
weighted towards the shape families that have kernels of their own (3x3 pad 1 at stride 1 and 2, 1x1, 2x2 images).
Every draw is printed before it runs, so a failure names its case.
"""
import random

import numpy as np
import pytest

from tests import test_gpu_gemm as gemm_cases
from tests.test_gpu_conv import run_layer
from tests.util import he_normal, normal, to_dev, to_np

pytestmark = pytest.mark.gpu


def draw_conv(rng):
    kind = rng.choice(["any", "any", "direct", "direct2", "pointwise", "tiny"])
    N = rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 33])
    IC = rng.choice([1, 2, 3, 4, 7, 8, 9, 12, 16, 17, 24, 32, 40, 64, 72])
    OC = rng.choice([1, 2, 3, 5, 8, 12, 16, 17, 31, 32, 48, 64, 65, 96, 130])
    if kind == "any":
        FH, FW = rng.randint(1, 5), rng.randint(1, 5)
        sH, sW = rng.randint(1, 3), rng.randint(1, 3)
        pH, pW = rng.randint(0, 2), rng.randint(0, 2)
        IH, IW = rng.randint(max(1, FH - 2 * pH), 20), rng.randint(max(1, FW - 2 * pW), 20)
    elif kind == "direct":
        FH = FW = 3
        sH = sW = pH = pW = 1
        IW = rng.choice([4, 8, 16, 32])
        IH = rng.choice([IW, IW, 4, 8, 12, 16, 24, 5])
    elif kind == "direct2":
        FH = FW = 3
        sH = sW = 2
        pH = pW = 1
        IW = rng.choice([16, 32, 64])
        IH = rng.choice([IW, 8, 16, 32])
    elif kind == "pointwise":
        FH = FW = sH = sW = 1
        pH = pW = 0
        IW = rng.choice([8, 16, 32, 5])
        IH = rng.choice([IW, 8, 16, 4])
    else:
        FH = FW = 3
        sH = sW = pH = pW = 1
        IH = IW = 2
        IC, OC = rng.choice([4, 16, 64, 130]), rng.choice([4, 16, 64, 100])
    if N * max(IC, OC) * IH * IW > 3_000_000:
        N = max(1, N // 8)
    return (N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_conv_geometries(dev, seed):
    import torch
    from crusaderbackend_amd import capi
    rng = random.Random(seed)
    for i in range(40):
        shape = draw_conv(rng)
        bias, own_ws = rng.random() < 0.5, rng.random() < 0.5
        print("conv", seed, i, shape, bias, own_ws, flush=True)
        run_layer(dev, *shape, bias=bias, seed=100 * seed + i, ws=own_ws)
        # the one-launch backward gives the same bits as the two separate calls, whichever kernels the geometry selects
        N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW = shape
        g = capi.ConvGeom.make(*shape)
        X, W, dY = normal(i, N, IC, IH, IW), he_normal(i + 1, OC, IC, FH, FW), normal(i + 2, N, OC, g.OH, g.OW)
        Xd, Wd, dYd, dW0 = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev), normal(i + 3, OC, IC, FH, FW)
        dX1, dW1 = torch.empty_like(Xd), to_dev(dW0, dev)
        capi.conv_dgrad(Wd, dYd, dX1, g)
        capi.conv_wgrad(dYd, Xd, dW1, g)
        dX2, dW2 = torch.empty_like(Xd), to_dev(dW0, dev)
        capi.conv_bwd(Wd, dYd, Xd, dX2, dW2, g)
        assert np.array_equal(to_np(dX1), to_np(dX2)) and np.array_equal(to_np(dW1), to_np(dW2)), shape


# 3x3 / pad 1 / stride 1 on extents that none of the width-specialised kernels takes: the tiled kernels, every tile shape
# (forward / data gradient 8 x 16, 16 x 8, 4 x 32 and 8 x 8, weight gradient 4 x 16, 8 x 8 and 2 x 32, by which pads least) and
# every channel blocking of the weight gradient, ragged right and bottom edges, ragged channel chunks and blocks
OFF_GRID = [(2, 64, 56, 56, 64), (2, 128, 28, 28, 128), (3, 256, 14, 14, 96), (8, 130, 7, 7, 70), (4, 3, 24, 40, 16), (1, 20, 33, 5, 100),
            (2, 12, 5, 33, 33), (5, 8, 1, 1, 8), (3, 9, 3, 3, 5), (2, 36, 12, 12, 64), (1, 17, 60, 17, 31), (2, 4, 9, 100, 12),
            (2, 40, 20, 20, 24), (9, 33, 13, 29, 33)]


@pytest.mark.parametrize("shape", OFF_GRID, ids=lambda s: "x".join(map(str, s)))
def test_3x3_layers_off_the_width_grid(dev, shape):
    N, IC, IH, IW, OC = shape
    run_layer(dev, N, IC, IH, IW, OC, 3, 3, 1, 1, 1, 1, bias=True, seed=sum(shape))


# 3x3 / pad 1 / stride 2 off the width grid: tiled forward (odd / even window columns de-interleaved in LDS), data gradient by
# residue classes; odd and even extents, ragged tiles and channel chunks
OFF_GRID_S2 = [(2, 64, 56, 56, 128), (3, 16, 7, 7, 24), (2, 9, 15, 22, 33), (1, 128, 28, 28, 40), (4, 8, 5, 64, 8), (2, 40, 24, 24, 64)]


@pytest.mark.parametrize("shape", OFF_GRID_S2, ids=lambda s: "x".join(map(str, s)))
def test_3x3_stride_2_layers_off_the_width_grid(dev, shape):
    N, IC, IH, IW, OC = shape
    run_layer(dev, N, IC, IH, IW, OC, 3, 3, 2, 2, 1, 1, bias=True, seed=sum(shape))


# 5x5 / pad 2 / stride 1: the tiled kernel with 25 taps (forward and data gradient), any extent
FIVE_BY_FIVE = [(4, 16, 28, 28, 32), (2, 3, 32, 32, 6), (3, 20, 9, 14, 50), (2, 64, 12, 12, 64), (1, 8, 5, 3, 9), (2, 33, 17, 40, 31)]


@pytest.mark.parametrize("shape", FIVE_BY_FIVE, ids=lambda s: "x".join(map(str, s)))
def test_5x5_same_padding_layers(dev, shape):
    N, IC, IH, IW, OC = shape
    run_layer(dev, N, IC, IH, IW, OC, 5, 5, 1, 1, 2, 2, bias=True, seed=sum(shape))


# 3x3 and 5x5 at stride 1 with paddings other than "same" (0 ... F - 1): output and input extents differ, the tiled kernels' window
# origin is an argument (forward and data gradient for both filter sizes, weight gradient for 3x3)
OTHER_PADDINGS = [
    # N, IC, IH, IW, OC, F, pad
    (4, 16, 28, 28, 32, 3, 0), (2, 64, 14, 30, 64, 3, 2), (3, 9, 11, 7, 20, 3, 0), (8, 32, 32, 32, 32, 3, 2), (2, 24, 3, 3, 8, 3, 0),
    (32, 96, 30, 30, 72, 3, 0), (96, 40, 20, 20, 48, 3, 2),  # the tiled weight gradient: enough tiles and channel blocks to be chosen
    (4, 6, 14, 14, 16, 5, 0), (2, 16, 28, 28, 32, 5, 1), (2, 32, 12, 20, 24, 5, 3), (1, 8, 6, 5, 40, 5, 4), (8, 20, 24, 24, 50, 5, 0),
]


@pytest.mark.parametrize("shape", OTHER_PADDINGS, ids=lambda s: "x".join(map(str, s)))
def test_3x3_and_5x5_layers_with_other_paddings(dev, shape):
    N, IC, IH, IW, OC, F, pad = shape
    run_layer(dev, N, IC, IH, IW, OC, F, F, 1, 1, pad, pad, bias=True, seed=sum(shape))


# Data gradients at stride > 1 that go through the tiled kernel one residue class of input pixels at a time: enough workgroups
# in the launch to be chosen (128, or 24 for a single class), tap grids 1 x 1 ... 4 x 4, 8 x 8 and 8 x 16 pixel tiles, ragged
# class grids, rectangular filters and strides, classes that no tap reaches
TILED_CLASSES = [
    # N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW
    (24, 40, 28, 28, 24, 4, 4, 2, 2, 1, 1), (24, 64, 30, 30, 16, 3, 3, 2, 2, 1, 1), (24, 33, 27, 31, 12, 5, 5, 2, 2, 2, 2),
    (24, 64, 32, 32, 8, 7, 7, 2, 2, 3, 3), (48, 24, 48, 48, 20, 3, 3, 3, 3, 1, 1), (96, 64, 16, 16, 32, 2, 2, 2, 2, 0, 0),
    (8, 96, 20, 20, 32, 1, 1, 2, 2, 0, 0), (16, 70, 17, 23, 40, 1, 1, 3, 3, 0, 0), (32, 32, 20, 20, 16, 3, 3, 2, 1, 1, 1),
    (24, 48, 24, 24, 16, 3, 5, 2, 2, 1, 2), (100, 36, 15, 15, 24, 2, 2, 2, 2, 1, 1), (24, 40, 29, 29, 17, 4, 4, 2, 2, 0, 0),
    # 1024 workgroups per class: one launch per tap grid (1x1, 1x2, 2x1, 2x2 / 2x2 ... 3x3 / 3x3 ... 4x4 / a class without a grid of its own)
    (256, 64, 30, 30, 8, 3, 3, 2, 2, 1, 1), (256, 64, 28, 28, 8, 5, 5, 2, 2, 2, 2), (256, 64, 28, 28, 6, 7, 7, 2, 2, 3, 3),
    (256, 64, 45, 45, 8, 4, 4, 3, 3, 1, 1), (256, 64, 28, 28, 8, 3, 5, 2, 2, 1, 2),
    # the same layers at half the batch: all classes in one launch on the shared tap grid, absent taps skipped
    (128, 64, 30, 30, 8, 3, 3, 2, 2, 1, 1), (128, 64, 28, 28, 8, 5, 5, 2, 2, 2, 2), (128, 64, 28, 28, 8, 3, 5, 2, 2, 1, 2),
    # class grids that 4 x 32 tiles pad less than 8 x 16 ones
    (24, 16, 56, 56, 8, 3, 3, 2, 2, 1, 1), (8, 40, 55, 57, 8, 5, 5, 2, 2, 2, 2),
]


@pytest.mark.parametrize("shape", TILED_CLASSES, ids=lambda s: "x".join(map(str, s)))
def test_strided_layers_whose_data_gradient_runs_by_tiled_residue_classes(dev, shape):
    run_layer(dev, *shape, bias=True, seed=sum(shape))


@pytest.mark.parametrize("seed", [41, 42])
def test_random_3x3_layers_of_any_extent(dev, seed):
    rng = random.Random(seed)
    for i in range(30):
        N, IC, OC = rng.choice([1, 2, 3, 5]), rng.choice([1, 3, 4, 8, 9, 16, 20, 33, 64]), rng.choice([1, 5, 8, 31, 32, 33, 64, 65, 100])
        IH, IW = rng.randint(1, 40), rng.randint(1, 70)
        print("3x3", seed, i, (N, IC, IH, IW, OC), flush=True)
        run_layer(dev, N, IC, IH, IW, OC, 3, 3, 1, 1, 1, 1, bias=rng.random() < 0.5, seed=100 * seed + i)


def test_3x3_off_grid_operands_aligned_to_4_bytes_only(dev):
    """The tiled kernel makes no alignment demands (scalar window loads; the 16-byte filter loads are chosen from the filter
    tensor's own address): every operand one float past a 16-byte boundary."""
    import torch
    from crusaderbackend_amd import capi
    from oracle import seblas_oracle as orc
    from tests.util import assert_close
    N, IC, H, W_, OC = 2, 16, 14, 22, 40
    g = capi.ConvGeom.make(N, IC, H, W_, OC, 3, 3, 1, 1, 1, 1)
    X, W, dY, b = normal(1, N, IC, H, W_), he_normal(2, OC, IC, 3, 3), normal(3, N, OC, H, W_), normal(4, OC)

    def shifted(a):
        buf = torch.empty(a.size + 1, dtype=torch.float32, device=dev)
        v = buf[1:].view(*a.shape)
        v.copy_(to_dev(a, dev))
        assert v.data_ptr() % 16 == 4
        return v

    Y = shifted(np.full((N, OC, H, W_), np.nan, np.float32))
    capi.conv_fwd(shifted(W), shifted(X), Y, shifted(b), g)
    assert_close(to_np(Y), orc.conv(W, X, b, 1, 1, 1, 1, threads=8), IC * 9, "fwd, 4-byte aligned")
    dX = shifted(np.full((N, IC, H, W_), np.nan, np.float32))
    capi.conv_dgrad(shifted(W), shifted(dY), dX, g)
    assert_close(to_np(dX), orc.convDerive(W, dY, (H, W_), 1, 1, 1, 1, threads=8), OC * 9, "dgrad, 4-byte aligned")


@pytest.mark.parametrize("seed", [31, 32])
def test_random_large_pointwise_layers(dev, seed):
    """1x1 layers with enough pixels per call for the kernels that stream the activations straight into the matrix
    instructions (at least 32768 pixels, at most 64 channels on the short side) and for the pixel-contraction weight
    gradient: ragged channel counts on both sides, 8- and 16-byte pixel vectors, more than one filter staging pass."""
    rng = random.Random(seed)
    for i in range(6):
        H, W = rng.choice([(32, 32), (32, 32), (16, 32), (64, 16), (16, 16)])
        N = rng.choice([32, 40, 64, 72, 136]) * (4 if H * W == 256 else (2 if H * W == 512 else 1))
        IC, OC = rng.choice([5, 24, 50, 97, 204, 270, 300]), rng.choice([1, 12, 20, 33, 48, 50, 64])
        if N * IC * H * W > 24_000_000:
            N = max(32 * 1024 // (H * W), N // 2)
        shape = (N, IC, H, W, OC, 1, 1, 1, 1, 0, 0)
        bias = rng.random() < 0.5
        print("pointwise", seed, i, shape, bias, flush=True)
        run_layer(dev, *shape, bias=bias, seed=100 * seed + i, ws=rng.random() < 0.5)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_gemm_shapes(dev, seed):
    rng = random.Random(seed)
    for i in range(40):
        M = rng.choice([2, 3, 17, 64, 65, 100, 128, 129, 200, 256, 300, 513, 768, 1000])
        N = rng.choice([4, 5, 36, 64, 66, 128, 130, 256, 260, 512, 700, 1024])
        K = rng.choice([1, 2, 7, 16, 33, 64, 100, 256, 500, 512, 1024, 2048, 2500, 4096])
        batch = rng.choice([1, 1, 1, 2, 3])
        if M * N * K * batch > 600_000_000:
            K = max(1, K // 8)
        print("gemm", seed, i, (M, N, K, batch), flush=True)
        gemm_cases.run_nn(dev, M, N, K, batch, seed=i)
        gemm_cases.run_tn(dev, M, N, K, batch, seed=i + 1)
        gemm_cases.run_nt(dev, M, N, K, seed=i + 2)
        gemm_cases.run_nta(dev, M, N, max(1, K // 16), batch, seed=i + 3)


@pytest.mark.parametrize("seed", [7, 8])
def test_random_full_batch_layers(dev, seed):
    """Layer shapes at batches of 64 to 128, where the workgroup-count gates of the kernel choice open (resident chunks, the
    two-half forward, many-small-workgroup 1x1 tiles, streamed 1x1 layers, shortcut kernels, 4x4-image tiles): 3x3 at stride
    1 and 2 and 1x1 at stride 1 and 2 on 4- to 32-wide grids, channel counts on and off the 16-channel blocks."""
    rng = random.Random(seed)
    done = 0
    while done < 30:
        W = rng.choice([4, 8, 16, 32])
        H = rng.choice([W, W, W // 2 if W > 4 else W, 8])
        F = rng.choice([3, 3, 1])
        s = rng.choice([1, 1, 1, 2]) if (W >= 8 or F == 1) else 1
        p = 1 if F == 3 else 0
        IC = rng.choice([3, 9, 12, 16, 24, 32, 48, 64, 100, 128, 204, 256])
        OC = rng.choice([10, 12, 16, 32, 48, 64, 96, 128])
        N = rng.choice([64, 96, 128])
        if N * max(IC, OC) * H * W > 12_000_000:
            N = 64
        if N * max(IC, OC) * H * W > 12_000_000:
            IC = min(IC, 64)
        shape = (N, IC, H * s, W * s, OC, F, F, s, s, p, p)
        bias, own_ws = rng.random() < 0.5, rng.random() < 0.5
        print("full batch", seed, done, shape, bias, own_ws, flush=True)
        run_layer(dev, *shape, bias=bias, seed=1000 * seed + done, ws=own_ws)
        done += 1
