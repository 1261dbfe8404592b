"""Dataset bytes -> network input on the device (crb_images_from_bytes) against the CPU restatement of the reference's
per-image host loops. Plain conversion and min-max scaling are elementwise float operations in the reference's order and
must match bit for bit; mean / deviation scaling sums a channel in another order, so it is compared within a tolerance."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPES = [(128, 3, 32, 32), (5, 3, 7, 9), (2, 3, 224, 224), (4, 1, 28, 28), (3, 4, 16, 16), (1, 64, 4, 4), (9, 2, 1, 1)]


def _mods():
    import torch

    from crusaderbackend_amd import capi
    from oracle import seio_oracle as sio

    return torch, capi, sio


def _images(seed, n, c, h, w):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    if n > 1:
        raw[1] = raw[1] // 3 + 17          # a narrow range
        raw[1, 0] = raw[1, 0] // 4 + 60    # first channel narrower than the ones after it
    return raw


def _run(torch, capi, dev, raw, norm, p0, p1, aug=None):
    n, c, h, w = raw.shape
    src = torch.from_numpy(raw).to(dev)
    dst = torch.full((n, c, h, w), float("nan"), dtype=torch.float32, device=dev)
    table = capi.image_aug_table(torch, dev, aug) if aug is not None else None
    capi.images_from_bytes(src, dst, n, c, h, w, norm, p0, p1, aug=table)
    torch.cuda.synchronize()
    return dst.cpu().numpy()


def _reference(sio, raw, norm, p0, p1, aug=None):
    x = sio.bytesToFloat(raw)
    if norm == 1:
        x = np.stack([sio.uniformNorm(im, p0, p1) for im in x])
    elif norm == 2:
        x = np.stack([sio.distribNorm(im, p0, p1) for im in x])
    if aug is not None:
        x = sio.mirrorW(x, [1 if f & 1 else 0 for _, _, f in aug])
        shifted = sio.randCrop(x, [dh for dh, _, _ in aug], [dw for _, dw, _ in aug])
        for i, (_, _, f) in enumerate(aug):
            if f & 2:
                x[i] = shifted[i]
    return x


@pytest.mark.parametrize("shape", SHAPES)
def test_plain_conversion(dev, shape):
    torch, capi, sio = _mods()
    raw = _images(1, *shape)
    assert np.array_equal(_run(torch, capi, dev, raw, capi.NORM_NONE, 0.0, 0.0), raw.astype(np.float32))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-1.0, 1.0)])
def test_uniform_norm_bit_exact(dev, shape, lo, hi):
    torch, capi, sio = _mods()
    raw = _images(2, *shape)
    got = _run(torch, capi, dev, raw, capi.NORM_UNIFORM, lo, hi)
    ref = _reference(sio, raw, 1, lo, hi)
    assert np.array_equal(got, ref, equal_nan=True)  # (9,2,1,1): one value per channel -> 0/0 in channel 0, as on the CPU


def test_uniform_norm_constant_image(dev):
    torch, capi, sio = _mods()
    raw = np.full((2, 3, 8, 8), 77, np.uint8)
    got = _run(torch, capi, dev, raw, capi.NORM_UNIFORM, 0.0, 1.0)
    ref = _reference(sio, raw, 1, 0.0, 1.0)
    assert np.isnan(ref).all() and np.isnan(got).all()  # max == min: 0/0 everywhere, on both sides


@pytest.mark.parametrize("shape", SHAPES[:6])
@pytest.mark.parametrize("mean,sd", [(0.0, 1.0), (0.5, 0.25)])
def test_distrib_norm(dev, shape, mean, sd):
    torch, capi, sio = _mods()
    raw = _images(3, *shape)
    got = _run(torch, capi, dev, raw, capi.NORM_DISTRIBUTION, mean, sd)
    ref = _reference(sio, raw, 2, mean, sd)
    # tolerance: the reference accumulates a plane's squared deviations one by one in float, which drifts by about
    # 2^-24 * sqrt(plane size) relative; the device sums in a tree. Outputs are O(1).
    tol = max(2e-6, 2e-7 * float(np.sqrt(shape[2] * shape[3])))
    np.testing.assert_allclose(got, ref, rtol=tol, atol=tol)


@pytest.mark.parametrize("shape", [(64, 3, 32, 32), (6, 3, 7, 9), (3, 1, 28, 28)])
@pytest.mark.parametrize("norm", [0, 1])
def test_mirror_and_shift(dev, shape, norm):
    torch, capi, sio = _mods()
    raw = _images(4, *shape)
    rng = np.random.default_rng(5)
    n = shape[0]
    aug = [(int(rng.integers(-4, 5)), int(rng.integers(-4, 5)), int(rng.integers(0, 4))) for _ in range(n)]
    aug[0] = (0, 0, 0)
    aug[1] = (0, 0, 2)   # a shift by nothing still blanks row 0 and column 0
    aug[2] = (-4, 4, 3)
    got = _run(torch, capi, dev, raw, norm, 0.0, 1.0, aug)
    ref = _reference(sio, raw, norm, 0.0, 1.0, aug)
    assert np.array_equal(got, ref, equal_nan=True)
    assert not got[1, :, 0, :].any() and not got[1, :, :, 0].any()


def test_argument_errors(dev):
    torch, capi, sio = _mods()
    src = torch.zeros(65 * 4, dtype=torch.uint8, device=dev)
    dst = torch.zeros(65 * 4, dtype=torch.float32, device=dev)
    with pytest.raises(capi.CrbError):
        capi.images_from_bytes(src, dst, 1, 65, 2, 2)          # too many channels
    with pytest.raises(capi.CrbError):
        capi.images_from_bytes(src, dst, 0, 3, 2, 2)           # no images
    with pytest.raises(capi.CrbError):
        capi.images_from_bytes(src, dst, 1, 3, 2, 2, norm=7)   # unknown normalisation
    with pytest.raises(capi.CrbError):
        capi.images_from_bytes(None, dst, 1, 3, 2, 2)
