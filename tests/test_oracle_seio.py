"""Pins the data-preparation oracle (oracle/seio_oracle.c, oracle/seio_oracle.py) by checks that do not restate its loops:
numpy library routines, closed forms and hand-written cases."""
import struct

import numpy as np
import pytest

from oracle import seio_oracle as sio


def img(seed, c=3, h=32, w=32):
    return np.random.default_rng(seed).integers(0, 256, (c, h, w), dtype=np.uint8)


def test_bytes_to_float():
    raw = img(1)
    assert np.array_equal(sio.bytesToFloat(raw), raw.astype(np.float32))


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-1.0, 1.0), (0.5, 3.0)])
def test_uniform_norm_running_extrema(lo, hi):
    raw = img(2)
    raw[0] = raw[0] // 2 + 40  # channel 0 spans less than the full byte range, so the later channels widen the extrema
    x = raw.astype(np.float64)
    mins = np.minimum.accumulate(x.reshape(3, -1).min(axis=1))
    maxs = np.maximum.accumulate(x.reshape(3, -1).max(axis=1))
    ref = (x - mins[:, None, None]) / (maxs - mins)[:, None, None] * (hi - lo) + lo
    out = sio.uniformNorm(raw.astype(np.float32), lo, hi)
    np.testing.assert_allclose(out, ref, rtol=3e-7, atol=3e-7)
    # channel 0 is scaled by its own extrema: it reaches both ends of the range exactly
    assert out[0].min() == np.float32(lo) and out[0].max() == np.float32(hi)


def test_uniform_norm_second_channel_uses_extrema_of_both():
    x = np.array([[[10, 20]], [[0, 15]]], np.float32)  # channel 0: 10..20; channels 0 and 1 together: 0..20
    out = sio.uniformNorm(x)
    assert np.array_equal(out[0], np.array([[0.0, 1.0]], np.float32))
    assert np.array_equal(out[1], np.array([[0.0, 0.75]], np.float32))  # not 0..1: scaled by 0..20


@pytest.mark.parametrize("mean,sd", [(0.0, 1.0), (0.5, 0.25)])
def test_distrib_norm(mean, sd):
    raw = img(3)
    x = raw.astype(np.float64)
    m = x.reshape(3, -1).mean(axis=1)[:, None, None]
    v = x.reshape(3, -1).var(axis=1)[:, None, None]
    ref = (x - m) * sd / np.sqrt(v + 1e-8) + mean
    out = sio.distribNorm(raw.astype(np.float32), mean, sd)
    np.testing.assert_allclose(out, ref, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(out.reshape(3, -1).astype(np.float64).mean(axis=1), mean, atol=1e-5)
    np.testing.assert_allclose(out.reshape(3, -1).astype(np.float64).std(axis=1), sd, rtol=1e-5)


def test_rand_crop_against_padded_slices():
    rng = np.random.default_rng(4)
    src = rng.standard_normal((5, 2, 6, 7)).astype(np.float32)
    ho, wo = np.array([0, 2, -2, 1, -1]), np.array([0, -3, 3, 0, 2])
    out = sio.randCrop(src, ho, wo)
    masked = src.copy()
    masked[:, :, 0, :] = 0  # row 0 and column 0 of the source are never taken ('> 0' in the reference)
    masked[:, :, :, 0] = 0
    P = 4
    padded = np.pad(masked, ((0, 0), (0, 0), (P, P), (P, P)))
    for i in range(5):
        ref = padded[i, :, P + ho[i]:P + ho[i] + 6, P + wo[i]:P + wo[i] + 7]
        assert np.array_equal(out[i], ref), i


def test_rand_crop_hand_case():
    src = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    assert np.array_equal(sio.randCrop(src, [0], [0])[0, 0], np.array([[0, 0, 0], [0, 5, 6], [0, 8, 9]], np.float32))
    assert np.array_equal(sio.randCrop(src, [1], [1])[0, 0], np.array([[5, 6, 0], [8, 9, 0], [0, 0, 0]], np.float32))
    assert np.array_equal(sio.randCrop(src, [-1], [0])[0, 0], np.array([[0, 0, 0], [0, 0, 0], [0, 5, 6]], np.float32))


def test_mirror():
    src = np.random.default_rng(5).standard_normal((4, 3, 5, 6)).astype(np.float32)
    flip = np.array([1, 0, 1, 0], np.uint8)
    out = sio.mirrorW(src, flip)
    assert np.array_equal(out[0], src[0, :, :, ::-1]) and np.array_equal(out[2], src[2, :, :, ::-1])
    assert np.array_equal(out[1], src[1]) and np.array_equal(out[3], src[3])


def test_crdat_record_layout():
    # two records of 4 pixels and 2 label values, written byte by byte
    data = bytes([1, 2, 3, 250]) + struct.pack("<2f", 0.0, 1.0) + bytes([9, 8, 7, 6]) + struct.pack("<2f", 1.0, 0.0)
    x, lab = sio.crdat_record(data, 4, 2, 1)
    assert np.array_equal(x, np.array([9, 8, 7, 6], np.float32)) and np.array_equal(lab, np.array([1, 0], np.float32))
    x, lab = sio.crdat_record(data, 4, 2, 0)
    assert np.array_equal(x, np.array([1, 2, 3, 250], np.float32)) and np.array_equal(lab, np.array([0, 1], np.float32))
    with pytest.raises(IndexError):
        sio.crdat_record(data, 4, 2, 2)
    assert sio.crdat_pack([[1, 2, 3, 250], [9, 8, 7, 6]], [[0, 1], [1, 0]]) == data


def test_cifar_record_layout():
    rec0 = bytes([3]) + bytes(range(256)) * 12
    rec1 = bytes([9]) + bytes([7]) * 3072
    x, lab = sio.cifar_bin_record(rec0 + rec1, 0)
    assert x.shape == (3072,) and x[0] == 0 and x[255] == 255 and x[256] == 0 and lab.argmax() == 3 and lab.sum() == 1
    x, lab = sio.cifar_bin_record(rec0 + rec1, 1)
    assert (x == 7).all() and lab.argmax() == 9
    with pytest.raises(IndexError):
        sio.cifar_bin_record(rec0 + rec1, 2)


def test_fetch_order_is_sampling_without_replacement():
    rng = np.random.default_rng(6)
    total, epoch = 12, 9
    draws, remained = [], total
    for _ in range(total + 2 * epoch):
        draws.append(int(rng.integers(0, remained)))
        remained = remained - 1 if remained > 1 else epoch
    order = sio.fetch_order(total, epoch, draws)
    assert sorted(order[:total]) == list(range(total))  # the first pass visits every record once
    # later passes visit `epoch` distinct records each
    assert len(set(order[total:total + epoch])) == epoch and len(set(order[total + epoch:])) == epoch
    # hand case: registry 0 1 2 3, draws 1, 1, 0, 0 -> 1, 2, 0, 3
    assert sio.fetch_order(4, 4, [1, 1, 0, 0]) == [1, 2, 0, 3]
