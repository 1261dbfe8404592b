"""The seio data pipeline of the C++ host layer (record readers, sampling without replacement, batch formation with
normalisation and augmentation on the device) against the CPU restatement. The C++ test program reads dataset files
written here and leaves what it produced; this test recomputes every batch from the files with the restatement."""
import os
import subprocess

import numpy as np
import pytest

from oracle import seio_oracle as sio

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# CRB_HOST_TEST_BIN: another build of the same program (e.g. one with host sanitizers)
BIN = os.environ.get("CRB_HOST_TEST_BIN") or os.path.join(ROOT, "tests", "cpp", "bin", "test_seblas_host")


@pytest.mark.gpu
def test_batches_formed_on_device_match_restatement(dev, tmp_path):
    assert os.path.exists(BIN), f"{BIN} missing: run `make -C crusaderbackend_amd/host`"
    d = str(tmp_path)
    rng = np.random.default_rng(8)
    n, xs, ls = 20, 3 * 8 * 8, 10
    images = rng.integers(0, 256, (n, 3, 8, 8), dtype=np.uint8)
    images[4] = images[4] // 5 + 100
    labels = np.eye(ls, dtype=np.float32)[rng.integers(0, ls, n)]
    crdat = sio.crdat_pack(images, labels)
    open(os.path.join(d, "set.crdat"), "wb").write(crdat)
    # draws valid for 24 fetches: 20 remaining at first, 16 again once none remain
    draws, remained = [], 20
    for _ in range(24):
        draws.append(int(rng.integers(0, remained)))
        remained = remained - 1 if remained > 1 else 16
    np.array(draws, np.uint32).tofile(os.path.join(d, "draws.u32"))
    # two CIFAR-style files of 6 records each
    cif = rng.integers(0, 256, (12, 3073), dtype=np.uint8)
    cif[:, 0] = rng.integers(0, 10, 12)
    cif[:6].tofile(os.path.join(d, "cifar_1.bin"))
    cif[6:].tofile(os.path.join(d, "cifar_2.bin"))

    r = subprocess.run([BIN, "data", d], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "data: OK" in r.stdout, r.stdout + r.stderr

    load = lambda name, dt=np.float32: np.fromfile(os.path.join(d, name), dt)
    # single record, the reference's float form
    x7, l7 = sio.crdat_record(crdat, xs, ls, 7)
    assert np.array_equal(load("rec7.x.f32"), x7) and np.array_equal(load("rec7.label.f32"), l7)
    assert np.array_equal(x7, images[7].ravel()) and np.array_equal(l7, labels[7])

    # the records of each batch follow from the draws
    assert np.array_equal(load("taken.u32", np.uint32), np.array(draws, np.uint32))
    order = sio.fetch_order(20, 16, draws)
    assert sorted(order[:20]) == list(range(20))
    for b in range(3):
        ids = order[8 * b:8 * b + 8]
        aug = load("batch%d.aug.i32" % b, np.int32).reshape(8, 3)
        assert ((aug[:, 2] & 2) == 2).all() and (np.abs(aug[:, :2]) <= 2).all()
        x = np.stack([sio.uniformNorm(sio.crdat_record(crdat, xs, ls, i)[0].reshape(3, 8, 8)) for i in ids])
        x = sio.mirrorW(x, (aug[:, 2] & 1).astype(np.uint8))
        x = sio.randCrop(x, aug[:, 0], aug[:, 1])
        got = load("batch%d.x.f32" % b).reshape(8, 3, 8, 8)
        assert np.array_equal(got, x, equal_nan=True), b
        assert np.array_equal(load("batch%d.label.f32" % b).reshape(8, ls), labels[ids])
    # over three batches both mirror decisions occur and the shifts vary
    allaug = np.concatenate([load("batch%d.aug.i32" % b, np.int32).reshape(8, 3) for b in range(3)])
    assert set((allaug[:, 2] & 1).tolist()) == {0, 1} and len(set(map(tuple, allaug[:, :2].tolist()))) > 3

    # no transform, no augmentation: the bytes as floats
    assert np.array_equal(load("plain.x.f32").reshape(4, 3, 8, 8), images[[3, 4, 0, 1]].astype(np.float32))
    # distribution scaling
    ref = np.stack([sio.distribNorm(images[i].astype(np.float32), 0.5, 0.25) for i in (19, 0, 6, 7)])
    np.testing.assert_allclose(load("dist.x.f32").reshape(4, 3, 8, 8), ref, rtol=2e-6, atol=2e-6)

    # CIFAR-10 binary records across two files
    cx, cl = load("cifar.x.f32").reshape(5, 3072), load("cifar.label.f32").reshape(5, 10)
    whole = cif.tobytes()
    for k, rec in enumerate((0, 5, 6, 11, 3)):
        x, lab = sio.cifar_bin_record(whole, rec)
        assert np.array_equal(cx[k], x) and np.array_equal(cl[k], lab), rec


@pytest.mark.gpu
def test_sequential_train_on_a_dataset_file(dev, tmp_path):
    """Sequential::train end to end: batches formed from a .crdat file on a second thread and stream, per-mini-batch
    forward / backward / update, test loss, log file and epoch model file."""
    assert os.path.exists(BIN), f"{BIN} missing: run `make -C crusaderbackend_amd/host`"
    d = str(tmp_path)
    rng = np.random.default_rng(21)
    n = 96 + 16
    cls = rng.integers(0, 2, n)
    images = rng.integers(0, 60, (n, 1, 8, 8), dtype=np.uint8)
    for i in range(n):  # class 0: bright left half, class 1: bright right half
        images[i, 0, :, (0 if cls[i] == 0 else 4):(4 if cls[i] == 0 else 8)] += 150
    labels = np.eye(2, dtype=np.float32)[cls]
    open(os.path.join(d, "toy.crdat"), "wb").write(sio.crdat_pack(images, labels))
    r = subprocess.run([BIN, "train", d], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "train: OK" in r.stdout, r.stdout + r.stderr
    log = open(os.path.join(d, "cache.log")).read()
    assert len([v for v in log.replace(" ", "").split(",") if v]) == 16  # 8 batches trained on: training loss and test loss each
