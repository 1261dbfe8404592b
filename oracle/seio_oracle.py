"""numpy-facing loader of the data-preparation oracle (oracle/seio_oracle.c) and the restatement of the dataset record
layouts and the fetch order.

TEST INFRASTRUCTURE ONLY: imported by tests/ and the benchmark's cpu_baseline leg. Nothing in the product imports it.
"""
import ctypes

import numpy as np

from . import seblas_oracle as _base

_u32 = ctypes.c_uint32
_f = ctypes.POINTER(ctypes.c_float)
_b = ctypes.POINTER(ctypes.c_uint8)
_i = ctypes.POINTER(ctypes.c_int32)


def _fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f)


def bytesToFloat(raw):
    raw = np.ascontiguousarray(raw, np.uint8)
    out = np.empty(raw.shape, np.float32)
    _base.load().oracle_bytesToFloat(raw.ctypes.data_as(_b), _fp(out), _u32(raw.size))
    return out


def uniformNorm(X, desiredMin=0.0, desiredMax=1.0):
    """X (c, h, w) float image -> normalised copy."""
    X = np.array(X, np.float32, order="C")
    c = X.shape[0]
    _base.load().oracle_uniformNorm(_fp(X), _u32(c), _u32(X.size // c), ctypes.c_float(desiredMin), ctypes.c_float(desiredMax))
    return X


def distribNorm(X, desiredMean=0.0, desiredVar=1.0):
    X = np.array(X, np.float32, order="C")
    c = X.shape[0]
    _base.load().oracle_distribNorm(_fp(X), _u32(c), _u32(X.size // c), ctypes.c_float(desiredMean), ctypes.c_float(desiredVar))
    return X


def randCrop(src, hOffset, wOffset):
    """src (n, c, h, w); offsets: one int per image."""
    src = np.ascontiguousarray(src, np.float32)
    n, c, h, w = src.shape
    ho, wo = np.ascontiguousarray(hOffset, np.int32), np.ascontiguousarray(wOffset, np.int32)
    assert ho.size == n and wo.size == n
    dst = np.empty_like(src)
    _base.load().oracle_randCrop(_fp(src), _fp(dst), _u32(n), _u32(c), _u32(h), _u32(w), ho.ctypes.data_as(_i), wo.ctypes.data_as(_i))
    return dst


def mirrorW(src, flip):
    src = np.ascontiguousarray(src, np.float32)
    n, c, h, w = src.shape
    fl = np.ascontiguousarray(flip, np.uint8)
    assert fl.size == n
    dst = np.empty_like(src)
    _base.load().oracle_mirrorW(_fp(src), _fp(dst), _u32(n), _u32(c), _u32(h), _u32(w), fl.ctypes.data_as(_b))
    return dst


# ---- record layouts ----------------------------------------------------------------------------------------------------
def crdat_record(data, x_size, label_size, offset):
    """Record `offset` of a .crdat file (CrdatLoader::loadData, seio/data/DataLoader.cu:14-41): x_size byte pixels, then
    label_size float32 label values; records follow each other without a header. -> (X float32, label float32)"""
    stride = x_size + 4 * label_size
    if offset >= len(data) // stride:
        raise IndexError("crdat: record %d of %d" % (offset, len(data) // stride))
    rec = data[offset * stride:(offset + 1) * stride]
    return np.frombuffer(rec, np.uint8, x_size).astype(np.float32), np.frombuffer(rec, "<f4", label_size, x_size).copy()


def crdat_pack(images_u8, labels_f32):
    """The .crdat bytes of a set of records (what the reader above expects)."""
    out = bytearray()
    for img, lab in zip(images_u8, labels_f32):
        out += np.ascontiguousarray(img, np.uint8).tobytes() + np.ascontiguousarray(lab, "<f4").tobytes()
    return bytes(out)


def cifar_bin_record(data, index, classes=10, x_size=3072):
    """Record `index` of a CIFAR-10 binary batch file: 1 label byte, then 3072 pixel bytes (red, green, blue planes of
    32 x 32, row-major) — the dataset's published layout, which the archived training programs read with
    fetchCIFAR(dataset, path, fileIndex) (archive/Resnet56:276-282; the function itself is no longer in the tree).
    -> (X float32 of 3072 values, one-hot label of `classes` values)"""
    stride = 1 + x_size
    if index >= len(data) // stride:
        raise IndexError("cifar: record %d of %d" % (index, len(data) // stride))
    rec = data[index * stride:(index + 1) * stride]
    label = np.zeros(classes, np.float32)
    label[rec[0]] = 1.0
    return np.frombuffer(rec, np.uint8, x_size, 1).astype(np.float32), label


def fetch_order(total, epoch_size, draws):
    """The record ids DataFetcher::fetchTrain loads for a given sequence of drawn positions (seio/data/DataFetcher.cu:10-47,
    DataFetcher.cuh:36-49): the registry starts as 0..total-1 (total = EPOCH_SIZE + TEST_SIZE) with all of it remaining;
    a draw in [0, remaining) selects registry[draw], which is then moved to the end of the remaining part; when nothing
    remains, the remaining count restarts at EPOCH_SIZE."""
    registry = list(range(total))
    remained = total
    out = []
    for d in draws:
        assert 0 <= d < remained
        out.append(registry[d])
        sel = registry.pop(d)
        registry.insert(remained - 1, sel)
        remained -= 1
        if remained <= 0:
            remained = epoch_size
    return out
