"""Model files (.crseq): the format restatement (oracle/crseq_oracle.py) is pinned against a file laid out by hand from
the reference's format description, and the C++ codec of the host layer is checked against the restatement — on the CPU
through its device-free inspector, on the GPU through files written, read and re-written by the C++ test program.

The reference ships no model file, so there is no fixture of its own to compare with; the hand-laid file below follows
seio/modelcache/codec.cuh:18-38 and the encodeInfo / encodeNetParams bodies of each operand word by word.
"""
import ctypes
import os
import struct
import subprocess

import numpy as np
import pytest

from oracle import crseq_oracle as crseq

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# CRB_HOST_TEST_BIN: another build of the same program (e.g. one with host sanitizers)
BIN = os.environ.get("CRB_HOST_TEST_BIN") or os.path.join(ROOT, "tests", "cpp", "bin", "test_seblas_host")
HOST_LIB = os.path.join(ROOT, "crusaderbackend_amd", "lib", "libseblas_host.so")


def rnd(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def tiny_network():
    """input (2,1,2,2): conv 1->2 1x1 with bias, relu, [shortcut 7: batchnorm | branch conv 2->2 1x1], pool 2, linear 3, softmax"""
    return [
        {"type": "conv2d", "W": np.array([0.5, -1.0], np.float32).reshape(2, 1, 1, 1), "stride": (1, 1), "pad": (0, 0),
         "b": np.array([0.25, 2.0], np.float32)},
        {"type": "relu"},
        {"type": "shortcut_beg", "uuid": 7},
        {"type": "batchnorm", "beta": np.arange(8, dtype=np.float32).reshape(2, 2, 2) * 0.125,
         "gamma": 1.0 + np.arange(8, dtype=np.float32).reshape(2, 2, 2)},
        {"type": "shortcut_end", "uuid": 7, "branch": [
            {"type": "conv2d", "W": np.array([1.5, 2.5, 3.5, 4.5], np.float32).reshape(2, 2, 1, 1), "stride": (1, 1), "pad": (0, 0),
             "b": None}]},
        {"type": "maxpool2d", "stride": (2, 2), "range": (2, 2)},
        {"type": "linear", "out": 3, "W": np.array([[1, 2], [3, 4], [5, 6]], np.float32), "b": np.array([-1, -2, -3], np.float32)},
        {"type": "softmax"},
    ]


# The same network, word by word. Integers are uint32, the rest float32, little-endian.
TINY_WORDS = [
    0x7921AEDF, 8, 5,                                                  # magic, operand count, epoch
    0x0002, 0xA002, 0xF002, 0x0003, 0xF003, 0xB003, 0x0001, 0x0005,    # type ids
    2, 1, 1, 1, 1, 1, 0, 0, 1,                                         # conv: filter n,c,h,w  strides  pads  has-bias
    7, 0,                                                              # opening endpoint: uuid, 0 branch operands
    7, 1, 0x0002, 2, 2, 1, 1, 1, 1, 0, 0, 0,                           # closing endpoint: uuid, count, branch ids, branch infos
    2, 2, 2, 2,                                                        # pool: strides, ranges
    3,                                                                 # linear: outputs
]
TINY_FLOATS = [
    0.5, -1.0, 0.25, 2.0,                                              # conv filter, conv bias
    0.0, 0.125, 0.25, 0.375, 0.5, 0.625, 0.75, 0.875,                  # batch-norm beta ...
    1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0,                            # ... then gamma
    1.5, 2.5, 3.5, 4.5,                                                # branch conv filter (no bias)
    1.0, 2.0, 3.0, 4.0, 5.0, 6.0, -1.0, -2.0, -3.0,                    # linear weights (OUT x IN), biases
]


def tiny_bytes():
    return struct.pack("<%dI" % len(TINY_WORDS), *TINY_WORDS) + struct.pack("<%df" % len(TINY_FLOATS), *TINY_FLOATS)


def same_network(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x["type"] == y["type"]
        for k in set(x) | set(y):
            if k == "branch":
                same_network(x.get(k, []), y.get(k, []))
            elif isinstance(x.get(k), np.ndarray) or isinstance(y.get(k), np.ndarray):
                assert np.array_equal(x[k], y[k]) and x[k].shape == y[k].shape, k
            elif k == "out" or k == "uuid" or k == "stride" or k == "pad" or k == "range" or k == "b":
                assert (x.get(k) is None and y.get(k) is None) or tuple(np.atleast_1d(x[k])) == tuple(np.atleast_1d(y[k])), k


# ---- the restatement against the hand-laid file ------------------------------------------------------------------------
def test_header_bytes_are_little_endian_words():
    assert tiny_bytes()[:12] == bytes.fromhex("dfae2179" "08000000" "05000000")
    assert crseq.encode([], epoch=3) == bytes.fromhex("dfae2179" "00000000" "03000000")


def test_encode_matches_hand_laid_file():
    assert crseq.encode(tiny_network(), epoch=5) == tiny_bytes()


def test_decode_reads_hand_laid_file():
    epoch, ops, out = crseq.decode(tiny_bytes(), (2, 1, 2, 2))
    assert epoch == 5 and out == (2, 1, 3, 1)
    same_network(ops, tiny_network())


def test_record_sizes_add_up():
    net = tiny_network()
    data = crseq.encode(net)
    infos = sum(crseq.info_size(op) for op in net)
    params = sum(len(crseq.encode_params(op)) for op in net)
    assert infos == 36 + 8 + (8 + 4 + 36) + 16 + 4
    assert params == 4 * len(TINY_FLOATS)
    assert len(data) == 12 + 4 * len(net) + infos + params


def random_network(seed, n=2, c=3, hw=8):
    """conv-bn-relu-pool, an identity block, a strided block with a two-operand projection branch, two dense layers."""
    k = iter(range(seed * 100, seed * 100 + 100))
    conv = lambda oc, ic, f, s, p, bias: {"type": "conv2d", "W": rnd(next(k), oc, ic, f, f) * 0.3, "stride": (s, s), "pad": (p, p),
                                          "b": rnd(next(k), oc) if bias else None}
    bn = lambda ch, h: {"type": "batchnorm", "beta": rnd(next(k), ch, h, h) * 0.2, "gamma": 1 + rnd(next(k), ch, h, h) * 0.2}
    h = hw // 2
    return [
        conv(8, c, 3, 1, 1, True), bn(8, hw), {"type": "relu"}, {"type": "maxpool2d", "stride": (2, 2), "range": (2, 2)},
        {"type": "shortcut_beg", "uuid": 1}, conv(8, 8, 3, 1, 1, False), bn(8, h), {"type": "shortcut_end", "uuid": 1, "branch": []},
        {"type": "relu"},
        {"type": "shortcut_beg", "uuid": 2}, conv(16, 8, 3, 2, 1, True),
        {"type": "shortcut_end", "uuid": 2, "branch": [conv(16, 8, 1, 2, 0, False), bn(16, h // 2)]},
        {"type": "relu"},
        {"type": "linear", "out": 12, "W": rnd(next(k), 12, 16 * (h // 2) ** 2) * 0.1, "b": rnd(next(k), 12)},
        {"type": "relu"},
        {"type": "linear", "out": 10, "W": rnd(next(k), 10, 12) * 0.3, "b": rnd(next(k), 10)},
        {"type": "softmax"},
    ]


@pytest.mark.parametrize("seed", [1, 2])
def test_round_trip_with_projection_branch(seed):
    net = random_network(seed)
    data = crseq.encode(net, epoch=40 + seed)
    epoch, ops, out = crseq.decode(data, (2, 3, 8, 8))
    assert epoch == 40 + seed and out == (2, 1, 10, 1)
    same_network(ops, net)
    assert crseq.encode(ops, epoch) == data


def test_cudnn_convolution_id_reads_as_conv2d():
    net = tiny_network()
    net[0]["cudnn"] = True
    data = crseq.encode(net)
    assert struct.unpack_from("<I", data, 12)[0] == 0xD002
    _, ops, _ = crseq.decode(data, (2, 1, 2, 2))
    assert ops[0]["type"] == "conv2d" and ops[0]["cudnn"] and np.array_equal(ops[0]["W"], net[0]["W"])


def test_malformed_files_are_rejected():
    good = tiny_bytes()
    with pytest.raises(ValueError, match="magic"):
        crseq.decode(b"\x00" + good[1:], (2, 1, 2, 2))
    with pytest.raises(ValueError, match="ends inside"):
        crseq.decode(good[:-4], (2, 1, 2, 2))
    with pytest.raises(ValueError, match="after the last"):
        crseq.decode(good + b"\x00" * 4, (2, 1, 2, 2))
    bad_id = bytearray(good)
    struct.pack_into("<I", bad_id, 12, 0xE001)  # a dense block: no operand for it here
    with pytest.raises(ValueError, match="not handled"):
        crseq.decode(bytes(bad_id), (2, 1, 2, 2))
    with pytest.raises(ValueError):  # another input shape: the dense layer's weights no longer fit the file
        crseq.decode(good, (2, 1, 4, 4))


# ---- the C++ codec, device-free part -----------------------------------------------------------------------------------
def _inspect(path):
    assert os.path.exists(HOST_LIB), f"{HOST_LIB} missing: run `make -C crusaderbackend_amd/host`"
    lib = ctypes.CDLL(HOST_LIB)
    lib.seio_inspect_sequence.restype = ctypes.c_int
    lib.seio_inspect_sequence.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_uint]
    buf = ctypes.create_string_buffer(1 << 16)
    rc = lib.seio_inspect_sequence(path.encode(), buf, len(buf))
    return rc, buf.value.decode()


def test_cpp_inspector_reads_restatement_file(tmp_path):
    path = str(tmp_path / "tiny.crseq")
    open(path, "wb").write(tiny_bytes())
    rc, text = _inspect(path)
    assert rc == len(text) and rc > 0
    assert text.splitlines() == [
        "operands=8 epoch=5 params_at=%d param_bytes=%d" % (12 + 4 * 8 + 112, 4 * len(TINY_FLOATS)),
        "conv2d filter=2,1,1,1 stride=1,1 pad=0,0 bias=1",
        "relu",
        "shortcut_beg uuid=7 branch=0",
        "batchnorm",
        "shortcut_end uuid=7 branch=1",
        "  conv2d filter=2,2,1,1 stride=1,1 pad=0,0 bias=0",
        "maxpool2d stride=2,2 range=2,2",
        "linear out=3",
        "softmax",
    ]


def test_cpp_inspector_rejects_malformed_files(tmp_path):
    good = tiny_bytes()
    cases = {"badmagic": b"\x00" + good[1:], "short": good[:40], "unknown": good[:12] + struct.pack("<I", 0xE001) + good[16:]}
    for name, data in cases.items():
        path = str(tmp_path / (name + ".crseq"))
        open(path, "wb").write(data)
        rc, text = _inspect(path)
        assert rc == -1 and text.startswith("crseq:"), (name, text)
    rc, text = _inspect(str(tmp_path / "missing.crseq"))
    assert rc == -1 and "cannot open" in text


# ---- the C++ codec on the device ------------------------------------------------------------------------------------------
def _forward(ops, x):
    """The network on the CPU with the operator restatements (checker for the values the loaded network computes)."""
    from oracle import seblas_oracle as orc

    opened = {}
    for op in ops:
        t = op["type"]
        if t == "conv2d":
            x = orc.conv(op["W"], x, op.get("b"), op["stride"][0], op["stride"][1], op["pad"][0], op["pad"][1])
        elif t == "batchnorm":
            x = orc.batchNorm(x, op["beta"].ravel(), op["gamma"].ravel())[0]
        elif t == "relu":
            x = orc.relu(x)
        elif t == "maxpool2d":
            x = orc.maxPool(x, op["range"][0], op["range"][1])[0]
        elif t == "linear":
            x = orc.linear(x.reshape(x.shape[0], -1), op["W"], op["b"]).reshape(x.shape[0], 1, -1, 1)
        elif t == "softmax":
            x = orc.softmax(x.reshape(x.shape[0], -1), x[0].size).reshape(x.shape)
        elif t == "shortcut_beg":
            opened[op["uuid"]] = x
        elif t == "shortcut_end":
            x = x + (_forward(op["branch"], opened[op["uuid"]]) if op["branch"] else opened[op["uuid"]])
    return x


@pytest.mark.gpu
def test_cpp_codec_files_match_restatement(dev, tmp_path):
    assert os.path.exists(BIN), f"{BIN} missing: run `make -C crusaderbackend_amd/host`"
    d = str(tmp_path)
    net = random_network(3, n=4)
    data = crseq.encode(net, epoch=9)
    open(os.path.join(d, "b.crseq"), "wb").write(data)
    x = rnd(55, 4, 3, 8, 8)
    x.tofile(os.path.join(d, "b.x.f32"))
    np.array([4, 3, 8, 8], np.float32).tofile(os.path.join(d, "b.shape.f32"))

    r = subprocess.run([BIN, "codec", d], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "codec: OK" in r.stdout, r.stdout + r.stderr

    # a file written by the C++ codec: the restatement reads it, finds the parameters the program dumped, in the
    # program's parameter order, and writes the very same bytes again
    for name, epoch_expected in (("a", 17), ("a2", 18)):
        a = open(os.path.join(d, name + ".crseq"), "rb").read()
        epoch, ops, out = crseq.decode(a, (4, 3, 8, 8))
        assert epoch == epoch_expected and out == (4, 1, 10, 1)
        assert [op["type"] for op in ops] == ["conv2d", "batchnorm", "relu", "maxpool2d", "shortcut_beg", "conv2d", "batchnorm",
                                              "shortcut_end", "relu", "shortcut_beg", "conv2d", "shortcut_end", "relu", "linear",
                                              "softmax"]
        assert [b["type"] for b in ops[11]["branch"]] == ["conv2d", "batchnorm"]
        assert crseq.encode(ops, epoch) == a
        flat = []

        def collect(lst):
            for op in lst:
                if op["type"] == "conv2d":
                    flat.extend([op["W"].ravel()] + ([] if op["b"] is None else [op["b"].ravel()]))
                elif op["type"] == "batchnorm":
                    flat.extend([op["beta"].ravel(), op["gamma"].ravel()])
                elif op["type"] == "linear":
                    flat.extend([op["W"].ravel(), op["b"].ravel()])
                elif op["type"] == "shortcut_end":
                    collect(op["branch"])

        collect(ops)
        dumped = np.fromfile(os.path.join(d, name + ".params.f32"), np.float32)
        assert np.array_equal(np.concatenate(flat), dumped)
        if name == "a":  # and the values the program computed with them are the network's values
            xa = np.fromfile(os.path.join(d, "a.x.f32"), np.float32).reshape(4, 3, 8, 8)
            ya = np.fromfile(os.path.join(d, "a.y.f32"), np.float32).reshape(4, 10)
            np.testing.assert_allclose(ya, _forward(ops, xa).reshape(4, 10), rtol=2e-4, atol=2e-6)

    # a file written by the restatement: the C++ codec loads it, computes the network's values and writes it back unchanged
    assert open(os.path.join(d, "b2.crseq"), "rb").read() == data
    yb = np.fromfile(os.path.join(d, "b.y.f32"), np.float32).reshape(4, 10)
    np.testing.assert_allclose(yb, _forward(net, x).reshape(4, 10), rtol=2e-4, atol=2e-6)
