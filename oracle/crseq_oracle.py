"""CPU restatement of the reference's `.crseq` model file format (pure Python + numpy).

TEST INFRASTRUCTURE ONLY: imported by tests/ as the checker of the C++ codec. Nothing in the product imports it.

A network is a list of operand descriptions (dicts); `encode` produces the bytes `saveSequence` writes for it and
`decode` parses such bytes back, inferring each parameter's element count from the network input shape the way
`loadSequence` does. Everything is little-endian uint32 / float32.

File architecture (seio/modelcache/codec.cuh:18-38, codec.cu:8-39):
    header      magic 0x7921aedf, operand count, epoch id                       3 x uint32
    id table    one uint32 operand type id per top-level operand
    info        per top-level operand, its construction arguments (may be empty)
    parameters  per top-level operand, its trainable tensors as raw float32

Operand descriptions and their info / parameter records:
    {"type": "linear", "out": OUT, "W": (OUT, IN), "b": (OUT,)}     id 0x0001  info: OUT                  (Linear.cu:62-75)
    {"type": "conv2d", "W": (OC, IC, FH, FW), "stride": (sH, sW), "pad": (pH, pW), "b": (OC,) or None}
                                                                    id 0x0002  info: filter n,c,h,w, sH, sW, pH, pW, has-bias
                                                                               params: filter, then bias (Conv2D.cu:59-80,
                                                                               NetParam.cuh:45-53)
    {"type": "batchnorm", "beta": (C,H,W), "gamma": (C,H,W)}        id 0x0003  no info; params: beta, then gamma
                                                                               (BatchNorm.cu:46-55)
    {"type": "softmax"}                                             id 0x0005  nothing
    {"type": "relu"}                                                id 0xa002  nothing
    {"type": "maxpool2d", "stride": (sH, sW), "range": (rH, rW)}    id 0xb003  info: sH, sW, rH, rW       (MaxPool2D.cu:22-33)
    {"type": "shortcut_beg", "uuid": U}                             id 0xf002  info: U, 0
    {"type": "shortcut_end", "uuid": U, "branch": [operands...]}    id 0xf003  info: U, count, the branch's id table, the
                                                                               branch's infos; params: the branch's params
                                                                               (ShortcutEndpoint.cu:151-177)
A convolution written by the reference's cuDNN operand (id 0xd002) has the same records as 0x0002
(OperandCodecs.cu:175-206) and decodes to "conv2d" with "cudnn": True.

Two places where the reference's reader does not accept what its writer produces, both for a closing shortcut endpoint
that has branch operands: the info cursor is not advanced past the branch's infos (OperandCodecs.cu:236-259: only the
local `subInfoOffset` moves), and the branch's parameter shapes are taken from `branchOperands[i-1]` with i = 0
(:261-269). `decode` here reads what the writer wrote: the cursor moves past the branch, and the branch's input shape is
the shape that entered the opening endpoint with the same uuid.
"""
import struct

import numpy as np

MAGIC = 0x7921AEDF
IDS = {"linear": 0x0001, "conv2d": 0x0002, "batchnorm": 0x0003, "softmax": 0x0005, "relu": 0xA002,
       "maxpool2d": 0xB003, "shortcut_beg": 0xF002, "shortcut_end": 0xF003}
NAMES = {v: k for k, v in IDS.items()}
ID_CUDNN_CONV2D = 0xD002


def _u32(*vals):
    return struct.pack("<%dI" % len(vals), *vals)


def _f32(a):
    return np.ascontiguousarray(a, dtype="<f4").tobytes()


# ---- writer (codec.cu:8-39) ----------------------------------------------------------------------------------------
def op_id(op):
    if op["type"] == "conv2d" and op.get("cudnn"):
        return ID_CUDNN_CONV2D
    return IDS[op["type"]]


def encode_info(op):
    t = op["type"]
    if t == "linear":
        return _u32(op["out"])
    if t == "conv2d":
        oc, ic, fh, fw = op["W"].shape
        return _u32(oc, ic, fh, fw, op["stride"][0], op["stride"][1], op["pad"][0], op["pad"][1], 0 if op.get("b") is None else 1)
    if t == "maxpool2d":
        return _u32(op["stride"][0], op["stride"][1], op["range"][0], op["range"][1])
    if t == "shortcut_beg":
        return _u32(op["uuid"], 0)
    if t == "shortcut_end":
        branch = op.get("branch", [])
        out = _u32(op["uuid"], len(branch))
        out += b"".join(_u32(op_id(b)) for b in branch)
        out += b"".join(encode_info(b) for b in branch)
        return out
    return b""  # batchnorm, softmax, relu


def encode_params(op):
    t = op["type"]
    if t == "linear":
        return _f32(op["W"]) + _f32(op["b"])
    if t == "conv2d":
        return _f32(op["W"]) + (b"" if op.get("b") is None else _f32(op["b"]))
    if t == "batchnorm":
        return _f32(op["beta"]) + _f32(op["gamma"])
    if t == "shortcut_end":
        return b"".join(encode_params(b) for b in op.get("branch", []))
    return b""


def encode(operands, epoch=0):
    out = _u32(MAGIC, len(operands), epoch)
    out += b"".join(_u32(op_id(op)) for op in operands)
    out += b"".join(encode_info(op) for op in operands)
    out += b"".join(encode_params(op) for op in operands)
    return out


# ---- reader (codec.cu:41-97, OperandCodecs.cu) ----------------------------------------------------------------------
class _Cursor:
    def __init__(self, data, pos):
        self.data, self.pos = data, pos

    def u32(self, n=1):
        if self.pos + 4 * n > len(self.data):
            raise ValueError("crseq: file ends inside a record")
        vals = struct.unpack_from("<%dI" % n, self.data, self.pos)
        self.pos += 4 * n
        return vals if n > 1 else vals[0]

    def f32(self, shape):
        count = int(np.prod(shape))
        if self.pos + 4 * count > len(self.data):
            raise ValueError("crseq: file ends inside a parameter tensor")
        a = np.frombuffer(self.data, "<f4", count, self.pos).reshape(shape).copy()
        self.pos += 4 * count
        return a


def decode_info(type_id, cur):
    """The operand description without its tensors; `cur` is the info cursor."""
    if type_id == ID_CUDNN_CONV2D or type_id == IDS["conv2d"]:
        oc, ic, fh, fw, sh, sw, ph, pw, has_bias = cur.u32(9)
        op = {"type": "conv2d", "filter": (oc, ic, fh, fw), "stride": (sh, sw), "pad": (ph, pw), "has_bias": has_bias > 0}
        if type_id == ID_CUDNN_CONV2D:
            op["cudnn"] = True
        return op
    if type_id not in NAMES:
        raise ValueError("crseq: operand type 0x%04x is not handled" % type_id)
    t = NAMES[type_id]
    if t == "linear":
        return {"type": t, "out": cur.u32()}
    if t == "maxpool2d":
        sh, sw, rh, rw = cur.u32(4)
        return {"type": t, "stride": (sh, sw), "range": (rh, rw)}
    if t == "shortcut_beg":
        uuid, _ = cur.u32(2)
        return {"type": t, "uuid": uuid}
    if t == "shortcut_end":
        uuid, count = cur.u32(2)
        ids = [cur.u32() for _ in range(count)]
        return {"type": t, "uuid": uuid, "branch": [decode_info(i, cur) for i in ids]}
    return {"type": t}


def out_shape(op, s):
    """Output shape (n, c, h, w) of an operand for input shape s (Conv2D.cuh:40-44, Linear.cuh, MaxPool2D.cuh:42-51)."""
    n, c, h, w = s
    t = op["type"]
    if t == "conv2d":
        oc, _, fh, fw = op["filter"] if "filter" in op else op["W"].shape
        return (n, oc, (h + 2 * op["pad"][0] - fh) // op["stride"][0] + 1, (w + 2 * op["pad"][1] - fw) // op["stride"][1] + 1)
    if t == "linear":
        return (n, 1, op["out"], 1)
    if t == "maxpool2d":
        return (n, c, h // op["stride"][0], w // op["stride"][1])
    return s


def decode_params(op, cur, s, open_shapes):
    """Reads op's tensors at the parameter cursor for input shape s; returns the output shape."""
    t = op["type"]
    if t == "linear":
        op["W"] = cur.f32((op["out"], s[1] * s[2] * s[3]))
        op["b"] = cur.f32((op["out"],))
    elif t == "conv2d":
        op["W"] = cur.f32(op.pop("filter"))
        op["b"] = cur.f32((op["W"].shape[0],)) if op.pop("has_bias") else None
    elif t == "batchnorm":
        op["beta"] = cur.f32(s[1:])
        op["gamma"] = cur.f32(s[1:])
    elif t == "shortcut_beg":
        open_shapes[op["uuid"]] = s
    elif t == "shortcut_end":
        if op["uuid"] not in open_shapes:
            raise ValueError("crseq: closing shortcut endpoint %d has no opening endpoint" % op["uuid"])
        bs = open_shapes[op["uuid"]]
        for b in op["branch"]:
            bs = decode_params(b, cur, bs, open_shapes)
        if op["branch"] and bs != s:
            raise ValueError("crseq: shortcut branch output %s differs from the main path %s" % (bs, s))
    return out_shape(op, s)


def decode(data, in_shape):
    """-> (epoch, operands, output shape). in_shape = (n, c, h, w) of the network input."""
    head = _Cursor(data, 0)
    magic, count, epoch = head.u32(3)
    if magic != MAGIC:
        raise ValueError("crseq: wrong magic number 0x%08x" % magic)
    info = _Cursor(data, 12 + 4 * count)
    operands = [decode_info(head.u32(), info) for _ in range(count)]
    par = _Cursor(data, info.pos)
    s, open_shapes = tuple(in_shape), {}
    for op in operands:
        s = decode_params(op, par, s, open_shapes)
    if par.pos != len(data):
        raise ValueError("crseq: %d bytes after the last parameter" % (len(data) - par.pos))
    return epoch, operands, s


# ---- record sizes as the operands report them (getInfoEncodingSize / getNetParamsEncodingSize) -----------------------
def info_size(op):
    t = op["type"]
    if t == "conv2d":
        return 36  # Conv2D.cuh:93-95
    if t == "linear":
        return 4  # Linear.cuh:66-68
    if t == "maxpool2d":
        return 16  # MaxPool2D.cuh:63-65
    if t == "shortcut_beg":
        return 8
    if t == "shortcut_end":  # uuid, count and the branch's id table and infos as written (ShortcutEndpoint.cu:151-167)
        return 8 + sum(4 + info_size(b) for b in op.get("branch", []))
    return 0
