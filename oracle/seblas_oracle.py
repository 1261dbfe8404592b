"""numpy-facing loader of the CPU oracle (oracle/seblas_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg. Nothing in the product package imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libseblas_oracle.so")

_u32 = ctypes.c_uint32
_f = ctypes.POINTER(ctypes.c_float)
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib


def _ptr(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def sgemm(A, B, threads=1):
    """A (M,K); B (batch,K,N) or (K,N) -> C with B's batch shape."""
    A, B = _f32(A), _f32(B)
    B3 = B.reshape(-1, B.shape[-2], B.shape[-1])
    M, K = A.shape
    N = B3.shape[2]
    C = np.empty((B3.shape[0], M, N), np.float32)
    load().oracle_sgemm(_ptr(A), _ptr(B3), _ptr(C), _u32(M), _u32(N), _u32(K), _u32(B3.shape[0]), threads)
    return C.reshape(B.shape[:-2] + (M, N))


def sgemmTN(A, B, threads=1):
    """A stored (K,M); B (batch,K,N) or (K,N)."""
    A, B = _f32(A), _f32(B)
    B3 = B.reshape(-1, B.shape[-2], B.shape[-1])
    K, M = A.shape
    N = B3.shape[2]
    C = np.empty((B3.shape[0], M, N), np.float32)
    load().oracle_sgemmTN(_ptr(A), _ptr(B3), _ptr(C), _u32(M), _u32(N), _u32(K), _u32(B3.shape[0]), threads)
    return C.reshape(B.shape[:-2] + (M, N))


def sgemmNT(A, B, threads=1):
    """A (M,K); B stored (N,K)."""
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[0]
    C = np.empty((M, N), np.float32)
    load().oracle_sgemmNT(_ptr(A), _ptr(B), _ptr(C), _u32(M), _u32(N), _u32(K), threads)
    return C


def sgemmNTA(A, B, C, threads=1):
    """A (batch,M,K); B (batch,N,K); returns C + sum_b A[b] B[b]^T (C is not modified)."""
    A, B = _f32(A), _f32(B)
    A3 = A.reshape(-1, A.shape[-2], A.shape[-1])
    B3 = B.reshape(-1, B.shape[-2], B.shape[-1])
    out = _f32(C).copy()
    M, K = A3.shape[1:]
    N = B3.shape[1]
    load().oracle_sgemmNTA(_ptr(A3), _ptr(B3), _ptr(out), _u32(M), _u32(N), _u32(K), _u32(A3.shape[0]), threads)
    return out


def linear(X, W, B, threads=1):
    X, W, B = _f32(X), _f32(W), _f32(B)
    batch, IN = X.shape
    OUT = W.shape[0]
    Y = np.empty((batch, OUT), np.float32)
    load().oracle_linear(_ptr(X), _ptr(W), _ptr(B), _ptr(Y), _u32(batch), _u32(IN), _u32(OUT), threads)
    return Y


def linearXGrad(dY, W, threads=1):
    dY, W = _f32(dY), _f32(W)
    batch, OUT = dY.shape
    IN = W.shape[1]
    dX = np.empty((batch, IN), np.float32)
    load().oracle_linearXGrad(_ptr(dY), _ptr(W), _ptr(dX), _u32(batch), _u32(IN), _u32(OUT), threads)
    return dX


def linearParamGrad(dY, X, dW, dB, threads=1):
    """Returns (dW + dY^T X, dB + colsum(dY)); inputs are not modified."""
    dY, X = _f32(dY), _f32(X)
    batch, OUT = dY.shape
    IN = X.shape[1]
    dW2, dB2 = _f32(dW).copy(), _f32(dB).copy()
    load().oracle_linearParamGrad(_ptr(dY), _ptr(X), _ptr(dW2), _ptr(dB2), _u32(batch), _u32(IN), _u32(OUT), threads)
    return dW2, dB2


def out_hw(IH, IW, FH, FW, sH, sW, pH, pW):
    return (IH - FH + 2 * pH) // sH + 1, (IW - FW + 2 * pW) // sW + 1


def _geom_args(N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW):
    return [_u32(v) for v in (N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW)]


def conv(W, X, bias, sH, sW, pH, pW, threads=1):
    W, X = _f32(W), _f32(X)
    bias = None if bias is None else _f32(bias)
    OC, IC, FH, FW = W.shape
    N, _, IH, IW = X.shape
    OH, OW = out_hw(IH, IW, FH, FW, sH, sW, pH, pW)
    Y = np.empty((N, OC, OH, OW), np.float32)
    load().oracle_conv(_ptr(W), _ptr(X), _ptr(Y), _ptr(bias),
                       *_geom_args(N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW), threads)
    return Y


def convDerive(W, dY, in_hw, sH, sW, pH, pW, threads=1):
    W, dY = _f32(W), _f32(dY)
    OC, IC, FH, FW = W.shape
    N, _, OH, OW = dY.shape
    IH, IW = in_hw
    dX = np.empty((N, IC, IH, IW), np.float32)
    load().oracle_convDerive(_ptr(W), _ptr(dY), _ptr(dX),
                             *_geom_args(N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW), threads)
    return dX


def convError(dY, X, dW, sH, sW, pH, pW, threads=1):
    """Returns dW + wgrad (dW is not modified)."""
    dY, X = _f32(dY), _f32(X)
    out = _f32(dW).copy()
    OC, IC, FH, FW = out.shape
    N, _, IH, IW = X.shape
    OH, OW = dY.shape[2:]
    load().oracle_convError(_ptr(dY), _ptr(X), _ptr(out),
                            *_geom_args(N, IC, IH, IW, OC, FH, FW, OH, OW, sH, sW, pH, pW), threads)
    return out


def convBias(Y, bias):
    out = _f32(Y).copy()
    N, C = out.shape[:2]
    HW = int(np.prod(out.shape[2:]))
    load().oracle_convBias(_ptr(out), _ptr(_f32(bias)), _u32(N), _u32(C), _u32(HW))
    return out


# ---- elementwise / reduction operators (oracle/seblas_oracle_ew.c) -------------------------------------------------
def relu(X):
    X = _f32(X)
    Y = np.empty_like(X)
    load().oracle_relu(_ptr(X), _ptr(Y), _u32(X.size))
    return Y


def reluGradFast(X, dY):
    X, dY = _f32(X), _f32(dY)
    dX = np.empty_like(X)
    load().oracle_reluGradFast(_ptr(X), _ptr(dY), _ptr(dX), _u32(X.size))
    return dX


def maxPool(X, rH, rW):
    """X (N,C,IH,IW) -> (Y (N,C,IH//rH,IW//rW), record (N,C,OH*rH,OW*rW))."""
    X = _f32(X)
    N, C, IH, IW = X.shape
    OH, OW = IH // rH, IW // rW
    Y = np.empty((N, C, OH, OW), np.float32)
    rec = np.empty((N, C, OH * rH, OW * rW), np.float32)
    load().oracle_maxPool(_ptr(X), _ptr(Y), _ptr(rec), _u32(N * C), _u32(IH), _u32(IW), _u32(rH), _u32(rW))
    return Y, rec


def maxPoolBack(dY, record, in_hw, rH, rW):
    """Returns (dX, record after the pass); `record` is not modified."""
    dY, rec = _f32(dY), _f32(record).copy()
    N, C = dY.shape[:2]
    IH, IW = in_hw
    dX = np.empty((N, C, IH, IW), np.float32)
    load().oracle_maxPoolBack(_ptr(dX), _ptr(dY), _ptr(rec), _u32(N * C), _u32(IH), _u32(IW), _u32(rH), _u32(rW))
    return dX, rec


def softmax(A, step):
    A = _f32(A)
    assert A.size % step == 0
    out = np.empty_like(A)
    load().oracle_softmax(_ptr(A), _ptr(out), _u32(A.size // step), _u32(step))
    return out


def crossEntropyLoss(Y, labels):
    Y, labels = _f32(Y), _f32(labels)
    dY = np.empty_like(Y)
    load().oracle_crossEntropyLoss(_ptr(Y), _ptr(labels), _ptr(dY), _u32(Y.size))
    return dY


def crossEntropyCalc(Y, labels):
    Y, labels = _f32(Y), _f32(labels)
    fn = load().oracle_crossEntropyCalc
    fn.restype = ctypes.c_float
    return float(fn(_ptr(Y), _ptr(labels), _u32(Y.size)))


def tensorAdd(A, B):
    A, B = _f32(A).copy(), _f32(B)
    load().oracle_tensorAdd(_ptr(A), _ptr(B), _u32(A.size))
    return A


def tensorSub(A, B):
    A, B = _f32(A).copy(), _f32(B)
    load().oracle_tensorSub(_ptr(A), _ptr(B), _u32(A.size))
    return A


def tensorScale(A, s):
    A = _f32(A).copy()
    load().oracle_tensorScale(_ptr(A), ctypes.c_float(s), _u32(A.size))
    return A


def constFill(A, v):
    A = _f32(A).copy()
    load().oracle_constFill(_ptr(A), ctypes.c_float(v), _u32(A.size))
    return A


def momentumApply(X, G, M, lr, beta, decay=1.0):
    """Returns the updated (X, G, M); the arguments are not modified."""
    X, G, M = _f32(X).copy(), _f32(G).copy(), _f32(M).copy()
    load().oracle_momentumApply(_ptr(X), _ptr(G), _ptr(M), _u32(X.size), ctypes.c_float(lr), ctypes.c_float(beta),
                                ctypes.c_float(decay))
    return X, G, M


def batchNorm(X, beta, gamma):
    """X (N, ...) -> (Y, xHat, mean, var); statistics per feature (every position after the batch axis) over N."""
    X = _f32(X)
    N, F = X.shape[0], X.size // X.shape[0]
    Y, xHat = np.empty_like(X), np.empty_like(X)
    mean, var = np.empty(F, np.float32), np.empty(F, np.float32)
    load().oracle_batchNorm(_ptr(X), _ptr(_f32(beta).ravel()), _ptr(_f32(gamma).ravel()), _ptr(mean), _ptr(var), _ptr(Y),
                            _ptr(xHat), _u32(N), _u32(F))
    return Y, xHat, mean, var


def batchNormGrad(dY, gamma, X):
    dY, X = _f32(dY), _f32(X)
    N, F = X.shape[0], X.size // X.shape[0]
    dX = np.empty_like(X)
    load().oracle_batchNormGrad(_ptr(dY), _ptr(_f32(gamma).ravel()), _ptr(X), _ptr(dX), _u32(N), _u32(F))
    return dX


def batchNormParamGrads(dY, xHat):
    """Returns (dGamma, dBeta), each with F values."""
    dY, xHat = _f32(dY), _f32(xHat)
    N, F = dY.shape[0], dY.size // dY.shape[0]
    dG, dB = np.empty(F, np.float32), np.empty(F, np.float32)
    load().oracle_batchNormParamGrads(_ptr(dY), _ptr(xHat), _ptr(dG), _ptr(dB), _u32(N), _u32(F))
    return dG, dB
