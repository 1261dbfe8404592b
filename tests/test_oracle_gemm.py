"""Pins the CPU oracle's GEMM and dense-layer functions (no GPU).

The reference holds no golden vectors for this path, so each function is pinned by checks that do not
restate its own formula: numpy float64 matmul on transposed/stacked operands, closed forms, and identities
between the entry points (the same ones the reference's linearUnitTest relies on).
"""
import numpy as np
import pytest

from oracle import seblas_oracle as orc
from tests.util import assert_close, normal, uniform


@pytest.mark.parametrize("M,N,K,batch", [(1, 1, 1, 1), (3, 5, 7, 2), (17, 33, 65, 3), (128, 64, 96, 1)])
def test_sgemm_vs_float64_matmul(M, N, K, batch):
    A, B = uniform(1, M, K), uniform(2, batch, K, N)
    ref = np.matmul(A.astype(np.float64)[None], B.astype(np.float64))
    assert_close(orc.sgemm(A, B), ref, K, "oracle sgemm")
    # A is shared by every batch slice (B.n loop of the reference), it is not batched itself
    assert_close(orc.sgemm(A, B)[batch - 1], A.astype(np.float64) @ B[batch - 1].astype(np.float64), K, "last slice")


@pytest.mark.parametrize("M,N,K,batch", [(1, 1, 1, 1), (3, 5, 7, 2), (17, 33, 65, 3)])
def test_sgemmTN_vs_float64_matmul(M, N, K, batch):
    A, B = uniform(3, K, M), uniform(4, batch, K, N)
    ref = np.matmul(A.astype(np.float64).T[None], B.astype(np.float64))
    assert_close(orc.sgemmTN(A, B), ref, K, "oracle sgemmTN")


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (17, 33, 65)])
def test_sgemmNT_vs_float64_matmul(M, N, K):
    A, B = uniform(5, M, K), uniform(6, N, K)
    assert_close(orc.sgemmNT(A, B), A.astype(np.float64) @ B.astype(np.float64).T, K, "oracle sgemmNT")


@pytest.mark.parametrize("M,N,K,batch", [(3, 5, 7, 1), (9, 4, 1, 16), (17, 33, 20, 3)])
def test_sgemmNTA_vs_float64_and_accumulates(M, N, K, batch):
    A, B, C0 = uniform(7, batch, M, K), uniform(8, batch, N, K), uniform(9, M, N)
    ref = C0.astype(np.float64) + np.einsum("bmk,bnk->mn", A.astype(np.float64), B.astype(np.float64))
    assert_close(orc.sgemmNTA(A, B, C0), ref, K * batch, "oracle sgemmNTA")
    # C is read-modify-write: starting from zero twice gives exactly twice (power-of-two scaling is exact)
    once = orc.sgemmNTA(A, B, np.zeros((M, N), np.float32))
    assert np.array_equal(orc.sgemmNTA(A, B, once), 2 * once)


def test_closed_forms():
    K, N = 37, 23
    B = uniform(10, K, N)
    assert np.array_equal(orc.sgemm(np.eye(K, dtype=np.float32), B), B)          # A = I  =>  C = B
    ones = np.ones((5, K), np.float32)
    assert np.array_equal(orc.sgemm(ones, np.ones((K, N), np.float32)), np.full((5, N), K, np.float32))
    u, v = uniform(11, 6, 1), uniform(12, 1, 9)                                      # rank-1: exact products
    assert np.array_equal(orc.sgemm(u, v), u * v)
    # a non-symmetric case where a transposed operand or swapped index would show
    A = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    Bm = np.array([[1, 0], [0, 1], [2, 3]], np.float32)
    assert np.array_equal(orc.sgemm(A, Bm), np.array([[7, 11], [16, 23]], np.float32))
    assert np.array_equal(orc.sgemmTN(A.T.copy(), Bm), np.array([[7, 11], [16, 23]], np.float32))
    assert np.array_equal(orc.sgemmNT(A, Bm.T.copy()), np.array([[7, 11], [16, 23]], np.float32))


def test_transposition_identities():
    M, N, K = 13, 11, 19
    A, B = uniform(13, M, K), uniform(14, K, N)
    C = orc.sgemm(A, B)
    assert np.array_equal(orc.sgemmNT(A, np.ascontiguousarray(B.T)), C)
    assert np.array_equal(orc.sgemmTN(np.ascontiguousarray(A.T), B), C)


@pytest.mark.parametrize("batch,IN,OUT", [(1, 1, 1), (4, 7, 5), (16, 40, 24)])
def test_linear_family_vs_float64(batch, IN, OUT):
    X, W, b, dY = normal(1, batch, IN), normal(2, OUT, IN), normal(3, OUT), normal(4, batch, OUT)
    X64, W64, dY64 = X.astype(np.float64), W.astype(np.float64), dY.astype(np.float64)
    assert_close(orc.linear(X, W, b), X64 @ W64.T + b, IN, "oracle linear")
    assert_close(orc.linearXGrad(dY, W), dY64 @ W64, OUT, "oracle linearXGrad")
    dW0, dB0 = normal(5, OUT, IN), normal(6, OUT)
    dW, dB = orc.linearParamGrad(dY, X, dW0, dB0)
    assert_close(dW, dW0 + dY64.T @ X64, batch, "oracle linearParamGrad dW")
    assert_close(dB, dB0 + dY64.sum(0), batch, "oracle linearParamGrad dB")


def test_linear_identity_weight_and_adjoint():
    batch, n = 6, 9
    X, b = normal(7, batch, n), normal(8, n)
    assert np.array_equal(orc.linear(X, np.eye(n, dtype=np.float32), b), X + b)
    IN, OUT = 12, 7
    X, W, dY = normal(9, batch, IN), normal(10, OUT, IN), normal(11, batch, OUT)
    zero_b = np.zeros(OUT, np.float32)
    lhs = np.vdot(orc.linear(X, W, zero_b).astype(np.float64), dY)
    mid = np.vdot(X.astype(np.float64), orc.linearXGrad(dY, W))
    dW, _ = orc.linearParamGrad(dY, X, np.zeros((OUT, IN), np.float32), zero_b)
    rhs = np.vdot(W.astype(np.float64), dW)
    assert abs(lhs - mid) < 1e-4 * abs(lhs) + 1e-4 and abs(lhs - rhs) < 1e-4 * abs(lhs) + 1e-4


def test_linear_param_grad_is_nta_of_outer_products():
    """validation/UnitTestTools.cu:143-144: linearParamGrad(dY,X) == sgemmNTA over K=1 outer products."""
    batch, IN, OUT = 8, 10, 6
    dY, X = normal(12, batch, OUT), normal(13, batch, IN)
    dW, _ = orc.linearParamGrad(dY, X, np.zeros((OUT, IN), np.float32), np.zeros(OUT, np.float32))
    nta = orc.sgemmNTA(dY.reshape(batch, OUT, 1), X.reshape(batch, IN, 1), np.zeros((OUT, IN), np.float32))
    np.testing.assert_allclose(dW, nta, atol=1e-3, rtol=0)


def test_thread_count_does_not_change_results():
    A, B = uniform(1, 37, 29), uniform(2, 2, 29, 31)
    assert np.array_equal(orc.sgemm(A, B, threads=1), orc.sgemm(A, B, threads=5))
    X, W, dY = normal(3, 3, 5, 9, 9), normal(4, 7, 5, 3, 3), normal(5, 3, 7, 9, 9)
    assert np.array_equal(orc.conv(W, X, None, 1, 1, 1, 1, threads=1), orc.conv(W, X, None, 1, 1, 1, 1, threads=4))
    z = np.zeros_like(W)
    assert np.array_equal(orc.convError(dY, X, z, 1, 1, 1, 1, threads=1), orc.convError(dY, X, z, 1, 1, 1, 1, threads=3))
