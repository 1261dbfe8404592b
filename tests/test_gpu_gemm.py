"""GPU parity of the GEMM and dense-layer entry points (through the C ABI) against the CPU oracle.

Case grids follow the reference's own differential tests (validation/UnitTestTools.cu:130-170 for the
linear/NTA identity) plus the sizes its `%4` kernel-selection rules and 128-wide tiles make interesting
(seblas/operations/cuGEMM.cu:1653-1660).
"""
import numpy as np
import pytest

from tests.util import assert_close, to_dev, to_np, uniform, normal

pytestmark = pytest.mark.gpu

ODD = [1, 2, 3, 5, 7, 127, 129, 130]


def _capi():
    from crusaderbackend_amd import capi
    return capi


def _oracle():
    from oracle import seblas_oracle
    return seblas_oracle


def _empty(dev, *shape):
    import torch
    return torch.full(shape, float("nan"), dtype=torch.float32, device=dev)


def run_nn(dev, M, N, K, batch, seed):
    A = uniform(seed, M, K)
    B = uniform(seed + 1, batch, K, N)
    C = _empty(dev, batch, M, N)
    _capi().sgemm_nn(to_dev(A, dev), to_dev(B, dev), C, M, N, K, batch)
    assert_close(to_np(C), _oracle().sgemm(A, B, threads=8), K, f"sgemm_nn {M}x{N}x{K} b{batch}")


def run_tn(dev, M, N, K, batch, seed):
    A = uniform(seed, K, M)
    B = uniform(seed + 1, batch, K, N)
    C = _empty(dev, batch, M, N)
    _capi().sgemm_tn(to_dev(A, dev), to_dev(B, dev), C, M, N, K, batch)
    assert_close(to_np(C), _oracle().sgemmTN(A, B, threads=8), K, f"sgemm_tn {M}x{N}x{K} b{batch}")


def run_nt(dev, M, N, K, seed):
    A = uniform(seed, M, K)
    B = uniform(seed + 1, N, K)
    C = _empty(dev, M, N)
    _capi().sgemm_nt(to_dev(A, dev), to_dev(B, dev), C, M, N, K)
    assert_close(to_np(C), _oracle().sgemmNT(A, B, threads=8), K, f"sgemm_nt {M}x{N}x{K}")


def run_nta(dev, M, N, K, batch, seed):
    A = uniform(seed, batch, M, K)
    B = uniform(seed + 1, batch, N, K)
    C0 = uniform(seed + 2, M, N)
    C = to_dev(C0, dev)
    _capi().sgemm_nta(to_dev(A, dev), to_dev(B, dev), C, M, N, K, batch)
    assert_close(to_np(C), _oracle().sgemmNTA(A, B, C0, threads=8), K * batch, f"sgemm_nta {M}x{N}x{K} b{batch}")


def test_sgemm_config1_1024(dev):
    """benchmark configuration 1: M=N=K=1024, uniform[-1,1], fixed seeds."""
    run_nn(dev, 1024, 1024, 1024, 1, seed=1)


@pytest.mark.parametrize("M,N,K", [(m, n, k) for m in ODD for n in (1, 5, 129) for k in (1, 7, 130)])
def test_sgemm_nn_odd(dev, M, N, K):
    run_nn(dev, M, N, K, 1, seed=100 + M + N + K)


@pytest.mark.parametrize("M,N,K,batch", [(64, 64, 64, 3), (130, 36, 20, 2), (256, 384, 128, 2), (8, 260, 24, 5)])
def test_sgemm_nn_batched(dev, M, N, K, batch):
    run_nn(dev, M, N, K, batch, seed=7)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (127, 129, 130), (128, 128, 16), (132, 260, 33),
                                   (512, 256, 100), (64, 512, 12)])
def test_sgemm_tn(dev, M, N, K):
    run_tn(dev, M, N, K, 1, seed=11)
    run_tn(dev, M, N, K, 2, seed=12)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (127, 129, 130), (129, 257, 64), (256, 130, 36),
                                   (260, 260, 260), (512, 512, 128)])
def test_sgemm_nt(dev, M, N, K):
    run_nt(dev, M, N, K, seed=21)


@pytest.mark.parametrize("M,N,K,batch", [(4, 6, 1, 128), (130, 66, 1, 16), (64, 64, 8, 4), (200, 100, 12, 3),
                                         (129, 3, 5, 7), (256, 256, 64, 2)])
def test_sgemm_nta(dev, M, N, K, batch):
    run_nta(dev, M, N, K, batch, seed=31)


def test_sgemm_nta_accumulates_twice(dev):
    """Calling the accumulate form twice on a zero C doubles the single-call result."""
    M, N, K, batch = 96, 80, 20, 3
    A, B = uniform(1, batch, M, K), uniform(2, batch, N, K)
    import torch
    C = torch.zeros(M, N, device=dev)
    dA, dB = to_dev(A, dev), to_dev(B, dev)
    _capi().sgemm_nta(dA, dB, C, M, N, K, batch)
    once = to_np(C).copy()
    _capi().sgemm_nta(dA, dB, C, M, N, K, batch)
    np.testing.assert_allclose(to_np(C), 2 * once, rtol=1e-6, atol=0)


@pytest.mark.parametrize("batch,IN,OUT", [(1, 1, 1), (3, 7, 5), (128, 512, 512), (128, 512, 10), (64, 130, 66),
                                          (33, 1024, 10), (256, 260, 132)])
def test_linear_family(dev, batch, IN, OUT):
    capi, orc = _capi(), _oracle()
    X, W, b = normal(1, batch, IN), normal(2, OUT, IN, std=(2.0 / IN) ** 0.5), normal(3, OUT)
    dY = normal(4, batch, OUT)
    Y = _empty(dev, batch, OUT)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, batch, IN, OUT)
    assert_close(to_np(Y), orc.linear(X, W, b, threads=8), IN, "linear")
    dX = _empty(dev, batch, IN)
    capi.linear_dgrad(to_dev(dY, dev), to_dev(W, dev), dX, batch, IN, OUT)
    assert_close(to_np(dX), orc.linearXGrad(dY, W, threads=8), OUT, "linearXGrad")
    dW0, dB0 = normal(5, OUT, IN), normal(6, OUT)
    dW, dB = to_dev(dW0, dev), to_dev(dB0, dev)
    capi.linear_wgrad(to_dev(dY, dev), to_dev(X, dev), dW, dB, batch, IN, OUT)
    rW, rB = orc.linearParamGrad(dY, X, dW0, dB0, threads=8)
    assert_close(to_np(dW), rW, batch, "linearParamGrad dW")
    assert_close(to_np(dB), rB, batch, "linearParamGrad dB")


def test_linear_param_grad_equals_nta_outer_products(dev):
    """The reference's linearUnitTest identity (validation/UnitTestTools.cu:143-144): dW from
    linearParamGrad equals sgemmNTA over the batch of K=1 outer products dY[n] x X[n]^T."""
    import torch
    capi = _capi()
    batch, IN, OUT = 32, 48, 40
    dY, X = normal(1, batch, OUT), normal(2, batch, IN)
    dW1 = torch.zeros(OUT, IN, device=dev)
    dB = torch.zeros(OUT, device=dev)
    capi.linear_wgrad(to_dev(dY, dev), to_dev(X, dev), dW1, dB, batch, IN, OUT)
    dW2 = torch.zeros(OUT, IN, device=dev)
    # A = dY viewed as (batch, OUT, 1), B = X viewed as (batch, IN, 1)
    capi.sgemm_nta(to_dev(dY, dev), to_dev(X, dev), dW2, OUT, IN, 1, batch)
    np.testing.assert_allclose(to_np(dW1), to_np(dW2), atol=1e-3, rtol=0)  # abs 1e-3 as in the reference test


def test_linear_relu_flag(dev):
    capi, orc = _capi(), _oracle()
    batch, IN, OUT = 16, 64, 48
    X, W, b = normal(1, batch, IN), normal(2, OUT, IN), normal(3, OUT)
    Y = _empty(dev, batch, OUT)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, batch, IN, OUT, flags=capi.CRB_FLAG_RELU)
    assert_close(to_np(Y), np.maximum(orc.linear(X, W, b), 0), IN, "linear+relu")


# Shapes whose tile grid fills the chip in whole rounds and whose contraction is a multiple of 32 run on the kernel that
# loads operand panels straight into LDS: 128 x 128 tiles (the first three), 64 x 64 tiles (the next three), the latter as
# eight-wave workgroups when there is at most one per CU (the last two); ragged edge tiles included.
DIRECT_TO_LDS = [(2048, 2048, 256), (2040, 2044, 288), (1024, 4096, 320), (512, 4096, 512), (508, 4092, 544), (32768, 64, 576),
                 (1000, 1020, 544), (768, 1024, 1024)]


@pytest.mark.parametrize("M,N,K", DIRECT_TO_LDS)
def test_sgemm_forms_on_chip_filling_shapes(dev, M, N, K):
    run_nn(dev, M, N, K, 1, seed=71)
    run_nt(dev, M, N, K, seed=72)
    run_tn(dev, M, N, K, 1, seed=73)
    run_nta(dev, M, N, K // 2 if K % 64 == 0 else K, 2 if K % 64 == 0 else 1, seed=74)


def test_sgemm_nn_batched_on_chip_filling_shape(dev):
    run_nn(dev, 512, 1024, 256, 4, seed=75)
    run_tn(dev, 512, 1024, 256, 4, seed=76)


@pytest.mark.parametrize("batch,IN,OUT", [(2048, 256, 2048), (512, 512, 4096), (2040, 288, 2044), (2048, 1024, 2048)])
def test_linear_family_on_chip_filling_shapes(dev, batch, IN, OUT):
    """Bias, ReLU, accumulation and the bias gradient riding along, on the whole-tile and the edge-tile epilogues."""
    capi, orc = _capi(), _oracle()
    X, W, b = normal(1, batch, IN), normal(2, OUT, IN, std=(2.0 / IN) ** 0.5), normal(3, OUT)
    dY = normal(4, batch, OUT)
    Y = _empty(dev, batch, OUT)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, batch, IN, OUT)
    ref = orc.linear(X, W, b, threads=8)
    assert_close(to_np(Y), ref, IN, "linear")
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, batch, IN, OUT, flags=capi.CRB_FLAG_RELU)
    assert_close(to_np(Y), np.maximum(ref, 0), IN, "linear+relu")
    dX = _empty(dev, batch, IN)
    capi.linear_dgrad(to_dev(dY, dev), to_dev(W, dev), dX, batch, IN, OUT)
    assert_close(to_np(dX), orc.linearXGrad(dY, W, threads=8), OUT, "linearXGrad")
    dW0, dB0 = normal(5, OUT, IN), normal(6, OUT)
    dW, dB = to_dev(dW0, dev), to_dev(dB0, dev)
    capi.linear_wgrad(to_dev(dY, dev), to_dev(X, dev), dW, dB, batch, IN, OUT)
    rW, rB = orc.linearParamGrad(dY, X, dW0, dB0, threads=8)
    assert_close(to_np(dW), rW, batch, "linearParamGrad dW")
    assert_close(to_np(dB), rB, batch, "linearParamGrad dB")


def test_error_paths(dev):
    import torch
    capi = _capi()
    t = torch.zeros(16, device=dev)
    lib = capi.load()
    assert lib.crb_sgemm_nn(None, t.data_ptr(), t.data_ptr(), 4, 4, 1, 1, None) == capi.CRB_ENULL
    assert lib.crb_sgemm_nn(t.data_ptr(), t.data_ptr(), t.data_ptr(), 0, 4, 1, 1, None) == capi.CRB_EINVAL_SHAPE
    assert b"zero dimension" in lib.crb_last_error_string()
    assert lib.crb_linear_fwd(t.data_ptr(), t.data_ptr(), None, t.data_ptr(), 1, 4, 4, 0, None) == capi.CRB_ENULL


@pytest.mark.parametrize("M,N,K", [(256, 256, 4096), (100, 200, 3000), (64, 48, 8192), (130, 1000, 2049), (1, 1, 5000)])
def test_split_k_paths(dev, M, N, K):
    """Few output tiles and a long contraction: the K range is split over workgroups and recombined in fixed order."""
    run_nn(dev, M, N, K, 1, seed=41)
    run_tn(dev, M, N, K, 1, seed=42)
    run_nt(dev, M, N, K, seed=43)


@pytest.mark.parametrize("M,N,K", [(256, 2048, 2048), (512, 512, 4096), (128, 2048, 2048), (250, 1020, 2048), (128, 512, 8192)])
def test_split_k_on_the_direct_to_lds_kernel(dev, M, N, K):
    """Few tiles, contraction a multiple of 32: slices of K on the kernel that loads straight into LDS (128-wide and 64-wide tiles,
    ragged edges), every form, and the dense-layer epilogues (bias, ReLU, accumulate with the bias gradient) behind the slice sum."""
    run_nn(dev, M, N, K, 1, seed=45)
    run_tn(dev, M, N, K, 1, seed=46)
    run_nt(dev, M, N, K, seed=47)
    capi, orc = _capi(), _oracle()
    X, W, b = normal(1, M, K), normal(2, N, K, std=(2.0 / K) ** 0.5), normal(3, N)
    Y = _empty(dev, M, N)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, M, K, N, flags=capi.CRB_FLAG_RELU)
    assert_close(to_np(Y), np.maximum(orc.linear(X, W, b, threads=8), 0), K, "linear + bias + relu behind the slice sum")
    Y2 = _empty(dev, M, N)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y2, M, K, N, flags=capi.CRB_FLAG_RELU)
    assert np.array_equal(to_np(Y), to_np(Y2)), "bit-reproducible"
    # weight gradient dW (M x N) += dY^T (K x M) * X (K x N), dB += column sums of dY: batch = K
    dY, Xb = normal(4, K, M), normal(5, K, N)
    dW0, dB0 = normal(6, M, N), normal(7, M)
    dW, dB = to_dev(dW0, dev), to_dev(dB0, dev)
    capi.linear_wgrad(to_dev(dY, dev), to_dev(Xb, dev), dW, dB, K, N, M)
    rW, rB = orc.linearParamGrad(dY, Xb, dW0, dB0, threads=8)
    assert_close(to_np(dW), rW, K, "linearParamGrad dW behind the slice sum")
    assert_close(to_np(dB), rB, K, "linearParamGrad dB")


def test_split_k_nta_small_output_and_bias_epilogue(dev):
    run_nta(dev, 48, 24, 1024, 64, seed=44)
    capi, orc = _capi(), _oracle()
    batch, IN, OUT = 32, 2048, 300
    X, W, b = normal(1, batch, IN), normal(2, OUT, IN, std=0.02), normal(3, OUT)
    Y = _empty(dev, batch, OUT)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y, batch, IN, OUT, flags=capi.CRB_FLAG_RELU)
    assert_close(to_np(Y), np.maximum(orc.linear(X, W, b, threads=8), 0), IN, "split-K linear + bias + relu")
    # bit-reproducible
    Y2 = _empty(dev, batch, OUT)
    capi.linear_fwd(to_dev(X, dev), to_dev(W, dev), to_dev(b, dev), Y2, batch, IN, OUT, flags=capi.CRB_FLAG_RELU)
    assert np.array_equal(to_np(Y), to_np(Y2))


def test_split_k_on_two_streams_keeps_scratch_apart(dev):
    """Split-K calls queued on two streams at once use separate scratch: each result equals the one the same call gives alone."""
    import torch
    capi = _capi()
    shapes = [(256, 256, 4096), (192, 320, 6144)]
    ops = []
    for i, (M, N, K) in enumerate(shapes):
        A, B = to_dev(uniform(60 + i, M, K), dev), to_dev(uniform(70 + i, K, N), dev)
        alone = _empty(dev, M, N)
        capi.sgemm_nn(A, B, alone, M, N, K)
        ops.append((A, B, alone, M, N, K))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=dev) for _ in shapes]
    outs = [[_empty(dev, M, N) for _ in range(8)] for (_, _, _, M, N, K) in ops]
    for rep in range(8):  # interleaved, so the two streams' kernels overlap on the device
        for (A, B, _, M, N, K), st, out in zip(ops, streams, outs):
            capi.sgemm_nn(A, B, out[rep], M, N, K, stream=st)
    torch.cuda.synchronize()
    for (_, _, alone, M, N, K), out in zip(ops, outs):
        for rep in range(8):
            assert torch.equal(out[rep], alone), f"{M}x{N}x{K} repeat {rep}"
    capi.load().crb_release_workspace()
    again = _empty(dev, *shapes[0][:2])
    capi.sgemm_nn(ops[0][0], ops[0][1], again, *shapes[0])  # the arena comes back after a release
    torch.cuda.synchronize()
    assert torch.equal(again, ops[0][2])


def test_sgemm_4096_cubed_full_size(dev):
    """The headline GEMM shape at full size: against the oracle on seeded uniform[-1,1] inputs, and exactly against a product
    whose value is known in closed form (B a signed permutation: every output element is one input element, sign flipped or not)."""
    import torch
    n = 4096
    capi = _capi()
    A = uniform(5, n, n)
    B = uniform(6, n, n)
    C = _empty(dev, n, n)
    Ad = to_dev(A, dev)
    capi.sgemm_nn(Ad, to_dev(B, dev), C, n, n, n)
    assert_close(to_np(C), _oracle().sgemm(A, B[None], threads=16)[0], n, "sgemm_nn 4096^3")
    perm = rng_perm(7, n)
    sign = np.where(np.arange(n) % 3 == 0, -1.0, 1.0).astype(np.float32)
    P = np.zeros((n, n), dtype=np.float32)
    P[perm, np.arange(n)] = sign  # column j of A*P is sign[j] * column perm[j] of A
    capi.sgemm_nn(Ad, to_dev(P, dev), C, n, n, n)
    assert np.array_equal(to_np(C), A[:, perm] * sign[None, :])
    # and the transposed-operand forms on the same inputs give the same matrix as the NN form, to rounding
    Ct = _empty(dev, n, n)
    capi.sgemm_tn(to_dev(np.ascontiguousarray(A.T), dev), to_dev(P, dev), Ct, n, n, n)
    assert np.array_equal(to_np(Ct), to_np(C))
    capi.sgemm_nt(Ad, to_dev(np.ascontiguousarray(P.T), dev), Ct, n, n, n)
    assert np.array_equal(to_np(Ct), to_np(C))


def rng_perm(seed, n):
    return np.random.default_rng(seed).permutation(n)


def test_dense_sweep_configuration_full_size(dev):
    """benchmark configuration 5: batch 256 through FC 4096 -> 4096 in the forward (NT), data-gradient (NN) and
    weight-gradient (TN) forms, plus the tall-skinny im2col product 32768 x 64 x 576; uniform[-1,1], fixed seeds."""
    capi, orc = _capi(), _oracle()
    batch, IN, OUT = 256, 4096, 4096
    X, W, b, dY = uniform(1, batch, IN), uniform(2, OUT, IN), uniform(3, OUT), uniform(4, batch, OUT)
    Xd, Wd, dYd = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev)
    Y = _empty(dev, batch, OUT)
    capi.linear_fwd(Xd, Wd, to_dev(b, dev), Y, batch, IN, OUT)
    assert_close(to_np(Y), orc.linear(X, W, b, threads=16), IN, "linear 256x4096x4096")
    dX = _empty(dev, batch, IN)
    capi.linear_dgrad(dYd, Wd, dX, batch, IN, OUT)
    assert_close(to_np(dX), orc.linearXGrad(dY, W, threads=16), OUT, "linearXGrad 256x4096x4096")
    dW0, dB0 = uniform(5, OUT, IN), uniform(6, OUT)
    dW, dB = to_dev(dW0, dev), to_dev(dB0, dev)
    capi.linear_wgrad(dYd, Xd, dW, dB, batch, IN, OUT)
    rW, rB = orc.linearParamGrad(dY, X, dW0, dB0, threads=16)
    assert_close(to_np(dW), rW, batch, "linearParamGrad dW 4096x4096x256")
    assert_close(to_np(dB), rB, batch, "linearParamGrad dB")
    run_nn(dev, 32768, 64, 576, 1, seed=9)


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (260, 132, 516), (64, 1024, 2048), (2048, 2048, 256)])
def test_gemm_operands_aligned_to_4_bytes_only(dev, M, N, K):
    """Every operand one float past a 16-byte boundary, sizes that would otherwise take the 16-byte-load paths."""
    import torch
    capi, orc = _capi(), _oracle()

    def shifted(a):
        buf = torch.empty(a.size + 1, dtype=torch.float32, device=dev)
        v = buf[1:].view(*a.shape)
        v.copy_(to_dev(a, dev))
        assert v.data_ptr() % 16 == 4
        return v

    A, B, Bt, At = uniform(1, M, K), uniform(2, K, N), uniform(3, N, K), uniform(4, K, M)
    C = shifted(np.full((M, N), np.nan, np.float32))
    capi.sgemm_nn(shifted(A), shifted(B), C, M, N, K)
    assert_close(to_np(C), orc.sgemm(A, B, threads=8), K, "nn, 4-byte aligned")
    capi.sgemm_nt(shifted(A), shifted(Bt), C, M, N, K)
    assert_close(to_np(C), orc.sgemmNT(A, Bt, threads=8), K, "nt, 4-byte aligned")
    capi.sgemm_tn(shifted(At), shifted(B), C, M, N, K)
    assert_close(to_np(C), orc.sgemmTN(At, B, threads=8), K, "tn, 4-byte aligned")
    C0 = uniform(5, M, N)
    Cacc = shifted(C0)
    capi.sgemm_nta(shifted(A[None]), shifted(Bt[None]), Cacc, M, N, K, 1)
    assert_close(to_np(Cacc), orc.sgemmNTA(A[None], Bt[None], C0, threads=8), K, "nta, 4-byte aligned")
    bias = uniform(6, N)
    Y = shifted(np.full((M, N), np.nan, np.float32))
    capi.linear_fwd(shifted(A), shifted(Bt), shifted(bias), Y, M, K, N)
    assert_close(to_np(Y), orc.linear(A, Bt, bias, threads=8), K, "linear, 4-byte aligned")


def test_two_host_threads_on_their_own_streams(dev):
    """Two host threads issue split-K GEMMs and weight gradients at once, each on its own stream (ctypes releases the
    interpreter lock during a call): every result equals the one the same call gives alone, and an error raised in one
    thread leaves the other thread's error text alone."""
    import threading
    import torch
    capi = _capi()
    lib = capi.load()
    M, N, K = 192, 256, 4096
    g = capi.ConvGeom.make(16, 16, 32, 32, 16, 3, 3, 1, 1, 1, 1)
    A, B = to_dev(uniform(80, M, K), dev), to_dev(uniform(81, K, N), dev)
    dY, X = to_dev(uniform(82, 16, 16, 32, 32), dev), to_dev(uniform(83, 16, 16, 32, 32), dev)
    C_alone, dW_alone = _empty(dev, M, N), torch.zeros(16, 16, 3, 3, device=dev)
    capi.sgemm_nn(A, B, C_alone, M, N, K)
    capi.conv_wgrad(dY, X, dW_alone, g)
    torch.cuda.synchronize()
    failures = []

    def worker(tag):
        try:
            st = torch.cuda.Stream(device=dev)
            outs = []
            for rep in range(25):
                C, dW = _empty(dev, M, N), torch.zeros(16, 16, 3, 3, device=dev)
                with torch.cuda.stream(st):  # allocations above are on the default stream and complete; work goes to st
                    capi.sgemm_nn(A, B, C, M, N, K, stream=st)
                    capi.conv_wgrad(dY, X, dW, g, stream=st)
                outs.append((C, dW))
                if rep == 10:  # a failing call in this thread: its text must be this thread's
                    assert lib.crb_sgemm_nn(None, B.data_ptr(), C.data_ptr(), M, N, K, 1, None) == capi.CRB_ENULL
                    assert b"crb_sgemm_nn" in lib.crb_last_error_string()
            st.synchronize()
            for C, dW in outs:
                if not (torch.equal(C, C_alone) and torch.equal(dW, dW_alone)):
                    failures.append(tag)
                    break
        except Exception as e:  # surfaced in the main thread below
            failures.append(f"{tag}: {e!r}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures
