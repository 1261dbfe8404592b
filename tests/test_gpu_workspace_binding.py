"""Split scratch from a block the caller binds to the stream (crb_bind_workspace): no entry point allocates while a block
is bound, the *_workspace_bytes queries say what a call needs, too small a block is refused, and a dense layer whose
contraction is cut records into a HIP graph without any earlier eager call."""
import numpy as np
import pytest

from oracle import seblas_oracle as orc
from tests.util import assert_close, he_normal, normal, to_dev, to_np, uniform

pytestmark = pytest.mark.gpu


def test_linear_fwd_needing_a_split_records_into_a_graph_without_warmup(dev):
    import torch
    from crusaderbackend_amd import capi

    batch, IN, OUT = 128, 2048, 40  # 2 x 1 tiles: the contraction is cut, so the call needs scratch
    need = capi.gemm_workspace_bytes(batch, OUT, IN, 1)
    assert need > 0
    X, W, b = uniform(1, batch, IN), uniform(2, OUT, IN), uniform(3, OUT)
    Xd, Wd, bd = to_dev(X, dev), to_dev(W, dev), to_dev(b, dev)
    Y = torch.empty(batch, OUT, device=dev)
    ws = torch.empty(need // 4, device=dev)
    side = torch.cuda.Stream(device=dev)  # a fresh stream: the library holds no arena for it
    capi.bind_workspace(ws, stream=side)
    try:
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            capi.linear_fwd(Xd, Wd, bd, Y, batch, IN, OUT, stream=torch.cuda.current_stream())
        torch.cuda.synchronize()
        ref = orc.linear(X, W, b)
        for replay in range(3):
            Y.fill_(float("nan"))
            ws.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert_close(to_np(Y), ref, IN, f"linear from a graph, replay {replay}")
    finally:
        capi.bind_workspace(None, stream=side)


def test_capture_without_scratch_is_refused_not_allocated(dev):
    import torch
    from crusaderbackend_amd import capi

    batch, IN, OUT = 64, 4096, 24
    assert capi.gemm_workspace_bytes(batch, OUT, IN, 1) > 0
    Xd, Wd, bd = (to_dev(uniform(i, *s), dev) for i, s in ((1, (batch, IN)), (2, (OUT, IN)), (3, (OUT,))))
    Y = torch.empty(batch, OUT, device=dev)
    side = torch.cuda.Stream(device=dev)  # fresh stream, nothing bound, arena empty
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        with pytest.raises(capi.CrbError) as ei:
            capi.linear_fwd(Xd, Wd, bd, Y, batch, IN, OUT, stream=torch.cuda.current_stream())
        capi.tensor_fill(Y, 1.0, Y.numel(), stream=torch.cuda.current_stream())  # the capture itself stays valid
    assert ei.value.status == capi.CRB_EWORKSPACE and "captured" in str(ei.value)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.all(Y == 1.0)


def test_bound_workspace_too_small_is_refused_and_exact_size_works(dev):
    import torch
    from crusaderbackend_amd import capi

    s = torch.cuda.Stream(device=dev)
    M, N, K = 96, 80, 3000
    need = capi.gemm_workspace_bytes(M, N, K, 1)
    assert need > 0
    A, B = uniform(4, M, K), uniform(5, K, N)
    Ad, Bd = to_dev(A, dev), to_dev(B, dev)
    C = torch.empty(M, N, device=dev)
    small = torch.empty(need // 4 - 64, device=dev)
    exact = torch.empty(need // 4, device=dev)
    torch.cuda.synchronize()
    try:
        capi.bind_workspace(small, stream=s)
        with pytest.raises(capi.CrbError) as ei:
            capi.sgemm_nn(Ad, Bd, C, M, N, K, stream=s)
        assert ei.value.status == capi.CRB_EWORKSPACE
        capi.bind_workspace(exact, stream=s)
        capi.sgemm_nn(Ad, Bd, C, M, N, K, stream=s)
        s.synchronize()
        assert_close(to_np(C), orc.sgemm(A, B), K, "sgemm on a bound workspace")
        # the other forms of the family on the same shapes
        At = to_dev(np.ascontiguousarray(A.T), dev)
        capi.sgemm_tn(At, Bd, C, M, N, K, stream=s)
        s.synchronize()
        assert_close(to_np(C), orc.sgemm(A, B), K, "sgemmTN on a bound workspace")
    finally:
        capi.bind_workspace(None, stream=s)
    with pytest.raises(capi.CrbError):
        capi.bind_workspace(exact[1:], stream=s)  # not 256-byte aligned


def test_conv_queries_and_general_path_on_a_bound_workspace(dev):
    import torch
    from crusaderbackend_amd import capi

    s = torch.cuda.Stream(device=dev)
    # shapes with kernels of their own need nothing
    for (N, IC, H, OC, F, st, p) in ((128, 16, 32, 16, 3, 1, 1), (128, 16, 32, 32, 3, 2, 1), (64, 204, 32, 48, 1, 1, 0)):
        g = capi.ConvGeom.make(N, IC, H, H, OC, F, F, st, st, p, p)
        assert capi.conv_fwd_workspace_bytes(g) == 0 and capi.conv_dgrad_workspace_bytes(g) == 0
    # 5x5 filters with pad 1 on 12x12 images (no kernel of their own), few pixels: the general path cuts the contraction
    N, IC, H, OC = 4, 64, 12, 48
    g = capi.ConvGeom.make(N, IC, H, H, OC, 5, 5, 1, 1, 1, 1)
    OH = g.OH
    nf, nd, nw, nb = (capi.conv_fwd_workspace_bytes(g), capi.conv_dgrad_workspace_bytes(g), capi.conv_wgrad_workspace_bytes(g),
                      capi.conv_bias_grad_workspace_bytes(N, OC, OH * OH))
    assert nf > 0 and nd > 0 and nw > 0 and nb > 0
    X, W, dY, b = normal(1, N, IC, H, H), he_normal(2, OC, IC, 5, 5), normal(3, N, OC, OH, OH), normal(4, OC)
    Xd, Wd, dYd, bd = to_dev(X, dev), to_dev(W, dev), to_dev(dY, dev), to_dev(b, dev)
    Y, dX = torch.empty(N, OC, OH, OH, device=dev), torch.empty(N, IC, H, H, device=dev)
    dW, dB = torch.zeros(OC, IC, 5, 5, device=dev), torch.zeros(OC, device=dev)
    ws = torch.empty(max(nf, nd, nw, nb) // 4, device=dev)
    torch.cuda.synchronize()
    try:
        capi.bind_workspace(ws, stream=s)
        capi.conv_fwd(Wd, Xd, Y, bd, g, stream=s)
        capi.conv_dgrad(Wd, dYd, dX, g, stream=s)
        capi.conv_wgrad(dYd, Xd, dW, g, stream=s)  # workspace argument NULL: the bound block serves it
        capi.conv_bias_grad(dYd, dB, N, OC, OH * OH, stream=s)
        s.synchronize()
    finally:
        capi.bind_workspace(None, stream=s)
    assert_close(to_np(Y), orc.conv(W, X, b, 1, 1, 1, 1), IC * 25, "conv fwd (bound workspace)")
    assert_close(to_np(dX), orc.convDerive(W, dY, (H, H), 1, 1, 1, 1), OC * 25, "conv dgrad (bound workspace)")
    assert_close(to_np(dW), orc.convError(dY, X, np.zeros_like(W), 1, 1, 1, 1), N * OH * OH, "conv wgrad (bound workspace)")
    assert_close(to_np(dB), dY.astype(np.float64).sum(axis=(0, 2, 3)), N * OH * OH, "conv bias grad (bound workspace)")


def test_pointwise_wgrad_honours_the_workspace_argument(dev):
    import torch
    from crusaderbackend_amd import capi

    N, IC, H, OC = 64, 24, 16, 48  # 1x1: the accumulate-NT GEMM form, one tile, contraction of 16384: cut
    g = capi.ConvGeom.make(N, IC, H, H, OC, 1, 1)
    need = capi.conv_wgrad_workspace_bytes(g)
    assert need > 0
    X, dY = normal(1, N, IC, H, H), normal(2, N, OC, H, H)
    dW = torch.zeros(OC, IC, 1, 1, device=dev)
    ws = torch.empty(need // 4, device=dev)
    capi.conv_wgrad(to_dev(dY, dev), to_dev(X, dev), dW, g, workspace=ws)
    torch.cuda.synchronize()
    assert_close(to_np(dW), orc.convError(dY, X, np.zeros((OC, IC, 1, 1), np.float32), 1, 1, 0, 0), N * H * H, "1x1 wgrad")
    with pytest.raises(capi.CrbError) as ei:
        capi.conv_wgrad(to_dev(dY, dev), to_dev(X, dev), dW, g, workspace=ws[: need // 8])
    assert ei.value.status == capi.CRB_EWORKSPACE


# (N, IC, H, OC, F, stride, pad, operands 16-byte aligned): 2x2 images (products over (channel, pixel) pairs on the tiled
# engine), 1x1 layers the batched GEMM forms take (odd image size; operands off the 16-byte grid), the general gather path,
# direct-kernel shapes on operands off the grid (which then take the general path too)
EXACT_SHAPES = [(128, 64, 2, 64, 3, 1, 1, True), (128, 512, 2, 512, 3, 1, 1, True), (8, 40, 2, 24, 3, 1, 1, True),
                (64, 24, 16, 48, 1, 1, 0, False), (4, 96, 7, 40, 1, 1, 0, True), (2, 300, 6, 20, 1, 1, 0, False),
                (2, 64, 12, 48, 5, 1, 2, True), (3, 20, 9, 12, 3, 2, 1, True), (16, 16, 32, 16, 3, 1, 1, False),
                (8, 16, 16, 32, 1, 2, 0, True), (4, 40, 14, 48, 3, 1, 1, True), (3, 24, 20, 70, 3, 1, 1, False), (2, 16, 15, 24, 3, 2, 1, True)]


@pytest.mark.parametrize("shape", EXACT_SHAPES, ids=lambda s: "x".join(map(str, s[:7])) + ("" if s[7] else "-unaligned"))
def test_a_workspace_of_exactly_the_queried_size_serves_every_conv_entry_point(dev, shape):
    """What the *_workspace_bytes queries return is what a call needs: each entry point runs on a bound block of exactly
    that size (a bound block is never grown, so a query that under-reports shows as CRB_EWORKSPACE)."""
    import torch
    from crusaderbackend_amd import capi

    N, IC, H, OC, F, st, p, aligned = shape
    g = capi.ConvGeom.make(N, IC, H, H, OC, F, F, st, st, p, p)
    X, W, dY, b = normal(1, N, IC, H, H), he_normal(2, OC, IC, F, F), normal(3, N, OC, g.OH, g.OW), normal(4, OC)

    def place(a):  # aligned: as allocated; otherwise 4 bytes past a 16-byte boundary
        if aligned:
            return to_dev(a, dev)
        buf = torch.empty(a.size + 1, device=dev)
        buf[1:].copy_(torch.from_numpy(a.reshape(-1)))
        return buf[1:].view(*a.shape)

    Xd, Wd, dYd, bd = place(X), to_dev(W, dev), place(dY), to_dev(b, dev)
    Y, dX = place(np.zeros_like(dY)), place(np.zeros_like(X))
    dW = torch.zeros(OC, IC, F, F, device=dev)
    s = torch.cuda.Stream(device=dev)
    need = {"fwd": capi.conv_fwd_workspace_bytes(g, aligned), "dgrad": capi.conv_dgrad_workspace_bytes(g, aligned),
            "wgrad": capi.conv_wgrad_workspace_bytes(g)}
    torch.cuda.synchronize()
    try:
        for name in ("fwd", "dgrad", "wgrad"):
            ws = torch.empty(max(need[name], 256) // 4, device=dev)  # nothing needed: a token block, still never grown
            capi.bind_workspace(ws, stream=s)
            if name == "fwd":
                capi.conv_fwd(Wd, Xd, Y, bd, g, stream=s)
            elif name == "dgrad":
                capi.conv_dgrad(Wd, dYd, dX, g, stream=s)
            else:
                capi.conv_wgrad(dYd, Xd, dW, g, stream=s)
            s.synchronize()
    finally:
        capi.bind_workspace(None, stream=s)
    assert_close(to_np(Y), orc.conv(W, X, b, st, st, p, p), IC * F * F, f"conv fwd {shape}")
    assert_close(to_np(dX), orc.convDerive(W, dY, (H, H), st, st, p, p), OC * F * F, f"conv dgrad {shape}")
    assert_close(to_np(dW), orc.convError(dY, X, np.zeros_like(W), st, st, p, p), N * g.OH * g.OW, f"conv wgrad {shape}")
