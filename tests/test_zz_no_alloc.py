"""crb_conv_wgrad_noalloc: the weight gradient on the library's built-in scratch buffer.

Same kernels and split plan as crb_conv_wgrad, so results must be bit-identical to it; two calls in a row share the one
buffer (the second, smaller, call must not see the first call's slices); geometries beyond the buffer are refused."""
import numpy as np
import pytest

from oracle import seblas_oracle as orc
from tests.util import assert_close, he_normal, normal, to_dev, to_np

pytestmark = pytest.mark.gpu


def _pair(dev, N, IC, H, OC, F, s, p, seed):
    import torch
    from crusaderbackend_amd import capi

    g = capi.ConvGeom.make(N, IC, H, H, OC, F, F, s, s, p, p)
    X, dY = normal(seed, N, IC, H, H), normal(seed + 1, N, OC, g.OH, g.OW)
    dW0 = he_normal(seed + 2, OC, IC, F, F)  # accumulate contract: start from a non-zero dW
    Xd, dYd = to_dev(X, dev), to_dev(dY, dev)
    want, got = to_dev(dW0, dev), to_dev(dW0, dev)
    nbytes = capi.conv_wgrad_workspace_bytes(g)
    ws = torch.empty(max(nbytes // 4, 4), device=dev)
    capi.conv_wgrad(dYd, Xd, want, g, workspace=ws)
    return g, X, dY, dW0, Xd, dYd, want, got, nbytes


# (N, IC, H, OC, F, stride, pad): direct 3x3 at three widths, stride 2, 1x1 (GEMM form, cut contraction), 1x1 stride-2
# shortcut, 2x2 images, a 5x5 filter on the general path
SHAPES = [(128, 16, 32, 16, 3, 1, 1), (64, 32, 16, 32, 3, 1, 1), (32, 64, 8, 64, 3, 1, 1), (32, 16, 32, 32, 3, 2, 1),
          (64, 24, 16, 48, 1, 1, 0), (16, 16, 32, 32, 1, 2, 0), (64, 32, 2, 32, 3, 1, 1), (4, 12, 12, 20, 5, 1, 2)]


def test_noalloc_two_calls_in_a_row_match_conv_wgrad(dev):
    import torch
    from crusaderbackend_amd import capi

    used_scratch = 0
    for i in range(len(SHAPES) - 1):
        big, small = SHAPES[i], SHAPES[i + 1]
        if i % 2:  # second call with the smaller input: fewer images of the same layer, then the next shape
            small = (max(big[0] // 4, 1),) + big[1:]
        a = _pair(dev, *big, seed=100 + 10 * i)
        b = _pair(dev, *small, seed=105 + 10 * i)
        torch.cuda.synchronize()
        capi.conv_wgrad_noalloc(a[5], a[4], a[7], a[0])
        capi.conv_wgrad_noalloc(b[5], b[4], b[7], b[0])
        torch.cuda.synchronize()
        for (g, X, dY, dW0, _, _, want, got, nbytes), shape in ((a, big), (b, small)):
            assert torch.equal(got, want), f"noalloc != conv_wgrad for {shape}"
            used_scratch += nbytes > 0
            if shape[0] * g.OH * g.OW <= 1 << 15:  # oracle too, where it is quick
                ref = orc.convError(dY, X, dW0.copy(), shape[5], shape[5], shape[6], shape[6])
                assert_close(to_np(got), ref, shape[0] * g.OH * g.OW, f"noalloc wgrad {shape}")
    assert used_scratch >= 8  # most of the shapes do go through the buffer


def test_noalloc_second_call_repeats_bit_for_bit_and_on_a_side_stream(dev):
    import torch
    from crusaderbackend_amd import capi

    g, X, dY, dW0, Xd, dYd, want, got, _ = _pair(dev, 128, 32, 16, 32, 3, 1, 1, seed=7)
    s = torch.cuda.Stream(device=dev)
    torch.cuda.synchronize()
    capi.conv_wgrad_noalloc(dYd, Xd, got, g, stream=s)
    s.synchronize()
    assert torch.equal(got, want)
    got2 = to_dev(dW0, dev)
    capi.conv_wgrad_noalloc(dYd, Xd, got2, g)
    torch.cuda.synchronize()
    assert torch.equal(got2, want)


def test_noalloc_refuses_what_does_not_fit_and_bad_arguments(dev):
    import torch
    from crusaderbackend_amd import capi

    # 3x3 on 12x12 images, 256 -> 256 channels: the general path's slices exceed the built-in buffer
    g = capi.ConvGeom.make(64, 256, 12, 12, 256, 3, 3, 1, 1, 1, 1)
    assert capi.conv_wgrad_workspace_bytes(g) > capi.NOALLOC_SCRATCH_BYTES
    X, dY = torch.zeros(64, 256, 12, 12, device=dev), torch.zeros(64, 256, 12, 12, device=dev)
    dW = torch.zeros(256, 256, 3, 3, device=dev)
    with pytest.raises(capi.CrbError) as ei:
        capi.conv_wgrad_noalloc(dY, X, dW, g)
    assert ei.value.status == capi.CRB_EWORKSPACE and "built-in buffer" in str(ei.value)
    with pytest.raises(capi.CrbError) as ei:
        capi.conv_wgrad_noalloc(None, X, dW, g)
    assert ei.value.status == capi.CRB_ENULL
    bad = capi.ConvGeom.make(1, 1, 4, 4, 1, 3, 3, 1, 1, 0, 0, OH=3, OW=2)
    with pytest.raises(capi.CrbError) as ei:
        capi.conv_wgrad_noalloc(dY, X, dW, bad)
    assert ei.value.status == capi.CRB_EINVAL_SHAPE


def test_noalloc_records_into_a_graph_with_nothing_bound_and_no_arena(dev):
    """The property the entry point exists for: it runs where nothing may be allocated. A capture on a fresh stream (no
    workspace bound, the library holds no arena for it) refuses any growth, so an allocation would surface as
    CRB_EWORKSPACE; the graph is replayed with eager work in between and checked against crb_conv_wgrad every time.
    Shapes: a direct 3x3 layer, a 1x1 layer on the pixel-contraction kernel, and a 1x1 layer whose operands are off the
    16-byte grid (the accumulate-NT GEMM form, its split scratch served through the scope)."""
    import torch
    from crusaderbackend_amd import capi

    cases = []
    for i, (N, IC, H, OC, F, st, p, off) in enumerate(((64, 16, 32, 16, 3, 1, 1, 0), (64, 64, 16, 48, 1, 1, 0, 0), (64, 24, 16, 48, 1, 1, 0, 1))):
        g = capi.ConvGeom.make(N, IC, H, H, OC, F, F, st, st, p, p)
        X, dY, dW0 = normal(50 + i, N, IC, H, H), normal(60 + i, N, OC, g.OH, g.OW), he_normal(70 + i, OC, IC, F, F)

        def place(a):
            buf = torch.empty(a.size + off, device=dev)
            buf[off:].copy_(torch.from_numpy(a.reshape(-1)))
            return buf[off:].view(*a.shape)

        Xd, dYd = place(X), place(dY)
        assert capi.conv_wgrad_workspace_bytes(g) > 0
        want = to_dev(dW0, dev)
        ws = torch.empty(capi.conv_wgrad_workspace_bytes(g) // 4, device=dev)
        capi.conv_wgrad(dYd, Xd, want, g, workspace=ws)
        cases.append((g, Xd, dYd, dW0, want, to_dev(dW0, dev)))
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)  # fresh: nothing bound, no arena
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for g, Xd, dYd, _, _, got in cases:
            capi.conv_wgrad_noalloc(dYd, Xd, got, g, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    for replay in range(3):
        for _, _, _, dW0, _, got in cases:  # eager work between the replays: reset the accumulated-into tensors
            got.copy_(torch.from_numpy(dW0))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for g, _, _, _, want, got in cases:
            assert torch.equal(got, want), (replay, g.IC, g.OC, g.FH)
