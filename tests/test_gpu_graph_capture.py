"""The entry points of a training step recorded into a HIP graph and replayed.

None of them allocates or synchronises when the caller brings the workspace (and the split scratch of the others has been
grown by an earlier eager call), so a stream capture can record them. Each replay is checked against the eager result,
with eager work and synchronisations between the replays.
"""
import numpy as np
import pytest

from tests.util import he_normal, normal, to_dev

pytestmark = pytest.mark.gpu


def test_conv_step_replays_from_a_graph(dev):
    import torch
    from crusaderbackend_amd import capi
    shapes = [(32, 16, 32, 16, 1), (32, 32, 16, 32, 1), (32, 16, 32, 32, 2), (32, 8, 12, 8, 1)]  # (N, IC, H, OC, stride); 12x12 images have no sliced form
    layers = []
    for i, (N, IC, H, OC, s) in enumerate(shapes):
        g = capi.ConvGeom.make(N, IC, H, H, OC, 3, 3, s, s, 1, 1)
        L = dict(g=g, X=to_dev(normal(10 + i, N, IC, H, H), dev), W=to_dev(he_normal(20 + i, OC, IC, 3, 3), dev),
                 b=to_dev(normal(30 + i, OC), dev), dY=to_dev(normal(40 + i, N, OC, g.OH, g.OW), dev),
                 Y=torch.empty(N, OC, g.OH, g.OW, device=dev), dX=torch.empty(N, IC, H, H, device=dev),
                 dW=torch.zeros(OC, IC, 3, 3, device=dev),
                 ws=torch.empty(max(capi.conv_wgrad_workspace_bytes(g) // 4, 4), device=dev), n=capi.conv_bwd_slices(g))
        layers.append(L)
    sliced = [L for L in layers if L["n"]]
    assert sliced and len(sliced) < len(layers)  # both kinds of layer are in the step
    table = capi.slice_sum_table([(L["ws"], L["dW"], L["n"]) for L in sliced])

    def step(stream):
        for L in layers:
            capi.tensor_fill(L["dW"], 0.0, L["dW"].numel(), stream=stream)  # a fill kernel, not a memset node
            capi.conv_fwd(L["W"], L["X"], L["Y"], L["b"], L["g"], flags=capi.CRB_FLAG_RELU, stream=stream)
        for L in reversed(layers):
            if L["n"]:
                capi.conv_bwd_sliced(L["W"], L["dY"], L["X"], L["dX"], L["g"], L["ws"], stream=stream)
            else:
                capi.conv_bwd(L["W"], L["dY"], L["X"], L["dX"], L["dW"], L["g"], workspace=L["ws"], stream=stream)
        capi.sum_slices_multi(table, stream=stream)

    step(None)  # eager: the results to reproduce (and any library scratch grown)
    torch.cuda.synchronize()
    want = [{k: L[k].clone() for k in ("Y", "dX", "dW")} for L in layers]

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(torch.cuda.current_stream())
    torch.cuda.synchronize()

    for replay in range(4):
        for L in layers:  # eager work between the replays: spoil every output
            L["Y"].fill_(float("nan")), L["dX"].fill_(float("nan")), L["dW"].fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for L, w in zip(layers, want):
            for k in ("Y", "dX", "dW"):
                assert torch.equal(L[k], w[k]), (replay, k, tuple(L[k].shape))
