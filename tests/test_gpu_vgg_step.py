"""End-to-end parity of a whole training step (convolutions, ReLU, pooling, dense layers, softmax, cross-entropy,
momentum update) driven through the C ABI, against the same step replayed with the CPU oracle on identical values.

Per-operator parity is covered elsewhere to the 1e-5*sqrt(K) bound; here rounding differences travel through up to
16 layers, so the comparison is on the relative L2 error of each tensor (bound 2e-4), and the loss to 1e-4 relative.
"""
import numpy as np
import pytest

from tests.util import to_np

pytestmark = pytest.mark.gpu


def cpu_step(orc, net, x, labels, params, threads=8):
    """The same call sequence as Vgg16Step.step(), on numpy arrays with the oracle's operators."""
    B = net.batch
    acts, cur = [], x
    convs = [p for p in params[:len(params) - len(net.fc)]]
    ci = 0
    for kind, st in net.stages:
        if kind == "conv":
            p = convs[ci]
            ci += 1
            z = orc.conv(p["W"], cur, p["b"], 1, 1, 1, 1, threads=threads)
            out = orc.relu(z)
            acts.append(("conv", p, cur, z, out))
        else:
            out, rec = orc.maxPool(cur, 2, 2)
            acts.append(("pool", rec, cur, None, out))
        cur = out
    cur = cur.reshape(B, -1)
    fcs = []
    for st, p in zip(net.fc, params[len(params) - len(net.fc):]):
        z = orc.linear(cur, p["W"], p["b"], threads=threads)
        out = orc.relu(z) if st["relu"] else z
        fcs.append((st, p, cur, z, out))
        cur = out
    probs = orc.softmax(cur, net.classes)
    loss = orc.crossEntropyCalc(probs, labels)
    d = orc.crossEntropyLoss(probs, labels)
    for st, p, xin, z, out in reversed(fcs):
        dz = orc.reluGradFast(z, d) if st["relu"] else d
        d = orc.linearXGrad(dz, p["W"], threads=threads)
        p["dW"], p["dB"] = orc.linearParamGrad(dz, xin, p["dW"], p["dB"], threads=threads)
    for kind, p, xin, z, out in reversed(acts):
        d = d.reshape(out.shape)
        if kind == "pool":
            d, _ = orc.maxPoolBack(d, p, xin.shape[2:], 2, 2)
        else:
            dz = orc.reluGradFast(z, d)
            d = orc.convDerive(p["W"], dz, xin.shape[2:], 1, 1, 1, 1, threads=threads)
            p["dW"] = orc.convError(dz, xin, p["dW"], 1, 1, 1, 1, threads=threads)
            p["dB"] = p["dB"] + dz.sum(axis=(0, 2, 3), dtype=np.float64).astype(np.float32)
    grads = [{"dW": p["dW"].copy(), "dB": p["dB"].copy()} for p in params]
    for p in params:
        p["W"], p["dW"], p["mW"] = [a.reshape(p["W"].shape) for a in
                                    orc.momentumApply(p["W"], p["dW"], p["mW"], net.lr, net.beta, 1.0 - net.l2)]
        p["b"], p["dB"], p["mB"] = orc.momentumApply(p["b"], p["dB"], p["mB"], net.lr, net.beta, 1.0)
    return probs, loss, d, grads


def rel_l2(got, ref):
    got, ref = np.asarray(got, np.float64).ravel(), np.asarray(ref, np.float64).ravel()
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))


@pytest.mark.parametrize("name,kw", [
    ("small", dict(batch=6, image=8, cfg=(8, "M", 16, 16, "M", 32, "M"), hidden=24)),
    ("vgg16", dict(batch=4, image=32)),
])
def test_training_step_matches_cpu_replica(dev, name, kw):
    import torch
    from crusaderbackend_amd import capi
    from crusaderbackend_amd.vgg16_step import Vgg16Step
    from oracle import seblas_oracle as orc

    net = Vgg16Step(torch, capi, dev, seed=7, **kw)
    params = net.params()
    x, labels = to_np(net.x), to_np(net.labels)
    # a non-trivial momentum state, so the update is not just a scaled gradient
    rng = np.random.default_rng(3)
    for st, p in zip(net.layers(), params):
        for k in ("mW", "mB"):
            p[k] = (rng.standard_normal(p[k].shape) * 1e-3).astype(np.float32)
            st[k].copy_(torch.from_numpy(p[k]))
    net.step()
    torch.cuda.synchronize()
    probs, loss, dx, grads = cpu_step(orc, net, x, labels, params)

    bound = 2e-4
    assert rel_l2(to_np(net.probs), probs) <= bound
    assert abs(float(to_np(net.loss)[0]) - loss) <= 1e-4 * abs(loss)
    assert rel_l2(to_np(net.dx), dx) <= bound
    for i, (st, p) in enumerate(zip(net.layers(), params)):
        for k in ("W", "b", "mW", "mB"):
            assert rel_l2(to_np(st[k]), p[k]) <= bound, f"{name}: layer {i} {k}"
        assert not to_np(st["dW"]).any() and not to_np(st["dB"]).any()  # gradients are cleared by the update
    # the momentum buffers carry the gradients: m_new = beta*m_old + (1-beta)*g
    for i, (st, g) in enumerate(zip(net.layers(), grads)):
        assert np.isfinite(g["dW"]).all() and np.abs(g["dW"]).max() > 0, f"{name}: layer {i} has a zero gradient"
