"""Shared helpers of the parity tests."""
import math

import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def uniform(seed, *shape):
    """uniform[-1,1] fp32, fixed seed."""
    return rng(seed).uniform(-1.0, 1.0, size=shape).astype(np.float32)


def normal(seed, *shape, std=1.0):
    return (rng(seed).standard_normal(size=shape) * std).astype(np.float32)


def he_normal(seed, OC, IC, FH, FW):
    """conv filter init of the reference: N(0, sqrt(2/(IC*FH*FW))) (seann/operands/seblas/Conv2D.cu:45-50)."""
    return normal(seed, OC, IC, FH, FW, std=math.sqrt(2.0 / (IC * FH * FW)))


def tolerance(ref, K):
    """Per-element bound 1e-5*sqrt(K)*max(|ref|, rms(ref)): accumulation order differs between CPU and GPU."""
    ref = np.asarray(ref, dtype=np.float64)
    rms = math.sqrt(float(np.mean(ref * ref))) if ref.size else 0.0
    return 1e-5 * math.sqrt(max(K, 1)) * np.maximum(np.abs(ref), rms)


# worst err / tol seen per checked quantity in this process (written out by conftest at the end of a GPU session)
MARGINS = {}


def assert_close(got, ref, K, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref64 = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref64.shape, f"{what}: shape {got.shape} vs {ref64.shape}"
    assert np.all(np.isfinite(got)), f"{what}: non-finite values"
    err = np.abs(got - ref64)
    tol = tolerance(ref64, K)
    if err.size:
        with np.errstate(divide="ignore", invalid="ignore"):
            ratio = float(np.nanmax(np.where(tol > 0, err / tol, 0.0)))
            # the same error against the plain relative bound 1e-5*sqrt(K)*|ref| (no RMS floor), on elements that are not tiny
            big = np.abs(ref64) >= 1e-3 * (np.sqrt(np.mean(ref64 * ref64)) + 1e-300)
            rel = float(np.max(err[big] / (1e-5 * math.sqrt(max(K, 1)) * np.abs(ref64[big])))) if big.any() else 0.0
        old = MARGINS.get(what)
        if old is None or ratio > old["err_over_tol"]:
            MARGINS[what] = {"err_over_tol": ratio, "err_over_plain_relative_bound": rel, "K": int(K), "elements": int(err.size)}
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} elements outside 1e-5*sqrt(K={K}) tolerance; worst at {idx}: "
            f"got {got[idx]!r} ref {ref64[idx]!r} err {err[idx]:.3e} tol {tol[idx]:.3e}")


def to_dev(a, dev):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def to_np(t):
    return t.detach().cpu().numpy()
