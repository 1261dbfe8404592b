"""Writes tests/golden/conv_fixtures.npz: small convolution input/output vectors computed with torch-CPU in
float64 (conv2d and its autograd — a textbook routine, independent of both the oracle and the HIP kernels).
Run from the repository root:  python tests/golden/make_conv_fixtures.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

# (N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW)
CASES = [
    (2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1),
    (2, 4, 9, 9, 6, 3, 3, 2, 2, 1, 1),
    (1, 5, 6, 10, 3, 1, 1, 1, 1, 0, 0),
    (2, 2, 7, 7, 3, 5, 3, 1, 2, 2, 0),
    (1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1),
]


def main():
    out = {"count": np.int64(len(CASES))}
    g = torch.Generator().manual_seed(1234)
    for i, (N, IC, IH, IW, OC, FH, FW, sH, sW, pH, pW) in enumerate(CASES):
        X = torch.randn(N, IC, IH, IW, generator=g).float()
        W = torch.randn(OC, IC, FH, FW, generator=g).float()
        b = torch.randn(OC, generator=g).float()
        Xd, Wd = X.double().requires_grad_(), W.double().requires_grad_()
        Y = F.conv2d(Xd, Wd, b.double(), stride=(sH, sW), padding=(pH, pW))
        dY = torch.randn(Y.shape, generator=g).float()
        Y.backward(dY.double())
        out.update({f"{i}_geom": np.array([sH, sW, pH, pW]), f"{i}_X": X.numpy(), f"{i}_W": W.numpy(),
                    f"{i}_b": b.numpy(), f"{i}_dY": dY.numpy(), f"{i}_Y": Y.detach().numpy(),
                    f"{i}_dX": Xd.grad.numpy(), f"{i}_dW": Wd.grad.numpy()})
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv_fixtures.npz"), **out)


if __name__ == "__main__":
    main()
