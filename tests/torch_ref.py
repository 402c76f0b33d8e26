"""Independent fp64 torch restatements of the FORWARD maths only.

Backward and second-order formulas of the oracle are pinned by running torch
autograd (and double backward) through these forwards; nothing here re-types a
backward formula.
"""
import numpy as np
import torch


def grid_forward(params, xyz, scale, offset, idx):
    """params: (n_params,) f64 tensor; xyz: (3, N) f64 tensor (may require grad);
    idx: (L, 8, N) integer entry indices (pinned separately as integers).
    Returns (2L, N).  Weights are built from xyz so autograd sees d/dxyz.
    """
    L = idx.shape[0]
    P = params.view(-1, 2)
    outs = []
    for l in range(L):
        pos = xyz * float(scale[l]) + 0.5
        w = pos - torch.floor(pos).detach()
        acc = 0
        for k in range(8):
            wt = 1
            for d in range(3):
                wt = wt * (w[d] if (k >> d) & 1 else (1 - w[d]))
            e = torch.as_tensor(idx[l, k].astype(np.int64)) + int(offset[l])
            acc = acc + wt[:, None] * P[e]
        outs.append(acc.t())
    return torch.cat(outs, 0)


def mlp_forward(Ws, x):
    """Ws: list of (out, in) f64 tensors; x: (in, N).  ReLU hidden, linear out."""
    h = x
    for W in Ws[:-1]:
        h = torch.relu(W @ h)
    return Ws[-1] @ h
