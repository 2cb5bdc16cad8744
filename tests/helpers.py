"""Shared builders for the parity tests."""
import numpy as np
import torch

import oracle
from oracle import mathref


def linear(W):
    lin = torch.nn.Linear(W.shape[1], W.shape[0], bias=False)
    lin.weight.data = W.clone()
    return lin


def expand_meta(v, R, C, gs):
    """flat [R*G] per-group meta -> per element [C, R] (identity order)."""
    G = (C + gs - 1) // gs
    return v.view(R, G).repeat_interleave(gs, dim=1)[:, :C].t().contiguous()


def random_problem(C, R, n=None, sym=True, gs=128, seed=0, outliers=3, mse=False):
    """W [R,C], per-element meta [C,R], normalised U from a float64 factorisation."""
    g = torch.Generator().manual_seed(seed)
    W = 0.02 * torch.randn(R, C, generator=g)
    X = torch.randn(n or 2 * C, C, generator=g)
    X[:, :outliers] *= 10
    H = (2.0 / X.shape[0]) * X.T @ X
    U = torch.from_numpy(mathref.factor(H.double().numpy(), 0.01)).float().contiguous()
    G = (C + gs - 1) // gs
    Wp = torch.nn.functional.pad(W, (0, G * gs - C))
    s, z = oracle.build_group_meta_packed(Wp.reshape(R * G, gs), 4, sym)
    if mse:
        p = torch.linspace(1.0, 0.2, 100)
        oracle.mse_scale_groups_packed(Wp.reshape(R * G, gs), s, z, p, 2.4, 4, sym)
    return dict(W=W, X=X, H=H, U=U, s=s, z=z, se=expand_meta(s, R, C, gs), ze=expand_meta(z, R, C, gs),
                G=G, gs=gs)


def flip_rate(a, b):
    return (a.cpu() != b.cpu()).float().mean().item()
