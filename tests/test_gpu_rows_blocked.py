"""The blocked closed form (layers that saw 129 .. ~1000 calibration rows: factor and sweep from
the rows as 128-column products on the matrix pipe) against dense float64 algebra.

As in test_gpu_lowrank the closed forms are pinned by the dense computation they replace, not by
a retyped formula: the lower factor M of D + B^T B (H = M^T M, numpy float64 Cholesky of the
index-reversed matrix) gives M[k,t] / M[k,k], which must equal HmT[:, k] . B[:, t] left of k's
block and -V inside it; the sweep is compared with a float64 column-by-column GPTQ on the dense
upper factor of inv(H), the reference's own form (gptq.py:160-164, solver.cu:9-154).
"""
import numpy as np
import pytest
import torch

import oracle
from test_gpu_lowrank import _lower_factor, _float64_gptq

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rows_problem(C, n, seed, dead=()):
    """BT [n, C]: sqrt(2/n) x rows with an activation-ordered spread; D [C]."""
    g = torch.Generator().manual_seed(seed)
    BT = torch.randn(n, C, generator=g) * (2.0 / n) ** 0.5
    BT *= torch.linspace(2.0, 0.5, C)[None, :]
    D = torch.full((C,), 0.01 * float((BT.double() ** 2).sum(0).mean()))
    for k in dead:
        BT[:, k] = 0
        D[k] += 1.0
    return BT, D


def _batch(C, ns, seed0, dead=()):
    nmax = max((n + 127) // 128 * 128 for n in ns)
    BT = torch.zeros(len(ns), nmax, C)
    D = torch.zeros(len(ns), C)
    for b, n in enumerate(ns):
        BT[b, :n], D[b] = _rows_problem(C, n, seed0 + b, dead if b == 1 else ())
    n_rows = torch.tensor([(n + 127) // 128 * 128 for n in ns], dtype=torch.int32)
    return BT, D, n_rows


@pytest.mark.parametrize("C,ns", [(512, (130, 300, 512, 1000)), (1024, (256, 129, 700)),
                                  (384, (200,) * 8)])
def test_blocked_factor_matches_the_dense_float64_factor(hip, C, ns):
    """Mixed row counts in one batch (each matrix's products stop at its own multiple of 128),
    pruned columns in one of them, and a batch of eight (the XCD-aware workgroup map)."""
    BT, D, n_rows = _batch(C, ns, 40, dead=(5, C - 130))
    HmT, V, info = hip.rows_factor_blocked(BT.to(DEV), D.to(DEV), n_rows.to(DEV))
    assert info.cpu().tolist() == [0] * len(ns)
    worst = 0.0
    for b, n in enumerate(ns):
        Bd = BT[b].double().numpy()
        H = np.diag(D[b].double().numpy()) + Bd.T @ Bd
        M = _lower_factor(H)
        want = np.tril(M / np.diag(M)[:, None], -1)               # [k, t], t < k
        nb = int(n_rows[b])
        got = HmT[b, :nb].cpu().double().numpy().T @ Bd[:nb]      # h_k . b_t
        Vb = V[b].cpu().double().numpy()                          # [t, k - c0]
        scale = max(1.0, float(np.abs(want).max()))
        for c0 in range(0, C, 128):
            if c0:
                worst = max(worst, np.abs(got[c0:c0 + 128, :c0] - want[c0:c0 + 128, :c0]).max() / scale)
            blk = -Vb[c0:c0 + 128].T                              # [k, t] of the block
            assert not np.triu(blk, 0).any()                      # nothing on or above the diagonal
            worst = max(worst, np.abs(blk - want[c0:c0 + 128, c0:c0 + 128]).max() / scale)
    print(f"C={C} ns={ns}: largest deviation from the float64 factor {worst:.2e}")
    # an fp32 Cholesky factorisation of the C x C matrix is 1-5e-5 from the float64 one here
    assert worst <= 2e-5


def test_blocked_factor_flags_a_pivot_that_is_not_positive(hip):
    BT, D, n_rows = _batch(256, (150, 150, 150), 7)
    D[1, 200] = -1e9
    HmT, V, info = hip.rows_factor_blocked(BT.to(DEV), D.to(DEV), n_rows.to(DEV))
    info = info.cpu().tolist()
    assert info[0] == 0 and info[2] == 0 and info[1] != 0
    assert not HmT[1].any() and not V[1].any() and HmT[0].any() and V[2].any()


@pytest.mark.parametrize("n,dtype", [(130, torch.bfloat16), (256, torch.float32), (300, torch.bfloat16)])
def test_blocked_sweep_matches_float64_gptq_on_the_dense_factor(hip, n, dtype):
    C, R, gs = 384, 256, 128
    G = C // gs
    BT, D, n_rows = _batch(C, (n, n + 100), 11)
    g = torch.Generator().manual_seed(5)
    W = (0.02 * torch.randn(2, R, C, generator=g)).to(dtype)
    s, z = oracle.build_group_meta_packed(W.float().reshape(2 * R * G, gs), 4, False)
    perm = torch.randperm(C, generator=g)                    # groups follow an arbitrary order
    g_idx = (perm // gs).to(torch.int32)
    W0 = W[:, :, perm].transpose(1, 2).contiguous()          # [2, C, R] solver order
    sT = s.view(2, R, G).transpose(1, 2).contiguous()
    zT = z.view(2, R, G).transpose(1, 2).contiguous()
    HmT, V, info = hip.rows_factor_blocked(BT.to(DEV), D.to(DEV), n_rows.to(DEV))
    assert info.cpu().tolist() == [0, 0]
    Bp = BT.transpose(1, 2).contiguous()
    X = W0.float().to(DEV)
    q = hip.gptq_sweep_rows_blocked(X, W0.to(DEV), HmT, Bp.to(DEV), V, n_rows.to(DEV), sT.to(DEV),
                                    zT.to(DEV), g_idx[None].expand(2, C).contiguous().to(DEV), 4).cpu()
    for b in range(2):
        Bd = BT[b].double().numpy()
        H = np.diag(D[b].double().numpy()) + Bd.T @ Bd
        se = sT[b][g_idx.long()].t().double().numpy()        # [R, C] per element, solver order
        ze = zT[b][g_idx.long()].t().double().numpy()
        Q, margin = _float64_gptq(W0[b].t().double().numpy(), H, se, ze)
        diff = q[b].t().double().numpy() != Q
        print(f"n={n} matrix {b}: {diff.mean():.2e} of the codes differ from float64 GPTQ")
        # fp32 against float64: rows may part ways at a near-tie and then stay apart; up to the
        # first difference of a row everything must agree, and that first difference must be a
        # near-tie of the rounding
        for r in np.nonzero(diff.any(1))[0]:
            c = int(np.argmax(diff[r]))
            assert margin[r, c] < 1e-3, (b, r, c, margin[r, c])
        assert diff.any(1).mean() <= 0.05
        # what is left in X: the displacements w0 - deq of the codes that were chosen
        deq = (q[b].float() - zT[b][g_idx.long()]) * sT[b][g_idx.long()]
        assert torch.allclose(X[b].cpu(), W0[b].float() - deq, atol=1e-6)
