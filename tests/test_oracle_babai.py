"""Pins the oracle's Babai solver (solver_babai.cu:123-322, gptq.py:107-108,157-158,231-246)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from helpers import random_problem


def _upper_factor(H, rel_damp=0.01):
    Hd = H.double().numpy().copy()
    Hd[np.diag_indices(Hd.shape[0])] += rel_damp * np.mean(np.diag(Hd))
    return torch.from_numpy(np.linalg.cholesky(Hd).T.copy()).float().contiguous()   # H = A^T A


def _problem(C, R, gs, sym=True, seed=0):
    pr = random_problem(C=C, R=R, sym=sym, gs=gs, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    perm = torch.randperm(C, generator=g)
    pr["g_idx"] = (perm // gs).to(torch.int32)
    pr["A"] = _upper_factor(pr["H"])
    return pr


def _meta_per_element(s, z, g_idx, R, G):
    """[C,R] per-element scales/zeros for solver column c of group g_idx[c]."""
    se = s.view(R, G).t()[g_idx.long()].contiguous()
    ze = z.view(R, G).t()[g_idx.long()].contiguous()
    return se, ze


@pytest.mark.parametrize("sym", [True, False])
def test_identity_factor_is_round_to_nearest(sym):
    C, R, gs = 256, 24, 128
    pr = _problem(C, R, gs, sym=sym)
    Wt = pr["W"].t().contiguous()
    q = oracle.babai_solver(Wt.clone(), torch.eye(C), pr["s"], pr["z"], gs, 4, gs // 4, pr["g_idx"], pr["G"])
    se, ze = _meta_per_element(pr["s"], pr["z"], pr["g_idx"], R, pr["G"])
    assert np.array_equal(q.numpy(), mathref.rtn(Wt.numpy(), se.numpy(), ze.numpy(), 4))


def test_float64_restatement_of_the_recurrence_agrees_away_from_ties():
    """Independent numpy/float64 form of solver_babai.cu:190-213,313-316: columns from the
    last to the first, W[:, :t] -= err_t * A[:t, t] / diag(A)[:t]."""
    C, R, gs = 64, 8, 32
    pr = _problem(C, R, gs)
    A = pr["A"].double().numpy()
    se, ze = _meta_per_element(pr["s"], pr["z"], pr["g_idx"], R, pr["G"])
    s64, z64 = se.t().double().numpy(), ze.t().double().numpy()         # [R, C]
    W = pr["W"].double().numpy().copy()
    Q = np.zeros((R, C), dtype=np.int64)
    margins = np.zeros((R, C))
    for t in range(C - 1, -1, -1):
        b = W[:, t] / (s64[:, t] + 1e-12) + z64[:, t]
        margins[:, t] = np.abs(b - np.floor(b) - 0.5)
        q = np.clip(np.rint(b), 0, 15)
        Q[:, t] = q
        err = W[:, t] - (q - z64[:, t]) * s64[:, t]
        W[:, :t] -= np.outer(err, A[:t, t] / np.diag(A)[:t])
    q = oracle.babai_solver(pr["W"].t().contiguous(), pr["A"], pr["s"], pr["z"], gs, 4, 8, pr["g_idx"],
                            pr["G"]).t().numpy()
    safe = margins.min(axis=1) > 1e-3
    assert safe.sum() >= R // 2
    assert np.array_equal(q[safe], Q[safe])


@pytest.mark.parametrize("block", [8, 32])
def test_equals_the_forward_sweep_of_the_reversed_problem(block):
    """With both index orders reversed the back-to-front recurrence IS the GPTQ sweep with
    U'[t',k'] = A[C-1-k', C-1-t'] / A[C-1-k', C-1-k'] (two separately written oracle functions,
    one of them pinned by the textbook GPTQ): bit for bit in the chain order."""
    C, R, gs = 192, 40, 64
    pr = _problem(C, R, gs, sym=False, seed=3)
    A = pr["A"]
    qb = oracle.babai_solver(pr["W"].t().contiguous(), A, pr["s"], pr["z"], gs, 4, block, pr["g_idx"], pr["G"])
    Af = A.flip(0, 1)                                            # lower
    inv = (1.0 / torch.diag(Af)).float()
    Up = torch.triu((Af * inv[:, None]).t().contiguous(), 1) + torch.eye(C)
    se, ze = _meta_per_element(pr["s"], pr["z"], pr["g_idx"], R, pr["G"])
    qf = oracle.gptq_solver(pr["W"].t().flip(0).contiguous(), Up.contiguous(), se.flip(0).contiguous(),
                            ze.flip(0).contiguous(), 4, block=block)
    assert torch.equal(qb, qf.flip(0))


def test_chain_and_gemm_orders_differ_only_rarely():
    C, R, gs = 256, 64, 128
    pr = _problem(C, R, gs)
    args = (pr["A"], pr["s"], pr["z"], gs, 4, 32, pr["g_idx"], pr["G"])
    q0 = oracle.babai_solver(pr["W"].t().contiguous(), *args, trail_mode=oracle.TRAIL_CHAIN)
    q1 = oracle.babai_solver(pr["W"].t().contiguous(), *args, trail_mode=oracle.TRAIL_GEMM)
    assert (q0 != q1).float().mean().item() < 2e-3


def test_host_checks_are_the_reference_ones():
    W = torch.zeros(64, 4)
    with pytest.raises(RuntimeError):
        oracle.babai_solver(W, torch.eye(64), torch.ones(8), torch.ones(8), 48, 4, 8, None, 2)    # 48 % 32
    with pytest.raises(RuntimeError):
        oracle.babai_solver(W, torch.eye(64), torch.ones(8), torch.ones(8), 32, 4, 8, None, 3)    # G mismatch


def test_class_path_ascending_order_and_identity_fallback():
    """gptq.py:107-108: act-order for Babai is ASCENDING; a layer without tokens gets H = I
    and the result is round-to-nearest."""
    g = torch.Generator().manual_seed(7)
    W = 0.02 * torch.randn(16, 128, generator=g)
    layer = torch.nn.Linear(128, 16, bias=False)
    layer.weight.data = W.clone()
    kw = dict(bits=4, group_size=32, symmetric=True, quantization_scale="absmax",
              quantization_order="activation", algorithm="babai")
    o = oracle.GPTQ(layer, **kw)
    X = torch.randn(300, 128, generator=g)
    X[:, 5] *= 9
    o.update(X)
    q, s, z = o.quantize()
    d = torch.diag(2.0 / 300 * X.T @ X)
    assert torch.equal(o.perm, torch.argsort(d))                 # ascending
    assert q.shape == (16, 128) and q.dtype == torch.uint8
    o2 = oracle.GPTQ(layer, **kw)                                 # no update: H = I
    q2, s2, z2 = o2.quantize()
    G = 4
    se = s2.view(16, G).repeat_interleave(32, 1)
    ze = z2.view(16, G).repeat_interleave(32, 1)
    assert np.array_equal(q2.numpy(), mathref.rtn(W.numpy(), se.numpy(), ze.numpy(), 4))
