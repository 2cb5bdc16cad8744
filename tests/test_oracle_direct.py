"""The displacement form of the sweep (factor of H instead of the factor of its inverse):
the algebra in float64, the fp32 checker against the reference-form oracle."""
import numpy as np
import torch

import oracle
from oracle import mathref
from helpers import random_problem, flip_rate


def _sweeps_float64(W, Ut, N, s, z):
    """Both forms column by column in float64 (W [R,C]; s, z [R,C])."""
    R, C = W.shape
    Xe, Xd = W.copy(), W.copy()
    Qe, Qd = np.zeros((R, C)), np.zeros((R, C))
    for t in range(C):
        inv = 1.0 / (s[:, t] + 1e-12)
        qe = np.clip(np.rint(Xe[:, t] * inv + z[:, t]), 0, 15)
        qd = np.clip(np.rint(Xd[:, t] * inv + z[:, t]), 0, 15)
        Qe[:, t], Qd[:, t] = qe, qd
        err = Xe[:, t] - (qe - z[:, t]) * s[:, t]
        d = W[:, t] - (qd - z[:, t]) * s[:, t]
        Xe[:, t + 1:] -= np.outer(err, Ut[t, t + 1:])
        Xd[:, t + 1:] += np.outer(d, N[t, t + 1:])
    return Qe, Qd, Xe, Xd


def test_direct_factor_is_the_inverse_of_the_reference_factor():
    pr = random_problem(C=96, R=4, n=60, seed=1)             # rank deficient + damping
    H = pr["H"].double().numpy()
    H = 0.5 * (H + H.T)                                      # fp32 X^T X is symmetric to 1 ulp only
    Ut = mathref.factor(H, 0.01)
    V = mathref.direct_factor(H, 0.01)
    N = 2 * np.eye(96) - V                                   # unit diagonal, +M/M_kk above
    assert np.allclose(N @ Ut, np.eye(96), atol=1e-9)
    assert np.allclose(np.tril(V, -1), 0) and np.allclose(np.diag(V), 1)


def test_both_forms_are_the_same_solve_in_float64():
    """Same codes and the same value at every column when it is reached."""
    pr = random_problem(C=128, R=16, n=100, seed=2)
    H = pr["H"].double().numpy()
    H = 0.5 * (H + H.T)
    Ut = mathref.factor(H, 0.01)
    N = 2 * np.eye(128) - mathref.direct_factor(H, 0.01)
    W = pr["W"].double().numpy()
    s, z = pr["se"].t().double().numpy(), pr["ze"].t().double().numpy()
    Qe, Qd, Xe, Xd = _sweeps_float64(W, Ut, N, s, z)
    assert np.array_equal(Qe, Qd)
    assert np.allclose(Xe, Xd, atol=1e-10)


def test_checker_identity_factor_is_round_to_nearest():
    pr = random_problem(C=64, R=8, seed=3)
    Wt = pr["W"].t().contiguous()
    q = oracle.gptq_solver_direct(Wt.clone(), torch.eye(64), pr["se"], pr["ze"], 4)
    ref = torch.clamp(torch.round(torch.addcmul(pr["ze"].double(), Wt.double(),
                                                (1.0 / (pr["se"] + 1e-12)).double()).float()), 0, 15)
    assert torch.equal(q.float(), ref)


def test_checker_against_the_reference_form():
    """fp32 displacement form vs the oracle's error form and the float64 solve: codes differ
    only at near-ties; the Hessian-weighted error is the same."""
    C, R = 256, 64
    pr = random_problem(C=C, R=R, n=512, seed=4)
    H = pr["H"].double().numpy()
    V = torch.from_numpy(mathref.direct_factor(H, 0.01)).float().contiguous()
    Wt = pr["W"].t().contiguous()
    qd = oracle.gptq_solver_direct(Wt.clone(), V, pr["se"], pr["ze"], 4)
    qe = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4)
    assert flip_rate(qd, qe) <= 1e-3
    W = pr["W"].double().numpy()
    s, z = pr["se"].t().double().numpy(), pr["ze"].t().double().numpy()
    Q64, _, _, _ = _sweeps_float64(W, mathref.factor(H, 0.01), 2 * np.eye(C) - V.double().numpy(), s, z)
    assert float((qd.t().double().numpy() != Q64).mean()) <= 1e-3
    def loss(q):
        D = W - (q.t().double().numpy() - z) * s
        return float(np.einsum("rc,cd,rd->", D, H, D))
    assert abs(loss(qd) / loss(qe) - 1) < 1e-3
