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


def _reverse_factor_diag(H, rel_damp):
    """diag of M for H + damp I = M M^T (M upper), float64."""
    C = H.shape[0]
    Hd = 0.5 * (H + H.T)
    Hd[np.diag_indices(C)] += rel_damp * np.mean(np.diag(H))
    return np.diag(np.linalg.cholesky(Hd[::-1, ::-1])[::-1, ::-1]).copy()


def test_sparse14_look_ahead_in_float64():
    """The 1:4 mask score reads three columns that have not received all their updates; in
    the displacement form those hold different numbers.  Rebuilt through the inverse of N's
    4x4 diagonal block they give the error form's masks and codes exactly; left as they are
    they do not."""
    C, R = 128, 32
    pr = random_problem(C=C, R=R, n=200, seed=5)
    H = pr["H"].double().numpy()
    H = 0.5 * (H + H.T)
    U0 = mathref.factor(H, 0.01, normalise=False)
    Ut, uinv = U0 / np.diag(U0)[:, None], 1.0 / np.diag(U0)
    assert np.allclose(uinv, _reverse_factor_diag(H, 0.01), rtol=1e-9)
    V = mathref.direct_factor(H, 0.01)
    W = pr["W"].double().numpy()
    s, z = pr["se"].t().double().numpy(), pr["ze"].t().double().numpy()

    def run(form):
        X, Q, mask = W.copy(), np.zeros((R, C)), np.zeros((R, C), bool)
        for t in range(C):
            if t % 4 == 0:
                look = X[:, t:t + 4]
                if form == "d":   # "d-uncorrected" skips this
                    v = V[t:t + 4, t:t + 4]
                    A = np.eye(4)
                    A[0, 1], A[1, 2], A[2, 3] = v[0, 1], v[1, 2], v[2, 3]
                    A[0, 2] = v[0, 2] + v[0, 1] * v[1, 2]
                    A[1, 3] = v[1, 3] + v[1, 2] * v[2, 3]
                    A[0, 3] = v[0, 3] + v[0, 1] * A[1, 3] + v[0, 2] * v[2, 3]
                    look = W[:, t:t + 4] + (X[:, t:t + 4] - W[:, t:t + 4]) @ A
                mask[np.arange(R), t + np.abs(look * uinv[None, t:t + 4]).argmax(1)] = True
            q = np.clip(np.rint(X[:, t] / (s[:, t] + 1e-12) + z[:, t]), 0, 15)
            deq = np.where(mask[:, t], (q - z[:, t]) * s[:, t], 0.0)
            Q[:, t] = np.where(mask[:, t], q, 0)
            if form == "e":
                X[:, t + 1:] -= np.outer(X[:, t] - deq, Ut[t, t + 1:])
            else:
                X[:, t + 1:] -= np.outer(W[:, t] - deq, V[t, t + 1:])
        return Q, mask

    (Qe, Me), (Qd, Md), (Qn, Mn) = run("e"), run("d"), run("d-uncorrected")
    assert np.array_equal(Me, Md) and np.array_equal(Qe, Qd)
    assert not np.array_equal(Me, Mn)


def test_sparse14_checker_against_the_reference_form():
    for C, R, n, seed in ((256, 64, 500, 1), (200, 33, 150, 2), (512, 32, 300, 3)):
        pr = random_problem(C=C, R=R, n=n, seed=seed)
        H = pr["H"].double().numpy()
        U0 = torch.from_numpy(mathref.factor(H, 0.01, normalise=False)).float().contiguous()
        V = torch.from_numpy(mathref.direct_factor(H, 0.01)).float().contiguous()
        mdiag = torch.from_numpy(_reverse_factor_diag(H, 0.01)).float()
        Wt = pr["W"].t().contiguous()
        qe, Me = oracle.sparsegptq14_solver(Wt.clone(), U0.clone(), pr["se"], pr["ze"], 4)
        qd, Md = oracle.sparsegptq14_solver_direct(Wt.clone(), V, mdiag, pr["se"], pr["ze"], 4)
        be = np.unpackbits(Me.numpy().view(np.uint8), bitorder="little")
        bd = np.unpackbits(Md.numpy().view(np.uint8), bitorder="little")
        assert bd.reshape(-1, 4).sum(1).max() <= 1          # at most one kept weight per group of four
        assert (be != bd).mean() <= 1e-3 and flip_rate(qe, qd) <= 3e-3
