"""Pins the oracle's column sweep (solver.cu:9-154, solver_sparsegptq14.cu:29-200)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from helpers import random_problem, flip_rate


@pytest.mark.parametrize("sym", [True, False])
def test_identity_factor_is_round_to_nearest(sym):
    pr = random_problem(C=256, R=48, sym=sym)
    Wt = pr["W"].t().contiguous()
    q = oracle.gptq_solver(Wt.clone(), torch.eye(256), pr["se"], pr["ze"], 4)
    ref = mathref.rtn(Wt.numpy(), pr["se"].numpy(), pr["ze"].numpy(), 4)
    assert np.array_equal(q.numpy(), ref)
    # dequantised weights written back: (q - q0) * s with one rounding
    deq = oracle.gptq_solver.last_W
    want = (q.double() * pr["se"].double() - (pr["ze"] * pr["se"]).double()).float()
    assert torch.equal(deq, want)


def test_textbook_gptq_float64_agrees_away_from_ties():
    C, R = 64, 8
    pr = random_problem(C=C, R=R, n=256, gs=32)
    Q, D, margins = mathref.gptq_textbook(pr["W"].numpy(), pr["H"].numpy(), pr["se"].t().numpy(),
                                          pr["ze"].t().numpy(), 4, 0.01)
    q = oracle.gptq_solver(pr["W"].t().contiguous(), pr["U"], pr["se"], pr["ze"], 4, block=32)
    q = q.t().numpy()
    # rows whose every decision had a clear margin must agree exactly
    safe = margins.min(axis=1) > 1e-3
    assert safe.sum() >= R // 2
    assert np.array_equal(q[safe], Q[safe])


@pytest.mark.parametrize("mode", [oracle.TRAIL_CHAIN, oracle.TRAIL_GEMM])
def test_block_size_invariance(mode):
    pr = random_problem(C=384, R=64)
    Wt = pr["W"].t().contiguous()
    base = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=mode, block=32)
    for B in (64, 128, 96):
        other = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=mode, block=B)
        if mode == oracle.TRAIL_CHAIN:
            assert torch.equal(base, other)           # one fma chain: independent of blocking
        else:
            assert flip_rate(base, other) < 5e-3      # a different summation order: ties only


def test_chain_and_gemm_orders_differ_only_at_ties():
    pr = random_problem(C=512, R=128)
    Wt = pr["W"].t().contiguous()
    a = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=oracle.TRAIL_CHAIN)
    b = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=oracle.TRAIL_GEMM)
    assert flip_rate(a, b) < 5e-3


def test_gptq_beats_rtn_in_hessian_weighted_error():
    pr = random_problem(C=512, R=64, outliers=8)
    Wt = pr["W"].t().contiguous()
    q = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4)
    rtn = mathref.rtn(Wt.numpy(), pr["se"].numpy(), pr["ze"].numpy(), 4)
    deq = lambda qq: ((torch.as_tensor(qq).float() - pr["ze"]) * pr["se"]).t().numpy()
    H = pr["H"].numpy()
    assert mathref.layer_error(pr["W"].numpy(), deq(q), H) < 0.9 * mathref.layer_error(pr["W"].numpy(), deq(rtn), H)


def test_ragged_last_block():
    # C not a multiple of the block width: the tail block must be swept too
    pr = random_problem(C=200, R=20, gs=128)
    Wt = pr["W"].t().contiguous()
    a = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, block=32)
    b = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, block=200)
    assert torch.equal(a, b)


# ---------------------------------------------------------------- 1:4 joint solve
def _sparse(pr, U0):
    Wt = pr["W"].t().contiguous()
    U = U0.clone()
    q, M = oracle.sparsegptq14_solver(Wt.clone(), U, pr["se"], pr["ze"], 4)
    return q, M.view(torch.int32), U, oracle.sparsegptq14_solver.last_W


def _bits(M, C):
    m = M.numpy().astype(np.uint32)
    cols = np.arange(C)
    return ((m[cols // 32] >> (cols % 32)[:, None]) & 1).astype(bool)     # [C, R]


def test_sparse_one_survivor_per_group_of_four():
    C, R = 256, 40
    pr = random_problem(C=C, R=R)
    U0 = torch.from_numpy(mathref.factor(pr["H"].double().numpy(), 0.01, normalise=False)).float().contiguous()
    q, M, Un, deq = _sparse(pr, U0)
    keep = _bits(M, C)
    assert np.all(keep.reshape(C // 4, 4, R).sum(axis=1) == 1)
    assert np.all(q.numpy()[~keep] == 0) and np.all(deq.numpy()[~keep] == 0)
    # the caller's U is row-normalised in place with a reciprocal multiply
    want = U0 * (1.0 / U0.diag())[:, None]
    assert torch.equal(Un, want)


def test_sparse_identity_factor_is_magnitude_pruning_plus_rtn():
    C, R = 128, 16
    pr = random_problem(C=C, R=R)
    q, M, _, _ = _sparse(pr, torch.eye(C))
    keep = _bits(M, C)
    Wt = pr["W"].t().numpy()
    first_argmax = np.abs(Wt).reshape(C // 4, 4, R).argmax(axis=1)         # first max wins
    want = np.zeros((C // 4, 4, R), dtype=bool)
    np.put_along_axis(want, first_argmax[:, None, :], True, axis=1)
    assert np.array_equal(keep, want.reshape(C, R))
    rtn = mathref.rtn(Wt, pr["se"].numpy(), pr["ze"].numpy(), 4)
    assert np.array_equal(q.numpy()[keep], rtn[keep])


def test_sparse_selection_uses_updated_weights_and_saliency():
    # brute force in float64 on a tiny case: saliency |x / U0_kk| with x updated by all
    # earlier columns but not by the group's own
    C, R = 32, 4
    pr = random_problem(C=C, R=R, n=128, gs=32)
    U0 = mathref.factor(pr["H"].double().numpy(), 0.01, normalise=False)
    q, M, _, _ = _sparse(pr, torch.from_numpy(U0).float().contiguous())
    keep = _bits(M, C)
    Un = U0 / np.diag(U0)[:, None]
    x = pr["W"].t().double().numpy().copy()
    s, z = pr["se"].double().numpy(), pr["ze"].double().numpy()
    mine = np.zeros((C, R), dtype=bool)
    clear = np.ones(R, dtype=bool)
    for t in range(C):
        if t % 4 == 0:
            sc = np.abs(x[t:t + 4] / np.diag(U0)[t:t + 4, None])
            srt = np.sort(sc, axis=0)
            clear &= (srt[-1] - srt[-2]) > 1e-4 * srt[-1]
            mine[t:t + 4][sc.argmax(axis=0), np.arange(R)] = True
        qq = np.clip(np.rint(x[t] / (s[t] + 1e-12) + z[t]), 0, 15)
        err = np.where(mine[t], x[t] - (qq - z[t]) * s[t], x[t])
        x[t + 1:] -= np.outer(Un[t, t + 1:], err)
    assert clear.any()
    assert np.array_equal(keep[:, clear], mine[:, clear])


def test_reference_shaped_host_loop_is_pinned():
    """TRAIL_BLAS: the 32-column kernel alone (oracle_gptq_inblock) followed by one BLAS SGEMM
    per block, the reference's host loop literally (solver.cu:118-150).  The in-block kernel by
    itself is the fma chain: with one block spanning the matrix it equals the chained solver
    bit for bit, and with U = I it is round-to-nearest.  With 32-column blocks the SGEMM's
    summation order differs from the chain's, so codes may move at ties only, and the
    Hessian-weighted error stays the same."""
    pr = random_problem(C=192, R=40)
    Wt = pr["W"].t().contiguous()
    one_block = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4,
                                   trail_mode=oracle.TRAIL_BLAS, block=192)
    chain = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4)
    assert torch.equal(one_block, chain)
    rtn = oracle.gptq_solver(Wt.clone(), torch.eye(192), pr["se"], pr["ze"], 4,
                             trail_mode=oracle.TRAIL_BLAS)
    assert np.array_equal(rtn.numpy(), mathref.rtn(Wt.numpy(), pr["se"].numpy(), pr["ze"].numpy(), 4))
    pr = random_problem(C=512, R=128)
    Wt = pr["W"].t().contiguous()
    a = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=oracle.TRAIL_CHAIN)
    b = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4, trail_mode=oracle.TRAIL_BLAS)
    Wb = oracle.gptq_solver.last_W                     # dequantised weights of the BLAS run
    assert flip_rate(a, b) < 5e-3
    want = (b.double() * pr["se"].double() - (pr["ze"] * pr["se"]).double()).float()
    assert torch.equal(Wb, want)
    H = pr["H"].double().numpy()
    deq = lambda q: ((q.double() - pr["ze"].double()) * pr["se"].double()).t().numpy()
    ea = mathref.layer_error(pr["W"].numpy(), deq(a), H)
    eb = mathref.layer_error(pr["W"].numpy(), deq(b), H)
    assert abs(eb / ea - 1) < 5e-3
