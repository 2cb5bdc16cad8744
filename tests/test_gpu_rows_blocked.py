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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rows_operands_and_diagonal_match_their_definitions(hip, dtype):
    """The front end of the closed forms: sqrt(2/n) X in solver order, pruned columns zero, in
    both layouts, and the float64-summed diagonal of (2/n) X^T X, straight from rows that lie
    end to end in one tensor (ragged counts, a feature count that is no multiple of the tile).
    Element by element against the definition in float64, rounded once: bit-exact for the
    operands; the diagonal's sum may be ordered differently, one ulp of f32 is allowed."""
    g = torch.Generator().manual_seed(3)
    C, nmax = 200, 96
    ns = [5, 96, 40, 1]
    row0 = [7, 20, 130, 0]                                   # not in batch order, with gaps
    rows = torch.randn(180, C, generator=g).to(dtype)
    perm = torch.stack([torch.randperm(C, generator=g) for _ in ns])
    dead = torch.rand(len(ns), C, generator=g) < 0.1
    root = torch.tensor([(2.0 / n) ** 0.5 for n in ns], dtype=torch.float64)
    BT, Bp = hip.rows_operands(rows.to(DEV), torch.tensor(row0).to(DEV), torch.tensor(ns, dtype=torch.int32).to(DEV),
                               root.to(DEV), perm.to(DEV), dead.to(DEV), nmax)
    _, Bp_only = hip.rows_operands(rows.to(DEV), torch.tensor(row0).to(DEV),
                                   torch.tensor(ns, dtype=torch.int32).to(DEV), root.to(DEV), perm.to(DEV),
                                   dead.to(torch.uint8).to(DEV), nmax, want_bt=False)
    want = torch.zeros(len(ns), nmax, C)
    for b, n in enumerate(ns):
        x = rows[row0[b]:row0[b] + n].double()[:, perm[b]] * root[b]
        want[b, :n] = x.float().masked_fill(dead[b][None, :], 0)
    assert torch.equal(BT.cpu(), want)
    assert torch.equal(Bp.cpu(), want.transpose(1, 2)) and torch.equal(Bp_only.cpu(), want.transpose(1, 2))
    alpha = torch.tensor([2.0 / n for n in ns], dtype=torch.float64)
    d = hip.rows_diagonal(rows.to(DEV), torch.tensor(row0).to(DEV), torch.tensor(ns, dtype=torch.int32).to(DEV),
                          alpha.to(DEV)).cpu()
    ref = torch.stack([(rows[row0[b]:row0[b] + n].double() ** 2).sum(0) * alpha[b] for b, n in enumerate(ns)])
    assert ((d.double() - ref).abs() <= 6e-8 * ref).all()
    assert (d == ref.float()).float().mean() > 0.99


def test_rows_that_arrive_in_several_updates_and_change_route():
    """Rows of one expert spread over several update() calls, in f32 and bf16, with experts that
    move from the per-row-vector form to the blocked form and from there to their Hessian:
    every expert ends up where the oracle, fed the same rows in the same pieces
    (forge/gptq.py:61-80), ends up, under the rule of the end-to-end tests."""
    from forge.moe import ExpertGroupGPTQ
    from helpers import linear, codes_at_floor
    g0 = torch.Generator().manual_seed(23)
    C, R = 1024, 128
    W = (0.02 * torch.randn(3, R, C, generator=g0)).bfloat16()
    first = [torch.randn(10, C, generator=g0), torch.randn(50, C, generator=g0), torch.randn(30, C, generator=g0)]
    later = [torch.randn(30, C, generator=g0).bfloat16(), torch.randn(20, C, generator=g0).bfloat16(),
             torch.randn(100, C, generator=g0).bfloat16()]
    first[1] = first[1].bfloat16().float()
    first[2] = first[2].bfloat16().float()                  # only expert 0's first rows need f32
    kw = dict(bits=4, group_size=128, symmetric=False, quantization_scale="absmax",
              quantization_order="activation", rel_damp=0.01)
    grp = ExpertGroupGPTQ([W.to(DEV)], device=DEV, low_rank_tokens=16, **kw)
    grp.update(torch.cat(first).to(DEV), [0, 10, 60, 90])
    assert grp.low_rank == [True, False, False] and grp.rows_route == [False, True, True]
    grp.prepare()                                           # lays the kept rows end to end; discarded below
    grp.update(torch.cat(later).to(DEV), [0, 30, 50, 150])
    # 40 and 70 rows: blocked form (up to 128 rows at 1024 features); 130 rows: through the Hessian
    assert grp.low_rank == [False] * 3 and grp.rows_route == [True, True, False]
    X2 = torch.cat([first[2].double(), later[2].double()])
    H2 = (2.0 / 130) * X2.t() @ X2
    assert ((grp.hessian(2).cpu().double() - H2).norm() / H2.norm()).item() < 2e-6
    q = grp.quantize(chunk=3)[0][0].cpu()
    assert not grp.issue_non_invertible.any()
    for e in range(3):
        o = oracle.GPTQ(linear(W[e]), **kw)
        o.update(first[e])
        o.update(later[e].float())
        qo = o.quantize()[0]
        codes_at_floor(f"expert {e}", qo, q[e], W[e], [torch.cat([first[e], later[e].float()])], kw,
                       order=o.perm)
