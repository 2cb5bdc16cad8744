"""HIP Babai path (forge_babai_solver, forge_chol_reverse_lower_batched,
forge_unit_upper_from_lower, GPTQ(algorithm="babai")) against the oracle and float64."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_problem, flip_rate, linear

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _upper_factor(H, rel_damp=0.01):
    Hd = H.double().numpy().copy()
    Hd[np.diag_indices(Hd.shape[0])] += rel_damp * np.mean(np.diag(Hd))
    return torch.from_numpy(np.linalg.cholesky(Hd).T.copy()).float().contiguous()


@pytest.mark.parametrize("C,R,gs,sym", [(256, 192, 128, True), (320, 100, 64, False), (96, 64, 32, True)])
def test_babai_solver_bit_exact(hip, C, R, gs, sym):
    """Same factor on both sides: the codes are those of the oracle's chain, bit for bit
    (ragged last 128-column block, R not a multiple of 64, permuted group lookup included)."""
    pr = random_problem(C=C, R=R, sym=sym, gs=gs, seed=C)
    g = torch.Generator().manual_seed(C + 1)
    g_idx = (torch.randperm(C, generator=g) // gs).to(torch.int32)
    A = _upper_factor(pr["H"])
    Wt = pr["W"].t().contiguous()
    qo = oracle.babai_solver(Wt.clone(), A, pr["s"], pr["z"], gs, 4, gs // 4, g_idx, pr["G"])
    qg = hip.babai_solver(Wt.to(DEV), A.to(DEV), pr["s"].to(DEV), pr["z"].to(DEV), gs, 4, gs // 4,
                          g_idx.to(DEV), pr["G"])
    assert torch.equal(qo, qg.cpu())


def test_full_size_babai_properties(hip):
    """Config-1 size (2048 x 2048).  An identity factor must give round-to-nearest bit for
    bit; the back-to-front solve must equal the forward sweep of the index-reversed problem
    (rows of the unit factor U'[t', k'] = A[k, t] / A[k, k] with k = C-1-k', t = C-1-t')
    composed from the library's other entry points; and the oracle's chain must agree."""
    C = R = 2048
    gs, G = 128, 16
    pr = random_problem(C=C, R=R, n=1024, seed=9)
    A = _upper_factor(pr["H"])
    Wt = pr["W"].t().contiguous()
    s, z = pr["s"].to(DEV), pr["z"].to(DEV)
    q_rtn = hip.babai_solver(Wt.to(DEV), torch.eye(C, device=DEV), s, z, gs, 4, 32, None, G)
    se, ze = pr["se"].to(DEV), pr["ze"].to(DEV)
    ref = torch.clamp(torch.round(torch.addcmul(ze.double(), Wt.to(DEV).double(),
                                                (1.0 / (se + 1e-12)).double()).float()), 0, 15)
    assert torch.equal(q_rtn.float(), ref)
    q = hip.babai_solver(Wt.to(DEV), A.to(DEV), s, z, gs, 4, 32, None, G)
    Ur = hip.unit_upper_from_lower(A.view(1, C, C).to(DEV), None, flipped_upper=True)
    sT = pr["s"].view(R, G).t().contiguous().view(1, G, R).to(DEV)
    zT = pr["z"].view(R, G).t().contiguous().view(1, G, R).to(DEV)
    g_rev = (torch.arange(C - 1, -1, -1) // gs).int().view(1, C).to(DEV)
    q_fwd = hip.gptq_sweep_batched(Wt.flip(0).contiguous().view(1, C, R).to(DEV), Ur, sT, zT, g_rev, 4)
    assert torch.equal(q, q_fwd[0].flip(0))
    qo = oracle.babai_solver(Wt.clone(), A, pr["s"], pr["z"], gs, 4, 32, None, G)
    assert torch.equal(qo, q.cpu())


def test_babai_solver_rejects_what_the_reference_rejects(hip):
    W = torch.zeros(64, 8, device=DEV)
    A = torch.eye(64, device=DEV)
    s = torch.ones(16, device=DEV)
    with pytest.raises(RuntimeError):
        hip.babai_solver(W, A, s, s, 48, 4, 8, None, 2)          # group size not a multiple of 32
    with pytest.raises(RuntimeError):
        hip.babai_solver(W, A, s, s, 32, 4, 8, None, 3)          # G does not match


@pytest.mark.parametrize("C", [100, 256])
def test_unit_upper_from_lower_bit_exact(hip, C):
    g = torch.Generator().manual_seed(C)
    L = torch.tril(torch.randn(2, C, C, generator=g)) + 3 * torch.eye(C)
    info = torch.tensor([0, 4], dtype=torch.int32)
    U = hip.unit_upper_from_lower(L.to(DEV), info.to(DEV)).cpu()
    inv = 1.0 / torch.diagonal(L[0])
    want = torch.triu((L[0] * inv[:, None]).t().contiguous(), 1) + torch.eye(C)
    assert torch.equal(U[0], want)
    assert torch.equal(U[1], torch.eye(C))                       # failed factorisation: identity
    # the reference's upper factor given instead of the reversed lower one
    A = L[0].flip(0, 1).contiguous()
    U2 = hip.unit_upper_from_lower(A.view(1, C, C).to(DEV), None, flipped_upper=True).cpu()
    assert torch.equal(U2[0], want)


@pytest.mark.parametrize("B,C", [(3, 200), (8, 512)])
def test_reverse_lower_factor_matches_float64(hip, B, C):
    g = torch.Generator().manual_seed(B * C)
    X = torch.randn(B, 2 * C, C, generator=g, dtype=torch.float64)
    X[:, :, :4] *= 7
    H = ((2.0 / X.shape[1]) * X.transpose(1, 2) @ X).float()
    H[B - 1, 3, 3] = -1.0                                        # not positive definite
    damp = (0.01 * torch.diagonal(H[0]).mean()).repeat(B).float()
    L, info = hip.chol_reverse_lower_batched(H.clone().to(DEV), damp.to(DEV))
    assert info.tolist()[:B - 1] == [0] * (B - 1) and info[B - 1].item() > 0
    for b in range(B - 1):
        Hd = H[b].double().numpy().copy()
        Hd[np.diag_indices(C)] += float(damp[b])
        # H = L^T L with L lower  <=>  flip(H) = A^T A with A = flip(L) upper
        A = np.linalg.cholesky(Hd[::-1, ::-1]).T
        ref = A[::-1, ::-1]
        got = torch.tril(L[b].cpu()).double().numpy()
        assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 5e-6


@pytest.mark.parametrize("order", ["activation", "default"])
def test_class_end_to_end_against_the_oracle(order):
    """forge.gptq.GPTQ(algorithm="babai") against oracle.GPTQ: same scales and zeros; codes
    differ only through the last bits of two fp32 factorisations (different routes)."""
    from forge.gptq import GPTQ
    g = torch.Generator().manual_seed(11)
    R, C, n = 256, 512, 1024
    W = 0.02 * torch.randn(R, C, generator=g)
    X = torch.randn(n, C, generator=g)
    # well separated column energies: the activation order must not hinge on the last bits
    # of two fp32 Hessians (a different order is a different, equally valid, solve)
    X *= torch.linspace(0.5, 3.0, C)[torch.randperm(C, generator=g)]
    kw = dict(bits=4, group_size=128, symmetric=False, quantization_scale="mse",
              quantization_order=order, rel_damp=0.01, algorithm="babai")
    o = oracle.GPTQ(linear(W), **kw)
    o.update(X)
    qo, so, zo = o.quantize()
    h = GPTQ(linear(W).to(DEV), device=DEV, **kw)
    h.update(X.to(DEV))
    qg, sg, zg = (t.cpu() for t in h.quantize())
    assert float((h.perm.cpu() != o.perm).float().mean()) < 0.01
    assert float((so != sg).float().mean()) <= 1e-3
    same = so == sg
    assert torch.equal(zo[same], zg[same])
    assert flip_rate(qo, qg) <= 5e-3


def test_expert_group_babai_matches_per_expert_oracle():
    """The batched front end with algorithm="babai": gate/up share Hessian and factor; one
    expert never saw a token (H = I: plain round-to-nearest, exact)."""
    from forge.moe import ExpertGroupGPTQ
    g = torch.Generator().manual_seed(21)
    E, R, C = 3, 96, 256
    Wg = 0.02 * torch.randn(E, R, C, generator=g)
    Wu = 0.02 * torch.randn(E, R, C, generator=g)
    col = torch.linspace(0.5, 3.0, C)[torch.randperm(C, generator=g)]
    xs = [torch.randn(n, C, generator=g) * col for n in (400, 0, 700)]
    offs = np.concatenate([[0], np.cumsum([x.shape[0] for x in xs])])
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="activation", algorithm="babai")
    grp = ExpertGroupGPTQ([Wg.to(DEV), Wu.to(DEV)], device=DEV, **kw)
    grp.update(torch.cat(xs).to(DEV), offs)
    (qg, sg, zg), (qu, su, zu) = grp.quantize(chunk=4)
    for e in range(E):
        for W, (q, s, z) in ((Wg[e], (qg, sg, zg)), (Wu[e], (qu, su, zu))):
            o = oracle.GPTQ(linear(W), **kw)
            o.update(xs[e])
            qo, so, zo = o.quantize()
            assert float((so != s[e].cpu()).float().mean()) <= 2e-3
            if xs[e].shape[0] == 0:
                assert torch.equal(qo, q[e].cpu())
            else:
                assert flip_rate(qo, q[e]) <= 5e-3
