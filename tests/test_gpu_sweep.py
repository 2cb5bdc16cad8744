"""HIP column sweep against the oracle: bit-exact codes, weights and masks."""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from helpers import random_problem

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("C,R,sym", [(128, 64, True), (256, 130, False), (640, 96, True),
                                     (200, 77, False), (36, 5, True), (1024, 512, True)])
def test_gptq_solver_bit_exact(hip, C, R, sym):
    pr = random_problem(C=C, R=R, sym=sym, seed=C + R)
    Wt = pr["W"].t().contiguous()
    q0 = oracle.gptq_solver(Wt.clone(), pr["U"], pr["se"], pr["ze"], 4)
    W0 = oracle.gptq_solver.last_W
    Wd = Wt.clone().to(DEV)
    q1 = hip.gptq_solver(Wd, pr["U"].to(DEV), pr["se"].to(DEV), pr["ze"].to(DEV), 4)
    assert torch.equal(q0, q1.cpu())
    assert torch.equal(W0, Wd.cpu())            # contiguous W is overwritten with deq


def test_gptq_solver_non_contiguous_input_is_left_alone(hip):
    pr = random_problem(C=128, R=64)
    Wd = pr["W"].to(DEV)
    before = Wd.clone()
    q1 = hip.gptq_solver(Wd.t(), pr["U"].to(DEV), pr["se"].to(DEV), pr["ze"].to(DEV), 4)
    q0 = oracle.gptq_solver(pr["W"].t().contiguous(), pr["U"], pr["se"], pr["ze"], 4)
    assert torch.equal(q0, q1.cpu()) and torch.equal(Wd, before)


@pytest.mark.parametrize("bits", [2, 3, 8])
def test_other_bit_widths(hip, bits):
    pr = random_problem(C=256, R=64)
    s, z = oracle.build_group_meta_packed(pr["W"].reshape(-1, 128), bits, False)
    from helpers import expand_meta
    se, ze = expand_meta(s, 64, 256, 128), expand_meta(z, 64, 256, 128)
    Wt = pr["W"].t().contiguous()
    q0 = oracle.gptq_solver(Wt.clone(), pr["U"], se, ze, bits)
    q1 = hip.gptq_solver(Wt.clone().to(DEV), pr["U"].to(DEV), se.to(DEV), ze.to(DEV), bits)
    assert torch.equal(q0, q1.cpu()) and int(q0.max()) <= 2 ** bits - 1


@pytest.mark.parametrize("C,R", [(256, 64), (384, 200), (100, 33)])
def test_sparse14_solver_bit_exact(hip, C, R):
    pr = random_problem(C=C, R=R, seed=C)
    U0 = torch.from_numpy(mathref.factor(pr["H"].double().numpy(), 0.01, normalise=False)).float().contiguous()
    Wt = pr["W"].t().contiguous()
    Uo = U0.clone()
    q0, M0 = oracle.sparsegptq14_solver(Wt.clone(), Uo, pr["se"], pr["ze"], 4)
    W0 = oracle.sparsegptq14_solver.last_W
    Ud, Wd = U0.clone().to(DEV), Wt.clone().to(DEV)
    q1, M1 = hip.sparsegptq14_solver(Wd, Ud, pr["se"].to(DEV), pr["ze"].to(DEV), 4)
    assert torch.equal(q0, q1.cpu())
    assert torch.equal(M0.view(torch.int32), M1.cpu().view(torch.int32))
    assert torch.equal(Uo, Ud.cpu())            # caller's U row-normalised in place
    assert torch.equal(W0, Wd.cpu())


@pytest.mark.parametrize("C,R", [(512, 192), (200, 70)])
def test_batched_sweep_with_group_lookup_and_permutation(hip, C, R):
    B, gs = 3, 128
    G = (C + gs - 1) // gs
    Xs, Us, sT, zT, gi, want = [], [], [], [], [], []
    for b in range(B):
        pr = random_problem(C=C, R=R, seed=100 + b, sym=bool(b % 2))
        perm = torch.randperm(C, generator=torch.Generator().manual_seed(b))
        Wt = pr["W"].t()[perm].contiguous()
        se, ze = pr["se"][perm].contiguous(), pr["ze"][perm].contiguous()
        want.append(oracle.gptq_solver(Wt.clone(), pr["U"], se, ze, 4))
        Xs.append(Wt); Us.append(pr["U"])
        sT.append(pr["s"].view(R, G).t().contiguous()); zT.append(pr["z"].view(R, G).t().contiguous())
        gi.append((perm // gs).int())
    X = torch.stack(Xs).to(DEV)
    q = hip.gptq_sweep_batched(X, torch.stack(Us).to(DEV), torch.stack(sT).to(DEV),
                               torch.stack(zT).to(DEV), torch.stack(gi).to(DEV), 4)
    for b in range(B):
        assert torch.equal(want[b], q[b].cpu())


@pytest.mark.parametrize("C,R", [(512, 256), (384, 192), (200, 70)])
def test_direct_sweep_bit_exact(hip, C, R):
    """Displacement form (factor of H itself) against its CPU checker: codes and the
    displacements left in X, bit for bit; whole-wavefront, 64-row and ragged variants."""
    B, gs = 3, 128
    G = (C + gs - 1) // gs
    Xs, Vs, sT, zT, gi, want, disp = [], [], [], [], [], [], []
    for b in range(B):
        pr = random_problem(C=C, R=R, seed=200 + b, sym=bool(b % 2), n=C // 2 if b == 2 else None)
        perm = torch.randperm(C, generator=torch.Generator().manual_seed(b))
        Wt = pr["W"].t()[perm].contiguous()
        se, ze = pr["se"][perm].contiguous(), pr["ze"][perm].contiguous()
        V = torch.from_numpy(mathref.direct_factor(pr["H"].double().numpy(), 0.01)).float().contiguous()
        want.append(oracle.gptq_solver_direct(Wt.clone(), V, se, ze, 4))
        disp.append(Wt - oracle.gptq_solver_direct.last_W)
        Xs.append(Wt); Vs.append(V)
        sT.append(pr["s"].view(R, G).t().contiguous()); zT.append(pr["z"].view(R, G).t().contiguous())
        gi.append((perm // gs).int())
    X = torch.stack(Xs).to(DEV)
    args = (torch.stack(Vs).to(DEV), torch.stack(sT).to(DEV), torch.stack(zT).to(DEV),
            torch.stack(gi).to(DEV), 4)
    q = hip.gptq_sweep_direct_batched(X, *args, exact_chain=True)
    for b in range(B):
        assert torch.equal(want[b], q[b].cpu())
        assert torch.equal(disp[b], X[b].cpu())
    # default: block updates as blocked sums (bf16 pieces where the tiles are full, fp32
    # elsewhere): fp32-grade, so codes move only at near-ties
    X2 = torch.stack(Xs).to(DEV)
    q2 = hip.gptq_sweep_direct_batched(X2, *args)
    assert (q2 != q).float().mean().item() <= 1e-3
    assert (X2 - X).abs().max().item() <= 0.05 * X.abs().max().item()


@pytest.mark.parametrize("C,R,dtype", [(512, 256, torch.bfloat16), (384, 192, torch.bfloat16),
                                       (200, 70, torch.bfloat16), (256, 128, torch.float32)])
def test_direct_sweep_untouched_weights_from_the_layout_pass(hip, C, R, dtype):
    """The layout pass writes the solver-order weights twice, as f32 (the values the sweep
    updates) and in the weights' own type (the untouched copy the displacement form reads):
    both equal the plain pass's output, also for a band of a taller matrix, and the sweep
    returns the same codes and displacements whether that copy is bf16, f32 or made inside the
    wrapper.  Fast (whole 256-row tiles) and general layout kernels."""
    B, gs = 2, 128
    G = (C + gs - 1) // gs
    g0 = torch.Generator().manual_seed(C + R)
    W = (0.02 * torch.randn(B, R, C, generator=g0)).to(dtype)
    perm = torch.stack([torch.randperm(C, generator=g0) for _ in range(B)])
    perm_inv = torch.argsort(perm, dim=1)
    Vs, sT, zT = [], [], []
    for b in range(B):
        pr = random_problem(C=C, R=R, seed=300 + b)
        Vs.append(torch.from_numpy(mathref.direct_factor(pr["H"].double().numpy(), 0.01)).float().contiguous())
        s_, z_ = oracle.build_group_meta_packed(
            torch.nn.functional.pad(W[b].float(), (0, G * gs - C)).reshape(R * G, gs), 4, True)
        sT.append(s_.view(R, G).t().contiguous()); zT.append(z_.view(R, G).t().contiguous())
    Wd, pd = W.to(DEV), perm_inv.to(DEV)
    X = hip.weight_to_solver_order(Wd, pd)
    W0 = torch.empty((B, C, R), dtype=dtype, device=DEV)
    X2 = hip.weight_to_solver_order(Wd, pd, out=torch.empty_like(X), out0=W0)
    assert torch.equal(X, X2) and torch.equal(W0.float(), X)
    assert torch.equal(X[0].cpu(), W[0].float().t()[perm[0]])
    # a band of a taller pair
    tall, tall0 = torch.zeros((B, C, 2 * R), device=DEV), torch.zeros((B, C, 2 * R), dtype=dtype, device=DEV)
    hip.weight_to_solver_order(Wd, pd, out=tall, row0=R, out0=tall0)
    assert torch.equal(tall[:, :, R:], X) and torch.equal(tall0[:, :, R:].float(), X)
    assert not tall[:, :, :R].any() and not tall0[:, :, :R].any()
    args = (torch.stack(Vs).to(DEV), torch.stack(sT).to(DEV), torch.stack(zT).to(DEV),
            (perm // gs).int().to(DEV), 4)
    Xa, Xb, Xc = X.clone(), X.clone(), X.clone()
    qa = hip.gptq_sweep_direct_batched(Xa, *args)
    qb = hip.gptq_sweep_direct_batched(Xb, *args, W0=W0)
    qc = hip.gptq_sweep_direct_batched(Xc, *args, W0=W0.float())
    assert torch.equal(qa, qb) and torch.equal(qa, qc)
    assert torch.equal(Xa, Xb) and torch.equal(Xa, Xc)


@pytest.mark.parametrize("C,products", [(512, 0), (640, 3), (384, 6)])
def test_direct_sweep_reads_its_v_operand_from_the_lower_factor(hip, C, products):
    """Given the lower factor, the long block updates form their V operand from its rows
    instead of reading V: same numbers, so codes and displacements are bit-identical, also
    when everything of V beyond one block of its diagonal was never written (NaN here), when X
    itself was never laid out (NaN; the products start from the untouched copy) and for a
    matrix whose factorisation failed (V = I).  Left-looking schedule, both piece kinds."""
    B, R, gs = 3, 256, 128
    G = C // gs
    g0 = torch.Generator().manual_seed(C)
    H = torch.stack([random_problem(C=C, R=8, seed=400 + b)["H"] for b in range(B)])
    H[2] = -H[2]                                                  # not positive definite
    W = 0.02 * torch.randn(B, R, C, generator=g0)
    perm = torch.stack([torch.randperm(C, generator=g0) for _ in range(B)])
    sT, zT = [], []
    for b in range(B):
        s_, z_ = oracle.build_group_meta_packed(W[b].reshape(R * G, gs), 4, True)
        sT.append(s_.view(R, G).t().contiguous()); zT.append(z_.view(R, G).t().contiguous())
    damp = torch.full((B,), 0.01) * H.diagonal(dim1=1, dim2=2).mean(dim=1).abs()
    L, info = hip.chol_reverse_lower_batched(H.to(DEV).clone(), damp.to(DEV))
    assert info.cpu().tolist()[:2] == [0, 0] and info.cpu().tolist()[2] != 0
    X = hip.weight_to_solver_order(W.to(DEV), torch.argsort(perm, dim=1).to(DEV))
    args = (torch.stack(sT).to(DEV), torch.stack(zT).to(DEV), (perm // gs).int().to(DEV), 4)
    hip.set_option("sweep_schedule", 1)
    old = hip.set_option("sweep_update_products", products)
    try:
        assert hip.sweep_direct_reads_band_only(B, C, R)
        assert not hip.sweep_direct_reads_band_only(B, C + 4, R)       # ragged last block
        V = hip.unit_upper_from_lower(L, info, negate=True, upper_only=True)
        Xa = X.clone()
        qa = hip.gptq_sweep_direct_batched(Xa, V, *args)
        Vb = torch.full_like(V, float("nan"))
        with torch.cuda.device(DEV):
            hip._check(hip._lib.forge_unit_upper_from_lower(
                L.data_ptr(), info.data_ptr(), Vb.data_ptr(), B, C, 2 | 4 | 8, None))
        idx = torch.arange(C, device=DEV)
        blk = idx // 128
        upper = idx[None, :] >= idx[:, None]                          # row t, column k >= t
        in_band = upper & (blk[None, :] <= blk[:, None] + 1)
        assert torch.equal(Vb[:, in_band], V[:, in_band])
        assert torch.isnan(Vb[:, upper & ~in_band]).all()
        Xb = X.clone()
        qb = hip.gptq_sweep_direct_batched(Xb, Vb, *args, L=L, info=info)
        assert torch.equal(qa, qb) and torch.equal(Xa, Xb)
        # X not laid out at all: every block is first written by its long product, which then
        # starts from the untouched copy (f32 here; bf16 in the layout-pass test's shapes)
        Xc = torch.full_like(X, float("nan"))
        qc = hip.gptq_sweep_direct_batched(Xc, Vb, *args, W0=X.clone(), L=L, info=info, x_from_w0=True)
        assert torch.equal(qa, qc) and torch.equal(Xa, Xc)
        Wb = W.bfloat16()
        X0 = torch.empty((B, C, R), dtype=torch.bfloat16, device=DEV)
        pinv = torch.argsort(perm, dim=1).to(DEV)
        Xd = hip.weight_to_solver_order(Wb.to(DEV), pinv, out=torch.full_like(X, float("nan")), out0=X0,
                                        skip_out=True)
        assert torch.isnan(Xd).all()
        qd = hip.gptq_sweep_direct_batched(Xd, Vb, *args, W0=X0, L=L, info=info, x_from_w0=True)
        Xe = hip.weight_to_solver_order(Wb.to(DEV), pinv)
        qe = hip.gptq_sweep_direct_batched(Xe, V, *args)
        assert torch.equal(qd, qe) and torch.equal(Xd, Xe)
    finally:
        hip.set_option("sweep_update_products", old)
        hip.set_option("sweep_schedule", 0)


@pytest.mark.parametrize("C,R,n", [(256, 64, 500), (512, 256, 300), (200, 33, 150)])
def test_direct_sparse14_sweep_bit_exact(hip, C, R, n):
    """1:4 joint solve in the displacement form against its CPU checker: codes and masks bit
    for bit with the fp32 chain; with the bf16-piece block updates only near-ties move."""
    gs = 128
    G = (C + gs - 1) // gs
    pr = random_problem(C=C, R=R, n=n, seed=C)
    H = pr["H"].double().numpy()
    V = torch.from_numpy(mathref.direct_factor(H, 0.01)).float().contiguous()
    Hd = 0.5 * (H + H.T)
    Hd[np.diag_indices(C)] += 0.01 * np.mean(np.diag(H))
    mdiag = torch.from_numpy(np.diag(np.linalg.cholesky(Hd[::-1, ::-1])[::-1, ::-1]).copy()).float()
    Wt = pr["W"].t().contiguous()
    qd, Md = oracle.sparsegptq14_solver_direct(Wt.clone(), V, mdiag, pr["se"], pr["ze"], 4)
    args = (V.view(1, C, C).to(DEV), pr["s"].view(R, G).t().contiguous().view(1, G, R).to(DEV),
            pr["z"].view(R, G).t().contiguous().view(1, G, R).to(DEV),
            (torch.arange(C) // gs).int().view(1, C).to(DEV), 4)
    kw = dict(sparse14=True, mdiag=mdiag.view(1, C).to(DEV))
    q, M = hip.gptq_sweep_direct_batched(Wt.clone().view(1, C, R).to(DEV), *args, exact_chain=True, **kw)
    assert torch.equal(qd, q[0].cpu())
    assert torch.equal(Md.view(torch.int32), M[0].cpu().view(torch.int32))
    q2, M2 = hip.gptq_sweep_direct_batched(Wt.clone().view(1, C, R).to(DEV), *args, **kw)
    assert (q2 != q).float().mean().item() <= 3e-3
    assert (M2.view(torch.int32) != M.view(torch.int32)).float().mean().item() <= 3e-3


def test_sweep_schedules_and_block_update_kernels_agree(hip, monkeypatch):
    """32 matrices of 512 rows (128 row tiles: the left-looking schedule by default).  The
    reference-form sweep gives the same codes under both schedules; the displacement form
    gives the same codes under both schedules with the fp32 chain, and with the bf16-piece
    block updates (left-looking only) all but near-ties."""
    B, C, R, gs = 32, 512, 512, 128
    G = C // gs
    g = torch.Generator().manual_seed(41)
    X = (0.02 * torch.randn(B, C, R, generator=g)).to(DEV)
    A = torch.randn(B, 2 * C, C, generator=g).to(DEV)
    H = (2.0 / (2 * C)) * A.transpose(1, 2) @ A
    damp = 0.01 * torch.diagonal(H, dim1=1, dim2=2).mean(1)
    U, _, info = hip.chol_inv_upper_batched(H.clone(), damp)
    L, info2 = hip.chol_reverse_lower_batched(H.clone(), damp)
    assert not info.any() and not info2.any()
    V = hip.unit_upper_from_lower(L, info2, negate=True, upper_only=True)
    amax = X.view(B, G, gs, R).abs().amax(2)
    sT = (2.0 / 15.0 * amax + 1e-12).contiguous()
    zT = torch.full_like(sT, 8.0)
    gi = (torch.arange(C) // gs).int().repeat(B, 1).to(DEV)
    out = {}
    try:
        for code, sched in ((1, "left"), (2, "right")):
            hip.set_option("sweep_schedule", code)
            out["ref", sched] = hip.gptq_sweep_batched(X.clone(), U, sT, zT, gi, 4)
            out["direct", sched] = hip.gptq_sweep_direct_batched(X.clone(), V, sT, zT, gi, 4, exact_chain=True)
    finally:
        hip.set_option("sweep_schedule", 0)
    assert torch.equal(out["ref", "left"], out["ref", "right"])
    assert torch.equal(out["direct", "left"], out["direct", "right"])
    q_bf16 = hip.gptq_sweep_direct_batched(X.clone(), V, sT, zT, gi, 4)
    assert (q_bf16 != out["direct", "left"]).float().mean().item() <= 1e-3
    assert (out["ref", "left"] != out["direct", "left"]).float().mean().item() <= 3e-3


def test_direct_factor_on_the_gpu(hip):
    """chol_reverse_lower_batched + unit_upper_from_lower(negate=True) give the V of the
    displacement form: against float64, and I - strict(V) inverts the reference's factor."""
    C = 384
    pr = random_problem(C=C, R=8, n=200, seed=31)
    H = pr["H"]
    damp = (0.01 * torch.diagonal(H).mean()).view(1)
    L, info = hip.chol_reverse_lower_batched(H.clone().view(1, C, C).to(DEV), damp.to(DEV))
    assert info.tolist() == [0]
    V = hip.unit_upper_from_lower(L, info, negate=True)[0].cpu().double().numpy()
    Up = hip.unit_upper_from_lower(L, info)[0].cpu().double().numpy()
    assert np.array_equal(V, 2 * np.eye(C) - Up)
    # tiles wholly below the diagonal may be left unwritten: everything on and above it agrees
    Vu = hip.unit_upper_from_lower(L, info, negate=True, upper_only=True)[0].cpu().double().numpy()
    tiles = (np.arange(C)[:, None] // 32) <= (np.arange(C)[None, :] // 32)
    assert np.array_equal(Vu[tiles], V[tiles])
    ref = mathref.direct_factor(H.double().numpy(), 0.01)
    assert np.linalg.norm(V - ref) / np.linalg.norm(ref) < 2e-5
    Ut = mathref.factor(H.double().numpy(), 0.01)
    assert np.abs((2 * np.eye(C) - V) @ Ut - np.eye(C)).max() < 1e-3


@pytest.mark.parametrize("spread", [0.0, 4.0])
def test_factor_of_h_from_fp16_halves(hip, spread):
    """Where only the factor of H is needed, the trailing updates form every fp32 product from
    two fp16 halves of the operands (three products), each column scaled by a power of two
    taken from its diagonal entry.  Against float64 it must be as accurate as the three-bf16-
    thirds form (six products), also when the diagonal spans 16 orders of magnitude (feature
    scales 1e-4 .. 1e4) and the batch mixes differently scaled matrices."""
    C, B = 640, 3
    g = torch.Generator().manual_seed(17)
    Hs = []
    for b in range(B):
        X = torch.randn(900, C, generator=g, dtype=torch.float64)
        X = X * (10.0 ** (spread * (2 * torch.rand(C, generator=g, dtype=torch.float64) - 1))) * 10.0 ** (b - 1)
        Hs.append((2.0 / 900) * X.T @ X)
    H = torch.stack(Hs)
    damp = 1e-4 * torch.diagonal(H, dim1=1, dim2=2).mean(1)       # small: the spread stays in the factor
    Hd = H + torch.diag_embed(damp[:, None].expand(B, C))
    errs = {}
    for tag, opt in (("halves", 0), ("thirds", 1)):
        old = hip.set_option("factor_pieces", opt)
        try:
            L, info = hip.chol_reverse_lower_batched(H.float().to(DEV), damp.float().to(DEV))
        finally:
            hip.set_option("factor_pieces", old)
        assert info.tolist() == [0] * B
        worst = 0.0
        for b in range(B):
            A = Hd[b].float().double().numpy()            # what the GPU was given
            Lr = np.linalg.cholesky(A[::-1, ::-1])[::-1, ::-1].T    # A = L2^T L2, L2 lower
            d = 1.0 / np.sqrt(np.diag(A))
            got = np.tril(L[b].cpu().double().numpy())
            worst = max(worst, np.linalg.norm((got - Lr) * d[None, :]) / np.linalg.norm(Lr * d[None, :]))
        errs[tag] = worst
    print(f"spread 1e+-{spread}: equilibrated factor error halves {errs['halves']:.2e} thirds {errs['thirds']:.2e}")
    assert errs["halves"] <= 1.5 * errs["thirds"] + 1e-7
    assert errs["halves"] < (2e-3 if spread else 1e-5)


def test_full_size_sweep_properties(hip):
    """Config-1 size (2048 x 2048): U = I must give round-to-nearest bit for bit, and the
    batched (left-looking) and single-matrix (right-looking) schedules must agree."""
    C = R = 2048
    pr = random_problem(C=C, R=R, n=1024, seed=7)
    Wt = pr["W"].t().contiguous().to(DEV)
    se, ze = pr["se"].to(DEV), pr["ze"].to(DEV)
    q_rtn = hip.gptq_solver(Wt.clone(), torch.eye(C, device=DEV), se, ze, 4)
    ref = torch.clamp(torch.round(torch.addcmul(ze.double(), Wt.double(), (1.0 / (se + 1e-12)).double()).float()), 0, 15)
    assert torch.equal(q_rtn.float(), ref)
    U = pr["U"].to(DEV)
    q_single = hip.gptq_solver(Wt.clone(), U, se, ze, 4)
    G = C // 128
    q_batched = hip.gptq_sweep_batched(Wt.clone().view(1, C, R), U.view(1, C, C),
                                       pr["s"].view(R, G).t().contiguous().view(1, G, R).to(DEV),
                                       pr["z"].view(R, G).t().contiguous().view(1, G, R).to(DEV),
                                       (torch.arange(C) // 128).int().view(1, C).to(DEV), 4)
    assert torch.equal(q_single, q_batched[0])
    q0 = oracle.gptq_solver(pr["W"].t().contiguous(), pr["U"], pr["se"], pr["ze"], 4)
    assert torch.equal(q0, q_single.cpu())
