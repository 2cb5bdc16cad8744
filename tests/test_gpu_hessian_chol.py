"""HIP Hessian accumulation, factorisation and layout kernels against float64 closed forms."""
import numpy as np
import pytest
import torch

from oracle import mathref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, b):
    a, b = a.double().cpu(), torch.as_tensor(b).double()
    return ((a - b).norm() / b.norm()).item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("C", [256, 200, 1000])
def test_grouped_ragged_hessian(hip, dtype, C):
    counts = [0, 3, 17, 300, 64, 0, 129]
    offs = np.concatenate([[0], np.cumsum(counts)])
    g = torch.Generator().manual_seed(C)
    X = torch.randn(int(offs[-1]), C, generator=g).to(dtype)
    E = len(counts)
    H = torch.full((E, C, C), float("nan"), device=DEV)
    hip.hessian_update_grouped(X.to(DEV), offs, H, [2.0 / max(c, 1) for c in counts], [0.0] * E)
    for e, c in enumerate(counts):
        if c == 0:
            assert bool(torch.isnan(H[e]).all())            # zero-token expert: untouched
            continue
        ref = mathref.hessian([X[offs[e]:offs[e + 1]].double().numpy()])
        assert _rel(H[e], ref) < 2e-6
        assert torch.equal(H[e], H[e].t())                  # exactly symmetric
    # second batch: running mean H <- (n/N) H + (2/N) X^T X   (gptq.py:73-79)
    X2 = torch.randn(int(offs[-1]), C, generator=g).to(dtype)
    hip.hessian_update_grouped(X2.to(DEV), offs, H, [2.0 / max(2 * c, 1) for c in counts], [0.5] * E)
    for e in (1, 3, 6):
        ref = mathref.hessian([X[offs[e]:offs[e + 1]].double().numpy(),
                               X2[offs[e]:offs[e + 1]].double().numpy()])
        assert _rel(H[e], ref) < 2e-6 and torch.equal(H[e], H[e].t())


@pytest.mark.parametrize("C", [256, 768])
def test_grouped_hessian_heavy_and_light_groups_in_one_call(hip, C):
    """Groups with 512 tokens and more take the 256 x 256 workgroup tiles with operands staged
    through LDS, the others (in the same call) the one-pass kernel; token counts that are not
    multiples of the 64-token stage, an empty group between them, then a running-mean update."""
    counts = [700, 5, 0, 1030, 513, 511, 64]
    offs = np.concatenate([[0], np.cumsum(counts)])
    g = torch.Generator().manual_seed(C + 1)
    X = torch.randn(int(offs[-1]), C, generator=g).bfloat16()
    E = len(counts)
    H = torch.full((E, C, C), float("nan"), device=DEV)
    hip.hessian_update_grouped(X.to(DEV), offs, H, [2.0 / max(c, 1) for c in counts], [0.0] * E)
    for e, c in enumerate(counts):
        if c == 0:
            assert bool(torch.isnan(H[e]).all())
            continue
        ref = mathref.hessian([X[offs[e]:offs[e + 1]].double().numpy()])
        assert _rel(H[e], ref) < 2e-6, (e, c)
        assert torch.equal(H[e], H[e].t())
    X2 = torch.randn(int(offs[-1]), C, generator=g).bfloat16()
    hip.hessian_update_grouped(X2.to(DEV), offs, H, [2.0 / max(2 * c, 1) for c in counts], [0.5] * E)
    for e, c in enumerate(counts):
        if c:
            ref = mathref.hessian([X[offs[e]:offs[e + 1]].double().numpy(),
                                   X2[offs[e]:offs[e + 1]].double().numpy()])
            assert _rel(H[e], ref) < 2e-6 and torch.equal(H[e], H[e].t())
    # every group heavy: only the big-tile kernel runs
    Hb = torch.full((2, C, C), float("nan"), device=DEV)
    hip.hessian_update_grouped(X[:1400].to(DEV), [0, 700, 1400], Hb, [2.0 / 700] * 2, [0.0] * 2)
    assert torch.equal(Hb[0], H.new_tensor(0) + Hb[0]) and _rel(Hb[0], mathref.hessian([X[:700].double().numpy()])) < 2e-6
    assert _rel(Hb[1], mathref.hessian([X[700:1400].double().numpy()])) < 2e-6


def test_hessian_strided_rows_and_empty_call(hip):
    X = torch.randn(40, 300, device=DEV).bfloat16()[:, :256]          # row pitch 300
    H = torch.zeros((1, 256, 256), device=DEV)
    hip.hessian_update_grouped(X, [0, 40], H, [2.0 / 40], [0.0])
    assert _rel(H[0], mathref.hessian([X.double().cpu().numpy()])) < 2e-6
    before = H.clone()
    hip.hessian_update_grouped(X, [7, 7], H, [1.0], [0.0])            # no rows: no-op
    assert torch.equal(before, H)


@pytest.mark.parametrize("C", [128, 256, 200, 36, 1024])
@pytest.mark.parametrize("normalise", [True, False])
def test_factor_matches_float64(hip, C, normalise):
    B = 3
    Hs = []
    for b in range(B):
        g = torch.Generator().manual_seed(10 * C + b)
        X = torch.randn(2 * C if b < 2 else max(C // 2, 4), C, generator=g, dtype=torch.float64)
        X[:, :3] *= 8
        Hs.append((2.0 / X.shape[0]) * X.T @ X)
    H = torch.stack(Hs).float()
    damp = (0.01 * torch.diagonal(H, dim1=1, dim2=2).mean(1)).float()
    U, ud, info = hip.chol_inv_upper_batched(H.clone().to(DEV), damp.to(DEV), normalise=normalise)
    assert info.tolist() == [0] * B
    for b in range(B):
        Hd = H[b].double().numpy().copy()
        Hd[np.diag_indices(C)] += float(damp[b])
        U0 = np.linalg.cholesky(np.linalg.inv(Hd)).T
        ref = U0 / np.diag(U0)[:, None] if normalise else U0
        # rank-deficient Hessian (b == 2) is far worse conditioned
        assert _rel(U[b], ref) < (2e-4 if b == 2 else 5e-6)
        assert _rel(ud[b], np.diag(U0).copy()) < (1e-4 if b == 2 else 5e-6)
        assert int((torch.tril(U[b], -1) != 0).sum()) == 0
        if normalise:
            assert bool((U[b].diagonal() == 1).all())


@pytest.mark.parametrize("B,C", [(8, 1536), (3, 640)])
def test_factor_bf16_split_and_fp32_updates_agree(hip, monkeypatch, B, C):
    """C a multiple of 128: the trailing updates run as three-piece bf16 products by default
    and as fp32 blocked sums with the option fp32_blocked_sum = 1; both are fp32-accurate."""
    g = torch.Generator().manual_seed(C)
    X = torch.randn(B, 2 * C, C, generator=g, dtype=torch.float64)
    X[:, :, :5] *= 6
    H = ((2.0 / X.shape[1]) * X.transpose(1, 2) @ X).float()
    H[B - 1, 7, 7] = float("nan")                       # one failing matrix among the good ones
    damp = (0.01 * torch.diagonal(H[:B - 1], dim1=1, dim2=2).mean()).repeat(B).float()
    assert hip.get_option("fp32_blocked_sum") == 0
    Us, uds, infos = hip.chol_inv_upper_batched(H.clone().to(DEV), damp.to(DEV))
    hip.set_option("fp32_blocked_sum", 1)
    try:
        Uf, udf, infof = hip.chol_inv_upper_batched(H.clone().to(DEV), damp.to(DEV))
        # upper_only: same values on and above the diagonal blocks, nothing promised left of them
        Uu, _, _ = hip.chol_inv_upper_batched(H.clone().to(DEV), damp.to(DEV), upper_only=True)
    finally:
        hip.set_option("fp32_blocked_sum", 0)
    assert torch.equal(torch.triu(Uu), torch.triu(Uf))
    assert infos.tolist()[:B - 1] == [0] * (B - 1) and infos[B - 1].item() > 0
    assert infof.tolist() == infos.tolist()
    assert torch.equal(Us[B - 1].cpu(), torch.eye(C))
    for b in range(B - 1):
        Hd = H[b].double().numpy().copy()
        Hd[np.diag_indices(C)] += float(damp[b])
        U0 = np.linalg.cholesky(np.linalg.inv(Hd)).T
        ref = U0 / np.diag(U0)[:, None]
        es, ef = _rel(Us[b], ref), _rel(Uf[b], ref)
        assert es < 5e-6 and ef < 5e-6 and es < 2 * ef + 1e-7
        assert int((torch.tril(Us[b], -1) != 0).sum()) == 0


def test_factor_failure_gives_identity(hip):
    H = torch.eye(256).repeat(3, 1, 1)
    H[1, 100, 100] = -1.0                               # not positive definite
    H[2, 5, 5] = float("nan")
    U, ud, info = hip.chol_inv_upper_batched(H.to(DEV), torch.zeros(3, device=DEV))
    assert info[0].item() == 0 and info[1].item() > 0 and info[2].item() > 0
    for b in range(3):
        assert torch.equal(U[b].cpu(), torch.eye(256))


def test_layout_kernels(hip):
    B, R, C = 2, 192, 320
    g = torch.Generator().manual_seed(0)
    W = torch.randn(B, R, C, generator=g).bfloat16()
    perm = torch.stack([torch.randperm(C, generator=g) for _ in range(B)])
    pinv = torch.argsort(perm, dim=1)
    dead = (torch.rand(B, C, generator=g) < 0.05).to(torch.uint8)
    Xo = hip.weight_to_solver_order(W.to(DEV), pinv.to(DEV), dead.to(DEV))
    q = torch.randint(0, 16, (B, C, R), dtype=torch.uint8, generator=g)
    qo = hip.codes_to_layer_order(q.to(DEV), pinv.to(DEV))
    Hh = torch.randn(B, C, C, generator=g)
    Hh = Hh + Hh.transpose(1, 2)
    Hp, dmp = hip.hessian_permute(Hh.to(DEV), perm.to(DEV), dead.to(DEV), 0.01)
    for b in range(B):
        Wz = W[b].float().clone()
        Wz[:, dead[b].bool()] = 0
        assert torch.equal(Xo[b].cpu(), Wz.t()[perm[b]].contiguous())          # W.T[perm]
        assert torch.equal(qo[b].cpu(), q[b][pinv[b]].t().contiguous())        # q[perm_inv].T
        ref = Hh[b][perm[b]][:, perm[b]].clone()
        d = dead[b].bool()
        ref[d, :] = 0; ref[:, d] = 0; ref[d, d] = 1
        assert torch.equal(Hp[b].cpu(), ref)
        assert dmp[b].item() == pytest.approx(0.01 * ref.diag().mean().item(), rel=1e-5)
    Wf = torch.randn(1, 50, 70, generator=g)                                    # f32, ragged tile
    ident = torch.arange(70).view(1, 70)
    assert torch.equal(hip.weight_to_solver_order(Wf.to(DEV), ident.to(DEV)).cpu()[0], Wf[0].t().contiguous())


def test_pack_int4_layout(hip):
    """compressed-tensors 'pack-quantized' int4: eight (code - zero) values per int32,
    offset binary (+8), lowest nibble first, along the input dimension
    (consumer: pack_quantized.py:279-313).  parity unpinned against the third-party packer
    itself (not installed here); pinned against its documented layout."""
    R, C, gs = 33, 330, 128
    g = torch.Generator().manual_seed(1)
    codes = torch.randint(0, 16, (R, C), dtype=torch.uint8, generator=g)
    G = (C + gs - 1) // gs
    z = torch.randint(0, 16, (R * G,), generator=g).float()
    pk = hip.pack_int4(codes.to(DEV), z.to(DEV), gs).cpu()
    zz = z.view(R, G).repeat_interleave(gs, 1)[:, :C].to(torch.int64)
    sh = (codes.to(torch.int64) - zz + 8) & 0xF
    sh = torch.nn.functional.pad(sh, (0, (-C) % 8)).view(R, -1, 8)
    ref = sum(sh[:, :, k] << (4 * k) for k in range(8))
    assert torch.equal(pk.to(torch.int64) & 0xFFFFFFFF, ref)
    pk8 = hip.pack_int4(codes.to(DEV), None, gs).cpu()                 # symmetric: zero = 8
    sh = torch.nn.functional.pad(codes.to(torch.int64), (0, (-C) % 8)).view(R, -1, 8)
    assert torch.equal(pk8.to(torch.int64) & 0xFFFFFFFF, sum(sh[:, :, k] << (4 * k) for k in range(8)))

@pytest.mark.gpu
@pytest.mark.parametrize("C,gs", [(1024, 128), (1024, 32), (1040, 128), (1008, 48), (1000, 40), (1000, 64)])
def test_pack_int4_aligned_rows(hip, C, gs):
    """C and the group size multiples of 16 (16-byte loads, groups tiling the row or not) or of
    8 (8-byte loads): same words as the general form."""
    R = 96
    g = torch.Generator().manual_seed(2)
    codes = torch.randint(0, 16, (R, C), dtype=torch.uint8, generator=g)
    G = (C + gs - 1) // gs
    z = torch.randint(0, 16, (R * G,), generator=g).float()
    for zeros in (z, None):
        pk = hip.pack_int4(codes.to(DEV), None if zeros is None else zeros.to(DEV), gs).cpu()
        zz = 8 if zeros is None else z.view(R, G).repeat_interleave(gs, 1)[:, :C].to(torch.int64)
        sh = ((codes.to(torch.int64) - zz + 8) & 0xF).view(R, -1, 8)
        ref = sum(sh[:, :, k] << (4 * k) for k in range(8))
        assert torch.equal(pk.to(torch.int64) & 0xFFFFFFFF, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("B,R,C", [(2, 512, 384), (1, 256, 1152)])
def test_layout_kernels_tall_tiles(hip, B, R, C):
    """bf16 weights with R % 256 == 0 and C % 128 == 0 take the tall-tile transposes."""
    g = torch.Generator().manual_seed(3)
    W = torch.randn(B, R, C, generator=g).bfloat16()
    perm = torch.stack([torch.randperm(C, generator=g) for _ in range(B)])
    pinv = torch.argsort(perm, dim=1)
    dead = (torch.rand(B, C, generator=g) < 0.05).to(torch.uint8)
    Xo = hip.weight_to_solver_order(W.to(DEV), pinv.to(DEV), dead.to(DEV))
    Xn = hip.weight_to_solver_order(W.to(DEV), pinv.to(DEV))
    q = torch.randint(0, 16, (B, C, R), dtype=torch.uint8, generator=g)
    qo = hip.codes_to_layer_order(q.to(DEV), pinv.to(DEV))
    for b in range(B):
        Wz = W[b].float().clone()
        assert torch.equal(Xn[b].cpu(), Wz.t()[perm[b]].contiguous())
        Wz[:, dead[b].bool()] = 0
        assert torch.equal(Xo[b].cpu(), Wz.t()[perm[b]].contiguous())
        assert torch.equal(qo[b].cpu(), q[b][pinv[b]].t().contiguous())


@pytest.mark.gpu
@pytest.mark.parametrize("C", [70, 1028, 2564, 4104])
def test_hessian_permute_sizes(hip, C):
    """Scalar form (C % 4 != 0) and the 2-, 4- and 8-chunk row forms, with a ragged last
    group of rows and dead columns."""
    g = torch.Generator().manual_seed(C)
    Hh = torch.randn(1, C, C, generator=g)
    Hh = Hh + Hh.transpose(1, 2)
    perm = torch.randperm(C, generator=g).view(1, C)
    dead = (torch.rand(1, C, generator=g) < 0.02).to(torch.uint8)
    Hp, dmp = hip.hessian_permute(Hh.to(DEV), perm.to(DEV), dead.to(DEV), 0.01)
    ref = Hh[0][perm[0]][:, perm[0]].clone()
    d = dead[0].bool()
    ref[d, :] = 0; ref[:, d] = 0; ref[d, d] = 1
    assert torch.equal(Hp[0].cpu(), ref)
    assert dmp[0].item() == pytest.approx(0.01 * ref.diag().mean().item(), rel=1e-5)
    # the form that writes, in each row, only up to the end of the row's own 128-column block
    # (the scalar form writes everything): equal there, and the same damping
    Hl, dl = hip.hessian_permute(Hh.to(DEV), perm.to(DEV), dead.to(DEV), 0.01, lower_blocks=True)
    idx = torch.arange(C)
    keep = (idx[None, :] // 128) <= (idx[:, None] // 128)
    assert torch.equal(Hl[0].cpu()[keep], ref[keep]) and torch.equal(dl, dmp)



