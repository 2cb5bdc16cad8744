"""Write-back dequant and the routed-row gather in front of the per-expert Hessians
(the callers either side of the solve)."""
import numpy as np
import pytest
import torch

import oracle

DEV = "cuda"


# ------------------------------------------------------------------ oracle pins (CPU)
def test_oracle_dequantize_closed_form():
    """(q - q0) * s element by element in numpy float32, ragged last group included."""
    R, C, gs = 5, 300, 128
    g = torch.Generator().manual_seed(0)
    q = torch.randint(0, 16, (R, C), dtype=torch.uint8, generator=g)
    G = (C + gs - 1) // gs
    s = torch.rand(R * G, generator=g) * 0.02 + 1e-4
    z = torch.randint(0, 16, (R * G,), generator=g).float()
    got = oracle.dequantize(q, s, z, gs).numpy()
    qn, sn, zn = q.numpy().astype(np.float32), s.numpy().reshape(R, G), z.numpy().reshape(R, G)
    for r in range(R):
        for c in range(C):
            assert got[r, c] == np.float32(np.float32(qn[r, c] - zn[r, c // gs]) * sn[r, c // gs])


def test_oracle_routed_rows_brute_force():
    """Every (token, k) pair lands once, under its expert, in ascending token order, scaled
    by its own routing weight."""
    T, H, E, K = 37, 16, 6, 3
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).bfloat16()
    ri = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    rw = torch.rand(T, K, generator=g)
    rows, offs = oracle.routed_rows(x, ri, rw, E)
    assert offs[0] == 0 and offs[-1] == T * K and len(offs) == E + 1
    for e in range(E):
        want = []
        for t in range(T):
            for k in range(K):
                if int(ri[t, k]) == e:
                    w = rw[t, k].to(torch.bfloat16)
                    want.append((x[t].float() * w.float()).to(torch.bfloat16))
        got = rows[offs[e]:offs[e + 1]]
        assert got.shape[0] == len(want)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
    plain, offs2 = oracle.routed_rows(x, ri, None, E)
    assert offs2 == offs and torch.equal(plain[offs[2]:offs[3]], x[(ri == 2).any(1).nonzero().flatten()])


# ------------------------------------------------------------------ HIP parity (bit-exact)
@pytest.mark.gpu
@pytest.mark.parametrize("B,R,C,gs", [(1, 33, 300, 128), (3, 64, 1024, 128), (2, 7, 70, 32),
                                      (2, 5, 1040, 128), (1, 3, 20480, 48), (2, 9, 1024, 40)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dequantize_groups_matches_oracle(hip, B, R, C, gs, dtype):
    g = torch.Generator().manual_seed(C)
    q = torch.randint(0, 16, (B, R, C), dtype=torch.uint8, generator=g)
    G = (C + gs - 1) // gs
    s = torch.rand(B, R * G, generator=g) * 0.02 + 1e-4
    z = torch.randint(0, 16, (B, R * G), generator=g).float()
    got = hip.dequantize_groups(q.to(DEV), s.to(DEV), z.to(DEV), gs, dtype).cpu()
    for b in range(B):
        assert torch.equal(got[b], oracle.dequantize(q[b], s[b], z[b], gs).to(dtype))


@pytest.mark.gpu
def test_dequantize_forge_full_signature_and_errors(hip):
    from forge.engine import dequantize_forge_full
    g = torch.Generator().manual_seed(2)
    q = torch.randint(0, 16, (16, 256), dtype=torch.uint8, generator=g)
    s = torch.rand(16 * 2, generator=g) * 0.01 + 1e-4
    z = torch.full((16 * 2,), 8.0)
    w = dequantize_forge_full(torch.bfloat16, q, s, z, 128, DEV)
    assert w.dtype == torch.bfloat16 and w.device.type == "cuda"
    assert torch.equal(w.cpu(), oracle.dequantize(q, s, z, 128).to(torch.bfloat16))
    with pytest.raises(ValueError):
        dequantize_forge_full(torch.bfloat16, q.view(-1), s, z, 128, DEV)
    with pytest.raises(ValueError):
        dequantize_forge_full(torch.bfloat16, q, s[:-1], z, 128, DEV)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H", [64, 70, 2048])
def test_gather_scaled_rows_matches_oracle(hip, dtype, H):
    g = torch.Generator().manual_seed(H)
    T, N = 50, 131
    x = torch.randn(T, H + 6, generator=g).to(dtype)[:, :H]                # row pitch H + 6
    idx = torch.randint(0, T, (N,), generator=g)
    w = torch.rand(N, generator=g)
    got = hip.gather_scaled_rows(x.to(DEV), idx.to(DEV), w.to(DEV)).cpu()
    assert torch.equal(got, oracle.gather_scaled_rows(x, idx, w))
    plain = hip.gather_scaled_rows(x.to(DEV), idx.to(DEV)).cpu()
    assert torch.equal(plain, x[idx])
    empty = hip.gather_scaled_rows(x.to(DEV), idx[:0].to(DEV))
    assert tuple(empty.shape) == (0, H)


@pytest.mark.gpu
def test_routed_rows_feed_the_grouped_hessian(hip):
    """Hook front end -> grouped Hessian update: equals the oracle's per-expert loop, and the
    Hessians equal the closed form on the scaled rows."""
    from forge.engine import routed_rows
    from oracle import mathref
    T, H, E, K = 300, 256, 8, 2
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=g).bfloat16()
    logits = torch.randn(T, E, generator=g)
    logits[:, 3] = -1e9                                                    # expert 3 gets no token
    rw, ri = torch.softmax(logits, -1).topk(K, dim=-1)
    ri = ri.clone(); ri[0, 0] = -1                                         # dropped entry
    rows, offs = routed_rows(x.to(DEV), ri.to(DEV), rw.to(DEV), E)
    want, woffs = oracle.routed_rows(x, ri, rw, E)
    assert offs == woffs and offs[4] == offs[3]
    assert torch.equal(rows.cpu(), want)
    Hs = torch.zeros(E, H, H, device=DEV)
    counts = [offs[e + 1] - offs[e] for e in range(E)]
    hip.hessian_update_grouped(rows, offs, Hs, [2.0 / max(c, 1) for c in counts], [0.0] * E)
    for e in (0, 5):
        ref = mathref.hessian([want[offs[e]:offs[e + 1]].double().numpy()])
        rel = (Hs[e].cpu().double() - torch.from_numpy(ref)).norm() / torch.from_numpy(ref).norm()
        assert rel < 2e-6
