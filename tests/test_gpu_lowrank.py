"""The low-rank route (layers that saw at most 128 calibration rows) against dense float64
algebra and against the route through the Hessian.

The closed forms are pinned by the dense computation they replace: the lower factor M of
D + B^T B (H = M^T M, numpy float64 Cholesky of the index-reversed matrix) gives
M[k,t] / M[k,k], which must equal Hm[k] . Bp[t]; the sweep is compared with a float64
column-by-column GPTQ on the dense factor of inv(H) (the reference's own form,
gptq.py:160-164 and solver.cu:9-154), i.e. with a different formula, not a retyped one.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import linear, flip_rate, codes_at_floor

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _lower_factor(H):
    """M lower with H = M^T M (elimination from the last row upwards), float64."""
    G = np.linalg.cholesky(H[::-1, ::-1])
    return np.ascontiguousarray(G.T[::-1, ::-1])


def _problem(C, n, seed, dead=()):
    g = torch.Generator().manual_seed(seed)
    Bp = torch.zeros(C, 4 if 0 < n <= 4 else 16 if n <= 16 else 32 if n <= 32 else 64 if n <= 64 else 128)
    Bp[:, :n] = torch.randn(C, n, generator=g) * (2.0 / max(n, 1)) ** 0.5
    Bp[:, 0] *= torch.linspace(3.0, 0.3, C)                 # an "activation-ordered" spread
    D = torch.full((C,), 0.02)
    for k in dead:
        Bp[k] = 0
        D[k] += 1.0
    return Bp, D


@pytest.mark.parametrize("n", [0, 1, 3, 5, 16, 23, 64, 100, 128])
def test_factor_matches_the_dense_float64_factor(hip, n):
    C = 384
    probs = [_problem(C, n, s, dead=(7, 200) if s == 1 else ()) for s in range(3)]
    Bp = torch.stack([p[0] for p in probs]).to(DEV)
    D = torch.stack([p[1] for p in probs]).to(DEV)
    Hm, info = hip.lowrank_factor(Bp, D)
    assert info.cpu().tolist() == [0, 0, 0]
    for b, (B1, D1) in enumerate(probs):
        Bd = B1.double().numpy()
        H = np.diag(D1.double().numpy()) + Bd @ Bd.T
        M = _lower_factor(H)
        want = np.tril(M / np.diag(M)[:, None], -1)          # [k, t], t < k
        got = np.tril(Hm[b].cpu().double().numpy() @ Bd.T, -1)
        scale = max(1.0, float(np.abs(want).max()))
        assert float(np.abs(got - want).max()) <= 2e-6 * scale, (n, b)
    # a pivot that is not positive is reported, not divided by
    Dbad = D.clone()
    Dbad[1, 5] = -1e9
    assert hip.lowrank_factor(Bp, Dbad)[1].cpu().tolist() == [0, 1, 0]


def _float64_gptq(W, H, s, z, maxq=15.0):
    """Column-by-column GPTQ in the reference's form: U = upper factor of inv(H), rows divided
    by their diagonal; err = x - deq is handed to the later columns.  W [R, C] float64."""
    Hinv = np.linalg.inv(H)
    U = np.ascontiguousarray(np.linalg.cholesky(Hinv).T)    # upper, U^T U = inv(H)
    U = U / np.diag(U)[:, None]
    X = W.copy()
    Q = np.zeros_like(W)
    margin = np.full(W.shape, np.inf)
    for t in range(W.shape[1]):
        v = X[:, t] / (s[:, t] + 1e-12) + z[:, t]
        q = np.clip(np.rint(v), 0, maxq)
        margin[:, t] = np.abs(v - np.floor(v) - 0.5)          # distance from a rounding tie
        Q[:, t] = q
        e = X[:, t] - (q - z[:, t]) * s[:, t]
        X[:, t + 1:] -= np.outer(e, U[t, t + 1:])
    return Q, margin


@pytest.mark.parametrize("n,dtype", [(1, torch.float32), (4, torch.bfloat16), (16, torch.bfloat16),
                                     (0, torch.float32), (30, torch.bfloat16), (64, torch.float32),
                                     (50, torch.bfloat16), (128, torch.bfloat16), (90, torch.float32), (3, torch.bfloat16)])
def test_sweep_matches_float64_gptq_on_the_dense_factor(hip, n, dtype):
    C, R, gs = 256, 300, 128
    G = C // gs
    Bp, D = _problem(C, n, 11)
    g = torch.Generator().manual_seed(5)
    W = (0.02 * torch.randn(R, C, generator=g)).to(dtype)
    s, z = oracle.build_group_meta_packed(W.float().reshape(R * G, gs), 4, False)
    perm = torch.randperm(C, generator=g)                    # groups follow an arbitrary order
    g_idx = (perm // gs).to(torch.int32)
    W0 = W[:, perm].t().contiguous()                         # [C, R] solver order
    sT = s.view(R, G).t().contiguous()
    zT = z.view(R, G).t().contiguous()
    Hm, info = hip.lowrank_factor(Bp[None].to(DEV), D[None].to(DEV))
    q = hip.gptq_sweep_lowrank(W0[None].to(DEV), Bp[None].to(DEV), Hm, info, sT[None].to(DEV),
                               zT[None].to(DEV), g_idx[None].to(DEV), 4)[0].cpu()
    Bd = Bp.double().numpy()
    H = np.diag(D.double().numpy()) + Bd @ Bd.T
    se = sT[g_idx.long()].t().double().numpy()               # [R, C] per element, solver order
    ze = zT[g_idx.long()].t().double().numpy()
    Q, margin = _float64_gptq(W0.t().double().numpy(), H, se, ze)
    diff = q.t().double().numpy() != Q
    print(f"n={n}: {diff.mean():.2e} of the codes differ from float64 GPTQ")
    # fp32 against float64: rows may part ways at a near-tie and then stay apart; up to the
    # first difference of a row everything must agree, and that first difference must be a
    # near-tie of the rounding
    for r in np.nonzero(diff.any(1))[0]:
        c = int(np.argmax(diff[r]))
        assert margin[r, c] < 1e-3, (r, c, margin[r, c])
    assert diff.any(1).mean() <= 0.05
    if n == 0:
        assert diff.sum() <= 1                               # no coupling: plain rounding


def test_failed_factor_sweeps_uncoupled(hip):
    C, R, gs = 128, 64, 128
    Bp, D = _problem(C, 3, 2)
    g = torch.Generator().manual_seed(1)
    W0 = 0.02 * torch.randn(C, R, generator=g)
    s, z = oracle.build_group_meta_packed(W0.t().contiguous().reshape(R, gs), 4, True)
    g_idx = torch.zeros(C, dtype=torch.int32)
    args = (s.view(1, 1, R).to(DEV), z.view(1, 1, R).to(DEV), g_idx[None].to(DEV), 4)
    Hm = torch.full((1, C, Bp.shape[1]), float("nan"), device=DEV)  # never read
    bad = torch.ones(1, dtype=torch.int32, device=DEV)
    q = hip.gptq_sweep_lowrank(W0[None].to(DEV), Bp[None].to(DEV), Hm, bad, *args)[0].cpu()
    # the quantiser's fma(x, 1/(s+eps), z): the product of two floats is exact in float64
    # (symmetric absmax scales put every group's extreme weight exactly on a rounding tie)
    inv = (1.0 / (s + 1e-12))[None, :]
    v = (W0.double() * inv.double() + z[None, :].double()).float()
    want = torch.clamp(torch.round(v), 0, 15).to(torch.uint8)
    assert torch.equal(q, want)


@pytest.mark.parametrize("dtype,C,gs", [(torch.bfloat16, 512, 128), (torch.float32, 200, 64),
                                         (torch.bfloat16, 77, 32)])
def test_round_to_nearest_is_the_quantiser_weight_by_weight(hip, dtype, C, gs):
    g = torch.Generator().manual_seed(4)
    B, R = 3, 37
    G = (C + gs - 1) // gs
    W = (0.02 * torch.randn(B, R, C + 8, generator=g)).to(dtype)[:, :, :C]     # pitched rows
    Wp = torch.nn.functional.pad(W.float(), (0, G * gs - C))
    s, z = oracle.build_group_meta_packed(Wp.reshape(B * R * G, gs), 4, False)
    s, z = s.view(B, R * G), z.view(B, R * G)
    q = hip.round_to_nearest(W.to(DEV), s.to(DEV), z.to(DEV), gs, 4).cpu()
    se = s.view(B, R, G).repeat_interleave(gs, dim=2)[:, :, :C]
    ze = z.view(B, R, G).repeat_interleave(gs, dim=2)[:, :, :C]
    inv = 1.0 / (se + 1e-12)
    v = (W.double() * inv.double() + ze.double()).float()    # fma: the product is exact in float64
    assert torch.equal(q, torch.clamp(torch.round(v), 0, 15).to(torch.uint8))


def test_hessian_ranges_skip_groups_in_place(hip):
    g = torch.Generator().manual_seed(0)
    C = 256
    X = torch.randn(50, C, generator=g).bfloat16().to(DEV)
    offs = [0, 7, 7, 30, 50]
    E = 4
    H0 = torch.randn(E, C, C, generator=g).to(DEV)
    al, be = [2 / 7, 1.0, 2 / 23, 0.1], [0.0, 0.5, 0.0, 0.5]
    want = hip.hessian_update_grouped(X, offs, H0.clone(), al, be)
    row0, counts = offs[:-1], [offs[i + 1] - offs[i] for i in range(E)]
    got = hip.hessian_update_ranges(X, row0, counts, H0.clone(), al, be)
    assert torch.equal(want, got)
    counts[2] = 0                                            # expert 2 left out: untouched
    got = hip.hessian_update_ranges(X, row0, counts, H0.clone(), al, be)
    assert torch.equal(got[2], H0[2]) and torch.equal(got[0], want[0]) and torch.equal(got[3], want[3])


def test_layout_passes_on_a_scattered_subset(hip):
    """The gather / scatter forms (one launch for a subset of a stack) against the plain forms on
    the same matrices one by one."""
    g = torch.Generator().manual_seed(6)
    B, R, C = 5, 256, 256
    W = (0.02 * torch.randn(B, R, C, generator=g)).bfloat16().to(DEV)
    perm_inv = torch.stack([torch.randperm(C, generator=g) for _ in range(B)]).to(DEV)
    dead = (torch.rand(B, C, generator=g) < 0.02).to(torch.uint8).to(DEV)
    H = torch.randn(B, C, C, generator=g).to(DEV)
    idx = torch.tensor([3, 0, 4], device=DEV)
    X = torch.empty((3, C, R), dtype=torch.float32, device=DEV)
    W0 = torch.empty((3, C, R), dtype=torch.bfloat16, device=DEV)
    hip.weight_to_solver_order(W, perm_inv, dead, out=X, out0=W0, index=idx)
    Hp, damp = hip.hessian_permute(H, perm_inv, dead, 0.01, lower_blocks=True, index=idx)
    codes = torch.randint(0, 16, (3, C, R), generator=g, dtype=torch.uint8).to(DEV)
    out = torch.zeros((B, R, C), dtype=torch.uint8, device=DEV)
    hip.codes_to_layer_order(codes, perm_inv, out=out, index=idx)
    for pos, e in enumerate(idx.tolist()):
        sl = slice(e, e + 1)
        X1 = hip.weight_to_solver_order(W[sl], perm_inv[sl].contiguous(), dead[sl].contiguous())
        assert torch.equal(X[pos], X1[0]) and torch.equal(W0[pos].float(), X1[0])
        H1, d1 = hip.hessian_permute(H[sl], perm_inv[sl].contiguous(), dead[sl].contiguous(), 0.01,
                                     lower_blocks=True)
        keep = torch.ones(C, C, dtype=torch.bool, device=DEV).tril()
        for blk in range(0, C, 128):                             # what lower_blocks writes
            keep[blk:blk + 128, :blk + 128] = True
        assert torch.equal(Hp[pos][keep], H1[0][keep]) and torch.equal(damp[pos], d1[0])
        q1 = hip.codes_to_layer_order(codes[pos:pos + 1], perm_inv[sl].contiguous())
        assert torch.equal(out[e], q1[0])
    assert not out[1].any() and not out[2].any()                 # untouched slots
    G = C // 128
    s, z = oracle.build_group_meta_packed(W.float().cpu().reshape(B * R * G, 128), 4, False)
    s, z = s.view(B, R * G).to(DEV), z.view(B, R * G).to(DEV)
    full = hip.round_to_nearest(W, s, z, 128, 4)
    part = torch.zeros_like(full)
    hip.round_to_nearest(W, s, z, 128, 4, out=part, index=idx)
    assert torch.equal(part[idx], full[idx]) and not part[1].any() and not part[2].any()


def test_expert_group_low_rank_route_against_the_dense_route_and_the_oracle():
    """Experts with 0 .. 16 rows through the low-rank route, the same experts with
    low_rank_tokens=0 through their Hessians, and the reference-form oracle: scales identical,
    codes within the tie-driven differences of two fp32 realisations; an expert that gets more
    rows in a later update leaves the route and its Hessian is rebuilt from all of them."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(8)
    C, R = 512, 128
    ns = (0, 2, 16, 5, 9, 40)
    E = len(ns)
    W = (0.02 * torch.randn(E, R, C, generator=g0)).bfloat16()
    W2 = (0.02 * torch.randn(E, R // 2, C, generator=g0)).bfloat16()
    xs = [torch.randn(n, C, generator=g0).bfloat16() for n in ns]
    xs[3][:, 17] = 0                                        # a dead input feature
    extra = torch.randn(12, C, generator=g0).bfloat16()     # expert 4: 9 + 12 rows in two calls
    offs = np.concatenate([[0], np.cumsum(ns)]).tolist()
    kw = dict(bits=4, group_size=128, symmetric=False, quantization_scale="absmax",
              quantization_order="activation", rel_damp=0.01)
    out = {}
    for lim in (16, 0):
        grp = ExpertGroupGPTQ([W.to(DEV), W2.to(DEV)], device=DEV, low_rank_tokens=lim, **kw)
        grp.update(torch.cat(xs).to(DEV), offs)
        assert grp.low_rank == ([True] * 5 + [False] if lim else [False] * E)
        grp.update(extra.to(DEV), [0, 0, 0, 0, 0, 12, 12])
        assert grp.low_rank == ([True] * 4 + [False] * 2 if lim else [False] * E)
        out[lim] = [tuple(t.cpu() for t in o) for o in grp.quantize(chunk=4)]
        assert not grp.issue_non_invertible.any()
        if lim:
            X4 = torch.cat([xs[4], extra]).double()
            H4 = (2.0 / 21) * X4.t() @ X4
            assert ((grp.hessian(4).cpu().double() - H4).norm() / H4.norm()).item() < 2e-6
    for i, Wi in enumerate((W, W2)):
        assert torch.equal(out[16][i][1], out[0][i][1]) and torch.equal(out[16][i][2], out[0][i][2])
        for e, n in enumerate(ns):
            X = torch.cat([xs[4], extra]) if e == 4 else xs[e]
            o = oracle.GPTQ(linear(Wi[e]), **kw)
            if X.shape[0]:
                o.update(X)
            qo = o.quantize()[0]
            ql, qd = out[16][i][0][e], out[0][i][0][e]
            rl = float((qo != ql).any(1).float().mean())
            rd = float((qo != qd).any(1).float().mean())
            print(f"stack {i} expert {e} ({X.shape[0]} rows): flips vs oracle low-rank "
                  f"{flip_rate(qo, ql):.2e}, dense {flip_rate(qo, qd):.2e}; rows that differ {rl:.3f}, {rd:.3f}")
            if n == 0:
                assert torch.equal(qo, ql) and torch.equal(qo, qd)   # H = I: plain rounding, exact
            elif e == 5:
                assert torch.equal(ql, qd)                   # through the Hessian either way
            else:
                # the rule of the end-to-end tests: within max(1e-3, 1.5 x floor) of the oracle,
                # the floor being what the reference's own codes move by between valid fp32
                # realisations of its library calls; on matrices this small (one diverging row is
                # 0.8 % of the codes) isolated rows that start from a one-level tie pass too
                codes_at_floor(f"low-rank stack {i} expert {e}", qo, ql, Wi[e], [X], kw, order=o.perm)


@pytest.mark.parametrize("dead", [False, True])
def test_prepare_ahead_of_other_work_changes_nothing(dead):
    """prepare() right after update(), then unrelated work on the same stream (another group's
    update, a large product), then quantize(): the same codes, scales and zeros as quantize()
    alone, with and without a dead input feature (with one the scale search waits for the
    stream after all); an update() after prepare() discards what was prepared."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(21)
    C, R = 512, 128
    ns = (0, 3, 16, 40, 200)
    W = (0.02 * torch.randn(len(ns), R, C, generator=g0)).bfloat16().to(DEV)
    xs = [torch.randn(n, C, generator=g0).bfloat16() for n in ns]
    if dead:
        for x in xs:
            x[:, 33] = 0
    X = torch.cat(xs).to(DEV)
    offs = np.concatenate([[0], np.cumsum(ns)]).tolist()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="activation", rel_damp=0.01, device=DEV)
    plain = ExpertGroupGPTQ([W], **kw)
    plain.update(X, offs)
    want = [t.cpu() for t in plain.quantize(chunk=8)[0]]

    early = ExpertGroupGPTQ([W], **kw)
    early.update(X, offs)
    early.prepare()
    other = ExpertGroupGPTQ([W.flip(0).contiguous()], **kw)       # unrelated work behind it
    other.update(X, offs)
    big = torch.randn(4096, 4096, device=DEV)
    for _ in range(8):
        big = (big @ big).clamp(-1, 1)
    got = [t.cpu() for t in early.quantize(chunk=8)[0]]
    for a, b in zip(want, got):
        assert torch.equal(a, b)

    again = ExpertGroupGPTQ([W], **kw)
    again.update(X[:offs[3]], offs[:4] + [offs[3]] * 2)           # the first three experts' rows
    again.prepare()
    again.update(X[offs[3]:], [0, 0, 0, 0, ns[3], ns[3] + ns[4]])  # the rest: prepare() is void
    assert again._prepared is None
    got = [t.cpu() for t in again.quantize(chunk=8)[0]]
    for a, b in zip(want, got):
        assert torch.equal(a, b)


def test_more_matrices_than_one_mixed_launch_holds(hip):
    """forge_gptq_sweep_lowrank_mixed splits a batch of more than 96 matrices into several
    launches, each with its own offsets into the weights, the vectors, the scales and the codes:
    100 small matrices of all five sizes in one call must equal the same matrices swept one
    by one."""
    g = torch.Generator().manual_seed(13)
    B, C, R, gs = 100, 128, 96, 128
    sizes = (4, 16, 32, 64, 128)
    ns = [sizes[int(i)] for i in torch.randint(0, 5, (B,), generator=g)]
    ns[0], ns[95], ns[96], ns[99] = 128, 4, 64, 16           # both sides of the split, all lane widths
    W0 = (0.02 * torch.randn(B, C, R, generator=g)).bfloat16().to(DEV)
    sT = (0.002 + 0.004 * torch.rand(B, 1, R, generator=g)).to(DEV)
    zT = torch.randint(5, 11, (B, 1, R), generator=g).float().to(DEV)
    g_idx = torch.zeros(B, C, dtype=torch.int32, device=DEV)
    Bps, Hms, infos = [], [], []
    for b, n in enumerate(ns):
        Bp, D = _problem(C, max(1, n - (b % 3)), 100 + b)    # some rows of the size left zero
        assert Bp.shape[1] <= n
        Bp = torch.nn.functional.pad(Bp, (0, n - Bp.shape[1]))
        Hm, info = hip.lowrank_factor(Bp[None].to(DEV), D[None].to(DEV))
        Bps.append(Bp.to(DEV))
        Hms.append(Hm[0])
        infos.append(info)
    info = torch.cat(infos)
    info[7] = 1                                              # one matrix swept uncoupled
    q = hip.gptq_sweep_lowrank_mixed(W0, torch.cat([b.flatten() for b in Bps]),
                                     torch.cat([h.flatten() for h in Hms]), ns, info, sT, zT, g_idx, 4)
    for b in range(B):
        one = hip.gptq_sweep_lowrank(W0[b:b + 1], Bps[b][None], Hms[b][None], info[b:b + 1],
                                     sT[b:b + 1], zT[b:b + 1], g_idx[b:b + 1], 4)
        assert torch.equal(q[b], one[0]), (b, ns[b])


def test_rows_kept_in_f32_are_not_rounded_when_an_expert_leaves_the_route():
    """An expert whose first rows came as f32 and whose later rows come as bf16 (and push it off
    the low-rank route): its Hessian is the f32 sum over all of them, as the route through the
    Hessian gives it, not the sum over kept rows rounded to bf16."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(17)
    C, R = 256, 64
    W = (0.02 * torch.randn(2, R, C, generator=g0)).bfloat16().to(DEV)
    first = torch.randn(10, C, generator=g0)                       # f32, not bf16-representable
    later = torch.randn(30, C, generator=g0).bfloat16()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="absmax",
              quantization_order="default", rel_damp=0.01, device=DEV)
    Hs = {}
    for lim in (16, 0):
        grp = ExpertGroupGPTQ([W], low_rank_tokens=lim, **kw)
        grp.update(first.to(DEV), [0, 10, 10])
        grp.update(later.to(DEV), [0, 30, 30])
        assert grp.low_rank == [False, lim > 0]
        Hs[lim] = grp.hessian(0).cpu().double()
        assert grp.hessian(1) is None
    X = torch.cat([first.double(), later.double()])
    want = (2.0 / 40) * X.t() @ X
    for lim, H in Hs.items():
        assert ((H - want).norm() / want.norm()).item() < 2e-6, lim
    rounded = torch.cat([first.bfloat16().double(), later.double()])
    assert (((2.0 / 40) * rounded.t() @ rounded - want).norm() / want.norm()).item() > 1e-4

