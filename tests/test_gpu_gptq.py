"""End-to-end: forge.gptq.GPTQ / forge.moe.ExpertGroupGPTQ on the GPU against oracle.GPTQ.

Tolerances.  Scales and zeros: equal (MSE: except candidate ties, <= 0.1 % of groups,
checked in test_gpu_grid).  Codes: with the SAME Hessian and factor every integer stage is
bit-exact at the benchmark shapes (test_gpu_stage_substitution).  End to end the Hessian sum
and the factorisation are fp32 library calls in the reference (an SGEMM and LAPACK's
potrf/potri/potrf, gptq.py:79,160-164) whose summation order it does not fix, and GPTQ's
rounding decisions amplify their last bits: a flipped code changes the error fed to every
later column of its row.  FLOOR = the largest share of codes that differ between any two
valid realisations of the reference out of three to five (helpers.reference_floor): the oracle,
the same with those two library stages computed in float64 and rounded to fp32 once
(helpers.Float64StagesGPTQ), and the oracle with its Hessian accumulated in two, three or five
calls instead of one and the trailing update's SGEMM (solver.cu:146-150) summing in another
valid order.  The GPU result must stay within max(1e-3, 1.5 * FLOOR) of the oracle, at benchmark
sizes also of the float64-stage result, and its layer output error ||WX - QX||^2 within 1 % of
the oracle's.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from forge import synth
from helpers import linear, flip_rate, expand_meta, reference_floor, codes_at_floor as _codes_at_floor

pytestmark = pytest.mark.gpu
DEV = "cuda"
from helpers import FLOORS  # noqa: E402


def _run_pair(W, X, chunks=2, **kw):
    from forge.gptq import GPTQ
    o = oracle.GPTQ(linear(W), **kw)
    g = GPTQ(linear(W).to(DEV), device=DEV, **kw)
    for part in torch.chunk(X, chunks):
        o.update(part)
        g.add_batch(part.to(DEV))
    assert int(g.num_samples) == int(o.num_samples) == X.shape[0]
    Hrel = ((g.H.cpu().double() - o.H.double()).norm() / o.H.double().norm()).item()
    assert Hrel < 2e-6
    H = o.H.double().numpy().copy()
    return o, g, H


@pytest.mark.parametrize("kw", [
    dict(symmetric=True, quantization_scale="absmax", quantization_order="default"),
    dict(symmetric=True, quantization_scale="mse", quantization_order="default"),
    dict(symmetric=False, quantization_scale="mse", quantization_order="activation"),
    dict(symmetric=False, quantization_scale="absmax", quantization_order="activation", group_size=64),
], ids=["sym-absmax", "sym-mse", "asym-mse-actorder", "asym-absmax-actorder-g64"])
def test_dense_layer_end_to_end(kw):
    case = synth.dense_outlier(R=256, C=1024, n=1024, seed=1)
    kw = dict(bits=4, rel_damp=0.01, **kw)
    kw.setdefault("group_size", 128)
    o, g, H = _run_pair(case.W, case.X, **kw)
    qo, so, zo = o.quantize()
    qg, sg, zg = g.quantize()
    assert qg.dtype == torch.uint8 and tuple(qg.shape) == (256, 1024) and qg.is_contiguous()
    assert sg.shape == so.shape and zg.shape == zo.shape and g.G == o.G
    same = so == sg.cpu()
    assert float((~same).float().mean()) <= 1e-3
    assert torch.equal(zo[same], zg.cpu()[same])
    _codes_at_floor("dense 256x1024", qo, qg, case.W, torch.chunk(case.X, 2), kw)
    gs = kw["group_size"]
    Wf = case.W.numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, gs).numpy(), H)
    eg = mathref.layer_error(Wf, oracle.dequantize(qg.cpu(), sg.cpu(), zg.cpu(), gs).numpy(), H)
    assert abs(eg / eo - 1) < 0.01


def test_dense_layer_direct_route():
    """The class with factor_route="direct" (factor of H itself, displacement sweep): same
    tolerances against the reference-form oracle as the default route."""
    from forge.gptq import GPTQ
    case = synth.dense_outlier(R=256, C=1024, n=1024, seed=1)
    kw = dict(bits=4, rel_damp=0.01, group_size=128, symmetric=False, quantization_scale="mse",
              quantization_order="activation")
    o = oracle.GPTQ(linear(case.W), **kw)
    g = GPTQ(linear(case.W).to(DEV), device=DEV, factor_route="direct", **kw)
    o.update(case.X)
    g.update(case.X.to(DEV))
    H = o.H.double().numpy().copy()
    qo, so, zo = o.quantize()
    qg, sg, zg = (t.cpu() for t in g.quantize())
    same = so == sg
    assert float((~same).float().mean()) <= 1e-3 and torch.equal(zo[same], zg[same])
    _codes_at_floor("dense 256x1024 direct", qo, qg, case.W, [case.X], kw)
    Wf = case.W.numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, 128).numpy(), H)
    eg = mathref.layer_error(Wf, oracle.dequantize(qg, sg, zg, 128).numpy(), H)
    assert abs(eg / eo - 1) < 0.01


def test_fallbacks_zero_tokens_nan_dead_column_and_non_pd():
    from forge.gptq import GPTQ
    g0 = torch.Generator().manual_seed(2)
    W = 0.02 * torch.randn(64, 256, generator=g0)
    kw = dict(bits=4, symmetric=True, quantization_scale="absmax", quantization_order="activation")

    def rtn_of(q, s, z):
        se = expand_meta(s.cpu(), 64, 256, 128).t()
        ze = expand_meta(z.cpu(), 64, 256, 128).t()
        return np.array_equal(q.cpu().numpy(), mathref.rtn(W.numpy(), se.numpy(), ze.numpy(), 4))

    h = GPTQ(linear(W).to(DEV), device=DEV, **kw)                        # no tokens: H = I
    h.update(torch.empty(0, 256, device=DEV))
    assert rtn_of(*h.quantize())
    h = GPTQ(linear(W).to(DEV), device=DEV, **kw)                        # NaN activations: H = I
    X = torch.randn(16, 256, generator=g0); X[3, 7] = float("nan")
    h.update(X.to(DEV))
    assert rtn_of(*h.quantize())
    # dead input feature: pruned, weight column zeroed, same as the oracle
    X = torch.randn(512, 256, generator=g0) * torch.linspace(0.5, 2.0, 256)
    X[:, 9] = 0
    o = oracle.GPTQ(linear(W), **kw); o.update(X)
    h = GPTQ(linear(W).to(DEV), device=DEV, **kw); h.update(X.to(DEV))
    qo, so, zo = o.quantize(); qg, sg, zg = h.quantize()
    assert bool(h.pruned_ids[9]) and int(h.pruned_ids.sum()) == 1
    assert torch.equal(so, sg.cpu())
    _codes_at_floor("dead column", qo, qg, W, [X], kw, order=o.perm)
    assert torch.equal(qo[:, 9], qg.cpu()[:, 9])
    # not positive definite (rank 4, no damping): identity fallback + flag, like gptq.py:172-175
    h = GPTQ(linear(W).to(DEV), device=DEV, rel_damp=0.0, **kw)
    h.update((torch.randn(4, 256, generator=g0) + 0.5).to(DEV))
    assert rtn_of(*h.quantize()) and h.issue_non_invertible


def test_owner_sharing_reset_and_in_place_damping():
    from forge.gptq import GPTQ
    g0 = torch.Generator().manual_seed(3)
    Wg, Wu = 0.02 * torch.randn(48, 256, generator=g0), 0.02 * torch.randn(48, 256, generator=g0)
    X = torch.randn(400, 256, generator=g0) * torch.linspace(0.3, 2.0, 256)
    kw = dict(bits=4, symmetric=False, quantization_scale="absmax", quantization_order="activation")
    og = oracle.GPTQ(linear(Wg), **kw); ou = oracle.GPTQ(linear(Wu), owner=og, **kw)
    hg = GPTQ(linear(Wg).to(DEV), device=DEV, **kw); hu = GPTQ(linear(Wu).to(DEV), device=DEV, owner=hg, **kw)
    for h in (og, ou):
        h.update(X)
    for h in (hg, hu):
        h.update(X.to(DEV))
    assert hu.H is None and not hu._is_owner() and hg._is_owner()
    # owner first, then the non-owner (quant.py:414,514): the non-owner re-damps the
    # owner's already damped Hessian -- reproduced, see the oracle's host test
    qo_g, _, _ = og.quantize(); qo_u, so_u, _ = ou.quantize()
    qg_g, _, _ = hg.quantize(); qg_u, sg_u, _ = hu.quantize()
    assert torch.equal(hu.perm.cpu(), ou.perm) and int(hu.num_samples) == 400
    assert torch.equal(so_u, sg_u.cpu())
    _, floor, _ = _codes_at_floor("owner gate", qo_g, qg_g, Wg, [X], kw)
    assert flip_rate(qo_u, qg_u) <= max(1e-3, FLOORS * floor) + 1e-3   # 48 x 256 codes: 1e-3 = 12 codes
    ratio = (hu.H.diagonal().cpu() - ou.H.diagonal()).abs().max() / ou.H.diagonal().abs().max()
    assert ratio < 1e-5                      # both damped twice
    hg.reset()
    assert hg.H is None and int(hg.num_samples) == 0 and not hg.prepared and hg.perm is None


def test_sparse14_end_to_end():
    from forge.gptq import GPTQ
    case = synth.sparse14_down_proj(R=192, C=512, n=1024, seed=4)
    kw = dict(bits=4, symmetric=True, quantization_scale="mse", quantization_order="default",
              algorithm="sparsegptq")
    o, g, H = _run_pair(case.W, case.X, **kw)
    qo, so, zo, Mo = o.quantize()
    qg, sg, zg, Mg = g.quantize()
    assert tuple(Mg.shape) == (16, 192) and Mg.dtype == torch.uint32
    assert float((so != sg.cpu()).float().mean()) <= 1e-3
    _, floor, out64 = _codes_at_floor("sparse14 192x512", qo, qg, case.W, torch.chunk(case.X, 2), kw)
    bits = lambda M: ((M.view(torch.int32).cpu().numpy().astype(np.uint32)[np.arange(512) // 32]
                       >> (np.arange(512) % 32)[:, None]) & 1)
    keep = bits(Mg)
    assert np.all(keep.reshape(128, 4, 192).sum(axis=1) == 1)           # exactly 1 of 4 kept
    mask_floor = float((bits(Mo) != bits(out64[3])).mean())
    assert float((bits(Mo) != keep).mean()) <= max(1e-3, FLOORS * mask_floor)
    dq = lambda q, s, z, M: (oracle.dequantize(q, s, z, 128) * torch.from_numpy(bits(M).T.copy()).float()).numpy()
    eo = mathref.layer_error(case.W.float().numpy(), dq(qo, so, zo, Mo), H)
    eg = mathref.layer_error(case.W.float().numpy(), dq(qg.cpu(), sg.cpu(), zg.cpu(), Mg), H)
    assert abs(eg / eo - 1) < 0.01


@pytest.mark.parametrize("factor_route", ["direct", "inverse"])
def test_expert_group_matches_per_expert_handles(factor_route):
    """Qwen3-shaped miniature: ragged routed tokens, a zero-token expert, gate/up sharing
    one Hessian and one factorisation, down on its own.  Both routes to the sweep's matrix
    (the factor of H itself with displacements, the reference's factor of inv(H) with
    errors) against the reference-form oracle."""
    from forge.moe import ExpertGroupGPTQ
    moe = synth.qwen3_moe(experts=6, n_experts=48, hidden=512, inter=256, tokens=1024, seed=5)
    E = 6
    moe.rows[4] = moe.rows[4][:0]                                        # expert without tokens
    xs, hs = zip(*(moe.expert_inputs(e) for e in range(E)))
    offs = np.concatenate([[0], np.cumsum([x.shape[0] for x in xs])])
    kw = dict(bits=4, group_size=128, symmetric=False, quantization_scale="mse",
              quantization_order="activation")
    gu = ExpertGroupGPTQ([moe.Wg[:E].to(DEV), moe.Wu[:E].to(DEV)], device=DEV,
                         factor_route=factor_route, **kw)
    dn = ExpertGroupGPTQ([moe.Wd[:E].to(DEV)], device=DEV, factor_route=factor_route, **kw)
    half = [x.shape[0] // 2 for x in xs]                                 # two ragged calibration passes
    for sel in (lambda x, h: x[:h], lambda x, h: x[h:]):
        px = [sel(x, h) for x, h in zip(xs, half)]
        ph = [sel(y, h) for y, h in zip(hs, half)]
        o2 = np.concatenate([[0], np.cumsum([p.shape[0] for p in px])])
        gu.update(torch.cat(px).to(DEV), o2)
        dn.update(torch.cat(ph).to(DEV), o2)
    (qg, sg, zg), (qu, su, zu) = gu.quantize(chunk=4)
    (qd, sd, zd), = dn.quantize(chunk=4)
    for e in range(E):
        for W, X, (q, s, z) in ((moe.Wg[e], xs[e], (qg, sg, zg)), (moe.Wu[e], xs[e], (qu, su, zu)),
                                (moe.Wd[e], hs[e], (qd, sd, zd))):
            o = oracle.GPTQ(linear(W), **kw)
            o.update(X)
            qo, so, zo = o.quantize()
            assert float((so != s[e].cpu()).float().mean()) <= 2e-3
            same = so == s[e].cpu()
            assert torch.equal(zo[same], z[e].cpu()[same])
            if X.shape[0] == 0:
                assert torch.equal(qo, q[e].cpu())                       # H = I: pure RTN, exact
            else:
                _codes_at_floor(f"expert {e} {tuple(W.shape)} {factor_route}", qo, q[e], W, [X], kw,
                                order=o.perm)


@pytest.mark.parametrize("factor_route", ["direct", "inverse"])
def test_expert_group_non_positive_definite_falls_back(factor_route):
    """No damping and fewer tokens than features: the factorisation of that expert fails, it is
    quantised by plain round-to-nearest and flagged (gptq.py:172-175); its neighbour, with
    enough tokens, is solved as usual."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(8)
    E, R, C = 2, 64, 256
    W = 0.02 * torch.randn(E, R, C, generator=g0)
    xs = [torch.randn(4, C, generator=g0) + 0.5, torch.randn(600, C, generator=g0)]
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="absmax",
              quantization_order="default", rel_damp=0.0)
    grp = ExpertGroupGPTQ([W.to(DEV)], device=DEV, factor_route=factor_route, **kw)
    grp.update(torch.cat(xs).to(DEV), [0, 4, 604])
    (q, s, z), = grp.quantize(chunk=2)
    assert grp.issue_non_invertible.tolist() == [True, False]
    se = expand_meta(s[0].cpu(), R, C, 128).t()
    ze = expand_meta(z[0].cpu(), R, C, 128).t()
    assert np.array_equal(q[0].cpu().numpy(), mathref.rtn(W[0].numpy(), se.numpy(), ze.numpy(), 4))
    o = oracle.GPTQ(linear(W[1]), **kw)
    o.update(xs[1])
    qo, so, zo = o.quantize()
    assert torch.equal(so, s[1].cpu())
    _codes_at_floor(f"undamped neighbour {factor_route}", qo, q[1], W[1], [xs[1]], kw, order=o.perm)


@pytest.mark.parametrize("zero_weight_column", [False, True])
def test_expert_group_dead_and_zero_columns(zero_weight_column):
    """A feature that one expert never sees (dead column: zero Hessian diagonal) and, in the
    second case, an all-zero weight column in gate_proj only, which gives gate and up
    different pruning masks: they no longer share a factor."""
    from forge.moe import ExpertGroupGPTQ
    moe = synth.qwen3_moe(experts=3, n_experts=24, hidden=256, inter=128, tokens=768, seed=11)
    E = 3
    xs = [moe.expert_inputs(e)[0].clone() for e in range(E)]
    xs[1][:, 37] = 0
    xs[1][:, 200] = 0
    Wg, Wu = moe.Wg[:E].clone(), moe.Wu[:E].clone()
    if zero_weight_column:
        Wg[2, :, 5] = 0
    offs = np.concatenate([[0], np.cumsum([x.shape[0] for x in xs])])
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="activation")
    gu = ExpertGroupGPTQ([Wg.to(DEV), Wu.to(DEV)], device=DEV, **kw)
    gu.update(torch.cat(xs).to(DEV), offs)
    (qg, sg, zg), (qu, su, zu) = gu.quantize(chunk=4)
    for e in range(E):
        for W, (q, s, z) in ((Wg[e], (qg, sg, zg)), (Wu[e], (qu, su, zu))):
            o = oracle.GPTQ(linear(W), **kw)
            o.update(xs[e])
            qo, so, zo = o.quantize()
            assert float((so != s[e].cpu()).float().mean()) <= 2e-3
            _codes_at_floor(f"dead/zero columns, expert {e}", qo, q[e], W, [xs[e]], kw,
                            order=o.perm)
            if e == 1:      # dead columns are pruned: weight 0 -> the code of zero
                assert torch.equal(qo[:, [37, 200]], q[e].cpu()[:, [37, 200]])


@pytest.mark.parametrize("factor_route,R,C", [("direct", 64, 256), ("inverse", 64, 256),
                                              ("direct", 128, 384)])
def test_expert_group_sparse14_matches_per_expert_oracle(factor_route, R, C, hip):
    """algorithm="sparsegptq" through the batched front end: codes, keep-masks (solver order)
    and scales against oracle.GPTQ expert by expert; one kept weight in every group of four.
    Both routes to the sweep's matrix; the last case with the left-looking schedule a large
    batch takes (whole 128 x 128 tiles: long products from 16-bit pieces, their V operand from
    the factor's rows, X never laid out)."""
    from forge.moe import ExpertGroupGPTQ
    g = torch.Generator().manual_seed(31)
    E = 3
    left = R % 128 == 0
    Wg = (0.02 * torch.randn(E, R, C, generator=g)).bfloat16()
    Wu = (0.02 * torch.randn(E, R, C, generator=g)).bfloat16()
    xs = [torch.randn(n, C, generator=g).bfloat16() for n in (500, 320, 640)]
    offs = np.concatenate([[0], np.cumsum([x.shape[0] for x in xs])])
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="default", algorithm="sparsegptq")
    grp = ExpertGroupGPTQ([Wg.to(DEV), Wu.to(DEV)], device=DEV, factor_route=factor_route, **kw)
    grp.update(torch.cat(xs).to(DEV), offs)
    if left:
        hip.set_option("sweep_schedule", 1)
    try:
        assert hip.sweep_direct_reads_band_only(E, C, 2 * R) == left
        (qg, sg, zg, Mg), (qu, su, zu, Mu) = grp.quantize(chunk=4)
    finally:
        hip.set_option("sweep_schedule", 0)
    for e in range(E):
        for W, (q, s, z, M) in ((Wg[e], (qg, sg, zg, Mg)), (Wu[e], (qu, su, zu, Mu))):
            o = oracle.GPTQ(linear(W), **kw)
            o.update(xs[e])
            qo, so, zo, Mo = o.quantize()
            assert float((so != s[e].cpu()).float().mean()) <= 2e-3
            bits_o = np.unpackbits(Mo.numpy().view(np.uint8), bitorder="little")
            bits_g = np.unpackbits(M[e].cpu().numpy().view(np.uint8), bitorder="little")
            assert bits_g.reshape(-1, 4).sum(1).tolist() == [1] * (bits_g.size // 4)
            _, floor, out64 = _codes_at_floor(f"sparse14 expert {e} {factor_route}", qo, q[e], W, [xs[e]], kw)
            bits_64 = np.unpackbits(out64[3].numpy().view(np.uint8), bitorder="little")
            assert (bits_o != bits_g).mean() <= max(1e-3, FLOORS * (bits_o != bits_64).mean())


# ---------------------------------------------------------------- benchmark configurations
def _e2e(tag, W, X, kw, gs=128):
    o, g, H = _run_pair(W, X, chunks=1, **kw)
    ro, rg = o.quantize(), g.quantize()
    qo, so, zo = ro[:3]
    qg, sg, zg = (t.cpu() for t in rg[:3])
    assert float((so != sg).float().mean()) <= 1e-3
    same = so == sg
    assert torch.equal(zo[same], zg[same])
    flips = flip_rate(qo, qg)
    Wf = W.float().numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, gs).numpy(), H)
    eg = mathref.layer_error(Wf, oracle.dequantize(qg, sg, zg, gs).numpy(), H)
    assert abs(eg / eo - 1) < 0.01, eg / eo
    _codes_at_floor(tag, qo, qg, W, [X], kw, both=True)
    return flips, eg / eo, ro, rg


@pytest.mark.parametrize("scale", ["absmax", "mse"])
def test_config1_dense_2048_full_size(scale):
    """Config 1 as specified: 2048x2048 f32 weight, 1024 f32 tokens with 1 % outlier channels,
    4-bit symmetric g128, damp 0.01, no act-order."""
    case = synth.dense_outlier()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale=scale,
              quantization_order="default", rel_damp=0.01)
    flips, ratio, _, _ = _e2e(f"config1 {scale}", case.W, case.X, kw)
    print(f"config1 {scale}: flips {flips:.2e} error ratio {ratio:.5f}")


def test_config4_student_t_full_size_against_a_row_subset():
    """Config 4 as specified (4096 x 7168 bf16 weight with Student-t(3) rows, 2048 tokens,
    4-bit asymmetric g128, MSE search with 100 shrink factors and p = 2.4) solved in full on the
    GPU.  Rows are independent given the Hessian, so the CPU oracle solves the first 256 rows
    of the same weight with the same tokens and those rows are compared."""
    from forge.gptq import GPTQ
    case = synth.student_t_weight()
    rows = 256
    kw = dict(bits=4, group_size=128, symmetric=False, quantization_scale="mse",
              quantization_order="default", rel_damp=0.01)
    g = GPTQ(linear(case.W).to(DEV), device=DEV, **kw)
    g.add_batch(case.X.to(DEV))
    qg, sg, zg = (t.cpu() for t in g.quantize())
    assert tuple(qg.shape) == (4096, 7168) and g.G == 56
    Wsub = case.W[:rows].contiguous()
    o = oracle.GPTQ(linear(Wsub), **kw)
    o.update(case.X)
    H = o.H.double().numpy().copy()
    qo, so, zo = o.quantize()
    sg, zg, qg = sg[:rows * 56], zg[:rows * 56], qg[:rows]
    same = so == sg
    assert float((~same).float().mean()) <= 1e-3 and torch.equal(zo[same], zg[same])
    _codes_at_floor("config4 rows 0-255", qo, qg, Wsub, [case.X], kw, both=True)
    Wf = Wsub.float().numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, 128).numpy(), H)
    eg = mathref.layer_error(Wf, oracle.dequantize(qg, sg, zg, 128).numpy(), H)
    assert abs(eg / eo - 1) < 0.01, eg / eo


def test_config5_sparse14_full_size():
    """Config 5 as specified: 3072x1536 bf16 down_proj, 2048 bf16 tokens, 1:4 mask + 4-bit
    symmetric g128 on the survivors."""
    case = synth.sparse14_down_proj()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="default", algorithm="sparsegptq")
    o, g, H = _run_pair(case.W, case.X, chunks=1, **kw)
    qo, so, zo, Mo = o.quantize()
    qg, sg, zg, Mg = g.quantize()
    assert float((so != sg.cpu()).float().mean()) <= 1e-3
    C, R = 1536, 3072
    unpack = lambda M: ((M.view(torch.int32).cpu().numpy().astype(np.uint32)[np.arange(C) // 32]
                         >> (np.arange(C) % 32)[:, None]) & 1).astype(bool)
    ko, kg = unpack(Mo), unpack(Mg)
    assert np.all(kg.reshape(C // 4, 4, R).sum(axis=1) == 1)
    _, floor, out64 = _codes_at_floor("config5", qo, qg, case.W, [case.X], kw, both=True)
    assert float((ko != kg).mean()) <= max(1e-3, FLOORS * float((ko != unpack(out64[3])).mean()))
    dq = lambda q, s, z, k: (oracle.dequantize(q, s, z, 128) * torch.from_numpy(k.T.copy()).float()).numpy()
    Wf = case.W.float().numpy()
    eo = mathref.layer_error(Wf, dq(qo, so, zo, ko), H)
    eg = mathref.layer_error(Wf, dq(qg.cpu(), sg.cpu(), zg.cpu(), kg), H)
    assert abs(eg / eo - 1) < 0.01
    # the packed inference words built from the GPU result decode back to the same codes
    from forge.backend.hip import kernels
    s32 = sg.view(R, C // 128).repeat_interleave(4, dim=1).t().contiguous()      # [G32, R]
    words = kernels.pack_sparsegptq14_to_u64x2(qg, Mg, s32).view(torch.int64).cpu()
    want = oracle.pack_sparsegptq14_to_u64x2(qg.cpu(), Mg.cpu().view(torch.int32), s32.cpu())
    assert torch.equal(words, want)


@pytest.mark.parametrize("n_tokens", [1536, 200, 128, 100, 40])
def test_config3_all_routes_against_the_oracle_at_full_shape(n_tokens):
    """DeepSeek-V3-shaped gate_proj (C = 7168, fp8 block round trip, act-order, MSE; 512 of
    its 2048 rows, rows being independent, to keep the CPU oracle's sweeps short) with a heavy
    expert's tokens, with 200 (Hessian of rank 200 before damping; the batched front end's default
    route then takes the blocked closed form) and with 128 and 40 (that route then solves from the
    rows themselves, column by column: at 65-128 rows, i.e. 100 and 128 here, with four threads per
    row of the factor's recurrence and eight lanes per row of the sweep, at 40 with one).  At
    this size the
    problem is ill conditioned: the oracle's own codes move by 1-2 % between two valid fp32
    realisations of its library stages (the floor).  Three GPU routes are held to that floor
    against the reference-form oracle: the drop-in class (reference's factor of inv(H), fp32
    chain sweep), the batched front end on the same route, and the batched front end's default
    -- the route the benchmark times: factor of H itself, displacement sweep, block updates
    from bf16 pieces."""
    from forge.gptq import GPTQ
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(11)
    W = synth.fp8_block_roundtrip((0.02 * torch.randn(512, 7168, generator=g0)).bfloat16())
    X = torch.randn(1536, 7168, generator=g0).bfloat16()[:n_tokens].contiguous()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="activation", rel_damp=0.01)
    o = oracle.GPTQ(linear(W), **kw)
    o.update(X)
    H = o.H.double().numpy().copy()
    qo, so, zo = o.quantize()
    floor, out64 = reference_floor(W, [X], qo, **kw)
    bound = max(1e-3, FLOORS * floor)
    Wf = W.float().numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, 128).numpy(), H)
    # with fewer rows than the group size the error only sees the few directions the rows span
    # and is driven almost to zero: it then moves by a per cent between equally valid solutions,
    # the oracle's own float64-stage realisation included
    e64 = mathref.layer_error(Wf, oracle.dequantize(*out64[:3], 128).numpy(), H)
    allowed = 0.01 if n_tokens >= 128 else max(0.01, 2 * abs(e64 / eo - 1))

    def check(tag, q, s, z):
        q, s, z = q.cpu(), s.cpu(), z.cpu()
        assert float((so != s).float().mean()) <= 1e-3
        flips, to64 = flip_rate(qo, q), flip_rate(out64[0], q)
        eg = mathref.layer_error(Wf, oracle.dequantize(q, s, z, 128).numpy(), H)
        print(f"config3 n={n_tokens} {tag}: flips vs oracle {flips:.2e}, vs float64 stages {to64:.2e}, "
              f"floor {floor:.2e}, error ratio {eg / eo:.5f} (the float64-stage oracle's: {e64 / eo:.5f})")
        assert abs(eg / eo - 1) <= allowed, (tag, eg / eo, e64 / eo)
        assert flips <= bound and to64 <= bound

    g = GPTQ(linear(W).to(DEV), device=DEV, **kw)
    g.add_batch(X.to(DEV))
    check("class", *g.quantize())
    del g
    from forge.backend.hip import kernels
    # a single matrix would take the right-looking schedule (fp32 chain updates); the layer's
    # 64-expert chunks take the left-looking one with block updates from bf16 pieces: force
    # it, so that this is the arithmetic the benchmark times
    kernels.set_option("sweep_schedule", 1)
    try:
        # (100 and 128 rows: the default takes the blocked closed form from 65 rows on; with
        # low_rank_tokens=128 the column-by-column form with eight lanes per row of the sweep)
        variants = [("inverse", {}), ("direct", {})] + ([("direct", dict(low_rank_tokens=128))] if n_tokens in (100, 128) else [])
        for route, extra in variants:
            grp = ExpertGroupGPTQ([W.to(DEV).view(1, 512, 7168)], device=DEV, factor_route=route, **extra, **kw)
            grp.update(X.to(DEV), [0, n_tokens])
            (q, s, z), = grp.quantize(chunk=1)
            assert not grp.issue_non_invertible.any()
            if route == "direct":
                assert grp.low_rank == [n_tokens <= (extra.get("low_rank_tokens", 64))]
                assert grp.rows_route == [extra.get("low_rank_tokens", 64) < n_tokens <= 512]
            check(f"batched {route} {extra}", q[0], s[0], z[0])
            del grp
    finally:
        kernels.set_option("sweep_schedule", 0)


def test_expert_group_few_tokens_routes_agree():
    """Experts that saw 1 .. 700 tokens of 2048 features (rank-deficient Hessians, damping
    only): both routes of the batched front end against the oracle.  With a handful of tokens
    ||WX - QX||^2 only sees the few directions the tokens span and is driven almost to zero,
    so it moves by 1-2 % between equally valid solutions -- the oracle's own float64-stage
    realisation does (measured 0.7 %, 1.3 %, 1.7 % at 1, 3, 16 tokens).  Each route must
    therefore stay within max(1 %, twice that movement) of the oracle's error, within the
    floor-based bound of its codes, and far below round-to-nearest's error.  Where diagonal
    entries of the Hessian are exactly equal (one bf16 token) the activation order itself is
    not defined by the reference; there the error may differ by 5 % and codes are not compared."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(3)
    C, R = 2048, 256
    ns = (1, 3, 16, 100, 700)
    E = len(ns)
    W = (0.02 * torch.randn(E, R, C, generator=g0)).bfloat16()
    xs = [torch.randn(n, C, generator=g0).bfloat16() for n in ns]
    offs = np.concatenate([[0], np.cumsum(ns)]).tolist()
    kw = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
              quantization_order="activation", rel_damp=0.01)
    out = {}
    for route in ("direct", "inverse"):
        grp = ExpertGroupGPTQ([W.to(DEV)], device=DEV, factor_route=route, **kw)
        grp.update(torch.cat(xs).to(DEV), offs)
        (q, s, z), = grp.quantize(chunk=8)
        assert not grp.issue_non_invertible.any()
        out[route] = (q.cpu(), s.cpu(), z.cpu())
    assert torch.equal(out["direct"][1], out["inverse"][1])
    for e, n in enumerate(ns):
        X = xs[e].double()
        H = ((2.0 / n) * X.t() @ X).numpy()
        Wf = W[e].double().numpy()

        def err(q, s, z):
            D = Wf - oracle.dequantize(q, s, z, 128).double().numpy()
            return float(((D @ H) * D).sum())

        o = oracle.GPTQ(linear(W[e]), **kw)
        o.update(xs[e])
        qo, so, zo = o.quantize()
        floor, o64 = reference_floor(W[e], [xs[e]], qo, **kw)
        eo = err(qo, so, zo)
        spread = abs(err(*o64[:3]) / eo - 1)
        diag = (2.0 / n) * (xs[e].float() ** 2).sum(0)
        ties = C - torch.unique(diag).numel() > C // 100          # more than 1 % of the columns
        se = expand_meta(out["direct"][1][e], R, C, 128).t().double().numpy()
        ze = expand_meta(out["direct"][2][e], R, C, 128).t().double().numpy()
        Dr = Wf - (np.clip(np.rint(Wf / (se + 1e-12) + ze), 0, 15) - ze) * se
        rtn = float(((Dr @ H) * Dr).sum())
        for r in out:
            q, s, z = (t[e] for t in out[r])
            ratio = err(q, s, z) / eo
            flips = flip_rate(qo, q)
            print(f"n={n} {r}: error / oracle's {ratio:.4f} (float64-stage oracle moves by {spread:.4f}), "
                  f"flips {flips:.2e} (floor {floor:.2e})")
            assert abs(ratio - 1) <= (0.05 if ties else max(0.01, 2 * spread)), (n, r, ratio, spread)
            # exactly equal diagonal entries (certain with one bf16 token: many |x_j| coincide)
            # leave their activation order to argsort's tie-breaking, which the reference does
            # not fix (non-stable sort, gptq.py:110) and which differs between torch's CPU and
            # GPU sorts: the codes are then compared through the error only
            if not ties:
                assert flips <= max(1e-3, FLOORS * floor), (n, r, flips, floor)
            assert err(q, s, z) < 0.5 * rtn


@pytest.fixture(scope="module")
def config2_step(hip):
    """Eight Qwen3-30B-A3B-shaped experts (768x2048 / 2048x768 bf16, asymmetric, MSE) with the
    layer's ragged routing, batched.  With the left-looking schedule that the layer's 128
    experts take (eight alone would be swept right-looking): long products from fp16 halves,
    their V operand from the factor's rows, X never laid out."""
    from forge.moe import ExpertGroupGPTQ
    moe = synth.qwen3_moe(experts=8, seed=6)
    E = 8
    xs, hs = zip(*(moe.expert_inputs(e) for e in range(E)))
    offs = np.concatenate([[0], np.cumsum([x.shape[0] for x in xs])])
    gu = ExpertGroupGPTQ([moe.Wg.to(DEV), moe.Wu.to(DEV)], device=DEV, **CONFIG2_KW)
    dn = ExpertGroupGPTQ([moe.Wd.to(DEV)], device=DEV, **CONFIG2_KW)
    gu.update(torch.cat(xs).to(DEV), offs)
    dn.update(torch.cat(hs).to(DEV), offs)
    hip.set_option("sweep_schedule", 1)
    try:
        assert hip.sweep_direct_reads_band_only(8, 2048, 1536) and hip.sweep_direct_reads_band_only(8, 768, 2048)
        outs = [tuple(t.cpu() for t in o) for o in gu.quantize(chunk=8)]
        outs += [tuple(t.cpu() for t in o) for o in dn.quantize(chunk=8)]
    finally:
        hip.set_option("sweep_schedule", 0)
    del gu, dn
    torch.cuda.empty_cache()
    return moe, xs, hs, outs, {}


CONFIG2_KW = dict(bits=4, group_size=128, symmetric=False, quantization_scale="mse",
                  quantization_order="default")


def _config2_expert(step, e, floors):
    """One expert's three matrices against per-expert oracle handles: (error of the oracle's
    codes, error of the GPU's) as ||WX - QX||^2 summed over the tokens the expert saw."""
    moe, xs, hs, (og, ou, od), errors = step
    if e in errors and not floors:
        return errors[e]
    sum_o = sum_g = 0.0
    for W, X, (q, s, z) in ((moe.Wg[e], xs[e], og), (moe.Wu[e], xs[e], ou), (moe.Wd[e], hs[e], od)):
        o = oracle.GPTQ(linear(W), **CONFIG2_KW)
        o.update(X)
        n = X.shape[0]
        H = o.H.double().numpy().copy() if o.H is not None else np.eye(W.shape[1])
        qo, so, zo = o.quantize()
        assert float((so != s[e]).float().mean()) <= 2e-3
        if n and floors:
            _codes_at_floor(f"config2 expert {e} {tuple(W.shape)} n={n}", qo, q[e], W, [X], CONFIG2_KW)
        Wf = W.float().numpy()
        eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, 128).numpy(), H) * n / 2
        eg = mathref.layer_error(Wf, oracle.dequantize(q[e], s[e], z[e], 128).numpy(), H) * n / 2
        # Per expert the ratio is only meaningful with enough tokens (an expert that saw 3 tokens
        # has a rank-3 Hessian and its error moves by several % between equally good solutions).
        if floors and n >= 128:
            assert abs(eg / eo - 1) < 0.01, (e, tuple(W.shape), eg / eo)
        sum_o += eo
        sum_g += eg
    errors[e] = (sum_o, sum_g)
    return errors[e]


@pytest.mark.parametrize("e", range(8))
def test_config2_qwen3_expert_at_full_shape(config2_step, e):
    """Scales equal up to candidate near-ties, codes under the floor rule, the expert's output
    error within 1 % of the oracle's where it saw at least 128 tokens."""
    _config2_expert(config2_step, e, floors=True)


def test_config2_qwen3_layer_error(config2_step):
    """The layer's output error over all eight experts: within 1 % of the oracle's."""
    sums = [_config2_expert(config2_step, e, floors=False) for e in range(8)]
    so, sg = sum(a for a, _ in sums), sum(b for _, b in sums)
    print(f"config2 layer error ratio {sg / so:.5f}")
    assert abs(sg / so - 1) < 0.01


def test_quantize_refuses_a_chunk_whose_workspace_does_not_fit(monkeypatch):
    """quantize() adds up what its largest chunk allocates and raises before it queues anything
    when the device cannot hold it (a kernel that meets a full device mid-queue takes the queue
    down with it); a smaller chunk then goes through."""
    from forge.moe import ExpertGroupGPTQ
    g0 = torch.Generator().manual_seed(2)
    W = (0.02 * torch.randn(4, 128, 256, generator=g0)).bfloat16().to(DEV)
    X = torch.randn(600, 256, generator=g0).bfloat16().to(DEV)
    grp = ExpertGroupGPTQ([W], device=DEV, bits=4, group_size=128, symmetric=True,
                          quantization_scale="absmax", quantization_order="activation")
    grp.update(X, [0, 200, 400, 403, 600])
    need = grp.workspace_bytes(3, 1, 0, 0, 128)
    assert need > 3 * (2 * 256 * 256 * 4 + 256 * 128 * 7)
    real = ExpertGroupGPTQ.workspace_bytes
    monkeypatch.setattr(ExpertGroupGPTQ, "workspace_bytes",
                        lambda self, nd, *a: (1 << 50) if nd > 2 else real(self, nd, *a))
    with pytest.raises(RuntimeError, match="smaller `chunk`"):
        grp.quantize(chunk=4)
    (q, s, z), = grp.quantize(chunk=2)
    assert tuple(q.shape) == (4, 128, 256) and not grp.issue_non_invertible.any()
