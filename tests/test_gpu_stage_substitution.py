"""Stage substitution at the benchmark shapes: every stage of the GPU path that does integer
work is fed the ORACLE's own tensors (its Hessian, activation order, grid and factor) and must
then reproduce the oracle's codes bit for bit.  What is left to differ end to end is the fp32
rounding inside the Hessian sum and the factorisation (tests/test_gpu_gptq.py bounds that
against the reference's own sensitivity to it).

Shapes: config 1 (2048 x 2048, 1024 f32 tokens, no act-order), config 3's gate_proj (C = 7168,
fp8 block round trip, act-order; 512 of the 2048 rows, rows being independent, so that the
CPU oracle's sweeps stay short) and config 5 (3072 x 1536, 1:4 joint solve).
"""
import numpy as np
import pytest
import torch

import oracle
from forge import synth
from helpers import linear, reference_floor

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(name):
    if name == "config1":
        c = synth.dense_outlier()
        return c.W, c.X, dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
                              quantization_order="default", rel_damp=0.01)
    if name == "config3":
        g0 = torch.Generator().manual_seed(11)
        W = synth.fp8_block_roundtrip((0.02 * torch.randn(512, 7168, generator=g0)).bfloat16())
        X = torch.randn(1536, 7168, generator=g0).bfloat16()
        return W, X, dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
                          quantization_order="activation", rel_damp=0.01)
    c = synth.sparse14_down_proj()
    return c.W, c.X, dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
                          quantization_order="default", algorithm="sparsegptq", rel_damp=0.01)


def _oracle_stages(W, X, kw):
    """The oracle's flow stopped after each stage (oracle.GPTQ.quantize, gptq.py:128-139)."""
    o = oracle.GPTQ(linear(W), **kw)
    o.update(X)
    o._prep()
    scales, qzeros = o._quant_grid()
    U = o._h_factor().contiguous()          # o.H is now the permuted, damped Hessian
    Wt = o.W.clone().float().t()[o.perm].contiguous()
    return o, scales, qzeros, U, Wt


def _batched_meta(o, scales, qzeros, R):
    G = o.G
    sT = scales.view(R, G).t().contiguous().view(1, G, R).to(DEV)
    zT = qzeros.view(R, G).t().contiguous().view(1, G, R).to(DEV)
    g_idx = (o.perm // o.group_size).to(torch.int32).view(1, -1).to(DEV)
    return sT, zT, g_idx


@pytest.mark.parametrize("name", ["config1", "config3"])
def test_reference_form_sweep_on_the_oracles_factor(hip, name):
    """Oracle's H, order, grid and LAPACK factor -> the GPU's reference-form sweep (both the
    reference-signature operator and the batched g_idx form the class uses): 0 flips."""
    W, X, kw = _case(name)
    R, C = W.shape
    o, scales, qzeros, U, Wt = _oracle_stages(W, X, kw)
    se, ze = o._expand(scales, C, R).contiguous(), o._expand(qzeros, C, R).contiguous()
    q_ref = oracle.gptq_solver(Wt.clone(), U, se, ze, 4)
    q_op = hip.gptq_solver(Wt.clone().to(DEV), U.to(DEV), se.to(DEV), ze.to(DEV), 4)
    assert torch.equal(q_ref, q_op.cpu())
    del q_op, se, ze
    sT, zT, g_idx = _batched_meta(o, scales, qzeros, R)
    perm_inv = o.perm_inv.view(1, C).to(DEV)
    Xs = hip.weight_to_solver_order(W.to(DEV).view(1, R, C), perm_inv)
    assert torch.equal(Xs[0].cpu(), Wt)
    q_b = hip.gptq_sweep_batched(Xs, U.to(DEV).view(1, C, C), sT, zT, g_idx, 4)
    assert torch.equal(q_ref, q_b[0].cpu())
    # back to the layer's order: the oracle's returned codes
    q_layer = hip.codes_to_layer_order(q_b, perm_inv)[0].cpu()
    assert torch.equal(q_layer, q_ref[o.perm_inv].t().contiguous())


def test_reference_form_sparse14_on_the_oracles_factor(hip):
    """Config 5 at full size: codes, keep-masks and the in-place normalisation of U."""
    W, X, kw = _case("config5")
    R, C = W.shape
    o, scales, qzeros, U, Wt = _oracle_stages(W, X, kw)
    se, ze = o._expand(scales, C, R).contiguous(), o._expand(qzeros, C, R).contiguous()
    Uo = U.clone()
    q_ref, M_ref = oracle.sparsegptq14_solver(Wt.clone(), Uo, se, ze, 4)
    Ud = U.clone().to(DEV)
    q_op, M_op = hip.sparsegptq14_solver(Wt.clone().to(DEV), Ud, se.to(DEV), ze.to(DEV), 4)
    assert torch.equal(q_ref, q_op.cpu())
    assert torch.equal(M_ref.view(torch.int32), M_op.cpu().view(torch.int32))
    assert torch.equal(Uo, Ud.cpu())
    # batched form: row-normalised U and 1/diag of the un-normalised one
    sT, zT, g_idx = _batched_meta(o, scales, qzeros, R)
    uinv = (1.0 / U.diag()).view(1, C).contiguous().to(DEV)
    q_b, M_b = hip.gptq_sweep_batched(Wt.clone().to(DEV).view(1, C, R), Ud.view(1, C, C), sT, zT,
                                      g_idx, 4, sparse14=True, uinv=uinv)
    assert torch.equal(q_ref, q_b[0].cpu())
    assert torch.equal(M_ref.view(torch.int32), M_b[0].cpu().view(torch.int32))


@pytest.mark.parametrize("name", ["config1", "config3", "config5"])
def test_direct_route_sweep_on_the_oracles_hessian(hip, name):
    """The route the benchmark times.  The oracle's permuted, damped Hessian is factored on
    the GPU (factor of H itself), the matrix V is copied back, and the displacement-form
    sweep runs on both sides with that V: the fp32-chain form equals its CPU checker bit for
    bit.  The block updates the library ships for batches of experts (left-looking schedule,
    sums on the 16-bit matrix pipe) are a different fp32-grade summation, not a chain: their
    codes are compared with the chain's for two fp16 halves per operand (2) and
    for 6, 3 and 1 bf16 piece products per fp32 product.  All but the last must stay within
    max(0.1 %, a quarter of the floor) -- the floor being what the reference's own codes move
    by between two fp32 realisations of its library stages; plain bf16 operands (1 product)
    are reported: they move 2-16 %."""
    W, X, kw = _case(name)
    R, C = W.shape
    sparse = kw.get("algorithm") == "sparsegptq"
    o, scales, qzeros, U, Wt = _oracle_stages(W, X, kw)
    se, ze = o._expand(scales, C, R).contiguous(), o._expand(qzeros, C, R).contiguous()
    L, info = hip.chol_reverse_lower_batched(o.H.to(DEV).view(1, C, C).clone(), None)
    assert int(info.item()) == 0
    V = hip.unit_upper_from_lower(L, info, negate=True, upper_only=True)
    Vc = torch.triu(V[0].cpu()).contiguous()          # tiles below the diagonal are unwritten
    sT, zT, g_idx = _batched_meta(o, scales, qzeros, R)
    Xd = Wt.to(DEV).view(1, C, R)
    mdiag = L[0].diagonal().contiguous().view(1, C) if sparse else None

    def gpu(**k):
        r = hip.gptq_sweep_direct_batched(Xd.clone(), V, sT, zT, g_idx, 4, sparse14=sparse,
                                          mdiag=mdiag, **k)
        return r if sparse else (r, None)

    if sparse:
        q_ref, M_ref = oracle.sparsegptq14_solver_direct(Wt.clone(), Vc, mdiag[0].cpu(), se, ze, 4)
        q_orc, _ = oracle.sparsegptq14_solver(Wt.clone(), U.clone(), se, ze, 4)
    else:
        q_ref, M_ref = oracle.gptq_solver_direct(Wt.clone(), Vc, se, ze, 4), None
        q_orc = oracle.gptq_solver(Wt.clone(), U, se, ze, 4)
    q_x, M_x = gpu(exact_chain=True)
    assert torch.equal(q_ref, q_x[0].cpu())
    if sparse:
        assert torch.equal(M_ref.view(torch.int32), M_x[0].cpu().view(torch.int32))
    # floor: the oracle's own codes against its float64-stage realisation (solver order)
    floor, out64 = reference_floor(W, [X], q_orc[o.perm_inv].t().contiguous(), **kw)
    bound = max(1e-3, 0.25 * floor)
    hip.set_option("sweep_schedule", 1)               # what a batch of experts takes
    try:
        for products in (2, 6, 3, 1):
            old = hip.set_option("sweep_update_products", products)
            try:
                q_s, M_s = gpu()
            finally:
                hip.set_option("sweep_update_products", old)
            flips = (q_x != q_s).float().mean().item()
            what = "fp16 halves" if products == 2 else f"{products} bf16 piece product(s)"
            print(f"{name}: block updates from {what} vs fp32 chain: flips "
                  f"{flips:.2e} (floor {floor:.2e})")
            if products != 1:
                assert flips <= bound, (products, flips, floor)
                if sparse:
                    assert (M_x.view(torch.int32) != M_s.view(torch.int32)).float().mean().item() <= bound
            else:
                assert flips > bound                  # why plain bf16 operands are not shipped
    finally:
        hip.set_option("sweep_schedule", 0)
