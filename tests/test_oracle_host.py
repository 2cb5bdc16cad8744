"""Pins the oracle's host logic (forge/gptq.py:10-276 restated in oracle.GPTQ)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from helpers import linear, random_problem, flip_rate


def _handle(R=32, C=128, **kw):
    g = torch.Generator().manual_seed(1)
    W = 0.02 * torch.randn(R, C, generator=g)
    kw.setdefault("quantization_scale", "absmax")
    return oracle.GPTQ(linear(W), **kw), W


def test_hessian_closed_form_and_chunking_invariance():
    h, _ = _handle()
    g = torch.Generator().manual_seed(2)
    X = torch.randn(300, 128, generator=g)
    for part in (X[:7], X[7:7], X[7:150].reshape(11, 13, 128), X[150:]):   # incl. empty + 3-d batch
        h.update(part)
    ref = mathref.hessian([X.numpy()])
    assert int(h.num_samples) == 300
    assert np.allclose(h.H.numpy(), ref, rtol=1e-5, atol=1e-6)
    assert torch.equal(h.H, h.H.t()) or np.allclose(h.H.numpy(), h.H.numpy().T, rtol=1e-6)
    one, _ = _handle()
    one.update(X)
    assert np.allclose(one.H.numpy(), h.H.numpy(), rtol=1e-5, atol=1e-6)
    # first call: the beta = 0 update overwrites the preliminary product (gptq.py:75-79)
    assert np.allclose(one.H.numpy(), (2.0 / 300) * (X.T @ X).numpy(), rtol=1e-5, atol=1e-6)


def test_prep_activation_order_and_dead_columns():
    h, W = _handle(quantization_order="activation")
    g = torch.Generator().manual_seed(3)
    X = torch.randn(64, 128, generator=g) * torch.linspace(0.1, 3.0, 128)
    X[:, 5] = 0                                                    # dead feature
    h.update(X)
    Hfull = h.H.clone()
    h._prep()
    assert bool(h.pruned_ids[5]) and int(h.pruned_ids.sum()) == 1
    assert torch.all(h.W[:, 5] == 0)
    d = torch.diag(Hfull).clone(); d[5] = 1.0
    assert torch.all(d[h.perm][:-1] >= d[h.perm][1:])             # descending diagonal
    assert torch.equal(h.perm_inv[h.perm], torch.arange(128))
    p5 = int(h.perm_inv[5])
    assert h.H[p5, p5] == 1 and h.H[p5].abs().sum() == 1 and h.H[:, p5].abs().sum() == 1
    keep = [i for i in range(128) if i != p5]
    assert torch.equal(h.H[keep][:, keep], Hfull[h.perm][:, h.perm][keep][:, keep])


@pytest.mark.parametrize("case", ["no_tokens", "nan"])
def test_identity_fallback_gives_rtn(case):
    h, W = _handle(symmetric=True, quantization_order="default")
    if case == "nan":
        X = torch.randn(8, 128); X[0, 0] = float("nan")
        h.update(X)
    q, s, z = h.quantize()
    se = s.view(32, 1).repeat_interleave(128, 1); ze = z.view(32, 1).repeat_interleave(128, 1)
    assert np.array_equal(q.numpy(), mathref.rtn(W.numpy(), se.numpy(), ze.numpy(), 4))


def test_factor_matches_scipy_float64():
    pr = random_problem(C=256, R=8)
    h = oracle.GPTQ(linear(pr["W"]), quantization_order="default", quantization_scale="absmax")
    h.update(pr["X"]); h._prep()
    H64 = h.H.double().numpy().copy()
    U = h._h_factor()
    ref = mathref.factor(H64, 0.01)
    assert np.allclose(U.numpy(), ref, rtol=0, atol=2e-5 * np.abs(ref).max())
    assert torch.all(torch.tril(U, -1) == 0) and torch.all(U.diag() == 1)
    # U0^T U0 (H + damp I) = I for the un-normalised factor
    U0 = mathref.factor(H64, 0.01, normalise=False)
    Hd = H64 + 0.01 * np.mean(np.diag(H64)) * np.eye(256)
    assert np.allclose(U0.T @ U0 @ Hd, np.eye(256), atol=1e-8)


def test_non_positive_definite_falls_back_to_identity():
    h, W = _handle(rel_damp=0.0, quantization_order="default", symmetric=True)
    X = torch.randn(4, 128)                    # rank 4 < 128 and no damping: not PD
    X[:, 0] = 1.0                              # keep every diagonal entry non-zero
    h.update(X + 0.01)
    q, s, z = h.quantize()
    assert h.issue_non_invertible
    se = s.view(32, 1).repeat_interleave(128, 1); ze = z.view(32, 1).repeat_interleave(128, 1)
    assert np.array_equal(q.numpy(), mathref.rtn(W.numpy(), se.numpy(), ze.numpy(), 4))


def test_owner_sharing_and_unpermute():
    g = torch.Generator().manual_seed(5)
    Wg, Wu = 0.02 * torch.randn(24, 128, generator=g), 0.02 * torch.randn(24, 128, generator=g)
    X = torch.randn(200, 128, generator=g) * torch.linspace(0.2, 2.0, 128)

    def pair():
        gate = oracle.GPTQ(linear(Wg), quantization_scale="absmax")
        up = oracle.GPTQ(linear(Wu), quantization_scale="absmax", owner=gate)
        gate.update(X); up.update(torch.full((3, 128), 1e6))      # non-owner ignores its tokens
        return gate, up

    solo = oracle.GPTQ(linear(Wu), quantization_scale="absmax")
    solo.update(X)
    qs, ss, zs = solo.quantize()
    # non-owner first: it prepares the owner's Hessian and solves on a copy of it
    gate, up = pair()
    qu, su, zu = up.quantize()
    assert torch.equal(up.perm, gate.perm) and int(up.num_samples) == 200 and gate.prepared
    assert torch.equal(qu, qs) and torch.equal(su, ss) and torch.equal(zu, zs)
    # owner first (the order quant.py:414,514 uses): _h_factor damps the owner's H IN PLACE
    # (gptq.py:143,154), so the non-owner copies an already damped Hessian and damps it again
    gate, up = pair()
    gate.quantize()
    qu2, _, _ = up.quantize()
    twice = oracle.GPTQ(linear(Wu), quantization_scale="absmax")
    twice.update(X); twice._prep()
    twice.H.diagonal().add_(0.01 * twice.H.diag().mean())
    q2, _, _ = twice.quantize()
    assert torch.equal(qu2, q2) and not torch.equal(qu2, qs)
    # scales are indexed r*G + (original column // gs): dequantising in that layout is close
    deq = oracle.dequantize(qu, su, zu, 128)
    assert (deq - Wu).abs().max() < 3 * su.max()


def test_quantize_returns_reference_layouts_sparse():
    pr = random_problem(C=256, R=16)
    h = oracle.GPTQ(linear(pr["W"]), algorithm="sparsegptq", symmetric=True,
                    quantization_order="default", quantization_scale="absmax")
    h.update(pr["X"])
    q, s, z, M = h.quantize()
    assert q.shape == (16, 256) and q.dtype == torch.uint8
    assert s.shape == (32,) and z.shape == (32,) and tuple(M.shape) == (8, 16)
    kept = (q != 0).sum().item()
    assert kept <= 16 * 256 // 4
