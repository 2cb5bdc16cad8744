"""Pins the oracle's scale/zero search (quant_grid.cu:42-183) with closed forms and brute force."""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref

EPS = np.float32(1e-12)


@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("gs", [32, 64, 128, 96])
def test_minmax_matches_closed_form(sym, gs):
    g = torch.Generator().manual_seed(gs + sym)
    X = 0.05 * torch.randn(513, gs, generator=g)
    X[7] = 0                       # all-zero group
    X[8] = X[8].abs() + 0.01       # all-positive group
    X[9] = -X[9].abs() - 0.01      # all-negative group
    s, z = oracle.build_group_meta_packed(X, 4, sym)
    s_ref, z_ref = mathref.minmax_grid(X.numpy(), 4, sym)
    assert np.array_equal(s.numpy(), s_ref)
    assert np.array_equal(z.numpy(), z_ref)


def test_minmax_special_cases():
    X = torch.zeros(3, 128)
    X[1] = torch.linspace(0.5, 1.5, 128)      # all positive
    X[2] = torch.linspace(-1.0, 1.0, 128)
    s, z = oracle.build_group_meta_packed(X, 4, True)
    assert s[0].item() == pytest.approx(1e-12) and z[0].item() == 8.0      # zero group: s = eps, code 8
    assert s[2].item() == np.float32(np.float64(np.float32(2) / np.float32(15)) * 1.0 + 1e-12)
    s, z = oracle.build_group_meta_packed(X, 4, False)
    assert z[0].item() == 0.0 and s[0].item() == pytest.approx(1e-12)
    # asymmetric: the reference does NOT force zero into the range; -xmin/s < 0 clamps to 0
    assert z[1].item() == 0.0
    assert s[1].item() == pytest.approx((1.5 - 0.5) / 15, rel=1e-6)
    assert z[2].item() == np.rint(np.float32(1.0) / s[2].numpy())


def test_padding_zeros_enter_minmax():
    # an all-positive tail group padded with zeros must see xmin = 0 (gptq.py:190-195)
    W = torch.full((1, 100), 0.3)
    Wp = torch.nn.functional.pad(W, (0, 28)).reshape(1, 128)
    s, z = oracle.build_group_meta_packed(Wp, 4, False)
    assert s.item() == pytest.approx(0.3 / 15, rel=1e-6) and z.item() == 0.0


@pytest.mark.parametrize("sym", [True, False])
def test_mse_against_float64_brute_force(sym):
    g = torch.Generator().manual_seed(3)
    X = 0.02 * torch.randn(64, 128, generator=g) / torch.rand(64, 128, generator=g).clamp_min(0.05)
    s0, z0 = oracle.build_group_meta_packed(X, 4, sym)
    p = torch.linspace(1.0, 0.2, 100)
    s, z, L = oracle.mse_scale_groups_packed(X, s0.clone(), z0.clone(), p, 2.4, 4, sym, return_losses=True)
    for gi in range(64):
        ref, ss, zs = mathref.mse_losses(X[gi].numpy(), s0[gi].item(), z0[gi].item(), p.numpy(), 4, sym, 2.4)
        # fp32 loss of every candidate agrees with the float64 brute force
        assert np.allclose(L[gi].numpy(), ref, rtol=2e-5)
        best = int(np.argmin(ref))
        chosen = int(np.nonzero(ss == s[gi].item())[0][0])
        # chosen candidate is a minimiser up to fp32 rounding of the loss
        assert ref[chosen] <= ref[best] * (1 + 2e-5)
        assert z[gi].item() == zs[chosen]
        # first strict minimum of the oracle's own fp32 losses
        assert chosen == int(np.argmin(L[gi].numpy()))
        assert ref[chosen] <= ref[0] * (1 + 2e-5)          # never worse than no shrink
        if sym:
            assert z[gi].item() == z0[gi].item()


def test_mse_returns_scale_without_eps_and_first_minimum_on_ties():
    # an all-zero group: every candidate has the same loss, the first (p = 1.0) must win
    X = torch.zeros(1, 128)
    s0, z0 = oracle.build_group_meta_packed(X, 4, True)
    p = torch.linspace(1.0, 0.2, 100)
    s, z = oracle.mse_scale_groups_packed(X, s0.clone(), z0.clone(), p, 2.4, 4, True)
    assert s.item() == s0.item() * 1.0 and z.item() == 8.0


def test_mse_rejects_other_group_sizes():
    X = torch.zeros(4, 48)
    with pytest.raises(RuntimeError):
        oracle.mse_scale_groups_packed(X, torch.ones(4), torch.ones(4), torch.ones(3), 2.4, 4, True)
