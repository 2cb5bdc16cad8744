"""A benchmark step in small, at the DeepSeek-V3 layer's own matrix shapes, against the oracle.

One ``ExpertGroupGPTQ.quantize()`` call per projection carries experts of every kind that a
step of the benchmark layer holds: experts without a single routed row (plain rounding),
with 3 .. 64 rows (solved from the rows, the sizes of the per-row-vector sweep in ONE mixed
launch), with 100, 128 and 200 rows (the blocked closed form, sizes 128 and 256 in one batch)
and with 1536 (through the Hessian).  gate_proj
and up_proj are two stacks of their full shape that share one factor (R = 2048 each, C = 7168);
down_proj has its full shape too, R = 7168, C = 2048.  The oracle checks a
regular subset of each expert's rows (every eighth of gate/up's, every seventh of down's: the
grid is per row and group, the sweep per row, gptq.py:128-139 / solver.cu:9-154), which
touches every row tile of the kernels and keeps an expert's CPU side to a few seconds.  Every expert is then
compared with ``oracle.GPTQ`` (forge/gptq.py:128-139 on the handles that quant.py:386-396
creates) under the rules of test_gpu_gptq: scales equal up to candidate near-ties, codes
within max(1e-3, 1.5 x floor) of the oracle AND of the float64-stage realisation, layer
output error within 1 % (experts with a handful of rows: within twice what the oracle's own
float64-stage realisation moves by, as in test_expert_group_few_tokens_routes_agree).

The GPU side runs once per module; each parametrised case is one expert's CPU comparison
(an oracle solve and the realisations of the floor, each with its factorisations of a
7168 x 7168 Hessian: about ten seconds).
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import mathref
from forge import synth
from helpers import linear, flip_rate, reference_floor, FLOORS

pytestmark = pytest.mark.gpu
DEV = "cuda"
KW = dict(bits=4, group_size=128, symmetric=True, quantization_scale="mse",
          quantization_order="activation", rel_damp=0.01)
#        rows each expert saw: none, the per-row-vector sizes 4/16/32/64, then beyond
NS = (0, 3, 16, 40, 100, 128, 200, 1536, 0, 64, 128, 5)
GATE_UP_CASES = tuple(range(len(NS)))
DOWN_CASES = tuple(range(len(NS)))


def _rows(seed, C):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(n, C, generator=g).bfloat16() for n in NS]


@pytest.fixture(scope="module")
def gate_up():
    from forge.moe import ExpertGroupGPTQ
    g = torch.Generator().manual_seed(31)
    E, R, C = len(NS), 2048, 7168
    W = [torch.stack([synth.fp8_block_roundtrip((0.02 * torch.randn(R, C, generator=g)).bfloat16())
                      for _ in range(E)]) for _ in range(2)]
    xs = _rows(32, C)
    offs = np.concatenate([[0], np.cumsum(NS)]).tolist()
    grp = ExpertGroupGPTQ([w.to(DEV) for w in W], device=DEV, **KW)
    grp.update(torch.cat(xs).to(DEV), offs)
    outs = [tuple(t.cpu() for t in o) for o in grp.quantize(chunk=E)]
    assert not grp.issue_non_invertible.any()
    routes = (list(grp.low_rank), list(grp.rows_route))
    del grp
    torch.cuda.empty_cache()
    return W, xs, outs, routes


@pytest.fixture(scope="module")
def down():
    from forge.moe import ExpertGroupGPTQ
    g = torch.Generator().manual_seed(33)
    E, R, C = len(NS), 7168, 2048
    W = torch.stack([synth.fp8_block_roundtrip((0.02 * torch.randn(R, C, generator=g)).bfloat16())
                     for _ in range(E)])
    xs = _rows(34, C)
    offs = np.concatenate([[0], np.cumsum(NS)]).tolist()
    grp = ExpertGroupGPTQ([W.to(DEV)], device=DEV, **KW)
    grp.update(torch.cat(xs).to(DEV), offs)
    outs = [tuple(t.cpu() for t in o) for o in grp.quantize(chunk=E)]
    assert not grp.issue_non_invertible.any()
    routes = (list(grp.low_rank), list(grp.rows_route))
    del grp
    torch.cuda.empty_cache()
    return W, xs, outs, routes


def _against_the_oracle(tag, W, X, q, s, z):
    n = X.shape[0]
    o = oracle.GPTQ(linear(W), **KW)
    if n:
        o.update(X)
    H = o.H.double().numpy().copy() if n else None
    qo, so, zo = o.quantize()
    assert float((so != s).float().mean()) <= 2e-3, tag
    if n == 0:
        # H = I: nothing couples the columns, the sweep is the quantiser weight by weight
        same = (so.view(W.shape[0], -1) == s.view(W.shape[0], -1)).all(1)
        assert torch.equal(qo[same], q[same]), tag
        return
    floor, o64 = reference_floor(W, [X], qo, **KW)
    bound = max(1e-3, FLOORS * floor)
    flips, to64 = flip_rate(qo, q), flip_rate(o64[0], q)
    Wf = W.float().numpy()
    eo = mathref.layer_error(Wf, oracle.dequantize(qo, so, zo, 128).numpy(), H)
    e64 = mathref.layer_error(Wf, oracle.dequantize(*o64[:3], 128).numpy(), H)
    eg = mathref.layer_error(Wf, oracle.dequantize(q, s, z, 128).numpy(), H)
    spread = abs(e64 / eo - 1)
    print(f"{tag}: flips vs oracle {flips:.2e}, vs float64 stages {to64:.2e}, floor {floor:.2e}, "
          f"error ratio {eg / eo:.5f} (the float64-stage oracle's: {e64 / eo:.5f})")
    assert flips <= bound and to64 <= bound, (tag, flips, to64, floor)
    # with fewer rows than features the error only sees the few directions the rows span and is
    # driven almost to zero: it then moves by a per cent or two between equally valid solutions
    assert abs(eg / eo - 1) <= (0.01 if n >= 128 else max(0.01, 2 * spread)), (tag, eg / eo, spread)


def test_routes_taken(gate_up, down):
    """What the step is meant to mix in one call: experts without rows and with up to 64 rows
    solved from the rows themselves column by column, those with 100, 128 and 200 rows by the
    blocked closed form (256 x 7 does not exceed 2048 nor 7168), the one with 1536 rows through
    its Hessian."""
    for _, _, _, (low, blocked) in (gate_up, down):
        assert low == [n <= 64 for n in NS]
        assert blocked == [64 < n <= 256 for n in NS]


@pytest.mark.parametrize("e", GATE_UP_CASES)
def test_gate_up_expert_against_the_oracle(gate_up, e):
    """gate_proj and up_proj of one expert share their Hessian and factor (the reference's
    owner mechanism, forge/gptq.py:36,84-94): one oracle solve on the two matrices' rows
    stacked, with the owner's single damping, as the batched front end defines the unit of work."""
    W, xs, outs, _ = gate_up
    R, G = W[0].shape[1], W[0].shape[2] // 128
    rows = torch.arange(0, R, 8)
    pick = lambda t: t[e].view(R, G)[rows].reshape(-1)
    Wst = torch.cat([W[0][e][rows], W[1][e][rows]])
    q = torch.cat([outs[0][0][e][rows], outs[1][0][e][rows]])
    s = torch.cat([pick(outs[0][1]), pick(outs[1][1])])
    z = torch.cat([pick(outs[0][2]), pick(outs[1][2])])
    _against_the_oracle(f"gate/up expert {e} ({NS[e]} rows)", Wst, xs[e], q, s, z)


@pytest.mark.parametrize("e", DOWN_CASES)
def test_down_expert_against_the_oracle(down, e):
    W, xs, outs, _ = down
    rows = torch.arange(0, W.shape[1], 7)
    G = W.shape[2] // 128
    pick = lambda t: t[e].view(W.shape[1], G)[rows].reshape(-1)
    _against_the_oracle(f"down expert {e} ({NS[e]} rows)", W[e][rows], xs[e], outs[0][0][e][rows],
                        pick(outs[0][1]), pick(outs[0][2]))
