"""Seeded synthetic workloads shaped like the layers 4Bit-Forge quantises.

Five generators, one per benchmark configuration: a dense linear with outlier channels,
a Qwen3-style and a DeepSeek-V3-style MoE layer with Zipf-routed tokens, a heavy-tailed
weight for the scale search, and a MiniMax-style down projection for the 1:4 solve.
Everything is drawn from a ``torch.Generator`` so that a CPU run and a GPU run of the
same seed see the same numbers when generated on the CPU and moved.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch


def _gen(seed: int, device="cpu") -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


@dataclass
class DenseCase:
    W: torch.Tensor            # [R, C]
    X: torch.Tensor            # [n, C]
    opts: dict = field(default_factory=dict)


def dense_outlier(R=2048, C=2048, n=1024, seed=0, device="cpu") -> DenseCase:
    """Config 1: W = 0.02 randn f32; X = randn f32 with 1 % channels scaled x20."""
    g = _gen(seed, device)
    W = 0.02 * torch.randn(R, C, generator=g, device=device)
    X = torch.randn(n, C, generator=g, device=device)
    k = max(1, round(0.01 * C))
    idx = torch.randperm(C, generator=g, device=device)[:k]
    X[:, idx] *= 20.0
    return DenseCase(W, X, dict(bits=4, group_size=128, symmetric=True, rel_damp=0.01,
                                quantization_order="default"))


def student_t_weight(R=4096, C=7168, n=2048, nu=3.0, seed=0, device="cpu") -> DenseCase:
    """Config 4: rows 0.02 * Student-t(nu) as randn / sqrt(chi2(nu)/nu), bf16."""
    g = _gen(seed, device)
    z = torch.randn(R, C, generator=g, device=device)
    chi = torch.zeros(R, C, device=device)
    for _ in range(int(nu)):
        chi += torch.randn(R, C, generator=g, device=device) ** 2
    W = (0.02 * z / torch.sqrt(chi / nu)).to(torch.bfloat16)
    X = torch.randn(n, C, generator=g, device=device)
    return DenseCase(W, X, dict(bits=4, group_size=128, symmetric=False,
                                quantization_scale="mse", quantization_order="default"))


def sparse14_down_proj(R=3072, C=1536, n=2048, seed=0, device="cpu") -> DenseCase:
    """Config 5: MiniMax-M2-style expert down_proj, bf16."""
    g = _gen(seed, device)
    W = (0.02 * torch.randn(R, C, generator=g, device=device)).to(torch.bfloat16)
    X = torch.randn(n, C, generator=g, device=device).to(torch.bfloat16)
    return DenseCase(W, X, dict(bits=4, group_size=128, symmetric=True, algorithm="sparsegptq",
                                quantization_order="default"))


def fp8_block_roundtrip(W: torch.Tensor, tile: int = 128) -> torch.Tensor:
    """Encode to float8_e4m3fn with one fp32 scale per tile x tile block (scale_inv =
    amax/448) and decode fp8 -> f32 * scale_inv -> bf16, the way DeepSeek checkpoints
    are materialised (forge/utils/io.py:533-563)."""
    R, C = W.shape
    nR, nC = (R + tile - 1) // tile, (C + tile - 1) // tile
    Wp = torch.zeros(nR * tile, nC * tile, dtype=torch.float32, device=W.device)
    Wp[:R, :C] = W.float()
    blk = Wp.view(nR, tile, nC, tile)
    s_inv = blk.abs().amax(dim=(1, 3)).clamp_min(1e-12) / 448.0
    q = (blk / s_inv[:, None, :, None]).to(torch.float8_e4m3fn)
    out = q.float() * s_inv[:, None, :, None]
    return out.reshape(nR * tile, nC * tile)[:R, :C].to(torch.bfloat16).contiguous()


@dataclass
class MoECase:
    hidden: int
    inter: int
    n_experts: int
    X: torch.Tensor                     # [T, hidden] bf16
    Wg: torch.Tensor                    # [E, inter, hidden] bf16
    Wu: torch.Tensor                    # [E, inter, hidden] bf16
    Wd: torch.Tensor                    # [E, hidden, inter] bf16
    rows: List[torch.Tensor]            # per expert: token indices routed to it
    opts: dict = field(default_factory=dict)

    def expert_inputs(self, e: int):
        """(x for gate/up, x for down) of expert e, as one calibration forward with the
        unquantised weights would hand them to the hooks (quant.py:371-375,406)."""
        x = self.X[self.rows[e]]
        h = torch.nn.functional.silu(x @ self.Wg[e].T) * (x @ self.Wu[e].T)
        return x, h.to(torch.bfloat16)


def route_topk(T: int, E: int, k: int, g: torch.Generator, zipf_a: float = 1.1,
               device="cpu") -> List[torch.Tensor]:
    """Top-k of softmax(randn logits + log popularity); popularity ~ rank^-a over a seeded
    permutation of the experts.  Returns the routed token indices per expert (ragged)."""
    order = torch.randperm(E, generator=g, device=device)
    pop = torch.empty(E, device=device)
    pop[order] = torch.arange(1, E + 1, device=device, dtype=torch.float32) ** (-zipf_a)
    logits = torch.randn(T, E, generator=g, device=device) + torch.log(pop / pop.sum())
    top = torch.topk(torch.softmax(logits, dim=-1), k, dim=-1).indices       # [T, k]
    flat_e = top.reshape(-1)
    flat_t = torch.arange(T, device=device).repeat_interleave(k)
    srt = torch.argsort(flat_e, stable=True)
    counts = torch.bincount(flat_e, minlength=E).tolist()
    return list(torch.split(flat_t[srt], counts))


def moe_layer(hidden, inter, n_experts, tokens, topk=8, seed=0, fp8=False, device="cpu",
              experts: Optional[int] = None, opts: Optional[dict] = None) -> MoECase:
    """Configs 2 and 3.  ``experts`` limits how many experts' weights are materialised
    (routing is still over all ``n_experts``) so that reduced cases stay small."""
    g = _gen(seed, device)
    X = torch.randn(tokens, hidden, generator=g, device=device).to(torch.bfloat16)
    rows = route_topk(tokens, n_experts, topk, g, device=device)
    E = n_experts if experts is None else experts

    def w(*shape):
        t = (0.02 * torch.randn(*shape, generator=g, device=device)).to(torch.bfloat16)
        if fp8:
            t = torch.stack([fp8_block_roundtrip(t[i]) for i in range(t.shape[0])])
        return t

    return MoECase(hidden, inter, n_experts, X, w(E, inter, hidden), w(E, inter, hidden),
                   w(E, hidden, inter), rows, opts or {})


def qwen3_moe(seed=0, device="cpu", experts=None, n_experts=128, hidden=2048, inter=768,
              tokens=4096) -> MoECase:
    return moe_layer(hidden, inter, n_experts, tokens, seed=seed, device=device, experts=experts,
                     opts=dict(bits=4, group_size=128, symmetric=False,
                               quantization_order="default"))


def deepseek_v3_moe(seed=0, device="cpu", experts=None, n_experts=256, hidden=7168, inter=2048,
                    tokens=8192) -> MoECase:
    return moe_layer(hidden, inter, n_experts, tokens, seed=seed, fp8=True, device=device,
                     experts=experts,
                     opts=dict(bits=4, group_size=128, symmetric=True,
                               quantization_order="activation"))
