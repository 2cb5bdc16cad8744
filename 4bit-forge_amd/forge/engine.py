"""Callers either side of the solve (forge/utils/engine.py, forge/utils/quant.py of the
reference): the dequantised weight that is written back into the layer before the block is
run again, and the routed-row gather in front of the per-expert Hessian update."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from forge.backend.hip import kernels


@torch.no_grad()
def dequantize_forge_full(dtype, qweight, scales, qzeros, group_size, device):
    """Same call as forge/utils/engine.py:71-97: (q - q0) * s with flat [R*G] per-group
    meta, computed in f32 and rounded to `dtype`; qweight [R, C] unpacked codes."""
    if qweight.dim() != 2:
        raise ValueError(f"Expected qweight (R,C) unpacked, got shape={tuple(qweight.shape)}")
    R, C = qweight.shape
    G = (C + group_size - 1) // group_size
    scales = scales.reshape(-1)
    qzeros = qzeros.reshape(-1)
    if scales.numel() != R * G or qzeros.numel() != R * G:
        raise ValueError(f"Expected scales/qzeros numel == R*G ({R * G}), "
                         f"got scales={scales.numel()}, qzeros={qzeros.numel()}")
    dev = torch.device(device)
    return kernels.dequantize_groups(qweight.to(dev).to(torch.uint8), scales.to(dev),
                                     qzeros.to(dev), group_size, dtype)


@torch.no_grad()
def routed_rows(x: torch.Tensor, router_indices: torch.Tensor,
                routing_weights: Optional[torch.Tensor], num_experts: int
                ) -> Tuple[torch.Tensor, list]:
    """What the fused-expert hook of forge/utils/engine.py:210-238 feeds to the per-expert
    handles, for all experts at once: the rows of `x` [tokens, H] routed to each expert,
    scaled by their routing weight, grouped by expert in ascending token order.
    router_indices / routing_weights: [tokens, top_k].  Returns (rows [N, H], offsets
    [num_experts + 1]) as ExpertGroupGPTQ.update takes them.  Entries with an expert id
    outside [0, num_experts) are dropped, as the hook skips them."""
    ri = router_indices.reshape(router_indices.shape[0], -1).to(x.device)
    tok = torch.arange(ri.shape[0], device=x.device).unsqueeze(1).expand_as(ri).reshape(-1)
    exp = ri.reshape(-1).to(torch.int64)
    ok = (exp >= 0) & (exp < num_experts)
    # stable sort by expert keeps (token, k) order inside an expert, as nonzero() yields it
    order = torch.argsort(torch.where(ok, exp, torch.full_like(exp, num_experts)), stable=True)
    n_ok = int(ok.sum())
    order = order[:n_ok]
    counts = torch.bincount(exp[order], minlength=num_experts).cpu().tolist()
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + int(c))
    w = None
    if routing_weights is not None:
        w = routing_weights.reshape(ri.shape[0], -1).to(x.device).reshape(-1)[order].to(x.dtype)
    x2 = x if x.stride(-1) == 1 else x.contiguous()
    rows = kernels.gather_scaled_rows(x2, tok[order].contiguous(), w)
    return rows, offsets
