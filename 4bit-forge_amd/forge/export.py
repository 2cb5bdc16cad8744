"""What leaves the path: the per-layer record that the calibration driver stores and the
tensor set the compressed-tensors consumer reads.

``layer_record`` builds the dict of quant.py:498-511 from ``GPTQ.quantize()``'s results;
``pack_weight`` is pack_quantized.py:279-313 with the nibble packing done on the GPU
(``forge_pack_int4``).  Nothing here touches files: writing the record (``torch.save``) and
assembling checkpoint shards stay with the caller.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from forge.backend.hip import kernels


def layer_record(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                 group_size: int, bits: int, shape: Sequence[int]) -> Dict[str, object]:
    """The dict quant.py:498-511 saves per layer: codes as int8 (still one code per byte),
    fp32 scales, int32 zeros (flat, index r*G + g), group size, bit width, weight shape."""
    return {
        "qweight": qweight.to(torch.int8),
        "scales": scales.to(torch.float32),
        "qzeros": qzeros.to(torch.int32),
        "group_size": int(group_size),
        "bits": int(bits),
        "shape": tuple(int(s) for s in shape),
    }


def _first(weight: Dict[str, torch.Tensor], *names: str) -> torch.Tensor:
    for n in names:
        if n in weight:
            return weight[n]
    raise KeyError(f"none of {names} in the layer record (keys: {sorted(weight)})")


def pack_weight(weight: Dict[str, torch.Tensor], bits: int, sym: bool,
                group_size: Optional[int] = None) -> Dict[str, torch.Tensor]:
    """pack_quantized.py:279-313: ``weight_packed`` [R, ceil(C/8)] int32 (each code minus its
    group's zero, offset binary +8, eight per word along C, lowest nibble first),
    ``weight_shape`` int64 [2], ``weight_scale`` [R, G] and, when not symmetric,
    ``weight_zero_point`` [R, G].  The record may name its per-group tensors ``scale``/``zero``
    (what the reference's function reads) or ``scales``/``qzeros`` (what quant.py:498-511
    writes), flat [R*G] or [R, G].  Tensors must be on the GPU; 4-bit only (the reference
    delegates other widths to a third-party packer that has no counterpart here)."""
    if int(bits) != 4:
        raise NotImplementedError(f"bits={bits}: only the 4-bit nibble layout is packed here")
    qweight = weight["qweight"]
    scale = _first(weight, "scale", "scales")
    zero = _first(weight, "zero", "qzeros")
    if not qweight.is_cuda:
        raise RuntimeError("pack_weight runs on the GPU only; there is no CPU fallback")
    R, C = qweight.shape
    group_size = int(group_size or C)
    G = (C + group_size - 1) // group_size
    if scale.numel() != R * G or zero.numel() != R * G:
        raise ValueError(f"expected {R * G} scales and zeros for a {R} x {C} weight in groups of "
                         f"{group_size}, got {scale.numel()} and {zero.numel()}")
    codes = qweight.view(torch.uint8) if qweight.dtype == torch.int8 else qweight.to(torch.uint8)
    zero_f = zero.to(device=qweight.device, dtype=torch.float32).reshape(R * G).contiguous()
    out = {
        "weight_packed": kernels.pack_int4(codes.contiguous(), zero_f, group_size),
        "weight_shape": torch.tensor([R, C], dtype=torch.int64),
        "weight_scale": scale.reshape(R, G),
    }
    if not sym:
        out["weight_zero_point"] = zero.reshape(R, G)
    return out
