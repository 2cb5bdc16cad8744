"""Batched GPTQ over the experts of one MoE layer (no counterpart in the reference, which
walks its ``GPTQ`` handles one linear layer at a time, quant.py:414-417).

``ExpertGroupGPTQ`` holds E equally shaped experts.  Several weight stacks may share one
Hessian stack (gate_proj and up_proj see the same tokens: the reference's ``owner``
mechanism, forge/gptq.py:36,84-94), so they also share one factorisation.  ``update``
takes the routed tokens of ALL experts at once (rows grouped by expert + offsets) and
issues one ragged MFMA launch; ``quantize`` runs the scale search, the factorisation
and the sweep for a chunk of experts per launch so that every kernel fills the GPU.
Arithmetic per expert is the one of ``forge.gptq.GPTQ``.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from forge.backend.hip import kernels


class ExpertGroupGPTQ:
    def __init__(self, weights: Sequence[torch.Tensor], bits: int = 4, group_size: int = 128,
                 symmetric: bool = False, quantization_scale: str = "mse",
                 quantization_order: str = "activation", rel_damp: float = 1e-2,
                 device=None):
        """weights: stacks [E, R_i, C] (bf16 or f32) that share the input features C."""
        self.device = torch.device(device) if device is not None else weights[0].device
        if self.device.type != "cuda":
            raise RuntimeError("ExpertGroupGPTQ runs on the GPU only; there is no CPU fallback")
        self.W: List[torch.Tensor] = []
        for w in weights:
            if w.dim() != 3 or w.shape[0] != weights[0].shape[0] or w.shape[2] != weights[0].shape[2]:
                raise ValueError("weights must be [E, R, C] stacks sharing E and C")
            w = w.to(self.device)
            if w.dtype not in (torch.bfloat16, torch.float32):
                w = w.float()
            self.W.append(w.contiguous())
        self.E, _, self.C = self.W[0].shape
        self.bits, self.group_size, self.symmetric = bits, group_size, symmetric
        self.quantization_scale = quantization_scale
        self.quantization_order = quantization_order
        self.rel_damp = rel_damp
        self.H: Optional[torch.Tensor] = None           # [E, C, C] f32
        self.num_samples = [0] * self.E                 # host-side counts
        self.issue_non_invertible = torch.zeros(self.E, dtype=torch.bool)

    # ------------------------------------------------------------------ Hessians
    @torch.no_grad()
    def update(self, X: torch.Tensor, offsets: Sequence[int]):
        """X [T, C]: calibration rows grouped by expert; expert e owns rows
        offsets[e]:offsets[e+1].  Running mean per expert as in forge/gptq.py:61-80."""
        if len(offsets) != self.E + 1:
            raise ValueError("offsets must have E+1 entries")
        X = X.to(self.device)
        if X.dtype not in (torch.bfloat16, torch.float32):
            X = X.float()
        if X.stride(-1) != 1:
            X = X.contiguous()
        if self.H is None:
            self.H = torch.empty((self.E, self.C, self.C), dtype=torch.float32, device=self.device)
        alpha, beta = [], []
        for e in range(self.E):
            new = int(offsets[e + 1]) - int(offsets[e])
            n = self.num_samples[e]
            total = max(n + new, 1)
            alpha.append(2.0 / total)
            beta.append(n / total)
            self.num_samples[e] = n + new
        kernels.hessian_update_grouped(X, [int(o) for o in offsets], self.H, alpha, beta)

    add_batch = update

    # ------------------------------------------------------------------ solve
    @torch.no_grad()
    def quantize(self, chunk: int = 32, max_shrink: float = 0.2, n_grid: int = 100,
                 norm: float = 2.4):
        """Returns one (qweight [E,R,C] u8, scales [E,R*G] f32, qzeros [E,R*G] f32) per stack."""
        E, C, gs, dev = self.E, self.C, self.group_size, self.device
        G = (C + gs - 1) // gs
        mse = self.quantization_scale == "mse"
        cand = torch.linspace(1.0, max_shrink, n_grid, dtype=torch.float32, device=dev) if mse else None
        if self.H is None:
            self.H = torch.empty((E, C, C), dtype=torch.float32, device=dev)
        # experts that never saw a token (or whose Hessian went NaN) fall back to H = I
        seen = torch.tensor([n > 0 for n in self.num_samples], device=dev)
        bad = ~seen
        if bool(seen.any()):
            nan = torch.isnan(self.H[seen].diagonal(dim1=1, dim2=2)).any(dim=1)
            bad[seen.nonzero().flatten()[nan]] = True
        if bool(bad.any()):
            self.H[bad] = torch.eye(C, device=dev, dtype=torch.float32)

        outs = [[None, None, None] for _ in self.W]
        for i, W in enumerate(self.W):
            R = W.shape[1]
            outs[i][0] = torch.empty((E, R, C), dtype=torch.uint8, device=dev)
        for e0 in range(0, E, chunk):
            e1 = min(E, e0 + chunk)
            B = e1 - e0
            H = self.H[e0:e1]
            diag = H.diagonal(dim1=1, dim2=2)
            dead = diag == 0                                             # [B, C]
            has_dead = bool(dead.any())
            if self.quantization_order == "activation":
                perm = torch.argsort(torch.where(dead, torch.ones_like(diag), diag), dim=1,
                                     descending=True)
            else:
                perm = torch.arange(C, device=dev).expand(B, C).contiguous()
            perm_inv = torch.argsort(perm, dim=1)
            g_idx = (perm // gs).to(torch.int32).contiguous()
            dead_u8 = dead.to(torch.uint8).contiguous()
            dead_perm = torch.gather(dead, 1, perm)
            # weights with pruned columns zeroed decide the (unpermuted-index) zero-column
            # mask that the reference applies to the permuted Hessian (forge/gptq.py:145-149)
            masks = []
            for W in self.W:
                Wc = W[e0:e1]
                zero_cols = ((Wc == 0) | dead[:, None, :]).all(dim=1)
                masks.append((dead_perm | zero_cols).to(torch.uint8).contiguous())
            shared = all(torch.equal(masks[0], m) for m in masks[1:])
            U = None
            for i, W in enumerate(self.W):
                Wc = W[e0:e1]
                R = Wc.shape[1]
                if U is None or not shared:
                    Hp, damp = kernels.hessian_permute(H, perm, masks[i], float(self.rel_damp))
                    U, _, info = kernels.chol_inv_upper_batched(Hp, damp, normalise=True)
                    del Hp
                    self.issue_non_invertible[e0:e1] |= (info > 0).cpu()
                # pruned columns are zero in the reference's W before the grid is built
                Wsrc = Wc.masked_fill(dead[:, None, :], 0) if has_dead else Wc
                scales, qzeros = kernels.quant_grid(Wsrc, gs, self.bits, self.symmetric, mse, cand,
                                                    norm)
                del Wsrc
                X = kernels.weight_to_solver_order(Wc, perm_inv, dead_u8)
                sT = scales.view(B, R, G).transpose(1, 2).contiguous()
                zT = qzeros.view(B, R, G).transpose(1, 2).contiguous()
                q = kernels.gptq_sweep_batched(X, U, sT, zT, g_idx, self.bits)
                del X
                outs[i][0][e0:e1] = kernels.codes_to_layer_order(q, perm_inv)
                if outs[i][1] is None:
                    outs[i][1] = torch.empty((E, R * G), dtype=torch.float32, device=dev)
                    outs[i][2] = torch.empty((E, R * G), dtype=torch.float32, device=dev)
                outs[i][1][e0:e1] = scales
                outs[i][2][e0:e1] = qzeros
            del U
        return [tuple(o) for o in outs]
