"""Per-layer GPTQ handle on MI355X: drop-in for the reference's ``forge.gptq.GPTQ``.

Same constructor, methods, attributes and return values as forge/gptq.py:10-276 of the
reference (``update``/``add_batch`` accumulate the Hessian from calibration activations,
``quantize`` returns ``(qweight [R,C] u8, scales [R*G] f32, qzeros [R*G] f32[, M])``), but
every stage is a HIP kernel from ``forge.backend.hip``:

=====================  ==============================================================
reference (torch/CUDA)  here
=====================  ==============================================================
``H.addmm_``            ragged rank-k MFMA update (``hessian_update_grouped``)
``H[perm][:, perm]``    fused gather + dead-column fix-up (``hessian_permute``)
3 x cuSOLVER            one batched factorisation (``chol_inv_upper_batched``)
grid kernels            ``quant_grid`` (min/max + shrink search, straight from bf16/f32)
``repeat_interleave``   none: the sweep looks scales up by group (``g_idx = perm // gs``)
32-column sweep + SGEMM  128-column register sweep + chained f32 MFMA GEMM
=====================  ==============================================================

There is no CPU path: tensors must live on the GPU and the HIP library must be built.
"""
from __future__ import annotations

import uuid

import torch

from forge.backend.hip import kernels


def _as_calibration_rows(X: torch.Tensor, device) -> torch.Tensor:
    """Flatten to [n, C]; bf16 and f32 are consumed as they are, anything else as f32."""
    X = X.reshape(-1, X.shape[-1]).to(device=device)
    if X.dtype not in (torch.bfloat16, torch.float32):
        X = X.to(torch.float32)
    if X.stride(-1) != 1:
        X = X.contiguous()
    return X


class GPTQ(object):
    def __init__(self, layer, bits: int = 4, group_size: int = 128, symmetric: bool = False,
                 quantization_scale: str = "mse", quantization_order: str = "activation",
                 rel_damp: float = 1e-2, algorithm: str = "gptq", owner=None, device=None,
                 factor_route: str = "inverse"):
        """Arguments of the reference's class (forge/gptq.py:11-22) plus ``factor_route``
        (algorithms "gptq" and "sparsegptq"; Babai has its own factor): "inverse", the default, follows the reference's
        factorisation (Cholesky, inverse, Cholesky of the inverse) and its error-propagating
        sweep; "direct" stops at the factor of H itself and sweeps with the displacements
        w - deq, which is the same solve in exact arithmetic at half the factorisation work
        (see ``forge.moe.ExpertGroupGPTQ``)."""
        if algorithm not in ("gptq", "sparsegptq", "babai"):
            raise NotImplementedError(f"algorithm={algorithm!r}: 'gptq', 'sparsegptq' or 'babai'")
        if factor_route not in ("direct", "inverse"):
            raise ValueError(f"factor_route={factor_route!r}: 'direct' or 'inverse'")
        self.factor_route = factor_route
        self.layer = layer
        self.device = torch.device(device) if device is not None else layer.weight.device
        if self.device.type != "cuda":
            raise RuntimeError("forge.gptq.GPTQ runs on the GPU only (device must be a cuda "
                               f"device, got {self.device}); there is no CPU fallback")
        self.W = layer.weight.detach().clone().to(self.device)      # [R, C]
        self.H = None
        self.num_samples = torch.zeros((), device=self.device, dtype=torch.int64)
        self._n_host = 0                    # same count, kept on the host: no sync per update
        self.bits = bits
        self.group_size = group_size
        self.symmetric = symmetric
        self.quantization_scale = quantization_scale
        self.quantization_order = quantization_order
        self.rel_damp = rel_damp
        self.algorithm = algorithm
        self.owner = owner if owner is not None else self
        self.perm = None
        self.perm_inv = None
        self.pruned_ids = None
        self.prepared = False
        self.issue_non_invertible = False
        self.G = None
        self.id = uuid.uuid4()

    def _is_owner(self):
        return self.id == self.owner.id

    # ------------------------------------------------------------------ state
    @torch.no_grad()
    def reset(self):
        self.W = self.layer.weight.detach().clone().to(self.device)
        self.H = None
        self.num_samples = torch.zeros((), device=self.device, dtype=torch.int64)
        self._n_host = 0
        self.prepared = False
        self.perm = self.perm_inv = self.pruned_ids = None
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Hessian
    @torch.no_grad()
    def update(self, X: torch.Tensor):
        """H <- (n/N) H + (2/N) X^T X with N = n + rows(X); the owner accumulates."""
        if not self._is_owner():
            return
        o = self.owner
        X = _as_calibration_rows(X, o.device)
        new = int(X.shape[0])
        if new == 0:
            return
        C = int(X.shape[1])
        n = o._n_host
        total = n + new
        if o.H is None:
            o.H = torch.empty((C, C), dtype=torch.float32, device=o.device)
        # first call: beta == 0, H is written without being read
        kernels.hessian_update_grouped(X, [0, new], o.H.view(1, C, C), [2.0 / total], [n / total])
        o._n_host = total
        o.num_samples.add_(new)

    add_batch = update

    # ------------------------------------------------------------------ prepare
    def _copy_owner_state(self):
        o = self.owner
        self.H = o.H.clone()
        self.pruned_ids = o.pruned_ids.clone()
        self.perm = o.perm.clone()
        self.perm_inv = o.perm_inv.clone()
        self.W[:, self.pruned_ids] = 0
        self.num_samples = o.num_samples.clone()
        self._n_host = o._n_host
        self.prepared = True

    @torch.no_grad()
    def _prep(self):
        o = self.owner
        if self._is_owner() and self.prepared:
            return
        if not self._is_owner() and o.prepared:
            if not self.prepared:
                self._copy_owner_state()
            return
        C = int(o.W.shape[-1])
        if o.H is None or o._n_host == 0 or bool(torch.isnan(o.H).any()):
            o.H = torch.eye(C, device=o.device, dtype=torch.float32)
        dead = torch.diag(o.H) == 0
        o.pruned_ids = dead
        if o.quantization_order == "activation":
            diag = torch.where(dead, torch.ones_like(torch.diag(o.H)), torch.diag(o.H))
            # Babai walks the columns back to front: ascending order (forge/gptq.py:107-108)
            o.perm = torch.argsort(diag, descending=o.algorithm != "babai")
        else:
            o.perm = torch.arange(C, device=o.device)
        o.perm_inv = torch.argsort(o.perm)
        o.W[:, dead] = 0
        # H[perm][:, perm] with the dead rows/columns cleared and their diagonal set to 1
        Hp, _ = kernels.hessian_permute(o.H.view(1, C, C), o.perm.view(1, C),
                                        dead[o.perm].to(torch.uint8).view(1, C), 0.0)
        o.H = Hp[0]
        o.prepared = True
        if not self._is_owner():
            self._copy_owner_state()

    # ------------------------------------------------------------------ stages
    @torch.no_grad()
    def _quant_grid(self, max_shrink: float = 0.2, n_grid: int = 100, norm: float = 2.4):
        R, C = self.W.shape
        mse = self.quantization_scale == "mse"
        cand = None
        if mse:
            cand = torch.linspace(1.0, max_shrink, n_grid, dtype=torch.float32, device=self.device)
        W = self.W if self.W.dtype in (torch.float32, torch.bfloat16) else self.W.float()
        scales, qzeros = kernels.quant_grid(W, self.group_size, self.bits, self.symmetric, mse,
                                            cand, norm)
        self.G = (C + self.group_size - 1) // self.group_size
        return scales, qzeros

    @torch.no_grad()
    def _h_factor(self):
        """Row-normalised ('gptq') or raw ('sparsegptq') upper Cholesky factor of
        inv(H + damp I); identity when the factorisation fails.  As in the reference the
        fix-ups and the damping are applied to self.H in place (forge/gptq.py:143-154), so
        a non-owner that copies its owner's Hessian afterwards sees the damped matrix."""
        H = self.H
        C = int(self.W.shape[-1])
        zero_cols = self.W.eq(0).all(dim=0)      # original column order, used on permuted H
        if bool(zero_cols.any()):
            H[zero_cols, :] = 0
            H[:, zero_cols] = 0
            H[zero_cols, zero_cols] = 1.0
        H.diagonal().add_(float(self.rel_damp) * torch.diag(H).mean())
        if self.algorithm == "babai":
            # The reference factors H = A^T A (A upper, forge/gptq.py:157-158) and sweeps from
            # the last column to the first.  With both index orders reversed that is a forward
            # sweep whose unit upper matrix comes from the LOWER factor of the reversed H.
            L, info = kernels.chol_reverse_lower_batched(H.flip(0, 1).contiguous().view(1, C, C), None)
            if int(info.item()) > 0:
                self.issue_non_invertible = True
            return kernels.unit_upper_from_lower(L, info)[0]
        sparse = self.algorithm == "sparsegptq"
        if self.factor_route == "direct":
            L, info = kernels.chol_reverse_lower_batched(H.clone().view(1, C, C), None)
            if int(info.item()) > 0:
                self.issue_non_invertible = True
            if sparse:
                # 1/diag(U) of the mask score (solver_sparsegptq14.cu:153) is the diagonal of
                # the factor of H itself; 1 where the factorisation failed (U = I)
                self._score_weight = torch.where(info[:, None] != 0, torch.ones((), device=H.device),
                                                 L.diagonal(dim1=1, dim2=2)).contiguous()
            return kernels.unit_upper_from_lower(L, info, negate=True, upper_only=True)[0]
        U, udiag, info = kernels.chol_inv_upper_batched(H.clone().view(1, C, C), None,
                                                        normalise=not sparse)
        if int(info.item()) > 0:
            self.issue_non_invertible = True
        if sparse:
            # rows scaled by the rounded reciprocal of the diagonal, as
            # solver_sparsegptq14.cu:153-155 does to its caller's tensor
            self._score_weight = (1.0 / udiag).contiguous()
            U.mul_(self._score_weight.unsqueeze(-1))
        return U[0]

    @torch.no_grad()
    def quantize(self):
        self._prep()
        scales, qzeros = self._quant_grid()
        U = self._h_factor()
        R, C = self.W.shape
        G, gs = self.G, self.group_size
        W = self.W if self.W.dtype in (torch.float32, torch.bfloat16) else self.W.float()
        if self.algorithm == "babai":
            # solver order = the reference's permuted order reversed (see _h_factor)
            perm_r = self.perm.flip(0)
            perm_r_inv = torch.argsort(perm_r)
            X = kernels.weight_to_solver_order(W.view(1, R, C), perm_r_inv.view(1, C))
            g_idx = (perm_r // gs).to(torch.int32).view(1, C)
            sT = scales.view(R, G).t().contiguous().view(1, G, R)
            zT = qzeros.view(R, G).t().contiguous().view(1, G, R)
            q = kernels.gptq_sweep_batched(X, U.view(1, C, C), sT, zT, g_idx, self.bits)
            return kernels.codes_to_layer_order(q, perm_r_inv.view(1, C))[0], scales, qzeros
        W0 = None
        if self.factor_route == "direct":
            W0 = torch.empty((1, C, R), dtype=W.dtype, device=W.device)
        X = kernels.weight_to_solver_order(W.view(1, R, C), self.perm_inv.view(1, C), out0=W0)
        g_idx = (self.perm // gs).to(torch.int32).view(1, C)
        sT = scales.view(R, G).t().contiguous().view(1, G, R)
        zT = qzeros.view(R, G).t().contiguous().view(1, G, R)
        # per-group scales and zeros are looked up through g_idx inside the sweep: the two
        # [C, R] expansions of forge/gptq.py:251-252 are never materialised
        if self.algorithm == "sparsegptq":
            if self.factor_route == "direct":
                q, M = kernels.gptq_sweep_direct_batched(X, U.view(1, C, C), sT, zT, g_idx, self.bits,
                                                         W0=W0, sparse14=True, mdiag=self._score_weight)
            else:
                q, M = kernels.gptq_sweep_batched(X, U.view(1, C, C), sT, zT, g_idx, self.bits,
                                                  sparse14=True, uinv=self._score_weight)
            qw = kernels.codes_to_layer_order(q, self.perm_inv.view(1, C))[0]
            return qw, scales, qzeros, M[0]
        if self.factor_route == "direct":
            q = kernels.gptq_sweep_direct_batched(X, U.view(1, C, C), sT, zT, g_idx, self.bits, W0=W0)
        else:
            q = kernels.gptq_sweep_batched(X, U.view(1, C, C), sT, zT, g_idx, self.bits)
        qw = kernels.codes_to_layer_order(q, self.perm_inv.view(1, C))[0]
        return qw, scales, qzeros
