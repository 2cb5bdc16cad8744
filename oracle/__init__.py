"""CPU oracle for the GPTQ calibration-and-solve path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module.  It exists so that tests, the
smoke check and the benchmark's ``cpu_baseline`` leg can compare the HIP kernels with a
CPU restatement of the reference's arithmetic:

* ``kernels``  -- the four hot-path operators with the reference's Python signatures
  (forge/backend/cuda/kernels.cpp:92-120), executed by ``libforge_oracle.so``
  (scalar C, see forge_oracle.c) on CPU tensors;
* ``GPTQ``     -- the per-layer host logic of forge/gptq.py:10-276 on ``device="cpu"``
  (torch's CPU ``addmm_``, LAPACK ``cholesky_ex``/``cholesky_inverse`` and ``argsort``
  stand where the reference calls the same torch routines on its device);
* ``mathref``  -- float64 closed forms used to pin the two above.

Pinned by (tests/test_oracle_*.py): closed forms for the min/max grid, brute-force
float64 search for the MSE grid, U = I reducing the sweep to round-to-nearest, the
textbook unblocked GPTQ recursion in float64, block-size invariance, scipy's float64
``cholesky(inv(H))`` for the factor, and the 1:4 mask invariants.
parity unpinned: bits of nvcc's ``__logf``/``__expf`` and of cuBLAS' SGEMM summation
order (no reference fixture exists and CUDA cannot run here); the oracle uses libm and
a stated fmaf order for them.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import uuid
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import torch

_HERE = Path(__file__).resolve().parent
_LIB = None

TRAIL_CHAIN = 0
TRAIL_GEMM = 1
TRAIL_BLAS = 2      # in-block in C, trailing update with torch's CPU SGEMM (addmm_)


def build(force: bool = False) -> Path:
    """Compile forge_oracle.c with gcc (recipe: oracle/Makefile)."""
    so = _HERE / "libforge_oracle.so"
    if force and so.exists():
        so.unlink()
    subprocess.run(["make", "-C", str(_HERE), "-s"], check=True)
    return so


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        so = _HERE / "libforge_oracle.so"
        if not so.exists():
            build()
        L = ctypes.CDLL(str(so))
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.oracle_build_group_meta.argtypes = [vp, i64, i64, i32, i32, vp, vp]
        L.oracle_mse_scale_groups.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, f32, i32, vp]
        L.oracle_gptq_solver.argtypes = [vp, vp, vp, vp, i32, i64, i64, vp, i32, i64]
        L.oracle_sparsegptq14_solver.argtypes = [vp, vp, vp, vp, i32, i64, i64, vp, vp, i32]
        L.oracle_gptq_inblock.argtypes = [vp, vp, vp, vp, i32, i64, i64, i64, i64, vp, vp]
        L.oracle_babai_solver.argtypes = [vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, vp, i32, i64]
        L.oracle_babai_solver.restype = None
        L.oracle_gptq_solver_direct.argtypes = [vp, vp, vp, vp, i32, i64, i64, vp]
        L.oracle_gptq_solver_direct.restype = None
        L.oracle_sparsegptq14_solver_direct.argtypes = [vp, vp, vp, vp, vp, i32, i64, i64, vp, vp]
        L.oracle_sparsegptq14_solver_direct.restype = None
        L.oracle_pack_sparsegptq14.argtypes = [vp, vp, vp, vp, i64, i64]
        L.oracle_pack_sparsegptq14.restype = None
        for f in (L.oracle_build_group_meta, L.oracle_mse_scale_groups, L.oracle_gptq_solver,
                  L.oracle_sparsegptq14_solver, L.oracle_gptq_inblock):
            f.restype = None
        _LIB = L
    return _LIB


def _f32c(t: torch.Tensor) -> torch.Tensor:
    assert t.device.type == "cpu"
    return t.to(torch.float32).contiguous()


def build_group_meta_packed(X: torch.Tensor, bit_width: int, symmetric: bool):
    """kernels.cpp:93-97 -> quant_grid.cu:186-224.  X [RG, gs] f32."""
    X = _f32c(X)
    RG, gs = X.shape
    scales = torch.empty(RG, dtype=torch.float32)
    qzeros = torch.empty(RG, dtype=torch.float32)
    lib().oracle_build_group_meta(X.data_ptr(), RG, gs, int(bit_width), int(bool(symmetric)),
                                  scales.data_ptr(), qzeros.data_ptr())
    return scales, qzeros


def mse_scale_groups_packed(X, scales, qzeros, candidates, norm, bit_width, symmetric,
                            return_losses: bool = False):
    """kernels.cpp:98-102 -> quant_grid.cu:227-287.  Overwrites scales/qzeros in place."""
    X = _f32c(X)
    RG, gs = X.shape
    if gs not in (32, 64, 128):
        raise RuntimeError(f"Unsupported group_size={gs} (expected 32/64/128)")
    assert scales.dtype == torch.float32 and scales.is_contiguous()
    assert qzeros.dtype == torch.float32 and qzeros.is_contiguous()
    cand = _f32c(candidates)
    P = cand.numel()
    losses = torch.empty((RG, P), dtype=torch.float32) if return_losses else None
    lib().oracle_mse_scale_groups(X.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
                                  cand.data_ptr(), RG, gs, P, int(bit_width), float(norm),
                                  int(bool(symmetric)),
                                  losses.data_ptr() if return_losses else None)
    if return_losses:
        return scales, qzeros, losses
    return scales, qzeros


def gptq_solver(W, U, scales, qzeros, bits, trail_mode: int = TRAIL_CHAIN, block: int = 32):
    """kernels.cpp:104-108 -> solver.cu:99-154.  W [C,R] f32 (made contiguous; the
    contiguous copy receives the dequantised weights), returns qweight [C,R] u8."""
    W = W.contiguous() if W.dtype == torch.float32 else W.to(torch.float32).contiguous()
    U = _f32c(U); scales = _f32c(scales); qzeros = _f32c(qzeros)
    C, R = W.shape
    q = torch.empty((C, R), dtype=torch.uint8)
    if trail_mode == TRAIL_BLAS:
        # the reference's host loop literally: 32-column kernel, then one SGEMM per block
        E = torch.empty((block, R), dtype=torch.float32)
        for start in range(0, C, block):
            end = min(start + block, C)
            lib().oracle_gptq_inblock(W.data_ptr(), U.data_ptr(), scales.data_ptr(),
                                      qzeros.data_ptr(), int(bits), C, R, start, end - start,
                                      q.data_ptr(), E.data_ptr())
            if end < C:
                W[end:].addmm_(U[start:end, end:].t(), E[:end - start], beta=1.0, alpha=-1.0)
    else:
        lib().oracle_gptq_solver(W.data_ptr(), U.data_ptr(), scales.data_ptr(),
                                 qzeros.data_ptr(), int(bits), C, R, q.data_ptr(),
                                 int(trail_mode), int(block))
    gptq_solver.last_W = W
    return q


def gptq_solver_direct(W, V, scales, qzeros, bits):
    """Checker for the library's displacement form of the sweep (no reference counterpart):
    V [C,C] = -M[t,k]/M[k,k] above the diagonal for H + damp I = M M^T, columns hand on
    d = w0 - deq.  W [C,R], scales/qzeros [C,R] per element; returns qweight [C,R] u8."""
    W = W.contiguous() if W.dtype == torch.float32 else W.to(torch.float32).contiguous()
    V = _f32c(V); scales = _f32c(scales); qzeros = _f32c(qzeros)
    C, R = W.shape
    q = torch.empty((C, R), dtype=torch.uint8)
    lib().oracle_gptq_solver_direct(W.data_ptr(), V.data_ptr(), scales.data_ptr(),
                                    qzeros.data_ptr(), int(bits), C, R, q.data_ptr())
    gptq_solver_direct.last_W = W
    return q


def sparsegptq14_solver_direct(W, V, mdiag, scales, qzeros, bits):
    """Checker for the displacement form of the 1:4 joint solve: V as for gptq_solver_direct,
    mdiag [C] = diag of the factor M of H + damp I = M M^T.  Returns (qweight [C,R] u8,
    M [ceil(C/32), R] uint32)."""
    W = W.contiguous() if W.dtype == torch.float32 else W.to(torch.float32).contiguous()
    V = _f32c(V); mdiag = _f32c(mdiag); scales = _f32c(scales); qzeros = _f32c(qzeros)
    C, R = W.shape
    q = torch.empty((C, R), dtype=torch.uint8)
    M = torch.zeros(((C + 31) // 32, R), dtype=torch.uint32)
    lib().oracle_sparsegptq14_solver_direct(W.data_ptr(), V.data_ptr(), mdiag.data_ptr(),
                                            scales.data_ptr(), qzeros.data_ptr(), int(bits), C, R,
                                            q.data_ptr(), M.data_ptr())
    sparsegptq14_solver_direct.last_W = W
    return q, M


def babai_solver(W, A, scales, qzeros, group_size, bits, block_size, g_idx, G,
                 trail_mode: int = TRAIL_CHAIN):
    """kernels.cpp:46-56 -> solver_babai.cu:217-322.  W [C,R] f32 (the contiguous copy
    receives the dequantised weights), A [C,C] upper factor of H, scales/qzeros [R*G],
    g_idx [C] int32.  Returns qweight [C,R] u8.  The host checks are the reference's."""
    W = W.contiguous() if W.dtype == torch.float32 else W.to(torch.float32).contiguous()
    A = _f32c(A); scales = _f32c(scales); qzeros = _f32c(qzeros)
    C, R = W.shape
    gs = min(int(group_size), C)
    if gs <= 0 or gs % 32 != 0:
        raise RuntimeError("group_size must be multiple of 32 (effective group_size)")
    if (C + gs - 1) // gs != int(G):
        raise RuntimeError("qmeta G mismatch")
    block = int(block_size)
    if block <= 0 or block > 32:
        block = 32
    block = min(block, C)
    gi = None if g_idx is None else g_idx.to(torch.int32).contiguous()
    q = torch.zeros((C, R), dtype=torch.uint8)
    lib().oracle_babai_solver(W.data_ptr(), A.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
                              None if gi is None else gi.data_ptr(), gs, int(bits), C, R, int(G),
                              q.data_ptr(), int(trail_mode), block)
    babai_solver.last_W = W
    return q


def sparsegptq14_solver(W, U, scales, qzeros, bits, trail_mode: int = TRAIL_CHAIN):
    """kernels.cpp:110-120 -> solver_sparsegptq14.cu:142-200.  Row-normalises U in place."""
    W = W.contiguous() if W.dtype == torch.float32 else W.to(torch.float32).contiguous()
    assert U.dtype == torch.float32 and U.is_contiguous()
    scales = _f32c(scales); qzeros = _f32c(qzeros)
    C, R = W.shape
    q = torch.empty((C, R), dtype=torch.uint8)
    M = torch.empty(((C + 31) // 32, R), dtype=torch.int32)
    lib().oracle_sparsegptq14_solver(W.data_ptr(), U.data_ptr(), scales.data_ptr(),
                                     qzeros.data_ptr(), int(bits), C, R, q.data_ptr(),
                                     M.data_ptr(), int(trail_mode))
    sparsegptq14_solver.last_W = W
    return q, M.view(torch.uint32) if hasattr(torch, "uint32") else M


def pack_sparsegptq14_to_u64x2(qweight_rc, M, scales):
    """kernels.cpp:122-126 -> bitpacking_sparsegptq14.cu:110-172.  Returns int64 [G2,R,2]
    holding the u64 bit patterns."""
    q = qweight_rc.contiguous()
    R, C = q.shape
    G32 = (C + 31) // 32
    Mi = M.contiguous().view(torch.int32)
    sc = _f32c(scales)
    assert tuple(Mi.shape) == (G32, R) and tuple(sc.shape) == (G32, R) and q.dtype == torch.uint8
    out = torch.empty(((G32 + 1) // 2, R, 2), dtype=torch.int64)
    lib().oracle_pack_sparsegptq14(q.data_ptr(), Mi.data_ptr(), sc.data_ptr(), out.data_ptr(), R, C)
    return out


def fp8_block_dequant(w_fp8, scale_inv, dtype=torch.bfloat16):
    """The reference's own torch expression for DeepSeek fp8 weights
    (forge/utils/io.py:533-563,863-872): f32(w) * scale_inv per so x si tile -> dtype."""
    w = w_fp8.to(torch.float32)
    O, I = w.shape
    nO, nI = scale_inv.shape
    assert I % nI == 0
    si = I // nI
    so = si if (O + si - 1) // si == nO else (O + nO - 1) // nO
    rows = torch.arange(O) // so
    cols = torch.arange(I) // si
    return (w * scale_inv.float()[rows][:, cols]).to(dtype)


kernels = SimpleNamespace(
    build_group_meta_packed=build_group_meta_packed,
    mse_scale_groups_packed=mse_scale_groups_packed,
    gptq_solver=gptq_solver,
    sparsegptq14_solver=sparsegptq14_solver,
    pack_sparsegptq14_to_u64x2=pack_sparsegptq14_to_u64x2,
)


class GPTQ:
    """CPU restatement of the reference's per-layer solver object (forge/gptq.py:10-276).

    Same constructor, attributes and return values; always runs on the CPU.  ``trail_mode``
    selects the oracle's trailing-update summation order (see forge_oracle.c).
    """

    def __init__(self, layer, bits=4, group_size=128, symmetric=False,
                 quantization_scale="mse", quantization_order="activation", rel_damp=1e-2,
                 algorithm="gptq", owner=None, device=None, trail_mode=TRAIL_CHAIN):
        # gptq.py:11-43
        self.layer = layer
        self.W = layer.weight.detach().clone().cpu()
        self.device = "cpu"
        self.H = None
        self.num_samples = torch.zeros((), dtype=torch.int64)
        self.bits, self.group_size, self.symmetric = bits, group_size, symmetric
        self.quantization_scale = quantization_scale
        self.quantization_order = quantization_order
        self.rel_damp = rel_damp
        self.algorithm = algorithm
        self.owner = self if owner is None else owner
        self.perm = self.perm_inv = self.pruned_ids = None
        self.prepared = False
        self.issue_non_invertible = False
        self.trail_mode = trail_mode
        self.id = uuid.uuid4()

    def _is_owner(self):
        return self.id == self.owner.id

    @torch.no_grad()
    def reset(self):
        # gptq.py:49-59
        self.W = self.layer.weight.detach().clone().cpu()
        self.H = None
        self.num_samples = torch.zeros((), dtype=torch.int64)
        self.prepared = False
        self.perm = self.perm_inv = self.pruned_ids = None

    @torch.no_grad()
    def update(self, X):
        # gptq.py:61-80: running mean H <- (n/N) H + (2/N) X^T X, owner only.
        if not self._is_owner():
            return
        o = self.owner
        X = X.reshape(-1, X.shape[-1]).to(device="cpu", dtype=torch.float32)
        new = int(X.shape[0])
        if new == 0:
            return
        n = int(o.num_samples.item())
        total = n + new
        alpha = 2.0 / total
        if o.H is None:
            o.H = X.T @ (alpha * X)          # gptq.py:75-76 (overwritten below, beta == 0)
        o.H.addmm_(X.transpose(-2, -1), X, alpha=alpha, beta=n / total)
        o.num_samples.add_(new)

    add_batch = update

    def _adopt_owner_state(self):
        # gptq.py:86-94 / 119-126
        o = self.owner
        self.H = o.H.clone()
        self.pruned_ids = o.pruned_ids.clone()
        self.perm = o.perm.clone()
        self.perm_inv = o.perm_inv.clone()
        self.W[:, self.pruned_ids] = 0
        self.num_samples = o.num_samples.clone()
        self.prepared = True

    @torch.no_grad()
    def _prep(self):
        # gptq.py:82-126
        o = self.owner
        if self._is_owner() and self.prepared:
            return
        if (not self._is_owner()) and o.prepared and not self.prepared:
            self._adopt_owner_state()
            return
        C = int(o.W.shape[-1])
        if o.H is None or int(o.num_samples.item()) == 0 or bool(torch.isnan(o.H).any()):
            o.H = torch.eye(C, dtype=torch.float32)
        dead = torch.diag(o.H) == 0
        o.pruned_ids = dead
        o.H[dead, :] = 0
        o.H[:, dead] = 0
        o.H[dead, dead] = 1            # paired boolean index: hits the diagonal only
        if o.quantization_order == "activation":
            o.perm = torch.argsort(o.H.diag(), descending=(o.algorithm != "babai"))
        else:
            o.perm = torch.arange(C)
        o.perm_inv = torch.argsort(o.perm)
        o.W[:, dead] = 0
        o.prepared = True
        o.H = o.H[o.perm][:, o.perm]
        if (not self._is_owner()) and not self.prepared:
            self._adopt_owner_state()

    @torch.no_grad()
    def _quant_grid(self, max_shrink=0.2, n_grid=100, norm=2.4):
        # gptq.py:180-227: contiguous gs-wide groups of the UNPERMUTED weight, zero padded.
        W = self.W.clone()
        R, C = W.shape
        gs = self.group_size
        G = (C + gs - 1) // gs
        if G * gs != C:
            W = torch.nn.functional.pad(W, (0, G * gs - C))
        Wg = W.reshape(R * G, gs).to(torch.float32).contiguous()
        scales, qzeros = build_group_meta_packed(Wg, self.bits, self.symmetric)
        if self.quantization_scale == "mse":
            p = torch.linspace(1.0, max_shrink, n_grid, dtype=torch.float32)
            scales, qzeros = mse_scale_groups_packed(Wg, scales, qzeros, p, float(norm),
                                                     self.bits, self.symmetric)
        self.G = int(G)
        return scales, qzeros

    @torch.no_grad()
    def _h_factor(self):
        # gptq.py:141-177 (mutates self.H in place up to the first factorisation).
        H = self.H
        C = self.W.shape[-1]
        zero_cols = self.W.eq(0).all(dim=0)       # unpermuted columns on the permuted H
        if bool(zero_cols.any()):
            H[zero_cols, :] = 0
            H[:, zero_cols] = 0
            H[zero_cols, zero_cols] = 1.0
        damp = float(self.rel_damp) * torch.diag(H).mean()
        idx = torch.arange(C)
        H[idx, idx] += damp
        if self.algorithm == "babai":
            A, info = torch.linalg.cholesky_ex(H, upper=True)      # gptq.py:157-158: H = A^T A
            if int(info.item()) > 0:
                self.issue_non_invertible = True
                A = torch.eye(C, dtype=torch.float32)
            return A
        U, info = self._factor_upper(H)
        if int(info) > 0:
            self.issue_non_invertible = True
            U = torch.eye(C, dtype=torch.float32)
        return U

    def _factor_upper(self, H):
        """gptq.py:160-166: upper Cholesky factor of inv(H) through LAPACK's potrf, potri,
        potrf in fp32, rows divided by the diagonal for "gptq".  Returns (U, info)."""
        L, info = torch.linalg.cholesky_ex(H, upper=False)
        U = None
        try:
            Hinv = torch.cholesky_inverse(L, upper=False)
            U, info2 = torch.linalg.cholesky_ex(Hinv, upper=True)
            info = info + info2
            if self.algorithm == "gptq":
                U = U / U.diag()[:, None]
        except RuntimeError:
            # torch's CPU potri raises on a singular factor instead of carrying on; the
            # outcome the reference codes for is the identity fallback of the caller
            info = info + 1
        return U, int(info.item())

    def _expand(self, v, C, R):
        # gptq.py:251-252: per-element [C,R] meta in solver (permuted) column order.
        return (v.clone().view(R, self.G).repeat_interleave(self.group_size, dim=1)[:, :C]
                .transpose(-2, -1)[self.perm])

    @torch.no_grad()
    def quantize(self):
        # gptq.py:128-139
        self._prep()
        scales, qzeros = self._quant_grid()
        U = self._h_factor()
        self.last_factor = U            # kept for tests that swap single stages
        W = self.W.clone().transpose(-2, -1)[self.perm]
        C, R = W.shape
        if self.algorithm == "babai":
            # gptq.py:231-246
            g_idx = (self.perm // self.group_size).to(torch.int32)
            q = babai_solver(W.to(torch.float32), U, scales, qzeros, self.group_size, self.bits,
                             self.group_size // 4, g_idx, self.G, trail_mode=self.trail_mode)
            return q[self.perm_inv].transpose(-2, -1).contiguous(), scales, qzeros
        s_e, z_e = self._expand(scales, C, R), self._expand(qzeros, C, R)
        if self.algorithm == "sparsegptq":
            q, M = sparsegptq14_solver(W.to(torch.float32), U.contiguous(), s_e, z_e, self.bits,
                                       trail_mode=self.trail_mode)
            return q[self.perm_inv].transpose(-2, -1).contiguous(), scales, qzeros, M
        q = gptq_solver(W.to(torch.float32), U, s_e, z_e, self.bits, trail_mode=self.trail_mode)
        return q[self.perm_inv].transpose(-2, -1).contiguous(), scales, qzeros


def dequantize(qweight, scales, qzeros, group_size):
    """(q - q0) * s with flat [R*G] per-group meta (forge/utils/engine.py:71-97)."""
    R, C = qweight.shape
    G = (C + group_size - 1) // group_size
    s = scales.reshape(R, G).repeat_interleave(group_size, dim=1)[:, :C]
    z = qzeros.reshape(R, G).repeat_interleave(group_size, dim=1)[:, :C]
    return (qweight.to(torch.float32) - z.to(torch.float32)) * s.to(torch.float32)


def gather_scaled_rows(X, row_idx, weight=None):
    """x_e = x[tok_idx]; x_e_w = x_e * w.unsqueeze(-1) with w in x's dtype
    (forge/utils/engine.py:229-238)."""
    rows = X[row_idx]
    if weight is None:
        return rows
    return rows * weight.to(X.dtype).unsqueeze(-1)


def routed_rows(x, router_indices, routing_weights, num_experts):
    """The per-expert loop of the fused-expert hook (forge/utils/engine.py:224-238), its
    scaled rows concatenated in expert order with their offsets."""
    ri2 = router_indices.reshape(-1, router_indices.shape[-1] if router_indices.ndim > 1 else 1)
    rw2 = None if routing_weights is None else routing_weights.reshape(ri2.shape)
    parts, offsets = [], [0]
    for e in range(num_experts):
        tok_idx, k_idx = (ri2 == e).nonzero(as_tuple=True)
        x_e = x[tok_idx]
        if rw2 is not None:
            x_e = x_e * rw2[tok_idx, k_idx].to(x.dtype).unsqueeze(-1)
        parts.append(x_e)
        offsets.append(offsets[-1] + int(tok_idx.numel()))
    return torch.cat(parts, 0), offsets
