"""Float64 closed forms that pin the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Each routine is what the mathematics fixes, written independently of forge_oracle.c:
a dropped term, a wrong sign or a transposed operand in the oracle fails against one
of these.
"""
from __future__ import annotations

import numpy as np
import torch

EPS = np.float32(1e-12)


def hessian(batches):
    """H = (2/N) * sum_b X_b^T X_b, the fixed point of the running mean in
    forge/gptq.py:61-80."""
    n = sum(int(b.shape[0]) for b in batches)
    C = batches[0].shape[1]
    H = np.zeros((C, C), dtype=np.float64)
    for b in batches:
        b = np.asarray(b, dtype=np.float64)
        H += b.T @ b
    return 2.0 * H / n


def _raise_if_failed(info):
    if int(info) != 0:
        raise np.linalg.LinAlgError("matrix is not positive definite")


def factor(H, rel_damp, normalise=True):
    """Upper Cholesky factor of inv(H + damp*I) (forge/gptq.py:152-164) in float64: the three
    LAPACK steps of gptq.py:160-164 through torch's float64 routines (all host threads; the
    general inverse plus scipy's Cholesky that this replaces gave the same matrix to 1e-13 and
    took five times as long at 7168 features)."""
    H = np.array(H, dtype=np.float64)
    H[np.diag_indices_from(H)] += rel_damp * np.mean(np.diag(H))
    L, info = torch.linalg.cholesky_ex(torch.from_numpy(H))
    _raise_if_failed(info)
    U0, info = torch.linalg.cholesky_ex(torch.cholesky_inverse(L), upper=True)
    _raise_if_failed(info)
    U0 = U0.numpy()
    return U0 / np.diag(U0)[:, None] if normalise else U0


def direct_factor(H, rel_damp):
    """V for the displacement form of the sweep: with H + damp*I = M M^T (M upper, the
    Cholesky factor taken from the last row upwards), V[t,k] = -M[t,k]/M[k,k] above the
    diagonal and 1 on it.  I - strict(V) is the inverse of ``factor(H, rel_damp)``."""
    H = np.array(H, dtype=np.float64)
    H[np.diag_indices_from(H)] += rel_damp * np.mean(np.diag(H))
    H = 0.5 * (H + H.T)
    Lr, info = torch.linalg.cholesky_ex(torch.from_numpy(np.ascontiguousarray(H[::-1, ::-1])))
    _raise_if_failed(info)
    M = Lr.numpy()[::-1, ::-1]
    V = -(M / np.diag(M)[None, :])
    V[np.diag_indices_from(V)] = 1.0
    return np.triu(V)


def minmax_grid(Xg, bits, symmetric):
    """Closed form of the per-group scale/zero (forge/backend/cuda/quant_grid.cu:78-93),
    evaluated with numpy float32 scalars."""
    Xg = np.asarray(Xg, dtype=np.float32)
    maxq = np.float32(2 ** bits - 1)
    lo, hi = Xg.min(axis=1), Xg.max(axis=1)
    if symmetric:
        amax = np.maximum(np.abs(lo), np.abs(hi))
        # one rounding (fused) for (2/maxq)*amax+eps: do it in float64, then round once
        s = (np.float64(np.float32(2.0) / maxq) * amax.astype(np.float64) + np.float64(EPS)).astype(np.float32)
        q0 = np.full_like(s, (maxq + 1) / 2)
    else:
        s = ((hi - lo) / maxq + EPS).astype(np.float32)
        q0 = np.clip(np.rint((-lo / s).astype(np.float32)), 0, maxq).astype(np.float32)
    return s, q0


def mse_losses(xg, sg, q0g, cands, bits, symmetric, norm):
    """Float64 loss of every shrink candidate for ONE group (quant_grid.cu:142-170);
    quantisation itself follows the fp32 rule so that the codes are the same."""
    maxq = np.float32(2 ** bits - 1)
    xg = np.asarray(xg, dtype=np.float32)
    out = np.empty(len(cands), dtype=np.float64)
    zs = np.empty(len(cands), dtype=np.float32)
    ss = np.empty(len(cands), dtype=np.float32)
    xmin = np.float32(0) if symmetric else -(np.float32(sg) * np.float32(q0g))
    for i, p in enumerate(np.asarray(cands, dtype=np.float32)):
        s = np.float32(sg) * p
        rcp = np.float32(1) / (s + EPS)
        q0 = np.float32(q0g) if symmetric else np.clip(np.rint(-xmin * rcp), 0, maxq).astype(np.float32)
        biased = (xg.astype(np.float64) * np.float64(rcp) + np.float64(q0)).astype(np.float32)  # fma
        q = np.clip(np.rint(biased), 0, maxq)
        diff = (q.astype(np.float64) - np.float64(q0)) * np.float64(s) - xg.astype(np.float64)
        out[i] = np.sum(np.maximum(np.abs(diff), 1e-20) ** norm)
        zs[i], ss[i] = q0, s
    return out, ss, zs


def gptq_textbook(W, H, scales_e, zeros_e, bits, rel_damp):
    """Unblocked GPTQ (Frantar et al., Alg. 1 with static groups) in float64 using the
    UN-normalised factor: err = (w - deq)/U0[t,t]; W[:, t:] -= err * U0[t, t:].
    W [R,C]; scales_e/zeros_e per element [R,C].  Returns codes [R,C] and dequantised."""
    maxq = 2 ** bits - 1
    W = np.array(W, dtype=np.float64)
    R, C = W.shape
    U0 = factor(H, rel_damp, normalise=False)
    Q = np.zeros((R, C), dtype=np.int64)
    D = np.zeros((R, C), dtype=np.float64)
    s = np.asarray(scales_e, dtype=np.float64)
    z = np.asarray(zeros_e, dtype=np.float64)
    margins = np.zeros((R, C))
    for t in range(C):
        w = W[:, t]
        b = w / (s[:, t] + 1e-12) + z[:, t]
        margins[:, t] = np.abs(b - np.floor(b) - 0.5)
        q = np.clip(np.rint(b), 0, maxq)
        d = (q - z[:, t]) * s[:, t]
        Q[:, t], D[:, t] = q, d
        err = (w - d) / U0[t, t]
        W[:, t:] -= np.outer(err, U0[t, t:])
    return Q, D, margins


def rtn(W, scales_e, zeros_e, bits):
    """Round-to-nearest with the fp32 rule of solver.cu:9-23 (what the sweep must give
    bit-for-bit when U = I)."""
    maxq = 2 ** bits - 1
    W = np.asarray(W, dtype=np.float32)
    s = np.asarray(scales_e, dtype=np.float32)
    z = np.asarray(zeros_e, dtype=np.float32)
    inv = (np.float32(1) / (s + EPS)).astype(np.float32)
    biased = (W.astype(np.float64) * inv.astype(np.float64) + z.astype(np.float64)).astype(np.float32)
    return np.clip(np.rint(biased), 0, maxq).astype(np.uint8)


def layer_error(W, Q, H):
    """tr((W-Q) H (W-Q)^T): proportional to ||WX - QX||^2 for the Hessian's tokens."""
    D = torch.from_numpy(np.asarray(W, dtype=np.float64) - np.asarray(Q, dtype=np.float64))
    Hd = torch.from_numpy(np.ascontiguousarray(H, dtype=np.float64))
    # (one float64 matrix product on all host threads, then a dot product)
    return float(((D @ Hd) * D).sum())
