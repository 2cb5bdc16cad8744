"""Operator boundary of the MI355X backend.

``kernels`` exposes the hot-path operators under the names the reference binds in
forge/backend/cuda/kernels.cpp:92-120 (``build_group_meta_packed``,
``mse_scale_groups_packed``, ``gptq_solver``, ``sparsegptq14_solver``) with the same
positional signatures and return conventions, plus the batched entry points of
include/forge_hip.h.  Everything goes through the C ABI of ``csrc/libforge_hip.so``
(ctypes; device pointers and the current HIP stream), torch only provides the memory.

There is no CPU fallback: without a GPU or without the built library every attribute
access raises ``RuntimeError`` (the reference's stub does the same when CUDA is missing,
forge/backend/cuda/__init__.py:74-87).
"""
from __future__ import annotations

import ctypes
from pathlib import Path
from types import ModuleType

import torch

__all__ = ["kernels", "library_path", "load_library"]

_CSRC = Path(__file__).resolve().parents[3] / "csrc"
FORGE_F32, FORGE_BF16 = 0, 1


def library_path() -> Path:
    return _CSRC / "libforge_hip.so"


def _declare(lib: ctypes.CDLL) -> ctypes.CDLL:
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    sigs = {
        "forge_hip_abi_version": ([], i32),
        "forge_last_error": ([], ctypes.c_char_p),
        "forge_kernel_timing_enable": ([i32], i32),
        "forge_kernel_timing_collect": ([], i32),
        "forge_kernel_timing_get": ([i32, ctypes.c_char_p, i32, ctypes.POINTER(i64),
                                     ctypes.POINTER(ctypes.c_double),
                                     ctypes.POINTER(ctypes.c_double), ctypes.POINTER(i32)], i32),
        "forge_set_option": ([ctypes.c_char_p, i64], i32),
        "forge_get_option": ([ctypes.c_char_p], i64),
        "forge_build_group_meta_packed": ([vp, i64, i64, i32, i32, vp, vp, vp], i32),
        "forge_mse_scale_groups_packed": ([vp, vp, vp, vp, i64, i64, i64, f32, i32, i32, vp], i32),
        "forge_quant_grid": ([vp, i32, i64, i64, i64, i64, i64, i64, i32, i32, i32, vp, i64, f32,
                              vp, vp, vp], i32),
        "forge_gptq_solver": ([vp, vp, vp, vp, i32, i64, i64, vp, vp, vp], i32),
        "forge_sparsegptq14_solver": ([vp, vp, vp, vp, i32, i64, i64, vp, vp, vp, vp, vp], i32),
        "forge_gptq_sweep_batched": ([vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, i32,
                                      vp], i32),
        "forge_gptq_sweep_direct_batched": ([vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64,
                                             i32, i32, vp, i64, vp], i32),
        "forge_gptq_sweep_direct_batched_w0": ([vp, vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64,
                                                i64, i64, i64, i32, i32, vp, i64, vp], i32),
        "forge_gptq_sweep_direct_reads_band_only": ([i64, i64, i64], i32),
        "forge_gptq_sweep_direct_workspace_bytes": ([i64, i64, i64], i64),
        "forge_hessian_update_grouped": ([vp, i32, i64, i64, vp, i64, vp, vp, vp, vp, i64, vp], i32),
        "forge_hessian_workspace_bytes": ([i64, i64, i64, i32], i64),
        "forge_hessian_update_ranges": ([vp, i32, i64, i64, vp, vp, i64, vp, vp, vp, vp, i64, vp], i32),
        "forge_lowrank_factor": ([vp, vp, vp, vp, i64, i64, i64, vp, i64, vp], i32),
        "forge_lowrank_workspace_bytes": ([i64, i64, i64], i64),
        "forge_gptq_sweep_lowrank_mixed": ([vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32,
                                            vp], i32),
        "forge_round_to_nearest": ([vp, i32, i64, i64, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp], i32),
        "forge_hessian_permute_gather": ([vp, vp, vp, vp, vp, vp, f32, i64, i64, i32, vp], i32),
        "forge_weight_to_solver_order_gather": ([vp, i32, i64, i64, vp, vp, vp, vp, vp, i64, i64, i64, i64,
                                                 i64, vp], i32),
        "forge_codes_to_layer_order_scatter": ([vp, i64, i64, vp, vp, vp, i64, i64, i64, vp], i32),
        "forge_gptq_sweep_lowrank": ([vp, i32, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, i64,
                                      vp], i32),
        "forge_rows_factor_blocked": ([vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, vp, i64, vp], i32),
        "forge_rows_factor_workspace_bytes": ([i64, i64, i64], i64),
        "forge_gptq_sweep_rows_blocked": ([vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64,
                                           i32, i64, vp, i64, vp], i32),
        "forge_gptq_sweep_rows_workspace_bytes": ([i64, i64, i64], i64),
        "forge_hessian_update_static": ([vp, i32, i64, i64, i64, f32, f32, vp, vp], i32),
        "forge_hessian_update_static_max_rows": ([i64, i32], i64),
        "forge_chol_inv_upper_batched": ([vp, vp, vp, vp, vp, i64, i64, i32, vp, i64, vp], i32),
        "forge_chol_workspace_bytes": ([i64, i64], i64),
        "forge_chol_reverse_lower_batched": ([vp, vp, vp, i64, i64, vp, i64, vp], i32),
        "forge_unit_upper_from_lower": ([vp, vp, vp, i64, i64, i32, vp], i32),
        "forge_babai_solver": ([vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, vp, vp, i64, vp], i32),
        "forge_babai_workspace_bytes": ([i64, i64, i64], i64),
        "forge_hessian_permute": ([vp, vp, vp, vp, vp, f32, i64, i64, vp], i32),
        "forge_hessian_permute_lower": ([vp, vp, vp, vp, vp, f32, i64, i64, vp], i32),
        "forge_weight_to_solver_order": ([vp, i32, i64, i64, vp, vp, vp, i64, i64, i64, vp], i32),
        "forge_codes_to_layer_order": ([vp, vp, vp, i64, i64, i64, vp], i32),
        "forge_weight_to_solver_order_strided": ([vp, i32, i64, i64, vp, vp, vp, i64, i64, i64, i64, i64,
                                                  vp], i32),
        "forge_weight_to_solver_order_pair": ([vp, i32, i64, i64, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                               vp], i32),
        "forge_codes_to_layer_order_strided": ([vp, i64, i64, vp, vp, i64, i64, i64, vp], i32),
        "forge_pack_int4": ([vp, vp, vp, i64, i64, i64, vp], i32),
        "forge_fp8_e4m3_block_dequant": ([vp, vp, vp, i32, i64, i64, i64, i64, i64, vp], i32),
        "forge_pack_sparsegptq14_to_u64x2": ([vp, vp, vp, vp, i64, i64, vp], i32),
        "forge_dequantize_groups": ([vp, vp, vp, vp, i32, i64, i64, i64, i64, vp], i32),
        "forge_gather_scaled_rows": ([vp, i32, i64, i64, i64, vp, vp, vp, i64, vp], i32),
        "forge_rows_operands": ([vp, i32, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, vp], i32),
        "forge_rows_diagonal": ([vp, i32, vp, vp, vp, vp, i64, i64, vp], i32),
    }
    for name, (args, res) in sigs.items():
        fn = getattr(lib, name)          # AttributeError here = library/header mismatch
        fn.argtypes, fn.restype = args, res
    return lib


EXPORTED_SYMBOLS = (
    "forge_hip_abi_version", "forge_last_error", "forge_kernel_timing_enable",
    "forge_kernel_timing_collect", "forge_kernel_timing_get", "forge_set_option",
    "forge_get_option", "forge_build_group_meta_packed",
    "forge_mse_scale_groups_packed", "forge_quant_grid", "forge_gptq_solver",
    "forge_sparsegptq14_solver", "forge_gptq_sweep_batched", "forge_gptq_sweep_direct_batched",
    "forge_gptq_sweep_direct_workspace_bytes",
    "forge_hessian_update_grouped",
    "forge_hessian_workspace_bytes",
    "forge_hessian_update_static", "forge_hessian_update_static_max_rows",
    "forge_chol_inv_upper_batched", "forge_chol_workspace_bytes", "forge_hessian_permute",
    "forge_hessian_permute_lower",
    "forge_weight_to_solver_order", "forge_codes_to_layer_order", "forge_pack_int4",
    "forge_weight_to_solver_order_strided", "forge_codes_to_layer_order_strided",
    "forge_weight_to_solver_order_pair", "forge_gptq_sweep_direct_batched_w0",
    "forge_gptq_sweep_direct_reads_band_only",
    "forge_fp8_e4m3_block_dequant", "forge_pack_sparsegptq14_to_u64x2",
    "forge_dequantize_groups", "forge_gather_scaled_rows",
    "forge_chol_reverse_lower_batched", "forge_unit_upper_from_lower", "forge_babai_solver",
    "forge_babai_workspace_bytes", "forge_hessian_update_ranges", "forge_lowrank_factor",
    "forge_gptq_sweep_lowrank", "forge_round_to_nearest", "forge_lowrank_workspace_bytes",
    "forge_gptq_sweep_lowrank_mixed", "forge_hessian_permute_gather",
    "forge_weight_to_solver_order_gather", "forge_codes_to_layer_order_scatter",
    "forge_rows_factor_blocked", "forge_rows_factor_workspace_bytes",
    "forge_gptq_sweep_rows_blocked", "forge_gptq_sweep_rows_workspace_bytes",
    "forge_rows_operands", "forge_rows_diagonal",
)


def load_library() -> ctypes.CDLL:
    """dlopen the C-ABI library and declare its prototypes (no GPU needed for this)."""
    path = library_path()
    if not path.exists():
        raise RuntimeError(f"{path} is missing: run `python 4bit-forge_amd/build.py` "
                           "(hipcc --offload-arch=gfx950)")
    return _declare(ctypes.CDLL(str(path)))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return FORGE_F32
    if t.dtype == torch.bfloat16:
        return FORGE_BF16
    raise RuntimeError(f"unsupported dtype {t.dtype} (float32 or bfloat16 expected)")


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("forge HIP kernels need tensors on the GPU "
                               f"(got a tensor on {t.device}); there is no CPU fallback")


class _HipKernels:
    """The operator table.  Method names and argument order follow kernels.cpp."""

    def __init__(self, lib: ctypes.CDLL):
        self._lib = lib

    def _check(self, rc: int):
        if rc != 0:
            raise RuntimeError(self._lib.forge_last_error().decode())

    # -- per-kernel timing (benchmarks) ------------------------------------------------
    def set_option(self, name: str, value: int):
        """Library-wide setting ("sweep_schedule", "fp32_blocked_sum", "sweep_update_products",
        "factor_pieces";
        see forge_set_option in forge_hip.h).  Returns the previous value."""
        old = int(self._lib.forge_get_option(name.encode()))
        self._check(self._lib.forge_set_option(name.encode(), int(value)))
        return old

    def get_option(self, name: str) -> int:
        return int(self._lib.forge_get_option(name.encode()))

    def timing_enable(self, on: bool):
        self._check(self._lib.forge_kernel_timing_enable(int(bool(on))))

    def timing_collect(self):
        """-> {kernel name: dict(launches, ms, work, unit)} for the launches since enable."""
        n = self._lib.forge_kernel_timing_collect()
        if n < 0:
            raise RuntimeError(self._lib.forge_last_error().decode())
        out = {}
        for i in range(n):
            name = ctypes.create_string_buffer(64)
            launches, ms, work, kind = (ctypes.c_int64(), ctypes.c_double(), ctypes.c_double(),
                                        ctypes.c_int())
            self._check(self._lib.forge_kernel_timing_get(i, name, 64, ctypes.byref(launches),
                                                          ctypes.byref(ms), ctypes.byref(work),
                                                          ctypes.byref(kind)))
            out[name.value.decode()] = dict(launches=launches.value, ms=ms.value, work=work.value,
                                            unit="flop" if kind.value == 0 else "byte")
        return out

    def build_group_meta_packed(self, X, bit_width, symmetric):
        _need_cuda(X)
        if X.dtype != torch.float32 or not X.is_contiguous() or X.dim() != 2:
            raise RuntimeError("build_group_meta_packed: X must be a contiguous f32 [RG, gs] tensor")
        RG, gs = X.shape
        scales = torch.empty(RG, dtype=torch.float32, device=X.device)
        qzeros = torch.empty(RG, dtype=torch.float32, device=X.device)
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_build_group_meta_packed(
                _ptr(X), RG, gs, int(bit_width), int(bool(symmetric)), _ptr(scales), _ptr(qzeros),
                _stream()))
        return scales, qzeros

    def mse_scale_groups_packed(self, X, scales, qzeros, candidates, norm, bit_width, symmetric):
        _need_cuda(X, scales, qzeros, candidates)
        for t in (X, scales, qzeros, candidates):
            if t.dtype != torch.float32 or not t.is_contiguous():
                raise RuntimeError("mse_scale_groups_packed: contiguous f32 tensors expected")
        RG, gs = X.shape
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_mse_scale_groups_packed(
                _ptr(X), _ptr(scales), _ptr(qzeros), _ptr(candidates), RG, gs,
                candidates.numel(), float(norm), int(bit_width), int(bool(symmetric)), _stream()))
        return scales, qzeros

    def gptq_solver(self, W, U, scales, qzeros, bits):
        _need_cuda(W, U, scales, qzeros)
        W = W.contiguous()          # as solver.cu:107: a non-contiguous W is solved on a copy
        U, scales, qzeros = U.contiguous(), scales.contiguous(), qzeros.contiguous()
        for t in (W, U, scales, qzeros):
            if t.dtype != torch.float32:
                raise RuntimeError("gptq_solver: f32 tensors expected")
        C, R = W.shape
        if tuple(U.shape) != (C, C) or tuple(scales.shape) != (C, R) or tuple(qzeros.shape) != (C, R):
            raise RuntimeError("gptq_solver: shape mismatch (W [C,R], U [C,C], scales/qzeros [C,R])")
        q = torch.empty((C, R), dtype=torch.uint8, device=W.device)
        E = torch.empty((C, R), dtype=torch.float32, device=W.device)
        with torch.cuda.device(W.device):
            self._check(self._lib.forge_gptq_solver(_ptr(W), _ptr(U), _ptr(scales), _ptr(qzeros),
                                                    int(bits), C, R, _ptr(q), _ptr(E), _stream()))
        return q

    def sparsegptq14_solver(self, W, U, scales, qzeros, bits):
        _need_cuda(W, U, scales, qzeros)
        W = W.contiguous()
        Uc = U.contiguous()
        scales, qzeros = scales.contiguous(), qzeros.contiguous()
        for t in (W, Uc, scales, qzeros):
            if t.dtype != torch.float32:
                raise RuntimeError("sparsegptq14_solver: f32 tensors expected")
        C, R = W.shape
        if tuple(Uc.shape) != (C, C) or tuple(scales.shape) != (C, R) or tuple(qzeros.shape) != (C, R):
            raise RuntimeError("sparsegptq14_solver: shape mismatch")
        q = torch.empty((C, R), dtype=torch.uint8, device=W.device)
        M = torch.empty(((C + 31) // 32, R), dtype=torch.uint32, device=W.device)
        E = torch.empty((C, R), dtype=torch.float32, device=W.device)
        uinv = torch.empty(C, dtype=torch.float32, device=W.device)
        with torch.cuda.device(W.device):
            self._check(self._lib.forge_sparsegptq14_solver(
                _ptr(W), _ptr(Uc), _ptr(scales), _ptr(qzeros), int(bits), C, R, _ptr(q), _ptr(M),
                _ptr(E), _ptr(uinv), _stream()))
        if Uc.data_ptr() != U.data_ptr():
            U.copy_(Uc)             # the reference row-normalises the caller's U in place
        return q, M

    # -- batched / fused entry points (no reference counterpart) -------------------------
    def quant_grid(self, W, gs, bits, symmetric, mse, candidates=None, norm=2.4):
        """W [R,C] or [B,R,C] (f32/bf16, last dim contiguous) -> scales, qzeros [B?, R*G]."""
        _need_cuda(W, candidates)
        squeeze = W.dim() == 2
        W3 = W.unsqueeze(0) if squeeze else W
        if W3.stride(2) != 1:
            W3 = W3.contiguous()
        B, R, C = W3.shape
        G = (C + gs - 1) // gs
        scales = torch.empty((B, R * G), dtype=torch.float32, device=W.device)
        qzeros = torch.empty_like(scales)
        P = 0 if candidates is None else candidates.numel()
        with torch.cuda.device(W.device):
            self._check(self._lib.forge_quant_grid(
                _ptr(W3), _dtype_code(W3), B, W3.stride(0), R, C, W3.stride(1), gs, int(bits),
                int(bool(symmetric)), int(bool(mse)), _ptr(candidates), P, float(norm),
                _ptr(scales), _ptr(qzeros), _stream()))
        return (scales[0], qzeros[0]) if squeeze else (scales, qzeros)

    def gptq_sweep_batched(self, X, U, scalesT, qzerosT, g_idx, bits, sparse14=False, uinv=None):
        """X [B,C,R] f32 in/out (errors on exit); returns qweight [B,C,R] u8 (and M)."""
        _need_cuda(X, U, scalesT, qzerosT, g_idx)
        B, C, R = X.shape
        G = scalesT.shape[1]
        assert X.is_contiguous() and U.is_contiguous() and scalesT.is_contiguous()
        assert qzerosT.is_contiguous() and g_idx.is_contiguous() and g_idx.dtype == torch.int32
        assert tuple(U.shape) == (B, C, C) and tuple(scalesT.shape) == (B, G, R)
        assert tuple(qzerosT.shape) == (B, G, R) and tuple(g_idx.shape) == (B, C)
        q = torch.empty((B, C, R), dtype=torch.uint8, device=X.device)
        M = None
        if sparse14:
            M = torch.empty((B, (C + 31) // 32, R), dtype=torch.uint32, device=X.device)
            assert uinv is not None and tuple(uinv.shape) == (B, C) and uinv.is_contiguous()
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_gptq_sweep_batched(
                _ptr(X), _ptr(U), _ptr(scalesT), _ptr(qzerosT), _ptr(g_idx), _ptr(q), _ptr(M),
                _ptr(uinv), B, C, R, G, int(bits), int(bool(sparse14)), _stream()))
        return (q, M) if sparse14 else q

    def sweep_direct_reads_band_only(self, B, C, R) -> bool:
        """True when gptq_sweep_direct_batched(..., L=...) reads V only within one 128-column
        block of its diagonal for this shape (unit_upper_from_lower(band=True) then suffices)."""
        return bool(self._lib.forge_gptq_sweep_direct_reads_band_only(int(B), int(C), int(R)))

    def gptq_sweep_direct_batched(self, X, V, scalesT, qzerosT, g_idx, bits, W0=None,
                                  exact_chain=False, sparse14=False, mdiag=None, L=None, info=None,
                                  x_from_w0=False):
        """The sweep fed by the factor of H itself: V [B,C,C] = -M[t,k]/M[k,k] above the
        diagonal (``unit_upper_from_lower(L, info, negate=True)``).  X [B,C,R] f32 in/out
        (displacements w0 - deq on exit); W0: untouched copy of X (made here when None).
        exact_chain: keep the block updates as one fp32 fma chain per element (reproducible
        on a CPU) instead of blocked sums on the bf16 matrix pipe.  sparse14: the 1:4 joint
        solve, with mdiag [B,C] = diag(L) (1 where the factorisation failed).  L [B,C,C], info
        [B] int32: the lower factor V was made from and its failure flags; the long block
        updates then take their V operand from L's rows (same numbers).  x_from_w0: X is
        uninitialised on entry (shapes with sweep_direct_reads_band_only only).
        Returns qweight [B,C,R] u8 (and M [B, ceil(C/32), R] u32)."""
        _need_cuda(X, V, scalesT, qzerosT, g_idx, W0, L, info)
        B, C, R = X.shape
        assert L is None or (L.is_contiguous() and L.dtype == torch.float32 and L.shape == V.shape)
        assert info is None or (info.dtype == torch.int32 and info.is_contiguous() and info.numel() == B)
        if exact_chain:
            L = None
        G = scalesT.shape[1]
        assert X.is_contiguous() and V.is_contiguous() and scalesT.is_contiguous()
        assert qzerosT.is_contiguous() and g_idx.is_contiguous() and g_idx.dtype == torch.int32
        assert tuple(V.shape) == (B, C, C) and tuple(scalesT.shape) == (B, G, R)
        assert tuple(qzerosT.shape) == (B, G, R) and tuple(g_idx.shape) == (B, C)
        if W0 is None:
            W0 = X.clone()
        assert W0.is_contiguous() and W0.shape == X.shape and W0.dtype in (torch.float32, torch.bfloat16)
        assert W0.data_ptr() != X.data_ptr() or X.numel() == 0
        q = torch.empty((B, C, R), dtype=torch.uint8, device=X.device)
        M = None
        if sparse14:
            M = torch.empty((B, (C + 31) // 32, R), dtype=torch.uint32, device=X.device)
            assert mdiag is not None and tuple(mdiag.shape) == (B, C) and mdiag.is_contiguous()
            assert mdiag.dtype == torch.float32
        nbytes = 0 if exact_chain else int(self._lib.forge_gptq_sweep_direct_workspace_bytes(B, C, R))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device) if nbytes else None
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_gptq_sweep_direct_batched_w0(
                _ptr(X), _ptr(W0), _dtype_code(W0), int(bool(x_from_w0)), _ptr(V), _ptr(L),
                _ptr(info if L is not None else None),
                _ptr(scalesT), _ptr(qzerosT), _ptr(g_idx), _ptr(q),
                _ptr(M), _ptr(mdiag), B, C, R, G, int(bits), int(bool(sparse14)), _ptr(ws), nbytes,
                _stream()))
        return (q, M) if sparse14 else q

    def hessian_update_grouped(self, X, offsets, H, alpha, beta):
        """X [T,C] (bf16/f32) rows grouped by expert; offsets: host int64 [E+1];
        H [E,C,C] f32; alpha/beta: host float sequences [E]."""
        _need_cuda(X, H)
        E = H.shape[0]
        C = H.shape[-1]
        offs = (ctypes.c_int64 * (E + 1))(*[int(o) for o in offsets])
        al = (ctypes.c_float * E)(*[float(a) for a in alpha])
        be = (ctypes.c_float * E)(*[float(b) for b in beta])
        assert X.stride(1) == 1 and H.is_contiguous() and H.dtype == torch.float32
        total = int(offsets[-1]) - int(offsets[0])
        nbytes = int(self._lib.forge_hessian_workspace_bytes(total, E, C, _dtype_code(X)))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=X.device)
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_hessian_update_grouped(
                _ptr(X), _dtype_code(X), X.stride(0), C, offs, E, al, be, _ptr(H), _ptr(ws),
                nbytes, _stream()))
        return H

    def hessian_update_ranges(self, X, row0, counts, H, alpha, beta):
        """hessian_update_grouped with every group's rows given as (row0[e], counts[e]): groups
        with counts[e] == 0 leave H[e] untouched wherever their rows lie in X."""
        _need_cuda(X, H)
        E = H.shape[0]
        C = H.shape[-1]
        assert len(row0) == E and len(counts) == E
        assert all(int(c) >= 0 and int(o) >= 0 and (int(c) == 0 or int(o) + int(c) <= X.shape[0])
                   for o, c in zip(row0, counts)), "row range outside X"
        r0 = (ctypes.c_int64 * E)(*[int(o) for o in row0])
        cn = (ctypes.c_int64 * E)(*[int(o) for o in counts])
        al = (ctypes.c_float * E)(*[float(a) for a in alpha])
        be = (ctypes.c_float * E)(*[float(b) for b in beta])
        assert X.stride(1) == 1 and H.is_contiguous() and H.dtype == torch.float32
        total = sum(int(c) for c in counts)
        nbytes = int(self._lib.forge_hessian_workspace_bytes(total, E, C, _dtype_code(X)))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=X.device)
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_hessian_update_ranges(
                _ptr(X), _dtype_code(X), X.stride(0), C, r0, cn, E, al, be, _ptr(H), _ptr(ws), nbytes,
                _stream()))
        return H

    def round_to_nearest(self, W, scales, qzeros, gs, bits, out=None, index=None):
        """W [B,R,C] (bf16/f32, layer layout), scales/qzeros [B,R*G] -> codes [B,R,C] u8 of the
        reference's quantiser applied weight by weight (a layer with H = I).  index (int64,
        device): only these matrices of the stacks are worked on (``out`` required then)."""
        _need_cuda(W, scales, qzeros, out, index)
        B, R, C = W.shape
        G = (C + gs - 1) // gs
        assert W.stride(2) == 1 and scales.is_contiguous() and qzeros.is_contiguous()
        assert tuple(scales.shape) == (B, R * G) and tuple(qzeros.shape) == (B, R * G)
        assert scales.dtype == torch.float32 and qzeros.dtype == torch.float32
        if out is None:
            assert index is None
            out = torch.empty((B, R, C), dtype=torch.uint8, device=W.device)
        assert out.is_contiguous() and out.dtype == torch.uint8 and tuple(out.shape) == (B, R, C)
        n = B
        if index is not None:
            assert index.dtype == torch.int64 and index.is_contiguous() and index.dim() == 1
            n = index.numel()
        with torch.cuda.device(W.device):
            self._check(self._lib.forge_round_to_nearest(
                _ptr(W), _dtype_code(W), W.stride(0), W.stride(1), _ptr(index), _ptr(scales), _ptr(qzeros),
                _ptr(out), n, R, C, int(gs), int(bits), _stream()))
        return out

    def lowrank_factor(self, Bp, D, out=None):
        """Bp [B,C,n] f32 (n = 4, 16, 32, 64 or 128), D [B,C] f32 -> (Hm [B,C,n] f32, info [B] i32): the
        factor of D + Bp^T Bp as the n-vectors the low-rank sweep reads (see forge_hip.h)."""
        _need_cuda(Bp, D)
        B, C, n = Bp.shape
        assert Bp.is_contiguous() and Bp.dtype == torch.float32 and n in (4, 16, 32, 64, 128)
        assert D.is_contiguous() and D.dtype == torch.float32 and tuple(D.shape) == (B, C)
        if out is not None:
            Hm, info = out
            _need_cuda(Hm, info)
            assert Hm.is_contiguous() and Hm.dtype == torch.float32 and Hm.shape == Bp.shape
            assert info.is_contiguous() and info.dtype == torch.int32 and info.numel() == B
        else:
            Hm = torch.empty_like(Bp)
            info = torch.empty(B, dtype=torch.int32, device=Bp.device)
        nbytes = int(self._lib.forge_lowrank_workspace_bytes(B, C, n))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=Bp.device)
        with torch.cuda.device(Bp.device):
            self._check(self._lib.forge_lowrank_factor(_ptr(Bp), _ptr(D), _ptr(Hm), _ptr(info), B, C, n,
                                                       _ptr(ws), nbytes, _stream()))
        return Hm, info

    def gptq_sweep_lowrank_mixed(self, W0, Bp, Hm, ns, info, scalesT, qzerosT, g_idx, bits):
        """gptq_sweep_lowrank for matrices of different n in one launch: ns[b] in (4, 16, 32, 64, 128);
        Bp/Hm flat f32 buffers holding matrix b's [C, ns[b]] vectors one after the other."""
        _need_cuda(W0, Bp, Hm, info, scalesT, qzerosT, g_idx)
        B, C, R = W0.shape
        G = scalesT.shape[1]
        assert len(ns) == B and all(int(n) in (4, 16, 32, 64, 128) for n in ns)
        total = C * sum(int(n) for n in ns)
        assert W0.is_contiguous() and Bp.is_contiguous() and Hm.is_contiguous()
        assert Bp.numel() == total and Hm.numel() == total and Bp.dtype == Hm.dtype == torch.float32
        assert scalesT.is_contiguous() and qzerosT.is_contiguous() and tuple(scalesT.shape) == (B, G, R)
        assert tuple(qzerosT.shape) == (B, G, R) and scalesT.dtype == torch.float32
        assert g_idx.dtype == torch.int32 and g_idx.is_contiguous() and tuple(g_idx.shape) == (B, C)
        assert info.dtype == torch.int32 and info.is_contiguous() and info.numel() == B
        q = torch.empty((B, C, R), dtype=torch.uint8, device=W0.device)
        nh = (ctypes.c_int64 * max(B, 1))(*[int(n) for n in ns])
        with torch.cuda.device(W0.device):
            self._check(self._lib.forge_gptq_sweep_lowrank_mixed(
                _ptr(W0), _dtype_code(W0), _ptr(Bp), _ptr(Hm), nh, _ptr(info), _ptr(scalesT),
                _ptr(qzerosT), _ptr(g_idx), _ptr(q), B, C, R, G, int(bits), _stream()))
        return q

    def gptq_sweep_lowrank(self, W0, Bp, Hm, info, scalesT, qzerosT, g_idx, bits):
        """W0 [B,C,R] (f32/bf16, solver order), Bp/Hm [B,C,n] (n = 4, 16, 32, 64 or 128), scalesT/qzerosT
        [B,G,R], g_idx [B,C] i32 -> codes [B,C,R] u8."""
        _need_cuda(W0, Bp, Hm, info, scalesT, qzerosT, g_idx)
        B, C, R = W0.shape
        G = scalesT.shape[1]
        n = Bp.shape[2]
        assert W0.is_contiguous() and Bp.is_contiguous() and Hm.is_contiguous()
        assert n in (4, 16, 32, 64, 128) and tuple(Bp.shape) == (B, C, n) and tuple(Hm.shape) == (B, C, n)
        assert scalesT.is_contiguous() and qzerosT.is_contiguous() and tuple(scalesT.shape) == (B, G, R)
        assert tuple(qzerosT.shape) == (B, G, R) and scalesT.dtype == torch.float32
        assert g_idx.dtype == torch.int32 and g_idx.is_contiguous() and tuple(g_idx.shape) == (B, C)
        assert info.dtype == torch.int32 and info.numel() == B
        q = torch.empty((B, C, R), dtype=torch.uint8, device=W0.device)
        with torch.cuda.device(W0.device):
            self._check(self._lib.forge_gptq_sweep_lowrank(
                _ptr(W0), _dtype_code(W0), _ptr(Bp), _ptr(Hm), _ptr(info), _ptr(scalesT), _ptr(qzerosT),
                _ptr(g_idx), _ptr(q), B, C, R, G, int(bits), n, _stream()))
        return q

    def workspace_bytes(self, what: str, *dims) -> int:
        """The size queries of forge_hip.h: what = "chol" (batch, C), "sweep_direct" (batch, C, R),
        "lowrank" (batch, C, n), "rows_factor" (batch, C, nmax), "sweep_rows" (batch, R, nmax)."""
        fn = {"chol": self._lib.forge_chol_workspace_bytes,
              "sweep_direct": self._lib.forge_gptq_sweep_direct_workspace_bytes,
              "lowrank": self._lib.forge_lowrank_workspace_bytes,
              "rows_factor": self._lib.forge_rows_factor_workspace_bytes,
              "sweep_rows": self._lib.forge_gptq_sweep_rows_workspace_bytes}[what]
        return int(fn(*[int(d) for d in dims]))

    def rows_factor_blocked(self, BT, D, n_rows, n_rows_host=None):
        """BT [B,nmax,C] f32 (row j = sqrt(2/n) x_j in solver order, zero rows beyond a matrix's own),
        D [B,C] f32, n_rows [B] int32 on the device (each a multiple of 128, <= nmax) ->
        (HmT [B,nmax,C], V [B,C,128], info [B] i32): the factor of D + BT^T BT as the blocked
        sweep reads it (see forge_rows_factor_blocked in forge_hip.h).  n_rows_host: the same
        numbers as a host list (only the timing records' work figures use them)."""
        _need_cuda(BT, D, n_rows)
        B, nmax, C = BT.shape
        assert BT.is_contiguous() and BT.dtype == torch.float32 and nmax % 128 == 0 and C % 128 == 0
        assert D.is_contiguous() and D.dtype == torch.float32 and tuple(D.shape) == (B, C)
        assert n_rows.is_contiguous() and n_rows.dtype == torch.int32 and n_rows.numel() == B
        HmT = torch.empty_like(BT)
        V = torch.empty((B, C, 128), dtype=torch.float32, device=BT.device)
        info = torch.empty(B, dtype=torch.int32, device=BT.device)
        nbytes = int(self._lib.forge_rows_factor_workspace_bytes(B, C, nmax))
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=BT.device)
        with torch.cuda.device(BT.device):
            nh = (ctypes.c_int32 * B)(*[int(n) for n in n_rows_host]) if n_rows_host is not None else None
            self._check(self._lib.forge_rows_factor_blocked(_ptr(BT), _ptr(D), _ptr(n_rows), nh, _ptr(HmT),
                                                            _ptr(V), _ptr(info), B, C, nmax, _ptr(ws),
                                                            nbytes, _stream()))
        return HmT, V, info

    def rows_operands(self, rows, row0, n, root, perm, dead, nmax, want_bt=True, out=None):
        """rows [*, C] bf16/f32 (matrix b owns rows row0[b] .. row0[b]+n[b]-1; row0 [B] i64, n [B]
        i32, root [B] f64 = sqrt(2/n), all on the device), perm [B,C] i64, dead [B,C] u8 or bool
        in solver order -> (BT [B,nmax,C] or None, Bp [B,C,nmax]) f32: sqrt(2/n) X in solver
        order with pruned columns zero, row-major and column-major.  out: Bp's storage."""
        _need_cuda(rows, row0, n, root, perm, dead)
        B, C = perm.shape
        assert rows.dim() == 2 and rows.shape[1] == C and rows.is_contiguous()
        assert row0.dtype == torch.int64 and n.dtype == torch.int32 and root.dtype == torch.float64
        assert row0.numel() == B and n.numel() == B and root.numel() == B
        assert perm.dtype == torch.int64 and perm.is_contiguous()
        if dead.dtype == torch.bool:
            dead = dead.view(torch.uint8)
        assert dead.dtype == torch.uint8 and dead.is_contiguous() and tuple(dead.shape) == (B, C)
        BT = torch.empty((B, nmax, C), dtype=torch.float32, device=rows.device) if want_bt else None
        Bp = out if out is not None else torch.empty((B, C, nmax), dtype=torch.float32, device=rows.device)
        assert Bp.is_contiguous() and Bp.dtype == torch.float32 and tuple(Bp.shape) == (B, C, nmax)
        with torch.cuda.device(rows.device):
            self._check(self._lib.forge_rows_operands(
                _ptr(rows), _dtype_code(rows), _ptr(row0), _ptr(n), _ptr(root), _ptr(perm), _ptr(dead),
                _ptr(BT), _ptr(Bp), B, C, int(nmax), _stream()))
        return BT, Bp

    def rows_diagonal(self, rows, row0, n, alpha):
        """diag((2/n) X^T X) per matrix, summed in float64 and rounded once: rows [*, C] bf16/f32,
        row0 [B] i64, n [B] i32, alpha [B] f64 (device) -> [B, C] f32."""
        _need_cuda(rows, row0, n, alpha)
        C = rows.shape[1]
        B = row0.numel()
        assert rows.dim() == 2 and rows.is_contiguous()
        assert row0.dtype == torch.int64 and n.dtype == torch.int32 and alpha.dtype == torch.float64
        assert n.numel() == B and alpha.numel() == B
        out = torch.empty((B, C), dtype=torch.float32, device=rows.device)
        with torch.cuda.device(rows.device):
            self._check(self._lib.forge_rows_diagonal(_ptr(rows), _dtype_code(rows), _ptr(row0), _ptr(n),
                                                      _ptr(alpha), _ptr(out), B, C, _stream()))
        return out

    def gptq_sweep_rows_blocked(self, X, W0, HmT, Bp, V, n_rows, scalesT, qzerosT, g_idx, bits,
                                n_rows_host=None):
        """X [B,C,R] f32 (weights in solver order; displacements on return), W0 the same untouched
        (f32/bf16), HmT [B,nmax,C], Bp [B,C,nmax], V [B,C,128], n_rows [B] i32 (device),
        scalesT/qzerosT [B,G,R], g_idx [B,C] i32 -> codes [B,C,R] u8."""
        _need_cuda(X, W0, HmT, Bp, V, n_rows, scalesT, qzerosT, g_idx)
        B, C, R = X.shape
        nmax = HmT.shape[1]
        G = scalesT.shape[1]
        assert X.is_contiguous() and X.dtype == torch.float32 and W0.is_contiguous() and W0.shape == X.shape
        assert HmT.is_contiguous() and tuple(HmT.shape) == (B, nmax, C) and HmT.dtype == torch.float32
        assert Bp.is_contiguous() and tuple(Bp.shape) == (B, C, nmax) and Bp.dtype == torch.float32
        assert V.is_contiguous() and tuple(V.shape) == (B, C, 128) and V.dtype == torch.float32
        assert n_rows.is_contiguous() and n_rows.dtype == torch.int32 and n_rows.numel() == B
        assert scalesT.is_contiguous() and qzerosT.is_contiguous() and tuple(scalesT.shape) == (B, G, R)
        assert tuple(qzerosT.shape) == (B, G, R) and scalesT.dtype == torch.float32
        assert g_idx.dtype == torch.int32 and g_idx.is_contiguous() and tuple(g_idx.shape) == (B, C)
        q = torch.empty((B, C, R), dtype=torch.uint8, device=X.device)
        nbytes = int(self._lib.forge_gptq_sweep_rows_workspace_bytes(B, R, nmax))
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=X.device)
        with torch.cuda.device(X.device):
            nh = (ctypes.c_int32 * B)(*[int(n) for n in n_rows_host]) if n_rows_host is not None else None
            self._check(self._lib.forge_gptq_sweep_rows_blocked(
                _ptr(X), _ptr(W0), _dtype_code(W0), _ptr(HmT), _ptr(Bp), _ptr(V), _ptr(n_rows), nh,
                _ptr(scalesT), _ptr(qzerosT), _ptr(g_idx), _ptr(q), B, C, R, G, int(bits), nmax,
                _ptr(ws), nbytes, _stream()))
        return q

    def hessian_update_static(self, X, H, alpha, beta):
        """H [C,C] f32 <- beta*H + alpha * X^T X for X [n,C] (bf16/f32) through the entry point
        that allocates nothing (its workspace is a device array of the library's own; see
        forge_hessian_update_static in forge_hip.h for the size limits)."""
        _need_cuda(X, H)
        C = H.shape[-1]
        assert X.dim() == 2 and X.shape[1] == C and X.stride(1) == 1
        assert tuple(H.shape) == (C, C) and H.is_contiguous() and H.dtype == torch.float32
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_hessian_update_static(
                _ptr(X), _dtype_code(X), X.stride(0), X.shape[0], C, float(alpha), float(beta),
                _ptr(H), _stream()))
        return H

    def chol_inv_upper_batched(self, H, damp, normalise=True, upper_only=False):
        """H [B,C,C] f32 (destroyed); damp [B] f32 or None -> U [B,C,C], udiag [B,C], info [B].
        upper_only: U is only valid on and above the diagonal blocks (what the sweeps read)."""
        _need_cuda(H, damp)
        B, C, _ = H.shape
        assert H.is_contiguous() and H.dtype == torch.float32
        assert damp is None or (damp.dtype == torch.float32 and damp.numel() == B)
        U = torch.empty_like(H)
        udiag = torch.empty((B, C), dtype=torch.float32, device=H.device)
        info = torch.empty(B, dtype=torch.int32, device=H.device)
        nbytes = int(self._lib.forge_chol_workspace_bytes(B, C))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=H.device)
        with torch.cuda.device(H.device):
            self._check(self._lib.forge_chol_inv_upper_batched(
                _ptr(H), _ptr(damp), _ptr(U), _ptr(udiag), _ptr(info), B, C,
                int(bool(normalise)) | (2 if upper_only else 0), _ptr(ws), nbytes, _stream()))
        return U, udiag, info

    def chol_reverse_lower_batched(self, H, damp):
        """H [B,C,C] f32: H + damp I = L^T L with L lower, left in H's lower triangle (the
        strict upper triangle is destroyed).  Returns (H, info [B])."""
        _need_cuda(H, damp)
        B, C, _ = H.shape
        assert H.is_contiguous() and H.dtype == torch.float32
        assert damp is None or (damp.dtype == torch.float32 and damp.numel() == B)
        info = torch.empty(B, dtype=torch.int32, device=H.device)
        nbytes = int(self._lib.forge_chol_workspace_bytes(B, C))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=H.device)
        with torch.cuda.device(H.device):
            self._check(self._lib.forge_chol_reverse_lower_batched(
                _ptr(H), _ptr(damp), _ptr(info), B, C, _ptr(ws), nbytes, _stream()))
        return H, info

    def unit_upper_from_lower(self, L, info=None, flipped_upper=False, negate=False,
                              upper_only=False, band=False):
        """U [B,C,C]: U[t,k] = L[k,t] / L[k,k] (k > t), unit diagonal, zero below; identity
        where info != 0.  flipped_upper: L is the upper factor A with both orders reversed.
        negate: entries above the diagonal with the opposite sign.  upper_only: 32x32 tiles
        wholly below the diagonal are left unwritten (uninitialised memory).  band: only the
        columns of each row's own 128-column block and of the next one are written."""
        _need_cuda(L, info)
        B, C, _ = L.shape
        assert L.is_contiguous() and L.dtype == torch.float32
        U = torch.empty_like(L)
        with torch.cuda.device(L.device):
            self._check(self._lib.forge_unit_upper_from_lower(
                _ptr(L), _ptr(info), _ptr(U), B, C,
                int(bool(flipped_upper)) | (2 if negate else 0) | (4 if upper_only else 0) | (8 if band else 0),
                _stream()))
        return U

    def babai_solver(self, W, A, scales, qzeros, group_size, bits, block_size, g_idx, G):
        """Reference operator (kernels.cpp:46-56): W [C,R] f32, A [C,C] upper factor,
        scales/qzeros [R*G], g_idx [C] int32 -> qweight [C,R] u8.  block_size is accepted for
        signature compatibility; the result does not depend on it."""
        _need_cuda(W, A, scales, qzeros, g_idx)
        C, R = W.shape
        W = W.to(torch.float32).contiguous()
        A = A.to(torch.float32).contiguous()
        scales, qzeros = scales.contiguous(), qzeros.contiguous()
        g_idx = None if g_idx is None else g_idx.to(torch.int32).contiguous()
        gs = min(int(group_size), C)
        if gs <= 0 or gs % 32 != 0:
            raise RuntimeError("group_size must be a positive multiple of 32 (effective group_size)")
        if (C + gs - 1) // gs != int(G):
            raise RuntimeError(f"qmeta G mismatch: got G={G} expected ceil(C/group_size)={(C + gs - 1) // gs}")
        q = torch.empty((C, R), dtype=torch.uint8, device=W.device)
        nbytes = int(self._lib.forge_babai_workspace_bytes(C, R, int(G)))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=W.device)
        with torch.cuda.device(W.device):
            self._check(self._lib.forge_babai_solver(
                _ptr(W), _ptr(A), _ptr(scales), _ptr(qzeros), _ptr(g_idx), gs, int(bits), C, R,
                int(G), _ptr(q), _ptr(ws), nbytes, _stream()))
        return q

    def hessian_permute(self, H, perm, dead, rel_damp, lower_blocks=False, out=None, index=None):
        """Hp[b] = H[b][perm][:, perm] with dead rows/columns cleared (unit diagonal), damp[b] =
        rel_damp * mean(diag).  lower_blocks: in row i only the columns up to the end of its own
        128-column block are written (what the factorisations read).  out = (Hp, damp): write
        into these instead of new tensors.  index (int64 [n], device): output b is made from
        matrix index[b] of H and rows index[b] of perm and dead."""
        _need_cuda(H, perm, dead, index)
        B, C, _ = H.shape
        assert H.is_contiguous() and perm.dtype == torch.int64 and perm.is_contiguous()
        assert dead.dtype == torch.uint8 and dead.is_contiguous()
        assert tuple(perm.shape) == (B, C) and tuple(dead.shape) == (B, C)
        n = B
        if index is not None:
            assert index.dtype == torch.int64 and index.is_contiguous() and index.dim() == 1
            n = index.numel()
        if out is not None:
            Hp, damp = out
            _need_cuda(Hp, damp)
            assert Hp.is_contiguous() and Hp.dtype == torch.float32 and tuple(Hp.shape) == (n, C, C)
            assert damp.is_contiguous() and damp.dtype == torch.float32 and damp.numel() == n
        else:
            Hp = torch.empty((n, C, C), dtype=torch.float32, device=H.device)
            damp = torch.empty(n, dtype=torch.float32, device=H.device)
        with torch.cuda.device(H.device):
            if index is not None:
                self._check(self._lib.forge_hessian_permute_gather(
                    _ptr(H), _ptr(index), _ptr(perm), _ptr(dead), _ptr(Hp), _ptr(damp), float(rel_damp), n,
                    C, int(bool(lower_blocks)), _stream()))
            else:
                fn = self._lib.forge_hessian_permute_lower if lower_blocks else self._lib.forge_hessian_permute
                self._check(fn(_ptr(H), _ptr(perm), _ptr(dead), _ptr(Hp), _ptr(damp), float(rel_damp), B, C,
                               _stream()))
        return Hp, damp

    def weight_to_solver_order(self, W, perm_inv, dead=None, out=None, row0=0, out0=None, skip_out=False,
                               index=None):
        """W [B,R,C] (bf16/f32) -> X [B,C,R] f32, X[b, perm_inv[b,c], r] = W[b, r, c].
        With ``out`` [B,C,Rtot] (f32, contiguous) the rows land at out[:, :, row0:row0+R]: stacks
        that share a factor fill one tall matrix without being concatenated first.  ``out0``
        (shape of ``out``, dtype of W) receives the same values in W's own type: the untouched
        copy for gptq_sweep_direct_batched(W0=...).  skip_out: only ``out0`` is written
        (``out`` then only gives the shape; for gptq_sweep_direct_batched(x_from_w0=True)).
        index (int64 [n], device): output b is made from W[index[b]], perm_inv[index[b]] and
        dead[index[b]]; ``out`` / ``out0`` are then [n,C,Rtot]."""
        _need_cuda(W, perm_inv, dead, out, index)
        B, R, C = W.shape
        assert W.stride(2) == 1 and perm_inv.dtype == torch.int64 and perm_inv.is_contiguous()
        assert tuple(perm_inv.shape) == (B, C)
        assert dead is None or (dead.dtype == torch.uint8 and dead.is_contiguous())
        n = B
        if index is not None:
            assert index.dtype == torch.int64 and index.is_contiguous() and index.dim() == 1
            n = index.numel()
        if out is None and skip_out and out0 is not None:
            shape = tuple(out0.shape)                 # only out0 is written: it also gives the shape
        else:
            if out is None:
                out = torch.empty((n, C, R), dtype=torch.float32, device=W.device)
                row0 = 0
            assert out.is_contiguous() and out.dtype == torch.float32
            shape = tuple(out.shape)
        assert len(shape) == 3
        Rtot = shape[2]
        assert shape[:2] == (n, C) and 0 <= row0 and row0 + R <= Rtot
        p0 = None
        if out0 is not None:
            _need_cuda(out0)
            assert out0.is_contiguous() and out0.dtype == W.dtype and tuple(out0.shape) == shape
            p0 = ctypes.c_void_p(out0.data_ptr() + out0.element_size() * row0)
        px = None if skip_out else ctypes.c_void_p(out.data_ptr() + 4 * row0)
        with torch.cuda.device(W.device):
            if index is not None:
                self._check(self._lib.forge_weight_to_solver_order_gather(
                    _ptr(W), _dtype_code(W), W.stride(0), W.stride(1), _ptr(index), _ptr(perm_inv),
                    _ptr(dead), px, p0, Rtot, C * Rtot, n, R, C, _stream()))
            else:
                self._check(self._lib.forge_weight_to_solver_order_pair(
                    _ptr(W), _dtype_code(W), W.stride(0), W.stride(1), _ptr(perm_inv), _ptr(dead),
                    px, p0, Rtot, C * Rtot, B, R, C, _stream()))
        return out

    def codes_to_layer_order(self, q, perm_inv, out=None, row0=0, rows=None, index=None):
        """q [B,C,R] u8 (solver order) -> [B,R,C] u8, out[b, r, c] = q[b, perm_inv[b,c], r].
        ``row0``/``rows`` select a band of q's rows (a stack of a tall shared-factor matrix);
        ``out`` [B,rows,C] (contiguous) receives it.  index (int64 [B], device): q[b] goes to
        out[index[b]] through perm_inv[index[b]] (``out`` and ``perm_inv`` are then the larger
        stack's)."""
        _need_cuda(q, perm_inv, out, index)
        B, C, Rtot = q.shape
        R = Rtot - row0 if rows is None else int(rows)
        assert q.is_contiguous() and q.dtype == torch.uint8 and perm_inv.is_contiguous()
        assert perm_inv.dtype == torch.int64 and perm_inv.shape[1] == C
        assert 0 <= row0 and R >= 0 and row0 + R <= Rtot
        if index is None:
            assert perm_inv.shape[0] == B
            if out is None:
                out = torch.empty((B, R, C), dtype=torch.uint8, device=q.device)
            assert tuple(out.shape) == (B, R, C)
        else:
            assert index.dtype == torch.int64 and index.is_contiguous() and index.numel() == B
            assert out is not None and tuple(out.shape) == (perm_inv.shape[0], R, C)
        assert out.is_contiguous() and out.dtype == torch.uint8
        with torch.cuda.device(q.device):
            if index is not None:
                self._check(self._lib.forge_codes_to_layer_order_scatter(
                    q.data_ptr() + row0, Rtot, C * Rtot, _ptr(index), _ptr(perm_inv), _ptr(out), B, R, C,
                    _stream()))
            else:
                self._check(self._lib.forge_codes_to_layer_order_strided(
                    q.data_ptr() + row0, Rtot, C * Rtot, _ptr(perm_inv), _ptr(out), B, R, C, _stream()))
        return out

    def pack_int4(self, codes, qzeros, group_size):
        _need_cuda(codes, qzeros)
        R, C = codes.shape
        assert codes.is_contiguous() and codes.dtype == torch.uint8
        out = torch.empty((R, (C + 7) // 8), dtype=torch.int32, device=codes.device)
        with torch.cuda.device(codes.device):
            self._check(self._lib.forge_pack_int4(_ptr(codes), _ptr(qzeros), _ptr(out), R, C,
                                                  int(group_size), _stream()))
        return out


    def fp8_block_dequant(self, w, scale_inv, dtype=torch.bfloat16):
        """w [O,I] or [B,O,I] float8_e4m3fn (or its uint8 view), scale_inv [.., nO, nI] f32 ->
        dequantised weights; tile sizes are inferred as forge/utils/io.py:533-548 does."""
        _need_cuda(w, scale_inv)
        squeeze = w.dim() == 2
        w3 = (w.unsqueeze(0) if squeeze else w).contiguous()
        s3 = (scale_inv.unsqueeze(0) if squeeze else scale_inv).contiguous().float()
        B, O, I = w3.shape
        nO, nI = s3.shape[1:]
        if I % nI:
            raise RuntimeError("fp8_block_dequant: I must be a multiple of the scale grid width")
        si = I // nI
        so = si if (O + si - 1) // si == nO else (O + nO - 1) // nO
        out = torch.empty((B, O, I), dtype=dtype, device=w.device)
        with torch.cuda.device(w.device):
            self._check(self._lib.forge_fp8_e4m3_block_dequant(
                _ptr(w3.view(torch.uint8)), _ptr(s3), _ptr(out), _dtype_code(out), B, O, I, so, si,
                _stream()))
        return out[0] if squeeze else out

    def pack_sparsegptq14_to_u64x2(self, qweight_rc, M, scales):
        """kernels.cpp:122-126: qweight_rc [R,C] u8, M [G32,R] u32, scales [G32,R] f32 ->
        uint64 [G2, R, 2]."""
        _need_cuda(qweight_rc, M, scales)
        qweight_rc, M, scales = qweight_rc.contiguous(), M.contiguous(), scales.contiguous()
        if qweight_rc.dim() != 2 or M.dim() != 2 or scales.dim() != 2:
            raise RuntimeError("pack_sparsegptq14_to_u64x2: 2-d tensors expected")
        R, C = qweight_rc.shape
        G32 = (C + 31) // 32
        if M.shape[0] != G32 or M.shape[1] != R or tuple(scales.shape) != (G32, R):
            raise RuntimeError("pack_sparsegptq14_to_u64x2: M/scales must be [ceil(C/32), R]")
        out = torch.empty(((G32 + 1) // 2, R, 2), dtype=torch.uint64, device=qweight_rc.device)
        with torch.cuda.device(qweight_rc.device):
            self._check(self._lib.forge_pack_sparsegptq14_to_u64x2(
                _ptr(qweight_rc), _ptr(M), _ptr(scales.float()), _ptr(out), R, C, _stream()))
        return out

    def dequantize_groups(self, qweight, scales, qzeros, group_size, dtype=torch.bfloat16):
        """qweight [R,C] or [B,R,C] u8, scales/qzeros [.., R*G] f32 -> (q - q0) * s in `dtype`
        (forge/utils/engine.py:71-97)."""
        _need_cuda(qweight, scales, qzeros)
        squeeze = qweight.dim() == 2
        q3 = (qweight.unsqueeze(0) if squeeze else qweight).contiguous()
        B, R, C = q3.shape
        G = (C + group_size - 1) // group_size
        s2 = scales.reshape(B, -1).float().contiguous()
        z2 = qzeros.reshape(B, -1).float().contiguous()
        if q3.dtype != torch.uint8 or s2.shape[1] != R * G or z2.shape[1] != R * G:
            raise ValueError(f"Expected uint8 codes and scales/qzeros numel == R*G ({R * G})")
        out = torch.empty((B, R, C), dtype=dtype, device=q3.device)
        with torch.cuda.device(q3.device):
            self._check(self._lib.forge_dequantize_groups(
                _ptr(q3), _ptr(s2), _ptr(z2), _ptr(out), _dtype_code(out), B, R, C, group_size,
                _stream()))
        return out[0] if squeeze else out

    def gather_scaled_rows(self, X, row_idx, weight=None):
        """out[i] = X[row_idx[i]] * weight[i] in X's dtype (weight None: plain gather);
        X [T,C] bf16/f32 with unit column stride, row_idx [N] int64."""
        _need_cuda(X, row_idx, weight)
        assert X.dim() == 2 and X.stride(1) == 1 and row_idx.dtype == torch.int64
        row_idx = row_idx.contiguous()
        if weight is not None:
            weight = weight.to(X.dtype).contiguous()
            assert weight.numel() == row_idx.numel()
        T, C = X.shape
        N = row_idx.numel()
        out = torch.empty((N, C), dtype=X.dtype, device=X.device)
        with torch.cuda.device(X.device):
            self._check(self._lib.forge_gather_scaled_rows(
                _ptr(X), _dtype_code(X), X.stride(0), T, C, _ptr(row_idx), _ptr(weight), _ptr(out),
                N, _stream()))
        return out


class _HipUnavailable(ModuleType):
    def __init__(self, why: str) -> None:
        super().__init__("forge.backend.hip.kernels")
        self.__dict__["_why"] = why

    def __getattr__(self, name: str):
        raise RuntimeError(f"4Bit-Forge HIP kernels are unavailable: {self.__dict__['_why']}")


def _make_kernels():
    if not torch.cuda.is_available():
        return _HipUnavailable("torch.cuda.is_available() is False (no MI355X visible)")
    try:
        return _HipKernels(load_library())
    except (OSError, RuntimeError, AttributeError) as exc:
        return _HipUnavailable(str(exc))


kernels = _make_kernels()
