"""Batched GPTQ over the experts of one MoE layer (no counterpart in the reference, which
walks its ``GPTQ`` handles one linear layer at a time, quant.py:414-417).

``ExpertGroupGPTQ`` holds E equally shaped experts.  Several weight stacks may share one
Hessian stack (gate_proj and up_proj see the same tokens: the reference's ``owner``
mechanism, forge/gptq.py:36,84-94), so they also share one factorisation.  ``update``
takes the routed tokens of ALL experts at once (rows grouped by expert + offsets) and
issues one ragged MFMA launch; ``quantize`` runs the scale search, the factorisation
and the sweep for a chunk of experts per launch so that every kernel fills the GPU.
Arithmetic per expert is the one of ``forge.gptq.GPTQ``.

Experts that saw at most ``low_rank_tokens`` rows (most experts of a large routed layer see a
handful of the calibration tokens, many none) never get a C x C Hessian: their rows are kept,
and the solve runs on the closed form that H = D + B^T B has in those few rows
(``kernels.lowrank_factor`` / ``kernels.gptq_sweep_lowrank``): the same result in exact
arithmetic.  Experts with more rows than that, but still few against their number of input
features (``rows_route_tokens``), take the same closed form in its blocked shape
(``kernels.rows_factor_blocked`` / ``kernels.gptq_sweep_rows_blocked``): products of inner
dimension n on the matrix pipe instead of a C x C factorisation and products of inner
dimension C.
"""
from __future__ import annotations

import collections
import threading
from typing import List, Optional, Sequence

import torch

from forge.backend.hip import kernels


class ExpertGroupGPTQ:
    # quantize() queues its work and returns without waiting for the GPU.  A caller that builds
    # group after group (a layer's chunks, a model's layers) would otherwise run arbitrarily far
    # ahead of the device, each call holding tens of GB of workspace that cannot be reused before
    # its kernels have run: every call waits for the call before the last MAX_IN_FLIGHT to finish.
    MAX_IN_FLIGHT = 2
    # The blocked closed form costs 4 n C R multiply-adds, half of them as products of inner
    # dimension 128 that are bound by the traffic of the n x R accumulator, plus a chain of small
    # launches per 128-column block, against C^2 R / 2 + C^3 / 6 of the route through the
    # Hessian: measured on the DeepSeek-V3-shaped layer (256 experts a step) it wins up to 512
    # rows at C = 7168 (232.4 / 231.2 / 237.1 ms with a limit of 256 / 512 / 1024 against 235.6
    # without), i.e. while n (a multiple of 128) times this factor is at most C.
    ROWS_ROUTE_COST = 7
    _in_flight = collections.deque()
    _in_flight_lock = threading.Lock()
    # The device runs the kernels of one hardware queue one after the other, and a process has
    # four such queues for all of its streams: a fresh pair of side streams per call ends up
    # sharing queues with the callers' streams in patterns that change from call to call (a
    # chain of small kernels then waits behind a 20 ms scale search).  So every group of a
    # device shares ONE stream for the scale searches (each fills the device: they run one
    # after the other anyway, in the order of the quantize() calls) and ONE for the low-rank
    # experts' chains: with two callers' streams that is four streams, one queue each.
    _side_streams = {}
    _side_streams_lock = threading.Lock()

    @classmethod
    def _streams_of(cls, dev):
        key = dev.index if dev.index is not None else torch.cuda.current_device()
        with cls._side_streams_lock:
            if key not in cls._side_streams:
                cls._side_streams[key] = (torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev))
            return cls._side_streams[key]                   # default priority

    def __init__(self, weights: Sequence[torch.Tensor], bits: int = 4, group_size: int = 128,
                 symmetric: bool = False, quantization_scale: str = "mse",
                 quantization_order: str = "activation", rel_damp: float = 1e-2,
                 algorithm: str = "gptq", device=None, factor_route: str = "direct",
                 low_rank_tokens: Optional[int] = None, rows_route_tokens: Optional[int] = None):
        """weights: stacks [E, R_i, C] (bf16 or f32) that share the input features C.
        algorithm: "gptq", "sparsegptq" (1:4 joint solve; quantize() then also returns the
        keep-masks M [E, ceil(C/32), R_i] u32 per stack) or "babai".
        factor_route (algorithms "gptq" and "sparsegptq"): "inverse" computes the reference's factor, the
        upper Cholesky factor of inv(H) (forge/gptq.py:160-166), and sweeps with the column
        errors; "direct" stops at the factor of H itself and sweeps with the displacements
        w0 - deq (``kernels.gptq_sweep_direct_batched``): the same solve in exact arithmetic
        at half the factorisation work, codes differing only where fp32 rounding decides a
        near-tie.
        low_rank_tokens (0..128; algorithm "gptq" on the direct route, C a multiple of 16):
        experts with at most this many calibration rows are solved from the rows themselves,
        see the module text; 0 = every expert through its Hessian.  None = 64 where the blocked
        closed form can take over from there (rows_route_tokens), else 128: at 65-128 rows the
        per-row-vector sweep, which runs on the vector ALU, costs more than the blocked form's
        matrix products and in-block chains (benchmark layer: 230.7 ms a step with 128, 223.7
        with 64, 228.1 with 32).  Such an expert has no stored Hessian: read Hessians through
        ``hessian(e)``.
        rows_route_tokens (needs low_rank_tokens > 0, C and every R a multiple of 128): experts
        with more rows than low_rank_tokens and at most this many, rounded up to a multiple of
        128, are solved from their rows by the blocked closed form, as long as that count times
        ``ROWS_ROUTE_COST`` does not exceed C (beyond that the route through the Hessian is the
        cheaper one).  None = 512; 0 = off."""
        if algorithm not in ("gptq", "sparsegptq", "babai"):
            raise NotImplementedError(f"algorithm={algorithm!r}: 'gptq', 'sparsegptq' or 'babai'")
        if factor_route not in ("direct", "inverse"):
            raise ValueError(f"factor_route={factor_route!r}: 'direct' or 'inverse'")
        self.algorithm = algorithm
        self.factor_route = factor_route
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
        # Hessians of the experts that go through one, [slots, C, C] f32: expert e owns
        # _Hpool[_slot[e]] (-1: none yet).  Experts that are solved from their rows never get one
        # (a DeepSeek-V3 layer: 38 of 256 experts x 205 MB instead of 256).
        self._Hpool: Optional[torch.Tensor] = None
        self._slot = [-1] * self.E
        self._slot_expert: List[int] = []
        self.num_samples = [0] * self.E                 # host-side counts
        if low_rank_tokens is not None and not 0 <= int(low_rank_tokens) <= 128:
            raise ValueError(f"low_rank_tokens={low_rank_tokens}: 0..128")
        ok = algorithm == "gptq" and factor_route == "direct" and self.C % 16 == 0 \
            and len({w.dtype for w in self.W}) == 1
        rows_ok = ok and low_rank_tokens != 0 and self.C % 128 == 0 and all(w.shape[1] % 128 == 0 for w in self.W)
        want = 512 if rows_route_tokens is None else int(rows_route_tokens)
        if want < 0 or want % 128 != 0:
            raise ValueError(f"rows_route_tokens={rows_route_tokens}: a multiple of 128")
        self.rows_route_tokens = min(want, self.C // self.ROWS_ROUTE_COST // 128 * 128) if rows_ok else 0
        if low_rank_tokens is None:
            low_rank_tokens = 64 if self.rows_route_tokens >= 128 else 128
        self.low_rank_tokens = int(low_rank_tokens) if ok else 0
        if self.rows_route_tokens <= self.low_rank_tokens:
            self.rows_route_tokens = 0
        # experts on the blocked route: rows_route[e], their rows as they came (a list of [k, C]
        # tensors per expert, copies)
        self.rows_route = [False] * self.E
        self._rows = [[] for _ in range(self.E)]
        # rows of the experts that are still on the low-rank route, [E, _cap, C] f32 (zero rows
        # beyond num_samples[e]); low_rank[e] turns False for good once an expert has seen more
        self._cap = next(n for n in (16, 32, 64, 128) if n >= max(self.low_rank_tokens, 1))
        self.low_rank = [self.low_rank_tokens > 0] * self.E
        self._kept: Optional[torch.Tensor] = None
        self._kept_wide = [False] * self.E               # an f32 row among the kept ones
        self._non_invertible = torch.zeros(self.E, dtype=torch.bool)
        self._pending_info = []                          # (expert ids, device flags) not yet fetched
        self._prepared = None                            # what prepare() queued, until quantize() uses it

    @property
    def issue_non_invertible(self) -> torch.Tensor:
        """[E] bool: experts whose factorisation failed in a quantize() so far (they were solved
        with the identity instead, forge/gptq.py:168-175).  Reading it waits for the GPU."""
        for ids, info in self._pending_info:
            self._non_invertible[ids] |= (info > 0).cpu()
        self._pending_info = []
        return self._non_invertible

    @torch.no_grad()
    def hessian(self, e: int) -> torch.Tensor:
        """H of expert e, [C, C] f32, as forge/gptq.py:61-80 would have accumulated it.  An
        expert that is solved from its rows has no stored Hessian (that is the point of those
        routes); it is formed here from the rows that were kept, (2/n) X^T X in float64
        rounded once; an expert that saw nothing has none (the reference's ``H is None``)."""
        n = self.num_samples[e]
        if n == 0:
            return None
        if self.low_rank[e]:
            X = self._kept[e, :n].double()
            return ((2.0 / n) * X.t() @ X).float()
        if self.rows_route[e]:
            X = torch.cat(self._rows[e]).double()
            return ((2.0 / n) * X.t() @ X).float()
        return self._Hpool[self._slot[e]]

    def _give_slots(self, experts):
        """Hessian storage for these experts (those that have none yet); the pool grows by what
        is asked for, existing Hessians are copied over."""
        fresh = [e for e in experts if self._slot[e] < 0]
        if not fresh:
            return
        have = len(self._slot_expert)
        if self._Hpool is None or self._Hpool.shape[0] < have + len(fresh):
            pool = torch.empty((have + len(fresh), self.C, self.C), dtype=torch.float32, device=self.device)
            if have:
                pool[:have] = self._Hpool[:have]
            self._Hpool = pool
        for e in fresh:
            self._slot[e] = len(self._slot_expert)
            self._slot_expert.append(e)

    def workspace_bytes(self, n_dense: int, n_low: int, n_rows: int, rows_nmax: int, R: int) -> int:
        """Device memory that quantize() allocates while one of its jobs is in flight (a job = the
        stacks that share a factor, R rows in all) for n_dense experts through their Hessians,
        n_low solved from at most 128 rows and n_rows by the blocked closed form with up to
        rows_nmax rows: permuted Hessian, factor band, solver-order weights (fp32 and their own
        type), codes and the kernels' workspaces.  The three routes run on two streams, so their
        needs add up."""
        C, esz = self.C, self.W[0].element_size()
        per_matrix = C * R * (4 + esz + 1)                    # X, W0, codes
        need = 0
        if n_dense:
            need += n_dense * (2 * C * C * 4 + per_matrix) + kernels.workspace_bytes("chol", n_dense, C) \
                + kernels.workspace_bytes("sweep_direct", n_dense, C, R)
        if n_low:
            need += n_low * (C * R * (esz + 1) + 2 * C * 128 * 4) + kernels.workspace_bytes("lowrank", n_low, C, 128)
        if n_rows:
            need += n_rows * (per_matrix + 3 * rows_nmax * C * 4 + C * 128 * 4) \
                + kernels.workspace_bytes("rows_factor", n_rows, C, rows_nmax) \
                + kernels.workspace_bytes("sweep_rows", n_rows, R, rows_nmax)
        return need

    def _require_memory(self, need: int):
        """Raises before anything is queued when the device cannot hold a solve's workspace: a
        kernel that meets a full device in the middle of the queue takes the queue down with it."""
        free, _ = torch.cuda.mem_get_info(self.device)
        cached = torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
        if need > free + cached:
            raise RuntimeError(
                f"ExpertGroupGPTQ.quantize needs about {need / 2**30:.1f} GiB of workspace for a chunk, "
                f"{(free + cached) / 2**30:.1f} GiB are free on {self.device}: pass a smaller `chunk`")

    def _per_slot(self, per_expert):
        """a per-expert host list rearranged by Hessian slot"""
        return [per_expert[e] for e in self._slot_expert]

    def _dev(self, values, dtype=None):
        """A small host list as a device tensor without stopping the host: through pinned memory
        and an asynchronous copy (torch.tensor(..., device=...) copies from pageable memory and
        returns only when the stream has reached the copy, i.e. when all the work queued before
        it is done)."""
        return torch.tensor(values, dtype=dtype).pin_memory().to(self.device, non_blocking=True)

    # ------------------------------------------------------------------ Hessians
    @torch.no_grad()
    def update(self, X: torch.Tensor, offsets: Sequence[int]):
        """X [T, C]: calibration rows grouped by expert; expert e owns rows
        offsets[e]:offsets[e+1].  Running mean per expert as in forge/gptq.py:61-80."""
        if len(offsets) != self.E + 1:
            raise ValueError("offsets must have E+1 entries")
        self._prepared = None
        X = X.to(self.device)
        if X.dtype not in (torch.bfloat16, torch.float32):
            X = X.float()
        if X.stride(-1) != 1:
            X = X.contiguous()
        if self._kept is None and self.low_rank_tokens:
            self._kept = torch.zeros((self.E, self._cap, self.C), dtype=torch.float32, device=self.device)
        if not self.low_rank_tokens:
            self._give_slots(range(self.E))          # every expert through its Hessian, in order
        row0, counts, alpha, beta = [], [], [], []
        src, dst, late, keep = [], [], [], []
        for e in range(self.E):
            o, new = int(offsets[e]), int(offsets[e + 1]) - int(offsets[e])
            n = self.num_samples[e]
            total = n + new
            self.num_samples[e] = total
            if self.low_rank[e] and total <= self.low_rank_tokens:
                src.extend(range(o, o + new))                     # keep the rows, no Hessian
                self._kept_wide[e] |= new > 0 and X.dtype == torch.float32
                dst.extend(range(e * self._cap + n, e * self._cap + total))
                new = 0
            elif (self.low_rank[e] or self.rows_route[e]) and total <= self.rows_route_tokens:
                if self.low_rank[e]:                              # outgrew the per-row-vector sizes
                    self.low_rank[e], self.rows_route[e] = False, True
                    if n > 0:
                        self._rows[e].append(self._kept[e, :n].clone())
                        self._kept[e].zero_()
                if new > 0:
                    keep.append((e, o, new))
                new = 0
            elif self.low_rank[e] or self.rows_route[e]:
                if n > 0:
                    late.append((e, n, o, new))                   # H[e] was never written
                    new = 0
                else:
                    self.low_rank[e] = self.rows_route[e] = False
            row0.append(o)
            counts.append(new)
            alpha.append(2.0 / max(total, 1))
            beta.append(n / max(total, 1))
        if src:
            self._kept.view(self.E * self._cap, self.C)[self._dev(dst)] = X[self._dev(src)].float()
        if keep:
            # one copy for all of them; each expert holds a view of its rows
            block = torch.cat([X[o:o + new] for _, o, new in keep])
            at = 0
            for e, _, new in keep:
                self._rows[e].append(block[at:at + new])
                at += new
        self._give_slots([e for e in range(self.E) if counts[e] > 0] + [e for e, *_ in late])
        if any(counts):
            kernels.hessian_update_ranges(X, self._per_slot(row0), self._per_slot(counts),
                                          self._Hpool[:len(self._slot_expert)], self._per_slot(alpha),
                                          self._per_slot(beta))
        if late:
            # experts that leave the low-rank route: their Hessian from the kept rows and the
            # new ones together, (2/total) X^T X, what the running mean equals
            parts, row0, counts, alpha = [], [0] * self.E, [0] * self.E, [0.0] * self.E
            at = 0
            # kept rows that came in as f32 are not rounded to a later call's bf16: the route
            # through the Hessian would have summed them in f32 too
            dt = torch.float32 if any(self._kept_wide[e] for e, *_ in late) else X.dtype
            dt = torch.float32 if any(r.dtype == torch.float32 for e, *_ in late for r in self._rows[e]) else dt
            for e, n, o, new in late:
                if self.rows_route[e]:
                    parts += [r.to(dt) for r in self._rows[e]] + [X[o:o + new].to(dt)]
                else:
                    parts += [self._kept[e, :n].to(dt), X[o:o + new].to(dt)]
                row0[e], counts[e], alpha[e] = at, n + new, 2.0 / (n + new)
                at += n + new
            rows = torch.cat(parts)               # (a copy: the kept rows are cleared next)
            for e, *_ in late:
                if self.low_rank[e]:
                    self._kept[e].zero_()
                self._rows[e] = []
                self.low_rank[e] = self.rows_route[e] = False
            kernels.hessian_update_ranges(rows, self._per_slot(row0), self._per_slot(counts),
                                          self._Hpool[:len(self._slot_expert)], self._per_slot(alpha),
                                          [0.0] * len(self._slot_expert))

    add_batch = update

    # ------------------------------------------------------------------ solve
    @torch.no_grad()
    def prepare(self):
        """Queues what quantize() has to know on the host before it can queue the solve (which
        experts have no usable Hessian, which have dead features, which may have all-zero
        weight columns) and the transfer of those few flags, and returns without waiting.
        quantize() calls it itself; a caller that calls it earlier, right after its last
        update() and on the same stream, with other work queued behind it, finds the flags
        there when it calls quantize(), which then neither waits for that other work nor makes
        its scale search wait for it.  Another update() discards it."""
        E, C, dev = self.E, self.C, self.device
        lr_host = list(self.low_rank)
        rr_host = list(self.rows_route)
        # every expert that is not solved from its rows has a Hessian (one that saw nothing gets
        # the identity written into its slot by quantize())
        self._give_slots([e for e in range(E) if not (lr_host[e] or rr_host[e])])
        # experts that never saw a token (or whose Hessian went NaN) fall back to H = I
        seen = self._dev([n > 0 for n in self.num_samples])
        if self._slot_expert == list(range(E)):
            diag_all = self._Hpool.diagonal(dim1=1, dim2=2)                # [E, C] view
        else:
            diag_all = torch.zeros((E, C), dtype=torch.float32, device=dev)
            if self._slot_expert:
                diag_all[self._dev(self._slot_expert)] = self._Hpool[:len(self._slot_expert)].diagonal(dim1=1, dim2=2)
        any_lr = any(lr_host)
        lr_dev = alpha32 = None
        if any_lr:
            # low-rank experts: diag(H) = (2/n) sum of squares of their kept rows (float64, rounded
            # once, as the Hessian kernel does for the others); H[e] itself holds nothing
            if self._kept is None:
                self._kept = torch.zeros((E, self._cap, C), dtype=torch.float32, device=dev)
            lr_dev = self._dev(lr_host)
            alpha32 = self._dev([2.0 / max(n, 1) for n in self.num_samples], dtype=torch.float32)
            cap = self._cap
            d_lr = kernels.rows_diagonal(
                self._kept.view(E * cap, C), self._dev([e * cap for e in range(E)]),
                self._dev([n if lr else 0 for n, lr in zip(self.num_samples, lr_host)], dtype=torch.int32),
                alpha32.double())
            diag_all = torch.where(lr_dev[:, None], d_lr, diag_all)
        rows_all, rows_at = None, {}
        rr_list = [e for e in range(E) if rr_host[e]]
        if rr_list:
            # experts on the blocked route: the same diagonal from their own rows, which from
            # here on lie end to end in ONE tensor (each expert keeps a view of its part)
            pieces = [p for e in rr_list for p in self._rows[e]]
            if any(p.dtype == torch.float32 for p in pieces):
                pieces = [p.float() for p in pieces]
            rows_all = pieces[0] if len(pieces) == 1 else torch.cat(pieces)
            at = 0
            for e in rr_list:
                rows_at[e] = at
                self._rows[e] = [rows_all[at:at + self.num_samples[e]]]
                at += self.num_samples[e]
            d_rr = kernels.rows_diagonal(
                rows_all, self._dev([rows_at[e] for e in rr_list]),
                self._dev([self.num_samples[e] for e in rr_list], dtype=torch.int32),
                self._dev([2.0 / self.num_samples[e] for e in rr_list], dtype=torch.float64))
            diag_all = diag_all.index_copy(0, self._dev(rr_list), d_rr)
        bad = (~seen) | torch.isnan(diag_all).any(dim=1)
        if any_lr or any(rr_host):
            off_h = self._dev([a or b for a, b in zip(lr_host, rr_host)])
            diag_all = torch.where((bad & off_h)[:, None], torch.ones((), device=dev), diag_all)
        # Weights with pruned columns zeroed decide the (unpermuted-index) zero-column mask
        # that the reference applies to the permuted Hessian (forge/gptq.py:145-149).  A column
        # can only be all zero if its first rows are: one look at 8 rows of every expert (fp8-
        # or int-derived weights do contain single zeros) and at the Hessian diagonals tells
        # which experts need the full pass over their weights at all.  These flags and `bad`
        # reach the host in ONE transfer (pinned memory, asynchronous), the only thing that
        # quantize() waits for before it queues the solve.
        dead_any = ((diag_all == 0) & ~bad[:, None]).any(dim=1)
        maybe_zero = [(W[:, :8, :] == 0).all(dim=1).any(dim=1) for W in self.W]
        flags = torch.stack([bad, dead_any] + maybe_zero)                  # [2 + stacks, E]
        host_flags = torch.empty(flags.shape, dtype=flags.dtype, pin_memory=True)
        host_flags.copy_(flags, non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        self._prepared = dict(diag_all=diag_all, bad=bad, host_flags=host_flags, ready=ready,
                              lr_host=lr_host, any_lr=any_lr, lr_dev=lr_dev, alpha32=alpha32,
                              rr_host=rr_host, rows_all=rows_all, rows_at=rows_at, keep=flags)
        return self._prepared

    @torch.no_grad()
    def quantize(self, chunk: int = 32, max_shrink: float = 0.2, n_grid: int = 100,
                 norm: float = 2.4, overlap_scale_search: bool = True):
        """Returns one (qweight [E,R,C] u8, scales [E,R*G] f32, qzeros [E,R*G] f32) per stack;
        with algorithm="sparsegptq" a fourth element M [E, ceil(C/32), R] u32 (bit i of word w
        <-> column 32 w + i of the SOLVER order, as the reference returns it).
        overlap_scale_search=False keeps the scale search on the caller's stream instead of a
        side stream (same results; for per-kernel timing, where no kernel's time should include
        another stream's work)."""
        E, C, gs, dev = self.E, self.C, self.group_size, self.device
        G = (C + gs - 1) // gs
        mse = self.quantization_scale == "mse"
        prep = self._prepared if self._prepared is not None else self.prepare()
        self._prepared = None
        prep["ready"].synchronize()        # the only wait for the GPU before the solve is queued
        diag_all, bad, host_flags = prep["diag_all"], prep["bad"], prep["host_flags"]
        lr_host, any_lr = prep["lr_host"], prep["any_lr"]
        lr_dev, alpha32 = prep["lr_dev"], prep["alpha32"]
        rr_host, rows_all, rows_at = prep["rr_host"], prep["rows_all"], prep["rows_at"]
        any_rr = any(rr_host)
        # (per expert: an indexed assignment of a broadcast identity moves the same bytes at a
        # fraction of the fill rate)
        for e in host_flags[0].nonzero().flatten().tolist():
            if lr_host[e] or rr_host[e]:
                continue                       # no matrix: its rows count as none (below)
            He = self._Hpool[self._slot[e]]
            He.zero_()
            He.diagonal().fill_(1.0)
            diag_all = diag_all.index_fill(0, self._dev([e]), 1.0)
        # the largest chunk's workspace must fit before anything is queued
        sizes_all = sum(int(W.shape[1]) for W in self.W)
        need = 0
        for c0 in range(0, E, chunk):
            ids = range(c0, min(E, c0 + chunk))
            rr = [self.num_samples[e] for e in ids if rr_host[e] and not bool(host_flags[0, e])]
            need = max(need, self.workspace_bytes(
                sum(1 for e in ids if not (lr_host[e] or rr_host[e])),
                sum(1 for e in ids if lr_host[e] and not bool(host_flags[0, e])),
                len(rr), max([(n + 127) // 128 * 128 for n in rr], default=0), sizes_all))
        self._require_memory(need)
        failed = []
        cand = None                                   # the shrink factors, made on the search stream
        side, lr_shared = self._streams_of(dev) if overlap_scale_search else (None, None)
        # the low-rank experts' kernels are chains of dependent steps on a few wavefronts: on a
        # stream of their own they run beside the other experts' matrix products
        lr_side = lr_shared if (any_lr or any_rr) else None

        sizes = [int(W.shape[1]) for W in self.W]
        sparse = self.algorithm == "sparsegptq"
        direct = self.algorithm in ("gptq", "sparsegptq") and self.factor_route == "direct"
        babai = self.algorithm == "babai"
        outs = [[torch.empty((E, R, C), dtype=torch.uint8, device=dev),
                 torch.empty((E, R * G), dtype=torch.float32, device=dev),
                 torch.empty((E, R * G), dtype=torch.float32, device=dev)]
                + ([torch.empty((E, (C + 31) // 32, R), dtype=torch.uint32, device=dev)] if sparse else [])
                for R in sizes]

        for e0 in range(0, E, chunk):
            e1 = min(E, e0 + chunk)
            B = e1 - e0
            diag = diag_all[e0:e1]
            dead = diag == 0                                             # [B, C]
            if self.quantization_order == "activation":
                # Babai walks back to front: ascending order (forge/gptq.py:107-108)
                perm = torch.argsort(torch.where(dead, torch.ones_like(diag), diag), dim=1,
                                     descending=not babai)
            else:
                perm = torch.arange(C, device=dev).expand(B, C).contiguous()
            dead_perm = torch.gather(dead, 1, perm)
            if babai:
                # the solve runs as a forward sweep over the reversed order (see forge/gptq.py)
                perm = perm.flip(1).contiguous()
            # the inverse permutation by a scatter (argsort(perm), forge/gptq.py:113, sorts again)
            perm_inv = torch.empty_like(perm).scatter_(
                1, perm, torch.arange(C, device=dev).expand(B, C))
            g_idx = (perm // gs).to(torch.int32).contiguous()
            dead_u8 = dead.to(torch.uint8).contiguous()
            has_dead = bool(host_flags[1, e0:e1].any())
            flags = [bool(host_flags[2 + i, e0:e1].any()) for i in range(len(self.W))]
            masks = []
            for W, maybe in zip(self.W, flags):
                if maybe or has_dead:
                    # all_r(W[r, c] == 0 or dead[c]) = all_r(W[r, c] == 0) or dead[c]
                    zero_cols = (W[e0:e1] == 0).all(dim=1) | dead
                    masks.append((dead_perm | zero_cols).to(torch.uint8).contiguous())
                else:
                    masks.append(None)
            if all(m is None for m in masks):
                shared = True
                masks = [torch.zeros((B, C), dtype=torch.uint8, device=dev)] * len(self.W)
            else:
                zero = torch.zeros((B, C), dtype=torch.uint8, device=dev)
                masks = [zero if m is None else m for m in masks]
                shared = all(torch.stack([(masks[0] == m).all() for m in masks[1:]]).cpu().tolist()) \
                    if len(masks) > 1 else True
                if babai:   # positions of the reference's order -> positions of the reversed one
                    masks = [m.flip(1).contiguous() for m in masks]
            # the experts of the chunk by route (positions in the chunk, ascending)
            none_ids = [e - e0 for e in range(e0, e1) if (lr_host[e] or rr_host[e]) and bool(host_flags[0, e])]
            lr_ids = [e - e0 for e in range(e0, e1) if lr_host[e] and not bool(host_flags[0, e])]
            rr_ids = [e - e0 for e in range(e0, e1) if rr_host[e] and not bool(host_flags[0, e])]
            dn_ids = [e - e0 for e in range(e0, e1) if not (lr_host[e] or rr_host[e])]
            # stacks that share the factor are swept as ONE tall matrix (rows are independent)
            jobs = [list(range(len(self.W)))] if shared else [[i] for i in range(len(self.W))]
            for job in jobs:
                # the stacks of a job share the factor and are swept as ONE tall matrix, their rows
                # one after the other; nothing is concatenated: each stack is searched and laid
                # out from where it is
                R = sum(sizes[i] for i in job)
                # the scale search only needs the weights: it runs on a side stream so that
                # its VALU/transcendental work shares the CUs with the MFMA-bound factorisation
                main = torch.cuda.current_stream()
                search = side if side is not None else main
                # the search reads the weights and, where features are dead, their mask: without
                # dead features it only waits for what prepare() saw queued, not for whatever
                # the caller has queued on this stream since
                if has_dead:
                    search.wait_stream(main)
                else:
                    search.wait_event(prep["ready"])
                with torch.cuda.stream(search):
                    if mse and cand is None:
                        cand = torch.linspace(1.0, max_shrink, n_grid, dtype=torch.float32, device=dev)
                    parts = []
                    for i in job:
                        # pruned columns are zero in the reference's W before the grid is built
                        Wi = self.W[i][e0:e1]
                        Wsrc = Wi.masked_fill(dead[:, None, :], 0) if has_dead else Wi
                        parts.append(kernels.quant_grid(Wsrc, gs, self.bits, self.symmetric, mse,
                                                        cand, norm))
                        Wsrc.record_stream(search)
                        del Wsrc
                    if len(parts) == 1:
                        scales, qzeros = parts[0]
                    else:
                        scales = torch.cat([p[0].view(B, sizes[i], G) for p, i in zip(parts, job)], dim=1)
                        qzeros = torch.cat([p[1].view(B, sizes[i], G) for p, i in zip(parts, job)], dim=1)
                    sT = scales.view(B, R, G).transpose(1, 2).contiguous()
                    zT = qzeros.view(B, R, G).transpose(1, 2).contiguous()
                mask = masks[job[0]]

                def layout_in(ids, W0, X=None, skip_out=False):
                    """weights of the chunk's experts `ids` -> solver order: one launch per stack"""
                    whole = len(ids) == B
                    idx = None if whole else self._dev(ids)
                    r0 = 0
                    for i in job:
                        kernels.weight_to_solver_order(self.W[i][e0:e1], perm_inv, dead_u8, out=X, row0=r0,
                                                       out0=W0, skip_out=skip_out, index=idx)
                        r0 += sizes[i]

                def layout_out(ids, q, M=None):
                    whole = len(ids) == B
                    idx = None if whole else self._dev(ids)
                    r0 = 0
                    for i in job:
                        Ri = sizes[i]
                        kernels.codes_to_layer_order(q, perm_inv, out=outs[i][0][e0:e1], row0=r0, rows=Ri,
                                                     index=idx)
                        if M is not None:
                            if whole:
                                outs[i][3][e0:e1] = M[:, :, r0:r0 + Ri]
                            else:
                                outs[i][3][e0:e1][idx] = M[:, :, r0:r0 + Ri]
                        r0 += Ri

                # ---------------------------------------------------------- low-rank experts
                lr_stream = main
                if lr_ids or none_ids or rr_ids:
                    lr_stream = lr_side if lr_side is not None and dn_ids else main
                    lr_stream.wait_stream(main)
                with torch.cuda.stream(lr_stream):
                    # by the number of rows the kernels are compiled for: 4, 16, 32, 64 or 128; the
                    # largest first: the sweep's workgroups start in launch order and run in
                    # proportion to their rows, the short ones fill in behind the long ones
                    buckets = []
                    for lo, nr in ((64, 128), (32, 64), (16, 32), (4, 16), (0, 4)):
                        ids = [i for i in lr_ids if lo < self.num_samples[e0 + i] <= nr]
                        if ids:
                            buckets.append((nr, ids))
                    # one sweep launch for all of them: their vectors laid end to end
                    ids_all = [i for _, ids in buckets for i in ids]
                    ns = [nr for nr, ids in buckets for _ in ids]
                    if ids_all:
                        Bp_all = torch.empty(C * sum(ns), dtype=torch.float32, device=dev)
                        Hm_all = torch.empty_like(Bp_all)
                        info = torch.empty(len(ids_all), dtype=torch.int32, device=dev)
                        W0 = torch.empty((len(ids_all), C, R), dtype=self.W[job[0]].dtype, device=dev)
                    pos = at = 0
                    for nr, ids in buckets:
                        li = self._dev(ids)
                        msk = mask[li].bool()                               # [Bl, C], solver order
                        span = slice(at, at + len(ids) * C * nr)
                        Bpv = Bp_all[span].view(len(ids), C, nr)
                        own = [self.num_samples[e0 + i] for i in ids]
                        # sqrt(2/n) X in solver order with pruned columns zero, [Bl, C, nr]
                        kernels.rows_operands(
                            self._kept.view(E * self._cap, C), self._dev([(e0 + i) * self._cap for i in ids]),
                            self._dev(own, dtype=torch.int32), alpha32[e0:e1][li].double().sqrt(),
                            perm[li], mask[li], nr, want_bt=False, out=Bpv)
                        dp = torch.where(msk, torch.ones((), device=dev), torch.gather(diag[li], 1, perm[li]))
                        D = (float(self.rel_damp) * dp.mean(dim=1))[:, None] + msk.float()
                        # (the layout pass ahead of the factor: it runs beside the scale search,
                        # which the factor's kernels, with their many registers, wait out)
                        layout_in(ids, W0[pos:pos + len(ids)], skip_out=True)
                        kernels.lowrank_factor(Bpv, D.contiguous(),
                                               out=(Hm_all[span].view(len(ids), C, nr), info[pos:pos + len(ids)]))
                        pos += len(ids)
                        at += len(ids) * C * nr
                    # ---------------------------------------------------- blocked closed form
                    if rr_ids:
                        ri = self._dev(rr_ids)
                        msk = mask[ri].bool()                               # [Br, C], solver order
                        n_own = [self.num_samples[e0 + i] for i in rr_ids]
                        nmax = max((n + 127) // 128 * 128 for n in n_own)
                        n_pad = [(n + 127) // 128 * 128 for n in n_own]
                        n_rows = self._dev(n_pad, dtype=torch.int32)
                        perm_r = perm[ri]
                        BT, Bp_r = kernels.rows_operands(
                            rows_all, self._dev([rows_at[e0 + i] for i in rr_ids]),
                            self._dev(n_own, dtype=torch.int32),
                            self._dev([(2.0 / n) ** 0.5 for n in n_own], dtype=torch.float64),
                            perm_r, mask[ri], nmax)
                        dp = torch.where(msk, torch.ones((), device=dev), torch.gather(diag[ri], 1, perm_r))
                        D = (float(self.rel_damp) * dp.mean(dim=1))[:, None] + msk.float()
                        Xr = torch.empty((len(rr_ids), C, R), dtype=torch.float32, device=dev)
                        W0r = torch.empty((len(rr_ids), C, R), dtype=self.W[job[0]].dtype, device=dev)
                        layout_in(rr_ids, W0r, Xr)
                        HmT, V, info_r = kernels.rows_factor_blocked(BT, D.contiguous(), n_rows, n_pad)
                        del BT
                        failed.append((torch.tensor([e0 + i for i in rr_ids]), info_r))
                    if lr_ids or none_ids or rr_ids:
                        lr_stream.wait_stream(search)
                        for t in (scales, qzeros, sT, zT) + tuple(x for p in parts for x in p):
                            t.record_stream(lr_stream)
                    if rr_ids:
                        q = kernels.gptq_sweep_rows_blocked(Xr, W0r, HmT, Bp_r, V, n_rows, sT[ri], zT[ri],
                                                            g_idx[ri].contiguous(), self.bits, n_pad)
                        layout_out(rr_ids, q)
                        del Xr, W0r, HmT, Bp_r, V, q
                    if ids_all:
                        failed.append((torch.tensor([e0 + i for i in ids_all]), info))
                        la = self._dev(ids_all)
                        q = kernels.gptq_sweep_lowrank_mixed(W0, Bp_all, Hm_all, ns, info, sT[la], zT[la],
                                                             g_idx[la].contiguous(), self.bits)
                        pos = 0
                        for nr, ids in buckets:
                            layout_out(ids, q[pos:pos + len(ids)])
                            pos += len(ids)
                        del W0, q, Bp_all, Hm_all
                    # experts without a single row (or with NaN rows): H = I, plain rounding
                    if none_ids:
                        ni = self._dev(none_ids)
                        for (sc_i, qz_i), i in zip(parts, job):
                            kernels.round_to_nearest(self.W[i][e0:e1], sc_i, qz_i, gs, self.bits,
                                                     out=outs[i][0][e0:e1], index=ni)

                # ---------------------------------------------------------- through the Hessian
                if dn_ids:
                    whole = len(dn_ids) == B
                    di = None if whole else self._dev(dn_ids)
                    pick = (lambda t: t) if whole else (lambda t: t[di].contiguous())
                    Bd = len(dn_ids)
                    X = torch.empty((Bd, C, R), dtype=torch.float32, device=dev)
                    # the displacement form also reads the untouched weights: the layout pass writes
                    # them a second time in their own type instead of X being copied afterwards
                    W0 = None
                    if direct and len({self.W[i].dtype for i in job}) == 1:
                        W0 = torch.empty((Bd, C, R), dtype=self.W[job[0]].dtype, device=dev)
                    # where every column block is first written by its long product, that product
                    # starts from W0 and X is not laid out at all
                    band = direct and not babai and kernels.sweep_direct_reads_band_only(Bd, C, R)
                    lazy_x = W0 is not None and band
                    # (ahead of the factorisation: see the closed forms above)
                    layout_in(dn_ids, W0, X, skip_out=lazy_x)
                    # the factorisations read their input's lower triangle in 128 x 128 blocks only
                    slots = [self._slot[e0 + i] for i in dn_ids]
                    if slots == list(range(e0, e1)) and self._Hpool.shape[0] >= e1:
                        Hp, damp = kernels.hessian_permute(self._Hpool[e0:e1], perm, mask, float(self.rel_damp),
                                                           lower_blocks=True)
                    else:
                        # the kernel takes ONE index for the Hessian, the order and the mask: the
                        # latter two are laid out by slot as well
                        si = self._dev(slots)
                        n_slots = len(self._slot_expert)
                        perm_s = torch.empty((n_slots, C), dtype=perm.dtype, device=dev)
                        mask_s = torch.empty((n_slots, C), dtype=mask.dtype, device=dev)
                        perm_s[si] = pick(perm)
                        mask_s[si] = pick(mask)
                        Hp, damp = kernels.hessian_permute(self._Hpool[:n_slots], perm_s, mask_s,
                                                           float(self.rel_damp), lower_blocks=True, index=si)
                    if babai:
                        L, info = kernels.chol_reverse_lower_batched(Hp, damp)
                        U = kernels.unit_upper_from_lower(L, info, upper_only=True)
                        del L
                    elif direct:
                        L, info = kernels.chol_reverse_lower_batched(Hp, damp)
                        # the sweep's long products read V straight from L's rows; where that covers
                        # everything beyond one block of the diagonal, only that band of V is written
                        U = kernels.unit_upper_from_lower(L, info, negate=True, upper_only=True, band=band)
                        if sparse:
                            # 1/diag(U) of the mask score (solver_sparsegptq14.cu:153) is the
                            # diagonal of the factor of H itself; U = I where it failed
                            uinv = torch.where((info != 0)[:, None], torch.ones((), device=dev),
                                               L.diagonal(dim1=1, dim2=2)).contiguous()
                        Lf = L
                        del L
                    elif sparse:
                        # un-normalised factor, rows then scaled by the rounded reciprocal of the
                        # diagonal as solver_sparsegptq14.cu:153-155 does
                        U, udiag, info = kernels.chol_inv_upper_batched(Hp, damp, normalise=False,
                                                                       upper_only=True)
                        uinv = (1.0 / udiag).contiguous()
                        U.mul_(uinv.unsqueeze(-1))
                    else:
                        U, _, info = kernels.chol_inv_upper_batched(Hp, damp, normalise=True, upper_only=True)
                    del Hp
                    failed.append((torch.tensor([e0 + i for i in dn_ids]), info))
                    main.wait_stream(search)
                    for t in (scales, qzeros, sT, zT):
                        t.record_stream(main)
                    sTd, zTd, gd = pick(sT), pick(zT), pick(g_idx)
                    M = None
                    if direct and sparse:
                        q, M = kernels.gptq_sweep_direct_batched(X, U, sTd, zTd, gd, self.bits, W0=W0,
                                                                 sparse14=True, mdiag=uinv, L=Lf, info=info,
                                                                 x_from_w0=lazy_x)
                    elif sparse:
                        q, M = kernels.gptq_sweep_batched(X, U, sTd, zTd, gd, self.bits, sparse14=True,
                                                          uinv=uinv)
                    elif direct:
                        q = kernels.gptq_sweep_direct_batched(X, U, sTd, zTd, gd, self.bits, W0=W0, L=Lf,
                                                              info=info, x_from_w0=lazy_x)
                    else:
                        q = kernels.gptq_sweep_batched(X, U, sTd, zTd, gd, self.bits)
                    del X, U, W0
                    Lf = None
                    layout_out(dn_ids, q, M)
                main.wait_stream(search)
                main.wait_stream(lr_stream)
                for t in (scales, qzeros):
                    t.record_stream(main)
                r0 = 0
                for i in job:
                    Ri = sizes[i]
                    outs[i][1][e0:e1] = scales.view(B, R, G)[:, r0:r0 + Ri].reshape(B, Ri * G)
                    outs[i][2][e0:e1] = qzeros.view(B, R, G)[:, r0:r0 + Ri].reshape(B, Ri * G)
                    r0 += Ri
        # the failure flags stay on the device until someone looks (issue_non_invertible): quantize()
        # itself never waits for the GPU after its one look at the Hessian diagonals
        self._pending_info.extend(failed)
        done = torch.cuda.Event()
        done.record()
        oldest = None
        with ExpertGroupGPTQ._in_flight_lock:
            ExpertGroupGPTQ._in_flight.append(done)
            if len(ExpertGroupGPTQ._in_flight) > ExpertGroupGPTQ.MAX_IN_FLIGHT:
                oldest = ExpertGroupGPTQ._in_flight.popleft()
        if oldest is not None:
            oldest.synchronize()
        return [tuple(o) for o in outs]
