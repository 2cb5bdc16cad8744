/*
 * forge_hip.h -- C ABI of libforge_hip.so, the MI355X (gfx950) implementation of
 * 4Bit-Forge's GPTQ calibration-and-solve kernels.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the name ends in _host.
 *   - Matrices are dense row-major; "ld" arguments are row pitches in elements.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  All work is
 *     enqueued asynchronously on it; no entry point synchronises unless it says so.
 *   - Return value: 0 on success, FORGE_ERR_* otherwise; forge_last_error() then gives
 *     a message (thread-local).  Invalid shapes are rejected BEFORE any launch.
 *   - dtype codes: FORGE_F32 = 0, FORGE_BF16 = 1.
 *
 * The first four entry points are what the reference binds through pybind11 in
 * forge/backend/cuda/kernels.cpp:92-120; the rest are batched forms of the same
 * arithmetic plus the torch library calls of forge/gptq.py that sit on the hot path.
 */
#ifndef FORGE_HIP_H
#define FORGE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FORGE_OK 0
#define FORGE_ERR_INVALID 1   /* bad argument / unsupported shape */
#define FORGE_ERR_HIP 2       /* a HIP runtime call failed */

#define FORGE_F32 0
#define FORGE_BF16 1

typedef void* forge_stream_t;

/* Library identification and error text. */
int forge_hip_abi_version(void);
const char* forge_last_error(void);

/* Optional per-kernel timing, for benchmarks: while enabled every kernel launch of this
 * library is bracketed by two HIP events on its stream.  _enable(on) clears all records;
 * _collect() waits for the bracketed launches and returns the number of distinct kernel
 * names (negative on error); _get(i) returns name, launches, summed duration (ms) and
 * summed algorithmic work of entry i (work_kind 0 = flops, 1 = HBM bytes).  No
 * counterpart in the reference. */
int forge_kernel_timing_enable(int on);
int forge_kernel_timing_collect(void);
int forge_kernel_timing_get(int index, char* name, int name_cap, int64_t* launches,
                            double* total_ms, double* work, int* work_kind);

/* Library-wide settings; no counterpart in the reference.  Each starts from an environment
 * variable that is read once, when the library is loaded, and is changed afterwards only
 * through forge_set_option (an atomic store; a launch reads the value it finds).
 *   "sweep_schedule"        FORGE_SWEEP_SCHEDULE=left|right   0 (default): by tile count,
 *                           1: left-looking, 2: right-looking -- see forge_gptq_sweep_batched
 *   "fp32_blocked_sum"      FORGE_FP32_BLOCKED_SUM=1          1: the factorisation's and the direct
 *                           sweep's blocked sums stay on the fp32 matrix instruction
 *   "sweep_update_products" FORGE_SWEEP_UPDATE_PRODUCTS=n     how the block updates of
 *                           forge_gptq_sweep_direct_batched form an fp32 product on the 16-bit
 *                           matrix pipe.  2: two fp16 halves per operand, three products,
 *                           fp32-grade (columns of V scaled by powers of two from their largest
 *                           entry, rows of displacements from a running maximum).  bf16 piece
 *                           products: 6 (three truncated pieces, every product of weight
 *                           >= 2^-16: fp32-grade), 3 (two pieces per operand, each rounded to
 *                           nearest, products (2,1) (1,2) (1,1), within ~2^-17 of the fp32
 *                           product), 4 (adds (2,2)), 1 (operands rounded to bf16; for
 *                           measurements: it moves 2-16 % of the codes).  0 (default): 3 from
 *                           C = 4096 on, 2 below
 *   "factor_pieces"         FORGE_FACTOR_PIECES=1             0 (default): where only the factor of H is
 *                           computed (forge_chol_reverse_lower_batched, C a multiple of 128) the
 *                           trailing updates take two fp16 halves of every operand, each column
 *                           scaled by a power of two from its diagonal entry, and three
 *                           products (fp32-grade: the halves hold 22+ bits); 1: three bf16 thirds
 *                           and six products everywhere, as forge_chol_inv_upper_batched always does
 *   "mse_reference_quantiser" FORGE_MSE_REFERENCE_QUANTISER=1   how the shrink search (forge_quant_grid,
 *                           forge_mse_scale_groups_packed) finds the level of a weight inside the
 *                           candidate's loss.  0 (default): rint(x * rcp) clamped to [-zero, maxq - zero],
 *                           one instruction less per weight and candidate; it picks the other of two
 *                           levels only where the reference's single rounding of x * rcp + zero lands on
 *                           a half-integer that x * rcp is not on, i.e. where both levels are equally
 *                           far from x to one ulp (it moves the loss by ~1e-7 of one term).
 *                           1: clamp(rint(fma(x, rcp, zero)), 0, maxq) - zero, quant_grid.cu:160-163
 *                           literally (12 % slower)
 * forge_set_option returns FORGE_ERR_INVALID for an unknown name or a value out of range;
 * forge_get_option returns -1 for an unknown name. */
int forge_set_option(const char* name, int64_t value);
int64_t forge_get_option(const char* name);

/* ------------------------------------------------------------------ quant grid */

/* Replaces kernels.build_group_meta_packed (kernels.cpp:93-97, quant_grid.cu:186-224).
 * X [RG, gs] f32.  Writes scales[RG], qzeros[RG] (f32).  Any gs >= 1. */
int forge_build_group_meta_packed(const float* X, int64_t RG, int64_t gs, int bits,
                                  int symmetric, float* scales, float* qzeros,
                                  forge_stream_t stream);

/* Replaces kernels.mse_scale_groups_packed (kernels.cpp:98-102, quant_grid.cu:227-287).
 * Overwrites scales/qzeros in place.  gs must be 32, 64 or 128 (as the reference). */
int forge_mse_scale_groups_packed(const float* X, float* scales, float* qzeros,
                                  const float* candidates, int64_t RG, int64_t gs, int64_t P,
                                  float norm, int bits, int symmetric, forge_stream_t stream);

/* Fused form of GPTQ._quant_grid (gptq.py:180-227) for `batch` weight matrices
 * W[b] = W + b*w_stride, each [R, C] with row pitch ldw, dtype w_dtype: contiguous
 * gs-wide column groups, the last one zero padded; min/max grid, then (if mse != 0)
 * the shrink search over `candidates`[P].  scales/qzeros: [batch, R*G] f32, index
 * r*G + g, G = ceil(C/gs).  gs in {32,64,128}. */
int forge_quant_grid(const void* W, int w_dtype, int64_t batch, int64_t w_stride, int64_t R,
                     int64_t C, int64_t ldw, int64_t gs, int bits, int symmetric, int mse,
                     const float* candidates, int64_t P, float norm, float* scales,
                     float* qzeros, forge_stream_t stream);

/* ------------------------------------------------------------------ column sweep */

/* Replaces kernels.gptq_solver (kernels.cpp:104-108, solver.cu:99-154).
 * W [C, R] f32 contiguous: solver-order columns x rows; overwritten with the dequantised
 * weights.  U [C, C] f32: row-normalised upper factor.  scales/qzeros [C, R] f32 per
 * element.  qweight [C, R] u8 receives codes 0..2^bits-1.  E [C, R] f32 is workspace
 * (receives the per-column errors). */
int forge_gptq_solver(float* W, const float* U, const float* scales, const float* qzeros,
                      int bits, int64_t C, int64_t R, uint8_t* qweight, float* E,
                      forge_stream_t stream);

/* Replaces kernels.sparsegptq14_solver (kernels.cpp:110-120,
 * solver_sparsegptq14.cu:142-200).  U holds the UN-normalised upper factor and is
 * row-normalised in place, as the reference does to its caller's tensor.
 * M [ceil(C/32), R] u32: bit i of word w <-> solver column 32*w+i kept.
 * uinv [C] f32 workspace (1/diag(U)). */
int forge_sparsegptq14_solver(float* W, float* U, const float* scales, const float* qzeros,
                              int bits, int64_t C, int64_t R, uint8_t* qweight, uint32_t* M,
                              float* E, float* uinv, forge_stream_t stream);

/* Batched sweep with per-group metadata (no [C,R] expansion, gptq.py:251-252 folded in).
 * For b in [0,batch): X[b] [C, R] f32 workspace holding the permuted transposed weight on
 * entry and the per-column errors on exit; U[b] [C, C]; scalesT/qzerosT[b] [G, R] f32
 * (group-major); g_idx[b] [C] int32 = group of solver column c; qweight[b] [C, R] u8.
 * sparse14 != 0 selects the 1:4 joint solve (then M[b] [ceil(C/32), R] u32 and
 * uinv[b] [C] must be given and U must already be row-normalised).
 * Schedule: with at least 128 tiles of 128 rows (batch * ceil(R/128)) each column block is
 * brought up to date by one long product over all earlier columns just before it is swept;
 * with fewer, every finished block is pushed into all later columns at once (more tiles per
 * launch).  Same fma chain per element either way, identical results.  The option
 * "sweep_schedule" forces one of them. */
int forge_gptq_sweep_batched(float* X, const float* U, const float* scalesT,
                             const float* qzerosT, const int32_t* g_idx, uint8_t* qweight,
                             uint32_t* M, const float* uinv, int64_t batch, int64_t C,
                             int64_t R, int64_t G, int bits, int sparse14,
                             forge_stream_t stream);

/* The same sweep fed by the factor of H itself instead of the factor of its inverse, so that
 * the second half of gptq.py:160-166 (cholesky_inverse and the second Cholesky) is never
 * computed.  With H + damp*I = M M^T (M upper; M = L^T of forge_chol_reverse_lower_batched)
 * and N[t][k] = M[t][k] / M[k][k], N is the inverse of the unit matrix that
 * forge_gptq_sweep_batched takes, and the value column k has when solver.cu:85-94 reaches it
 * equals w0[k] + sum_{t<k} d[t] N[t][k] with d[t] = w0[t] - deq[t], the column's original
 * weight minus what it was rounded to.  V[b] [C, C] holds -N above the diagonal
 * (forge_unit_upper_from_lower with flag 2); W0[b] [C, R] is an untouched copy of X[b] as
 * passed in.  Same quantiser and chain order as forge_gptq_sweep_batched; codes are equal in
 * exact arithmetic and differ in fp32 only where a value sits within rounding error of a
 * tie.  X holds the displacements d on exit.
 * sparse14 != 0: the 1:4 joint solve (solver_sparsegptq14.cu:29-200) in the same form; then
 * M[b] [ceil(C/32), R] u32 receives the keep-masks and mdiag[b] [C] must hold the diagonal of
 * L (= 1/diag(U) of the reference's un-normalised factor, the weight of the mask score;
 * 1 where the factorisation failed).  A pruned column hands on its whole original weight; the
 * values of the three columns the score looks ahead at are rebuilt from V's 4 x 4 diagonal block.
 * ws == NULL: the update of a column block by all earlier columns is one fp32 fused
 * multiply-add per earlier column, in ascending order (the chain of solver.cu:91-94 carried
 * across blocks), reproducible bit for bit on a CPU.  With a workspace of
 * forge_gptq_sweep_direct_workspace_bytes(batch, C, R) bytes that update is summed from
 * 16-bit pieces of the fp32 operands on the fp16 / bf16 matrix pipe wherever a block is a full
 * 128 x 128 tile and the left-looking schedule applies (see "sweep_update_products" under
 * forge_set_option: different rounding than the chain, faster). */
int forge_gptq_sweep_direct_batched(float* X, const float* W0, const float* V,
                                    const float* scalesT, const float* qzerosT,
                                    const int32_t* g_idx, uint8_t* qweight, uint32_t* M,
                                    const float* mdiag, int64_t batch, int64_t C, int64_t R,
                                    int64_t G, int bits, int sparse14, void* ws,
                                    int64_t ws_bytes, forge_stream_t stream);
int64_t forge_gptq_sweep_direct_workspace_bytes(int64_t batch, int64_t C, int64_t R);
/* The same with the untouched weights W0 in f32 (w0_dtype = FORGE_F32) or in bf16 (FORGE_BF16:
 * exact when the layer's weights are bf16, and half the bytes to read);
 * forge_weight_to_solver_order_pair writes X and W0 in one pass.
 * L, info (may be NULL): the lower factor that V was made from
 * (forge_chol_reverse_lower_batched) and its failure flags.  With them the long block updates
 * take their V operand straight from the rows of L, the same numbers, and when
 * forge_gptq_sweep_direct_reads_band_only(batch, C, R) returns 1 (left-looking schedule, whole
 * 128 x 128 tiles, workspace given) V is read only within one 128-column block of its diagonal:
 * forge_unit_upper_from_lower with bit 3 then suffices (the answer depends on the library's
 * options: do not change them between the query and the sweep).
 * x_from_w0 != 0 (only where that function returns 1; an error otherwise): X need not hold the
 * weights on entry -- forge_weight_to_solver_order_pair may be called with Xout = NULL -- since
 * every column block is then first written by its long product, which starts from W0. */
int forge_gptq_sweep_direct_reads_band_only(int64_t batch, int64_t C, int64_t R);
int forge_gptq_sweep_direct_batched_w0(float* X, const void* W0, int w0_dtype, int x_from_w0,
                                       const float* V, const float* L, const int32_t* info,
                                       const float* scalesT, const float* qzerosT,
                                       const int32_t* g_idx, uint8_t* qweight, uint32_t* M,
                                       const float* mdiag, int64_t batch, int64_t C, int64_t R,
                                       int64_t G, int bits, int sparse14, void* ws,
                                       int64_t ws_bytes, forge_stream_t stream);

/* GPTQ.quantize for a layer that saw n <= 128 calibration rows (gptq.py:128-166 with
 * solver.cu:9-154), without the C x C Hessian.  Such a layer's damped, pruned, permuted Hessian
 * (gptq.py:97-119,145-153) is  D + Bp^T Bp  with  Bp[k][j] = sqrt(2/n) x_j[perm[k]]  (0 in pruned
 * and all-zero-weight columns) and D[k] = damp (+ 1 in those columns), and every number the sweep
 * takes from the factor of that matrix is an n-term dot product:
 *   forge_lowrank_factor: Bp [batch][C][n] f32 (rows beyond the layer's own count zero), D
 *     [batch][C] f32 -> Hm [batch][C][n] f32 with  Hm[k] . Bp[t] = M[k][t] / M[k][k]  (t < k) for the lower factor
 *     M of forge_chol_reverse_lower_batched; info[b] = 1 where a pivot is not positive (or NaN).
 *     Recurrence in float64, 128-column blocks side by side; ws: device workspace of
 *     forge_lowrank_workspace_bytes(batch, C, n), 16-byte aligned.
 *   forge_gptq_sweep_lowrank: W0 [batch][C][R] (w0_dtype f32 or bf16, solver order, pruned columns
 *     zero: forge_weight_to_solver_order_pair's W0out), scalesT/qzerosT [batch][G][R], g_idx
 *     [batch][C] -> qweight [batch][C][R] u8.  Column k of a row is quantised at
 *     w0_k + Hm[k] . a  and then adds (w0_k - deq_k) Bp[k] to the row's n-vector a: the values
 *     forge_gptq_sweep_direct_batched reaches in exact arithmetic, the reference's quantiser
 *     (solver.cu:9-23).  Matrices with info != 0 are swept uncoupled (gptq.py:172-175).
 * n is 4, 16, 32, 64 or 128 (pad with zero rows), C % 16 == 0. */
/* GPTQ.quantize for a layer that saw NO calibration rows: H = I (gptq.py:97-99), its factor is
 * the identity, nothing couples the columns and the sweep of solver.cu:9-154 is its quantiser
 * (solver.cu:9-23) applied to every weight.  W [batch][R][C] (w_dtype f32 or bf16, row pitch ldw,
 * batch stride w_stride, layer layout), scales/qzeros [batch][R*G] (index r*G + c/gs) ->
 * qweight [batch][R][C] u8, layer layout: no permutation, no layout pass.  index (device, int64
 * [batch], may be NULL): launch entry b works on matrix index[b] of all three arrays, so that a
 * scattered subset of a stack is handled in place by one launch. */
int forge_round_to_nearest(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                           const int64_t* index, const float* scales, const float* qzeros,
                           uint8_t* qweight, int64_t batch, int64_t R, int64_t C, int64_t gs, int bits,
                           forge_stream_t stream);
int forge_lowrank_factor(const float* Bp, const float* D, float* Hm, int32_t* info, int64_t batch,
                         int64_t C, int64_t n, void* ws, int64_t ws_bytes, forge_stream_t stream);
int64_t forge_lowrank_workspace_bytes(int64_t batch, int64_t C, int64_t n);
/* forge_gptq_sweep_lowrank for matrices of different n in ONE launch (each of the three sizes
 * alone leaves most of the GPU idle): n_host[b] in {4, 16, 32, 64, 128} (host array), and matrix b's
 * vectors start C * (n_host[0] + ... + n_host[b-1]) floats into Bp and into Hm, i.e. the per-size
 * [batch_n][C][n] arrays laid end to end in batch order.  Everything else as above. */
int forge_gptq_sweep_lowrank_mixed(const void* W0, int w0_dtype, const float* Bp, const float* Hm,
                                   const int64_t* n_host, const int32_t* info, const float* scalesT,
                                   const float* qzerosT, const int32_t* g_idx, uint8_t* qweight,
                                   int64_t batch, int64_t C, int64_t R, int64_t G, int bits,
                                   forge_stream_t stream);
int forge_gptq_sweep_lowrank(const void* W0, int w0_dtype, const float* Bp, const float* Hm,
                             const int32_t* info, const float* scalesT, const float* qzerosT,
                             const int32_t* g_idx, uint8_t* qweight, int64_t batch, int64_t C,
                             int64_t R, int64_t G, int bits, int64_t n, forge_stream_t stream);

/* Front end of the two closed forms (layers that saw fewer calibration rows than they have
 * features): their operands straight from the rows the layer saw, without the Hessian that the
 * reference sums from them (forge/gptq.py:61-80: H = (2/n) X^T X as the running mean of
 * X^T (alpha X)).  rows [*, C] (x_dtype FORGE_BF16 or FORGE_F32, row pitch C): matrix b owns the
 * rows row0[b] .. row0[b] + n[b] - 1.  row0 [batch] int64, n [batch] int32, device memory.
 *
 * forge_rows_operands: root [batch] f64 (sqrt(2 / n[b]) as the caller rounds it), perm
 * [batch, C] int64 (solver column j is feature perm[b][j]), dead [batch, C] u8 in solver order
 * (pruned columns, gptq.py:145-149, read as zero).
 *   BT[b][r][j] = Bp[b][j][r] = (float)((double)rows[row0[b] + r][perm[b][j]] * root[b])
 * for r < n[b] and dead[b][j] == 0, else 0; BT [batch, nmax, C] f32 (may be NULL), Bp
 * [batch, C, nmax] f32, every element written.
 *
 * forge_rows_diagonal: out[b][c] = (float)(alpha[b] * sum_r (double)rows[row0[b] + r][c]^2),
 * the diagonal of H summed in float64 and rounded once (what the activation order and the
 * damping are taken from, gptq.py:100-108,151-153).  alpha [batch] f64, out [batch, C] f32. */
int forge_rows_operands(const void* rows, int x_dtype, const int64_t* row0, const int32_t* n,
                        const double* root, const int64_t* perm, const uint8_t* dead, float* BT,
                        float* Bp, int64_t batch, int64_t C, int64_t nmax, forge_stream_t stream);
int forge_rows_diagonal(const void* rows, int x_dtype, const int64_t* row0, const int32_t* n,
                        const double* alpha, float* out, int64_t batch, int64_t C,
                        forge_stream_t stream);

/* GPTQ.quantize for a layer that saw 129 .. ~1000 calibration rows, fewer than a fraction of its
 * input features (gptq.py:128-166 with solver.cu:9-154), again without the C x C Hessian: the
 * closed forms of forge_lowrank_factor as 128-column blocked products on the matrix pipe.
 *   forge_rows_factor_blocked: BT [batch][nmax][C] f32 = the rows of forge_lowrank_factor's Bp,
 *     transposed (row j = sqrt(2/n) x_j in solver order, 0 in pruned columns; zero rows beyond a
 *     layer's own count), D [batch][C], n_rows [batch] int32 on the DEVICE = each matrix's own row
 *     count rounded up to a multiple of 128 (<= nmax; products skip what lies beyond it),
 *     n_rows_host the same numbers on the host (may be NULL: only the work figures of the
 *     forge_kernel_timing_* records use it, which otherwise count every matrix as nmax rows)
 *     -> HmT [batch][nmax][C] (HmT[j][k] = entry j of h_k: h_k . b_t = M[k][t] / M[k][k] for t
 *     left of k's 128-column block), V [batch][C][128] (V[t][k - c0] = -M[k][t] / M[k][k] for t < k
 *     inside the block that starts at c0; 0 elsewhere) and info [batch] (1-based position of a pivot that is not
 *     positive; that matrix's HmT and V are then zero: swept uncoupled, gptq.py:172-175).
 *     fp32; C a multiple of 128, nmax a multiple of 128; ws of forge_rows_factor_workspace_bytes,
 *     256-byte aligned.
 *   forge_gptq_sweep_rows_blocked: X [batch][C][R] f32 holding the weights in solver order on
 *     entry and the displacements on exit, W0 the same weights untouched (f32 or bf16), Bp
 *     [batch][C][nmax] (the transpose of BT) -> qweight [batch][C][R] u8.  Before a block is swept
 *     its columns receive Hm_J A, after it A += B_J^T (displacements), A [nmax][R] per matrix in
 *     ws (forge_gptq_sweep_rows_workspace_bytes); the block itself runs the in-block chain of
 *     forge_gptq_sweep_direct_batched on V.  R a multiple of 128.
 * No counterpart in the reference, which forms and factors the C x C matrix whatever the number
 * of rows. */
int forge_rows_factor_blocked(const float* BT, const float* D, const int32_t* n_rows,
                              const int32_t* n_rows_host, float* HmT, float* V, int32_t* info,
                              int64_t batch, int64_t C, int64_t nmax, void* ws, int64_t ws_bytes,
                              forge_stream_t stream);
int64_t forge_rows_factor_workspace_bytes(int64_t batch, int64_t C, int64_t nmax);
int forge_gptq_sweep_rows_blocked(float* X, const void* W0, int w0_dtype, const float* HmT,
                                  const float* Bp, const float* V, const int32_t* n_rows,
                                  const int32_t* n_rows_host, const float* scalesT,
                                  const float* qzerosT, const int32_t* g_idx,
                                  uint8_t* qweight, int64_t batch, int64_t C, int64_t R, int64_t G,
                                  int bits, int64_t nmax, void* ws, int64_t ws_bytes,
                                  forge_stream_t stream);
int64_t forge_gptq_sweep_rows_workspace_bytes(int64_t batch, int64_t R, int64_t nmax);

/* Replaces kernels.babai_solver (kernels.cpp:46-56,147-149; solver_babai.cu:123-322).
 * W [C, R] f32 solver-order weights (read only; the reference also overwrites its private
 * copy with the dequantised values), A [C, C] f32 upper Cholesky factor of H (H = A^T A),
 * scales/qzeros [R*G] f32 (index r*G + g), g_idx [C] int32 group of solver column c (null:
 * c / group_size), qweight [C, R] u8.  Columns are quantised from the last to the first with
 * the reference's quantiser and fused multiply-adds; every element receives its updates as
 * one fma chain in that order (the reference applies those of other 32-column blocks
 * through an SGEMM whose summation order is not defined).  The block_size argument of the
 * reference has no effect on such a chain and is not taken.  ws: forge_babai_workspace_bytes. */
int forge_babai_solver(const float* W, const float* A, const float* scales, const float* qzeros,
                       const int32_t* g_idx, int64_t group_size, int bits, int64_t C, int64_t R,
                       int64_t G, uint8_t* qweight, void* ws, int64_t ws_bytes,
                       forge_stream_t stream);
int64_t forge_babai_workspace_bytes(int64_t C, int64_t R, int64_t G);

/* ------------------------------------------------------------------ Hessian */

/* Grouped ragged rank-k update, the batched form of GPTQ.update (gptq.py:61-80):
 * for each group e in [0, n_groups): rows offsets_host[e] .. offsets_host[e+1] of X
 * ([*, C], pitch ldx, dtype x_dtype) are that expert's tokens, and
 *   H[e] <- beta[e]*H[e] + alpha[e] * X_e^T X_e      (H[e] = H + e*C*C, f32 [C,C], full)
 * alpha_host/beta_host [n_groups] are host arrays (the caller owns the running-mean
 * bookkeeping); H[e] is not read when beta[e] == 0.  Groups with zero rows are left
 * untouched.  bf16 inputs use bf16 MFMA with fp32 accumulation (products exact); f32
 * inputs use f32 MFMA.  The diagonal entries, which decide the activation order
 * (gptq.py:107-110), are summed in float64 and rounded to f32 once per call.  ws: device
 * workspace of forge_hessian_workspace_bytes(total rows, n_groups, C, x_dtype).  The host
 * arrays are consumed before the call returns; nothing waits for the stream (the group
 * table travels through pinned memory that the library keeps). */
int forge_hessian_update_grouped(const void* X, int x_dtype, int64_t ldx, int64_t C,
                                 const int64_t* offsets_host, int64_t n_groups,
                                 const float* alpha_host, const float* beta_host, float* H,
                                 void* ws, int64_t ws_bytes, forge_stream_t stream);
int64_t forge_hessian_workspace_bytes(int64_t total_rows, int64_t n_groups, int64_t C,
                                      int x_dtype);
/* The same update with each group's rows given as a range of its own, rows row0_host[e] ..
 * row0_host[e] + n_host[e] - 1 of X: groups need not follow one another, so that a caller can
 * leave out the experts it handles by forge_lowrank_factor (n_host[e] = 0 leaves H[e] untouched)
 * while their rows stay where they are in X.  total_rows of the workspace query = sum of n_host. */
int forge_hessian_update_ranges(const void* X, int x_dtype, int64_t ldx, int64_t C,
                                const int64_t* row0_host, const int64_t* n_host, int64_t n_groups,
                                const float* alpha_host, const float* beta_host, float* H, void* ws,
                                int64_t ws_bytes, forge_stream_t stream);

/* GPTQ.update for ONE matrix without any allocation: H <- beta*H + alpha * X^T X for the
 * n_rows rows of X ([n_rows, C], pitch ldx, dtype x_dtype), the same kernels and the same
 * bits as forge_hessian_update_grouped with a single group.  No counterpart in the
 * reference; it is for callers that cannot allocate or bring a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  The group table, the
 * float64 diagonal and the bf16 operand panels live in a device array of the library's own
 * (32 MiB + 64.25 KiB per GPU, held until the process ends), which fixes the limits:
 * C <= 16384 and n_rows <= forge_hessian_update_static_max_rows(C, x_dtype) (bf16: the
 * panels, ceil(n_rows/16) * ceil(C/32) KiB, must fit in 32 MiB -- 2336 rows at C = 7168,
 * 8192 at C = 2048; f32: no limit on rows); larger inputs are rejected with
 * FORGE_ERR_INVALID before any launch.  Calls no hipMalloc/hipFree/hipHostMalloc and creates
 * no events (its launches never appear in the forge_kernel_timing_* records).  Every call on
 * a GPU uses that GPU's one array: calls that overlap on one GPU (different streams or
 * threads) race; calls on one stream are ordered.  Nothing in the array has to be cleared
 * between calls: every byte a call reads it has written first. */
int forge_hessian_update_static(const void* X, int x_dtype, int64_t ldx, int64_t n_rows,
                                int64_t C, float alpha, float beta, float* H,
                                forge_stream_t stream);
int64_t forge_hessian_update_static_max_rows(int64_t C, int x_dtype);

/* ------------------------------------------------------------------ factorisation */

/* Batched form of GPTQ._h_factor's torch.linalg calls (gptq.py:152-175):
 * for each b: A = H[b] + damp[b]*I (lower triangle of H[b] read), U0 = upper Cholesky
 * factor of inv(A); writes U[b] = U0 / diag(U0)[:,None] (normalise & 1) or U0, upper
 * triangle + zeroed lower; udiag[b] [C] receives diag(U0).  normalise & 2: the caller reads
 * the upper triangle only (the sweeps do) and the part of U[b] left of the 128x128 diagonal
 * blocks is left unwritten.  info[b] (int32) is 0 on
 * success or the 1-based index of the first non-positive pivot, in which case U[b] = I.
 * H[b] is destroyed (used as workspace).  ws: workspace of forge_chol_workspace_bytes
 * (128x128 inverse diagonal blocks, plus 1540 bytes per column and matrix for the 16-bit
 * pieces of two panels and the column scales), 256-byte aligned.
 * When C is a multiple of 128 the trailing updates are computed from three bf16 pieces per
 * fp32 operand on the bf16 matrix pipe (fp32-grade accuracy; not bit-identical to the fp32
 * update).  The option "fp32_blocked_sum" selects the fp32 update. */
int forge_chol_inv_upper_batched(float* H, const float* damp, float* U, float* udiag,
                                 int32_t* info, int64_t batch, int64_t C, int normalise,
                                 void* ws, int64_t ws_bytes, forge_stream_t stream);
int64_t forge_chol_workspace_bytes(int64_t batch, int64_t C);

/* The factor that the Babai branch of GPTQ._h_factor needs (gptq.py:157-158,
 * torch.linalg.cholesky_ex(H, upper=True)), in the index order of the sweep that consumes it:
 * for each b, A = H[b] + damp[b]*I is factored as A = L^T L with L LOWER triangular
 * (elimination from the last row upwards), and L is left in the lower triangle of H[b]
 * (the strict upper triangle of H[b] is destroyed).  Reversing both index orders of H gives
 * the reference's upper factor: chol(H_ref, upper)[i][j] = L[C-1-i][C-1-j] for
 * H[i][j] = H_ref[C-1-i][C-1-j].  info and ws as for forge_chol_inv_upper_batched. */
int forge_chol_reverse_lower_batched(float* H, const float* damp, int32_t* info, int64_t batch,
                                     int64_t C, void* ws, int64_t ws_bytes, forge_stream_t stream);

/* U[b][t][k] = L[b][k][t] * (1 / L[b][k][k]) for k > t, 1 on the diagonal, 0 below it: the
 * coefficients alpha = A[i][t] * invD[i] of solver_babai.cu:133-141,232-236 arranged as the unit
 * upper matrix of a forward sweep.  U[b] = I where info[b] != 0 (info may be null).
 * flipped_upper bit 0: L is given as the reference's upper factor A instead,
 * L[k][t] = A[C-1-k][C-1-t].  Bit 1: the entries above the diagonal are negated (the matrix V
 * of forge_gptq_sweep_direct_batched).  Bit 2: 32 x 32 tiles that lie wholly below the
 * diagonal are left unwritten (no sweep reads them).  Bit 3: only the columns of each row's own
 * 128-column block and of the next block are written (all that
 * forge_gptq_sweep_direct_batched_w0 reads when it is given L and
 * forge_gptq_sweep_direct_reads_band_only says so).  L and U must not overlap. */
int forge_unit_upper_from_lower(const float* L, const int32_t* info, float* U, int64_t batch,
                                int64_t C, int flipped_upper, forge_stream_t stream);

/* Fused gather for GPTQ._prep/_h_factor (gptq.py:100-117,145-154): for each b builds
 * Hp[b][i][j] = H[b][perm[i]][perm[j]] with rows/cols flagged in dead[b] (u8, in PERMUTED
 * position) zeroed and their diagonal set to 1; writes damp[b] = rel_damp * mean(diag). */
int forge_hessian_permute(const float* H, const int64_t* perm, const uint8_t* dead, float* Hp,
                          float* damp, float rel_damp, int64_t batch, int64_t C,
                          forge_stream_t stream);
/* The same, but in row i only the columns up to the end of the row's own 128-column block are
 * written (three quarters of the bytes): all that forge_chol_reverse_lower_batched and
 * forge_chol_inv_upper_batched read of their input. */
int forge_hessian_permute_lower(const float* H, const int64_t* perm, const uint8_t* dead, float* Hp,
                                float* damp, float rel_damp, int64_t batch, int64_t C,
                                forge_stream_t stream);
/* The same for a scattered subset of a larger stack in one launch: output b (Hp[b], damp[b]) is
 * made from matrix index[b] of H and rows index[b] of perm and dead (index: device, int64
 * [batch]); lower_blocks != 0 as forge_hessian_permute_lower. */
int forge_hessian_permute_gather(const float* H, const int64_t* index, const int64_t* perm,
                                 const uint8_t* dead, float* Hp, float* damp, float rel_damp,
                                 int64_t batch, int64_t C, int lower_blocks, forge_stream_t stream);

/* ------------------------------------------------------------------ layout helpers */

/* Xout[b][perm_inv[b][c]][r] = (f32) W[b][r][c]: the W.T[perm] of gptq.py:133 written as a
 * scatter of whole rows (perm_inv = argsort(perm), gptq.py:113).  W of dtype w_dtype
 * [R, C] pitch ldw; columns flagged in dead[b] (u8 [C], original order, may be NULL) read
 * as zero (gptq.py:115). */
int forge_weight_to_solver_order(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                 const int64_t* perm_inv, const uint8_t* dead, float* Xout,
                                 int64_t batch, int64_t R, int64_t C, forge_stream_t stream);

/* qout[b][r][c] = qin[b][perm_inv[b][c]][r]: back to [R, C] in original column order
 * (qweight[perm_inv].T of gptq.py:139). */
int forge_codes_to_layer_order(const uint8_t* qin, const int64_t* perm_inv, uint8_t* qout,
                               int64_t batch, int64_t R, int64_t C, forge_stream_t stream);

/* The two layout passes on a band of rows of a taller solver-order matrix: weight stacks that
 * share one factor (gate_proj and up_proj, gptq.py:36,84-94) are swept as ONE matrix whose
 * rows are the stacks' rows one after the other, without first concatenating the stacks.
 * _strided forms: Xout / qin point at the band's first row inside the tall matrix, ldo / ldi is
 * the tall matrix's row pitch in elements (>= R) and o_stride / i_stride its batch stride;
 * everything else as above (the plain forms are the case ldo = R, o_stride = C*R). */
int forge_weight_to_solver_order_strided(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                         const int64_t* perm_inv, const uint8_t* dead, float* Xout,
                                         int64_t ldo, int64_t o_stride, int64_t batch, int64_t R,
                                         int64_t C, forge_stream_t stream);
/* _pair: additionally writes W0out (may be NULL), the same matrix in the weights' own type
 * (w_dtype) with the same pitches in elements: the untouched copy that
 * forge_gptq_sweep_direct_batched_w0 reads beside the values it updates, produced in the pass
 * that lays X out instead of by a copy of X afterwards.  Xout may be NULL when only W0out is
 * wanted. */
int forge_weight_to_solver_order_pair(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                      const int64_t* perm_inv, const uint8_t* dead, float* Xout,
                                      void* W0out, int64_t ldo, int64_t o_stride, int64_t batch,
                                      int64_t R, int64_t C, forge_stream_t stream);
int forge_codes_to_layer_order_strided(const uint8_t* qin, int64_t ldi, int64_t i_stride,
                                       const int64_t* perm_inv, uint8_t* qout, int64_t batch,
                                       int64_t R, int64_t C, forge_stream_t stream);
/* The two strided layout passes for a scattered subset of a larger stack in one launch (index:
 * device, int64 [batch]).  _gather: output b (Xout / W0out + b * o_stride) is made from matrix
 * index[b] of W and rows index[b] of perm_inv and dead.  _scatter: input b (qin + b * i_stride)
 * goes to matrix index[b] of qout, through row index[b] of perm_inv. */
int forge_weight_to_solver_order_gather(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                        const int64_t* index, const int64_t* perm_inv,
                                        const uint8_t* dead, float* Xout, void* W0out, int64_t ldo,
                                        int64_t o_stride, int64_t batch, int64_t R, int64_t C,
                                        forge_stream_t stream);
int forge_codes_to_layer_order_scatter(const uint8_t* qin, int64_t ldi, int64_t i_stride,
                                       const int64_t* index, const int64_t* perm_inv, uint8_t* qout,
                                       int64_t batch, int64_t R, int64_t C, forge_stream_t stream);

/* Nibble packing of [R, C] u8 codes into the compressed-tensors "pack-quantized" int32
 * layout consumed by pack_quantized.py:279-313: value = code - zero + 8 (offset binary of
 * the zero-shifted int4), eight values per int32 along C, lowest nibble first.
 * qzeros [R*G] f32 (NULL = 8 for every group).  packed [R, ceil(C/8)] int32. */
int forge_pack_int4(const uint8_t* codes, const float* qzeros, int32_t* packed, int64_t R,
                    int64_t C, int64_t gs, forge_stream_t stream);

/* ------------------------------------------------------------------ formats around the path */

/* DeepSeek-style fp8 checkpoint weights -> bf16/f32 (forge/utils/io.py:533-563,863-872):
 * out[b][r][c] = (f32) w[b][r][c] * scale_inv[b][r / so][c / si], w holding OCP float8
 * e4m3fn bytes [batch, O, I], scale_inv [batch, ceil(O/so), ceil(I/si)] f32; the product is
 * rounded to out_dtype (FORGE_BF16: round to nearest even, or FORGE_F32). */
int forge_fp8_e4m3_block_dequant(const uint8_t* w, const float* scale_inv, void* out,
                                 int out_dtype, int64_t batch, int64_t O, int64_t I, int64_t so,
                                 int64_t si, forge_stream_t stream);

/* Replaces kernels.pack_sparsegptq14_to_u64x2 (kernels.cpp:122-126,
 * bitpacking_sparsegptq14.cu:58-172): qweight_rc [R, C] u8 codes, M [ceil(C/32), R] u32 keep
 * masks, scales [ceil(C/32), R] f32 -> out [ceil(ceil(C/32)/2), R, 2] u64, each
 * bf16(scale) << 48 | idx16 << 32 | qw32. */
int forge_pack_sparsegptq14_to_u64x2(const uint8_t* qweight_rc, const uint32_t* M,
                                     const float* scales, uint64_t* out, int64_t R, int64_t C,
                                     forge_stream_t stream);

/* Quantised weight back to the layer's dtype, for the re-forward that feeds the next
 * block's calibration (dequantize_forge_full, forge/utils/engine.py:71-97):
 * out[b][r][c] = ((f32) q[b][r][c] - qzeros[b][r*G + c/gs]) * scales[b][r*G + c/gs], a
 * subtraction and a multiplication in f32, then rounded to out_dtype (FORGE_BF16: nearest
 * even, or FORGE_F32).  q [batch, R, C] u8, scales/qzeros [batch, R*G] f32, G = ceil(C/gs). */
int forge_dequantize_groups(const uint8_t* q, const float* scales, const float* qzeros, void* out,
                            int out_dtype, int64_t batch, int64_t R, int64_t C, int64_t gs,
                            forge_stream_t stream);

/* The front of the Hessian update for fused-expert layers (the per-expert gather of
 * forge/utils/engine.py:229-238: x_e = x[tok_idx]; x_e_w = x_e * w[:, None]):
 * out[i][:] = X[row_idx[i]][:] * weight[i], the product rounded to x_dtype (weight NULL =
 * plain gather).  X [T, C] with row pitch ldx, row_idx [N] int64 (rows already grouped by
 * expert by the caller), weight [N] in x_dtype, out [N, C] contiguous.  Indices outside
 * [0, T) are an error of the caller; they are not checked on the device. */
int forge_gather_scaled_rows(const void* X, int x_dtype, int64_t ldx, int64_t T, int64_t C,
                             const int64_t* row_idx, const void* weight, void* out, int64_t N,
                             forge_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FORGE_HIP_H */
