/*
 * CPU oracle for the GPTQ calibration-and-solve kernels of 4Bit-Forge.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in scalar C, the arithmetic of the
 * reference's CUDA kernels so that the HIP kernels can be checked against it.  It is
 * never linked into, imported by, or called from the product library; only tests,
 * the smoke check and the benchmark's cpu_baseline leg use it.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC  (see oracle/Makefile).
 * -ffp-contract=off matters: every fused multiply-add below is an explicit fmaf()
 * and every other a*b+c must stay two roundings.
 *
 * Restated reference functions (paths relative to the reference checkout):
 *   oracle_build_group_meta      forge/backend/cuda/quant_grid.cu:42-99
 *   oracle_mse_scale_groups      forge/backend/cuda/quant_grid.cu:101-183
 *   oracle_gptq_solver           forge/backend/cuda/solver.cu:9-154
 *   oracle_sparsegptq14_solver   forge/backend/cuda/solver_sparsegptq14.cu:12-200
 *   oracle_pack_sparsegptq14     forge/backend/cuda/bitpacking_sparsegptq14.cu:58-107
 *   oracle_babai_solver          forge/backend/cuda/solver_babai.cu:123-322
 *   oracle_gptq_solver_direct    (the library's own displacement form of solver.cu:9-154;
 *                                checks that kernel's arithmetic, see its comment)
 *   oracle_sparsegptq14_solver_direct   (the same for solver_sparsegptq14.cu:29-200)
 *
 * Where the reference leaves fp32 bits undefined, the oracle fixes them as follows
 * (each choice is within the reference's own numerical freedom):
 *   - nvcc contracts `x*inv_s+q0` (solver.cu:13) and `(2/maxq)*amax+eps`
 *     (quant_grid.cu:83) into one FMA by default (--fmad=true); written as fmaf here.
 *   - __logf/__expf (quant_grid.cu:165-166) are hardware approximations whose bits are
 *     not specified; the oracle uses libm logf/expf.  Only exact near-ties of the
 *     candidate losses can therefore resolve differently.
 *   - The trailing update W[end:,:] -= U[blk,end:]^T * Eblk is a cuBLAS SGEMM
 *     (solver.cu:146-150) whose summation order is a library detail.  Two orders are
 *     offered: TRAIL_CHAIN applies the block's rank-1 updates one after another,
 *     x = fmaf(-U[t,k], err_t, x) for t ascending, i.e. the very chain the reference
 *     uses inside a block (solver.cu:91-94); the result is then independent of the
 *     block size.  TRAIL_GEMM accumulates acc = sum_t U[t,k]*err_t from zero with fmaf
 *     in ascending t and then stores W - acc (alpha=-1, beta=1 epilogue).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

#define ORACLE_EPS 1e-12f

static inline float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }

/* lrintf in the default rounding mode is round-to-nearest-even, like CUDA's lrintf. */
static inline float rne(float v) { return nearbyintf(v); }

/* quant_grid.cu:42-99.  X is [RG, gs] row-major fp32. */
void oracle_build_group_meta(const float* X, int64_t RG, int64_t gs, int bits, int symmetric,
                             float* scales, float* qzeros) {
    const float maxq = (float)((1 << bits) - 1);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < RG; ++g) {
        const float* grp = X + g * gs;
        float lo = 1e30f, hi = -1e30f;
        for (int64_t i = 0; i < gs; ++i) { hi = fmaxf(hi, grp[i]); lo = fminf(lo, grp[i]); }
        float s, q0;
        if (symmetric) {
            float amax = fmaxf(fabsf(lo), fabsf(hi));
            s = fmaf(2.0f / maxq, amax, ORACLE_EPS);
            q0 = 0.5f * (maxq + 1.0f);
        } else {
            s = (hi - lo) / maxq + ORACLE_EPS;
            q0 = clampf(rne(-lo / s), 0.0f, maxq);
        }
        scales[g] = s;
        qzeros[g] = q0;
    }
}

/* Loss of one shrink candidate for one group, in the reference's summation order:
 * 32 lanes, lane l adds elements l, l+32, l+64, ... in that order, then a shuffle-down
 * tree with offsets 16,8,4,2,1 (quant_grid.cu:15-22,156-169). */
static float group_loss(const float* grp, int64_t gs, float s, float rcp_s, float q0,
                        float maxq, float norm) {
    float lane[32];
    const int64_t vpl = gs / 32;
    for (int l = 0; l < 32; ++l) {
        float loss = 0.0f;
        for (int64_t i = 0; i < vpl; ++i) {
            float v = grp[l + 32 * i];
            float q = clampf(rne(fmaf(v, rcp_s, q0)), 0.0f, maxq);
            float diff = fmaf(q - q0, s, -v);
            float e = fmaxf(fabsf(diff), 1e-20f);
            loss += expf(logf(e) * norm);
        }
        lane[l] = loss;
    }
    for (int off = 16; off > 0; off >>= 1)
        for (int l = 0; l < off; ++l) lane[l] += lane[l + off];
    return lane[0];
}

/* quant_grid.cu:101-183.  Overwrites scales/qzeros in place.  losses_out (optional,
 * [RG,P]) receives every candidate's loss so that tests can recognise near-ties. */
void oracle_mse_scale_groups(const float* X, float* scales, float* qzeros, const float* cand,
                             int64_t RG, int64_t gs, int64_t P, int bits, float norm,
                             int symmetric, float* losses_out) {
    const float maxq = (float)((1 << bits) - 1);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < RG; ++g) {
        const float sg = scales[g], q0g = qzeros[g];
        float xmin = 0.0f;
        if (!symmetric) xmin = -(sg * q0g);
        float best_s = sg, best_q = q0g, best_loss = FLT_MAX;
        for (int64_t p = 0; p < P; ++p) {
            float s = sg * cand[p];
            float rcp_s = 1.0f / (s + ORACLE_EPS);
            float q0;
            if (symmetric) q0 = q0g;
            else q0 = clampf(rne(-xmin * rcp_s), 0.0f, maxq);
            float loss = group_loss(X + g * gs, gs, s, rcp_s, q0, maxq, norm);
            if (losses_out) losses_out[g * P + p] = loss;
            if (loss < best_loss) { best_loss = loss; best_s = s; best_q = q0; }
        }
        scales[g] = best_s;
        qzeros[g] = best_q;
    }
}

/* solver.cu:9-23 */
static inline void quantize_scalar(float x, float inv_s, float s, float q0, int maxq_i,
                                   float* err, uint8_t* qb, float* deq) {
    float biased = fmaf(x, inv_s, q0);
    long q = lrintf(biased);
    if (q < 0) q = 0; else if (q > maxq_i) q = maxq_i;
    *deq = fmaf((float)q, s, -q0 * s);
    *err = x - *deq;
    *qb = (uint8_t)q;
}

enum { TRAIL_CHAIN = 0, TRAIL_GEMM = 1 };

/* Apply one finished block's errors to every later column.  E is [B, R]. */
static void trailing_update(float* W, const float* U, const float* E, int64_t C, int64_t R,
                            int64_t start, int64_t B, int mode) {
    const int64_t end = start + B;
#pragma omp parallel for schedule(static)
    for (int64_t k = end; k < C; ++k) {
        float* wk = W + k * R;
        if (mode == TRAIL_CHAIN) {
            for (int64_t t = 0; t < B; ++t) {
                const float a = -U[(start + t) * C + k];
                const float* e = E + t * R;
                for (int64_t r = 0; r < R; ++r) wk[r] = fmaf(a, e[r], wk[r]);
            }
        } else {
            float* acc = (float*)calloc((size_t)R, sizeof(float));
            for (int64_t t = 0; t < B; ++t) {
                const float a = U[(start + t) * C + k];
                const float* e = E + t * R;
                for (int64_t r = 0; r < R; ++r) acc[r] = fmaf(a, e[r], acc[r]);
            }
            for (int64_t r = 0; r < R; ++r) wk[r] = wk[r] - acc[r];
            free(acc);
        }
    }
}

/* The in-block kernel alone (solver.cu:26-96) for one block of B <= 256 columns starting at
 * `start`; E [B,R] receives the errors.  Lets a caller do the trailing update with a BLAS
 * SGEMM exactly as the reference's host loop does (solver.cu:146-150). */
void oracle_gptq_inblock(float* W, const float* U, const float* scales, const float* qzeros,
                         int bits, int64_t C, int64_t R, int64_t start, int64_t B,
                         uint8_t* qweight, float* E) {
    const int maxq_i = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        float x[256];
        for (int64_t i = 0; i < B; ++i) x[i] = W[(start + i) * R + r];
        for (int64_t t = 0; t < B; ++t) {
            const int64_t c = start + t;
            const float s = scales[c * R + r], q0 = qzeros[c * R + r];
            const float inv_s = 1.0f / (s + ORACLE_EPS);
            float err, deq; uint8_t qb;
            quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
            qweight[c * R + r] = qb;
            W[c * R + r] = deq;
            E[t * R + r] = err;
            for (int64_t k = t + 1; k < B; ++k)
                x[k] = fmaf(-U[c * C + start + k], err, x[k]);
        }
    }
}

/* solver.cu:26-154.  W [C,R] fp32 is updated in place to the dequantised weights,
 * qweight [C,R] receives the codes.  U [C,C] is the row-normalised upper factor.
 * scales/qzeros are per element [C,R].  B is the in-block width (reference: 32). */
void oracle_gptq_solver(float* W, const float* U, const float* scales, const float* qzeros,
                        int bits, int64_t C, int64_t R, uint8_t* qweight, int trail_mode,
                        int64_t B) {
    const int maxq_i = (1 << bits) - 1;
    float* E = (float*)malloc((size_t)(B * R) * sizeof(float));
    for (int64_t start = 0; start < C; start += B) {
        const int64_t Bc = (start + B <= C) ? B : (C - start);
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < R; ++r) {
            float x[256];
            for (int64_t i = 0; i < Bc; ++i) x[i] = W[(start + i) * R + r];
            for (int64_t t = 0; t < Bc; ++t) {
                const int64_t c = start + t;
                const float s = scales[c * R + r], q0 = qzeros[c * R + r];
                const float inv_s = 1.0f / (s + ORACLE_EPS);
                float err, deq; uint8_t qb;
                quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
                qweight[c * R + r] = qb;
                W[c * R + r] = deq;
                E[t * R + r] = err;
                for (int64_t k = t + 1; k < Bc; ++k)
                    x[k] = fmaf(-U[c * C + start + k], err, x[k]);
            }
        }
        if (start + Bc < C) trailing_update(W, U, E, C, R, start, Bc, trail_mode);
    }
    free(E);
}

/* Checker for the library's displacement form of the same sweep (no counterpart in the
 * reference): V [C,C] holds -M[t,k]/M[k,k] above the diagonal, M being the upper factor of
 * H + damp*I = M M^T; a column hands on d = w0 - deq, its original weight minus what it was
 * rounded to, instead of err = x - deq.  I - strict(V) is the inverse of the unit matrix U
 * that oracle_gptq_solver takes, so err = d (I - strict(V)) and both forms reach every column
 * with the same value in exact arithmetic.  Quantiser and chain (one fmaf per earlier column,
 * ascending) are those of solver.cu:9-23,91-94.  W [C,R] is updated in place to the
 * dequantised weights. */
void oracle_gptq_solver_direct(float* W, const float* V, const float* scales,
                               const float* qzeros, int bits, int64_t C, int64_t R,
                               uint8_t* qweight) {
    const int maxq_i = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        float* x = (float*)malloc((size_t)C * sizeof(float));
        for (int64_t c = 0; c < C; ++c) x[c] = W[c * R + r];
        for (int64_t t = 0; t < C; ++t) {
            const float s = scales[t * R + r], q0 = qzeros[t * R + r];
            const float inv_s = 1.0f / (s + ORACLE_EPS);
            float err, deq; uint8_t qb;
            quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
            const float d = W[t * R + r] - deq;          /* W[t] is still the original weight */
            qweight[t * R + r] = qb;
            W[t * R + r] = deq;
            for (int64_t k = t + 1; k < C; ++k) x[k] = fmaf(-V[t * C + k], d, x[k]);
        }
        free(x);
    }
}

/* The 1:4 joint solve in the displacement form (checker for the library's kernel, no
 * counterpart in the reference).  mdiag [C] = diagonal of the factor M (= 1/diag(U0) of
 * solver_sparsegptq14.cu:153).  A pruned column hands on its whole original weight.  The mask
 * score reads the three columns after t before they have received the group's updates; those
 * values differ between the forms, so the error form's are rebuilt from d_j = x_j - w0_j and
 * the inverse A of the 4x4 unit diagonal block of N = I - strict(V):
 * value_k = w0_k + sum_{j<=k} d_j A[j,k], evaluated with the fused multiply-adds below. */
void oracle_sparsegptq14_solver_direct(float* W, const float* V, const float* mdiag,
                                       const float* scales, const float* qzeros, int bits,
                                       int64_t C, int64_t R, uint8_t* qweight, uint32_t* M) {
    const int maxq_i = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        float* x = (float*)calloc((size_t)C + 4, sizeof(float));
        float* w0 = (float*)calloc((size_t)C + 4, sizeof(float));
        for (int64_t c = 0; c < C; ++c) x[c] = w0[c] = W[c * R + r];
        uint32_t mask = 0u;
        for (int64_t t = 0; t < C; ++t) {
            if ((t & 31) == 0) mask = 0u;
            if (t % 4 == 0) {
                float v[4][4] = {{0}};
                for (int j = 0; j < 4; ++j)
                    for (int k = j + 1; k < 4; ++k)
                        if (t + k < C) v[j][k] = V[(t + j) * C + t + k];
                const float a02 = fmaf(v[0][1], v[1][2], v[0][2]);
                const float a13 = fmaf(v[1][2], v[2][3], v[1][3]);
                const float a03 = fmaf(v[0][1], a13, fmaf(v[0][2], v[2][3], v[0][3]));
                const float d0 = x[t] - w0[t], d1 = x[t + 1] - w0[t + 1], d2 = x[t + 2] - w0[t + 2];
                float look[4];
                look[0] = x[t];
                look[1] = fmaf(d0, v[0][1], x[t + 1]);
                look[2] = fmaf(d1, v[1][2], fmaf(d0, a02, x[t + 2]));
                look[3] = fmaf(d2, v[2][3], fmaf(d1, a13, fmaf(d0, a03, x[t + 3])));
                float best = -1e30f; int best_k = -1;
                for (int k = 0; k < 4; ++k) {
                    if (t + k >= C) continue;
                    float score = fabsf(look[k] * mdiag[t + k]);
                    if (best < score) { best = score; best_k = k; }
                }
                if (best_k > -1) mask |= (1u << ((t & 31) + best_k));
            }
            float err, deq = 0.0f, d; uint8_t qb = 0;
            if ((mask >> (t & 31)) & 1u) {
                const float s = scales[t * R + r], q0 = qzeros[t * R + r];
                const float inv_s = 1.0f / (s + ORACLE_EPS);
                quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
                d = w0[t] - deq;
            } else {
                d = w0[t];
            }
            qweight[t * R + r] = qb;
            W[t * R + r] = deq;
            for (int64_t k = t + 1; k < C; ++k) x[k] = fmaf(-V[t * C + k], d, x[k]);
            if ((t & 31) == 31 || t == C - 1) M[(t >> 5) * R + r] = mask;
        }
        free(x); free(w0);
    }
}

/* solver_sparsegptq14.cu:29-200.  U [C,C] holds the un-normalised upper factor on entry
 * and is row-normalised in place (lines 153-155), as the reference does to the caller's
 * tensor.  M is [ceil(C/32), R] uint32, bit i of word w <-> solver column 32*w+i. */
void oracle_sparsegptq14_solver(float* W, float* U, const float* scales, const float* qzeros,
                                int bits, int64_t C, int64_t R, uint8_t* qweight, uint32_t* M,
                                int trail_mode) {
    const int maxq_i = (1 << bits) - 1;
    const int64_t B = 32;
    float* Uinv = (float*)malloc((size_t)C * sizeof(float));
    for (int64_t i = 0; i < C; ++i) Uinv[i] = 1.0f / U[i * C + i];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < C; ++i)
        for (int64_t j = 0; j < C; ++j) U[i * C + j] = U[i * C + j] * Uinv[i];
    float* E = (float*)malloc((size_t)(B * R) * sizeof(float));
    for (int64_t start = 0; start < C; start += B) {
        const int64_t Bc = (start + B <= C) ? B : (C - start);
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < R; ++r) {
            float x[32];
            uint32_t mask = 0u;
            for (int64_t i = 0; i < Bc; ++i) x[i] = W[(start + i) * R + r];
            for (int64_t t = 0; t < Bc; ++t) {
                const int64_t c = start + t;
                if (t % 4 == 0) {
                    float best = -1e30f; int best_k = -1;
                    for (int k = 0; k < 4; ++k) {
                        if (c + k >= C) continue;
                        float score = fabsf(x[t + k] * Uinv[c + k]);
                        if (best < score) { best = score; best_k = k; }
                    }
                    if (best_k > -1) mask |= (1u << (t + best_k));
                }
                float err, deq = 0.0f; uint8_t qb = 0;
                if ((mask >> t) & 1u) {
                    const float s = scales[c * R + r], q0 = qzeros[c * R + r];
                    const float inv_s = 1.0f / (s + ORACLE_EPS);
                    quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
                } else {
                    err = x[t];
                }
                qweight[c * R + r] = qb;
                W[c * R + r] = deq;
                E[t * R + r] = err;
                for (int64_t k = t + 1; k < Bc; ++k)
                    x[k] = fmaf(-U[c * C + start + k], err, x[k]);
            }
            M[(start >> 5) * R + r] = mask;
        }
        if (start + Bc < C) trailing_update(W, U, E, C, R, start, Bc, trail_mode);
    }
    free(E);
    free(Uinv);
}

/* bitpacking_sparsegptq14.cu:58-107.  q_rc [R,C] codes, M [G32,R], scales [G32,R] ->
 * out [G2,R,2] u64 = bf16(scale) << 48 | idx16 << 32 | qw32. */
/* solver_babai.cu:123-322.  W [C,R] fp32 (updated in place to the dequantised weights),
 * A [C,C] upper Cholesky factor of H (H = A^T A), scales/qzeros [R*G] (index r*G + g),
 * g_idx [C] (group of solver column; NULL: c / group_size), B the block width (reference:
 * at most 32).  Blocks and the columns of a block are walked from the last to the first;
 * after column t every earlier column i receives x_i = fmaf(-A[i,t] * (1/A[i,i]), err_t, x_i).
 * For the rows above a block the reference does this with an SGEMM (`addmm_`, :313-316)
 * whose summation order is not defined: TRAIL_CHAIN continues the in-block chain (t
 * descending), TRAIL_GEMM accumulates the block's sum from zero (k ascending) and subtracts. */
void oracle_babai_solver(float* W, const float* A, const float* scales, const float* qzeros,
                         const int32_t* g_idx, int64_t group_size, int bits, int64_t C, int64_t R,
                         int64_t G, uint8_t* qweight, int trail_mode, int64_t B) {
    const int maxq_i = (1 << bits) - 1;
    float* invD = (float*)malloc((size_t)C * sizeof(float));
    for (int64_t i = 0; i < C; ++i) invD[i] = 1.0f / A[i * C + i];
    float* E = (float*)malloc((size_t)(B * R) * sizeof(float));
    for (int64_t block_end = C; block_end > 0; block_end -= B) {
        const int64_t start = block_end - B > 0 ? block_end - B : 0;
        const int64_t Bc = block_end - start;
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < R; ++r) {
            float x[256];
            for (int64_t i = 0; i < Bc; ++i) x[i] = W[(start + i) * R + r];
            for (int64_t t = Bc - 1; t >= 0; --t) {
                const int64_t row = start + t;
                int64_t g = g_idx ? (int64_t)g_idx[row] : row / group_size;
                if (g >= G) g = G - 1;
                const float s = scales[r * G + g], q0 = qzeros[r * G + g];
                const float inv_s = 1.0f / (s + ORACLE_EPS);
                float err, deq; uint8_t qb;
                quantize_scalar(x[t], inv_s, s, q0, maxq_i, &err, &qb, &deq);
                qweight[row * R + r] = qb;
                W[row * R + r] = deq;
                E[t * R + r] = err;
                for (int64_t i = 0; i < t; ++i) {
                    const float alpha = A[(start + i) * C + row] * invD[start + i];
                    x[i] = fmaf(-alpha, err, x[i]);
                }
            }
        }
        if (start > 0) {
#pragma omp parallel for schedule(static)
            for (int64_t i = 0; i < start; ++i) {
                float* wi = W + i * R;
                if (trail_mode == TRAIL_CHAIN) {
                    for (int64_t t = Bc - 1; t >= 0; --t) {
                        const float alpha = A[i * C + start + t] * invD[i];
                        const float* e = E + t * R;
                        for (int64_t r = 0; r < R; ++r) wi[r] = fmaf(-alpha, e[r], wi[r]);
                    }
                } else {
                    float* acc = (float*)calloc((size_t)R, sizeof(float));
                    for (int64_t t = 0; t < Bc; ++t) {
                        const float alpha = A[i * C + start + t] * invD[i];
                        const float* e = E + t * R;
                        for (int64_t r = 0; r < R; ++r) acc[r] = fmaf(alpha, e[r], acc[r]);
                    }
                    for (int64_t r = 0; r < R; ++r) wi[r] = wi[r] - acc[r];
                    free(acc);
                }
            }
        }
    }
    free(E);
    free(invD);
}

static uint16_t bf16_rne_bits(float x) {
    uint32_t u; memcpy(&u, &x, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void oracle_pack_sparsegptq14(const uint8_t* q_rc, const uint32_t* M, const float* scales,
                              uint64_t* out, int64_t R, int64_t C) {
    const int64_t G32 = (C + 31) / 32, G2 = (G32 + 1) / 2;
    for (int64_t g2 = 0; g2 < G2; ++g2)
        for (int64_t r = 0; r < R; ++r)
            for (int h = 0; h < 2; ++h) {
                const int64_t gid = 2 * g2 + h;
                uint64_t packed = 0;
                if (gid < G32) {
                    const uint32_t bitmask = M[gid * R + r];
                    uint32_t idx16 = 0, qw32 = 0x88888888u;
                    for (int i = 0; i < 8; ++i) {
                        const uint32_t sub = (bitmask >> (4 * i)) & 0xFu;
                        if (!sub) continue;
                        int c = 0;
                        while (!((sub >> c) & 1u)) ++c;            /* __ffs(sub) - 1 */
                        idx16 |= (uint32_t)(c & 3) << (2 * i);
                        const int64_t cid = gid * 32 + i * 4 + c;
                        if (cid < C) {
                            const uint32_t q = q_rc[r * C + cid] & 0xFu;
                            qw32 = (qw32 & ~(0xFu << (4 * i))) | (q << (4 * i));
                        }
                    }
                    packed = ((uint64_t)bf16_rne_bits(scales[gid * R + r]) << 48) |
                             ((uint64_t)(idx16 & 0xFFFFu) << 32) | (uint64_t)qw32;
                }
                out[(g2 * R + r) * 2 + h] = packed;
            }
}
