// fp32 MFMA GEMM whose K loop is one fma chain per output element (see chain_gemm.hip).
#pragma once
#include "common.h"

namespace forge {

// X[m, n] <- chain_{k = k0 .. k1-1} fma(sA * At[k, m], Bm[k, n], acc),  m in [m0, m1),
// n in [0, n1), acc starting from X[m, n] (or 0 when init_zero), sA = -1 when negate_a.
// Operands are "K-major": row k of At holds the m index contiguously, row k of Bm the n
// index.  All three may point into the same allocation as long as the rows written
// ([m0, m1) of X) are not among the rows read ([k0, k1) of At/Bm), or, when they are
// (in-place triangular solve), as long as n-tiles do not overlap: each workgroup reads
// all of its K range before it writes.
struct GemmArgs {
    float* X;         // accumulator / output, pitch ldx, batch stride xs
    const float* At;  // [K, M], pitch lda, batch stride as
    const float* Bm;  // [K, N], pitch ldb, batch stride bs
    int64_t ldx, xs, lda, as, ldb, bs;
    int m0, m1, n0, n1, k0, k1;
    bool negate_a;
    bool init_zero;
    bool b_upper_tri;  // Bm[k, n] == 0 for k > n: stop each tile's K loop at its last column
    bool b_lower_tri;  // Bm[k, n] == 0 for k < n: start each tile's K loop at its first column
    bool blocked_sum;  // sum K in blocks of 128 (more accurate; NOT the sweep's single chain)
    int products;      // bf16-piece path only: piece products per fp32 product (1, 3, 4; else 6)
    // piece path only: both not null = two fp16 pieces of every operand, three products,
    // fp32-grade.  bound_a[matrix * bound_a_stride + m] >= |At[k, m]| and
    // bound_b[matrix * bound_b_stride + n] >= |Bm[k, n]| for every k of the product: column m of
    // At and column n of Bm are scaled by the largest powers of two that keep them at or below
    // 2^14 (fp16 overflows at 2^16), and the two factors are divided out of the sums, exactly.
    const float* bound_a;
    int64_t bound_a_stride;
    const float* bound_b;
    int64_t bound_b_stride;
    // piece path only: not null = At is not read; its panel is formed from a lower triangular
    // matrix instead, At[k, m] = -(Al[m, k] * (1 / Al[m, m])) for k < m (the matrix V of the
    // displacement-form sweep straight from the factor of H; zero where a_info[matrix] != 0).
    // Al has pitch a_lower_ld and batch stride a_lower_stride.  Problems that do not take the
    // piece path need At.
    const float* a_lower;
    int64_t a_lower_ld, a_lower_stride;
    const int32_t* a_info;
    // piece path only: not null = the sums start from x_init (same pitch and batch stride as X,
    // in elements; f32 or, with x_init_bf16, bf16) instead of from X, which is then only written.
    // Problems that do not take the piece path ignore it and start from X.
    const void* x_init;
    bool x_init_bf16;
    // not null = the matrices of the batch differ in size inside their common, zero-padded
    // allocation: lim[matrix] (a multiple of 128, device memory) replaces k1 (lim_k), m1 (lim_m)
    // and/or n1 (lim_n) for that matrix where it is smaller.  Tiles that lie wholly beyond it
    // are skipped; the host still sizes the grid for the largest matrix.
    const int32_t* lim;
    bool lim_k, lim_m, lim_n;
    // with lim: the share of the nominal 2*M*N*K (largest matrix's sizes times the batch) that
    // the batch's own sizes amount to, for the timing records' work figure; 0 = all of it
    double work_frac;
    // filled in by launch_chain_gemm
    int n_tiles, m_tiles;
    bool xcd_map;
};

// Two problems for one grid (see launch_chain_gemm_pair).
struct GemmPair {
    GemmArgs first, second;
    int first_wgs;  // workgroups [0, first_wgs) belong to `first`
};

int launch_chain_gemm(const GemmArgs& g, int64_t batch, hipStream_t st);

// Runs two problems that do not depend on each other (neither writes what the other reads
// or writes).  When both are full-tile problems of the same kind they share one launch, the
// first problem's tiles ahead of the second's; otherwise they are launched one after the
// other.  Either may be empty.
// With a workspace of split_gemm_workspace_bytes(batch, k1 - k0), two blocked-sum problems
// of full tiles that share their A panel (same At, pitch, m0 and k0) run on the bf16 matrix
// pipe instead (three-piece split of every operand, fp32-grade accuracy, different
// rounding); the option fp32_blocked_sum = 1 keeps them on the fp32 kernel.
int launch_chain_gemm_pair(const GemmArgs& first, const GemmArgs& second, int64_t batch,
                           hipStream_t st, void* split_ws = nullptr, int64_t split_ws_bytes = 0);
int64_t split_gemm_workspace_bytes(int64_t batch, int64_t k_rows);
// True when launch_chain_gemm_pair(g, {}, batch, st, ws, ws_bytes) with a workspace of that
// size would run `g` on the piece path (and so would not read g.At when g.a_lower is set).
bool split_path_applies(const GemmArgs& g, int64_t batch, int64_t ws_bytes);

}  // namespace forge
