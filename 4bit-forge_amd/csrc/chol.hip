// Batched "upper Cholesky factor of the inverse" for the GPTQ solve on gfx950.
//
// The reference obtains U with three LAPACK-style calls (forge/gptq.py:160-164):
// L = chol(H), Hinv = potri(L), U0 = chol(Hinv, upper), then divides each row by its
// diagonal.  U0 is the unique upper-triangular matrix with positive diagonal and
// U0^T U0 = H^-1.  The same matrix is reached with half the arithmetic and no explicit
// inverse of H: factor H = L2^T L2 with L2 LOWER triangular (a Cholesky factorisation
// that eliminates from the last row/column upwards), then U0 = L2^-T.  Proof:
// H^-1 = L2^-1 L2^-T = (L2^-T)^T (L2^-T) and L2^-T is upper triangular with positive
// diagonal, so it is U0 by uniqueness.
//
// Both phases are organised so that every GEMM has K-major operands (row index = k),
// which is what chain_gemm.hip wants, and so that no transposes or index flips occur:
//
//   for block row a = last .. 0            (128 rows each)
//     1a  P[a, 0..a]  = H[a, 0..a] - sum_{k>a} L2[k,a]^T L2[k, 0..a]        (MFMA GEMM)
//     1b  P[a,a] = D^T D, D lower;  Dinv = D^-1                             (one workgroup)
//     1c  L2[a, 0..a-1] = Dinv^T P[a, 0..a-1]                               (MFMA GEMM)
//     2a  S[a, b] = sum_{a<k<=b} L2[k,a]^T U0[k,b]     for b > a            (MFMA GEMM)
//     2b  U0[a, b] = -Dinv^T S[a, b],   U0[a,a] = Dinv^T                    (MFMA GEMM)
//
// With `normalise`, a last pass divides every row of U0 by its diagonal entry (the
// H.div_(H.diag()[:, None]) of gptq.py:164); diag(U0) is returned separately.  Flops:
// C^3/3 for phase 1 and C^3/3 for phase 2 against 4/3 C^3 for the three-call route.
#include "chain_gemm.h"

namespace {

constexpr int NB = 128;       // block size
constexpr int LDP = NB + 4;   // LDS pitch

__global__ void add_damp_kernel(float* __restrict__ H, const float* __restrict__ damp, int64_t C) {
    const int64_t b = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < C) H[b * C * C + i * C + i] += damp[b];
}

// 1b for one diagonal block of every matrix in the batch.  256 threads as a 16x16 grid,
// thread (ty,tx) owns the 8x8 sub-block P[8ty.., 8tx..] in registers.  Each elimination
// step publishes the (unscaled) pivot row through LDS and costs one barrier:
//   P[i][j] -= (row[i] / piv) * row[j],   D[c][j] = row[j] / sqrt(piv) afterwards.
__device__ __forceinline__ void select_row(const float (&P)[8][8], int which, float (&out)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = P[0][j];
#pragma unroll
    for (int i = 1; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) out[j] = (which == i) ? P[i][j] : out[j];
}

__global__ __launch_bounds__(256) void diag_block_kernel(
    const float* __restrict__ A, float* __restrict__ U, float* __restrict__ Dinv,
    float* __restrict__ udiag, int32_t* __restrict__ info, int64_t C, int a, int nblk) {
    extern __shared__ float smem[];                      // 2 * NB * LDP floats (135 KB)
    float (*Dm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem);
    float (*Zm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem + NB * LDP);
    __shared__ float dsq[NB], drc[NB];
    __shared__ int s_fail;

    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const int64_t m0 = (int64_t)a * NB;
    const int n = (int)((C - m0) < NB ? (C - m0) : NB);
    const float* __restrict__ Ab = A + b * C * C;

    float P[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = 8 * ty + i, c = 8 * tx + j;
            // symmetric tile: both halves were produced by the same GEMM; read the lower one
            const int rr = r > c ? r : c, cc = r > c ? c : r;
            float v = (r == c) ? 1.0f : 0.0f;
            if (rr < n) v = Ab[(m0 + rr) * C + m0 + cc];
            P[i][j] = v;
        }
    if (tid == 0) s_fail = 0;

    // ---- P = D^T D, eliminating from the last row upwards
    for (int c = NB - 1; c >= 0; --c) {
        if (ty == (c >> 3)) {
            float row[8];
            select_row(P, c & 7, row);
#pragma unroll
            for (int j = 0; j < 8; ++j) Dm[c][8 * tx + j] = row[j];
        }
        __syncthreads();
        const float piv = Dm[c][c];
        const bool ok = piv > 0.0f;
        if (!ok && tid == 0 && s_fail == 0) s_fail = c + 1;
        const float inv = ok ? 1.0f / piv : 0.0f;
        float ri[8], rj[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) ri[i] = Dm[c][8 * ty + i] * inv;
#pragma unroll
        for (int j = 0; j < 8; ++j) rj[j] = Dm[c][8 * tx + j];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) P[i][j] = __builtin_fmaf(-ri[i], rj[j], P[i][j]);
    }
    __syncthreads();
    if (tid < NB) {
        const float piv = Dm[tid][tid];
        const float d = piv > 0.0f ? sqrtf(piv) : 1.0f;
        dsq[tid] = d;
        drc[tid] = 1.0f / d;
    }
    __syncthreads();
    for (int e = tid; e < NB * NB; e += 256) {
        const int c = e >> 7, j = e & (NB - 1);
        Dm[c][j] = j < c ? Dm[c][j] * drc[c] : (j == c ? dsq[c] : 0.0f);
    }
    __syncthreads();

    // ---- Z = D^-1 (lower), row by row from the top; P now accumulates D[i,k] Z[k,j]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) P[i][j] = 0.0f;
    for (int k = 0; k < NB; ++k) {
        if (ty == (k >> 3)) {
            float row[8];
            select_row(P, k & 7, row);
            const float rc = drc[k];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int col = 8 * tx + j;
                Zm[k][col] = col <= k ? ((col == k ? 1.0f : 0.0f) - row[j]) * rc : 0.0f;
            }
        }
        __syncthreads();
        float di[8], zj[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) di[i] = Dm[8 * ty + i][k];
#pragma unroll
        for (int j = 0; j < 8; ++j) zj[j] = Zm[k][8 * tx + j];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) P[i][j] = __builtin_fmaf(di[i], zj[j], P[i][j]);
    }
    __syncthreads();

    // ---- outputs
    float* __restrict__ Di = Dinv + (b * nblk + a) * NB * NB;
    for (int e = tid; e < NB * NB; e += 256) Di[e] = Zm[e >> 7][e & (NB - 1)];
    float* __restrict__ Ub = U + b * C * C;
    for (int e = tid; e < NB * NB; e += 256) {
        const int m = e >> 7, k = e & (NB - 1);   // U0[a-block row m, column k] = Z[k, m]
        if (m < n && k < n) Ub[(m0 + m) * C + m0 + k] = Zm[k][m];
    }
    if (tid < n) udiag[b * C + m0 + tid] = Zm[tid][tid];
    if (tid == 0 && s_fail != 0 && info[b] == 0) info[b] = (int32_t)(m0 + s_fail);
}

// Last pass over the rows of U0: divide by the diagonal when asked to (gptq.py:164); a
// failed factorisation hands back the identity instead, as gptq.py:172-175 does.
__global__ void finish_rows_kernel(float* __restrict__ U, float* __restrict__ udiag,
                                   const int32_t* __restrict__ info, int64_t C, bool normalise) {
    const int64_t b = blockIdx.y;
    const int64_t row = blockIdx.x;
    float* __restrict__ Ur = U + b * C * C + row * C;
    if (info[b] != 0) {
        for (int64_t j = threadIdx.x; j < C; j += blockDim.x) Ur[j] = (j == row) ? 1.0f : 0.0f;
        if (threadIdx.x == 0) udiag[b * C + row] = 1.0f;
        return;
    }
    if (!normalise) return;
    const float d = udiag[b * C + row];
    for (int64_t j = row + threadIdx.x; j < C; j += blockDim.x) Ur[j] = Ur[j] / d;
}

}  // namespace

extern "C" int64_t forge_chol_workspace_bytes(int64_t batch, int64_t C) {
    if (batch <= 0 || C <= 0) return 0;
    const int64_t nblk = forge::ceil_div(C, NB);
    return batch * nblk * NB * NB * (int64_t)sizeof(float);
}

extern "C" int forge_chol_inv_upper_batched(float* H, const float* damp, float* U, float* udiag,
                                            int32_t* info, int64_t batch, int64_t C,
                                            int normalise, void* ws, int64_t ws_bytes,
                                            forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1 << 30), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(H && U && udiag && info && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_chol_workspace_bytes(batch, C), "workspace too small");
    hipStream_t st = (hipStream_t)stream;
    const int nblk = (int)forge::ceil_div(C, NB);
    float* Dinv = (float*)ws;

    // the diagonal-block kernel keeps two 128x132 fp32 tiles in LDS (gfx950 has 160 KB/CU)
    constexpr size_t kDiagLds = 2 * NB * LDP * sizeof(float);
    FORGE_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(diag_block_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDiagLds));
    FORGE_HIP_CHECK(hipMemsetAsync(info, 0, batch * sizeof(int32_t), st));
    {
        forge::KernelTiming timing("chol_clear_u", st, 4.0 * C * C * (double)batch, forge::WORK_BYTES);
        FORGE_HIP_CHECK(hipMemsetAsync(U, 0, batch * C * C * sizeof(float), st));
    }
    if (damp) {
        add_damp_kernel<<<dim3((unsigned)forge::ceil_div(C, 256), (unsigned)batch), dim3(256), 0, st>>>(
            H, damp, C);
        FORGE_LAUNCH_CHECK();
    }

    for (int a = nblk - 1; a >= 0; --a) {
        const int m0 = a * NB;
        const int m1 = (int)(C < (int64_t)m0 + NB ? C : m0 + NB);
        forge::GemmArgs g{};
        if (m1 < C) {  // 1a
            g = forge::GemmArgs{};
            g.X = H; g.At = H; g.Bm = H; g.ldx = g.lda = g.ldb = C; g.xs = g.as = g.bs = C * C;
            g.m0 = m0; g.m1 = m1; g.n0 = 0; g.n1 = m1; g.k0 = m1; g.k1 = (int)C; g.negate_a = true; g.blocked_sum = true;
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
        }
        {
            forge::KernelTiming timing("chol_diag_block", st, 2.0 * NB * NB * NB * (double)batch,
                                       forge::WORK_FLOPS);
            diag_block_kernel<<<dim3((unsigned)batch), dim3(256), kDiagLds, st>>>(
                H, U, Dinv, udiag, info, C, a, nblk);
            FORGE_LAUNCH_CHECK();
        }
        // Dinv blocks addressed with global (k, m) indices: shift the base so that
        // element (m0 + k', m0 + m') lands on block entry (k', m').
        const int64_t shift = (int64_t)m0 * NB + m0;
        if (a > 0) {  // 1c
            g = forge::GemmArgs{};
            g.X = H; g.Bm = H; g.ldx = g.ldb = C; g.xs = g.bs = C * C;
            g.At = Dinv + (int64_t)a * NB * NB - shift; g.lda = NB; g.as = (int64_t)nblk * NB * NB;
            g.m0 = m0; g.m1 = m1; g.n0 = 0; g.n1 = m0; g.k0 = m0; g.k1 = m1; g.init_zero = true;
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
        }
        if (m1 < C) {  // 2a, 2b
            g = forge::GemmArgs{};
            g.X = U; g.At = H; g.Bm = U; g.ldx = g.lda = g.ldb = C; g.xs = g.as = g.bs = C * C;
            g.m0 = m0; g.m1 = m1; g.n0 = m1; g.n1 = (int)C; g.k0 = m1; g.k1 = (int)C;
            g.init_zero = true; g.b_upper_tri = true; g.blocked_sum = true;
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
            g = forge::GemmArgs{};
            g.X = U; g.Bm = U; g.ldx = g.ldb = C; g.xs = g.bs = C * C;
            g.At = Dinv + (int64_t)a * NB * NB - shift; g.lda = NB; g.as = (int64_t)nblk * NB * NB;
            g.m0 = m0; g.m1 = m1; g.n0 = m1; g.n1 = (int)C; g.k0 = m0; g.k1 = m1;
            g.init_zero = true; g.negate_a = true;
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
        }
    }
    forge::KernelTiming timing("chol_finish_rows", st, 4.0 * C * C * (double)batch, forge::WORK_BYTES);
    finish_rows_kernel<<<dim3((unsigned)C, (unsigned)batch), dim3(256), 0, st>>>(U, udiag, info, C,
                                                                               normalise != 0);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
