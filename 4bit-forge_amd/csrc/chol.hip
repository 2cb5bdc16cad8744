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
#include <type_traits>

namespace {

constexpr int NB = 128;       // block size
constexpr int LDP = NB + 4;   // LDS pitch

// (a fill kernel rather than hipMemsetAsync, so that a caller may capture the whole call
// into a HIP graph)
__global__ void clear_info_kernel(int32_t* __restrict__ info, int64_t batch) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < batch) info[i] = 0;
}

__global__ void add_damp_kernel(float* __restrict__ H, const float* __restrict__ damp, int64_t C) {
    const int64_t b = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < C) H[b * C * C + i * C + i] += damp[b];
}

// 1b for one diagonal block of every matrix in the batch.  256 threads as a 16x16 grid;
// thread (ty, tx) owns the elements (ty + 16 i, tx + 16 j), i, j < 8, of the block in
// registers (cyclic ownership: at every step of either phase the live part of the block is
// spread evenly over the threads, so a step costs (cb+1)^2 resp. (8-kb)(kb+1) fmas per
// thread instead of 64).  Each step publishes one row through LDS and costs one barrier;
// the row of the NEXT step is published as soon as the fmas that complete it are done, ahead
// of the rest of the step's fmas, so that its LDS write and the pivot's division are off the
// barrier-to-barrier path.
//   phase 1:  P[i][j] -= (row[i] / piv) * row[j],   D[c][j] = row[j] / sqrt(piv) afterwards
//   phase 2:  Z = D^-1 row by row, P accumulating D[i,k] Z[k,j]
__global__ __launch_bounds__(256) void diag_block_kernel(
    const float* __restrict__ A, float* __restrict__ U, float* __restrict__ Dinv,
    float* __restrict__ udiag, int32_t* __restrict__ info, int64_t C, int a, int nblk) {
    extern __shared__ __attribute__((aligned(16))) float smem[];   // 2 * NB * LDP floats (135 KB)
    float (*Dm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem);
    float (*Zm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem + NB * LDP);
    __shared__ float dsq[NB], drc[NB], s_inv[NB];
    __shared__ int s_fail;

    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const int64_t m0 = (int64_t)a * NB;
    const int n = (int)((C - m0) < NB ? (C - m0) : NB);
    const float* __restrict__ Ab = A + b * C * C;

    // symmetric tile: both halves were produced by the same GEMM; read the lower one.
    // (Full blocks load without per-element tests so that the 64 loads are in flight together.)
    float P[8][8];
    if (n == NB) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int r = ty + 16 * i, c = tx + 16 * j;
                const int rr = r > c ? r : c, cc = r > c ? c : r;
                P[i][j] = Ab[(m0 + rr) * C + m0 + cc];
            }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int r = ty + 16 * i, c = tx + 16 * j;
                const int rr = r > c ? r : c, cc = r > c ? c : r;
                float v = (r == c) ? 1.0f : 0.0f;
                if (rr < n) v = Ab[(m0 + rr) * C + m0 + cc];
                P[i][j] = v;
            }
    }
    if (tid == 0) s_fail = 0;
    __syncthreads();   // the pivot owners below test it

    // ---- P = D^T D, eliminating from the last row upwards.  Row c = 16 cb + r lives in
    // register row cb of the threads with ty == r; only rows and columns <= c are still
    // needed, i.e. register rows / columns <= cb.
    int my_fail = 0;   // first non-positive pivot this thread owned (1-based), in elimination order
    auto publish_row = [&](auto cb_tag, int r) {
        constexpr int cb = decltype(cb_tag)::value;
        if (ty == r) {
            const int c = 16 * cb + r;
#pragma unroll
            for (int j = 0; j <= cb; ++j) Dm[c][tx + 16 * j] = P[cb][j];
            // the owner of the pivot divides once for everybody
            if (tx == r) {
                const float piv = P[cb][cb];
                s_inv[c] = piv > 0.0f ? 1.0f / piv : 0.0f;
                if (!(piv > 0.0f) && my_fail == 0) my_fail = c + 1;
            }
        }
    };
    auto eliminate = [&](auto cb_tag) {
        constexpr int cb = decltype(cb_tag)::value;
        for (int r = 15; r >= 0; --r) {
            const int c = 16 * cb + r;
            __syncthreads();
            const float inv = s_inv[c];
            float ri[cb + 1], rj[cb + 1];
#pragma unroll
            for (int i = 0; i <= cb; ++i) {
                ri[i] = Dm[c][ty + 16 * i] * inv;
                rj[i] = Dm[c][tx + 16 * i];
            }
            // the two register rows that can hold the next pivot row first
#pragma unroll
            for (int i = cb; i >= (cb > 0 ? cb - 1 : 0); --i)
#pragma unroll
                for (int j = 0; j <= cb; ++j) P[i][j] = __builtin_fmaf(-ri[i], rj[j], P[i][j]);
            if (r > 0) publish_row(std::integral_constant<int, cb>{}, r - 1);
            else if constexpr (cb > 0) publish_row(std::integral_constant<int, cb - 1>{}, 15);
#pragma unroll
            for (int i = cb - 2; i >= 0; --i)
#pragma unroll
                for (int j = 0; j <= cb; ++j) P[i][j] = __builtin_fmaf(-ri[i], rj[j], P[i][j]);
        }
    };
    publish_row(std::integral_constant<int, 7>{}, 15);
    eliminate(std::integral_constant<int, 7>{});
    eliminate(std::integral_constant<int, 6>{});
    eliminate(std::integral_constant<int, 5>{});
    eliminate(std::integral_constant<int, 4>{});
    eliminate(std::integral_constant<int, 3>{});
    eliminate(std::integral_constant<int, 2>{});
    eliminate(std::integral_constant<int, 1>{});
    eliminate(std::integral_constant<int, 0>{});
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

    // ---- Z = D^-1 (lower), row by row from the top; P accumulates D[i,k] Z[k,j].  Row
    // k = 16 kb + r: only rows > k (register rows >= kb) and columns <= k (register columns
    // <= kb) are touched.
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) P[i][j] = 0.0f;
    auto publish_z = [&](auto kb_tag, int r, float rc) {
        constexpr int kb = decltype(kb_tag)::value;
        if (ty == r) {
            const int k = 16 * kb + r;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int col = tx + 16 * j;
                float z = 0.0f;
                if (j <= kb && col <= k) z = ((col == k ? 1.0f : 0.0f) - P[kb][j]) * rc;
                Zm[k][col] = z;
            }
        }
    };
    auto invert = [&](auto kb_tag) {
        constexpr int kb = decltype(kb_tag)::value;
        for (int r = 0; r < 16; ++r) {
            const int k = 16 * kb + r;
            // D does not change any more: its column k (and the next row's 1/d) are read
            // ahead of the barrier
            float d[8 - kb];
#pragma unroll
            for (int i = kb; i < 8; ++i) d[i - kb] = Dm[ty + 16 * i][k];
            const float rc_next = drc[k + 1 < NB ? k + 1 : k];
            __syncthreads();
            float zj[kb + 1];
#pragma unroll
            for (int j = 0; j <= kb; ++j) zj[j] = Zm[k][tx + 16 * j];
#pragma unroll
            for (int i = kb; i <= (kb < 7 ? kb + 1 : 7); ++i)
#pragma unroll
                for (int j = 0; j <= kb; ++j) P[i][j] = __builtin_fmaf(d[i - kb], zj[j], P[i][j]);
            if (r < 15) publish_z(std::integral_constant<int, kb>{}, r + 1, rc_next);
            else if constexpr (kb < 7) publish_z(std::integral_constant<int, kb + 1>{}, 0, rc_next);
#pragma unroll
            for (int i = kb + 2; i < 8; ++i)
#pragma unroll
                for (int j = 0; j <= kb; ++j) P[i][j] = __builtin_fmaf(d[i - kb], zj[j], P[i][j]);
        }
    };
    publish_z(std::integral_constant<int, 0>{}, 0, drc[0]);
    invert(std::integral_constant<int, 0>{});
    invert(std::integral_constant<int, 1>{});
    invert(std::integral_constant<int, 2>{});
    invert(std::integral_constant<int, 3>{});
    invert(std::integral_constant<int, 4>{});
    invert(std::integral_constant<int, 5>{});
    invert(std::integral_constant<int, 6>{});
    invert(std::integral_constant<int, 7>{});
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
    if (my_fail != 0) atomicMax(&s_fail, my_fail);   // the first failure = the largest row
    __syncthreads();
    if (tid == 0 && s_fail != 0 && info[b] == 0) info[b] = (int32_t)(m0 + s_fail);
}

// Last pass over the rows of U0: zero what lies left of the diagonal (the GEMMs only write
// the blocks on and right of it), and divide by the diagonal when asked to (gptq.py:164).
// A failed factorisation hands back the identity instead, as gptq.py:172-175 does.
__global__ void finish_rows_kernel(float* __restrict__ U, float* __restrict__ udiag,
                                   const int32_t* __restrict__ info, int64_t C, bool normalise,
                                   bool zero_left) {
    const int64_t b = blockIdx.y;
    const int64_t row = blockIdx.x;
    float* __restrict__ Ur = U + b * C * C + row * C;
    if (info[b] != 0) {
        for (int64_t j = threadIdx.x; j < C; j += blockDim.x) Ur[j] = (j == row) ? 1.0f : 0.0f;
        if (threadIdx.x == 0) udiag[b * C + row] = 1.0f;
        return;
    }
    // the diagonal block kernel wrote its whole tile, zeros below the diagonal included
    const int64_t left = zero_left ? row / NB * NB : 0;
    for (int64_t j = threadIdx.x; j < left; j += blockDim.x) Ur[j] = 0.0f;
    if (!normalise) return;
    const float d = udiag[b * C + row];
    for (int64_t j = row + threadIdx.x; j < C; j += blockDim.x) Ur[j] = Ur[j] / d;
}

}  // namespace

extern "C" int64_t forge_chol_workspace_bytes(int64_t batch, int64_t C) {
    if (batch <= 0 || C <= 0) return 0;
    const int64_t nblk = forge::ceil_div(C, NB);
    // inverse diagonal blocks, then the split A panel of the trailing updates
    return batch * nblk * NB * NB * (int64_t)sizeof(float) + forge::split_gemm_workspace_bytes(batch, C);
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
    const int64_t dinv_bytes = batch * nblk * NB * NB * (int64_t)sizeof(float);
    void* split_ws = (char*)ws + dinv_bytes;
    const int64_t split_ws_bytes = ws_bytes - dinv_bytes;

    // the diagonal-block kernel keeps two 128x132 fp32 tiles in LDS (gfx950 has 160 KB/CU)
    constexpr size_t kDiagLds = 2 * NB * LDP * sizeof(float);
    FORGE_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(diag_block_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDiagLds));
    clear_info_kernel<<<dim3((unsigned)forge::ceil_div(batch, 256)), dim3(256), 0, st>>>(info, batch);
    FORGE_LAUNCH_CHECK();
    if (damp) {
        add_damp_kernel<<<dim3((unsigned)forge::ceil_div(C, 256), (unsigned)batch), dim3(256), 0, st>>>(
            H, damp, C);
        FORGE_LAUNCH_CHECK();
    }

    for (int a = nblk - 1; a >= 0; --a) {
        const int m0 = a * NB;
        const int m1 = (int)(C < (int64_t)m0 + NB ? C : m0 + NB);
        // 1a and 2a of this step do not depend on each other (2a needs rows > a only), and
        // their tile counts are complementary, (a+1) and (nblk-1-a) per matrix: one grid
        forge::GemmArgs g1a{}, g2a{};   // left empty (m1 == m0) when there is nothing below
        if (m1 < C) {
            g1a.X = H; g1a.At = H; g1a.Bm = H; g1a.ldx = g1a.lda = g1a.ldb = C;
            g1a.xs = g1a.as = g1a.bs = C * C;
            g1a.m0 = m0; g1a.m1 = m1; g1a.n0 = 0; g1a.n1 = m1; g1a.k0 = m1; g1a.k1 = (int)C;
            g1a.negate_a = true; g1a.blocked_sum = true;
            g2a.X = U; g2a.At = H; g2a.Bm = U; g2a.ldx = g2a.lda = g2a.ldb = C;
            g2a.xs = g2a.as = g2a.bs = C * C;
            g2a.m0 = m0; g2a.m1 = m1; g2a.n0 = m1; g2a.n1 = (int)C; g2a.k0 = m1; g2a.k1 = (int)C;
            g2a.init_zero = true; g2a.b_upper_tri = true; g2a.blocked_sum = true;
            if (int e = forge::launch_chain_gemm_pair(g1a, g2a, batch, st, split_ws, split_ws_bytes)) return e;
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
        // 1c (rows of L2 left of the diagonal block) and 2b (rows of U0 right of it) both
        // multiply by Dinv^T and touch different matrices: one grid again
        forge::GemmArgs g1c{}, g2b{};
        if (a > 0) {
            g1c.X = H; g1c.Bm = H; g1c.ldx = g1c.ldb = C; g1c.xs = g1c.bs = C * C;
            g1c.At = Dinv + (int64_t)a * NB * NB - shift; g1c.lda = NB; g1c.as = (int64_t)nblk * NB * NB;
            g1c.m0 = m0; g1c.m1 = m1; g1c.n0 = 0; g1c.n1 = m0; g1c.k0 = m0; g1c.k1 = m1;
            g1c.init_zero = true;
        }
        if (m1 < C) {
            g2b.X = U; g2b.Bm = U; g2b.ldx = g2b.ldb = C; g2b.xs = g2b.bs = C * C;
            g2b.At = Dinv + (int64_t)a * NB * NB - shift; g2b.lda = NB; g2b.as = (int64_t)nblk * NB * NB;
            g2b.m0 = m0; g2b.m1 = m1; g2b.n0 = m1; g2b.n1 = (int)C; g2b.k0 = m0; g2b.k1 = m1;
            g2b.init_zero = true; g2b.negate_a = true;
        }
        if (int e = forge::launch_chain_gemm_pair(g1c, g2b, batch, st)) return e;
    }
    forge::KernelTiming timing("chol_finish_rows", st,
                               ((normalise & 2) ? 4.0 : 6.0) * C * C * (double)batch, forge::WORK_BYTES);
    finish_rows_kernel<<<dim3((unsigned)C, (unsigned)batch), dim3(256), 0, st>>>(
        U, udiag, info, C, (normalise & 1) != 0, (normalise & 2) == 0);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
