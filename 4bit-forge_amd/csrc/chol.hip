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

// Bounds for the fp16-piece products of the factorisation, one per column: every entry of the
// factor obeys |L2[k][j]| <= sqrt(A[j][j]) (column j of A = L2^T L2 sums its squares), whatever
// the spread of the diagonal (outlier channels).  The products scale each column by the largest
// power of two that keeps its bound at or below 2^14.
__global__ __launch_bounds__(256) void factor_bound_kernel(const float* __restrict__ H, int64_t C,
                                                           float* __restrict__ bound) {
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= C) return;
    const float d = H[(int64_t)blockIdx.y * C * C + j * C + j];
    // (NaN fails both tests: such a matrix fails anyway); 1.0001: sqrtf rounds to nearest
    bound[(int64_t)blockIdx.y * C + j] = (d > 0.0f && d < 3.0e38f) ? 1.0001f * sqrtf(d) : 1.0f;
}

// 1b for one diagonal block of every matrix in the batch: P = D^T D (D lower triangular,
// elimination from the last row upwards) and Z = D^-1, in one workgroup, blocked by 16 so
// that a phase is 8 block steps with a handful of barriers each rather than 128
// barrier-to-barrier pivot steps.
//   phase 1, block b = 7..0 (rows/columns 16b..16b+15), P = [[P11, P12], [P21, P22]]:
//     D22^T D22 = P22 by 16 lanes of ONE wavefront, a row of the 16x16 block per lane, the
//       pivot row taken through DPP row broadcasts: no LDS, no barrier inside
//     D22^T D21 = P21 by back substitution, a column per thread; P11 -= D21^T D21 (all
//       threads, P in registers)
//   W = D22^-1 of the eight diagonal blocks, all at once (16 lanes per block, DPP again)
//   phase 2, block kb = 0..7:  Z[kb, <kb] = -W (D[kb, <kb] Z[<kb, <kb]); the product in the
//     brackets is accumulated in registers by rank-16 updates as the rows of Z appear.
// Thread (ty, tx) of the 16x16 grid owns the elements (ty + 16 i, tx + 16 j), i, j < 8, in
// registers (cyclic ownership: the live part of the matrix stays spread over all threads).
template <int K>
__device__ __forceinline__ float row_bcast(float v) {   // lane K of this lane's row of 16
    float r;
    asm volatile("v_mov_b32_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v), "n"(K));
    return r;
}
// x -= bcast_K(u) * f   /   x += bcast_K(u) * f, one fused multiply-add each
template <int K>
__device__ __forceinline__ void fnma_bcast(float& x, float u, float f) {
    asm volatile("v_fmac_f32_dpp %0, -%1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(x) : "v"(u), "v"(f), "n"(K));
}
template <int K>
__device__ __forceinline__ void fma_bcast(float& x, float u, float f) {
    asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(x) : "v"(u), "v"(f), "n"(K));
}
// two wait states between a VALU write of a register and a DPP read of it
__device__ __forceinline__ void dpp_settle() { asm volatile("s_nop 1"); }
// the same, placed after whatever wrote these sixteen registers (they pass through the
// statement, so the compiler can move neither their producers below it nor their DPP
// readers above it)
__device__ __forceinline__ void dpp_settle16(float (&v)[16]) {
    asm volatile("s_nop 1"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]),
                   "+v"(v[7]), "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]),
                   "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
}

__global__ __launch_bounds__(256) void diag_block_kernel(
    const float* __restrict__ A, float* __restrict__ U, float* __restrict__ Dinv,
    float* __restrict__ udiag, int32_t* __restrict__ info, int64_t C, int a, int nblk,
    float* __restrict__ Lout) {
    // U/udiag may be null (factor-only call); Lout, when given, receives D (the diagonal block
    // of the lower factor) in the lower triangle of its tile.
    extern __shared__ __attribute__((aligned(16))) float smem[];   // 2 * NB * LDP floats (135 KB)
    float (*Dm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem);
    float (*Zm)[LDP] = reinterpret_cast<float (*)[LDP]>(smem + NB * LDP);
    __shared__ float Pp[16][LDP];   // the 16 rows of the current block, published by their owners
    __shared__ float s_rc[NB];      // 1 / D[k][k]
    __shared__ int s_fail;

    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const int64_t m0 = (int64_t)a * NB;
    const int n = (int)((C - m0) < NB ? (C - m0) : NB);
    const float* __restrict__ Ab = A + b * C * C;

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

    // ---- phase 1
    auto factor_block = [&](auto b_tag) {
        constexpr int bb = decltype(b_tag)::value;
        // 1. the owners publish rows 16 bb .. 16 bb + 15, columns < 16 (bb + 1)
#pragma unroll
        for (int j = 0; j <= bb; ++j) Pp[ty][tx + 16 * j] = P[bb][j];
        __syncthreads();
        // 2. one row of the 16x16 diagonal block per lane
        if (tid < 16) {
            const int li = tid;
            float p[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) p[j] = Pp[li][16 * bb + j];
            float mypiv = 1.0f;
            int fail = 0;
            dpp_settle16(p);
#define FORGE_ELIM(c)                                                                         \
    {                                                                                         \
        const float piv = row_bcast<c>(p[c]);                                                 \
        const bool ok = piv > 0.0f;                                                           \
        if (!ok && fail == 0) fail = 16 * bb + c + 1;                                         \
        mypiv = li == c ? piv : mypiv;                                                        \
        float inv = __builtin_amdgcn_rcpf(piv);                                               \
        inv = __builtin_fmaf(__builtin_fmaf(-piv, inv, 1.0f), inv, inv);                      \
        const float f = (ok && li < c) ? p[c] * inv : 0.0f;                                   \
        _Pragma("unroll") for (int j = 0; j < c; ++j) fnma_bcast<c>(p[j], p[j], f);          \
        dpp_settle();                                                                         \
    }
            FORGE_ELIM(15) FORGE_ELIM(14) FORGE_ELIM(13) FORGE_ELIM(12) FORGE_ELIM(11) FORGE_ELIM(10)
            FORGE_ELIM(9) FORGE_ELIM(8) FORGE_ELIM(7) FORGE_ELIM(6) FORGE_ELIM(5) FORGE_ELIM(4)
            FORGE_ELIM(3) FORGE_ELIM(2) FORGE_ELIM(1) FORGE_ELIM(0)
#undef FORGE_ELIM
            // lane li now holds row li of the unscaled factor in p[0..li]
            const float d = mypiv > 0.0f ? sqrtf(mypiv) : 1.0f;
            const float rc = 1.0f / d;
#pragma unroll
            for (int j = 0; j < 16; ++j)
                Dm[16 * bb + li][16 * bb + j] = j < li ? p[j] * rc : (j == li ? d : 0.0f);
            s_rc[16 * bb + li] = rc;
            if (li == 0 && fail != 0) atomicMax(&s_fail, fail);
        }
        __syncthreads();
        if constexpr (bb > 0) {
            // 3. D21 from D22^T D21 = P21, one column per thread, last row first
            if (tid < 16 * bb) {
                // (column form: once x[i] is known, the fmas that remove it from the rows
                // above are independent of each other)
                float x[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) x[i] = Pp[i][tid];
#pragma unroll
                for (int i = 15; i >= 0; --i) {
                    x[i] = x[i] * s_rc[16 * bb + i];
                    // row i of D22, the same for every thread: 16-byte broadcast reads
                    float drow[16];
#pragma unroll
                    for (int q = 0; 4 * q < i; ++q) {
                        const float4 v = *reinterpret_cast<const float4*>(&Dm[16 * bb + i][16 * bb + 4 * q]);
                        drow[4 * q] = v.x; drow[4 * q + 1] = v.y; drow[4 * q + 2] = v.z; drow[4 * q + 3] = v.w;
                    }
#pragma unroll
                    for (int k = 0; k < i; ++k) x[k] = __builtin_fmaf(-drow[k], x[i], x[k]);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) Dm[16 * bb + i][tid] = x[i];
            }
            __syncthreads();
            // 4. P11 -= D21^T D21
#pragma unroll 4
            for (int m = 0; m < 16; ++m) {
                float di[bb], dj2[bb];
#pragma unroll
                for (int i = 0; i < bb; ++i) {
                    di[i] = Dm[16 * bb + m][ty + 16 * i];
                    dj2[i] = Dm[16 * bb + m][tx + 16 * i];
                }
                // (blocks above the diagonal are never read again)
#pragma unroll
                for (int i = 0; i < bb; ++i)
#pragma unroll
                    for (int j = 0; j <= i; ++j) P[i][j] = __builtin_fmaf(-di[i], dj2[j], P[i][j]);
            }
        }
    };
    factor_block(std::integral_constant<int, 7>{});
    factor_block(std::integral_constant<int, 6>{});
    factor_block(std::integral_constant<int, 5>{});
    factor_block(std::integral_constant<int, 4>{});
    factor_block(std::integral_constant<int, 3>{});
    factor_block(std::integral_constant<int, 2>{});
    factor_block(std::integral_constant<int, 1>{});
    factor_block(std::integral_constant<int, 0>{});

    // ---- W = D22^-1 of all eight diagonal blocks at once: lanes 16 g .. 16 g + 15 take block g,
    // a row per lane, rows in lockstep: row m is finished by lane m at step m, then every
    // later row adds D[k][m] W[m][j] to its running sums
    __syncthreads();
    if (tid < 128) {
        const int g = tid >> 4, li = tid & 15;
        float dj[16], acc[16], w[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            dj[j] = Dm[16 * g + li][16 * g + j];
            acc[j] = 0.0f;
            w[j] = 0.0f;
        }
        const float rc = s_rc[16 * g + li];
#define FORGE_INV(m)                                                                          \
    {                                                                                         \
        _Pragma("unroll") for (int j = 0; j <= m; ++j) {                                      \
            const float val = ((j == m ? 1.0f : 0.0f) - acc[j]) * rc;                         \
            w[j] = li == m ? val : w[j];                                                      \
        }                                                                                     \
        dpp_settle16(w);                                                                      \
        _Pragma("unroll") for (int j = 0; j <= m; ++j) fma_bcast<m>(acc[j], w[j], dj[m]);     \
    }
        FORGE_INV(0) FORGE_INV(1) FORGE_INV(2) FORGE_INV(3) FORGE_INV(4) FORGE_INV(5) FORGE_INV(6)
        FORGE_INV(7) FORGE_INV(8) FORGE_INV(9) FORGE_INV(10) FORGE_INV(11) FORGE_INV(12)
        FORGE_INV(13) FORGE_INV(14) FORGE_INV(15)
#undef FORGE_INV
#pragma unroll
        for (int j = 0; j < 16; ++j) Zm[16 * g + li][16 * g + j] = j <= li ? w[j] : 0.0f;
    }
    __syncthreads();

    // ---- phase 2: P accumulates S = D[rows, < 16 kb] Z[< 16 kb, columns]
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) P[i][j] = 0.0f;
    auto invert_block = [&](auto kb_tag) {
        constexpr int kb = decltype(kb_tag)::value;
        if constexpr (kb > 0) {
            // 1. the owners publish S for the rows of block kb
#pragma unroll
            for (int j = 0; j < kb; ++j) Pp[ty][tx + 16 * j] = P[kb][j];
            __syncthreads();
            // 2. Z[kb, < kb] = -W S: row ty, columns tx + 16 j
            float wr[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) wr[k] = Zm[16 * kb + ty][16 * kb + k];   // W[ty][k], 0 for k > ty
            float z[kb];
#pragma unroll
            for (int j = 0; j < kb; ++j) z[j] = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; ++k)
#pragma unroll
                for (int j = 0; j < kb; ++j) z[j] = __builtin_fmaf(-wr[k], Pp[k][tx + 16 * j], z[j]);
#pragma unroll
            for (int j = 0; j < kb; ++j) Zm[16 * kb + ty][tx + 16 * j] = z[j];
        }
        // columns right of the diagonal block are zero
#pragma unroll
        for (int j = kb + 1; j < 8; ++j) Zm[16 * kb + ty][tx + 16 * j] = 0.0f;
        __syncthreads();
        if constexpr (kb < 7) {
            // 3. rows below: S += D[rows, block kb] Z[block kb, columns <= 16 kb + 15]
            // (the 16 values of D that a register row needs are consecutive in LDS: 16-byte reads)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float4 dq[7 - kb];
#pragma unroll
                for (int i = kb + 1; i < 8; ++i)
                    dq[i - kb - 1] = *reinterpret_cast<const float4*>(&Dm[ty + 16 * i][16 * kb + 4 * q]);
#pragma unroll
                for (int mm = 0; mm < 4; ++mm) {
                    const int m = 4 * q + mm;
                    float zrow[kb + 1];
#pragma unroll
                    for (int j = 0; j <= kb; ++j) zrow[j] = Zm[16 * kb + m][tx + 16 * j];
#pragma unroll
                    for (int i = kb + 1; i < 8; ++i) {
                        const float4 v = dq[i - kb - 1];
                        const float dv = mm == 0 ? v.x : (mm == 1 ? v.y : (mm == 2 ? v.z : v.w));
#pragma unroll
                        for (int j = 0; j <= kb; ++j) P[i][j] = __builtin_fmaf(dv, zrow[j], P[i][j]);
                    }
                }
            }
        }
    };
    invert_block(std::integral_constant<int, 0>{});
    invert_block(std::integral_constant<int, 1>{});
    invert_block(std::integral_constant<int, 2>{});
    invert_block(std::integral_constant<int, 3>{});
    invert_block(std::integral_constant<int, 4>{});
    invert_block(std::integral_constant<int, 5>{});
    invert_block(std::integral_constant<int, 6>{});
    invert_block(std::integral_constant<int, 7>{});
    __syncthreads();

    // ---- outputs
    float* __restrict__ Di = Dinv + (b * nblk + a) * NB * NB;
    for (int e = tid; e < NB * NB / 4; e += 256) {
        const int k = e >> 5, m4 = (e & 31) * 4;
        *reinterpret_cast<float4*>(Di + k * NB + m4) = *reinterpret_cast<const float4*>(&Zm[k][m4]);
    }
    if (U != nullptr) {
        float* __restrict__ Ub = U + b * C * C;
        for (int e = tid; e < NB * NB; e += 256) {
            const int m = e >> 7, k = e & (NB - 1);   // U0[a-block row m, column k] = Z[k, m]
            if (m < n && k < n) Ub[(m0 + m) * C + m0 + k] = Zm[k][m];
        }
        if (tid < n) udiag[b * C + m0 + tid] = Zm[tid][tid];
    }
    if (Lout != nullptr) {
        float* __restrict__ Lb = Lout + b * C * C;
        for (int e = tid; e < NB * NB; e += 256) {
            const int r = e >> 7, c = e & (NB - 1);
            if (r < n && c <= r) Lb[(m0 + r) * C + m0 + c] = Dm[r][c];
        }
    }
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
    // inverse diagonal blocks, then the split A panels of the trailing updates (two block rows
    // per product on the factor-only route)
    return batch * nblk * NB * NB * (int64_t)sizeof(float) + 2 * forge::split_gemm_workspace_bytes(batch, C) +
           (batch * C * (int64_t)sizeof(float) + 255) / 256 * 256;   // + one bound per column
}

namespace {

// U0^T-route factorisation (factor_only = false) or only its first phase: H = L2^T L2 with L2
// lower, left in the lower triangle of H (factor_only = true; U and udiag are not touched).
int chol_run(float* H, const float* damp, float* U, float* udiag, int32_t* info, int64_t batch,
             int64_t C, int normalise, bool factor_only, void* ws, int64_t ws_bytes, hipStream_t st) {
    const int nblk = (int)forge::ceil_div(C, NB);
    float* Dinv = (float*)ws;
    const int64_t dinv_bytes = batch * nblk * NB * NB * (int64_t)sizeof(float);
    void* split_ws = (char*)ws + dinv_bytes;
    const int64_t split_ws_bytes = 2 * forge::split_gemm_workspace_bytes(batch, C);
    float* bound = (float*)((char*)ws + dinv_bytes + split_ws_bytes);   // one per column and matrix
    // Factor only (no triangular inverse follows): every operand of the trailing updates is a
    // finished row of the factor, whose entries are bounded by the diagonal of the matrix, so
    // the products can be formed from two fp16 halves (three products) instead of three bf16
    // thirds (six).  The inverse's entries have no such bound: that route keeps the thirds.
    const bool halves = factor_only && (C % NB) == 0 && forge::option(forge::OPT_FACTOR_PIECES) == 0 &&
                        forge::option(forge::OPT_FP32_BLOCKED_SUM) == 0;

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

    if (halves) {
        factor_bound_kernel<<<dim3((unsigned)forge::ceil_div(C, 256), (unsigned)batch), dim3(256), 0, st>>>(
            H, C, bound);
        FORGE_LAUNCH_CHECK();
    }
    // 1a (+ 2a) for block rows [a_lo, a]: P[rows, 0..a] -= sum_{k > a} L2[k, rows]^T L2[k, 0..a].
    // 1a and 2a of a step do not depend on each other (2a needs rows > a only), and their tile
    // counts are complementary, (a+1) and (nblk-1-a) per matrix: one grid.
    auto trailing_update = [&](int a_lo, int a) -> int {
        const int m0 = a_lo * NB;
        const int m1 = (int)(C < (int64_t)(a + 1) * NB ? C : (int64_t)(a + 1) * NB);
        if (m1 >= C) return FORGE_OK;                       // nothing below
        forge::GemmArgs g1a{}, g2a{};
        g1a.X = H; g1a.At = H; g1a.Bm = H; g1a.ldx = g1a.lda = g1a.ldb = C;
        g1a.xs = g1a.as = g1a.bs = C * C;
        g1a.m0 = m0; g1a.m1 = m1; g1a.n0 = 0; g1a.n1 = m1; g1a.k0 = m1; g1a.k1 = (int)C;
        g1a.negate_a = true; g1a.blocked_sum = true;
        if (halves) { g1a.bound_a = g1a.bound_b = bound; g1a.bound_a_stride = g1a.bound_b_stride = C; }
        if (!factor_only) {
            g2a.X = U; g2a.At = H; g2a.Bm = U; g2a.ldx = g2a.lda = g2a.ldb = C;
            g2a.xs = g2a.as = g2a.bs = C * C;
            g2a.m0 = m0; g2a.m1 = m1; g2a.n0 = m1; g2a.n1 = (int)C; g2a.k0 = m1; g2a.k1 = (int)C;
            g2a.init_zero = true; g2a.b_upper_tri = true; g2a.blocked_sum = true;
        }
        return forge::launch_chain_gemm_pair(g1a, g2a, batch, st, split_ws, split_ws_bytes);
    };
    // 1b, 1c (+ 2b) of block row a: diagonal block, then the row's panels times Dinv^T.
    auto finish_block_row = [&](int a) -> int {
        const int m0 = a * NB;
        const int m1 = (int)(C < (int64_t)m0 + NB ? C : m0 + NB);
        {
            forge::KernelTiming timing("chol_diag_block", st, 2.0 * NB * NB * NB * (double)batch,
                                       forge::WORK_FLOPS);
            diag_block_kernel<<<dim3((unsigned)batch), dim3(256), kDiagLds, st>>>(
                H, factor_only ? nullptr : U, Dinv, factor_only ? nullptr : udiag, info, C, a, nblk,
                factor_only ? H : nullptr);
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
        if (m1 < C && !factor_only) {
            g2b.X = U; g2b.Bm = U; g2b.ldx = g2b.ldb = C; g2b.xs = g2b.bs = C * C;
            g2b.At = Dinv + (int64_t)a * NB * NB - shift; g2b.lda = NB; g2b.as = (int64_t)nblk * NB * NB;
            g2b.m0 = m0; g2b.m1 = m1; g2b.n0 = m1; g2b.n1 = (int)C; g2b.k0 = m0; g2b.k1 = m1;
            g2b.init_zero = true; g2b.negate_a = true;
        }
        return forge::launch_chain_gemm_pair(g1c, g2b, batch, st);
    };
    // With the fp16 halves the long product is bound by reading the rows of the factor below
    // the block from HBM (64 flops per byte at 128 columns), so two block rows are brought up to
    // date per product: every row read serves 256 columns (one workgroup computes both blocks'
    // tiles).  The upper of the two then only lacks what the lower one adds once it is finished, a
    // K = 128 product on the fp32 pipe.  (The pair's product also touches the block above the
    // upper row's diagonal block; nothing reads the upper triangle.)
    for (int a = nblk - 1; a >= 0;) {
        const bool pair = halves && a >= 1;
        if (int e = trailing_update(pair ? a - 1 : a, a)) return e;
        if (int e = finish_block_row(a)) return e;
        if (pair) {
            forge::GemmArgs fix{};
            fix.X = H; fix.At = H; fix.Bm = H; fix.ldx = fix.lda = fix.ldb = C;
            fix.xs = fix.as = fix.bs = C * C;
            fix.m0 = (a - 1) * NB; fix.m1 = a * NB; fix.n0 = 0; fix.n1 = a * NB;
            fix.k0 = a * NB; fix.k1 = (a + 1) * NB;
            fix.negate_a = true;
            if (int e = forge::launch_chain_gemm(fix, batch, st)) return e;
            if (int e = finish_block_row(a - 1)) return e;
            a -= 2;
        } else {
            a -= 1;
        }
    }
    if (factor_only) return FORGE_OK;
    forge::KernelTiming timing("chol_finish_rows", st,
                               ((normalise & 2) ? 4.0 : 6.0) * C * C * (double)batch, forge::WORK_BYTES);
    finish_rows_kernel<<<dim3((unsigned)C, (unsigned)batch), dim3(256), 0, st>>>(
        U, udiag, info, C, (normalise & 1) != 0, (normalise & 2) == 0);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

// U[t][k] = L[k][t] / L[k][k] for k > t (as a multiplication by the rounded reciprocal, the
// way solver_babai.cu:133-141 forms its coefficients), 1 on the diagonal, 0 below; identity
// where info says that the factorisation failed.  FLIP: L is given as an UPPER factor A with
// both index orders reversed, L[k][t] = A[C-1-k][C-1-t].  32x32 tiles through LDS so that
// both sides are accessed along rows.
template <bool FLIP>
__global__ __launch_bounds__(256) void unit_upper_from_lower_kernel(
    const float* __restrict__ L, const int32_t* __restrict__ info, float* __restrict__ U, int64_t C,
    float sign, bool upper_tiles_only, bool band) {
    __shared__ float tile[32][33];
    // band: the grid's x covers the eight tile columns of the row's own 128-column block and
    // the next one only
    const unsigned tile_col = band ? 4u * (blockIdx.y / 4u) + blockIdx.x : blockIdx.x;
    if (band && (int64_t)tile_col * 32 >= C) return;
    if (upper_tiles_only && blockIdx.y > tile_col) return;   // whole tile below the diagonal
    const int64_t b = blockIdx.z;
    const float* __restrict__ Lb = L + b * C * C;
    float* __restrict__ Ub = U + b * C * C;
    const int64_t t0 = (int64_t)blockIdx.y * 32, k0 = (int64_t)tile_col * 32;   // U tile rows t, columns k
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;                      // 32 x 8
    const bool failed = info != nullptr && info[b] != 0;
    if (!failed && k0 + 31 >= t0) {
        // L rows k0.., columns t0..: tile[kk][tt] = L[k0 + kk][t0 + tt] * rcp(L[k0+kk][k0+kk])
        for (int kk = ty; kk < 32; kk += 8) {
            const int64_t k = k0 + kk, t = t0 + tx;
            float v = 0.0f;
            if (k < C && t < C) {
                const float a = FLIP ? Lb[(C - 1 - k) * C + (C - 1 - t)] : Lb[k * C + t];
                const float d = FLIP ? Lb[(C - 1 - k) * (C + 1)] : Lb[k * (C + 1)];
                v = sign * (a * (1.0f / d));
            }
            tile[kk][tx] = v;
        }
    }
    __syncthreads();
    for (int tt = ty; tt < 32; tt += 8) {
        const int64_t t = t0 + tt, k = k0 + tx;
        if (t < C && k < C) {
            float v = (k == t) ? 1.0f : 0.0f;
            if (!failed && k > t) v = tile[tx][tt];
            Ub[t * C + k] = v;
        }
    }
}

}  // namespace

extern "C" int forge_chol_inv_upper_batched(float* H, const float* damp, float* U, float* udiag,
                                            int32_t* info, int64_t batch, int64_t C,
                                            int normalise, void* ws, int64_t ws_bytes,
                                            forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1 << 30), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(H && U && udiag && info && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_chol_workspace_bytes(batch, C), "workspace too small");
    return chol_run(H, damp, U, udiag, info, batch, C, normalise, false, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int forge_chol_reverse_lower_batched(float* H, const float* damp, int32_t* info,
                                                int64_t batch, int64_t C, void* ws, int64_t ws_bytes,
                                                forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1 << 30), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(H && info && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_chol_workspace_bytes(batch, C), "workspace too small");
    return chol_run(H, damp, nullptr, nullptr, info, batch, C, 0, true, ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int forge_unit_upper_from_lower(const float* L, const int32_t* info, float* U,
                                           int64_t batch, int64_t C, int flipped_upper,
                                           forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1 << 30), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(L && U && L != U, "null or aliased pointer");
    hipStream_t st = (hipStream_t)stream;
    const unsigned nt = (unsigned)forge::ceil_div(C, 32);
    forge::KernelTiming timing("unit_upper_from_lower", st,
                               ((flipped_upper & 8) ? 8.0 * 256.0 * C : 6.0 * C * C) * (double)batch,
                               forge::WORK_BYTES);
    const float sign = (flipped_upper & 2) ? -1.0f : 1.0f;
    const bool skip = (flipped_upper & 4) != 0;
    const bool band = (flipped_upper & 8) != 0;
    const dim3 grid(band ? 8u : nt, nt, (unsigned)batch);
    if (flipped_upper & 1)
        unit_upper_from_lower_kernel<true><<<grid, dim3(256), 0, st>>>(L, info, U, C, sign, skip, band);
    else
        unit_upper_from_lower_kernel<false><<<grid, dim3(256), 0, st>>>(L, info, U, C, sign, skip, band);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

// ------------------------------------------------------------------ factor from the rows
// A layer that saw n rows, n below its number of input features, has H = D + B^T B with B only n
// rows tall (B = sqrt(2/N) X in solver order, D = damp, + 1 in pruned columns).  Eliminating the
// columns from the last 128-column block upwards, the matrix that is left when block J is
// reached is D + B^T S_J B with S_J = (I + B_> D_>^-1 B_>^T)^-1 (n x n; "_>" = the columns after
// the block), so with Y = S_J B_J:
//     T    = D_J + B_J^T Y              the block's own 128 x 128 matrix, = M_JJ^T M_JJ
//     G    = Y M_JJ^-1                  n x 128
//     M[k, t] = G[:, k] . b_t           every entry of the factor's rows k in J left of the block
//     S_{J-1} = S_J - G G^T
// Everything the displacement-form sweep reads of the factor follows: h_k = G[:, k] / M[k, k]
// (M[k, t] / M[k, k] = h_k . b_t for t left of the block) and, inside the block,
// -M[k, t] / M[k, k].  4 n^2 C multiply-adds instead of C^3 / 3, no C x C matrix, all of it
// 128-wide products on the matrix pipe plus the 128 x 128 diagonal-block kernel above.  fp32
// throughout: measured against the float64 factor the h_k . b_t come out 2-20 times CLOSER than
// those of an fp32 Cholesky factorisation of the C x C matrix (56 rank-128 downdates of a
// matrix that starts as the identity, against C^2 / 2 entries that each collect C / 2 products).
namespace {

// T[b] <- diag(D[b][c0 .. c0 + 127])
__global__ __launch_bounds__(256) void rows_block_diag_kernel(float* __restrict__ T,
                                                              const float* __restrict__ D, int64_t C,
                                                              int64_t c0) {
    const int64_t b = blockIdx.y;
    const int e = blockIdx.x * 256 + threadIdx.x;           // 128 * 128 / 4 float4 per matrix
    const int r = e >> 5, c4 = (e & 31) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (r >= c4 && r < c4 + 4) (&v.x)[r - c4] = D[b * C + c0 + r];
    *reinterpret_cast<float4*>(T + b * NB * NB + r * NB + c4) = v;
}

// From the block's factor M (lower triangle of Mj) and its inverse Z:
//   Zs[c][k] = Z[c][k] * (1 / M[k][k])                 (columns of the inverse, scaled: G -> h)
//   V[c0 + t][k] = -(M[k][t] * (1 / M[k][k]))  (t < k), 0 otherwise     (the sweep's in-block rows)
// and the next block's T = diag(D) (next_c0 >= 0).
__global__ __launch_bounds__(256) void rows_block_scale_kernel(
    const float* __restrict__ Mj, const float* __restrict__ Z, float* __restrict__ Zs,
    float* __restrict__ V, float* __restrict__ T, const float* __restrict__ D, int64_t C, int64_t c0,
    int64_t next_c0) {
    // sixteen workgroups per matrix, eight rows of the tile each
    __shared__ float rc[NB];
    const int64_t b = blockIdx.y;
    const float* __restrict__ Mb = Mj + b * NB * NB;
    if (threadIdx.x < NB) rc[threadIdx.x] = 1.0f / Mb[threadIdx.x * NB + threadIdx.x];
    __syncthreads();
    for (int e = blockIdx.x * (NB * NB / 16) + threadIdx.x; e < (blockIdx.x + 1) * (NB * NB / 16); e += 256) {
        const int r = e >> 7, c = e & (NB - 1);
        Zs[b * NB * NB + e] = Z[b * NB * NB + e] * rc[c];
        // V[t = r][k = c] from M[k][t] = Mb[c][r]
        V[(b * C + c0 + r) * NB + c] = r < c ? -(Mb[c * NB + r] * rc[c]) : 0.0f;
        if (next_c0 >= 0) T[b * NB * NB + e] = r == c ? D[b * C + next_c0 + r] : 0.0f;
    }
}

__global__ __launch_bounds__(256) void rows_identity_kernel(float* __restrict__ S, int64_t n) {
    const int64_t b = blockIdx.y;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n * n; e += (int64_t)gridDim.x * 256)
        S[b * n * n + e] = (e / n == e % n) ? 1.0f : 0.0f;
}

// A matrix whose factorisation met a pivot that is not positive is swept uncoupled
// (gptq.py:172-175): its vectors and in-block rows become zero.
__global__ __launch_bounds__(256) void rows_failed_kernel(float* __restrict__ HmT, float* __restrict__ V,
                                                          const int32_t* __restrict__ info, int64_t n_hm,
                                                          int64_t n_v) {
    const int64_t b = blockIdx.y;
    if (info[b] == 0) return;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n_hm; e += (int64_t)gridDim.x * 256)
        HmT[b * n_hm + e] = 0.0f;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n_v; e += (int64_t)gridDim.x * 256)
        V[b * n_v + e] = 0.0f;
}

}  // namespace

extern "C" int64_t forge_rows_factor_workspace_bytes(int64_t batch, int64_t C, int64_t nmax) {
    if (batch <= 0 || C <= 0 || nmax <= 0) return 0;
    // S, Y, Y^T, G^T, and four 128 x 128 tiles per matrix: T, its factor, the inverse, the scaled inverse
    return batch * (nmax * nmax + 3 * nmax * NB + 4 * NB * NB) * (int64_t)sizeof(float);
}

extern "C" int forge_rows_factor_blocked(const float* BT, const float* D, const int32_t* n_rows,
                                         const int32_t* n_rows_host, float* HmT, float* V, int32_t* info,
                                         int64_t batch, int64_t C, int64_t nmax, void* ws,
                                         int64_t ws_bytes, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= NB && C < (1 << 22) && C % NB == 0,
                  "bad shape batch=%lld C=%lld (C: a multiple of 128)", (long long)batch, (long long)C);
    FORGE_REQUIRE(nmax >= NB && nmax <= 4096 && nmax % NB == 0, "nmax=%lld: a multiple of 128 up to 4096",
                  (long long)nmax);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(BT && D && n_rows && HmT && V && info && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_rows_factor_workspace_bytes(batch, C, nmax), "workspace too small");
    FORGE_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 255u) == 0, "ws must be 256-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    float* S = (float*)ws;
    float* Y = S + batch * nmax * nmax;
    float* YT = Y + batch * nmax * NB;
    float* GT = YT + batch * nmax * NB;
    float* T = GT + batch * nmax * NB;
    float* Mj = T + batch * NB * NB;
    float* Z = Mj + batch * NB * NB;
    float* Zs = Z + batch * NB * NB;
    constexpr size_t kDiagLds = 2 * NB * LDP * sizeof(float);
    FORGE_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(diag_block_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDiagLds));
    clear_info_kernel<<<dim3((unsigned)forge::ceil_div(batch, 256)), dim3(256), 0, st>>>(info, batch);
    FORGE_LAUNCH_CHECK();
    rows_identity_kernel<<<dim3((unsigned)(nmax * nmax / 256 < 1024 ? nmax * nmax / 256 : 1024), (unsigned)batch),
                           dim3(256), 0, st>>>(S, nmax);
    FORGE_LAUNCH_CHECK();
    const dim3 tile_grid(NB * NB / 4 / 256, (unsigned)batch);
    rows_block_diag_kernel<<<tile_grid, dim3(256), 0, st>>>(T, D, C, C - NB);
    FORGE_LAUNCH_CHECK();

    const int n = (int)nmax;
    // (for the timing records only: what the batch's own sizes leave of the nominal work)
    double f1 = 1.0, f2 = 1.0;
    if (n_rows_host) {
        f1 = f2 = 0.0;
        for (int64_t b = 0; b < batch; ++b) {
            FORGE_REQUIRE(n_rows_host[b] >= NB && n_rows_host[b] <= nmax && n_rows_host[b] % NB == 0,
                          "n_rows[%lld]=%d: a multiple of 128 up to nmax", (long long)b, n_rows_host[b]);
            const double r = (double)n_rows_host[b] / (double)nmax;
            f1 += r / (double)batch;
            f2 += r * r / (double)batch;
        }
    }
    for (int64_t c0 = C - NB; c0 >= 0; c0 -= NB) {
        // Y = S B_J and its transpose (each is an operand of a later product in that layout)
        forge::GemmArgs ya{}, yb{};
        ya.X = Y; ya.ldx = NB; ya.xs = nmax * NB;
        ya.At = S; ya.lda = nmax; ya.as = nmax * nmax;
        ya.Bm = BT + c0; ya.ldb = C; ya.bs = nmax * C;
        ya.m1 = n; ya.n1 = NB; ya.k1 = n; ya.init_zero = true; ya.blocked_sum = true;
        ya.lim = n_rows; ya.lim_m = ya.lim_k = true; ya.work_frac = f2;
        yb.X = YT; yb.ldx = nmax; yb.xs = nmax * NB;
        yb.At = BT + c0; yb.lda = C; yb.as = nmax * C;
        yb.Bm = S; yb.ldb = nmax; yb.bs = nmax * nmax;
        yb.m1 = NB; yb.n1 = n; yb.k1 = n; yb.init_zero = true; yb.blocked_sum = true;
        yb.lim = n_rows; yb.lim_n = yb.lim_k = true; yb.work_frac = f2;
        if (int e = forge::launch_chain_gemm_pair(ya, yb, batch, st)) return e;
        // T = D_J + B_J^T Y
        forge::GemmArgs t{};
        t.X = T; t.ldx = NB; t.xs = NB * NB;
        t.At = BT + c0; t.lda = C; t.as = nmax * C;
        t.Bm = Y; t.ldb = NB; t.bs = nmax * NB;
        t.m1 = NB; t.n1 = NB; t.k1 = n; t.blocked_sum = true;
        t.lim = n_rows; t.lim_k = true; t.work_frac = f1;
        if (int e = forge::launch_chain_gemm(t, batch, st)) return e;
        // T = M^T M, Z = M^-1
        {
            forge::KernelTiming timing("chol_diag_block", st, 2.0 * NB * NB * NB * (double)batch,
                                       forge::WORK_FLOPS);
            diag_block_kernel<<<dim3((unsigned)batch), dim3(256), kDiagLds, st>>>(
                T, nullptr, Z, nullptr, info, NB, 0, 1, Mj);
            FORGE_LAUNCH_CHECK();
        }
        rows_block_scale_kernel<<<dim3(16, (unsigned)batch), dim3(256), 0, st>>>(Mj, Z, Zs, V, T, D, C, c0,
                                                                                 c0 - NB);
        FORGE_LAUNCH_CHECK();
        // G^T = Z^T Y^T (for the downdate) and the h_k = G[:, k] / M[k, k] into their columns of HmT
        forge::GemmArgs ga{}, gb{};
        ga.X = GT; ga.ldx = nmax; ga.xs = nmax * NB;
        ga.At = Z; ga.lda = NB; ga.as = NB * NB;
        ga.Bm = YT; ga.ldb = nmax; ga.bs = nmax * NB;
        ga.m1 = NB; ga.n1 = n; ga.k1 = NB; ga.init_zero = true; ga.blocked_sum = true;
        ga.lim = n_rows; ga.lim_n = true; ga.work_frac = f1;
        gb.X = HmT + c0; gb.ldx = C; gb.xs = nmax * C;
        gb.At = YT; gb.lda = nmax; gb.as = nmax * NB;
        gb.Bm = Zs; gb.ldb = NB; gb.bs = NB * NB;
        gb.m1 = n; gb.n1 = NB; gb.k1 = NB; gb.init_zero = true; gb.blocked_sum = true;
        gb.lim = n_rows; gb.lim_m = true; gb.work_frac = f1;
        if (int e = forge::launch_chain_gemm_pair(ga, gb, batch, st)) return e;
        // S -= G G^T
        if (c0 > 0) {
            forge::GemmArgs s{};
            s.X = S; s.ldx = nmax; s.xs = nmax * nmax;
            s.At = GT; s.lda = nmax; s.as = nmax * NB;
            s.Bm = GT; s.ldb = nmax; s.bs = nmax * NB;
            s.m1 = n; s.n1 = n; s.k1 = NB; s.negate_a = true; s.blocked_sum = true;
            s.lim = n_rows; s.lim_m = s.lim_n = true; s.work_frac = f2;
            if (int e = forge::launch_chain_gemm(s, batch, st)) return e;
        }
    }
    rows_failed_kernel<<<dim3(64, (unsigned)batch), dim3(256), 0, st>>>(HmT, V, info, nmax * C, C * NB);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
