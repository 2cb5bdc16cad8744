// GPTQ for a layer that saw FEWER calibration rows than it has input features, on gfx950.
//
// The reference sums H = (2/n) X^T X over the n rows a layer saw (forge/gptq.py:61-80), adds
// damp to the diagonal (gptq.py:151-153), factors the C x C matrix three times (gptq.py:160-164)
// and sweeps the columns with the factor's rows (solver.cu:9-154).  For an expert of a routed
// layer n is often tiny (most experts of a 256-expert layer see a handful of the calibration
// tokens), and then H = D + B^T B with D diagonal and B = sqrt(2/n) X only n rows tall.  Every
// quantity the sweep reads from the factor has a closed form in B:
//
//   eliminate the columns from the last one upwards (H = M^T M, M lower, the factor the
//   displacement form of the sweep uses): with S_k = (I + B_{>k} D_{>k}^-1 B_{>k}^T)^-1 (n x n),
//     s = S_k b_k,  p_k = D_k + b_k . s = M[k,k]^2,  h_k = s / p_k,  S_{k-1} = S_k - s s^T / p_k
//   and  M[k,t] / M[k,k] = h_k . b_t  for t < k.
//
// The sweep's value of column k when it is reached, w0_k + sum_{t<k} (w0_t - deq_t) M[k,t]/M[k,k],
// is therefore  w0_k + h_k . a  with  a = sum_{t<k} (w0_t - deq_t) b_t  an n-vector per output
// row: 2 n multiply-adds per weight instead of C/2, no C x C matrix at all.  Same numbers as the
// dense route in exact arithmetic; in floating point this route is the more accurate one (the
// recurrence runs in float64, where S shrinks from 1 to damp / |b|^2 without losing its digits).
//
// Compiled for n = 4, 16, 32, 64 and 128 rows of B (rows beyond a layer's own count are zero rows;
// 128 with four threads per row of S in the factor):
//   lowrank_gram/suffix/block_kernel   the recurrence, cut into blocks of 128 columns that
//                                      start from their own S and run side by side; writes h_k.
//   lowrank_sweep_kernel               n/16 lanes per output row walk k = 0 .. C-1: dot,
//                                      quantise, update.
#include <vector>
#include "common.h"

namespace {

constexpr float kEps = 1e-12f;    // the quantiser's epsilon (solver.cu:12)

// ---------------------------------------------------------------- factor
// The recurrence is serial in k, but S_k = (I + sum_{j>k} b_j b_j^T / D_j)^-1 is the inverse of
// a SUM over the later columns: the columns are cut into blocks of FB, every block's Gram
// matrix sum b b^T / D is formed on its own (gram), summed from the last block backwards
// (suffix), and then every block inverts its own start matrix and walks only its FB columns
// (block): C / FB wavefronts per matrix at work instead of one, FB + n serial steps instead of C.
constexpr int FB = 128;

// What every lane of a wavefront needs of a column, the n entries of b_k, goes through LDS: lane
// i < NR loads entry i (the next column's while this one is worked on), all read all of them
// back with broadcast reads.
template <int NR>
struct ColumnFeed {
    float (*sh)[NR];
    const float* src;     // this lane's entry of column 0
    float nxt;
    bool owner;
    __device__ void start(int64_t k) {
        if (owner) sh[k & 1][threadIdx.x & (NR - 1)] = src[k * NR];
    }
    __device__ void request(int64_t k) { nxt = owner ? src[k * NR] : 0.0f; }
    __device__ void publish(int64_t k) {
        if (owner) sh[k & 1][threadIdx.x & (NR - 1)] = nxt;
    }
    __device__ void read(int64_t k, double (&bd)[NR]) const {
#pragma unroll
        for (int j = 0; j < NR; j += 4) {
            const float4 v = *reinterpret_cast<const float4*>(&sh[k & 1][j]);
            bd[j + 0] = (double)v.x; bd[j + 1] = (double)v.y;
            bd[j + 2] = (double)v.z; bd[j + 3] = (double)v.w;
        }
    }
};

// gram[b][blk][i][:] = sum over the block's columns of b_k[i] b_k / D_k; lane i < NR holds row i.
template <int NR>
__global__ __launch_bounds__(64) void lowrank_gram_kernel(const float* __restrict__ Bp,
                                                          const float* __restrict__ D,
                                                          double* __restrict__ gram, int64_t C,
                                                          int nblk) {
    __shared__ __attribute__((aligned(16))) float bsh[2][NR];
    const int row = threadIdx.x & (NR - 1);
    const int blk = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int64_t k_lo = (int64_t)blk * FB, k_hi = (k_lo + FB < C ? k_lo + FB : C) - 1;
    ColumnFeed<NR> feed{bsh, Bp + b * C * NR + row, 0.0f, threadIdx.x < NR};
    const float* __restrict__ Db = D + b * C;
    double acc[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) acc[j] = 0.0;
    feed.start(k_hi);
    float nd = Db[k_hi];
    for (int64_t k = k_hi; k >= k_lo; --k) {
        const double dk = (double)nd;
        if (k > k_lo) {
            feed.request(k - 1);
            nd = Db[k - 1];
        }
        __syncthreads();
        double bd[NR];
        feed.read(k, bd);
        const double mine = (double)bsh[k & 1][row] / dk;
#pragma unroll
        for (int j = 0; j < NR; ++j) acc[j] = __builtin_fma(mine, bd[j], acc[j]);
        if (k > k_lo) feed.publish(k - 1);
    }
    if (threadIdx.x < NR) {
        double* __restrict__ out = gram + ((b * nblk + blk) * NR + row) * NR;
#pragma unroll
        for (int j = 0; j < NR; ++j) out[j] = acc[j];
    }
}

// In place: gram[b][blk] <- sum of gram[b][blk'] over blk' > blk (a thread per matrix entry);
// also clears the failure flags.
__global__ __launch_bounds__(256) void lowrank_suffix_kernel(double* __restrict__ gram,
                                                             int32_t* __restrict__ info, int nblk,
                                                             int nn) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int64_t b = blockIdx.y;
    if (idx == 0) info[b] = 0;
    if (idx >= nn) return;
    double run = 0.0;
    for (int blk = nblk - 1; blk >= 0; --blk) {
        double* p = gram + (b * nblk + blk) * nn + idx;
        const double g = *p;
        *p = run;
        run += g;
    }
}

// One wavefront per (block, matrix); lane i < NR holds row i of S in float64 (lanes NR..63 repeat
// the first NR and store nothing).  S starts as the inverse of I + (the suffix sum above) by
// Gauss-Jordan elimination in place (symmetric positive definite: no pivoting), pivot row
// through LDS; then the block's columns from the last to the first.
template <int NR>
__global__ __launch_bounds__(64) void lowrank_block_kernel(const float* __restrict__ Bp,
                                                           const float* __restrict__ D,
                                                           const double* __restrict__ later,
                                                           float* __restrict__ Hm,
                                                           int32_t* __restrict__ info, int64_t C,
                                                           int nblk) {
    __shared__ __attribute__((aligned(16))) float bsh[2][NR];
    __shared__ __attribute__((aligned(16))) double ssh[NR];
    const int row = threadIdx.x & (NR - 1);
    const bool owner = threadIdx.x < NR;
    const int blk = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int64_t k_lo = (int64_t)blk * FB, k_hi = (k_lo + FB < C ? k_lo + FB : C) - 1;
    ColumnFeed<NR> feed{bsh, Bp + b * C * NR + row, 0.0f, owner};
    const float* __restrict__ Db = D + b * C;
    float* __restrict__ Hb = Hm + b * C * NR + row;
    feed.start(k_hi);
    float nd = Db[k_hi];
    bool bad = false;

    double S[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) S[j] = (j == row) ? 1.0 : 0.0;
    if (blk + 1 < nblk) {
        const double* __restrict__ src = later + ((b * nblk + blk) * NR + row) * NR;
#pragma unroll
        for (int j = 0; j < NR; ++j) S[j] += src[j];
#pragma unroll
        for (int m = 0; m < NR; ++m) {
            __syncthreads();                       // the previous pivot row has been read
            if (threadIdx.x == m) {
#pragma unroll
                for (int j = 0; j < NR; ++j) ssh[j] = S[j];
            }
            __syncthreads();
            double piv[NR];
#pragma unroll
            for (int j = 0; j < NR; j += 2) {
                const double2 v = *reinterpret_cast<const double2*>(&ssh[j]);
                piv[j] = v.x;
                piv[j + 1] = v.y;
            }
            bad |= !(piv[m] > 0.0);
            const double rp = 1.0 / piv[m];
            // rows other than m: S[j] -= (S[m] / p) piv[j], then S[m] = -S[m] / p;
            // row m itself: S[j] = piv[j] / p, S[m] = 1 / p
            const bool is_m = row == m;
            const double keep = is_m ? 0.0 : 1.0;
            const double g = is_m ? rp : -(S[m] * rp);
#pragma unroll
            for (int j = 0; j < NR; ++j) S[j] = __builtin_fma(g, piv[j], keep * S[j]);
            S[m] = g;
        }
        __syncthreads();
    }

    for (int64_t k = k_hi; k >= k_lo; --k) {
        const double dk = (double)nd;
        if (k > k_lo) {
            feed.request(k - 1);
            nd = Db[k - 1];
        }
        __syncthreads();
        double bd[NR];
        feed.read(k, bd);
        // s_row = S[row, :] . b   (four chains)
        double c0 = 0.0, c1 = 0.0, c2 = 0.0, c3 = 0.0;
#pragma unroll
        for (int j = 0; j < NR; j += 4) {
            c0 = __builtin_fma(S[j + 0], bd[j + 0], c0);
            c1 = __builtin_fma(S[j + 1], bd[j + 1], c1);
            c2 = __builtin_fma(S[j + 2], bd[j + 2], c2);
            c3 = __builtin_fma(S[j + 3], bd[j + 3], c3);
        }
        const double s = (c0 + c1) + (c2 + c3);
        if (owner) ssh[row] = s;
        __syncthreads();
        double sj[NR];
#pragma unroll
        for (int j = 0; j < NR; j += 2) {
            const double2 v = *reinterpret_cast<const double2*>(&ssh[j]);
            sj[j] = v.x;
            sj[j + 1] = v.y;
        }
        double p0 = dk, p1 = 0.0, p2 = 0.0, p3 = 0.0;
#pragma unroll
        for (int j = 0; j < NR; j += 4) {
            p0 = __builtin_fma(bd[j + 0], sj[j + 0], p0);
            p1 = __builtin_fma(bd[j + 1], sj[j + 1], p1);
            p2 = __builtin_fma(bd[j + 2], sj[j + 2], p2);
            p3 = __builtin_fma(bd[j + 3], sj[j + 3], p3);
        }
        const double p = (p0 + p1) + (p2 + p3);
        bad |= !(p > 0.0);                       // also catches NaN
        const double h = s / p;
        if (owner) Hb[k * NR] = (float)h;
#pragma unroll
        for (int j = 0; j < NR; ++j) S[j] = __builtin_fma(-h, sj[j], S[j]);
        if (k > k_lo) feed.publish(k - 1);
    }
    if (threadIdx.x == 0 && bad) atomicOr(info + b, 1);
}

// ---- n = 128: a row of S no longer fits one lane's registers.  NS = 4 threads share a row, 32
// columns each (512 threads, thread = (row, quarter)); what crosses threads goes through LDS
// with a workgroup barrier.  Same arithmetic as the one-wavefront kernels above except that the
// dot products are summed quarter by quarter.
constexpr int WN = 128, WS = 4, WQ = WN / WS;      // rows, threads per row, columns per thread

__global__ __launch_bounds__(WN * WS) void lowrank_gram_wide_kernel(const float* __restrict__ Bp,
                                                                    const float* __restrict__ D,
                                                                    double* __restrict__ gram,
                                                                    int64_t C, int nblk) {
    __shared__ __attribute__((aligned(16))) float bsh[2][WN];
    const int row = threadIdx.x & (WN - 1), qt = threadIdx.x / WN;
    const int blk = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int64_t k_lo = (int64_t)blk * FB, k_hi = (k_lo + FB < C ? k_lo + FB : C) - 1;
    const float* __restrict__ Bb = Bp + b * C * WN + row;
    const float* __restrict__ Db = D + b * C;
    double acc[WQ];
#pragma unroll
    for (int j = 0; j < WQ; ++j) acc[j] = 0.0;
    if (qt == 0) bsh[k_hi & 1][row] = Bb[k_hi * WN];
    float nd = Db[k_hi];
    for (int64_t k = k_hi; k >= k_lo; --k) {
        const double dk = (double)nd;
        float nxt = 0.0f;
        if (k > k_lo) {
            if (qt == 0) nxt = Bb[(k - 1) * WN];
            nd = Db[k - 1];
        }
        __syncthreads();
        const double mine = (double)bsh[k & 1][row] / dk;
#pragma unroll
        for (int j = 0; j < WQ; j += 4) {
            const float4 v = *reinterpret_cast<const float4*>(&bsh[k & 1][qt * WQ + j]);
            acc[j + 0] = __builtin_fma(mine, (double)v.x, acc[j + 0]);
            acc[j + 1] = __builtin_fma(mine, (double)v.y, acc[j + 1]);
            acc[j + 2] = __builtin_fma(mine, (double)v.z, acc[j + 2]);
            acc[j + 3] = __builtin_fma(mine, (double)v.w, acc[j + 3]);
        }
        if (k > k_lo && qt == 0) bsh[(k - 1) & 1][row] = nxt;
    }
    double* __restrict__ out = gram + ((b * nblk + blk) * WN + row) * WN + qt * WQ;
#pragma unroll
    for (int j = 0; j < WQ; ++j) out[j] = acc[j];
}

__global__ __launch_bounds__(WN * WS) void lowrank_block_wide_kernel(const float* __restrict__ Bp,
                                                                     const float* __restrict__ D,
                                                                     const double* __restrict__ later,
                                                                     float* __restrict__ Hm,
                                                                     int32_t* __restrict__ info,
                                                                     int64_t C, int nblk) {
    __shared__ __attribute__((aligned(16))) float bsh[2][WN];
    __shared__ __attribute__((aligned(16))) double rowsh[WN];      // pivot row / s
    __shared__ __attribute__((aligned(16))) double colsh[WN];      // pivot column
    __shared__ __attribute__((aligned(16))) double part[WS][WN];   // partial dots
    __shared__ double psum[WS];
    const int row = threadIdx.x & (WN - 1), qt = threadIdx.x / WN;
    const int blk = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int64_t k_lo = (int64_t)blk * FB, k_hi = (k_lo + FB < C ? k_lo + FB : C) - 1;
    const float* __restrict__ Bb = Bp + b * C * WN + row;
    const float* __restrict__ Db = D + b * C;
    float* __restrict__ Hb = Hm + b * C * WN + row;
    if (qt == 0) bsh[k_hi & 1][row] = Bb[k_hi * WN];
    float nd = Db[k_hi];
    bool bad = false;

    double S[WQ];                                   // S[row][qt * WQ + j]
#pragma unroll
    for (int j = 0; j < WQ; ++j) S[j] = (qt * WQ + j == row) ? 1.0 : 0.0;
    if (blk + 1 < nblk) {
        const double* __restrict__ src = later + ((b * nblk + blk) * WN + row) * WN + qt * WQ;
#pragma unroll
        for (int j = 0; j < WQ; ++j) S[j] += src[j];
        // (the quarter of the pivot is a run-time loop, the position inside it unrolled: S is
        // indexed with constants, and the code is a quarter of the fully unrolled form's)
#pragma unroll 1
        for (int mq = 0; mq < WS; ++mq)
#pragma unroll
        for (int mi = 0; mi < WQ; ++mi) {
            const int m = mq * WQ + mi;
            __syncthreads();                       // the previous pivot row and column have been read
            if (row == m) {
#pragma unroll
                for (int j = 0; j < WQ; ++j) rowsh[qt * WQ + j] = S[j];
            }
            if (qt == mq) colsh[row] = S[mi];
            __syncthreads();
            double piv[WQ];
#pragma unroll
            for (int j = 0; j < WQ; j += 2) {
                const double2 v = *reinterpret_cast<const double2*>(&rowsh[qt * WQ + j]);
                piv[j] = v.x;
                piv[j + 1] = v.y;
            }
            const double p = rowsh[m];
            bad |= !(p > 0.0);
            const double rp = 1.0 / p;
            const bool is_m = row == m;
            const double keep = is_m ? 0.0 : 1.0;
            const double g = is_m ? rp : -(colsh[row] * rp);
#pragma unroll
            for (int j = 0; j < WQ; ++j) S[j] = __builtin_fma(g, piv[j], keep * S[j]);
            if (qt == mq) S[mi] = g;
        }
    }

    for (int64_t k = k_hi; k >= k_lo; --k) {
        const double dk = (double)nd;
        float nxt = 0.0f;
        if (k > k_lo) {
            if (qt == 0) nxt = Bb[(k - 1) * WN];
            nd = Db[k - 1];
        }
        __syncthreads();                           // b_k is in place; last column's LDS reads are done
        double bd[WQ];
#pragma unroll
        for (int j = 0; j < WQ; j += 4) {
            const float4 v = *reinterpret_cast<const float4*>(&bsh[k & 1][qt * WQ + j]);
            bd[j + 0] = (double)v.x; bd[j + 1] = (double)v.y;
            bd[j + 2] = (double)v.z; bd[j + 3] = (double)v.w;
        }
        double c0 = 0.0, c1 = 0.0, c2 = 0.0, c3 = 0.0;
#pragma unroll
        for (int j = 0; j < WQ; j += 4) {
            c0 = __builtin_fma(S[j + 0], bd[j + 0], c0);
            c1 = __builtin_fma(S[j + 1], bd[j + 1], c1);
            c2 = __builtin_fma(S[j + 2], bd[j + 2], c2);
            c3 = __builtin_fma(S[j + 3], bd[j + 3], c3);
        }
        part[qt][row] = (c0 + c1) + (c2 + c3);
        __syncthreads();
        const double s = (part[0][row] + part[1][row]) + (part[2][row] + part[3][row]);
        if (qt == 0) rowsh[row] = s;
        __syncthreads();
        double sj[WQ];
#pragma unroll
        for (int j = 0; j < WQ; j += 2) {
            const double2 v = *reinterpret_cast<const double2*>(&rowsh[qt * WQ + j]);
            sj[j] = v.x;
            sj[j + 1] = v.y;
        }
        // b . s: every thread of a quarter forms the same partial sum; one of them posts it
        double p0 = 0.0, p1 = 0.0, p2 = 0.0, p3 = 0.0;
#pragma unroll
        for (int j = 0; j < WQ; j += 4) {
            p0 = __builtin_fma(bd[j + 0], sj[j + 0], p0);
            p1 = __builtin_fma(bd[j + 1], sj[j + 1], p1);
            p2 = __builtin_fma(bd[j + 2], sj[j + 2], p2);
            p3 = __builtin_fma(bd[j + 3], sj[j + 3], p3);
        }
        if (row == 0) psum[qt] = (p0 + p1) + (p2 + p3);
        __syncthreads();
        const double p = dk + ((psum[0] + psum[1]) + (psum[2] + psum[3]));
        bad |= !(p > 0.0);
        const double h = s / p;
        if (qt == 0) Hb[k * WN] = (float)h;
#pragma unroll
        for (int j = 0; j < WQ; ++j) S[j] = __builtin_fma(-h, sj[j], S[j]);
        if (k > k_lo && qt == 0) bsh[(k - 1) & 1][row] = nxt;
    }
    if (threadIdx.x == 0 && bad) atomicOr(info + b, 1);
}

__device__ __forceinline__ float w0_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float w0_as_f32(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }

// ---------------------------------------------------------------- sweep
// A row's n-vector a is spread over L = NR / 16 neighbouring lanes, sixteen entries each (one
// lane with four entries for NR = 4, the experts with a handful of rows): the
// dot product is sixteen multiply-adds per lane and a butterfly over the L lanes (both
// partners add the same two numbers, so all of them hold the same value and quantise alike),
// the update sixteen more.  256 / L rows per workgroup.  h_k and b_k are the same for every row:
// the workgroup stages TK columns of both in LDS and every multiply-add takes them from
// broadcast reads.  The row's weights, scales and zero points of the next tile are requested
// while the current tile's chain runs.  Quantiser as in solver.cu:9-23:
// q = clamp(rint(fma(x, 1/(s+eps), z)), 0, maxq), deq = fma(q, s, -(z s)).
template <int CTRL>
__device__ __forceinline__ float quad_swap(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// (Bp and Hm point at this matrix's own vectors; everything else at the batch's first matrix.)
template <int NR, typename W0T>
__device__ __forceinline__ void lowrank_sweep_body(
    const W0T* __restrict__ W0, const float* __restrict__ Bp, const float* __restrict__ Hm,
    const float* __restrict__ scT, const float* __restrict__ qzT, const int32_t* __restrict__ g_idx,
    const int32_t* __restrict__ info, uint8_t* __restrict__ q, int64_t C, int64_t R, int64_t G,
    float maxq) {
    constexpr int TK = 8;                         // columns per staged tile (16: twice the registers for the
                                                  // prefetched weights, scales and zeros, half the wavefronts per
                                                  // SIMD, 28 % slower; 4: no faster)
    constexpr int NA = NR < 16 ? NR : 16;         // entries of a per lane
    constexpr int L = NR / NA;                    // lanes per row
    constexpr int Q = NR / 4;                     // float4 per column
    __shared__ float4 Ts[2][2][TK][Q];            // [buffer][0 = h, 1 = b][column][quarter]
    const int64_t b = blockIdx.y;
    // the grid is sized for the matrices with the most lanes per row: the others need fewer
    // workgroups (the whole workgroup leaves together)
    if ((int64_t)blockIdx.x * (256 / L) >= R) return;
    const int part = threadIdx.x & (L - 1);
    const int64_t r_raw = (int64_t)blockIdx.x * (256 / L) + threadIdx.x / L;
    const bool live = r_raw < R && part == 0;
    const int64_t r = r_raw < R ? r_raw : R - 1;   // idle lanes replay the last row, store nothing
    const W0T* __restrict__ w0 = W0 + b * C * R + r;
    const float* __restrict__ sc = scT + b * G * R + r;
    const float* __restrict__ qz = qzT + b * G * R + r;
    const int32_t* __restrict__ gi = g_idx + b * C;
    uint8_t* __restrict__ qo = q + b * C * R + r;
    // a failed factorisation sweeps with the identity (gptq.py:172-175): no coupling at all
    const bool coupled = info[b] == 0;
    // a tile is TK * Q float4 of h and as many of b, both contiguous in memory: thread t
    // carries float4 number t, t + 256, ... of the two laid end to end
    constexpr int PER_TILE = 2 * TK * Q, SLOTS = (PER_TILE + 255) / 256;
    const float4* __restrict__ Hsrc = reinterpret_cast<const float4*>(Hm);
    const float4* __restrict__ Bsrc = reinterpret_cast<const float4*>(Bp);
    auto fetch = [&](int64_t k0, float4 (&st)[SLOTS]) {
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            const int idx = threadIdx.x + 256 * i;
            st[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (idx < PER_TILE && coupled)
                st[i] = idx < TK * Q ? Hsrc[k0 * Q + idx] : Bsrc[k0 * Q + idx - TK * Q];
        }
    };
    auto stash = [&](int to, const float4 (&st)[SLOTS]) {
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            const int idx = threadIdx.x + 256 * i;
            if (idx < PER_TILE) (&Ts[to][0][0][0])[idx] = st[i];
        }
    };

    float a[NA];
#pragma unroll
    for (int j = 0; j < NA; ++j) a[j] = 0.0f;

    float wv[TK], sv[TK], rv[TK], zv[TK];
    auto load_meta = [&](int64_t k0, float (&w)[TK], float (&s)[TK], float (&z)[TK]) {
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            const int64_t g = gi[k0 + t];
            w[t] = w0_as_f32(w0 + (k0 + t) * R);
            s[t] = sc[g * R];
            z[t] = qz[g * R];
        }
    };
    load_meta(0, wv, sv, zv);
    {
        float4 st[SLOTS];
        fetch(0, st);
        stash(0, st);
    }
    __syncthreads();

    int buf = 0;
    for (int64_t k0 = 0; k0 < C; k0 += TK) {
        const bool more = k0 + TK < C;
        float nw[TK], ns[TK], nz[TK];
        float4 stage[SLOTS];
        if (more) {
            load_meta(k0 + TK, nw, ns, nz);
            fetch(k0 + TK, stage);
        }
#pragma unroll
        for (int t = 0; t < TK; ++t) rv[t] = 1.0f / (sv[t] + kEps);
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            float h[NA], bb[NA];
#pragma unroll
            for (int j = 0; j < NA / 4; ++j) {
                const float4 v = Ts[buf][0][t][(NA / 4) * part + j];
                h[4 * j + 0] = v.x; h[4 * j + 1] = v.y; h[4 * j + 2] = v.z; h[4 * j + 3] = v.w;
            }
            float c0 = 0.0f, c1 = 0.0f, c2 = 0.0f, c3 = 0.0f;
#pragma unroll
            for (int j = 0; j < NA; j += 4) {
                c0 = __builtin_fmaf(a[j + 0], h[j + 0], c0);
                c1 = __builtin_fmaf(a[j + 1], h[j + 1], c1);
                c2 = __builtin_fmaf(a[j + 2], h[j + 2], c2);
                c3 = __builtin_fmaf(a[j + 3], h[j + 3], c3);
            }
            float dot = (c0 + c1) + (c2 + c3);
            if constexpr (L >= 2) dot += quad_swap<0xB1>(dot);      // lanes 0<->1, 2<->3
            if constexpr (L >= 4) dot += quad_swap<0x4E>(dot);      // lanes 0<->2, 1<->3
            if constexpr (L >= 8) dot += quad_swap<0x141>(dot);     // lane i <-> 7 - i of every eight
            const float x = wv[t] + dot;
            const float qf = __builtin_amdgcn_fmed3f(
                __builtin_rintf(__builtin_fmaf(x, rv[t], zv[t])), 0.0f, maxq);
            const float deq = __builtin_fmaf(qf, sv[t], -(zv[t] * sv[t]));
            const float d = wv[t] - deq;
            if (live) qo[(k0 + t) * R] = (uint8_t)qf;
#pragma unroll
            for (int j = 0; j < NA / 4; ++j) {
                const float4 v = Ts[buf][1][t][(NA / 4) * part + j];
                bb[4 * j + 0] = v.x; bb[4 * j + 1] = v.y; bb[4 * j + 2] = v.z; bb[4 * j + 3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < NA; ++j) a[j] = __builtin_fmaf(d, bb[j], a[j]);
        }
        if (more) {
            stash(buf ^ 1, stage);
#pragma unroll
            for (int t = 0; t < TK; ++t) { wv[t] = nw[t]; sv[t] = ns[t]; zv[t] = nz[t]; }
        }
        __syncthreads();
        buf ^= 1;
    }
}

// One launch for matrices of all three sizes: matrix b has nr[b] rows of B and its vectors
// start off[b] floats into Bp and Hm (laid end to end in batch order).
constexpr int kMaxMixed = 96;
struct MixedTable {
    int64_t off[kMaxMixed];
    uint8_t nr[kMaxMixed];
};

template <typename W0T>
__global__ __launch_bounds__(256) void lowrank_sweep_kernel(
    const W0T* __restrict__ W0, const float* __restrict__ Bp, const float* __restrict__ Hm,
    const float* __restrict__ scT, const float* __restrict__ qzT, const int32_t* __restrict__ g_idx,
    const int32_t* __restrict__ info, uint8_t* __restrict__ q, int64_t C, int64_t R, int64_t G,
    float maxq, MixedTable tab) {
    const int nr = tab.nr[blockIdx.y];
    const int64_t off = tab.off[blockIdx.y];
    if (nr == 4)
        lowrank_sweep_body<4, W0T>(W0, Bp + off, Hm + off, scT, qzT, g_idx, info, q, C, R, G, maxq);
    else if (nr == 16)
        lowrank_sweep_body<16, W0T>(W0, Bp + off, Hm + off, scT, qzT, g_idx, info, q, C, R, G, maxq);
    else if (nr == 32)
        lowrank_sweep_body<32, W0T>(W0, Bp + off, Hm + off, scT, qzT, g_idx, info, q, C, R, G, maxq);
    else if (nr == 64)
        lowrank_sweep_body<64, W0T>(W0, Bp + off, Hm + off, scT, qzT, g_idx, info, q, C, R, G, maxq);
    else
        lowrank_sweep_body<128, W0T>(W0, Bp + off, Hm + off, scT, qzT, g_idx, info, q, C, R, G, maxq);
}

// A layer that saw no rows at all has H = I (gptq.py:97-99): nothing couples its columns and the
// sweep is the quantiser applied to every weight, in whatever order.  Layer layout in, layer
// layout out; a thread takes eight consecutive columns of a row.
// The same for bf16 weights whose rows, groups and addresses are multiples of eight columns: a
// thread's eight columns lie in one group, one 16-byte load and one 8-byte store.  Few enough
// registers (and the wave priority) to run beside another stream's scale search.
__global__ __launch_bounds__(256) void round_to_nearest_bf16x8_kernel(
    const uint16_t* __restrict__ W, int64_t w_stride, int64_t ldw, const float* __restrict__ scales,
    const float* __restrict__ qzeros, uint8_t* __restrict__ q, int64_t R, int64_t C, uint32_t gs,
    int64_t G, float maxq, const int64_t* __restrict__ index) {
    __builtin_amdgcn_s_setprio(3);
    const uint32_t c0 = (blockIdx.x * 256u + threadIdx.x) * 8u;
    if ((int64_t)c0 >= C) return;
    const int64_t b = index ? index[blockIdx.z] : blockIdx.z;
    const uint32_t g = c0 / gs;
#pragma unroll 1
    for (int64_t r = blockIdx.y; r < R; r += gridDim.y) {
        const uint4 w = *reinterpret_cast<const uint4*>(W + b * w_stride + r * ldw + c0);
        const float s = scales[(b * R + r) * G + g], z = qzeros[(b * R + r) * G + g];
        const float rcp = 1.0f / (s + kEps);
        auto code = [&](uint32_t bits) {
            return (uint32_t)__builtin_amdgcn_fmed3f(
                __builtin_rintf(__builtin_fmaf(__uint_as_float(bits), rcp, z)), 0.0f, maxq);
        };
        const uint32_t lo = code(w.x << 16) | (code(w.x & 0xffff0000u) << 8) | (code(w.y << 16) << 16) |
                            (code(w.y & 0xffff0000u) << 24);
        const uint32_t hi = code(w.z << 16) | (code(w.z & 0xffff0000u) << 8) | (code(w.w << 16) << 16) |
                            (code(w.w & 0xffff0000u) << 24);
        *reinterpret_cast<uint2*>(q + (b * R + r) * C + c0) = make_uint2(lo, hi);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void round_to_nearest_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t ldw, const float* __restrict__ scales,
    const float* __restrict__ qzeros, uint8_t* __restrict__ q, int64_t R, int64_t C, int64_t gs,
    int64_t G, float maxq, const int64_t* __restrict__ index) {
    // grid: (eight-column pieces of a row / 256, rows, matrices): no division to find the row,
    // one 32-bit division to find the first group, boundaries counted from there
    const uint32_t c0 = (blockIdx.x * 256u + threadIdx.x) * 8u;
    if ((int64_t)c0 >= C) return;
    const int64_t b = index ? index[blockIdx.z] : blockIdx.z;
    const uint32_t gs32 = (uint32_t)gs, C32 = (uint32_t)C;
    const bool whole = c0 + 8 <= C32;
    for (int64_t r = blockIdx.y; r < R; r += gridDim.y) {
        const T* __restrict__ src = W + b * w_stride + r * ldw + c0;
        const float* __restrict__ sc = scales + (b * R + r) * G;
        const float* __restrict__ qz = qzeros + (b * R + r) * G;
        uint8_t* __restrict__ dst = q + (b * R + r) * C + c0;
        float v[8];
        if (whole && (reinterpret_cast<uintptr_t>(src) & 15u) == 0 && sizeof(T) == 2) {
            const uint4 w = *reinterpret_cast<const uint4*>(src);
            v[0] = __uint_as_float(w.x << 16); v[1] = __uint_as_float(w.x & 0xffff0000u);
            v[2] = __uint_as_float(w.y << 16); v[3] = __uint_as_float(w.y & 0xffff0000u);
            v[4] = __uint_as_float(w.z << 16); v[5] = __uint_as_float(w.z & 0xffff0000u);
            v[6] = __uint_as_float(w.w << 16); v[7] = __uint_as_float(w.w & 0xffff0000u);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = (c0 + i < C32) ? w0_as_f32(src + i) : 0.0f;
        }
        uint32_t lo = 0, hi = 0;
        uint32_t g = c0 / gs32, next = (g + 1) * gs32;      // first column of the next group
        float s = sc[g], z = qz[g];
        float rcp = 1.0f / (s + kEps);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (c0 + i >= next && c0 + i < C32) {
                ++g;
                next += gs32;
                s = sc[g];
                z = qz[g];
                rcp = 1.0f / (s + kEps);
            }
            const uint32_t code = (uint32_t)__builtin_amdgcn_fmed3f(
                __builtin_rintf(__builtin_fmaf(v[i], rcp, z)), 0.0f, maxq);
            if (i < 4) lo |= code << (8 * i); else hi |= code << (8 * (i - 4));
        }
        if (whole && (reinterpret_cast<uintptr_t>(dst) & 7u) == 0) {
            *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (c0 + i < C32) dst[i] = (uint8_t)(((i < 4 ? lo : hi) >> (8 * (i & 3))) & 0xffu);
        }
    }
}

}  // namespace

extern "C" int forge_round_to_nearest(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                      const int64_t* index, const float* scales, const float* qzeros,
                                      uint8_t* qweight, int64_t batch, int64_t R, int64_t C, int64_t gs,
                                      int bits, forge_stream_t stream) {
    FORGE_REQUIRE(w_dtype == FORGE_F32 || w_dtype == FORGE_BF16, "w_dtype=%d", w_dtype);
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && R >= 0 && C >= 0 && gs >= 1 && ldw >= C &&
                      R < (1LL << 30) && C < (1LL << 30),
                  "bad shape batch=%lld R=%lld C=%lld gs=%lld ldw=%lld", (long long)batch, (long long)R,
                  (long long)C, (long long)gs, (long long)ldw);
    FORGE_REQUIRE(bits >= 1 && bits <= 8, "bits=%d", bits);
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(W && scales && qzeros && qweight, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int64_t G = forge::ceil_div(C, gs);
    const dim3 grid((unsigned)forge::ceil_div((C + 7) / 8, 256), (unsigned)(R < 65535 ? R : 65535),
                    (unsigned)batch),
        block(256);
    const float maxq = (float)((1 << bits) - 1);
    forge::KernelTiming timing("round_to_nearest", st,
                               (double)batch * R * C * ((w_dtype == FORGE_BF16 ? 2.0 : 4.0) + 1.0),
                               forge::WORK_BYTES);
    const bool x8 = w_dtype == FORGE_BF16 && C % 8 == 0 && gs % 8 == 0 && ldw % 8 == 0 && w_stride % 8 == 0 &&
                    (reinterpret_cast<uintptr_t>(W) & 15u) == 0 && (reinterpret_cast<uintptr_t>(qweight) & 7u) == 0 &&
                    gs < (1LL << 31);
    if (x8)
        round_to_nearest_bf16x8_kernel<<<grid, block, 0, st>>>((const uint16_t*)W, w_stride, ldw, scales, qzeros,
                                                               qweight, R, C, (uint32_t)gs, G, maxq, index);
    else if (w_dtype == FORGE_BF16)
        round_to_nearest_kernel<uint16_t><<<grid, block, 0, st>>>((const uint16_t*)W, w_stride, ldw, scales,
                                                                  qzeros, qweight, R, C, gs, G, maxq, index);
    else
        round_to_nearest_kernel<float><<<grid, block, 0, st>>>((const float*)W, w_stride, ldw, scales,
                                                               qzeros, qweight, R, C, gs, G, maxq, index);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int64_t forge_lowrank_workspace_bytes(int64_t batch, int64_t C, int64_t n) {
    if (batch <= 0 || C <= 0 || n <= 0) return 0;
    return batch * forge::ceil_div(C, FB) * n * n * (int64_t)sizeof(double);
}

template <int NR>
static int launch_lowrank_factor(const float* Bp, const float* D, float* Hm, int32_t* info,
                                 int64_t batch, int64_t C, double* gram, hipStream_t st) {
    const int nblk = (int)forge::ceil_div(C, FB);
    const dim3 grid((unsigned)nblk, (unsigned)batch), block(64);
    lowrank_gram_kernel<NR><<<grid, block, 0, st>>>(Bp, D, gram, C, nblk);
    FORGE_LAUNCH_CHECK();
    lowrank_suffix_kernel<<<dim3((unsigned)forge::ceil_div(NR * NR, 256), (unsigned)batch), dim3(256), 0,
                            st>>>(gram, info, nblk, NR * NR);
    FORGE_LAUNCH_CHECK();
    lowrank_block_kernel<NR><<<grid, block, 0, st>>>(Bp, D, gram, Hm, info, C, nblk);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_lowrank_factor(const float* Bp, const float* D, float* Hm, int32_t* info,
                                    int64_t batch, int64_t C, int64_t n, void* ws, int64_t ws_bytes,
                                    forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1LL << 22), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    FORGE_REQUIRE(n == 4 || n == 16 || n == 32 || n == 64 || n == 128,
                  "n=%lld: 4, 16, 32, 64 or 128 rows (pad with zero rows)", (long long)n);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(Bp && D && Hm && info && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_lowrank_workspace_bytes(batch, C, n), "workspace too small");
    FORGE_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15u) == 0, "ws must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    // per column: the block's Gram matrix, the two n x n products and the dot; per block: the
    // inverse of its start matrix
    const double nb = (double)forge::ceil_div(C, FB);
    forge::KernelTiming timing("lowrank_factor", st,
                               ((6.0 * n * n + 2.0 * n) * C + 2.0 * n * n * n * nb) * (double)batch,
                               forge::WORK_FLOPS);
    if (n == 4) return launch_lowrank_factor<4>(Bp, D, Hm, info, batch, C, (double*)ws, st);
    if (n == 16) return launch_lowrank_factor<16>(Bp, D, Hm, info, batch, C, (double*)ws, st);
    if (n == 32) return launch_lowrank_factor<32>(Bp, D, Hm, info, batch, C, (double*)ws, st);
    if (n == 64) return launch_lowrank_factor<64>(Bp, D, Hm, info, batch, C, (double*)ws, st);
    double* gram = (double*)ws;
    const int nblk = (int)forge::ceil_div(C, FB);
    const dim3 grid((unsigned)nblk, (unsigned)batch), block(WN * WS);
    lowrank_gram_wide_kernel<<<grid, block, 0, st>>>(Bp, D, gram, C, nblk);
    FORGE_LAUNCH_CHECK();
    lowrank_suffix_kernel<<<dim3((unsigned)forge::ceil_div(WN * WN, 256), (unsigned)batch), dim3(256), 0,
                            st>>>(gram, info, nblk, WN * WN);
    FORGE_LAUNCH_CHECK();
    lowrank_block_wide_kernel<<<grid, block, 0, st>>>(Bp, D, gram, Hm, info, C, nblk);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_gptq_sweep_lowrank_mixed(const void* W0, int w0_dtype, const float* Bp,
                                              const float* Hm, const int64_t* n_host,
                                              const int32_t* info, const float* scalesT,
                                              const float* qzerosT, const int32_t* g_idx,
                                              uint8_t* qweight, int64_t batch, int64_t C, int64_t R,
                                              int64_t G, int bits, forge_stream_t stream) {
    FORGE_REQUIRE(w0_dtype == FORGE_F32 || w0_dtype == FORGE_BF16, "w0_dtype=%d", w0_dtype);
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 0 && R >= 0 && G >= 1 && C < (1LL << 30) &&
                      R < (1LL << 30),
                  "bad shape batch=%lld C=%lld R=%lld G=%lld", (long long)batch, (long long)C,
                  (long long)R, (long long)G);
    FORGE_REQUIRE(bits >= 1 && bits <= 8, "bits=%d", bits);
    FORGE_REQUIRE(C % 16 == 0, "C=%lld must be a multiple of 16", (long long)C);
    if (batch == 0 || C == 0 || R == 0) return FORGE_OK;
    FORGE_REQUIRE(W0 && Bp && Hm && n_host && info && scalesT && qzerosT && g_idx && qweight,
                  "null pointer");
    FORGE_REQUIRE(((reinterpret_cast<uintptr_t>(Bp) | reinterpret_cast<uintptr_t>(Hm)) & 15u) == 0,
                  "Bp and Hm must be 16-byte aligned");
    double rows = 0.0;
    for (int64_t b = 0; b < batch; ++b) {
        FORGE_REQUIRE(n_host[b] == 4 || n_host[b] == 16 || n_host[b] == 32 || n_host[b] == 64 ||
                          n_host[b] == 128,
                      "n[%lld]=%lld: 4, 16, 32, 64 or 128 rows (pad with zero rows)", (long long)b,
                      (long long)n_host[b]);
        rows += (double)n_host[b];
    }
    hipStream_t st = (hipStream_t)stream;
    const float maxq = (float)((1 << bits) - 1);
    forge::KernelTiming timing("lowrank_sweep", st, 4.0 * rows * C * (double)R, forge::WORK_FLOPS);
    const size_t w0_size = w0_dtype == FORGE_BF16 ? 2 : 4;
    int64_t off = 0;
    for (int64_t b0 = 0; b0 < batch; b0 += kMaxMixed) {
        const int64_t nb = batch - b0 < kMaxMixed ? batch - b0 : kMaxMixed;
        MixedTable tab{};
        int most = 16;
        for (int64_t i = 0; i < nb; ++i) {
            tab.off[i] = off;
            tab.nr[i] = (uint8_t)n_host[b0 + i];
            off += C * n_host[b0 + i];
            if (n_host[b0 + i] > most) most = (int)n_host[b0 + i];
        }
        const dim3 grid((unsigned)forge::ceil_div(R, 256 / (most <= 16 ? 1 : most / 16)), (unsigned)nb), block(256);
        const char* w0 = (const char*)W0 + (size_t)(b0 * C * R) * w0_size;
        if (w0_dtype == FORGE_BF16)
            lowrank_sweep_kernel<uint16_t><<<grid, block, 0, st>>>(
                (const uint16_t*)w0, Bp, Hm, scalesT + b0 * G * R, qzerosT + b0 * G * R, g_idx + b0 * C,
                info + b0, qweight + b0 * C * R, C, R, G, maxq, tab);
        else
            lowrank_sweep_kernel<float><<<grid, block, 0, st>>>(
                (const float*)w0, Bp, Hm, scalesT + b0 * G * R, qzerosT + b0 * G * R, g_idx + b0 * C,
                info + b0, qweight + b0 * C * R, C, R, G, maxq, tab);
        FORGE_LAUNCH_CHECK();
    }
    return FORGE_OK;
}

extern "C" int forge_gptq_sweep_lowrank(const void* W0, int w0_dtype, const float* Bp, const float* Hm,
                                        const int32_t* info, const float* scalesT,
                                        const float* qzerosT, const int32_t* g_idx, uint8_t* qweight,
                                        int64_t batch, int64_t C, int64_t R, int64_t G, int bits,
                                        int64_t n, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536, "bad batch=%lld", (long long)batch);
    std::vector<int64_t> ns((size_t)batch, n);
    return forge_gptq_sweep_lowrank_mixed(W0, w0_dtype, Bp, Hm, ns.data(), info, scalesT, qzerosT, g_idx,
                                          qweight, batch, C, R, G, bits, stream);
}
