// Grouped ragged Hessian accumulation  H[e] <- beta[e] H[e] + alpha[e] X_e^T X_e  on gfx950.
//
// Batched form of GPTQ.update (forge/gptq.py:61-80): each group e is one expert's routed
// tokens (rows offsets[e] .. offsets[e+1] of X).  Only tiles on or above the diagonal are
// computed; the mirror image is written from the same registers, so H stays exactly
// symmetric and both triangles are valid, as the reference's full SGEMM leaves them.
//
// bf16 tokens: v_mfma_f32_32x32x16_bf16 (products of bf16 pairs are exact in fp32, the
// accumulation is fp32).  The instruction wants, per lane, 8 consecutive k (tokens) of one
// column, i.e. the transpose of the row-major activations.  A small pack kernel therefore
// rewrites each group's tokens once into "operand panels": for every 32-column tile and
// every 16-token chunk one 1 KiB block whose lane l holds
//     X[chunk*16 + 8*(l/32) + 0..7][tile*32 + l%32]
// so that the rank-k kernel fetches every MFMA operand with one fully coalesced 16-byte
// load per lane and never touches LDS in its K loop.  Tokens are zero padded to a
// multiple of 16 per group.  fp32 tokens use v_mfma_f32_32x32x2_f32 on K-major tiles
// staged through LDS (no transpose needed for that instruction's operand layout).
//
// The diagonal is not taken from the matrix pipe: H[c][c] decides the activation order
// (argsort of diag(H), forge/gptq.py:107-110), and with thousands of columns neighbouring
// diagonal entries lie closer together than the rounding error of an fp32 sum over the
// tokens, so the order -- and through it a few per cent of the codes -- would depend on the
// summation order.  A small kernel sums every column's squares in float64 (the squares of
// bf16 and f32 values are exact there) and the update beta*old + alpha*sum is rounded to
// fp32 once; the rank-k kernels write that value where row == column.
#include "common.h"
#include <type_traits>
#include <hip/hip_bf16.h>
#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct GroupDesc {
    int64_t row0;      // first token row in X
    int64_t pack_off;  // offset (in 16-byte units) of this group's panels in the pack buffer
    int32_t n;         // tokens
    int32_t nchunk;    // ceil(n/16)
    float alpha, beta;
};

// ---------------------------------------------------------------- pack (bf16)
// grid: (col tile of 32, chunk of 16 tokens (strided), group).  One wavefront per block.
__global__ __launch_bounds__(64) void pack_bf16_kernel(const uint16_t* __restrict__ X, int64_t ldx,
                                                       int64_t C, const GroupDesc* __restrict__ gd,
                                                       uint4* __restrict__ pack) {
    const GroupDesc g = gd[blockIdx.z];
    const int lane = threadIdx.x;
    const int64_t ct = blockIdx.x;
    const int64_t col = ct * 32 + (lane & 31);
    for (int kc = blockIdx.y; kc < g.nchunk; kc += gridDim.y) {
        uint16_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t t = (int64_t)kc * 16 + 8 * (lane >> 5) + j;
            v[j] = (t < g.n && col < C) ? X[(g.row0 + t) * ldx + col] : (uint16_t)0;
        }
        uint4 o;
        o.x = v[0] | ((uint32_t)v[1] << 16);
        o.y = v[2] | ((uint32_t)v[3] << 16);
        o.z = v[4] | ((uint32_t)v[5] << 16);
        o.w = v[6] | ((uint32_t)v[7] << 16);
        pack[g.pack_off + (ct * g.nchunk + kc) * 64 + lane] = o;
    }
}

// Decode a linear index over the upper-triangular tile pairs (ti <= tj) of an NT x NT grid.
__device__ __forceinline__ void tile_pair(int p, int NT, int& ti, int& tj) {
    int i = 0, rowlen = NT;
    while (p >= rowlen) { p -= rowlen; ++i; --rowlen; }
    ti = i;
    tj = i + p;
}

// ---------------------------------------------------------------- diagonal in float64
// grid: (128-column slab, group).  Four wavefronts take every fourth token, two adjacent
// columns per lane; partial sums meet in LDS and are added in wavefront order.
// dnew[group][c] = (float)(beta * H[c][c] + alpha * sum_t x[t][c]^2).
template <typename T>
__device__ __forceinline__ double as_double(T v);
template <>
__device__ __forceinline__ double as_double<uint16_t>(uint16_t v) {
    return (double)__uint_as_float((uint32_t)v << 16);
}
template <>
__device__ __forceinline__ double as_double<float>(float v) { return (double)v; }

template <typename T>
__global__ __launch_bounds__(256) void diag_float64_kernel(const T* __restrict__ X, int64_t ldx,
                                                           int64_t C, const GroupDesc* __restrict__ gd,
                                                           const float* __restrict__ Hall,
                                                           float* __restrict__ dnew) {
    __shared__ double part[4][128];
    const GroupDesc g = gd[blockIdx.y];
    if (g.n == 0) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t c0 = (int64_t)blockIdx.x * 128 + 2 * lane;
    const bool in0 = c0 < C, in1 = c0 + 1 < C;
    // columns past the end read column 0 instead and count as zero: unconditional loads, so that
    // the sixteen rows really are in flight together (a load inside a branch is waited for at once)
    const T* __restrict__ col = X + g.row0 * ldx + (in0 ? c0 : 0);
    const int off1 = in1 ? 1 : 0;
    const double m0 = in0 ? 1.0 : 0.0, m1 = in1 ? 1.0 : 0.0;
    double s0 = 0.0, s1 = 0.0;
    int t = wave;
    // sixteen rows in flight per wavefront: a heavy group's columns are walked by ONE workgroup,
    // whose time is the rows' load latency divided by what is in flight
    // (16-bit values are held one per 32-bit register: packed pairs would chain the loads)
    using Held = typename std::conditional<sizeof(T) == 2, uint32_t, T>::type;
    for (; t + 60 < g.n; t += 64) {
        Held a[16], b[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const T* r = col + (int64_t)(t + 4 * u) * ldx;
            a[u] = r[0];
            b[u] = r[off1];
        }
        __builtin_amdgcn_sched_barrier(0);      // all 32 loads are issued before the first is used
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const double x = m0 * as_double<T>((T)a[u]), y = m1 * as_double<T>((T)b[u]);
            s0 = __builtin_fma(x, x, s0);
            s1 = __builtin_fma(y, y, s1);
        }
    }
    for (; t < g.n; t += 4) {
        const T* r = col + (int64_t)t * ldx;
        const double x = m0 * as_double<T>(r[0]), y = m1 * as_double<T>(r[off1]);
        s0 = __builtin_fma(x, x, s0);
        s1 = __builtin_fma(y, y, s1);
    }
    part[wave][2 * lane] = s0;
    part[wave][2 * lane + 1] = s1;
    __syncthreads();
    if (threadIdx.x < 128) {
        const int64_t c = (int64_t)blockIdx.x * 128 + threadIdx.x;
        if (c < C) {
            const double s = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) +
                             part[3][threadIdx.x];
            double o = (double)g.alpha * s;
            if (g.beta != 0.0f)
                o += (double)g.beta * (double)Hall[(int64_t)blockIdx.y * C * C + c * C + c];
            dnew[(int64_t)blockIdx.y * C + c] = (float)o;
        }
    }
}

// Write one 32x32 accumulator tile (and its mirror image) with out = alpha*acc + beta*H.
// Called by all four wavefronts of the workgroup together (it synchronises them).
__device__ __forceinline__ void store_tile(float* __restrict__ H, int64_t C, int row0, int col0,
                                           const f32x16& acc, float alpha, float beta, bool mirror,
                                           float (*tbuf)[33], int lane, const float* __restrict__ dn) {
    f32x16 out;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = row0 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        const int j = col0 + (lane & 31);
        float o = alpha * acc[v];
        if (i < C && j < C) {
            if (i == j) o = dn[i];                     // the float64 diagonal
            else if (beta != 0.0f) o = __builtin_fmaf(beta, H[(int64_t)i * C + j], o);
            H[(int64_t)i * C + j] = o;
        }
        out[v] = o;
    }
    if (mirror) {
#pragma unroll
        for (int v = 0; v < 16; ++v)
            tbuf[(v >> 2) * 8 + (lane >> 5) * 4 + (v & 3)][lane & 31] = out[v];
        __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int jj = (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);   // column of the source tile
            const int i = col0 + jj, j = row0 + (lane & 31);
            if (i < C && j < C) H[(int64_t)i * C + j] = tbuf[lane & 31][jj];
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- rank-k (bf16 MFMA)
// grid: (tile pair, group).  128x128 tile, 4 wavefronts, each 64x64 = 2x2 MFMA tiles.
// BLEND = false: every group has beta == 0 (no old values, fewer registers).
template <bool BLEND>
__global__ __launch_bounds__(256) void syrk_bf16_kernel(const uint4* __restrict__ pack,
                                                        const GroupDesc* __restrict__ gd,
                                                        float* __restrict__ Hall, int64_t C,
                                                        int NT, const float* __restrict__ dnew,
                                                        int n_hi) {
    __shared__ float tbuf[4][32][33];
    const GroupDesc g = gd[blockIdx.y];
    if (g.n == 0 || g.n >= n_hi) return;           // groups with n_hi tokens and more: the kernel below
    int ti, tj;
    tile_pair(blockIdx.x, NT, ti, tj);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    float* __restrict__ H = Hall + (int64_t)blockIdx.y * C * C;
    const float* __restrict__ dn = dnew + (int64_t)blockIdx.y * C;
    const int nct = (int)((C + 31) / 32);

    int cta[2], ctb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        cta[i] = ti * 4 + wm * 2 + i;
        ctb[i] = tj * 4 + wn * 2 + i;
    }
    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

    const uint4* __restrict__ base = pack + g.pack_off + lane;
    const uint4* pa[2];
    const uint4* pb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        pa[i] = base + (int64_t)(cta[i] < nct ? cta[i] : 0) * g.nchunk * 64;
        pb[i] = base + (int64_t)(ctb[i] < nct ? ctb[i] : 0) * g.nchunk * 64;
    }
    // With few token rows per expert the kernel is one pass over H: the old values of a
    // whole tile are requested before the K loop so that their latency overlaps it (and
    // each other), instead of one load-wait-store round trip per accumulator register.
    const bool full = (ti + 1) * 128 <= C && (tj + 1) * 128 <= C;    // uniform
    const bool blend = BLEND && g.beta != 0.0f;
    f32x16 old[2][2];
    if (BLEND && full && blend) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const float* __restrict__ Ht =
                    H + (int64_t)(cta[mi] * 32 + (lane >> 5) * 4) * C + ctb[ni] * 32 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    old[mi][ni][v] = Ht[(int64_t)((v >> 2) * 8 + (v & 3)) * C];
            }
    }
    for (int kc = 0; kc < g.nchunk; ++kc) {
        bf16x8 a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4 ua = pa[i][(int64_t)kc * 64];
            const uint4 ub = pb[i][(int64_t)kc * 64];
            a[i] = *reinterpret_cast<const bf16x8*>(&ua);
            b[i] = *reinterpret_cast<const bf16x8*>(&ub);
        }
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] =
                    __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
    }
    const bool mirror = ti != tj;
    if (full) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const int row0 = cta[mi] * 32, col0 = ctb[ni] * 32;
                f32x16 out;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float o = g.alpha * acc[mi][ni][v];
                    if (BLEND && blend) o = __builtin_fmaf(g.beta, old[mi][ni][v], o);
                    out[v] = o;
                }
                if (row0 == col0) {                     // the float64 diagonal
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        if ((v >> 2) * 8 + (lane >> 5) * 4 + (v & 3) == (lane & 31))
                            out[v] = dn[row0 + (lane & 31)];
                }
                float* __restrict__ Ht = H + (int64_t)(row0 + (lane >> 5) * 4) * C + col0 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) Ht[(int64_t)((v >> 2) * 8 + (v & 3)) * C] = out[v];
                if (mirror) {   // the wavefront's own 32x32 staging tile: no workgroup barrier needed
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        tbuf[wave][(v >> 2) * 8 + (lane >> 5) * 4 + (v & 3)][lane & 31] = out[v];
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    float* __restrict__ Hm = H + (int64_t)(col0 + (lane >> 5) * 4) * C + row0 + (lane & 31);
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int jj = (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                        Hm[(int64_t)((v >> 2) * 8 + (v & 3)) * C] = tbuf[wave][lane & 31][jj];
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                }
            }
    } else {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                store_tile(H, C, cta[mi] * 32, ctb[ni] * 32, acc[mi][ni], g.alpha, g.beta, mirror,
                           tbuf[wave], lane, dn);
    }
}

// ---------------------------------------------------------------- rank-k (bf16 MFMA), many tokens
// For groups with hundreds of tokens and more the kernel above is bound by the path from L2
// to the registers: every wavefront fetches its own operand panels, 16 KiB per workgroup and
// 16-token chunk for 2 x 128^3/8 flops.  Here a workgroup of 8 wavefronts owns a 256 x 256
// tile; per chunk its 16 operand panels (8 column tiles of A, 8 of B, 1 KiB each, already in
// the lane order of the matrix instruction) go through LDS once, one panel of each per
// wavefront, and every wavefront reads the 4 + 2 it needs for its 128 x 64 part (8 matrix
// instructions per 6 LDS reads and 2 global loads).  Two LDS buffers, one barrier per chunk;
// the loads of chunk k+2 are in flight while chunk k is multiplied.
// grid: (pair of 256-column tiles, group); only groups with n_lo <= n tokens are taken, C must
// be a multiple of 256.
constexpr int BIG = 256;
constexpr int kBigTokens = 512;   // groups with this many tokens and more take the kernel below
__global__ __launch_bounds__(512, 1) void syrk_bf16_big_kernel(const uint4* __restrict__ pack,
                                                               const GroupDesc* __restrict__ gd,
                                                               float* __restrict__ Hall, int64_t C,
                                                               int NT2, const float* __restrict__ dnew,
                                                               int n_lo) {
    // two stages of KC chunks x 16 panels; reused as per-wavefront 32 x 33 transposition tiles
    // afterwards
    constexpr int KC = 4;
    __shared__ __attribute__((aligned(16))) uint4 stage[2][KC][16][64];
    const GroupDesc g = gd[blockIdx.y];
    if (g.n < n_lo) return;
    int ti, tj;
    tile_pair(blockIdx.x, NT2, ti, tj);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 2, wn = wave & 3;              // 2 x 4 wavefronts, 128 x 64 each
    float* __restrict__ H = Hall + (int64_t)blockIdx.y * C * C;
    const float* __restrict__ dn = dnew + (int64_t)blockIdx.y * C;

    f32x16 acc[4][2];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

    // this wavefront brings in panel `wave` of A (column tile ti*8 + wave) and of B, KC chunks
    // of 16 tokens per stage; chunks past the group's last one are zeros
    const uint4* __restrict__ srcA = pack + g.pack_off + (int64_t)(ti * 8 + wave) * g.nchunk * 64 + lane;
    const uint4* __restrict__ srcB = pack + g.pack_off + (int64_t)(tj * 8 + wave) * g.nchunk * 64 + lane;
    const int nchunk = g.nchunk;
    const int nstage = (nchunk + KC - 1) / KC;
    uint4 ra[KC], rb[KC];
    auto fetch = [&](int st) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            // (a branch on a wavefront-uniform condition: a select on the loaded value would make
            // the wavefront wait for the load right here instead of one stage later)
            const int chunk = st * KC + c;
            if (chunk < nchunk) {
                ra[c] = srcA[(int64_t)chunk * 64];
                rb[c] = srcB[(int64_t)chunk * 64];
            } else {
                ra[c] = make_uint4(0u, 0u, 0u, 0u);
                rb[c] = make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    auto put = [&](int buf) {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            stage[buf][c][wave][lane] = ra[c];
            stage[buf][c][8 + wave][lane] = rb[c];
        }
    };
    fetch(0);
    put(0);
    if (nstage > 1) fetch(1);
    // Operands of a chunk are read from LDS while the matrix instructions of the chunk before
    // run (two register sets, one LDS read slotted in after each of the first six instructions
    // of a chunk): a wavefront issues in order, so reads issued as a block of their own would
    // leave the matrix pipe waiting for them.
    bf16x8 a[2][4], b[2][2];
#define FORGE_BIG_READ(buf, c, set)                                                             \
    do {                                                                                        \
        _Pragma("unroll") for (int mi = 0; mi < 4; ++mi) {                                      \
            const uint4 u = stage[buf][c][wm * 4 + mi][lane];                                   \
            a[set][mi] = __builtin_bit_cast(bf16x8, u);                                         \
        }                                                                                       \
        _Pragma("unroll") for (int ni = 0; ni < 2; ++ni) {                                      \
            const uint4 u = stage[buf][c][8 + wn * 2 + ni][lane];                               \
            b[set][ni] = __builtin_bit_cast(bf16x8, u);                                         \
        }                                                                                       \
    } while (0)
#define FORGE_BIG_MFMAS(set)                                                                    \
    do {                                                                                        \
        _Pragma("unroll") for (int mi = 0; mi < 4; ++mi) _Pragma("unroll") for (int ni = 0; ni < 2; ++ni) \
            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[set][mi], b[set][ni], acc[mi][ni], \
                                                                  0, 0, 0);                     \
    } while (0)
    for (int st = 0; st < nstage; ++st) {
        const int cur = st & 1;
        __syncthreads();                                   // stage `cur` is complete, `cur^1` is free
        FORGE_BIG_READ(cur, 0, 0);
        if (st + 1 < nstage) put(cur ^ 1);
        if (st + 2 < nstage) fetch(st + 2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            if (c + 1 < KC) FORGE_BIG_READ(cur, c + 1, (c + 1) & 1);
            FORGE_BIG_MFMAS(c & 1);
            if (c + 1 < KC) {
#pragma unroll
                for (int i = 0; i < 6; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#undef FORGE_BIG_READ
#undef FORGE_BIG_MFMAS
    __syncthreads();                                       // the stages become transposition tiles
    float (*tbuf)[33] = reinterpret_cast<float (*)[33]>(reinterpret_cast<float*>(&stage[0][0][0][0]) +
                                                        wave * 32 * 33);
    const bool blend = g.beta != 0.0f;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int row0 = (ti * 8 + wm * 4 + mi) * 32, col0 = (tj * 8 + wn * 2 + ni) * 32;
            if (row0 > col0) continue;                     // below the diagonal: its mirror image writes it
            float* __restrict__ Ht = H + (int64_t)(row0 + (lane >> 5) * 4) * C + col0 + (lane & 31);
            f32x16 out;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float o = g.alpha * acc[mi][ni][v];
                if (blend) o = __builtin_fmaf(g.beta, Ht[(int64_t)((v >> 2) * 8 + (v & 3)) * C], o);
                out[v] = o;
            }
            if (row0 == col0) {                            // the float64 diagonal
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if ((v >> 2) * 8 + (lane >> 5) * 4 + (v & 3) == (lane & 31))
                        out[v] = dn[row0 + (lane & 31)];
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) Ht[(int64_t)((v >> 2) * 8 + (v & 3)) * C] = out[v];
            if (row0 != col0) {                            // mirror image through the wavefront's own tile
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    tbuf[(v >> 2) * 8 + (lane >> 5) * 4 + (v & 3)][lane & 31] = out[v];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                float* __restrict__ Hm = H + (int64_t)(col0 + (lane >> 5) * 4) * C + row0 + (lane & 31);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int jj = (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                    Hm[(int64_t)((v >> 2) * 8 + (v & 3)) * C] = tbuf[lane & 31][jj];
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
}

// ---------------------------------------------------------------- rank-k (f32 MFMA)
// Same tiling; operands are the token rows themselves (K-major), staged through LDS.
constexpr int TK = 16;
__global__ __launch_bounds__(256) void syrk_f32_kernel(const float* __restrict__ X, int64_t ldx,
                                                       const GroupDesc* __restrict__ gd,
                                                       float* __restrict__ Hall, int64_t C, int NT,
                                                       const float* __restrict__ dnew) {
    __shared__ __attribute__((aligned(16))) float As[2][TK][128];
    __shared__ __attribute__((aligned(16))) float Bs[2][TK][128];
    __shared__ float tbuf[4][32][33];
    const GroupDesc g = gd[blockIdx.y];
    if (g.n == 0) return;
    int ti, tj;
    tile_pair(blockIdx.x, NT, ti, tj);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    float* __restrict__ H = Hall + (int64_t)blockIdx.y * C * C;
    const float* __restrict__ Xg = X + g.row0 * ldx;
    const int mt = ti * 128, nt = tj * 128;

    f32x16 acc[2][2], tot[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = tot[mi][ni][v] = 0.0f;

    const int lrow = tid >> 5, lcol = (tid & 31) * 4;
    float4 ra[2], rb[2];
    auto fetch = [&](int kk) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = kk + lrow + 8 * h;
            float va[4] = {0.f, 0.f, 0.f, 0.f}, vb[4] = {0.f, 0.f, 0.f, 0.f};
            if (k < g.n) {
                const float* row = Xg + (int64_t)k * ldx;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (mt + lcol + e < C) va[e] = row[mt + lcol + e];
                    if (nt + lcol + e < C) vb[e] = row[nt + lcol + e];
                }
            }
            ra[h] = make_float4(va[0], va[1], va[2], va[3]);
            rb[h] = make_float4(vb[0], vb[1], vb[2], vb[3]);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<float4*>(&As[buf][lrow + 8 * h][lcol]) = ra[h];
            *reinterpret_cast<float4*>(&Bs[buf][lrow + 8 * h][lcol]) = rb[h];
        }
    };
    int buf = 0;
    fetch(0);
    stage(0);
    __syncthreads();
    for (int kk = 0; kk < g.n; kk += TK) {
        const bool more = kk + TK < g.n;
        if (more) fetch(kk + TK);
#pragma unroll
        for (int kp = 0; kp < TK / 2; ++kp) {
            const int kr = 2 * kp + (lane >> 5);
            float av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                av[i] = As[buf][kr][wm * 64 + i * 32 + (lane & 31)];
                bv[i] = Bs[buf][kr][wn * 64 + i * 32 + (lane & 31)];
            }
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mi], bv[ni], acc[mi][ni],
                                                                       0, 0, 0);
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
        // Blocked summation: the matrix instruction adds its products to the accumulator one
        // after the other, so a single chain over n tokens carries a rounding error that grows
        // like sqrt(n).  Every 128 tokens the chain is folded into a second set of sums.
        if (((kk / TK) & 7) == 7 && more) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        tot[mi][ni][v] += acc[mi][ni][v];
                        acc[mi][ni][v] = 0.0f;
                    }
        }
    }
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] += tot[mi][ni][v];
    const bool mirror = ti != tj;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
            store_tile(H, C, mt + wm * 64 + mi * 32, nt + wn * 64 + ni * 32, acc[mi][ni], g.alpha,
                       g.beta, mirror, tbuf[wave], lane, dnew + (int64_t)blockIdx.y * C);
}

int64_t pack_units(int64_t n, int64_t C) {  // 16-byte units for one group
    return forge::ceil_div(n, 16) * forge::ceil_div(C, 32) * 64;
}

int64_t round256(int64_t b) { return (b + 255) / 256 * 256; }

// Pinned host blocks through which group tables travel to the device.  A call fills a
// block whose previous upload has completed (its event says so), enqueues the copy and
// returns: the host thread never waits for the stream.  Blocks live until the process ends.
struct UploadBlock {
    void* host;
    int64_t bytes;
    hipEvent_t done;
    bool used;
};
std::mutex g_upload_mu;
std::vector<UploadBlock> g_upload;

int upload_async(const void* src, int64_t bytes, void* dst, hipStream_t st) {
    std::lock_guard<std::mutex> lock(g_upload_mu);
    UploadBlock* blk = nullptr;
    for (auto& b : g_upload)
        if (b.bytes >= bytes && (!b.used || hipEventQuery(b.done) == hipSuccess)) {
            blk = &b;
            break;
        }
    if (!blk) {
        UploadBlock b{nullptr, std::max<int64_t>(bytes, 16384), nullptr, false};
        FORGE_HIP_CHECK(hipHostMalloc(&b.host, (size_t)b.bytes, hipHostMallocDefault));
        FORGE_HIP_CHECK(hipEventCreateWithFlags(&b.done, hipEventDisableTiming));
        g_upload.push_back(b);
        blk = &g_upload.back();
    }
    memcpy(blk->host, src, (size_t)bytes);
    FORGE_HIP_CHECK(hipMemcpyAsync(dst, blk->host, (size_t)bytes, hipMemcpyHostToDevice, st));
    FORGE_HIP_CHECK(hipEventRecord(blk->done, st));
    blk->used = true;
    return FORGE_OK;
}

// The launches of one update; gd_dev already holds the group table.
int launch_update(const void* X, int x_dtype, int64_t ldx, int64_t C, const GroupDesc* gd_dev,
                  int64_t n_groups, int64_t total, int max_chunks, int min_tokens, bool any_blend,
                  float* H, float* dnew, uint4* pack, hipStream_t st, bool timed = true) {
    const int NT = (int)forge::ceil_div(C, 128);
    const unsigned pairs = (unsigned)(NT * (NT + 1) / 2);
    const dim3 dgrid((unsigned)NT, (unsigned)n_groups);
    if (x_dtype == FORGE_BF16) {
        // one record for the whole update (diagonal, operand panels, rank-k kernels); executed
        // flops: tiles on and above the diagonal only
        forge::KernelTiming timing(timed ? "hessian_syrk_bf16" : nullptr, st,
                                   2.0 * (double)total * 128.0 * 128.0 * (double)pairs,
                                   forge::WORK_FLOPS);
        diag_float64_kernel<uint16_t><<<dgrid, dim3(256), 0, st>>>((const uint16_t*)X, ldx, C, gd_dev,
                                                                   H, dnew);
        FORGE_LAUNCH_CHECK();
        const unsigned ychunks = (unsigned)(max_chunks < 64 ? max_chunks : 64);
        pack_bf16_kernel<<<dim3((unsigned)forge::ceil_div(C, 32), ychunks, (unsigned)n_groups),
                           dim3(64), 0, st>>>((const uint16_t*)X, ldx, C, gd_dev, pack);
        FORGE_LAUNCH_CHECK();
        // groups with many tokens take the 256 x 256 workgroup tiles (operands shared through
        // LDS), the others the one-pass kernel that overlaps the old tile's loads with its K loop
        const bool big = (C % BIG) == 0 && max_chunks * 16 >= kBigTokens;
        const int n_split = big ? kBigTokens : (1 << 30);
        if (max_chunks * 16 < kBigTokens || !big || min_tokens < kBigTokens) {
            if (any_blend)
                syrk_bf16_kernel<true><<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(
                    pack, gd_dev, H, C, NT, dnew, n_split);
            else
                syrk_bf16_kernel<false><<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(
                    pack, gd_dev, H, C, NT, dnew, n_split);
            FORGE_LAUNCH_CHECK();
        }
        if (big) {
            const int NT2 = (int)(C / BIG);
            syrk_bf16_big_kernel<<<dim3((unsigned)(NT2 * (NT2 + 1) / 2), (unsigned)n_groups), dim3(512), 0,
                                   st>>>(pack, gd_dev, H, C, NT2, dnew, n_split);
            FORGE_LAUNCH_CHECK();
        }
    } else {
        forge::KernelTiming timing(timed ? "hessian_syrk_f32" : nullptr, st,
                                   2.0 * (double)total * 128.0 * 128.0 * (double)pairs,
                                   forge::WORK_FLOPS);
        diag_float64_kernel<float><<<dgrid, dim3(256), 0, st>>>((const float*)X, ldx, C, gd_dev, H,
                                                                dnew);
        FORGE_LAUNCH_CHECK();
        syrk_f32_kernel<<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(
            (const float*)X, ldx, gd_dev, H, C, NT, dnew);
        FORGE_LAUNCH_CHECK();
    }
    return FORGE_OK;
}

// ---------------------------------------------------------------- entry point without allocation
// Device memory of the library's own for forge_hessian_update_static: one group table entry,
// the float64-summed diagonal and the bf16 operand panels.  Every GPU the library runs on
// holds its own copy at its own address until the process ends.
constexpr int64_t STATIC_MAX_C = 16384;
constexpr int64_t STATIC_PACK_BYTES = 32ll << 20;
constexpr int64_t STATIC_DESC_BYTES = 256;
constexpr int64_t STATIC_BYTES = STATIC_DESC_BYTES + STATIC_MAX_C * 4 + STATIC_PACK_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_static_mu;
void* g_static_ptr[MAX_DEVICES] = {nullptr};

// Address of `scratch` on the current device (looked up once per device; in host code the
// array's name is only a handle for this lookup, never an address).
int static_scratch(unsigned char** out) {
    int dev = -1;
    FORGE_HIP_CHECK(hipGetDevice(&dev));
    FORGE_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "device index %d not supported", dev);
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_ptr[dev]) {
        void* p = nullptr;
        FORGE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        FORGE_REQUIRE(p != nullptr, "no device address for the static workspace");
        g_static_ptr[dev] = p;
    }
    *out = (unsigned char*)g_static_ptr[dev];
    return FORGE_OK;
}

__global__ void write_desc_kernel(GroupDesc* __restrict__ gd, GroupDesc v) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *gd = v;
}

}  // namespace

extern "C" int64_t forge_hessian_workspace_bytes(int64_t total_rows, int64_t n_groups, int64_t C,
                                                 int x_dtype) {
    if (n_groups <= 0 || C <= 0) return 0;
    int64_t bytes = round256(n_groups * (int64_t)sizeof(GroupDesc)) + round256(n_groups * C * 4);
    if (x_dtype == FORGE_BF16) bytes += pack_units(total_rows + 16 * n_groups, C) * 16;
    return bytes;
}

// Shared body of the two grouped entry points: group e = rows row0[e] .. row0[e] + n[e] - 1.
static int update_ranges(const void* X, int x_dtype, int64_t ldx, int64_t C, const int64_t* row0_host,
                         const int64_t* n_host, int64_t n_groups, const float* alpha_host,
                         const float* beta_host, float* H, void* ws, int64_t ws_bytes,
                         hipStream_t st) {
    std::vector<GroupDesc> gd((size_t)n_groups);
    int64_t off = 0, total = 0;
    int max_chunks = 0, min_tokens = 1 << 30;
    bool any = false, any_blend = false;
    for (int64_t e = 0; e < n_groups; ++e) {
        const int64_t n = n_host[e];
        FORGE_REQUIRE(n >= 0 && n < (1LL << 31) && row0_host[e] >= 0, "bad row range of group %lld",
                      (long long)e);
        gd[e].row0 = row0_host[e];
        gd[e].n = (int32_t)n;
        gd[e].nchunk = (int32_t)forge::ceil_div(n, 16);
        gd[e].pack_off = off;
        gd[e].alpha = alpha_host[e];
        gd[e].beta = beta_host[e];
        off += pack_units(n, C);
        total += n;
        if (gd[e].nchunk > max_chunks) max_chunks = gd[e].nchunk;
        if (n > 0 && n < min_tokens) min_tokens = (int)n;
        any |= n > 0;
        any_blend |= n > 0 && beta_host[e] != 0.0f;
    }
    if (!any) return FORGE_OK;
    FORGE_REQUIRE(X, "X is null");
    FORGE_REQUIRE(ws_bytes >= forge_hessian_workspace_bytes(total, n_groups, C, x_dtype),
                  "workspace too small");
    GroupDesc* gd_dev = (GroupDesc*)ws;
    const int64_t desc_bytes = round256(n_groups * (int64_t)sizeof(GroupDesc));
    float* dnew = (float*)((char*)ws + desc_bytes);
    uint4* pack = (uint4*)((char*)ws + desc_bytes + round256(n_groups * C * 4));
    // through a pinned block of the library's own: the host does not wait for the copy
    if (int rc = upload_async(gd.data(), n_groups * (int64_t)sizeof(GroupDesc), gd_dev, st)) return rc;
    return launch_update(X, x_dtype, ldx, C, gd_dev, n_groups, total, max_chunks, min_tokens, any_blend,
                         H, dnew, pack, st);
}

extern "C" int forge_hessian_update_grouped(const void* X, int x_dtype, int64_t ldx, int64_t C,
                                            const int64_t* offsets_host, int64_t n_groups,
                                            const float* alpha_host, const float* beta_host,
                                            float* H, void* ws, int64_t ws_bytes,
                                            forge_stream_t stream) {
    FORGE_REQUIRE(x_dtype == FORGE_F32 || x_dtype == FORGE_BF16, "x_dtype=%d", x_dtype);
    FORGE_REQUIRE(n_groups >= 0 && n_groups < 65536 && C >= 1 && C < (1 << 24) && ldx >= C,
                  "bad shape n_groups=%lld C=%lld ldx=%lld", (long long)n_groups, (long long)C,
                  (long long)ldx);
    if (n_groups == 0) return FORGE_OK;
    FORGE_REQUIRE(offsets_host && alpha_host && beta_host && H && ws, "null pointer");
    std::vector<int64_t> n((size_t)n_groups);
    for (int64_t e = 0; e < n_groups; ++e) {
        n[e] = offsets_host[e + 1] - offsets_host[e];
        FORGE_REQUIRE(n[e] >= 0, "offsets must be non-decreasing");
    }
    return update_ranges(X, x_dtype, ldx, C, offsets_host, n.data(), n_groups, alpha_host, beta_host, H,
                         ws, ws_bytes, (hipStream_t)stream);
}

extern "C" int forge_hessian_update_ranges(const void* X, int x_dtype, int64_t ldx, int64_t C,
                                           const int64_t* row0_host, const int64_t* n_host,
                                           int64_t n_groups, const float* alpha_host,
                                           const float* beta_host, float* H, void* ws,
                                           int64_t ws_bytes, forge_stream_t stream) {
    FORGE_REQUIRE(x_dtype == FORGE_F32 || x_dtype == FORGE_BF16, "x_dtype=%d", x_dtype);
    FORGE_REQUIRE(n_groups >= 0 && n_groups < 65536 && C >= 1 && C < (1 << 24) && ldx >= C,
                  "bad shape n_groups=%lld C=%lld ldx=%lld", (long long)n_groups, (long long)C,
                  (long long)ldx);
    if (n_groups == 0) return FORGE_OK;
    FORGE_REQUIRE(row0_host && n_host && alpha_host && beta_host && H && ws, "null pointer");
    return update_ranges(X, x_dtype, ldx, C, row0_host, n_host, n_groups, alpha_host, beta_host, H, ws,
                         ws_bytes, (hipStream_t)stream);
}

extern "C" int64_t forge_hessian_update_static_max_rows(int64_t C, int x_dtype) {
    if (C < 1 || C > STATIC_MAX_C) return 0;
    if (x_dtype != FORGE_BF16) return (1LL << 31) - 1;
    const int64_t chunks = STATIC_PACK_BYTES / (forge::ceil_div(C, 32) * 64 * 16);
    return chunks * 16;
}

extern "C" int forge_hessian_update_static(const void* X, int x_dtype, int64_t ldx, int64_t n_rows,
                                           int64_t C, float alpha, float beta, float* H,
                                           forge_stream_t stream) {
    FORGE_REQUIRE(x_dtype == FORGE_F32 || x_dtype == FORGE_BF16, "x_dtype=%d", x_dtype);
    FORGE_REQUIRE(C >= 1 && ldx >= C && n_rows >= 0, "bad shape n_rows=%lld C=%lld ldx=%lld",
                  (long long)n_rows, (long long)C, (long long)ldx);
    FORGE_REQUIRE(C <= STATIC_MAX_C, "C=%lld exceeds the static workspace's limit of %lld columns",
                  (long long)C, (long long)STATIC_MAX_C);
    FORGE_REQUIRE(n_rows <= forge_hessian_update_static_max_rows(C, x_dtype),
                  "n_rows=%lld exceeds the static workspace's limit of %lld rows at C=%lld "
                  "(use forge_hessian_update_grouped with a workspace of the caller's)",
                  (long long)n_rows, (long long)forge_hessian_update_static_max_rows(C, x_dtype),
                  (long long)C);
    if (n_rows == 0) return FORGE_OK;
    FORGE_REQUIRE(X && H, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    unsigned char* base = nullptr;
    if (int rc = static_scratch(&base)) return rc;
    GroupDesc* gd_dev = (GroupDesc*)base;
    float* dnew = (float*)(base + STATIC_DESC_BYTES);
    uint4* pack = (uint4*)(base + STATIC_DESC_BYTES + STATIC_MAX_C * 4);
    GroupDesc g;
    g.row0 = 0;
    g.pack_off = 0;
    g.n = (int32_t)n_rows;
    g.nchunk = (int32_t)forge::ceil_div(n_rows, 16);
    g.alpha = alpha;
    g.beta = beta;
    // the table entry travels as a kernel argument: no staging buffer, nothing to allocate
    write_desc_kernel<<<dim3(1), dim3(64), 0, st>>>(gd_dev, g);
    FORGE_LAUNCH_CHECK();
    return launch_update(X, x_dtype, ldx, C, gd_dev, 1, n_rows, g.nchunk, (int)n_rows, beta != 0.0f, H,
                         dnew, pack, st, /*timed=*/false);
}
