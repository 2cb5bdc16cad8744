// fp32 GEMM on the gfx950 matrix cores with a defined summation order.
//
// v_mfma_f32_32x32x2_f32 computes, for each output element, acc = fma(a[k], b[k], acc)
// for its two k values one after the other, in fp32 with round-to-nearest.  Chaining the
// instruction over ascending k therefore reproduces, bit for bit, the scalar recurrence
//     for k: x = fmaf(a_k, b_k, x)
// which is exactly how the GPTQ sweep propagates quantisation errors.  The same kernel
// serves the Cholesky / triangular-inverse updates, where only fp32 accuracy matters.
//
// Tile: 128 (m) x 128 (n) per workgroup of 4 wavefronts; each wavefront owns a 64x64
// quadrant = 2x2 MFMA tiles (64 accumulator registers).  Operands are K-major in memory,
// so a half-wavefront reads 32 consecutive floats of one k row: global loads are
// coalesced float4, LDS reads are conflict-free ds_read_b32, and no transpose is needed.
// K advances 32 rows per LDS stage, as two sub-stages of 16 rows (32 MFMAs each).
//
// Two kernels share this layout (a third, split_gemm_kernel further down, does the
// factorisation's blocked sums on the bf16 matrix pipe and has its own layout).
// chain_gemm_fast_kernel handles full, aligned tiles and
// is a software pipeline: while the MFMAs of one sub-stage run, the wavefront issues the
// LDS reads of the next sub-stage, the LDS writes of the next stage and the global loads
// of the stage after that, one memory instruction between two MFMAs (a wavefront issues
// in order, so memory instructions issued in a block of their own leave the matrix pipe
// idle for their whole issue time).  chain_gemm_kernel<EDGE> is the simple, bounds-checked
// form for ragged shapes.
#include "chain_gemm.h"
#include <cstdlib>
#include <type_traits>

namespace forge {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int TM = 128, TN = 128;
#ifndef FORGE_GEMM_TK
#define FORGE_GEMM_TK 32
#endif
constexpr int TK = FORGE_GEMM_TK;   // k rows per LDS stage
constexpr int NH = TK / 8;          // float4 loads per thread, operand and stage

// The simple form.  EDGE: bounds-checked loads/stores for tiles that stick out of
// [m0,m1) x [n0,n1), a K range that is not a multiple of 32, or rows that are not 16-byte
// aligned (the launcher only uses EDGE = true; full tiles go to chain_gemm_fast_kernel).  CHUNK > 0: every CHUNK k values the running
// accumulators are folded into a second set and restarted from zero (blocked summation:
// the rounding error of each fma is then relative to a short partial sum instead of the
// whole accumulated value).  Used where only accuracy matters; CHUNK == 0 is the single
// chain that the sweep's bit-exactness needs.
template <bool EDGE, int CHUNK>
__global__ __launch_bounds__(256, 2) void chain_gemm_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) float As[2][TK][TM];
    __shared__ __attribute__((aligned(16))) float Bs[2][TK][TN];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // 1-D grid -> (n tile, m tile, matrix).  Workgroups are handed to the 8 XCDs round
    // robin by linear id, and each XCD has its own L2.  With xcd_map, matrix e is served
    // by XCD e % 8 only, so the At panel that all of its tiles share is fetched into one L2
    // once instead of into all eight.
    const int per_matrix = g.n_tiles * g.m_tiles;
    int bz, tile;
    if (g.xcd_map) {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        bz = xcd + 8 * (slot / per_matrix);
        tile = slot % per_matrix;
    } else {
        bz = blockIdx.x / per_matrix;
        tile = blockIdx.x % per_matrix;
    }
    float* __restrict__ X = g.X + (int64_t)bz * g.xs;
    const float* __restrict__ At = g.At + (int64_t)bz * g.as;
    const float* __restrict__ Bm = g.Bm + (int64_t)bz * g.bs;
    const int mt = g.m0 + (tile / g.n_tiles) * TM;  // first m of this tile
    // triangular operand: K grows with n, so hand out the long tiles first
    const int tn = g.b_upper_tri ? g.n_tiles - 1 - tile % g.n_tiles : tile % g.n_tiles;
    const int nt = g.n0 + tn * TN;                  // first n of this tile
    int k0 = g.k0, k1 = g.k1;
    if (g.lim != nullptr) {   // uniform over the workgroup; before any barrier
        const int own = g.lim[bz];
        if ((g.lim_m && mt >= own) || (g.lim_n && nt >= own)) return;
        if (g.lim_k && k1 > own) k1 = own;
    }
    if (g.b_upper_tri && k1 > nt + TN) k1 = nt + TN;
    if (g.b_lower_tri && k0 < nt) k0 = nt;

    // element (v, lane) of MFMA tile (mi, ni) <-> X[m_base + mi*32 + row(v), n_base + ni*32]
    const int m_base = mt + wm * 64 + (lane >> 5) * 4;
    const int n_base = nt + wn * 64 + (lane & 31);
    float* __restrict__ Xw = X + (int64_t)m_base * g.ldx + n_base;

    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int dm = mi * 32 + (v >> 2) * 8 + (v & 3), dn = ni * 32;
                float x = 0.0f;
                if (!g.init_zero && (!EDGE || (m_base + dm < g.m1 && n_base + dn < g.n1)))
                    x = Xw[(int64_t)dm * g.ldx + dn];
                acc[mi][ni][v] = x;
            }
    f32x16 tot[2][2];
    if constexpr (CHUNK > 0) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                tot[mi][ni] = acc[mi][ni];
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;
            }
    }

    // global -> LDS staging: thread loads k rows (tid>>5) and (tid>>5)+8, 4 columns each
    const int lrow = tid >> 5, lcol = (tid & 31) * 4;
    const float sign = g.negate_a ? -1.0f : 1.0f;
    const float* pa = At + (int64_t)(k0 + lrow) * g.lda + mt + lcol;
    const float* pb = Bm + (int64_t)(k0 + lrow) * g.ldb + nt + lcol;
    const int64_t a_step8 = 8 * g.lda, b_step8 = 8 * g.ldb;
    float4 ra[NH], rb[NH];
    auto fetch = [&](int kk) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            float4 va, vb;
            if constexpr (!EDGE) {
                va = *reinterpret_cast<const float4*>(pa + h * a_step8);
                vb = *reinterpret_cast<const float4*>(pb + h * b_step8);
            } else {
                va = make_float4(0.f, 0.f, 0.f, 0.f);
                vb = va;
                if (kk + lrow + 8 * h < k1) {
                    const float* qa = pa + h * a_step8;
                    const float* qb = pb + h * b_step8;
                    if (mt + lcol + 0 < g.m1) va.x = qa[0];
                    if (mt + lcol + 1 < g.m1) va.y = qa[1];
                    if (mt + lcol + 2 < g.m1) va.z = qa[2];
                    if (mt + lcol + 3 < g.m1) va.w = qa[3];
                    if (nt + lcol + 0 < g.n1) vb.x = qb[0];
                    if (nt + lcol + 1 < g.n1) vb.y = qb[1];
                    if (nt + lcol + 2 < g.n1) vb.z = qb[2];
                    if (nt + lcol + 3 < g.n1) vb.w = qb[3];
                }
            }
            ra[h] = va;
            rb[h] = vb;
        }
        pa += NH * a_step8;
        pb += NH * b_step8;
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            // the sign is applied here, not in fetch(): a use right after the loads would
            // make the wavefront wait out their latency before its first MFMA
            *reinterpret_cast<float4*>(&As[buf][lrow + 8 * h][lcol]) =
                make_float4(sign * ra[h].x, sign * ra[h].y, sign * ra[h].z, sign * ra[h].w);
            *reinterpret_cast<float4*>(&Bs[buf][lrow + 8 * h][lcol]) = rb[h];
        }
    };

    const int a_off = wm * 64 + (lane & 31), b_off = wn * 64 + (lane & 31), kr0 = lane >> 5;
    int buf = 0;
    if (k0 < k1) {
        fetch(k0);
        stage(0);
    }
    __syncthreads();
    int stage_no = 0;
    for (int kk = k0; kk < k1; kk += TK) {
        const bool more = kk + TK < k1;
        if (more) fetch(kk + TK);
        // 16 k rows (8 MFMA k-pairs) at a time: all their LDS reads first, then 32 MFMAs
#pragma unroll
        for (int sub = 0; sub < TK / 16; ++sub) {
            float av[8][2], bv[8][2];
#pragma unroll
            for (int kp = 0; kp < 8; ++kp)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    av[kp][i] = As[buf][sub * 16 + 2 * kp + kr0][a_off + i * 32];
                    bv[kp][i] = Bs[buf][sub * 16 + 2 * kp + kr0][b_off + i * 32];
                }
            // keep every LDS read ahead of its MFMAs (the scheduler would otherwise sink
            // each read next to its use and expose the LDS latency 8 times)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kp = 0; kp < 8; ++kp)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[kp][mi], bv[kp][ni],
                                                                           acc[mi][ni], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (CHUNK > 0) {
            if (++stage_no == CHUNK / TK) {
                stage_no = 0;
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni) {
                        tot[mi][ni] += acc[mi][ni];
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;
                    }
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if constexpr (CHUNK > 0) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = tot[mi][ni] + acc[mi][ni];
    }

#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int dm = mi * 32 + (v >> 2) * 8 + (v & 3), dn = ni * 32;
                if (!EDGE || (m_base + dm < g.m1 && n_base + dn < g.n1))
                    Xw[(int64_t)dm * g.ldx + dn] = acc[mi][ni][v];
            }
}


// Full 128x128 tiles, 16-byte aligned rows, K range a multiple of 32 (after triangular
// clipping).  One stage s of the K loop:
//   region A   32 MFMAs on operand set 0 (sub-stage 0 of stage s)
//              | 16 LDS reads: operand set 1 (sub-stage 1 of stage s)
//              | 8 LDS writes: stage s+1 from registers into the other LDS buffer
//   barrier
//   region B   32 MFMAs on operand set 1
//              | 8 global loads: stage s+2 into registers
//              | 16 LDS reads: operand set 0 of stage s+1
// A negated A operand is folded into the sign of the accumulator on the way in and out:
// fma(-a, b, x) == -fma(a, b, -x) exactly, so the result is the same chain bit for bit.
// A launch carries one or two independent problems (GemmPair): workgroups below
// first_wgs work on `first`, the rest on `second`, so that two under-filled or ragged-ended
// problems share one grid.
// SPI = stages per loop iteration.  4 (K a multiple of 128): the LDS buffer of every stage
// is a compile-time constant, so no address is computed in the loop at all, and with CHUNK =
// 128 the first MFMAs of a chunk take C = 0 (no registers to clear) and the chunk is folded
// into the totals once per iteration.  1: any K that is a multiple of 32 (CHUNK = 0 only).
template <int CHUNK, int SPI>
__global__ __launch_bounds__(256, 2) void chain_gemm_fast_kernel(GemmPair pair) {
    static_assert(TK == 32, "two 16-row sub-stages per stage");
    static_assert(SPI == 1 || SPI == 4, "one stage or one 128-row chunk per iteration");
    static_assert(CHUNK == 0 || (CHUNK == SPI * TK), "a chunk is one loop iteration");
    const bool in_first = blockIdx.x < (unsigned)pair.first_wgs;
    const GemmArgs& g = in_first ? pair.first : pair.second;
    const int wg = in_first ? (int)blockIdx.x : (int)blockIdx.x - pair.first_wgs;
    __shared__ __attribute__((aligned(16))) float As[2][TK][TM];
    __shared__ __attribute__((aligned(16))) float Bs[2][TK][TN];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int per_matrix = g.n_tiles * g.m_tiles;
    int bz, tile;
    if (g.xcd_map) {  // first_wgs is then a multiple of 8, so wg & 7 is still the XCD
        const int xcd = wg & 7, slot = wg >> 3;
        bz = xcd + 8 * (slot / per_matrix);
        tile = slot % per_matrix;
    } else {
        bz = wg / per_matrix;
        tile = wg % per_matrix;
    }
    float* __restrict__ X = g.X + (int64_t)bz * g.xs;
    const float* __restrict__ At = g.At + (int64_t)bz * g.as;
    const float* __restrict__ Bm = g.Bm + (int64_t)bz * g.bs;
    const int mt = g.m0 + (tile / g.n_tiles) * TM;
    const int tn = g.b_upper_tri ? g.n_tiles - 1 - tile % g.n_tiles : tile % g.n_tiles;
    const int nt = g.n0 + tn * TN;
    int k0 = g.k0, k1 = g.k1;
    if (g.lim != nullptr) {   // uniform over the workgroup; before any barrier
        const int own = g.lim[bz];
        if ((g.lim_m && mt >= own) || (g.lim_n && nt >= own)) return;
        if (g.lim_k && k1 > own) k1 = own;
    }
    if (g.b_upper_tri && k1 > nt + TN) k1 = nt + TN;
    if (g.b_lower_tri && k0 < nt) k0 = nt;

    const int m_base = mt + wm * 32 + (lane >> 5) * 4;
    const int n_base = nt + wn * 32 + (lane & 31);
    float* __restrict__ Xw = X + (int64_t)m_base * g.ldx + n_base;
    const float sgn = g.negate_a ? -1.0f : 1.0f;

    // One branch around all 64 loads: tested per element, every load would be followed by
    // its own wait and the tile would start 64 memory latencies late.
    f32x16 acc[2][2];
    if (g.init_zero) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;
    } else {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int dm = mi * 64 + (v >> 2) * 8 + (v & 3), dn = ni * 64;
                    acc[mi][ni][v] = Xw[(int64_t)dm * g.ldx + dn];
                }
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) acc[mi][ni] *= sgn;
    }
    f32x16 tot[2][2];   // CHUNK > 0: running totals; acc then holds one chunk at a time
    if constexpr (CHUNK > 0) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) tot[mi][ni] = acc[mi][ni];
    }

    if (k0 < k1) {  // uniform over the workgroup
        // global -> LDS staging: thread loads k rows (tid>>5) + 8h, 4 columns each, as
        // buffer loads: one resource descriptor per operand (scalar registers), per-thread
        // byte offsets that never change and a scalar offset that advances with k.  The
        // fp32 MFMA executes on the vector ALU's multipliers, so every vector instruction in
        // this loop (address arithmetic included) takes time from it; with this addressing
        // and the LDS reads below the loop has six of them per 64 MFMAs.
        // (The eight 16-byte registers are named scalars on purpose: as an array captured
        // by a lambda the compiler kept part of them in memory.)
        const int lrow = tid >> 5, lcol = (tid & 31) * 4;
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(At + (int64_t)k0 * g.lda + mt), 0, 0x7FFFFFFF, 0x00027000);
        const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(Bm + (int64_t)k0 * g.ldb + nt), 0, 0x7FFFFFFF, 0x00027000);
        const int a8 = (int)(8 * g.lda * 4), b8 = (int)(8 * g.ldb * 4);
        const int ao0 = (int)(((int64_t)lrow * g.lda + lcol) * 4), ao1 = ao0 + a8, ao2 = ao0 + 2 * a8,
                  ao3 = ao0 + 3 * a8;
        const int bo0 = (int)(((int64_t)lrow * g.ldb + lcol) * 4), bo1 = bo0 + b8, bo2 = bo0 + 2 * b8,
                  bo3 = bo0 + 3 * b8;
        int a_soff = 0, b_soff = 0;
        u32x4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
#define FORGE_GEMM_FETCH()                                                      \
    do {                                                                        \
        ra0 = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, ao0, a_soff, 0);    \
        rb0 = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, bo0, b_soff, 0);    \
        ra1 = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, ao1, a_soff, 0);    \
        rb1 = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, bo1, b_soff, 0);    \
        ra2 = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, ao2, a_soff, 0);    \
        rb2 = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, bo2, b_soff, 0);    \
        ra3 = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, ao3, a_soff, 0);    \
        rb3 = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, bo3, b_soff, 0);    \
        a_soff += a_adv;                                                        \
        b_soff += b_adv;                                                        \
    } while (0)
#define FORGE_GEMM_STAGE(buf)                                           \
    do {                                                                \
        *reinterpret_cast<u32x4*>(&As[buf][lrow][lcol]) = ra0;         \
        *reinterpret_cast<u32x4*>(&Bs[buf][lrow][lcol]) = rb0;         \
        *reinterpret_cast<u32x4*>(&As[buf][lrow + 8][lcol]) = ra1;     \
        *reinterpret_cast<u32x4*>(&Bs[buf][lrow + 8][lcol]) = rb1;     \
        *reinterpret_cast<u32x4*>(&As[buf][lrow + 16][lcol]) = ra2;    \
        *reinterpret_cast<u32x4*>(&Bs[buf][lrow + 16][lcol]) = rb2;    \
        *reinterpret_cast<u32x4*>(&As[buf][lrow + 24][lcol]) = ra3;    \
        *reinterpret_cast<u32x4*>(&Bs[buf][lrow + 24][lcol]) = rb3;    \
    } while (0)

        // The two MFMA tiles of a wavefront sit 64 columns apart (rows wm*32.. and 64+wm*32..
        // of the tile), so both values of a k-pair are one ds_read2st64_b32 and every read of
        // a stage is the lane's base address plus an immediate offset.
        const int kr0 = lane >> 5;
        const float* a_lane = &As[0][kr0][wm * 32 + (lane & 31)];
        const float* b_lane = &Bs[0][kr0][wn * 32 + (lane & 31)];
        float av0[8][2], bv0[8][2], av1[8][2], bv1[8][2];
        auto read_ops = [&](int buf, int sub, float (&av)[8][2], float (&bv)[8][2]) {
            const float* ap = a_lane + buf * (TK * TM);
            const float* bp = b_lane + buf * (TK * TN);
#pragma unroll
            for (int kp = 0; kp < 8; ++kp)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    av[kp][i] = ap[(sub * 16 + 2 * kp) * TM + i * 64];
                    bv[kp][i] = bp[(sub * 16 + 2 * kp) * TN + i * 64];
                }
        };
        // fresh: the accumulators start a new chunk, the first k-pair takes C = 0
        auto mfmas = [&](const float (&av)[8][2], const float (&bv)[8][2], auto fresh) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kp = 0; kp < 8; ++kp)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            av[kp][mi], bv[kp][ni],
                            (decltype(fresh)::value && kp == 0) ? zero : acc[mi][ni], 0, 0, 0);
        };

        // Every fetch reads rows below k1: the pointers advance only while a further stage
        // exists; past the end the last stage is fetched again and never used.
        const int a_full = 4 * a8, b_full = 4 * b8;                  // 32 rows, in bytes
        int a_adv = (k0 + TK < k1) ? a_full : 0, b_adv = (k0 + TK < k1) ? b_full : 0;
        FORGE_GEMM_FETCH();
        FORGE_GEMM_STAGE(0);
        __syncthreads();
        read_ops(0, 0, av0, bv0);
        if (k0 + 2 * TK >= k1) { a_adv = 0; b_adv = 0; }
        FORGE_GEMM_FETCH();

        // One stage; `buf` is a compile-time constant when the caller passes one.
        auto stage_body = [&](auto buf, int kk, auto fresh) {
            // ---- region A.  The group barriers give the order "MFMA, memory instruction,
            // MFMA, ..."; the plain barriers keep instructions from leaving their region.
            read_ops(buf, 1, av1, bv1);
            mfmas(av0, bv0, fresh);
            FORGE_GEMM_STAGE(buf ^ 1);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            // ---- region B
            read_ops(buf ^ 1, 0, av0, bv0);
            if (kk + 3 * TK >= k1) { a_adv = 0; b_adv = 0; }
            mfmas(av1, bv1, std::false_type{});
            FORGE_GEMM_FETCH();
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 1);  // one global load
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 1);
            __builtin_amdgcn_sched_barrier(0);
        };
        if constexpr (SPI == 1) {
            int buf = 0;
            for (int kk = k0; kk < k1; kk += TK) {
                stage_body(buf, kk, std::false_type{});
                buf ^= 1;
            }
        } else {
            using B0 = std::integral_constant<int, 0>;
            using B1 = std::integral_constant<int, 1>;
            for (int kk = k0; kk < k1; kk += 4 * TK) {
                stage_body(B0{}, kk, std::integral_constant<bool, (CHUNK > 0)>{});
                stage_body(B1{}, kk + TK, std::false_type{});
                stage_body(B0{}, kk + 2 * TK, std::false_type{});
                stage_body(B1{}, kk + 3 * TK, std::false_type{});
                if constexpr (CHUNK > 0) {
#pragma unroll
                    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                        for (int ni = 0; ni < 2; ++ni) tot[mi][ni] += acc[mi][ni];
                }
            }
        }
#undef FORGE_GEMM_FETCH
#undef FORGE_GEMM_STAGE
    }
    if constexpr (CHUNK > 0) {   // every chunk has been folded already
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = tot[mi][ni];
    }

#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int dm = mi * 64 + (v >> 2) * 8 + (v & 3), dn = ni * 64;
                Xw[(int64_t)dm * g.ldx + dn] = sgn * acc[mi][ni][v];
            }
}


// ---------------------------------------------------------------------------------------
// Blocked-sum GEMM on the bf16 matrix pipe ("bf16x3").  Used where only fp32 ACCURACY is
// needed (the factorisation's trailing updates), never for the sweep's bit-exact chain.
//
// Every fp32 operand is cut, by truncation, into three bf16 pieces a = a1 + a2 + a3 (exact:
// 8 + 8 + 8 significant bits), and a*b is summed from the six piece products of weight
// >= 2^-16, smallest first: (3,1) (1,3) (2,2) (2,1) (1,2) (1,1), accumulated in fp32 by
// v_mfma_f32_32x32x16_bf16.  The dropped products are below 2^-24 |a b|, and the accumulators
// are folded into running totals every 128 k like the fp32 blocked sum, so the error is that
// of an fp32 dot product.  Six bf16 MFMAs do the work of sixteen fp32 ones.
//
// Two-piece forms of the same kernel (template parameters NP, NPROD, HALF, MT below): two bf16
// pieces each rounded to nearest with three products (~2^-17), and two fp16 halves of operands
// scaled by powers of two with three products (fp32-grade); with two pieces one workgroup can
// compute both m tiles of a 256-row problem (MT = 2).  What the matrix pipe sustains is set by
// the device's power management (about two thirds of the nominal rate on operands with random
// bits), so the kernel's job is to keep the pipe issuing and everything else out of its way.
//
// The fp32 matrix instruction shares the vector ALU, the bf16 one does not, so here the
// split arithmetic has somewhere to run; but a wavefront that holds 128 accumulators and the
// operands of the next step has no registers left for it.  Hence 8 wavefronts with two roles:
//   wavefronts 0..3  multiply: LDS reads and MFMAs only, 64x64 outputs each
//   wavefronts 4..7  produce: global loads, the split of B, LDS writes
// A stage is 32 rows of K in two LDS buffers, with one barrier per stage placed in the middle
// of the multipliers' stage:
//   multipliers, stage s:  MFMAs of k-step 0 | reads of k-step 1;  barrier s;
//                          MFMAs of k-step 1 | reads of (stage s+1, k-step 0)
//   producers, between barriers s-1 and s: stage s+1 into buffer (s+1)&1, and between its
//                          pieces the global loads of stage s+4 into the registers that the
//                          previous iteration consumed
// The A panel is the same for every workgroup of a matrix, so it is split once by
// split_a_panel_kernel (or split_a_panel_lower_kernel, from the rows of a lower triangular
// factor) into the exact LDS image of each stage and the producers only copy it.
// The multipliers never touch global memory: they start from zero, and at the end hand their
// sums to the producers through LDS, who add the old X (X + s * sum, s = -1 for a negated A)
// with coalesced 16-byte accesses.
//
// LDS image of one operand and stage: [piece 3][k group of eight 4][position 128] 16-byte
// words, a word = 8 consecutive k as bf16.  Column c of the 128-wide tile sits at position
// (c & 3) * 32 + (c >> 2): a producer thread loads 4 consecutive columns with one 16-byte
// load and the writes of a wavefront are then contiguous in LDS.  A multiplier's MFMA tile
// at positions [32 e, 32 e + 32) therefore covers the columns 4 j + e, j = 0..31.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int SPLIT_TK = 32;                       // k rows per stage
constexpr int SPLIT_STAGE_WORDS = 3 * 4 * 128;     // 16-byte words per operand and stage (three pieces)
constexpr int split_stage_words(int np) { return np * 4 * 128; }
constexpr int SPLIT_SETS = 4;                      // producer register sets = stages in flight

// N fp32 values (consecutive k of one column) -> N/2 packed words of each piece.
template <int N, typename W>
__device__ __forceinline__ void split_pieces(const float (&x)[N], W& p1, W& p2, W& p3) {
    unsigned h1[N], h2[N], h3[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const unsigned a1 = __float_as_uint(x[j]) & 0xFFFF0000u;
        const float r1 = x[j] - __uint_as_float(a1);                 // exact
        const unsigned a2 = __float_as_uint(r1) & 0xFFFF0000u;
        const float r2 = r1 - __uint_as_float(a2);                   // exact, <= 8 bits
        h1[j] = a1; h2[j] = a2; h3[j] = __float_as_uint(r2);
    }
#pragma unroll
    for (int w = 0; w < N / 2; ++w) {   // upper halves of (k, k+1) -> one word, k in the low half
        p1[w] = __builtin_amdgcn_perm(h1[2 * w + 1], h1[2 * w], 0x07060302u);
        p2[w] = __builtin_amdgcn_perm(h2[2 * w + 1], h2[2 * w], 0x07060302u);
        p3[w] = __builtin_amdgcn_perm(h3[2 * w + 1], h3[2 * w], 0x07060302u);
    }
}

// Two pieces, each rounded to nearest even by the hardware's packing conversion
// (v_cvt_pk_bf16_f32): a = a1 + a2 + r with |r| <= 2^-18 |a|.  Used with the three products
// (2,1) (1,2) (1,1), whose sum is then within ~2^-17 of a*b with errors of either sign.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <int N, typename W>
__device__ __forceinline__ void split_pieces2(const float (&x)[N], W& p1, W& p2) {
#pragma unroll
    for (int w = 0; w < N / 2; ++w) {
        const f32x2 v = {x[2 * w], x[2 * w + 1]};
        const unsigned h1 = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
        const f32x2 r = {v[0] - __uint_as_float(h1 << 16), v[1] - __uint_as_float(h1 & 0xFFFF0000u)};
        p1[w] = h1;                                                  // k in the low half
        p2[w] = __builtin_bit_cast(unsigned, __builtin_convertvector(r, bf16x2));
    }
}

// Two fp16 pieces of sc * x, each rounded to nearest (v_cvt_pk_f16_f32).  fp16 carries 11
// significant bits, so a1 = fp16(x), a2 = fp16(x - a1) leave |x - a1 - a2| <= 2^-24 |x|: the pair
// holds an fp32 value to its own precision, and the three products (2,1) (1,2) (1,1) give a*b
// to ~2^-23 -- fp32-grade from THREE products of the fp16 matrix instruction instead of six of
// the bf16 one.  The price is fp16's range: sc is a power of two, one per column of the operand
// matrix, chosen by the caller so that the column's largest entry lands at or below 2^14 (no
// overflow; the result is divided by the two columns' factors afterwards, exactly); an entry
// below 2^-17 of its column's bound loses low bits of its second piece (subnormal or flushed),
// an absolute error of at most 2^-29 of that bound, far below the fp32 rounding of the sums it
// enters.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
// The largest power of two sc with bound * sc <= 2^14 (bound = f * 2^e, f in [0.5, 1): 2^(14 - e)),
// kept inside [2^-100, 2^114] so that it and its reciprocal are normal numbers.
__device__ __forceinline__ float pow2_scale(float bound) {
    int e = __builtin_amdgcn_frexp_expf(bound);
    e = e < -100 ? -100 : (e > 114 ? 114 : e);
    return __uint_as_float((unsigned)(127 + 14 - e) << 23);
}
template <int N, typename W>
__device__ __forceinline__ void split_pieces2h(const float (&x)[N], float sc, W& p1, W& p2) {
#pragma unroll
    for (int w = 0; w < N / 2; ++w) {
        const f32x2 v = {x[2 * w] * sc, x[2 * w + 1] * sc};
        const f16x2 h1 = __builtin_convertvector(v, f16x2);
        const f32x2 back = __builtin_convertvector(h1, f32x2);
        const f32x2 r = {v[0] - back[0], v[1] - back[1]};
        p1[w] = __builtin_bit_cast(unsigned, h1);                    // k in the low half
        p2[w] = __builtin_bit_cast(unsigned, __builtin_convertvector(r, f16x2));
    }
}

// Rows [k0, k1) x columns [m0, m0+128) of At -> the LDS images of its stages, stage after
// stage (SPLIT_STAGE_WORDS words each).  One workgroup of 128 threads per matrix and stage.
template <int NP, bool HALF>
__global__ __launch_bounds__(128) void split_a_panel_kernel(const float* __restrict__ At, int64_t lda,
                                                            int64_t as, int m0, int k0, int n_stage,
                                                            u32x4* __restrict__ Ap, int64_t aps,
                                                            const float* __restrict__ bound,
                                                            int64_t bound_stride) {
    const int bz = blockIdx.x / n_stage, st = blockIdx.x % n_stage;
    const int t = threadIdx.x, kg = t >> 5, cq = t & 31;
    const float* src = At + (int64_t)bz * as + (int64_t)(k0 + SPLIT_TK * st + 8 * kg) * lda + m0 + 4 * cq;
    f32x4 x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = *reinterpret_cast<const f32x4*>(src + (int64_t)j * lda);
    u32x4* dst = Ap + (int64_t)bz * aps + (int64_t)st * split_stage_words(NP) + kg * 128 + cq;
    f32x4 sc4 = {1.f, 1.f, 1.f, 1.f};
    if (HALF) {
        const f32x4 b4 = *reinterpret_cast<const f32x4*>(bound + (int64_t)bz * bound_stride + m0 + 4 * cq);
#pragma unroll
        for (int e = 0; e < 4; ++e) sc4[e] = pow2_scale(b4[e]);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float col[8];
        u32x4 p1, p2, p3;
#pragma unroll
        for (int j = 0; j < 8; ++j) col[j] = x[j][e];
        if (NP == 3) {
            split_pieces<8>(col, p1, p2, p3);
            dst[1024 + 32 * e] = p3;
        } else if (HALF) {
            split_pieces2h<8>(col, sc4[e], p1, p2);
        } else {
            split_pieces2<8>(col, p1, p2);
        }
        dst[32 * e] = p1;
        dst[512 + 32 * e] = p2;
    }
}

// The same panel taken from a lower triangular matrix: element (k, m) = -(Al[m, k] * (1 / Al[m, m]))
// for k < m, zero elsewhere and for matrices whose info is not 0.  A thread reads the 8
// consecutive k of a word from ONE row of Al (32 contiguous bytes; four neighbouring lanes cover
// the 128 bytes that a row contributes to the stage), so nothing is transposed.
template <int NP, bool HALF>
__global__ __launch_bounds__(128) void split_a_panel_lower_kernel(
    const float* __restrict__ Al, int64_t ldl, int64_t ls, const int32_t* __restrict__ info, int m0,
    int k0, int n_stage, u32x4* __restrict__ Ap, int64_t aps, const float* __restrict__ bound,
    int64_t bound_stride) {
    const int bz = blockIdx.x / n_stage, st = blockIdx.x % n_stage;
    const int t = threadIdx.x, kg = t & 3, mr = t >> 2;     // k group of 8, row within a pass of 32
    const int kb = k0 + SPLIT_TK * st + 8 * kg;             // first of this thread's 8 k
    const float* __restrict__ Ab = Al + (int64_t)bz * ls;
    const bool failed = info != nullptr && info[bz] != 0;
    u32x4* dst = Ap + (int64_t)bz * aps + (int64_t)st * split_stage_words(NP) + kg * 128;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int c = 32 * e + mr, m = m0 + c;              // column of the tile, row of Al
        const float* row = Ab + (int64_t)m * ldl;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(row + kb);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(row + kb + 4);
        const float rcp = 1.0f / row[m];
        float col[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float a = j < 4 ? lo[j] : hi[j - 4];
            col[j] = (failed || kb + j >= m) ? 0.0f : -(a * rcp);
        }
        const int pos = (c & 3) * 32 + (c >> 2);            // the stage image's place of column c
        u32x4 p1, p2, p3;
        if (NP == 3) {
            split_pieces<8>(col, p1, p2, p3);
            dst[1024 + pos] = p3;
        } else if (HALF) {
            split_pieces2h<8>(col, pow2_scale(bound[(int64_t)bz * bound_stride + m]), p1, p2);
        } else {
            split_pieces2<8>(col, p1, p2);
        }
        dst[pos] = p1;
        dst[512 + pos] = p2;
    }
}

struct SplitPair {
    GemmPair pair;
    const u32x4* Ap;   // split A panel of both problems (same At, m0, k0)
    int64_t aps;       // words per matrix
    int64_t apt;       // words per m tile (all matrices): a problem may have two m tiles
};

// Both problems: full 128x128 tiles, one m tile, 16-byte aligned rows, every tile's K range
// a whole number of 128-row chunks starting at k0.
// NP pieces per operand, NPROD piece products per fp32 product (the largest ones).
//   NP = 3, NPROD = 6: all products of weight >= 2^-16, fp32-grade (the factorisation).
//   NP = 2 (pieces rounded to nearest): NPROD = 3: (2,1) (1,2) (1,1), within ~2^-17 of a*b;
//   NPROD = 4 adds (2,2); NPROD = 1 is (1,1) alone, i.e. plain bf16 operands.  Only where the
//   caller asks for it (the direct sweep's block updates, option "sweep_update_products").
//   HALF (NP = 2, NPROD = 3): the pieces are fp16 halves of operands scaled by the powers of two
//   g.scale[matrix][column] (split_pieces2h): fp32-grade from three products.
//   MT = 2 (NP = 2 only; the problem has two m tiles): one workgroup computes both, 256 x 128
//   outputs.  Every row of B is then loaded and split once for 256 output rows, a stage holds
//   twice the matrix work behind the same number of B loads in flight (what the producers'
//   four register sets can cover of the HBM latency doubles), and the LDS traffic per matrix
//   instruction falls by a quarter.  The 128 accumulator registers leave no room for a second
//   set of totals, so K is summed in one run, as an SGEMM does.
template <int NP, int NPROD, bool HALF, int MT>
__global__ __launch_bounds__(512, 1) void split_gemm_kernel(SplitPair sp) {
    static_assert(MT == 1 || (MT == 2 && NP == 2), "two m tiles per workgroup: two-piece layouts only");
    const bool in_first = blockIdx.x < (unsigned)sp.pair.first_wgs;
    const GemmArgs& g = in_first ? sp.pair.first : sp.pair.second;
    const int wg = in_first ? (int)blockIdx.x : (int)blockIdx.x - sp.pair.first_wgs;
    // [buffer][operand: the A panel of each m tile, then B][piece][k group][position]
    __shared__ __attribute__((aligned(16))) u32x4 L[2][MT + 1][NP][4][128];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The m tiles of one (matrix, n tile) follow each other on the same XCD: they read the same
    // rows of B at about the same time, so the second reading is served by that XCD's L2.
    const int grid_m_tiles = MT == 2 ? 1 : g.m_tiles;
    const int per_matrix = g.n_tiles * grid_m_tiles;
    int bz, rem;
    if (g.xcd_map) {
        const int xcd = wg & 7, slot = wg >> 3;
        bz = xcd + 8 * (slot / per_matrix);
        rem = slot % per_matrix;
    } else {
        bz = wg / per_matrix;
        rem = wg % per_matrix;
    }
    const int tile = rem / grid_m_tiles, mtile = rem % grid_m_tiles;
    const int m0 = g.m0 + mtile * TM;
    const int tn = g.b_upper_tri ? g.n_tiles - 1 - tile : tile;
    const int nt = g.n0 + tn * TN;
    const int k0 = g.k0;
    int k1 = g.k1;
    if (g.lim != nullptr) {   // uniform over the workgroup; before any barrier
        const int own = g.lim[bz];
        if ((g.lim_m && m0 >= own) || (g.lim_n && nt >= own)) return;
        if (g.lim_k && k1 > own) k1 = own;
    }
    if (g.b_upper_tri && k1 > nt + TN) k1 = nt + TN;
    const int n_stage = (k1 - k0) / SPLIT_TK;     // a multiple of 4

    if (wave >= 4) {
        // ---------------- producers ----------------
        // B: thread = rows 4 kh .. 4 kh + 3 of the stage x columns 4 cq .. 4 cq + 3
        const int pt = tid - 256, kh = pt >> 5, cq = pt & 31;
        const float* Bm = g.Bm + (int64_t)bz * g.bs;
        const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(Bm + (int64_t)k0 * g.ldb + nt), 0, 0x7FFFFFFF, 0x00027000);
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<u32x4*>(sp.Ap + (int64_t)mtile * sp.apt + (int64_t)bz * sp.aps), 0, 0x7FFFFFFF,
            0x00027000);
        const __amdgpu_buffer_rsrc_t a_rsrc2 = __builtin_amdgcn_make_buffer_rsrc(   // second m tile
            const_cast<u32x4*>(sp.Ap + (int64_t)(MT - 1) * sp.apt + (int64_t)bz * sp.aps), 0, 0x7FFFFFFF,
            0x00027000);
        int ob[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) ob[j] = (int)(((int64_t)(4 * kh + j) * g.ldb + 4 * cq) * 4);
        // fp16 halves: the power-of-two factors of this thread's four B columns
        f32x4 scb = {1.f, 1.f, 1.f, 1.f};
        if (HALF) {
            const f32x4 b4 =
                *reinterpret_cast<const f32x4*>(g.bound_b + (int64_t)bz * g.bound_b_stride + nt + 4 * cq);
#pragma unroll
            for (int e = 0; e < 4; ++e) scb[e] = pow2_scale(b4[e]);
        }
        const int oa = pt * 16;
        // Every fetch stays inside [k0, k1): the offsets advance only while a further stage
        // exists; past the end the last stage is fetched again and never used.
        int b_soff = 0, a_soff = 0, fetched = 0;
        int b_adv = (int)(SPLIT_TK * g.ldb * 4), a_adv = split_stage_words(NP) * 16;
        f32x4 xb[SPLIT_SETS][4];
        u32x4 xa[SPLIT_SETS][MT * 2 * NP];
#define FORGE_SPLIT_FETCH(q)                                                                       \
    do {                                                                                           \
        ++fetched;                                                                                 \
        if (fetched >= n_stage) { b_adv = 0; a_adv = 0; }                                          \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) xb[q][j] = __builtin_bit_cast(               \
            f32x4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, ob[j], b_soff, 0));               \
        _Pragma("unroll") for (int j = 0; j < 2 * NP; ++j)                                         \
            xa[q][j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, oa + j * 4096, a_soff, 0);    \
        if (MT == 2) {                                                                             \
            _Pragma("unroll") for (int j = 0; j < 2 * NP; ++j) xa[q][(MT - 1) * 2 * NP + j] =      \
                __builtin_amdgcn_raw_buffer_load_b128(a_rsrc2, oa + j * 4096, a_soff, 0);          \
        }                                                                                          \
        b_soff += b_adv;                                                                           \
        a_soff += a_adv;                                                                           \
    } while (0)
        // B word (piece, k group kh >> 1, position 32 e + cq), half kh & 1; A: plain copy
        u32x2* const Lb = reinterpret_cast<u32x2*>(&L[0][MT][0][kh >> 1][cq]) + (kh & 1);
        u32x4* const La = &L[0][0][0][0][0] + pt;
        constexpr int BUF = (MT + 1) * split_stage_words(NP);   // words per buffer (all operands)
#define FORGE_SPLIT_STAGE(buf, q)                                                                  \
    do {                                                                                           \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                            \
            float col[4];                                                                          \
            u32x2 p1, p2, p3;                                                                      \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) col[j] = xb[q][j][e];                    \
            if (NP == 3) {                                                                         \
                split_pieces<4>(col, p1, p2, p3);                                                  \
                Lb[((buf) * BUF + (NP - 1) * 512 + 32 * e) * 2] = p3;                              \
            } else if (HALF) {                                                                     \
                split_pieces2h<4>(col, scb[e], p1, p2);                                            \
            } else {                                                                               \
                split_pieces2<4>(col, p1, p2);                                                     \
            }                                                                                      \
            Lb[((buf) * BUF + 32 * e) * 2] = p1;                                                   \
            Lb[((buf) * BUF + 512 + 32 * e) * 2] = p2;                                             \
        }                                                                                          \
        _Pragma("unroll") for (int j = 0; j < MT * 2 * NP; ++j) La[(buf) * BUF + j * 256] = xa[q][j]; \
    } while (0)
        // One stage's split and LDS writes, with the loads of a later stage (into the register
        // set qf, which the previous iteration consumed) spread between them: a wavefront does
        // not go on until the texture unit has taken its load, and the unit takes 16 cycles per
        // 1 KB instruction, so loads issued back to back by all four producers would hold them
        // for as long as the unit needs for the whole stage.
#define FORGE_SPLIT_STAGE_FETCH(buf, q, qf)                                                        \
    do {                                                                                           \
        ++fetched;                                                                                 \
        if (fetched >= n_stage) { b_adv = 0; a_adv = 0; }                                          \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                            \
            xb[qf][e] = __builtin_bit_cast(                                                        \
                f32x4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, ob[e], b_soff, 0));           \
            _Pragma("unroll") for (int j = e * NP / 2; j < (e + 1) * NP / 2; ++j) {                \
                xa[qf][j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, oa + j * 4096, a_soff, 0); \
                if (MT == 2) xa[qf][2 * NP + j] =                                                  \
                    __builtin_amdgcn_raw_buffer_load_b128(a_rsrc2, oa + j * 4096, a_soff, 0);      \
            }                                                                                      \
            float col[4];                                                                          \
            u32x2 p1, p2, p3;                                                                      \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) col[j] = xb[q][j][e];                    \
            if (NP == 3) {                                                                         \
                split_pieces<4>(col, p1, p2, p3);                                                  \
                Lb[((buf) * BUF + (NP - 1) * 512 + 32 * e) * 2] = p3;                              \
            } else if (HALF) {                                                                     \
                split_pieces2h<4>(col, scb[e], p1, p2);                                            \
            } else {                                                                               \
                split_pieces2<4>(col, p1, p2);                                                     \
            }                                                                                      \
            Lb[((buf) * BUF + 32 * e) * 2] = p1;                                                   \
            Lb[((buf) * BUF + 512 + 32 * e) * 2] = p2;                                             \
            _Pragma("unroll") for (int j = e * MT * NP / 2; j < (e + 1) * MT * NP / 2; ++j)        \
                La[(buf) * BUF + j * 256] = xa[q][j];                                              \
            __builtin_amdgcn_sched_barrier(0);                                                     \
        }                                                                                          \
        b_soff += b_adv;                                                                           \
        a_soff += a_adv;                                                                           \
    } while (0)
        FORGE_SPLIT_FETCH(0);
        FORGE_SPLIT_FETCH(1);
        FORGE_SPLIT_FETCH(2);
        FORGE_SPLIT_FETCH(3);
        FORGE_SPLIT_STAGE(0, 0);
        __syncthreads();
        for (int s0 = 0; s0 < n_stage; s0 += 4) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                FORGE_SPLIT_STAGE_FETCH((s + 1) & 1, (s + 1) & 3, s & 3);
                __syncthreads();
            }
        }
#undef FORGE_SPLIT_STAGE_FETCH
#undef FORGE_SPLIT_FETCH
#undef FORGE_SPLIT_STAGE
        // Epilogue, on the producers so that it is coalesced: the multipliers leave their
        // sums in LDS (over the stage buffers, free by then), one m tile at a time, row r of
        // the tile at S[r][position]; thread = 16 rows x 4 consecutive columns, X is read and
        // written in 16-byte pieces of whole 512-byte rows.
        const float sgn = g.negate_a ? -1.0f : 1.0f;
        // fp16 halves: element (row, column) of the sums carries the factors of A's column
        // m0 + row and of B's column; powers of two, so dividing them out is exact
        f32x4 ib = {1.f, 1.f, 1.f, 1.f};
        if (HALF) {
#pragma unroll
            for (int e = 0; e < 4; ++e) ib[e] = sgn / scb[e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) ib[e] = sgn;
        }
        const float* S = reinterpret_cast<const float*>(&L[0][0][0][0][0]);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            float* __restrict__ Xt = g.X + (int64_t)bz * g.xs + (int64_t)(m0 + t * TM) * g.ldx + nt + 4 * cq;
            const float* __restrict__ sca =
                HALF ? g.bound_a + (int64_t)bz * g.bound_a_stride + m0 + t * TM : nullptr;
            f32x4 xo[16];
            if (g.x_init && g.x_init_bf16) {
                const uint16_t* __restrict__ X0 = static_cast<const uint16_t*>(g.x_init) + (Xt - g.X);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const u32x2 w = *reinterpret_cast<const u32x2*>(X0 + (int64_t)(kh + 8 * i) * g.ldx);
                    xo[i] = f32x4{__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xFFFF0000u),
                                  __uint_as_float(w[1] << 16), __uint_as_float(w[1] & 0xFFFF0000u)};
                }
            } else if (g.x_init) {
                const float* __restrict__ X0 = static_cast<const float*>(g.x_init) + (Xt - g.X);
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    xo[i] = *reinterpret_cast<const f32x4*>(X0 + (int64_t)(kh + 8 * i) * g.ldx);
            } else if (!g.init_zero) {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    xo[i] = *reinterpret_cast<const f32x4*>(Xt + (int64_t)(kh + 8 * i) * g.ldx);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) xo[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            if (t == 0) __syncthreads();   // every multiplier has read its last operands
            __syncthreads();               // the sums of m tile t are in LDS
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float* Sr = S + (kh + 8 * i) * TN + cq;
                const float ia = HALF ? 1.0f / pow2_scale(sca[kh + 8 * i]) : 1.0f;
                f32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = xo[i][e] + (ib[e] * ia) * Sr[32 * e];
                *reinterpret_cast<f32x4*>(Xt + (int64_t)(kh + 8 * i) * g.ldx) = o;
            }
            if (t + 1 < MT) __syncthreads();   // the staging area is free for the next m tile
        }
        return;
    }

    // ---------------- multipliers ----------------
    const int wm = wave >> 1, wn = wave & 1;
    // MFMA tile (mi, ni) of this wavefront: positions 32 (wm + 2 mi) .. of A, 32 (wn + 2 ni) ..
    // of B, i.e. output rows m0 + 4 j + wm + 2 mi and columns nt + 4 j' + wn + 2 ni.  Lane
    // element v of the accumulator is MFMA row (lane >> 5) * 4 + (v >> 2) * 8 + (v & 3),
    // column lane & 31.
    const int jrow = (lane >> 5) * 4, jcol = lane & 31;
    // One m tile: acc holds the sum of the current 128-row chunk, tot the sum of the chunks.
    // Two m tiles: acc runs over all of K.  X itself is added in the epilogue.
    constexpr bool CHUNKED = MT == 1;
    f32x16 acc[MT][2][2], tot[2][2];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc[t][mi][ni][v] = 0.0f;
                    if (CHUNKED) tot[mi][ni][v] = 0.0f;
                }
    const int rk = lane >> 5, ra = wm * 32 + (lane & 31), rb = wn * 32 + (lane & 31);
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    bf16x8 A0[MT][NP][2], B0[NP][2], A1[MT][NP][2], B1[NP][2];   // operands of k-step 0 / 1
#define FORGE_SPLIT_READ(buf, u, A, B)                                                             \
    do {                                                                                           \
        _Pragma("unroll") for (int p = 0; p < NP; ++p) _Pragma("unroll") for (int i = 0; i < 2; ++i) { \
            _Pragma("unroll") for (int t = 0; t < MT; ++t)                                         \
                A[t][p][i] = __builtin_bit_cast(bf16x8, L[buf][t][p][2 * (u) + rk][ra + 64 * i]);  \
            B[p][i] = __builtin_bit_cast(bf16x8, L[buf][MT][p][2 * (u) + rk][rb + 64 * i]);        \
        }                                                                                          \
    } while (0)
    // piece products smallest first; the four tiles innermost so that consecutive MFMAs use
    // different accumulators; `fresh`: the first product of a chunk takes C = 0
#define FORGE_SPLIT_MFMAS(A, B, fresh)                                                             \
    do {                                                                                           \
        constexpr int PA[6] = {NP - 1, 0, 1, 1, 0, 0}, PB[6] = {0, NP - 1, 1, 0, 1, 0};            \
        _Pragma("unroll") for (int t = 6 - NPROD; t < 6; ++t) _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) \
            _Pragma("unroll") for (int mi = 0; mi < 2; ++mi) _Pragma("unroll") for (int ni = 0; ni < 2; ++ni) \
                acc[mt][mi][ni] = HALF ? __builtin_amdgcn_mfma_f32_32x32x16_f16(                   \
                    __builtin_bit_cast(f16x8, A[mt][PA[t]][mi]), __builtin_bit_cast(f16x8, B[PB[t]][ni]), \
                    (CHUNKED && (fresh) && t == 6 - NPROD) ? zero : acc[mt][mi][ni], 0, 0, 0)      \
                    : __builtin_amdgcn_mfma_f32_32x32x16_bf16(                                     \
                    A[mt][PA[t]][mi], B[PB[t]][ni],                                                \
                    (CHUNKED && (fresh) && t == 6 - NPROD) ? zero : acc[mt][mi][ni], 0, 0, 0);     \
    } while (0)
    // 4 NPROD MT MFMAs and 2 NP (MT + 1) LDS reads per k-step (24 and 12, or 12 and 8): the
    // reads spread evenly between the MFMAs
#define FORGE_SPLIT_SCHED()                                                                        \
    do {                                                                                           \
        if (NPROD * MT == 6) {                                                                          \
            _Pragma("unroll") for (int i = 0; i < 12; ++i) {                                       \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
            }                                                                                      \
        } else if (NPROD * MT == 3) {                                                              \
            _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                        \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                 \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
            }                                                                                      \
        }                                                                                          \
    } while (0)
    __syncthreads();
    FORGE_SPLIT_READ(0, 0, A0, B0);
    for (int s0 = 0; s0 < n_stage; s0 += 4) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            FORGE_SPLIT_READ(s & 1, 1, A1, B1);
            FORGE_SPLIT_MFMAS(A0, B0, s == 0);
            FORGE_SPLIT_SCHED();
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            FORGE_SPLIT_READ((s + 1) & 1, 0, A0, B0);
            FORGE_SPLIT_MFMAS(A1, B1, false);
            FORGE_SPLIT_SCHED();
            __builtin_amdgcn_sched_barrier(0);
        }
        if (CHUNKED) {
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) tot[mi][ni] += acc[0][mi][ni];
        }
    }
#undef FORGE_SPLIT_READ
#undef FORGE_SPLIT_MFMAS
#undef FORGE_SPLIT_SCHED
    __syncthreads();   // all operand reads done: the stage buffers become the output staging
    float* S = reinterpret_cast<float*>(&L[0][0][0][0][0]);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 4 * (jrow + (v >> 2) * 8 + (v & 3)) + wm + 2 * mi;
                    S[r * TN + 32 * (wn + 2 * ni) + jcol] = CHUNKED ? tot[mi][ni][v] : acc[t][mi][ni][v];
                }
        __syncthreads();                     // the producers add them to X
        if (t + 1 < MT) __syncthreads();     // and have read them all
    }
}

}  // namespace

namespace {

struct Prepared {
    GemmArgs g;
    bool empty, edge;
    bool k128;   // every tile's K range is a whole number of 128-row chunks
    int64_t n_wg;
    double flops;
};

// Fills in the tile counts and decides which kernel a problem needs.
Prepared prepare(const GemmArgs& g_in, int64_t batch) {
    Prepared p{};
    GemmArgs& g = p.g;
    g = g_in;
    p.empty = g.m1 <= g.m0 || g.n1 <= g.n0 || batch <= 0 || (g.k1 <= g.k0 && !g.init_zero);
    if (p.empty) return p;
    // float4 loads need 16-byte aligned rows; anything else takes the scalar EDGE path
    const bool aligned = (g.lda % 4) == 0 && (g.ldb % 4) == 0 && (g.m0 % 4) == 0 &&
                         (g.n0 % 4) == 0 && (g.as % 4) == 0 && (g.bs % 4) == 0 &&
                         (reinterpret_cast<uintptr_t>(g.At) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(g.Bm) % 16) == 0;
    g.n_tiles = (int)ceil_div(g.n1 - g.n0, TN);
    g.m_tiles = (int)ceil_div(g.m1 - g.m0, TM);
    g.xcd_map = (batch % 8) == 0;
    p.n_wg = (int64_t)g.n_tiles * g.m_tiles * batch;
    // the triangular K clipping keeps multiples of TK only when tiles and K origin line up
    const bool tri_ok = (!g.b_upper_tri || ((g.n0 + TN - g.k0) % TK) == 0) &&
                        (!g.b_lower_tri || ((g.n0 - g.k0) % TK) == 0);
    // the full-tile kernel addresses its operands with 32-bit byte offsets from row k0
    const int64_t ldmax = g.lda > g.ldb ? g.lda : g.ldb;
    const bool offsets_fit = ((int64_t)(g.k1 - g.k0) + TK) * ldmax * 4 + TM * 4 < (1LL << 31);
    p.edge = ((g.m1 - g.m0) % TM) != 0 || ((g.n1 - g.n0) % TN) != 0 ||
             ((g.k1 - g.k0) % TK) != 0 || !tri_ok || !aligned || !offsets_fit;
    p.k128 = ((g.k1 - g.k0) % 128) == 0 && (!g.b_upper_tri || ((g.n0 + TN - g.k0) % 128) == 0) &&
             (!g.b_lower_tri || ((g.n0 - g.k0) % 128) == 0);
    // blocked summation exists for whole chunks only (full tiles) or bounds-checked
    if (g.blocked_sum && !p.k128) p.edge = true;
    // useful flops: 2*M*N*K with K clipped per n-tile for the triangular variants
    double kn = 0.0;
    for (int nt = g.n0; nt < g.n1; nt += TN) {
        int k0 = g.k0, k1 = g.k1;
        if (g.b_upper_tri && k1 > nt + TN) k1 = nt + TN;
        if (g.b_lower_tri && k0 < nt) k0 = nt;
        const int ncols = (g.n1 - nt) < TN ? (g.n1 - nt) : TN;
        if (k1 > k0) kn += (double)(k1 - k0) * ncols;
    }
    p.flops = 2.0 * (g.m1 - g.m0) * kn * (double)batch * (g.work_frac > 0.0 ? g.work_frac : 1.0);
    return p;
}

int launch_prepared(const Prepared& a, const Prepared* b, hipStream_t st) {
    const int64_t n_wg = a.n_wg + (b ? b->n_wg : 0);
    FORGE_REQUIRE(n_wg < (1LL << 31), "chain_gemm: grid too large");
    dim3 grid((unsigned)n_wg);
    KernelTiming timing(a.g.blocked_sum ? "chain_gemm_blocked_sum" : "chain_gemm", st,
                        a.flops + (b ? b->flops : 0.0), WORK_FLOPS);
    if (a.edge) {
        if (a.g.blocked_sum) chain_gemm_kernel<true, 128><<<grid, dim3(256), 0, st>>>(a.g);
        else chain_gemm_kernel<true, 0><<<grid, dim3(256), 0, st>>>(a.g);
    } else {
        GemmPair pair{};
        pair.first = a.g;
        pair.second = b ? b->g : a.g;
        pair.first_wgs = (int)a.n_wg;
        const bool k128 = a.k128 && (!b || b->k128);
        if (a.g.blocked_sum) chain_gemm_fast_kernel<128, 4><<<grid, dim3(256), 0, st>>>(pair);
        else if (k128) chain_gemm_fast_kernel<0, 4><<<grid, dim3(256), 0, st>>>(pair);
        else chain_gemm_fast_kernel<0, 1><<<grid, dim3(256), 0, st>>>(pair);
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

}  // namespace

int launch_chain_gemm(const GemmArgs& g, int64_t batch, hipStream_t st) {
    const Prepared p = prepare(g, batch);
    if (p.empty) return FORGE_OK;
    return launch_prepared(p, nullptr, st);
}

namespace {

// The bf16x3 path: both problems blocked-sum, full tiles, whole 128-row chunks, and the same
// A panel (At, pitch, m0, k0), which is split once for both.
bool split_eligible(const Prepared& a, const Prepared* b, int64_t batch, int64_t ws_bytes,
                    int* n_stage_out) {
    if (option(OPT_FP32_BLOCKED_SUM) == 1) return false;
    auto ok = [](const Prepared& p) {
        return !p.edge && p.k128 && p.g.blocked_sum && !p.g.b_lower_tri &&
               (p.g.m_tiles == 1 || (p.g.m_tiles == 2 && !p.g.b_upper_tri)) &&
               p.g.k1 - p.g.k0 >= 128 && (!p.g.b_upper_tri || p.g.n0 + TN - p.g.k0 >= 128);
    };
    if (!ok(a) || (b && !ok(*b))) return false;
    if (b && (a.g.m_tiles != 1 || b->g.m_tiles != 1)) return false;   // two m tiles: alone in its grid
    int k1 = a.g.k1;
    if (b) {
        const GemmArgs &x = a.g, &y = b->g;
        if (x.At != y.At || x.lda != y.lda || x.as != y.as || x.m0 != y.m0 || x.k0 != y.k0) return false;
        if (x.a_lower != y.a_lower || x.a_lower_ld != y.a_lower_ld || x.a_lower_stride != y.a_lower_stride ||
            x.a_info != y.a_info)
            return false;
        if (x.bound_a != y.bound_a || x.bound_a_stride != y.bound_a_stride) return false;
        if ((x.bound_b != nullptr) != (y.bound_b != nullptr)) return false;
        if (b->g.xcd_map && a.n_wg % 8 != 0) return false;
        if (y.k1 > k1) k1 = y.k1;
    }
    const int n_stage = (k1 - a.g.k0) / SPLIT_TK;
    if (ws_bytes < a.g.m_tiles * split_gemm_workspace_bytes(batch, k1 - a.g.k0)) return false;
    *n_stage_out = n_stage;
    return true;
}

int launch_split(const Prepared& a, const Prepared* b, int64_t batch, int n_stage, void* ws,
                 hipStream_t st) {
    const int64_t n_wg = a.n_wg + (b ? b->n_wg : 0);
    FORGE_REQUIRE(n_wg < (1LL << 31) && batch * n_stage < (1LL << 31), "split_gemm: grid too large");
    SplitPair sp{};
    sp.pair.first = a.g;
    sp.pair.second = b ? b->g : a.g;
    sp.pair.first_wgs = (int)a.n_wg;
    sp.Ap = static_cast<const u32x4*>(ws);
    const bool half = a.g.bound_a != nullptr && a.g.bound_b != nullptr;                               // fp16 pieces, three products
    const int products = half ? 3 : a.g.products;
    const bool two = products == 1 || products == 3 || products == 4;     // two-piece layout
    const int np = two ? 2 : 3;
    sp.aps = (int64_t)n_stage * split_stage_words(np);
    sp.apt = sp.aps * batch;
    for (int mt = 0; mt < a.g.m_tiles; ++mt) {
        KernelTiming timing("split_a_panel", st, (4.0 + 2.0 * np) * n_stage * SPLIT_TK * TM * (double)batch,
                            WORK_BYTES);
        const dim3 pgrid((unsigned)(batch * n_stage)), pblock(128);
        u32x4* dst = static_cast<u32x4*>(ws) + (int64_t)mt * sp.apt;
        if (a.g.a_lower) {
            const int m0 = a.g.m0 + mt * TM;
            if (half)
                split_a_panel_lower_kernel<2, true><<<pgrid, pblock, 0, st>>>(
                    a.g.a_lower, a.g.a_lower_ld, a.g.a_lower_stride, a.g.a_info, m0, a.g.k0, n_stage, dst,
                    sp.aps, a.g.bound_a, a.g.bound_a_stride);
            else if (two)
                split_a_panel_lower_kernel<2, false><<<pgrid, pblock, 0, st>>>(
                    a.g.a_lower, a.g.a_lower_ld, a.g.a_lower_stride, a.g.a_info, m0, a.g.k0, n_stage, dst,
                    sp.aps, nullptr, 0);
            else
                split_a_panel_lower_kernel<3, false><<<pgrid, pblock, 0, st>>>(
                    a.g.a_lower, a.g.a_lower_ld, a.g.a_lower_stride, a.g.a_info, m0, a.g.k0, n_stage, dst,
                    sp.aps, nullptr, 0);
        } else if (half)
            split_a_panel_kernel<2, true><<<pgrid, pblock, 0, st>>>(
                a.g.At, a.g.lda, a.g.as, a.g.m0 + mt * TM, a.g.k0, n_stage, dst, sp.aps, a.g.bound_a,
                a.g.bound_a_stride);
        else if (two)
            split_a_panel_kernel<2, false><<<pgrid, pblock, 0, st>>>(
                a.g.At, a.g.lda, a.g.as, a.g.m0 + mt * TM, a.g.k0, n_stage, dst, sp.aps, nullptr, 0);
        else
            split_a_panel_kernel<3, false><<<pgrid, pblock, 0, st>>>(
                a.g.At, a.g.lda, a.g.as, a.g.m0 + mt * TM, a.g.k0, n_stage, dst, sp.aps, nullptr, 0);
        FORGE_LAUNCH_CHECK();
    }
    KernelTiming timing(half ? "split_gemm_f16x2" : two ? "split_gemm_bf16x2" : "split_gemm_bf16x3", st,
                        a.flops + (b ? b->flops : 0.0), WORK_FLOPS);
    // two m tiles of a two-piece layout: one workgroup computes both
    const bool wide = a.g.m_tiles == 2 && np == 2 && (half || products == 3);
    const dim3 grid((unsigned)(wide ? n_wg / 2 : n_wg)), block(512);
    if (half) {
        if (wide) split_gemm_kernel<2, 3, true, 2><<<grid, block, 0, st>>>(sp);
        else split_gemm_kernel<2, 3, true, 1><<<grid, block, 0, st>>>(sp);
    } else {
        switch (products) {
            case 1: split_gemm_kernel<2, 1, false, 1><<<grid, block, 0, st>>>(sp); break;
            case 3:
                if (wide) split_gemm_kernel<2, 3, false, 2><<<grid, block, 0, st>>>(sp);
                else split_gemm_kernel<2, 3, false, 1><<<grid, block, 0, st>>>(sp);
                break;
            case 4: split_gemm_kernel<2, 4, false, 1><<<grid, block, 0, st>>>(sp); break;
            default: split_gemm_kernel<3, 6, false, 1><<<grid, block, 0, st>>>(sp); break;
        }
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

}  // namespace

int64_t split_gemm_workspace_bytes(int64_t batch, int64_t k_rows) {
    if (batch <= 0 || k_rows <= 0) return 0;
    return batch * ceil_div(k_rows, (int64_t)SPLIT_TK) * SPLIT_STAGE_WORDS * 16;
}

bool split_path_applies(const GemmArgs& g, int64_t batch, int64_t ws_bytes) {
    const Prepared p = prepare(g, batch);
    int n_stage = 0;
    return !p.empty && split_eligible(p, nullptr, batch, ws_bytes, &n_stage);
}

int launch_chain_gemm_pair(const GemmArgs& first, const GemmArgs& second, int64_t batch,
                           hipStream_t st, void* split_ws, int64_t split_ws_bytes) {
    const Prepared a = prepare(first, batch), b = prepare(second, batch);
    if (a.empty && b.empty) return FORGE_OK;
    const Prepared* pa = a.empty ? &b : &a;
    const Prepared* pb = (a.empty || b.empty) ? nullptr : &b;
    int n_stage = 0;
    if (split_ws && split_eligible(*pa, pb, batch, split_ws_bytes, &n_stage))
        return launch_split(*pa, pb, batch, n_stage, split_ws, st);
    if (!pb) return launch_prepared(*pa, nullptr, st);
    // one grid needs the same kernel for both; a grid split at a multiple of 8 keeps the
    // workgroup -> XCD map of the second problem
    const bool fusable = !a.edge && !b.edge && a.g.blocked_sum == b.g.blocked_sum &&
                         (!b.g.xcd_map || a.n_wg % 8 == 0);
    if (fusable) return launch_prepared(a, &b, st);
    if (int e = launch_prepared(a, nullptr, st)) return e;
    return launch_prepared(b, nullptr, st);
}

}  // namespace forge
