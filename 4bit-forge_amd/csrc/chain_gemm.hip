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
// Two kernels share this layout.  chain_gemm_fast_kernel handles full, aligned tiles and
// is a software pipeline: while the MFMAs of one sub-stage run, the wavefront issues the
// LDS reads of the next sub-stage, the LDS writes of the next stage and the global loads
// of the stage after that, one memory instruction between two MFMAs (a wavefront issues
// in order, so memory instructions issued in a block of their own leave the matrix pipe
// idle for their whole issue time).  chain_gemm_kernel<EDGE> is the simple, bounds-checked
// form for ragged shapes.
#include "chain_gemm.h"
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
    p.flops = 2.0 * (g.m1 - g.m0) * kn * (double)batch;
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

int launch_chain_gemm_pair(const GemmArgs& first, const GemmArgs& second, int64_t batch,
                           hipStream_t st) {
    const Prepared a = prepare(first, batch), b = prepare(second, batch);
    if (a.empty && b.empty) return FORGE_OK;
    if (a.empty) return launch_prepared(b, nullptr, st);
    if (b.empty) return launch_prepared(a, nullptr, st);
    // one grid needs the same kernel for both; a grid split at a multiple of 8 keeps the
    // workgroup -> XCD map of the second problem
    const bool fusable = !a.edge && !b.edge && a.g.blocked_sum == b.g.blocked_sum &&
                         (!b.g.xcd_map || a.n_wg % 8 == 0);
    if (fusable) return launch_prepared(a, &b, st);
    if (int e = launch_prepared(a, nullptr, st)) return e;
    return launch_prepared(b, nullptr, st);
}

}  // namespace forge
