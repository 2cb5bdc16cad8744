// Blocked GPTQ column sweep (dense and 1:4 joint solve) for gfx950.
//
// Arithmetic follows forge/backend/cuda/solver.cu:9-154 and
// forge/backend/cuda/solver_sparsegptq14.cu:12-200: per column quantise with
// q = clamp(rint(fma(x, 1/(s+eps), q0))), deq = fma(q, s, -q0*s), err = x - deq, then
// x[k] = fma(-U[t,k], err, x[k]) for every later column k.  Every element therefore
// receives its rank-1 updates as ONE fp32 fma chain in ascending t.  The trailing update
// keeps that exact chain: on gfx950 v_mfma_f32_32x32x2_f32 accumulates
// acc = fma(a[k], b[k], acc) one k after the other in fp32, so a GEMM whose accumulator
// is initialised with the current weights and whose K loop runs in ascending t gives the
// same bits as the scalar chain, for any blocking.  Two kernels:
//
//   sweep_block_kernel   one lane per output row, BW consecutive columns of that row in
//                        registers; the serial quantise/propagate chain (VALU).
//   chain_gemm_kernel    X[m, n] <- chain_k fma(-U[k, m], E[k, n], X[m, n]) on the f32
//                        MFMA pipe, 128x128 tiles staged through LDS (chain_gemm.hip).
//
// The host schedules them left-looking (batched experts: each column block is brought
// up to date with ONE long-K GEMM over all earlier errors, so the weights stream through
// HBM once) or right-looking (a single matrix: more tiles in flight per step).
#include <cstdlib>
#include "common.h"
#include "chain_gemm.h"

namespace {

constexpr float kEps = 1e-12f;
#ifndef FORGE_SWEEP_BW
#define FORGE_SWEEP_BW 128
#endif
constexpr int forge_kBW = FORGE_SWEEP_BW;  // columns per in-register block


struct SweepArgs {
    float* A;              // [C,R] per matrix: x on entry; on exit err (batched form) or deq
    float* B;              // [C,R] per matrix: receives err in the per-element form
    const float* U;        // [C,C] per matrix, row-normalised upper factor
    const float* scales;   // PER_ELEM: [C,R]; else [G,R]
    const float* qzeros;
    const int32_t* g_idx;  // [C] per matrix (group of solver column), !PER_ELEM only
    uint8_t* q;            // [C,R] per matrix
    uint32_t* M;           // [ceil(C/32),R] per matrix (sparse only)
    const float* uinv;     // [C] per matrix (sparse only)
    const void* W0;        // [C,R] per matrix: the untouched weights (displacement form only),
    bool w0_bf16;          // as f32 or, when set, as bf16 (exact for weights that are bf16)
    float* dbound;         // [R] per matrix or null: running max |d| of each row (displacement form)
    // U's pitch and batch stride; 0 = C and C*C.  u_band: row t holds the columns of its own
    // 128-column block only, [C, 128] per matrix: entry (t, k) sits at U[t * ldu + k - c0].
    int64_t ldu, u_stride;
    bool u_band;
    int64_t C, R, G;
    int64_t c0;            // first column of this block
    int bw;                // columns in this block (<= BW)
    int maxq;
};

// Quantise one value (solver.cu:9-23): code, dequantised value and error.
__device__ __forceinline__ void quantize_scalar(float x, float s, float q0, float maxq, float& qf,
                                                float& deq, float& err) {
    const float inv_s = 1.0f / (s + kEps);
    // v_med3_f32: same value as fminf(fmaxf(., 0), maxq)
    qf = __builtin_amdgcn_fmed3f(__builtin_rintf(__builtin_fmaf(x, inv_s, q0)), 0.0f, maxq);
    deq = __builtin_fmaf(qf, s, -(q0 * s));
    err = x - deq;
}

// x + (-u_K) * e as ONE fused multiply-add, where u_K is the `u` register of lane K of this
// lane's row of 16 lanes (DPP row broadcast): sixteen U values sit in one VGPR, spread over
// the lanes of a row, instead of each being broadcast to every lane through LDS.  Same
// arithmetic as fmaf(-u, e, x).  The leading s_nop covers the two wait states a DPP read
// needs after a VALU write of its source, which the compiler cannot see inside the asm.
template <int K>
__device__ __forceinline__ void fnma_row_bcast(float& x, float u, float e) {
    asm("v_fmac_f32_dpp %0, -%1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
        : "+v"(x)
        : "v"(u), "v"(e), "n"(K));
}
__device__ __forceinline__ float dpp_source(float u) {
    asm volatile("s_nop 1" : "+v"(u));
    return u;
}
#define FORGE_FOR_16(M) M(0) M(1) M(2) M(3) M(4) M(5) M(6) M(7) M(8) M(9) M(10) M(11) M(12) M(13) M(14) M(15)

#ifndef FORGE_SWEEP_RING
#define FORGE_SWEEP_RING 3
#endif

// One lane per output row; the row's BW block columns live in x[].  The block is walked
// in sub-blocks of 32 columns: the serial quantise/propagate chain on x[0..31], then
// those 32 errors are pushed into the block's remaining columns, then x[] is shifted down
// by 32 so that the next sub-block again sits in x[0..31] (this keeps the unrolled code at
// one sub-block's size).  U[t,k] is the same for every lane: the workgroup stages the
// block's rows of U in LDS once, before the first column, and every fma takes its U operand
// from there.  TAIL is the guarded, slower variant (U straight from global memory)
// for blocks that are not a whole number of 32-column sub-blocks or whose U rows are not
// 16-byte aligned.
//
// DISP is the displacement form: what a column hands on is d = w0 - deq (its ORIGINAL
// weight minus what it was rounded to) instead of err = x - deq, and `U` holds
// V[t,k] = -M[t,k] / M[k,k] (k > t) of the factor H = M M^T (M upper) instead of the
// row-normalised factor of the inverse.  With N = I - strict(V) the inverse of the unit
// matrix the error form uses, err = d N, so the value a column has when it is reached,
// w0_k + sum_{t<k} d_t N[t,k], is the same number in exact arithmetic; only fp32 rounding
// differs.  The quantiser, the fused multiply-adds and their order are those of the error form.
// Values of columns that are NOT yet reached differ between the forms; the 1:4 mask score,
// which looks three columns ahead, rebuilds the error form's values from the 4x4 diagonal
// block of V (see select_and_quantize).
__device__ __forceinline__ float w0_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float w0_as_f32(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }

// The LDS-staged variants reach memory through buffer instructions: the matrix's base address
// sits in scalar registers (one descriptor per array), the lane's row is ONE 32-bit register
// and the column a scalar offset, where pointers cost two registers per array and lane -- the
// registers that x[], the scales and the errors leave no room for.  Offsets are bytes from the
// descriptor's base and stay below 2^31 (the launcher checks the shape).
using rsrc_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ rsrc_t row_rsrc(const void* base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7FFFFFFF, 0x00027000);
}
__device__ __forceinline__ float buf_ld_f32(rsrc_t rs, int voff, int soff) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff, 0));
}
__device__ __forceinline__ float buf_ld_w0(rsrc_t rs, int row, int64_t col_elems, const float*) {
    return buf_ld_f32(rs, row * 4, (int)(col_elems * 4));
}
__device__ __forceinline__ float buf_ld_w0(rsrc_t rs, int row, int64_t col_elems, const uint16_t*) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rs, row * 2, (int)(col_elems * 2), 0) << 16);
}
__device__ __forceinline__ void buf_st_f32(float v, rsrc_t rs, int voff, int soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rs, voff, soff, 0);
}

template <int BW, int NT, bool SPARSE, bool PER_ELEM, bool ERR_IN_A, bool TAIL, bool DISP = false,
          typename W0T = float>
__global__ __launch_bounds__(NT, (TAIL || NT >= 256) ? 2 : 1) void sweep_block_kernel(SweepArgs a) {
    constexpr int SB = 32, NSB = BW / SB;
    constexpr int RING = FORGE_SWEEP_RING;   // LDS read-ahead: RING-1 steps of 16 columns
    // (all of the block's rows of U at once, 64 KB for 128 columns: a panel per sub-block, fetched
    // one sub-block ahead, held the next panel in registers across the serial chain, and those
    // twelve registers were the ones that no longer fitted beside x[], the scales and the errors)
    __shared__ __attribute__((aligned(16))) float Up[TAIL ? 1 : BW][TAIL ? 4 : BW];
    // Lanes past the last row leave at once; that only happens in the TAIL variant (the
    // LDS-staged variants are launched for whole wavefronts only: every lane loads its
    // share of the panel and meets the others at the barriers).
    const int64_t r = (int64_t)blockIdx.x * NT + threadIdx.x;
    if (r >= a.R) return;
    const int64_t b = blockIdx.y;
    const int64_t C = a.C, R = a.R;
    float* __restrict__ A = a.A + b * C * R + r;
    float* __restrict__ Bo = ERR_IN_A ? nullptr : a.B + b * C * R + r;
    const int64_t ldu = a.ldu ? a.ldu : C;
    // (band form: this block's columns start at 0 of every row)
    const float* __restrict__ U = a.U + b * (a.ldu ? a.u_stride : C * C) - (a.u_band ? a.c0 : 0);
    const float* __restrict__ sc = a.scales + b * (PER_ELEM ? C * R : a.G * R) + r;
    const float* __restrict__ qz = a.qzeros + b * (PER_ELEM ? C * R : a.G * R) + r;
    const int32_t* __restrict__ gi = PER_ELEM ? nullptr : a.g_idx + b * C;
    const float* __restrict__ uinv = SPARSE ? a.uinv + b * C : nullptr;
    uint32_t* __restrict__ Mw = SPARSE ? a.M + b * ((C + 31) / 32) * R + r : nullptr;
    uint8_t* __restrict__ q = a.q + b * C * R + r;
    const W0T* __restrict__ W0 = DISP ? static_cast<const W0T*>(a.W0) + b * C * R + r : nullptr;
    const int bw = a.bw;
    const int nsub = (bw + SB - 1) / SB;
    const float maxq = (float)a.maxq;
    float dmax = 0.0f;     // largest |d| this lane hands on in this block

    // (fast variants only) descriptors at the matrix's first row of this block
    const int row = (int)r;
    const rsrc_t rsA = row_rsrc(a.A + b * C * R + a.c0 * R);
    const rsrc_t rsB = row_rsrc(ERR_IN_A ? nullptr : a.B + b * C * R + a.c0 * R);
    const rsrc_t rsQ = row_rsrc(a.q + b * C * R + a.c0 * R);
    const rsrc_t rsS = row_rsrc(a.scales + b * (PER_ELEM ? C * R : a.G * R) + (PER_ELEM ? a.c0 * R : 0));
    const rsrc_t rsZ = row_rsrc(a.qzeros + b * (PER_ELEM ? C * R : a.G * R) + (PER_ELEM ? a.c0 * R : 0));
    const rsrc_t rsW = row_rsrc(DISP ? static_cast<const W0T*>(a.W0) + b * C * R + a.c0 * R : nullptr);
    const rsrc_t rsM = row_rsrc(SPARSE ? a.M + b * ((C + 31) / 32) * R : nullptr);

    float x[BW];
    if constexpr (TAIL) {
#pragma unroll
        for (int i = 0; i < BW; ++i) x[i] = (i < bw) ? A[(a.c0 + i) * R] : 0.0f;
    } else {
#pragma unroll
        for (int i = 0; i < BW; ++i) x[i] = (i < bw) ? buf_ld_f32(rsA, row * 4, (int)(i * R * 4)) : 0.0f;
    }

    if constexpr (!TAIL) {
        // rows c0..c0+bw-1 of U; of the 32 rows of sub-block i the columns from that sub-block on
        for (int i = 0; i < nsub; ++i) {
            const int w4 = (bw - i * SB) / 4;
            for (int idx = threadIdx.x; idx < SB * w4; idx += NT) {
                const int t = i * SB + idx / w4, j = idx % w4;
                *reinterpret_cast<float4*>(&Up[t][i * SB + 4 * j]) =
                    *reinterpret_cast<const float4*>(U + (a.c0 + t) * ldu + a.c0 + i * SB + 4 * j);
            }
        }
        __syncthreads();
    }

    // Scale and zero of a column do not depend on the sweep: all 32 pairs of a sub-block
    // are requested together, one sub-block ahead (while the previous sub-block's errors are
    // pushed), so that the serial chain never waits on them column by column.
    float sv[TAIL ? 1 : SB], qv[TAIL ? 1 : SB];
    auto load_meta = [&](int64_t c_first) {
        if constexpr (!TAIL) {
#pragma unroll
            for (int t = 0; t < SB; ++t) {
                const int64_t c = c_first + t;
                if constexpr (PER_ELEM) {
                    sv[t] = buf_ld_f32(rsS, row * 4, (int)((c - a.c0) * R * 4));
                    qv[t] = buf_ld_f32(rsZ, row * 4, (int)((c - a.c0) * R * 4));
                } else {
                    const int64_t g = gi[c];
                    sv[t] = buf_ld_f32(rsS, row * 4, (int)(g * R * 4));
                    qv[t] = buf_ld_f32(rsZ, row * 4, (int)(g * R * 4));
                }
            }
        }
    };
    load_meta(a.c0);

    for (int sb = 0; sb < nsub; ++sb) {
        const int64_t cs = a.c0 + (int64_t)sb * SB;   // first column of this sub-block
        const int rem = bw - sb * SB;                 // block columns from cs on
        float err[SB];
        uint32_t mask = 0u;
        // this sub-block's rows of U, from its own first column on
        const float* __restrict__ Ub = &Up[0][0] + (TAIL ? 0 : sb * (SB * BW + SB));

        auto select_and_quantize = [&](int t, int64_t c, float s, float q0) {
            bool keep = true;
            if constexpr (SPARSE) {
                if ((t & 3) == 0) {
                    // the values the score looks at: column t as it is, and the three columns
                    // after it BEFORE they have received this group's updates
                    float look[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) look[k] = x[t + k];
                    if constexpr (DISP) {
                        // Those three are not the same number in the two forms (only a column
                        // that has been reached is).  With d_j = x_j - w0_j, what the earlier
                        // columns have added so far, the error form's value of column k is
                        // w0_k + sum_{j<=k} d_j A[j,k], A the inverse of the 4x4 unit diagonal
                        // block of N = I - strict(V).
                        auto vv = [&](int j, int k) -> float {
                            if constexpr (TAIL) return (c + k < C) ? U[(c + j) * ldu + c + k] : 0.0f;
                            else return Ub[(t + j) * BW + t + k];
                        };
                        const float v01 = vv(0, 1), v02 = vv(0, 2), v03 = vv(0, 3);
                        const float v12 = vv(1, 2), v13 = vv(1, 3), v23 = vv(2, 3);
                        const float a02 = __builtin_fmaf(v01, v12, v02);
                        const float a13 = __builtin_fmaf(v12, v23, v13);
                        const float a03 = __builtin_fmaf(v01, a13, __builtin_fmaf(v02, v23, v03));
                        const float d0 = x[t] - err[t], d1 = x[t + 1] - err[t + 1];
                        const float d2 = x[t + 2] - err[t + 2];
                        look[1] = __builtin_fmaf(d0, v01, x[t + 1]);
                        look[2] = __builtin_fmaf(d1, v12, __builtin_fmaf(d0, a02, x[t + 2]));
                        look[3] = __builtin_fmaf(d2, v23, __builtin_fmaf(d1, a13, __builtin_fmaf(d0, a03, x[t + 3])));
                    }
                    float best = -1e30f;
                    int best_k = -1;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (!TAIL || c + k < C) {
                            const float score = fabsf(look[k] * uinv[c + k]);
                            if (best < score) { best = score; best_k = k; }
                        }
                    }
                    if (best_k > -1) mask |= 1u << (t + best_k);
                }
                keep = (mask >> t) & 1u;
            }
            float e, deq, qf;
            quantize_scalar(x[t], s, q0, maxq, qf, deq, e);
            if constexpr (DISP) e = err[t] - deq;   // err[t] holds the original weight here
            if constexpr (SPARSE) {
                // pruned column: code 0, weight 0, the whole value becomes the error
                qf = keep ? qf : 0.0f;
                deq = keep ? deq : 0.0f;
                e = keep ? e : (DISP ? err[t] : x[t]);
            }
            err[t] = e;
            if constexpr (DISP) dmax = fmaxf(dmax, fabsf(e));
            if constexpr (TAIL) {
                q[c * R] = (uint8_t)qf;
                if constexpr (ERR_IN_A) {
                    A[c * R] = e;
                } else {
                    A[c * R] = deq;
                    Bo[c * R] = e;
                }
            } else {
                const int col = (int)((c - a.c0) * R);
                __builtin_amdgcn_raw_buffer_store_b8((uint8_t)qf, rsQ, row, col, 0);
                if constexpr (ERR_IN_A) {
                    buf_st_f32(e, rsA, row * 4, col * 4);
                } else {
                    buf_st_f32(deq, rsA, row * 4, col * 4);
                    buf_st_f32(e, rsB, row * 4, col * 4);
                }
            }
        };

        if constexpr (!TAIL) {
            // (the original weights of the sub-block's second half are requested when a quarter of
            // the chain is done and as many scale/zero registers are free again: all 32 at the
            // start were the registers that the kernel did not have)
            if constexpr (DISP) {
#pragma unroll
                for (int t = 0; t < SB / 2; ++t) err[t] = buf_ld_w0(rsW, row, (cs - a.c0 + t) * R, (const W0T*)nullptr);
            }
            const bool more = sb + 1 < nsub;
            // U operands come from LDS 16 columns (4 broadcast ds_read_b128) at a time, read
            // two steps ahead of their use; scheduling barriers pin that distance (left
            // alone the scheduler hoists hundreds of reads and spills the x registers).
            // serial chain inside the sub-block: step = (row t, half h) -> 2*SB steps
            {
                const int l16 = threadIdx.x & 15;
                float ring[RING];
                auto rd = [&](int step) { return Ub[(step >> 1) * BW + (step & 1) * 16 + l16]; };
                ring[0] = rd(0);
                if (RING > 2) ring[1] = rd(1);
#pragma unroll
                for (int step = 0; step < 2 * SB; ++step) {
                    const int t = step >> 1, h = step & 1;
                    if (step + RING - 1 < 2 * SB) ring[(step + RING - 1) % RING] = rd(step + RING - 1);
                    if constexpr (DISP) {
                        if (step == SB / 2) {
#pragma unroll
                            for (int i = SB / 2; i < SB; ++i) err[i] = buf_ld_w0(rsW, row, (cs - a.c0 + i) * R, (const W0T*)nullptr);
                        }
                    }
                    if (h == 0) select_and_quantize(t, cs + t, sv[t], qv[t]);
                    __builtin_amdgcn_sched_barrier(0);
                    const float u16 = dpp_source(ring[step % RING]);
                    const float e = err[t];
#define FORGE_DIAG_FMA(k) if (h * 16 + k > t) fnma_row_bcast<k>(x[h * 16 + k], u16, e);
                    FORGE_FOR_16(FORGE_DIAG_FMA)
#undef FORGE_DIAG_FMA
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if constexpr (SPARSE) __builtin_amdgcn_raw_buffer_store_b32(mask, rsM, row * 4, (int)((cs >> 5) * R * 4), 0);
            if (more) load_meta(cs + SB);
            // push the 32 errors into the rest of the block
#pragma unroll
            for (int u = 1; u < NSB; ++u) {
                if (sb + u < nsub) {
                    const int l16 = threadIdx.x & 15;
                    float ring[RING];
                    auto rd = [&](int step) { return Ub[(step >> 1) * BW + u * SB + (step & 1) * 16 + l16]; };
                    ring[0] = rd(0);
                    if (RING > 2) ring[1] = rd(1);
#pragma unroll
                    for (int step = 0; step < 2 * SB; ++step) {
                        const int t = step >> 1, h = step & 1;
                        if (step + RING - 1 < 2 * SB) ring[(step + RING - 1) % RING] = rd(step + RING - 1);
                        __builtin_amdgcn_sched_barrier(0);
                        const float u16 = dpp_source(ring[step % RING]);
                        const float e = err[t];
#define FORGE_PUSH_FMA(k) fnma_row_bcast<k>(x[u * SB + h * 16 + k], u16, e);
                        FORGE_FOR_16(FORGE_PUSH_FMA)
#undef FORGE_PUSH_FMA
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        } else {
            if constexpr (DISP) {
#pragma unroll 1
                for (int t = 0; t < SB; ++t) err[t] = (t < rem) ? w0_as_f32(W0 + (cs + t) * R) : 0.0f;
            }
#pragma unroll 1
            for (int t = 0; t < SB; ++t) {
                if constexpr (!DISP) err[t] = 0.0f;
                if (t < rem) {
                    float s_t, q0_t;
                    if constexpr (PER_ELEM) {
                        s_t = sc[(cs + t) * R];
                        q0_t = qz[(cs + t) * R];
                    } else {
                        const int64_t g = gi[cs + t];
                        s_t = sc[g * R];
                        q0_t = qz[g * R];
                    }
                    select_and_quantize(t, cs + t, s_t, q0_t);
                    const float* __restrict__ Urow = U + (cs + t) * ldu + cs;
                    for (int k = t + 1; k < rem; ++k)
                        x[k] = __builtin_fmaf(-Urow[k], err[t], x[k]);
                }
            }
            if constexpr (SPARSE) Mw[(cs >> 5) * R] = mask;
        }
#pragma unroll
        for (int i = 0; i + SB < BW; ++i) x[i] = x[i + SB];
    }
    if constexpr (DISP) {
        // one lane per row: no other lane touches this entry (the first block starts it)
        if (a.dbound) {
            float* p = a.dbound + b * R + r;
            *p = a.c0 == 0 ? dmax : fmaxf(*p, dmax);
        }
    }
}

// The same bounds from the lower factor that V is made of, V[t, m] = -(Al[m, t] * (1 / Al[m, m])):
// the largest |Al[m, t]|, t < m, times |1 / Al[m, m]| (rounding is monotone, so this is the
// largest |V[t, m]| exactly).  One wavefront per row; 0 for matrices whose info is not 0.
__global__ __launch_bounds__(256) void lower_row_bound_kernel(const float* __restrict__ Al, int64_t C,
                                                              const int32_t* __restrict__ info,
                                                              float* __restrict__ bound) {
    const int64_t b = blockIdx.y, m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (m >= C) return;
    const int lane = threadIdx.x & 63;
    const float* __restrict__ row = Al + b * C * C + m * C;
    float mx = 0.0f;
    for (int64_t t = lane; t < m; t += 64) mx = fmaxf(mx, fabsf(row[t]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (lane == 0) {
        const bool failed = info != nullptr && info[b] != 0;
        bound[b * C + m] = failed ? 0.0f : fabsf(mx * (1.0f / row[m]));
    }
}

// X[b][c][r] = W0[b][c][r] for the first `rows` solver columns c of every matrix (the blocks that
// no long product writes before they are swept).
template <typename W0T>
__global__ __launch_bounds__(256) void rows_from_w0_kernel(float* __restrict__ X, const W0T* __restrict__ W0,
                                                           int64_t C, int64_t R, int64_t rows) {
    const int64_t b = blockIdx.y, n = rows * R;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        X[b * C * R + i] = w0_as_f32(W0 + b * C * R + i);
}

// bound[m] = max_{t < m} |V[t, m]| for every column of the unit upper matrix V (the strict upper
// triangle is all that the block updates read).  One workgroup per (128 columns, matrix).
__global__ __launch_bounds__(256) void upper_column_bound_kernel(const float* __restrict__ V, int64_t C,
                                                                 float* __restrict__ bound) {
    __shared__ float red[8][128];
    const int64_t b = blockIdx.y, m0 = (int64_t)blockIdx.x * 128;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const float* __restrict__ Vb = V + b * C * C;
    float mx[4] = {0.f, 0.f, 0.f, 0.f};
    const int64_t rows = (m0 + 128) < C ? (m0 + 128) : C;
    for (int64_t t = ty; t < rows; t += 8) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t m = m0 + 4 * tx + e;
            if (m < C && t < m) mx[e] = fmaxf(mx[e], fabsf(Vb[t * C + m]));
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[ty][4 * tx + e] = mx[e];
    __syncthreads();
    if (threadIdx.x < 128) {
        float v = red[0][threadIdx.x];
#pragma unroll
        for (int i = 1; i < 8; ++i) v = fmaxf(v, red[i][threadIdx.x]);
        if (m0 + threadIdx.x < C) bound[b * C + m0 + threadIdx.x] = v;
    }
}

// U[i, :] *= 1/U[i,i]; uinv[i] = 1/U[i,i]   (solver_sparsegptq14.cu:153-155)
__global__ void row_normalise_kernel(float* __restrict__ U, float* __restrict__ uinv, int64_t C) {
    const int64_t i = blockIdx.x;
    const float inv = 1.0f / U[i * C + i];
    for (int64_t j = threadIdx.x; j < C; j += blockDim.x) U[i * C + j] = U[i * C + j] * inv;
    if (threadIdx.x == 0) uinv[i] = inv;
}

template <bool SPARSE, bool PER_ELEM, bool DISP = false, typename W0T = float>
int launch_block(const SweepArgs& a, int64_t batch, hipStream_t st) {
    constexpr bool ERR_IN_A = !PER_ELEM;  // batched form keeps the errors in place
    forge::KernelTiming timing(SPARSE ? "sweep_block_sparse14" : "sweep_block", st,
                               (double)a.bw * (a.bw - 1) * (double)a.R * (double)batch,
                               forge::WORK_FLOPS);
    // the LDS-staged variants need whole wavefronts (every lane helps to load the panel)
    // (and their byte offsets from a block's or a matrix's first row fit 31 bits)
    const int64_t far = 128 > a.G ? (128 > a.C / 32 + 1 ? 128 : a.C / 32 + 1)
                                  : (a.G > a.C / 32 + 1 ? a.G : a.C / 32 + 1);
    const bool fast = a.bw % 32 == 0 && (a.ldu ? a.ldu : a.C) % 4 == 0 && a.c0 % 4 == 0 && a.R % 64 == 0 &&
                      (reinterpret_cast<uintptr_t>(a.U) % 16) == 0 && (far + 1) * a.R * 4 < (1LL << 31);
    if (fast && a.R % 256 == 0) {
        dim3 grid((unsigned)(a.R / 256), (unsigned)batch);
        sweep_block_kernel<forge_kBW, 256, SPARSE, PER_ELEM, ERR_IN_A, false, DISP, W0T>
            <<<grid, dim3(256), 0, st>>>(a);
    } else {
        dim3 grid((unsigned)forge::ceil_div(a.R, 64), (unsigned)batch);
        if (fast)
            sweep_block_kernel<forge_kBW, 64, SPARSE, PER_ELEM, ERR_IN_A, false, DISP, W0T>
                <<<grid, dim3(64), 0, st>>>(a);
        else
            sweep_block_kernel<forge_kBW, 64, SPARSE, PER_ELEM, ERR_IN_A, true, DISP, W0T>
                <<<grid, dim3(64), 0, st>>>(a);
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

int check_sweep_shape(int64_t C, int64_t R, int bits) {
    FORGE_REQUIRE(bits >= 1 && bits <= 8, "bits=%d outside 1..8", bits);
    FORGE_REQUIRE(C >= 1 && R >= 1 && C < (1 << 30) && R < (1 << 30), "bad shape C=%lld R=%lld",
                  (long long)C, (long long)R);
    return FORGE_OK;
}

}  // namespace

namespace forge {
constexpr int kBW = forge_kBW;
}

// Right-looking schedule for one matrix with per-element metadata (reference signature).
template <bool SPARSE>
static int solve_single(float* W, const float* U, const float* scales, const float* qzeros,
                        int bits, int64_t C, int64_t R, uint8_t* q, uint32_t* M, float* E,
                        const float* uinv, hipStream_t st) {
    for (int64_t start = 0; start < C; start += forge::kBW) {
        const int bw = (int)((C - start) < forge::kBW ? (C - start) : forge::kBW);
        SweepArgs a{};
        a.A = W; a.B = E; a.U = U; a.scales = scales; a.qzeros = qzeros; a.g_idx = nullptr;
        a.q = q; a.M = M; a.uinv = uinv; a.C = C; a.R = R; a.G = 0; a.c0 = start; a.bw = bw;
        a.maxq = (1 << bits) - 1;
        if (int e = launch_block<SPARSE, true>(a, 1, st)) return e;
        forge::GemmArgs g{};
        g.X = W; g.At = U; g.Bm = E; g.ldx = R; g.lda = C; g.ldb = R; g.xs = g.as = g.bs = 0;
        g.m0 = (int)(start + bw); g.m1 = (int)C; g.n1 = (int)R; g.k0 = (int)start;
        g.k1 = (int)(start + bw); g.negate_a = true;
        if (int e = forge::launch_chain_gemm(g, 1, st)) return e;
    }
    return FORGE_OK;
}

extern "C" int forge_gptq_solver(float* W, const float* U, const float* scales,
                                 const float* qzeros, int bits, int64_t C, int64_t R,
                                 uint8_t* qweight, float* E, forge_stream_t stream) {
    if (int e = check_sweep_shape(C, R, bits)) return e;
    FORGE_REQUIRE(W && U && scales && qzeros && qweight && E, "null pointer");
    return solve_single<false>(W, U, scales, qzeros, bits, C, R, qweight, nullptr, E, nullptr,
                               (hipStream_t)stream);
}

extern "C" int forge_sparsegptq14_solver(float* W, float* U, const float* scales,
                                         const float* qzeros, int bits, int64_t C, int64_t R,
                                         uint8_t* qweight, uint32_t* M, float* E, float* uinv,
                                         forge_stream_t stream) {
    if (int e = check_sweep_shape(C, R, bits)) return e;
    FORGE_REQUIRE(W && U && scales && qzeros && qweight && M && E && uinv, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    row_normalise_kernel<<<dim3((unsigned)C), dim3(256), 0, st>>>(U, uinv, C);
    FORGE_LAUNCH_CHECK();
    return solve_single<true>(W, U, scales, qzeros, bits, C, R, qweight, M, E, uinv, st);
}

// Few matrices: a left-looking step has only batch * R/128 tiles, far fewer than the GPU
// has CUs.  Then every finished block is pushed into ALL later columns at once instead
// (K = 128, (C - start)/128 times as many tiles); the weights are re-read per step, which
// a batch could not afford.  Same fma chain per element, hence the same bits.
static bool right_looking_schedule(int64_t batch, int64_t R) {
    bool right_looking = batch * forge::ceil_div(R, 128) < 128;
    const int64_t forced = forge::option(forge::OPT_SWEEP_SCHEDULE);
    if (forced == 1) right_looking = false;
    if (forced == 2) right_looking = true;
    return right_looking;
}

// The even blocks' long product, as sweep_batched launches it for block `start`.
static forge::GemmArgs even_block_update(float* X, const float* U, int64_t C, int64_t R, int64_t start) {
    forge::GemmArgs g{};
    g.X = X; g.At = U; g.Bm = X; g.ldx = R; g.lda = C; g.ldb = R;
    g.xs = C * R; g.as = C * C; g.bs = C * R;
    g.m0 = (int)start; g.n1 = (int)R; g.k0 = 0; g.k1 = (int)start;
    g.m1 = (int)(start + 2 * forge::kBW <= C ? start + 2 * forge::kBW : start + forge::kBW);
    g.negate_a = true;
    g.blocked_sum = true;
    g.products = 3;
    return g;
}

// True when, given the lower factor, the displacement-form sweep reads V only within one
// 128-column block of its diagonal: left-looking schedule and every even block's product on the
// piece path (whole 128 x 128 tiles, aligned rows), whose A panels then come from the factor.
static bool sweep_reads_band_only(float* X, const float* U, int64_t batch, int64_t C, int64_t R,
                                  int64_t split_bytes) {
    if (right_looking_schedule(batch, R) || C % forge::kBW != 0 || C <= forge::kBW) return false;
    // the last even block has the longest K (and the largest offsets); alignment is the same for all
    const int64_t nblk = C / forge::kBW, last_even = ((nblk - 1) / 2) * 2;
    if (last_even == 0) return false;
    return forge::split_path_applies(even_block_update(X, U, C, R, last_even * forge::kBW), batch, split_bytes) &&
           forge::split_path_applies(even_block_update(X, U, C, R, 2 * forge::kBW), batch, split_bytes);
}

// Left-looking schedule for a batch of equally shaped matrices, errors (or, with W0, the
// displacements) kept in X.
static int sweep_batched(float* X, const void* W0, bool w0_bf16, bool x_from_w0, const float* U,
                         const float* Lf, const int32_t* Linfo, const float* scalesT,
                         const float* qzerosT, const int32_t* g_idx, uint8_t* qweight,
                         uint32_t* M, const float* uinv, int64_t batch, int64_t C, int64_t R,
                         int64_t G, int bits, int sparse14, void* ws, int64_t ws_bytes,
                         forge_stream_t stream) {
    if (int e = check_sweep_shape(C, R, bits)) return e;
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && G >= 1, "bad batch=%lld G=%lld", (long long)batch,
                  (long long)G);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(X && U && scalesT && qzerosT && g_idx && qweight, "null pointer");
    FORGE_REQUIRE(!sparse14 || (M && uinv), "sparse14 needs M and uinv");
    FORGE_REQUIRE(W0 != X, "W0 must be a copy of X, not X itself");
    hipStream_t st = (hipStream_t)stream;
    const bool right_looking = right_looking_schedule(batch, R);
    // The direct route's block updates on the 16-bit matrix pipe, three products per fp32
    // product.  Below 4096 columns two fp16 halves per operand, fp32-grade: the columns of V are
    // scaled from their largest entry above the diagonal, the rows of displacements from a
    // running maximum that the block kernel keeps.  From 4096 columns on two bf16 pieces, each
    // rounded to nearest (~2^-17): there the codes' own sensitivity to fp32 rounding is an order
    // of magnitude above what the shorter pieces add, the updates are most of the sweep's time,
    // and under the power limit the bf16 instruction runs ~5 % faster than the fp16 one.  The
    // option sweep_update_products overrides (2: fp16 halves; bf16 pieces: 6 three truncated
    // pieces, fp32-grade; 3 / 4 two rounded pieces; 1 plain bf16).
    int products = (int)forge::option(forge::OPT_SWEEP_PRODUCTS);
    if (products == 0) products = C >= 4096 ? 3 : 2;
    const bool halves = ws && W0 && products == 2 && !right_looking && C > forge::kBW;
    const int64_t split_bytes = C > forge::kBW ? 2 * forge::split_gemm_workspace_bytes(batch, C - forge::kBW) : 0;
    float* vbound = nullptr;
    float* dbound = nullptr;
    if (halves) {
        vbound = (float*)((char*)ws + split_bytes);
        dbound = (float*)((char*)ws + split_bytes + (batch * C * 4 + 255) / 256 * 256);
    }
    // With the lower factor at hand the even blocks' A panels are formed from its rows: V is
    // then read only within one block of its diagonal (in-block chains, odd blocks' K = 128
    // products), provided every even block takes the piece path.
    const bool all_pieces = ws && W0 && sweep_reads_band_only(X, U, batch, C, R, split_bytes);
    const bool from_lower = Lf != nullptr && all_pieces;
    // X not laid out by the caller: every block from the third on is first written by its long
    // product, which then starts from W0; the first two are copied here
    FORGE_REQUIRE(!x_from_w0 || all_pieces,
                  "x_from_w0 needs the shape for which forge_gptq_sweep_direct_reads_band_only returns 1");
    if (x_from_w0) {
        const int64_t rows = C < 2 * forge::kBW ? C : 2 * forge::kBW;
        const dim3 grid((unsigned)forge::ceil_div(rows * R, 256 * 8), (unsigned)batch);
        if (w0_bf16)
            rows_from_w0_kernel<uint16_t><<<grid, dim3(256), 0, st>>>(X, (const uint16_t*)W0, C, R, rows);
        else
            rows_from_w0_kernel<float><<<grid, dim3(256), 0, st>>>(X, (const float*)W0, C, R, rows);
        FORGE_LAUNCH_CHECK();
    }
    if (halves) {
        if (from_lower)
            lower_row_bound_kernel<<<dim3((unsigned)forge::ceil_div(C, 4), (unsigned)batch), dim3(256), 0, st>>>(
                Lf, C, Linfo, vbound);
        else
            upper_column_bound_kernel<<<dim3((unsigned)forge::ceil_div(C, 128), (unsigned)batch), dim3(256), 0, st>>>(
                U, C, vbound);
        FORGE_LAUNCH_CHECK();
    }
    for (int64_t start = 0; start < C; start += forge::kBW) {
        const int bw = (int)((C - start) < forge::kBW ? (C - start) : forge::kBW);
        forge::GemmArgs g{};
        g.X = X; g.At = U; g.Bm = X; g.ldx = R; g.lda = C; g.ldb = R;
        g.xs = C * R; g.as = C * C; g.bs = C * R;
        g.m0 = (int)start; g.m1 = (int)(start + bw); g.n1 = (int)R; g.k0 = 0; g.k1 = (int)start;
        g.negate_a = true;
        if (right_looking) {
            // nothing to do here: the earlier blocks have already been pushed into this one
        } else if (ws) {
            // sums from 16-bit pieces of the operands on the fp16 / bf16 matrix pipe where the
            // block is a full tile (fp32 matrix pipe otherwise).  That product is
            // bound by reading the displacement rows of all earlier columns from HBM, so full
            // blocks are brought up to date two at a time: every row read then serves 256
            // columns (one workgroup computes both blocks' tiles where the pieces allow it), and
            // the odd block only lacks what its even neighbour adds, a K = 128 product on the
            // fp32 pipe.
            const bool pairs = C % forge::kBW == 0;
            const bool odd = pairs && ((start / forge::kBW) & 1) != 0;
            if (!odd) {
                g.blocked_sum = true;
                g.products = products == 2 ? 6 : products;
                if (halves) {
                    g.bound_a = vbound; g.bound_a_stride = C;
                    g.bound_b = dbound; g.bound_b_stride = R;
                }
                if (from_lower) {
                    g.a_lower = Lf; g.a_lower_ld = C; g.a_lower_stride = C * C; g.a_info = Linfo;
                }
                if (x_from_w0) { g.x_init = W0; g.x_init_bf16 = w0_bf16; }
                if (pairs && start + 2 * forge::kBW <= C) g.m1 = (int)(start + 2 * forge::kBW);
                if (int e = forge::launch_chain_gemm_pair(g, forge::GemmArgs{}, batch, st, ws, split_bytes)) return e;
                g.m1 = (int)(start + bw);
                g.a_lower = nullptr;
                g.x_init = nullptr;
            } else {
                g.k0 = (int)(start - forge::kBW);
                if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
            }
        } else {
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
        }
        SweepArgs a{};
        a.A = X; a.B = nullptr; a.U = U; a.scales = scalesT; a.qzeros = qzerosT; a.g_idx = g_idx;
        a.q = qweight; a.M = M; a.uinv = uinv; a.C = C; a.R = R; a.G = G; a.c0 = start; a.bw = bw;
        a.W0 = W0;
        a.w0_bf16 = w0_bf16;
        a.dbound = halves ? dbound : nullptr;
        a.maxq = (1 << bits) - 1;
        int e;
        if (!W0) e = sparse14 ? launch_block<true, false>(a, batch, st) : launch_block<false, false>(a, batch, st);
        else if (w0_bf16)
            e = sparse14 ? launch_block<true, false, true, uint16_t>(a, batch, st)
                         : launch_block<false, false, true, uint16_t>(a, batch, st);
        else
            e = sparse14 ? launch_block<true, false, true>(a, batch, st)
                         : launch_block<false, false, true>(a, batch, st);
        if (e) return e;
        if (right_looking && start + bw < C) {
            g.m0 = (int)(start + bw); g.m1 = (int)C; g.k0 = (int)start; g.k1 = (int)(start + bw);
            if (int e2 = forge::launch_chain_gemm(g, batch, st)) return e2;
        }
    }
    return FORGE_OK;
}

extern "C" int forge_gptq_sweep_batched(float* X, const float* U, const float* scalesT,
                                        const float* qzerosT, const int32_t* g_idx,
                                        uint8_t* qweight, uint32_t* M, const float* uinv,
                                        int64_t batch, int64_t C, int64_t R, int64_t G, int bits,
                                        int sparse14, forge_stream_t stream) {
    return sweep_batched(X, nullptr, false, false, U, nullptr, nullptr, scalesT, qzerosT, g_idx, qweight, M,
                         uinv, batch, C, R, G, bits, sparse14, nullptr, 0, stream);
}

extern "C" int64_t forge_gptq_sweep_direct_workspace_bytes(int64_t batch, int64_t C, int64_t R) {
    if (batch <= 0 || C <= forge::kBW || R <= 0) return 0;
    // the split A panels of two column blocks per product, one bound per column of V and one
    // per row of displacements
    return 2 * forge::split_gemm_workspace_bytes(batch, C - forge::kBW) +
           (batch * C * 4 + 255) / 256 * 256 + (batch * R * 4 + 255) / 256 * 256;
}

extern "C" int forge_gptq_sweep_direct_reads_band_only(int64_t batch, int64_t C, int64_t R) {
    if (batch <= 0 || C <= 0 || R <= 0) return 0;
    // stand-in pointers: only their alignment is looked at (device allocations are aligned)
    float* aligned = reinterpret_cast<float*>(uintptr_t(256));
    const int64_t split_bytes = C > forge::kBW ? 2 * forge::split_gemm_workspace_bytes(batch, C - forge::kBW) : 0;
    return sweep_reads_band_only(aligned, aligned, batch, C, R, split_bytes) ? 1 : 0;
}

extern "C" int forge_gptq_sweep_direct_batched_w0(float* X, const void* W0, int w0_dtype, int x_from_w0,
                                                  const float* V, const float* L, const int32_t* info,
                                                  const float* scalesT, const float* qzerosT,
                                                  const int32_t* g_idx, uint8_t* qweight,
                                                  uint32_t* M, const float* mdiag,
                                                  int64_t batch, int64_t C, int64_t R, int64_t G,
                                                  int bits, int sparse14, void* ws, int64_t ws_bytes,
                                                  forge_stream_t stream) {
    FORGE_REQUIRE(W0 || batch == 0, "null pointer");
    FORGE_REQUIRE(w0_dtype == FORGE_F32 || w0_dtype == FORGE_BF16, "w0_dtype=%d", w0_dtype);
    FORGE_REQUIRE(!ws || ws_bytes >= forge_gptq_sweep_direct_workspace_bytes(batch, C, R),
                  "workspace of %lld bytes, %lld needed", (long long)ws_bytes,
                  (long long)forge_gptq_sweep_direct_workspace_bytes(batch, C, R));
    return sweep_batched(X, W0, w0_dtype == FORGE_BF16, x_from_w0 != 0, V, L, info, scalesT, qzerosT, g_idx,
                         qweight, M, mdiag, batch, C, R, G, bits, sparse14, ws, ws_bytes, stream);
}

extern "C" int forge_gptq_sweep_direct_batched(float* X, const float* W0, const float* V,
                                               const float* scalesT, const float* qzerosT,
                                               const int32_t* g_idx, uint8_t* qweight,
                                               uint32_t* M, const float* mdiag,
                                               int64_t batch, int64_t C, int64_t R, int64_t G,
                                               int bits, int sparse14, void* ws, int64_t ws_bytes,
                                               forge_stream_t stream) {
    return forge_gptq_sweep_direct_batched_w0(X, W0, FORGE_F32, 0, V, nullptr, nullptr, scalesT, qzerosT, g_idx,
                                              qweight, M, mdiag, batch, C, R, G, bits, sparse14, ws,
                                              ws_bytes, stream);
}

// ------------------------------------------------------------------ sweep from the rows, blocked
// The displacement-form sweep for matrices whose factor is given by forge_rows_factor_blocked:
// the entries of the factor's row k left of k's own 128-column block are h_k . b_t, so all that
// the earlier blocks hand to block J is the n x R matrix  A = sum_{t before J} b_t d_t^T  (d_t the
// displacements of column t, one per output row):
//     X_J  = W0_J + Hm_J A          128 x R, inner dimension n     (before the block is swept)
//     A   += B_J^T D_J              n x R, inner dimension 128     (after it)
// 4 n C R multiply-adds per matrix instead of C^2 R / 2, and the in-block chains unchanged.
extern "C" int64_t forge_gptq_sweep_rows_workspace_bytes(int64_t batch, int64_t R, int64_t nmax) {
    if (batch <= 0 || R <= 0 || nmax <= 0) return 0;
    // A, and the 16-bit pieces of a block's h vectors (the shared operand of its product)
    return (batch * nmax * R * (int64_t)sizeof(float) + 255) / 256 * 256 +
           forge::split_gemm_workspace_bytes(batch, nmax);
}

extern "C" int forge_gptq_sweep_rows_blocked(float* X, const void* W0, int w0_dtype, const float* HmT,
                                             const float* Bp, const float* V, const int32_t* n_rows,
                                             const int32_t* n_rows_host, const float* scalesT,
                                             const float* qzerosT,
                                             const int32_t* g_idx, uint8_t* qweight, int64_t batch,
                                             int64_t C, int64_t R, int64_t G, int bits, int64_t nmax,
                                             void* ws, int64_t ws_bytes, forge_stream_t stream) {
    if (int e = check_sweep_shape(C, R, bits)) return e;
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && G >= 1, "bad batch=%lld G=%lld", (long long)batch,
                  (long long)G);
    FORGE_REQUIRE(C % forge::kBW == 0 && R % 128 == 0, "C=%lld and R=%lld must be multiples of 128",
                  (long long)C, (long long)R);
    FORGE_REQUIRE(nmax >= 128 && nmax % 128 == 0, "nmax=%lld: a multiple of 128", (long long)nmax);
    FORGE_REQUIRE(w0_dtype == FORGE_F32 || w0_dtype == FORGE_BF16, "w0_dtype=%d", w0_dtype);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(X && W0 && HmT && Bp && V && n_rows && scalesT && qzerosT && g_idx && qweight && ws,
                  "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_gptq_sweep_rows_workspace_bytes(batch, R, nmax), "workspace too small");
    hipStream_t st = (hipStream_t)stream;
    float* A = (float*)ws;
    double f1 = 1.0;         // for the timing records only: the batch's own share of the nominal work
    if (n_rows_host) {
        f1 = 0.0;
        for (int64_t b = 0; b < batch; ++b) {
            FORGE_REQUIRE(n_rows_host[b] >= 128 && n_rows_host[b] <= nmax && n_rows_host[b] % 128 == 0,
                          "n_rows[%lld]=%d: a multiple of 128 up to nmax", (long long)b, n_rows_host[b]);
            f1 += (double)n_rows_host[b] / (double)nmax / (double)batch;
        }
    }
    void* split_ws = (char*)ws + (batch * nmax * R * (int64_t)sizeof(float) + 255) / 256 * 256;
    const int64_t split_bytes = forge::split_gemm_workspace_bytes(batch, nmax);
    const bool w0_bf16 = w0_dtype == FORGE_BF16;
    for (int64_t start = 0; start < C; start += forge::kBW) {
        if (start > 0) {
            // on the 16-bit matrix pipe from two rounded bf16 pieces per operand (three products,
            // within ~2^-17 of the fp32 product: what the route through the Hessian takes for
            // its block updates from 4096 columns on), starting from the untouched weights;
            // fp32 matrix instruction from X where the option fp32_blocked_sum asks for it
            forge::GemmArgs g{};
            g.X = X; g.ldx = R; g.xs = C * R;
            g.At = HmT; g.lda = C; g.as = nmax * C;
            g.Bm = A; g.ldb = R; g.bs = nmax * R;
            g.m0 = (int)start; g.m1 = (int)(start + forge::kBW); g.n1 = (int)R; g.k1 = (int)nmax;
            g.blocked_sum = true;
            g.products = 3;
            g.x_init = W0; g.x_init_bf16 = w0_bf16;
            g.lim = n_rows; g.lim_k = true; g.work_frac = f1;
            if (int e = forge::launch_chain_gemm_pair(g, forge::GemmArgs{}, batch, st, split_ws, split_bytes))
                return e;
        }
        SweepArgs a{};
        a.A = X; a.U = V; a.ldu = forge::kBW; a.u_stride = C * forge::kBW; a.u_band = true;
        a.scales = scalesT; a.qzeros = qzerosT; a.g_idx = g_idx; a.q = qweight;
        a.C = C; a.R = R; a.G = G; a.c0 = start; a.bw = forge::kBW;
        a.W0 = W0; a.w0_bf16 = w0_bf16; a.maxq = (1 << bits) - 1;
        if (int e = w0_bf16 ? launch_block<false, false, true, uint16_t>(a, batch, st)
                            : launch_block<false, false, true>(a, batch, st))
            return e;
        if (start + forge::kBW < C) {
            forge::GemmArgs g{};
            g.X = A; g.ldx = R; g.xs = nmax * R;
            g.At = Bp; g.lda = nmax; g.as = C * nmax;
            g.Bm = X; g.ldb = R; g.bs = C * R;
            g.m1 = (int)nmax; g.n1 = (int)R; g.k0 = (int)start; g.k1 = (int)(start + forge::kBW);
            g.init_zero = start == 0;
            g.blocked_sum = true;
            g.lim = n_rows; g.lim_m = true; g.work_frac = f1;
            if (int e = forge::launch_chain_gemm(g, batch, st)) return e;
        }
    }
    return FORGE_OK;
}

// ------------------------------------------------------------------ Babai (nearest plane)
// solver_babai.cu:123-322 walks the columns from the last to the first and, after
// quantising column t, removes err_t * A[i,t] / A[i,i] from every earlier column i, A being
// the upper Cholesky factor of H.  With both index orders reversed (t' = C-1-t) this is the
// forward sweep above with the unit upper matrix U'[t',k'] = A[C-1-k', C-1-t'] / A[C-1-k', C-1-k']:
// same quantiser, same fused multiply-adds, one chain per element in the same order.  So the
// operator is a few index-reversing copies around gptq_sweep_batched.
namespace {

template <typename T>
__global__ void reverse_rows_kernel(const T* __restrict__ src, T* __restrict__ dst, int64_t C, int64_t R) {
    // rows on grid.x (no 65535 limit), row pieces on grid.y
    const int64_t c = blockIdx.x;
    for (int64_t r = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; r < R; r += (int64_t)gridDim.y * blockDim.x)
        dst[c * R + r] = src[(C - 1 - c) * R + r];
}

// scales/qzeros [R*G] (index r*G + g) -> [G, R]; g_idx reversed and clamped to G-1
// (solver_babai.cu:196-197)
__global__ void babai_meta_kernel(const float* __restrict__ scales, const float* __restrict__ qzeros,
                                  const int32_t* __restrict__ g_idx, float* __restrict__ sT,
                                  float* __restrict__ zT, int32_t* __restrict__ g_rev, int64_t C,
                                  int64_t R, int64_t G, int64_t group_size) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < R * G) {
        const int64_t g = i / R, r = i - g * R;
        sT[i] = scales[r * G + g];
        zT[i] = qzeros[r * G + g];
    }
    if (i < C) {
        const int64_t row = C - 1 - i;
        int64_t g = g_idx ? (int64_t)g_idx[row] : row / group_size;
        if (g >= G) g = G - 1;
        if (g < 0) g = 0;
        g_rev[i] = (int32_t)g;
    }
}

int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

extern "C" int64_t forge_babai_workspace_bytes(int64_t C, int64_t R, int64_t G) {
    if (C <= 0 || R <= 0 || G <= 0) return 0;
    return align256(C * C * 4) + align256(C * R * 4) + 2 * align256(G * R * 4) + align256(C * 4) +
           align256(C * R);
}

extern "C" int forge_unit_upper_from_lower(const float* L, const int32_t* info, float* U,
                                           int64_t batch, int64_t C, int flipped_upper,
                                           forge_stream_t stream);

extern "C" int forge_babai_solver(const float* W, const float* A, const float* scales,
                                  const float* qzeros, const int32_t* g_idx, int64_t group_size,
                                  int bits, int64_t C, int64_t R, int64_t G, uint8_t* qweight,
                                  void* ws, int64_t ws_bytes, forge_stream_t stream) {
    if (int e = check_sweep_shape(C, R, bits)) return e;
    FORGE_REQUIRE(G >= 1 && group_size >= 1, "bad G=%lld group_size=%lld", (long long)G, (long long)group_size);
    FORGE_REQUIRE(W && A && scales && qzeros && qweight && ws, "null pointer");
    FORGE_REQUIRE(ws_bytes >= forge_babai_workspace_bytes(C, R, G), "workspace too small");
    hipStream_t st = (hipStream_t)stream;
    char* p = (char*)ws;
    float* Ur = (float*)p; p += align256(C * C * 4);
    float* Xr = (float*)p; p += align256(C * R * 4);
    float* sT = (float*)p; p += align256(G * R * 4);
    float* zT = (float*)p; p += align256(G * R * 4);
    int32_t* g_rev = (int32_t*)p; p += align256(C * 4);
    uint8_t* qr = (uint8_t*)p;
    if (int e = forge_unit_upper_from_lower(A, nullptr, Ur, 1, C, 1, stream)) return e;
    const int64_t pieces = forge::ceil_div(R, 256);
    const unsigned gx = (unsigned)(pieces < 65535 ? pieces : 65535);   // the kernel strides over the rest
    reverse_rows_kernel<float><<<dim3((unsigned)C, gx), dim3(256), 0, st>>>(W, Xr, C, R);
    FORGE_LAUNCH_CHECK();
    const int64_t nmeta = R * G > C ? R * G : C;
    babai_meta_kernel<<<dim3((unsigned)forge::ceil_div(nmeta, 256)), dim3(256), 0, st>>>(
        scales, qzeros, g_idx, sT, zT, g_rev, C, R, G, group_size);
    FORGE_LAUNCH_CHECK();
    if (int e = forge_gptq_sweep_batched(Xr, Ur, sT, zT, g_rev, qr, nullptr, nullptr, 1, C, R, G, bits, 0, stream))
        return e;
    reverse_rows_kernel<uint8_t><<<dim3((unsigned)C, gx), dim3(256), 0, st>>>(qr, qweight, C, R);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
