// Group scale/zero search: min/max grid and MSE (Lp) shrink search.
//
// Arithmetic follows forge/backend/cuda/quant_grid.cu:42-183 of the reference: the same
// fp32 formulas, the same first-strict-minimum rule and the same summation tree for the
// candidate loss (32 partial sums of gs/32 elements each, then a halving tree), so that
// only the hardware log2/exp2 approximations can make a near-tie resolve differently.
//
// Mapping to CDNA4: the min/max kernel is HBM-bound and gives half a wavefront to each
// group (coalesced 128 B rows); the shrink search is VALU/transcendental-bound and gives
// one LANE to each group: all gs values sit in that lane's registers, the P candidates
// are evaluated without any cross-lane traffic, and the per-candidate scalar work
// (scale, reciprocal, zero point) is paid once per group instead of once per lane.
#include "common.h"
#include <hip/hip_bf16.h>

namespace {

constexpr float kEps = 1e-12f;

__device__ __forceinline__ float ld_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_as_f32(const __hip_bfloat16* p) {
    return __uint_as_float(static_cast<uint32_t>(*reinterpret_cast<const uint16_t*>(p)) << 16);
}

__device__ __forceinline__ float clampf(float v, float lo, float hi) {
    // one v_med3_f32; equal to fminf(fmaxf(v, lo), hi) for lo <= hi (a NaN gives lo in both)
    return __builtin_amdgcn_fmed3f(v, lo, hi);
}

// Scale and zero of one group from its extrema (quant_grid.cu:74-97).
__device__ __forceinline__ void meta_from_extrema(float xmin, float xmax, float maxq,
                                                  bool symmetric, float& s, float& q0) {
    if (symmetric) {
        float amax = fmaxf(fabsf(xmin), fabsf(xmax));
        s = __builtin_fmaf(2.0f / maxq, amax, kEps);
        q0 = 0.5f * (maxq + 1.0f);
    } else {
        s = (xmax - xmin) / maxq + kEps;
        q0 = clampf(__builtin_rintf(-xmin / s), 0.0f, maxq);
    }
}

// ---------------------------------------------------------------- min/max grid
// One half-wavefront (32 lanes) per group.  Group `g` of the flattened [batch*R*G] list
// covers columns [grp*gs, grp*gs+gs) of row r, columns >= C read as zero.
template <typename T>
__global__ __launch_bounds__(256) void minmax_grid_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t R, int64_t C, int64_t ldw, int64_t gs,
    int64_t G, int64_t n_groups, float maxq, bool symmetric, float* __restrict__ scales,
    float* __restrict__ qzeros) {
    const int lane = threadIdx.x & 31;
    const int64_t half = (int64_t)blockIdx.x * (blockDim.x >> 5) + (threadIdx.x >> 5);
    const int64_t stride = (int64_t)gridDim.x * (blockDim.x >> 5);
    for (int64_t g = half; g < n_groups; g += stride) {
        const int64_t b = g / (R * G);
        const int64_t rg = g - b * R * G;
        const int64_t r = rg / G, grp = rg - r * G;
        const T* row = W + b * w_stride + r * ldw;
        const int64_t c0 = grp * gs;
        float lo = 1e30f, hi = -1e30f;
        for (int64_t i = lane; i < gs; i += 32) {
            const int64_t c = c0 + i;
            const float v = (c < C) ? ld_as_f32(row + c) : 0.0f;
            hi = fmaxf(hi, v);
            lo = fminf(lo, v);
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
            hi = fmaxf(hi, __shfl_down(hi, off, 32));
            lo = fminf(lo, __shfl_down(lo, off, 32));
        }
        if (lane == 0) {
            float s, q0;
            meta_from_extrema(lo, hi, maxq, symmetric, s, q0);
            scales[g] = s;
            qzeros[g] = q0;
        }
    }
}

// Groups of exactly 128 elements, every group whole and 16-byte aligned: eight lanes per
// group, 16 consecutive elements per lane as 16-byte loads (two for bf16, four for fp32), so a
// wavefront has 2-4 KB in flight instead of 128 bytes.  Same extrema, hence the same bits.
template <typename T>
__global__ __launch_bounds__(256) void minmax_grid128_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t R, int64_t ldw, int64_t G,
    int64_t n_groups, float maxq, bool symmetric, float* __restrict__ scales,
    float* __restrict__ qzeros) {
    const int sub = threadIdx.x & 7;
    const int64_t g_raw = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 3;
    const int64_t g = g_raw < n_groups ? g_raw : n_groups - 1;   // all lanes take part in the shuffles
    const int64_t b = g / (R * G);
    const int64_t rg = g - b * R * G;
    const int64_t r = rg / G, grp = rg - r * G;
    const T* src = W + b * w_stride + r * ldw + grp * 128 + sub * 16;
    float v[16];
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 w = reinterpret_cast<const float4*>(src)[i];
            v[4 * i + 0] = w.x; v[4 * i + 1] = w.y; v[4 * i + 2] = w.z; v[4 * i + 3] = w.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4 w = reinterpret_cast<const uint4*>(src)[i];
            v[8 * i + 0] = __uint_as_float(w.x << 16); v[8 * i + 1] = __uint_as_float(w.x & 0xffff0000u);
            v[8 * i + 2] = __uint_as_float(w.y << 16); v[8 * i + 3] = __uint_as_float(w.y & 0xffff0000u);
            v[8 * i + 4] = __uint_as_float(w.z << 16); v[8 * i + 5] = __uint_as_float(w.z & 0xffff0000u);
            v[8 * i + 6] = __uint_as_float(w.w << 16); v[8 * i + 7] = __uint_as_float(w.w & 0xffff0000u);
        }
    }
    float lo = 1e30f, hi = -1e30f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        hi = fmaxf(hi, v[i]);
        lo = fminf(lo, v[i]);
    }
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) {
        hi = fmaxf(hi, __shfl_xor(hi, off, 8));
        lo = fminf(lo, __shfl_xor(lo, off, 8));
    }
    if (sub == 0 && g_raw < n_groups) {
        float s, q0;
        meta_from_extrema(lo, hi, maxq, symmetric, s, q0);
        scales[g] = s;
        qzeros[g] = q0;
    }
}

template <typename T>
bool minmax128_ok(const T* W, int64_t w_stride, int64_t C, int64_t ldw, int64_t gs, int64_t n_groups) {
    constexpr int64_t per16 = 16 / sizeof(T);
    return gs == 128 && C % 128 == 0 && ldw % per16 == 0 && w_stride % per16 == 0 &&
           (reinterpret_cast<uintptr_t>(W) % 16) == 0 && n_groups < (1LL << 33);
}

// ---------------------------------------------------------------- shrink search
// |diff|^norm as exp2(norm*log2(.)) on the hardware transcendental units (v_log_f32,
// v_exp_f32: 1 ulp each); mathematically the reference's __expf(__logf(e)*norm).
__device__ __forceinline__ float pow_abs(float e, float norm) {
    return __builtin_amdgcn_exp2f(__builtin_amdgcn_logf(e) * norm);
}

// Loss of one element for one candidate (quant_grid.cu:159-167).  FLOOR = false drops the
// max(|diff|, 1e-20): for norm >= 2.3 the floor's own loss 1e-20^norm is below the smallest
// fp32 denormal, i.e. 0, which is also what |diff| = 0 gives without it (log2 0 = -inf,
// exp2 -inf = 0); the launcher chooses.
template <bool FLOOR, bool REFQ = false>
__device__ __forceinline__ float element_loss(float x, float s, float rcp, float q0, float maxq,
                                              float norm) {
    // q - q0 directly: round(x*rcp) clamped to [-q0, maxq - q0].  q0 is a small integer, so
    // this is the reference's clamp(round(fma(x, rcp, q0)), 0, maxq) - q0 except where the
    // fma's own rounding lands x*rcp + q0 on a half-integer that x*rcp is not; there the two
    // neighbouring levels are equally far from x to within one ulp of the sum.  REFQ is the
    // reference's form itself (one more instruction per weight and candidate).
    const float qc = REFQ ? __builtin_amdgcn_fmed3f(__builtin_rintf(__builtin_fmaf(x, rcp, q0)), 0.0f, maxq) - q0
                          : __builtin_amdgcn_fmed3f(__builtin_rintf(x * rcp), -q0, maxq - q0);
    const float diff = __builtin_fmaf(qc, s, -x);
    return pow_abs(FLOOR ? fmaxf(fabsf(diff), 1e-20f) : fabsf(diff), norm);
}

// Sum over the 8 "reference lanes" l = Q, Q+4, ..., Q+28 (each the in-order sum of its
// GS/32 elements), combined exactly as the reference's halving tree combines them:
// ((p[Q] + p[Q+16]) + (p[Q+8] + p[Q+24])) + ((p[Q+4] + p[Q+20]) + (p[Q+12] + p[Q+28])).
template <int GS, int Q, bool FLOOR, bool REFQ>
__device__ __forceinline__ float quarter_loss(const float (&v)[GS], float s, float rcp, float q0,
                                              float maxq, float norm) {
    constexpr int VPL = GS / 32;
    auto lane_sum = [&](int j) {
        const int l = Q + 4 * j;
        // (the reference starts from 0 and adds: the same value, every term being >= +0)
        float loss = element_loss<FLOOR, REFQ>(v[l], s, rcp, q0, maxq, norm);
#pragma unroll
        for (int i = 1; i < VPL; ++i) loss += element_loss<FLOOR, REFQ>(v[l + 32 * i], s, rcp, q0, maxq, norm);
        return loss;
    };
    // the two halves of the tree one after the other: four lane sums in flight instead of eight
    // (the registers that saves are what lets small kernels of other streams share a SIMD with
    // three wavefronts of this one)
    const float even = (lane_sum(0) + lane_sum(4)) + (lane_sum(2) + lane_sum(6));
    __builtin_amdgcn_sched_barrier(0);
    const float odd = (lane_sum(1) + lane_sum(5)) + (lane_sum(3) + lane_sum(7));
    return even + odd;
}

// Loss of one candidate in the reference's summation order (32 lane sums, then the
// halving tree: total = (Q0 + Q2) + (Q1 + Q3) with Qi the quarter above).  Every term is
// >= 0 and fp32 addition is monotone, so each partial sum is a lower bound of the total:
// once it reaches `bound` for every group of the wavefront the candidate cannot be a new
// strict minimum and the rest of its evaluation is skipped (returns +inf for it).  The
// selected candidate and its loss are exactly those of the full evaluation.
template <int GS, bool FLOOR, bool REFQ>
__device__ __forceinline__ float candidate_loss(const float (&v)[GS], float s, float rcp,
                                                float q0, float maxq, float norm, float bound) {
    constexpr float kInf = __builtin_inff();
    const float a0 = quarter_loss<GS, 0, FLOOR, REFQ>(v, s, rcp, q0, maxq, norm);
    if (__builtin_amdgcn_ballot_w64(a0 < bound) == 0) return kInf;
    const float h0 = a0 + quarter_loss<GS, 2, FLOOR, REFQ>(v, s, rcp, q0, maxq, norm);
    if (__builtin_amdgcn_ballot_w64(h0 < bound) == 0) return kInf;
    const float a1 = quarter_loss<GS, 1, FLOOR, REFQ>(v, s, rcp, q0, maxq, norm);
    if (__builtin_amdgcn_ballot_w64(h0 + a1 < bound) == 0) return kInf;
    const float h1 = a1 + quarter_loss<GS, 3, FLOOR, REFQ>(v, s, rcp, q0, maxq, norm);
    return h0 + h1;
}

// One lane per group.  FUSED: derive (sg, q0g) from the group's own extrema first;
// otherwise read them from scales/qzeros (the reference's two-call protocol).
// SYM: symmetric grids as a compile-time fact: the zero point (maxq + 1) / 2 and what derives
// from it are then the same for every lane and live in scalar registers.
template <typename T, int GS, bool FUSED, bool FLOOR, bool REFQ, bool SYM>
__global__ __launch_bounds__(64) void mse_grid_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t R, int64_t C, int64_t ldw, int64_t G,
    int64_t n_groups, const float* __restrict__ cand, int P, float maxq, float norm,
    bool search, float* __restrict__ scales, float* __restrict__ qzeros) {
    constexpr bool symmetric = SYM;
    // lanes past the end replay the last group (the wavefront votes together below)
    const int64_t g_raw = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t g = g_raw < n_groups ? g_raw : n_groups - 1;
    const int64_t b = g / (R * G);
    const int64_t rg = g - b * R * G;
    const int64_t r = rg / G, grp = rg - r * G;
    const T* src = W + b * w_stride + r * ldw + grp * GS;
    const int64_t valid = (C - grp * GS) < GS ? (C - grp * GS) : GS;

    float v[GS];
    if (valid == GS && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
        constexpr int PER = 16 / sizeof(T);
        const uint4* s4 = reinterpret_cast<const uint4*>(src);
#pragma unroll
        for (int i = 0; i < GS / PER; ++i) {
            const uint4 w = s4[i];
            if constexpr (sizeof(T) == 4) {
                v[4 * i + 0] = __uint_as_float(w.x);
                v[4 * i + 1] = __uint_as_float(w.y);
                v[4 * i + 2] = __uint_as_float(w.z);
                v[4 * i + 3] = __uint_as_float(w.w);
            } else {
                v[8 * i + 0] = __uint_as_float(w.x << 16);
                v[8 * i + 1] = __uint_as_float(w.x & 0xffff0000u);
                v[8 * i + 2] = __uint_as_float(w.y << 16);
                v[8 * i + 3] = __uint_as_float(w.y & 0xffff0000u);
                v[8 * i + 4] = __uint_as_float(w.z << 16);
                v[8 * i + 5] = __uint_as_float(w.z & 0xffff0000u);
                v[8 * i + 6] = __uint_as_float(w.w << 16);
                v[8 * i + 7] = __uint_as_float(w.w & 0xffff0000u);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < GS; ++i) v[i] = (i < valid) ? ld_as_f32(src + i) : 0.0f;
    }

    float sg, q0g;
    float lo = 1e30f, hi = -1e30f;
#pragma unroll
    for (int i = 0; i < GS; ++i) {
        hi = fmaxf(hi, v[i]);
        lo = fminf(lo, v[i]);
    }
    if constexpr (FUSED) {
        meta_from_extrema(lo, hi, maxq, symmetric, sg, q0g);
    } else {
        sg = scales[g];
        q0g = qzeros[g];
    }

    float best_s = sg, best_q = q0g;
    if (search) {
        const float xmin = symmetric ? 0.0f : -(sg * q0g);
        float best_loss = 3.402823466e+38f;
        // The group's extreme values are two of the summands; shrinking the scale clips them
        // first.  A single summand is a lower bound of the (monotone, non-negative) fp32 sum,
        // so once it reaches the best loss for every group of the wavefront the candidate is
        // out without touching the other gs-2 elements.
        //
        // Symmetric grids (the zero point does not move with the candidate) make that test
        // before the candidate's reciprocal is even divided out, on |diff| instead of the loss:
        // `reach` is the |diff| from which one element's loss is certain to reach best_loss
        // (its 1/norm-th power plus a margin of 1e-4 against the few ulp of the log/exp pair;
        // the power is monotone for norm >= 1).  An extreme whose quotient by the approximate
        // reciprocal lies a whole level beyond the clamp is clamped under the exact reciprocal
        // as well (the two quotients differ by a few 1e-6), and then fma(bound, s, -x) IS its
        // diff.  Anything less clear counts as 0, which only means that the candidate is
        // evaluated: the test is an optimisation, candidate_loss decides.
        const bool early = symmetric && norm >= 1.0f;
        const float inv_norm = 1.0f / norm;
        const float top = maxq - q0g, bot = -q0g;
        float reach = 3.402823466e+38f;
        // Both |diff| grow as the scale shrinks and best_loss only changes when a candidate is
        // evaluated: a candidate that is out for the whole wavefront, each lane by an extreme
        // that is clamped with room to spare (1.01 levels: the next, smaller scale keeps it
        // beyond 1), takes every later candidate with a factor no larger out with it.
        bool rest_out = false;
        float out_from = 0.0f;
        for (int p = 0; p < P; ++p) {
            const float factor = cand[p];
            if (rest_out && factor <= out_from) continue;
            const float s = sg * factor;
            if (early) {
                const float approx = __builtin_amdgcn_rcpf(s + kEps);
                const float qh = hi * approx, ql = lo * approx;
                const float over = (qh >= top + 1.0f) ? -__builtin_fmaf(top, s, -hi) : 0.0f;
                const float under = (ql <= bot - 1.0f) ? __builtin_fmaf(bot, s, -lo) : 0.0f;
                if (__builtin_amdgcn_ballot_w64(!(fmaxf(over, under) >= reach)) == 0) {
                    // (a grid handed in with its zero point outside [0, maxq] or a scale below
                    // zero would turn the growth around: never settled)
                    const bool settled = sg > 0.0f && top >= 0.0f && bot <= 0.0f &&
                                         ((qh >= top + 1.01f && over >= reach) ||
                                          (ql <= bot - 1.01f && under >= reach));
                    if (__builtin_amdgcn_ballot_w64(!settled) == 0) {
                        rest_out = true;
                        out_from = factor;
                    }
                    continue;
                }
            }
            const float rcp = 1.0f / (s + kEps);
            const float q0 = symmetric ? q0g : clampf(__builtin_rintf(-xmin * rcp), 0.0f, maxq);
            if (!early) {
                const float clip = fmaxf(element_loss<FLOOR, REFQ>(lo, s, rcp, q0, maxq, norm),
                                         element_loss<FLOOR, REFQ>(hi, s, rcp, q0, maxq, norm));
                if (__builtin_amdgcn_ballot_w64(clip < best_loss) == 0) continue;
            }
            const float loss = candidate_loss<GS, FLOOR, REFQ>(v, s, rcp, q0, maxq, norm, best_loss);
            if (loss < best_loss) {
                best_loss = loss;
                best_s = s;
                best_q = q0;
                // (a loss of exactly 0 cannot be improved on: everything is out; losses down
                // where the log would see a denormal: no early test)
                reach = loss == 0.0f ? 0.0f
                        : loss < 1e-30f ? 3.402823466e+38f
                        : __builtin_amdgcn_exp2f(__builtin_amdgcn_logf(loss) * inv_norm) * 1.0001f;
            }
        }
    }
    if (g_raw < n_groups) {
        scales[g] = best_s;
        qzeros[g] = best_q;
    }
}

template <typename T, bool FUSED>
int launch_mse(const T* W, int64_t w_stride, int64_t R, int64_t C, int64_t ldw, int64_t gs,
               int64_t G, int64_t n_groups, const float* cand, int64_t P, float maxq, float norm,
               bool symmetric, bool search, float* scales, float* qzeros, hipStream_t st) {
    const dim3 block(64), grid((unsigned)forge::ceil_div(n_groups, 64));
    forge::KernelTiming timing(search ? "mse_grid" : "minmax_grid_lane", st,
                               (double)n_groups * (gs * sizeof(T) + 8.0 + (FUSED ? 0.0 : 8.0)),
                               forge::WORK_BYTES);
    const bool floor_needed = !(norm >= 2.3f);
    const bool refq = forge::option(forge::OPT_MSE_REFERENCE_QUANTISER) != 0;
#define FORGE_MSE_LAUNCH(GS, FL, RQ)                                                          \
    if (symmetric)                                                                            \
        mse_grid_kernel<T, GS, FUSED, FL, RQ, true><<<grid, block, 0, st>>>(                  \
            W, w_stride, R, C, ldw, G, n_groups, cand, (int)P, maxq, norm, search, scales, qzeros); \
    else                                                                                      \
        mse_grid_kernel<T, GS, FUSED, FL, RQ, false><<<grid, block, 0, st>>>(                 \
            W, w_stride, R, C, ldw, G, n_groups, cand, (int)P, maxq, norm, search, scales, qzeros)
#define FORGE_MSE_CASE(GS)                                                                    \
    case GS:                                                                                  \
        if (floor_needed && refq) { FORGE_MSE_LAUNCH(GS, true, true); }                       \
        else if (floor_needed) { FORGE_MSE_LAUNCH(GS, true, false); }                         \
        else if (refq) { FORGE_MSE_LAUNCH(GS, false, true); }                                 \
        else { FORGE_MSE_LAUNCH(GS, false, false); }                                          \
        break;
    switch (gs) {
        FORGE_MSE_CASE(32)
        FORGE_MSE_CASE(64)
        FORGE_MSE_CASE(128)
        default:
            return forge::fail(FORGE_ERR_INVALID, "Unsupported group_size=%lld (expected 32/64/128)",
                               (long long)gs);
    }
#undef FORGE_MSE_CASE
#undef FORGE_MSE_LAUNCH
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

int check_bits(int bits) {
    FORGE_REQUIRE(bits >= 1 && bits <= 8, "bits=%d outside 1..8", bits);
    return FORGE_OK;
}

}  // namespace

extern "C" int forge_build_group_meta_packed(const float* X, int64_t RG, int64_t gs, int bits,
                                             int symmetric, float* scales, float* qzeros,
                                             forge_stream_t stream) {
    if (int e = check_bits(bits)) return e;
    FORGE_REQUIRE(RG >= 0 && gs >= 1, "bad shape RG=%lld gs=%lld", (long long)RG, (long long)gs);
    FORGE_REQUIRE(RG == 0 || (X && scales && qzeros), "null pointer");
    if (RG == 0) return FORGE_OK;
    const float maxq = (float)((1 << bits) - 1);
    const int64_t halves_per_block = 8;
    int64_t blocks = forge::ceil_div(RG, halves_per_block);
    if (blocks > (1 << 20)) blocks = 1 << 20;
    forge::KernelTiming timing("minmax_grid", (hipStream_t)stream, (double)RG * (gs * 4.0 + 8.0),
                               forge::WORK_BYTES);
    if (minmax128_ok(X, 0, gs, gs, gs, RG))
        minmax_grid128_kernel<float><<<dim3((unsigned)forge::ceil_div(RG, 32)), dim3(256), 0,
                                       (hipStream_t)stream>>>(X, 0, RG, gs, 1, RG, maxq,
                                                              symmetric != 0, scales, qzeros);
    else
        minmax_grid_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
            X, 0, RG, gs, gs, gs, 1, RG, maxq, symmetric != 0, scales, qzeros);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_mse_scale_groups_packed(const float* X, float* scales, float* qzeros,
                                             const float* candidates, int64_t RG, int64_t gs,
                                             int64_t P, float norm, int bits, int symmetric,
                                             forge_stream_t stream) {
    if (int e = check_bits(bits)) return e;
    FORGE_REQUIRE(gs == 32 || gs == 64 || gs == 128,
                  "Unsupported group_size=%lld (expected 32/64/128)", (long long)gs);
    FORGE_REQUIRE(RG >= 0 && P >= 0 && P < (1 << 30), "bad shape RG=%lld P=%lld", (long long)RG,
                  (long long)P);
    FORGE_REQUIRE(RG == 0 || (X && scales && qzeros && (candidates || P == 0)), "null pointer");
    if (RG == 0) return FORGE_OK;
    const float maxq = (float)((1 << bits) - 1);
    return launch_mse<float, false>(X, 0, RG, gs, gs, gs, 1, RG, candidates, P, maxq, norm,
                                    symmetric != 0, true, scales, qzeros, (hipStream_t)stream);
}

extern "C" int forge_quant_grid(const void* W, int w_dtype, int64_t batch, int64_t w_stride,
                                int64_t R, int64_t C, int64_t ldw, int64_t gs, int bits,
                                int symmetric, int mse, const float* candidates, int64_t P,
                                float norm, float* scales, float* qzeros,
                                forge_stream_t stream) {
    if (int e = check_bits(bits)) return e;
    FORGE_REQUIRE(w_dtype == FORGE_F32 || w_dtype == FORGE_BF16, "w_dtype=%d", w_dtype);
    FORGE_REQUIRE(batch >= 0 && R >= 0 && C >= 1 && ldw >= C && gs >= 1,
                  "bad shape batch=%lld R=%lld C=%lld ldw=%lld gs=%lld", (long long)batch,
                  (long long)R, (long long)C, (long long)ldw, (long long)gs);
    FORGE_REQUIRE(!mse || P == 0 || candidates, "candidates is null");
    const int64_t G = forge::ceil_div(C, gs);
    const int64_t n_groups = batch * R * G;
    if (n_groups == 0) return FORGE_OK;
    FORGE_REQUIRE(W && scales && qzeros, "null pointer");
    const float maxq = (float)((1 << bits) - 1);
    hipStream_t st = (hipStream_t)stream;
    if (mse) {
        FORGE_REQUIRE(gs == 32 || gs == 64 || gs == 128,
                      "Unsupported group_size=%lld (expected 32/64/128)", (long long)gs);
        if (w_dtype == FORGE_F32)
            return launch_mse<float, true>((const float*)W, w_stride, R, C, ldw, gs, G, n_groups,
                                           candidates, P, maxq, norm, symmetric != 0, true, scales,
                                           qzeros, st);
        return launch_mse<__hip_bfloat16, true>((const __hip_bfloat16*)W, w_stride, R, C, ldw, gs,
                                                G, n_groups, candidates, P, maxq, norm,
                                                symmetric != 0, true, scales, qzeros, st);
    }
    int64_t blocks = forge::ceil_div(n_groups, 8);
    if (blocks > (1 << 20)) blocks = 1 << 20;
    forge::KernelTiming timing("minmax_grid", st,
                               (double)batch * R * C * (w_dtype == FORGE_F32 ? 4.0 : 2.0) +
                                   8.0 * n_groups,
                               forge::WORK_BYTES);
    const dim3 grid128((unsigned)forge::ceil_div(n_groups, 32));
    if (w_dtype == FORGE_F32 && minmax128_ok((const float*)W, w_stride, C, ldw, gs, n_groups))
        minmax_grid128_kernel<float><<<grid128, dim3(256), 0, st>>>(
            (const float*)W, w_stride, R, ldw, G, n_groups, maxq, symmetric != 0, scales, qzeros);
    else if (w_dtype == FORGE_BF16 &&
             minmax128_ok((const __hip_bfloat16*)W, w_stride, C, ldw, gs, n_groups))
        minmax_grid128_kernel<__hip_bfloat16><<<grid128, dim3(256), 0, st>>>(
            (const __hip_bfloat16*)W, w_stride, R, ldw, G, n_groups, maxq, symmetric != 0, scales,
            qzeros);
    else if (w_dtype == FORGE_F32)
        minmax_grid_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(
            (const float*)W, w_stride, R, C, ldw, gs, G, n_groups, maxq, symmetric != 0, scales,
            qzeros);
    else
        minmax_grid_kernel<__hip_bfloat16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(
            (const __hip_bfloat16*)W, w_stride, R, C, ldw, gs, G, n_groups, maxq, symmetric != 0,
            scales, qzeros);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
