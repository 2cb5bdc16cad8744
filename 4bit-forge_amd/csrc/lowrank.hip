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
// Two kernels, both for n <= 16 (rows beyond n are zero rows of B):
//   lowrank_factor_kernel   one wavefront per matrix walks k = C-1 .. 0 and writes h_k.
//   lowrank_sweep_kernel    one lane per output row walks k = 0 .. C-1: dot, quantise, update.
#include "common.h"

namespace {

constexpr int NR = 16;            // rows of B the kernels are written for
constexpr float kEps = 1e-12f;    // the quantiser's epsilon (solver.cu:12)

__device__ __forceinline__ double readlane_f64(double v, int lane) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}

// Lane i < 16 holds row i of S in float64 (lanes 16..63 repeat lanes 0..15: every value that
// crosses lanes is read from the first sixteen).  b_k and D_k are the same for every lane, one
// column ahead of their use in registers.
__global__ __launch_bounds__(64) void lowrank_factor_kernel(const float* __restrict__ Bp,
                                                            const float* __restrict__ D,
                                                            float* __restrict__ Hm,
                                                            int32_t* __restrict__ info, int64_t C) {
    const int row = threadIdx.x & (NR - 1);
    const int64_t b = blockIdx.x;
    const float4* __restrict__ Bb = reinterpret_cast<const float4*>(Bp + b * C * NR);
    const float* __restrict__ Db = D + b * C;
    float* __restrict__ Hb = Hm + b * C * NR;

    double S[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) S[j] = (j == row) ? 1.0 : 0.0;
    bool bad = false;

    float4 nb[NR / 4];
#pragma unroll
    for (int j = 0; j < NR / 4; ++j) nb[j] = Bb[(C - 1) * (NR / 4) + j];
    float nd = Db[C - 1];
    for (int64_t k = C - 1; k >= 0; --k) {
        double bd[NR];
#pragma unroll
        for (int j = 0; j < NR / 4; ++j) {
            bd[4 * j + 0] = (double)nb[j].x;
            bd[4 * j + 1] = (double)nb[j].y;
            bd[4 * j + 2] = (double)nb[j].z;
            bd[4 * j + 3] = (double)nb[j].w;
        }
        const double dk = (double)nd;
        if (k > 0) {
#pragma unroll
            for (int j = 0; j < NR / 4; ++j) nb[j] = Bb[(k - 1) * (NR / 4) + j];
            nd = Db[k - 1];
        }
        // s_row = S[row, :] . b   (four chains of four)
        double c0 = 0.0, c1 = 0.0, c2 = 0.0, c3 = 0.0;
#pragma unroll
        for (int j = 0; j < NR; j += 4) {
            c0 = __builtin_fma(S[j + 0], bd[j + 0], c0);
            c1 = __builtin_fma(S[j + 1], bd[j + 1], c1);
            c2 = __builtin_fma(S[j + 2], bd[j + 2], c2);
            c3 = __builtin_fma(S[j + 3], bd[j + 3], c3);
        }
        const double s = (c0 + c1) + (c2 + c3);
        double sj[NR];
#pragma unroll
        for (int j = 0; j < NR; ++j) sj[j] = readlane_f64(s, j);
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
        if (threadIdx.x < NR) Hb[k * NR + row] = (float)h;
#pragma unroll
        for (int j = 0; j < NR; ++j) S[j] = __builtin_fma(-h, sj[j], S[j]);
    }
    if (threadIdx.x == 0) info[b] = bad ? 1 : 0;
}

__device__ __forceinline__ float w0_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float w0_as_f32(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }

// One lane per output row, 256 rows per workgroup.  h_k and b_k are the same for every lane:
// the workgroup stages TK columns of both in LDS (one float4 per thread and tile) and every
// multiply-add takes them from broadcast reads.  The row's weights, scales and zero points of
// the next tile are requested while the current tile's chain runs.  Quantiser as in
// solver.cu:9-23: q = clamp(rint(fma(x, 1/(s+eps), z)), 0, maxq), deq = fma(q, s, -(z s)).
template <typename W0T>
__global__ __launch_bounds__(256) void lowrank_sweep_kernel(
    const W0T* __restrict__ W0, const float* __restrict__ Bp, const float* __restrict__ Hm,
    const float* __restrict__ scT, const float* __restrict__ qzT, const int32_t* __restrict__ g_idx,
    const int32_t* __restrict__ info, uint8_t* __restrict__ q, int64_t C, int64_t R, int64_t G,
    float maxq) {
    constexpr int TK = 16;
    __shared__ float4 Ts[2][2][TK][NR / 4];       // [buffer][0 = h, 1 = b][column][quarter]
    const int64_t b = blockIdx.y;
    const int64_t r_raw = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = r_raw < R;
    const int64_t r = live ? r_raw : R - 1;        // idle lanes replay the last row, store nothing
    const W0T* __restrict__ w0 = W0 + b * C * R + r;
    const float* __restrict__ sc = scT + b * G * R + r;
    const float* __restrict__ qz = qzT + b * G * R + r;
    const int32_t* __restrict__ gi = g_idx + b * C;
    uint8_t* __restrict__ qo = q + b * C * R + r;
    // a failed factorisation sweeps with the identity (gptq.py:172-175): no coupling at all
    const bool coupled = info[b] == 0;
    // thread t < 64 carries one float4 of the h tile, 64 <= t < 128 one of the b tile
    const int which = threadIdx.x >> 6, slot = threadIdx.x & 63;
    const float4* __restrict__ src =
        reinterpret_cast<const float4*>((which ? Bp : Hm) + b * C * NR) + slot;
    const bool stager = threadIdx.x < 128;

    float a[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) a[j] = 0.0f;

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
    if (stager) {
        const float4 v = src[0];
        Ts[0][which][slot >> 2][slot & 3] = coupled ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();

    int buf = 0;
    for (int64_t k0 = 0; k0 < C; k0 += TK) {
        const bool more = k0 + TK < C;
        float nw[TK], ns[TK], nz[TK];
        float4 stage = make_float4(0.f, 0.f, 0.f, 0.f);
        if (more) {
            load_meta(k0 + TK, nw, ns, nz);
            if (stager && coupled) stage = src[(k0 + TK) * (NR / 4)];
        }
#pragma unroll
        for (int t = 0; t < TK; ++t) rv[t] = 1.0f / (sv[t] + kEps);
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            float h[NR], bb[NR];
#pragma unroll
            for (int j = 0; j < NR / 4; ++j) {
                const float4 v = Ts[buf][0][t][j];
                h[4 * j + 0] = v.x; h[4 * j + 1] = v.y; h[4 * j + 2] = v.z; h[4 * j + 3] = v.w;
            }
            float c0 = wv[t], c1 = 0.0f, c2 = 0.0f, c3 = 0.0f;
#pragma unroll
            for (int j = 0; j < NR; j += 4) {
                c0 = __builtin_fmaf(a[j + 0], h[j + 0], c0);
                c1 = __builtin_fmaf(a[j + 1], h[j + 1], c1);
                c2 = __builtin_fmaf(a[j + 2], h[j + 2], c2);
                c3 = __builtin_fmaf(a[j + 3], h[j + 3], c3);
            }
            const float x = (c0 + c1) + (c2 + c3);
            const float qf = __builtin_amdgcn_fmed3f(
                __builtin_rintf(__builtin_fmaf(x, rv[t], zv[t])), 0.0f, maxq);
            const float deq = __builtin_fmaf(qf, sv[t], -(zv[t] * sv[t]));
            const float d = wv[t] - deq;
            if (live) qo[(k0 + t) * R] = (uint8_t)qf;
#pragma unroll
            for (int j = 0; j < NR / 4; ++j) {
                const float4 v = Ts[buf][1][t][j];
                bb[4 * j + 0] = v.x; bb[4 * j + 1] = v.y; bb[4 * j + 2] = v.z; bb[4 * j + 3] = v.w;
            }
#pragma unroll
            for (int j = 0; j < NR; ++j) a[j] = __builtin_fmaf(d, bb[j], a[j]);
        }
        if (more) {
            if (stager) Ts[buf ^ 1][which][slot >> 2][slot & 3] = stage;
#pragma unroll
            for (int t = 0; t < TK; ++t) { wv[t] = nw[t]; sv[t] = ns[t]; zv[t] = nz[t]; }
        }
        __syncthreads();
        buf ^= 1;
    }
}

}  // namespace

extern "C" int forge_lowrank_factor(const float* Bp, const float* D, float* Hm, int32_t* info,
                                    int64_t batch, int64_t C, int64_t n, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1 && C < (1LL << 30), "bad shape batch=%lld C=%lld",
                  (long long)batch, (long long)C);
    FORGE_REQUIRE(n == NR, "n=%lld: the kernels are written for %d rows (pad with zero rows)",
                  (long long)n, NR);
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(Bp && D && Hm && info, "null pointer");
    FORGE_REQUIRE((reinterpret_cast<uintptr_t>(Bp) & 15u) == 0, "Bp must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    // per column: two n x n products and the dot
    forge::KernelTiming timing("lowrank_factor", st, (4.0 * NR * NR + 2.0 * NR) * C * (double)batch,
                               forge::WORK_FLOPS);
    lowrank_factor_kernel<<<dim3((unsigned)batch), dim3(64), 0, st>>>(Bp, D, Hm, info, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_gptq_sweep_lowrank(const void* W0, int w0_dtype, const float* Bp, const float* Hm,
                                        const int32_t* info, const float* scalesT,
                                        const float* qzerosT, const int32_t* g_idx, uint8_t* qweight,
                                        int64_t batch, int64_t C, int64_t R, int64_t G, int bits,
                                        int64_t n, forge_stream_t stream) {
    FORGE_REQUIRE(w0_dtype == FORGE_F32 || w0_dtype == FORGE_BF16, "w0_dtype=%d", w0_dtype);
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 0 && R >= 0 && G >= 1 && C < (1LL << 30) &&
                      R < (1LL << 30),
                  "bad shape batch=%lld C=%lld R=%lld G=%lld", (long long)batch, (long long)C,
                  (long long)R, (long long)G);
    FORGE_REQUIRE(bits >= 1 && bits <= 8, "bits=%d", bits);
    FORGE_REQUIRE(n == NR, "n=%lld: the kernels are written for %d rows (pad with zero rows)",
                  (long long)n, NR);
    FORGE_REQUIRE(C % 16 == 0, "C=%lld must be a multiple of 16", (long long)C);
    if (batch == 0 || C == 0 || R == 0) return FORGE_OK;
    FORGE_REQUIRE(W0 && Bp && Hm && info && scalesT && qzerosT && g_idx && qweight, "null pointer");
    FORGE_REQUIRE(((reinterpret_cast<uintptr_t>(Bp) | reinterpret_cast<uintptr_t>(Hm)) & 15u) == 0,
                  "Bp and Hm must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)forge::ceil_div(R, 256), (unsigned)batch), block(256);
    const float maxq = (float)((1 << bits) - 1);
    forge::KernelTiming timing("lowrank_sweep", st, 4.0 * NR * C * (double)R * (double)batch,
                               forge::WORK_FLOPS);
    if (w0_dtype == FORGE_BF16)
        lowrank_sweep_kernel<uint16_t><<<grid, block, 0, st>>>((const uint16_t*)W0, Bp, Hm, scalesT,
                                                               qzerosT, g_idx, info, qweight, C, R, G,
                                                               maxq);
    else
        lowrank_sweep_kernel<float><<<grid, block, 0, st>>>((const float*)W0, Bp, Hm, scalesT, qzerosT,
                                                            g_idx, info, qweight, C, R, G, maxq);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
