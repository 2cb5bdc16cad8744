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
#include "common.h"
#include <hip/hip_bf16.h>
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

// Write one 32x32 accumulator tile (and its mirror image) with out = alpha*acc + beta*H.
// Called by all four wavefronts of the workgroup together (it synchronises them).
__device__ __forceinline__ void store_tile(float* __restrict__ H, int64_t C, int row0, int col0,
                                           const f32x16& acc, float alpha, float beta, bool mirror,
                                           float (*tbuf)[33], int lane) {
    f32x16 out;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int i = row0 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        const int j = col0 + (lane & 31);
        float o = alpha * acc[v];
        if (i < C && j < C) {
            if (beta != 0.0f) o = __builtin_fmaf(beta, H[(int64_t)i * C + j], o);
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
                                                        int NT) {
    __shared__ float tbuf[4][32][33];
    const GroupDesc g = gd[blockIdx.y];
    if (g.n == 0) return;
    int ti, tj;
    tile_pair(blockIdx.x, NT, ti, tj);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    float* __restrict__ H = Hall + (int64_t)blockIdx.y * C * C;
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
                           tbuf[wave], lane);
    }
}

// ---------------------------------------------------------------- rank-k (f32 MFMA)
// Same tiling; operands are the token rows themselves (K-major), staged through LDS.
constexpr int TK = 16;
__global__ __launch_bounds__(256) void syrk_f32_kernel(const float* __restrict__ X, int64_t ldx,
                                                       const GroupDesc* __restrict__ gd,
                                                       float* __restrict__ Hall, int64_t C, int NT) {
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

    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.0f;

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
    }
    const bool mirror = ti != tj;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
            store_tile(H, C, mt + wm * 64 + mi * 32, nt + wn * 64 + ni * 32, acc[mi][ni], g.alpha,
                       g.beta, mirror, tbuf[wave], lane);
}

int64_t pack_units(int64_t n, int64_t C) {  // 16-byte units for one group
    return forge::ceil_div(n, 16) * forge::ceil_div(C, 32) * 64;
}

}  // namespace

extern "C" int64_t forge_hessian_workspace_bytes(int64_t total_rows, int64_t n_groups, int64_t C,
                                                 int x_dtype) {
    if (n_groups <= 0 || C <= 0) return 0;
    int64_t bytes = n_groups * (int64_t)sizeof(GroupDesc) + 256;
    if (x_dtype == FORGE_BF16) bytes += pack_units(total_rows + 16 * n_groups, C) * 16;
    return bytes;
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
    const int64_t total = offsets_host[n_groups] - offsets_host[0];
    FORGE_REQUIRE(total >= 0, "offsets must be non-decreasing");
    FORGE_REQUIRE(total == 0 || X, "X is null");
    FORGE_REQUIRE(ws_bytes >= forge_hessian_workspace_bytes(total, n_groups, C, x_dtype),
                  "workspace too small");
    hipStream_t st = (hipStream_t)stream;

    std::vector<GroupDesc> gd((size_t)n_groups);
    int64_t off = 0;
    int max_chunks = 0;
    bool any = false;
    for (int64_t e = 0; e < n_groups; ++e) {
        const int64_t n = offsets_host[e + 1] - offsets_host[e];
        FORGE_REQUIRE(n >= 0 && n < (1LL << 31), "offsets must be non-decreasing");
        gd[e].row0 = offsets_host[e];
        gd[e].n = (int32_t)n;
        gd[e].nchunk = (int32_t)forge::ceil_div(n, 16);
        gd[e].pack_off = off;
        gd[e].alpha = alpha_host[e];
        gd[e].beta = beta_host[e];
        off += pack_units(n, C);
        if (gd[e].nchunk > max_chunks) max_chunks = gd[e].nchunk;
        any |= n > 0;
    }
    if (!any) return FORGE_OK;
    GroupDesc* gd_dev = (GroupDesc*)ws;
    const int64_t desc_bytes = ((n_groups * (int64_t)sizeof(GroupDesc) + 255) / 256) * 256;
    FORGE_HIP_CHECK(hipMemcpyAsync(gd_dev, gd.data(), n_groups * sizeof(GroupDesc),
                                   hipMemcpyHostToDevice, st));
    // the host vector dies with this call: make sure the copy has been consumed
    FORGE_HIP_CHECK(hipStreamSynchronize(st));

    const int NT = (int)forge::ceil_div(C, 128);
    const unsigned pairs = (unsigned)(NT * (NT + 1) / 2);
    if (x_dtype == FORGE_BF16) {
        uint4* pack = (uint4*)((char*)ws + desc_bytes);
        const unsigned ychunks = (unsigned)(max_chunks < 64 ? max_chunks : 64);
        pack_bf16_kernel<<<dim3((unsigned)forge::ceil_div(C, 32), ychunks, (unsigned)n_groups),
                           dim3(64), 0, st>>>((const uint16_t*)X, ldx, C, gd_dev, pack);
        FORGE_LAUNCH_CHECK();
        // executed flops: tiles on and above the diagonal only
        forge::KernelTiming timing("hessian_syrk_bf16", st,
                                   2.0 * (double)total * 128.0 * 128.0 * (double)pairs,
                                   forge::WORK_FLOPS);
        bool any_blend = false;
        for (int e = 0; e < n_groups; ++e) any_blend = any_blend || beta_host[e] != 0.0f;
        if (any_blend)
            syrk_bf16_kernel<true><<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(pack, gd_dev,
                                                                                         H, C, NT);
        else
            syrk_bf16_kernel<false><<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(pack, gd_dev,
                                                                                          H, C, NT);
        FORGE_LAUNCH_CHECK();
    } else {
        forge::KernelTiming timing("hessian_syrk_f32", st,
                                   2.0 * (double)total * 128.0 * 128.0 * (double)pairs,
                                   forge::WORK_FLOPS);
        syrk_f32_kernel<<<dim3(pairs, (unsigned)n_groups), dim3(256), 0, st>>>(
            (const float*)X, ldx, gd_dev, H, C, NT);
        FORGE_LAUNCH_CHECK();
    }
    return FORGE_OK;
}
