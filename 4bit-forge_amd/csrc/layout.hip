// Layout changes around the solve: weight -> solver order, codes -> layer order, the
// Hessian's symmetric permutation, and int4 nibble packing.  All HBM-bound byte/float
// movers; each one reads and writes every element once with coalesced rows.
#include "common.h"
#include <hip/hip_bf16.h>

namespace {

constexpr int64_t kPermuteLdsFloats = 16384;   // 64 KB of LDS per workgroup at most

__device__ __forceinline__ float ld_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_as_f32(const __hip_bfloat16* p) {
    return __uint_as_float(static_cast<uint32_t>(*reinterpret_cast<const uint16_t*>(p)) << 16);
}

// Xout[b][perm_inv[c]][r] = W[b][r][c]  (64x64 tiles through LDS; the W.T[perm] of
// forge/gptq.py:133 written as a scatter of whole output rows so that both sides coalesce).
template <typename T>
__global__ __launch_bounds__(256) void to_solver_order_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t ldw, const int64_t* __restrict__ perm_inv,
    const uint8_t* __restrict__ dead, float* __restrict__ Xout, int64_t R, int64_t C) {
    __shared__ float tile[64][65];
    const int64_t b = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const T* __restrict__ Wb = W + b * w_stride;
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        float v = 0.0f;
        if (r < R && c < C && !(dead && dead[b * C + c])) v = ld_as_f32(Wb + r * ldw + c);
        tile[i][tx] = v;
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int64_t c = c0 + j, r = r0 + tx;
        if (c < C && r < R) Xout[b * C * R + perm_inv[b * C + c] * R + r] = tile[tx][j];
    }
}

// qout[b][r][c] = qin[b][perm_inv[c]][r]   (qweight[perm_inv].T of forge/gptq.py:139)
__global__ __launch_bounds__(256) void to_layer_order_kernel(
    const uint8_t* __restrict__ qin, const int64_t* __restrict__ perm_inv,
    uint8_t* __restrict__ qout, int64_t R, int64_t C) {
    __shared__ uint8_t tile[64][65];
    const int64_t b = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int j = ty; j < 64; j += 4) {
        const int64_t c = c0 + j, r = r0 + tx;
        tile[j][tx] = (c < C && r < R) ? qin[b * C * R + perm_inv[b * C + c] * R + r] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        if (r < R && c < C) qout[b * R * C + r * C + c] = tile[tx][i];
    }
}

// Hp[b][i][j] = H[b][perm[i]][perm[j]], dead rows/columns zeroed with a unit diagonal
// (forge/gptq.py:100-103,117,145-149).  One workgroup per output row: the source row is
// streamed into LDS with coalesced loads, gathered from there in permuted order and
// written out coalesced, so HBM sees one sequential read and one sequential write.
__global__ __launch_bounds__(256) void hessian_permute_kernel(
    const float* __restrict__ H, const int64_t* __restrict__ perm, const uint8_t* __restrict__ dead,
    float* __restrict__ Hp, int64_t C) {
    extern __shared__ float srow[];                 // C floats, or nothing when C is too large
    const int64_t b = blockIdx.y, i = blockIdx.x;
    const int64_t* __restrict__ pb = perm + b * C;
    const uint8_t* __restrict__ db = dead ? dead + b * C : nullptr;
    const float* __restrict__ src = H + b * C * C + pb[i] * C;
    float* __restrict__ dst = Hp + b * C * C + i * C;
    const bool dead_i = db && db[i];
    const bool staged = C <= kPermuteLdsFloats;
    if (staged) {
        for (int64_t j = threadIdx.x; j < C; j += blockDim.x) srow[j] = src[j];
        __syncthreads();
    }
    for (int64_t j = threadIdx.x; j < C; j += blockDim.x) {
        float v = staged ? srow[pb[j]] : src[pb[j]];
        if (dead_i || (db && db[j])) v = (i == j) ? 1.0f : 0.0f;
        dst[j] = v;
    }
}

// damp[b] = rel_damp * mean(diag(Hp[b]))   (forge/gptq.py:152-153); fixed-order tree sum.
__global__ __launch_bounds__(256) void damp_kernel(const float* __restrict__ Hp,
                                                   float* __restrict__ damp, float rel_damp,
                                                   int64_t C) {
    __shared__ float part[256];
    const int64_t b = blockIdx.x;
    float s = 0.0f;
    for (int64_t i = threadIdx.x; i < C; i += 256) s += Hp[b * C * C + i * C + i];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) part[threadIdx.x] += part[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) damp[b] = rel_damp * (part[0] / (float)C);
}

// Eight zero-shifted codes per int32, lowest nibble first, offset binary (+8).
__global__ __launch_bounds__(256) void pack_int4_kernel(const uint8_t* __restrict__ codes,
                                                        const float* __restrict__ qzeros,
                                                        int32_t* __restrict__ packed, int64_t R,
                                                        int64_t C, int64_t gs, int64_t G) {
    const int64_t W8 = (C + 7) / 8;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= R * W8) return;
    const int64_t r = idx / W8, w = idx - r * W8;
    uint32_t word = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int64_t c = w * 8 + k;
        if (c < C) {
            const int z = qzeros ? (int)qzeros[r * G + c / gs] : 8;
            const int v = (int)codes[r * C + c] - z + 8;
            word |= (uint32_t)(v & 0xF) << (4 * k);
        }
    }
    packed[idx] = (int32_t)word;
}

}  // namespace

extern "C" int forge_weight_to_solver_order(const void* W, int w_dtype, int64_t w_stride,
                                            int64_t ldw, const int64_t* perm_inv,
                                            const uint8_t* dead, float* Xout, int64_t batch,
                                            int64_t R, int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(w_dtype == FORGE_F32 || w_dtype == FORGE_BF16, "w_dtype=%d", w_dtype);
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && R >= 0 && C >= 0 && ldw >= C, "bad shape");
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(W && perm_inv && Xout, "null pointer");
    dim3 grid((unsigned)forge::ceil_div(C, 64), (unsigned)forge::ceil_div(R, 64), (unsigned)batch);
    FORGE_REQUIRE(grid.y < 65536, "R too large");
    forge::KernelTiming timing("weight_to_solver_order", (hipStream_t)stream,
                               (double)batch * R * C * (4.0 + (w_dtype == FORGE_F32 ? 4.0 : 2.0)),
                               forge::WORK_BYTES);
    if (w_dtype == FORGE_F32)
        to_solver_order_kernel<float><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            (const float*)W, w_stride, ldw, perm_inv, dead, Xout, R, C);
    else
        to_solver_order_kernel<__hip_bfloat16><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            (const __hip_bfloat16*)W, w_stride, ldw, perm_inv, dead, Xout, R, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_codes_to_layer_order(const uint8_t* qin, const int64_t* perm_inv,
                                          uint8_t* qout, int64_t batch, int64_t R, int64_t C,
                                          forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && R >= 0 && C >= 0, "bad shape");
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(qin && perm_inv && qout, "null pointer");
    dim3 grid((unsigned)forge::ceil_div(C, 64), (unsigned)forge::ceil_div(R, 64), (unsigned)batch);
    FORGE_REQUIRE(grid.y < 65536, "R too large");
    forge::KernelTiming timing("codes_to_layer_order", (hipStream_t)stream, 2.0 * batch * R * C,
                               forge::WORK_BYTES);
    to_layer_order_kernel<<<grid, dim3(256), 0, (hipStream_t)stream>>>(qin, perm_inv, qout, R, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_hessian_permute(const float* H, const int64_t* perm, const uint8_t* dead,
                                     float* Hp, float* damp, float rel_damp, int64_t batch,
                                     int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1, "bad shape");
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(H && perm && Hp && damp, "null pointer");
    FORGE_REQUIRE(H != Hp, "hessian_permute cannot run in place");
    hipStream_t st = (hipStream_t)stream;
    forge::KernelTiming timing("hessian_permute", st, 8.0 * C * C * (double)batch, forge::WORK_BYTES);
    const size_t lds = C <= kPermuteLdsFloats ? (size_t)C * sizeof(float) : 0;
    hessian_permute_kernel<<<dim3((unsigned)C, (unsigned)batch), dim3(256), lds, st>>>(H, perm, dead,
                                                                                     Hp, C);
    FORGE_LAUNCH_CHECK();
    damp_kernel<<<dim3((unsigned)batch), dim3(256), 0, st>>>(Hp, damp, rel_damp, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_pack_int4(const uint8_t* codes, const float* qzeros, int32_t* packed,
                               int64_t R, int64_t C, int64_t gs, forge_stream_t stream) {
    FORGE_REQUIRE(R >= 0 && C >= 0 && gs >= 1, "bad shape");
    if (R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(codes && packed, "null pointer");
    const int64_t n = R * ((C + 7) / 8);
    forge::KernelTiming timing("pack_int4", (hipStream_t)stream,
                               1.5 * R * C + 4.0 * R * forge::ceil_div(C, gs), forge::WORK_BYTES);
    pack_int4_kernel<<<dim3((unsigned)forge::ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream>>>(
        codes, qzeros, packed, R, C, gs, forge::ceil_div(C, gs));
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
