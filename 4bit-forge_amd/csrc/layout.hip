// Layout changes around the solve: weight -> solver order, codes -> layer order, the
// Hessian's symmetric permutation, and int4 nibble packing.  All HBM-bound byte/float
// movers; each one reads and writes every element once with coalesced rows.
#include "common.h"
#include <hip/hip_bf16.h>

namespace {

constexpr int64_t kPermuteLdsFloats = 16384;   // 64 KB of LDS per workgroup at most

// First statement of the movers that are meant to run BESIDE the scale search (another stream's
// kernel that saturates the vector ALU with three wavefronts of 160 registers per SIMD).  Measured
// on gfx950: a kernel gets onto such a SIMD when its wavefronts need no more than the 32 registers
// left (16 for two of them), and it makes progress there only when it asks the instruction
// arbiter for precedence: the older wavefronts of the scale search are ready in nearly every cycle
// (layout pass beside the search: 14.6 ms one after the other, 14.0 ms together without the
// priority, 9.5 ms with it, 7.6 ms being the search alone).
__device__ __forceinline__ void run_beside_the_search() { __builtin_amdgcn_s_setprio(3); }

__device__ __forceinline__ float ld_as_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_as_f32(const __hip_bfloat16* p) {
    return __uint_as_float(static_cast<uint32_t>(*reinterpret_cast<const uint16_t*>(p)) << 16);
}

__device__ __forceinline__ void st_from_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void st_from_f32(__hip_bfloat16* p, float v) {   // v is a bf16 value
    *reinterpret_cast<uint16_t*>(p) = (uint16_t)(__float_as_uint(v) >> 16);
}

// Xout[b][perm_inv[c]][r] = W[b][r][c]  (64x64 tiles through LDS; the W.T[perm] of
// forge/gptq.py:133 written as a scatter of whole output rows so that both sides coalesce).
// W0out (may be null): the same matrix once more in the weights' own type, the untouched copy
// that the displacement-form sweep reads beside the values it updates.
template <typename T>
__global__ __launch_bounds__(256) void to_solver_order_kernel(
    const T* __restrict__ W, int64_t w_stride, int64_t ldw, const int64_t* __restrict__ perm_inv,
    const uint8_t* __restrict__ dead, float* __restrict__ Xout, T* __restrict__ W0out, int64_t R,
    int64_t C, int64_t ldo, int64_t o_stride, const int64_t* __restrict__ index) {
    __shared__ float tile[64][65];
    const int64_t b = blockIdx.z, sb = index ? index[b] : b;    // output slot, source slot
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const T* __restrict__ Wb = W + sb * w_stride;
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        float v = 0.0f;
        if (r < R && c < C && !(dead && dead[sb * C + c])) v = ld_as_f32(Wb + r * ldw + c);
        tile[i][tx] = v;
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int64_t c = c0 + j, r = r0 + tx;
        if (c < C && r < R) {
            const int64_t at = b * o_stride + perm_inv[sb * C + c] * ldo + r;
            if (Xout) Xout[at] = tile[tx][j];
            if (W0out) st_from_f32(W0out + at, tile[tx][j]);
        }
    }
}

// qout[b][r][c] = qin[b][perm_inv[c]][r]   (qweight[perm_inv].T of forge/gptq.py:139)
__global__ __launch_bounds__(256) void to_layer_order_kernel(
    const uint8_t* __restrict__ qin, const int64_t* __restrict__ perm_inv,
    uint8_t* __restrict__ qout, int64_t R, int64_t C, int64_t ldi, int64_t i_stride,
    const int64_t* __restrict__ index) {
    __shared__ uint8_t tile[64][65];
    const int64_t b = blockIdx.z, sb = index ? index[b] : b;    // input slot, destination slot
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int j = ty; j < 64; j += 4) {
        const int64_t c = c0 + j, r = r0 + tx;
        tile[j][tx] = (c < C && r < R) ? qin[b * i_stride + perm_inv[sb * C + c] * ldi + r] : 0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        if (r < R && c < C) qout[sb * R * C + r * C + c] = tile[tx][i];
    }
}

// Fast forms of the two transposes for the shapes the batched solve uses (bf16 weights,
// R % 256 == 0, C % 64 == 0 resp. C % 128 == 0).  Tiles are 256 rows of R tall so that a
// wavefront moves whole 128..1024-byte runs on both sides, with 4..16 bytes per lane.

// 64 (c) x 256 (r) tile, bf16 in, f32 out.  LDS holds the tile as [c][r] 16-bit words.
template <bool DEAD, bool XOUT>
__global__ __launch_bounds__(256) void to_solver_order_bf16_kernel(
    const uint16_t* __restrict__ W, int64_t w_stride, int64_t ldw,
    const int64_t* __restrict__ perm_inv, const uint8_t* __restrict__ dead,
    float* __restrict__ Xout, uint16_t* __restrict__ W0out, int64_t R, int64_t C, int64_t ldo,
    int64_t o_stride, const int64_t* __restrict__ index) {
    constexpr int TC = 64, TR = 256, PITCH = TR + 4;     // rows stay 8-byte aligned
    // (LDS asked for at launch, not declared: for a kernel whose declared LDS limits its
    // occupancy the compiler raises the register count in the kernel descriptor to what that
    // occupancy allows -- 97 for 33 KB -- and the wavefronts no longer fit beside the search's)
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint16_t (*tile)[PITCH] = reinterpret_cast<uint16_t (*)[PITCH]>(lds_raw);
    run_beside_the_search();
    const int64_t b = blockIdx.z, sb = index ? index[b] : b;
    const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
    const int tid = threadIdx.x;
    const uint16_t* __restrict__ Wb = W + sb * w_stride;
    {   // 16 lanes x 8 bytes cover one 128-byte row piece.  A lane takes a block of 4 rows x 4
        // columns, transposes it in registers and stores four rows of r into LDS, 8 bytes each.
        // (Two passes in flight, and two output rows at a time below: 26 registers, which fit
        // into the 32 that three wavefronts of the scale search leave free on a SIMD; all four
        // passes in flight need 48 and gain 4 % alone.  Two rows x four columns per lane -- 16
        // registers, two wavefronts beside the search -- moved 22 % less alone and gained nothing
        // beside it.)
        const int rb = tid >> 4, c4 = (tid & 15) * 4;
        uint32_t keep = 0xF;
        if constexpr (DEAD) {
            const uint8_t* d = dead + sb * C + c0 + c4;
            keep = (d[0] ? 0u : 1u) | (d[1] ? 0u : 2u) | (d[2] ? 0u : 4u) | (d[3] ? 0u : 8u);
        }
#pragma unroll 2
        for (int p = 0; p < TR / 64; ++p) {
            const int r = 4 * (16 * p + rb);
            const uint16_t* src = Wb + (r0 + r) * ldw + c0 + c4;
            const uint2 v0 = *reinterpret_cast<const uint2*>(src);
            const uint2 v1 = *reinterpret_cast<const uint2*>(src + ldw);
            const uint2 v2 = *reinterpret_cast<const uint2*>(src + 2 * ldw);
            const uint2 v3 = *reinterpret_cast<const uint2*>(src + 3 * ldw);
            // perm(hi, lo, sel): result byte i = byte sel[i] of {hi, lo} (0..3 = lo, 4..7 = hi)
            uint2 o0 = make_uint2(__builtin_amdgcn_perm(v1.x, v0.x, 0x05040100u),    // column c4
                                  __builtin_amdgcn_perm(v3.x, v2.x, 0x05040100u));
            uint2 o1 = make_uint2(__builtin_amdgcn_perm(v1.x, v0.x, 0x07060302u),    // c4 + 1
                                  __builtin_amdgcn_perm(v3.x, v2.x, 0x07060302u));
            uint2 o2 = make_uint2(__builtin_amdgcn_perm(v1.y, v0.y, 0x05040100u),    // c4 + 2
                                  __builtin_amdgcn_perm(v3.y, v2.y, 0x05040100u));
            uint2 o3 = make_uint2(__builtin_amdgcn_perm(v1.y, v0.y, 0x07060302u),    // c4 + 3
                                  __builtin_amdgcn_perm(v3.y, v2.y, 0x07060302u));
            if constexpr (DEAD) {
                if (!(keep & 1u)) o0 = make_uint2(0u, 0u);
                if (!(keep & 2u)) o1 = make_uint2(0u, 0u);
                if (!(keep & 4u)) o2 = make_uint2(0u, 0u);
                if (!(keep & 8u)) o3 = make_uint2(0u, 0u);
            }
            *reinterpret_cast<uint2*>(&tile[c4 + 0][r]) = o0;
            *reinterpret_cast<uint2*>(&tile[c4 + 1][r]) = o1;
            *reinterpret_cast<uint2*>(&tile[c4 + 2][r]) = o2;
            *reinterpret_cast<uint2*>(&tile[c4 + 3][r]) = o3;
        }
    }
    __syncthreads();
    {   // a wavefront writes the 256 floats (1 KiB) of one output row per instruction
        const int cw = tid >> 6, r4 = (tid & 63) * 4;
#pragma unroll 2
        for (int cc = 0; cc < TC; cc += 4) {
            const int c = cc + cw;
            const uint2 v = *reinterpret_cast<const uint2*>(&tile[c][r4]);
            const int64_t at = b * o_stride + perm_inv[sb * C + c0 + c] * ldo + r0 + r4;
            if (W0out) *reinterpret_cast<uint2*>(W0out + at) = v;
            if constexpr (XOUT)
                *reinterpret_cast<float4*>(Xout + at) =
                    make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xFFFF0000u),
                                __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xFFFF0000u));
        }
    }
}

// 128 (c) x 256 (r) byte tile.  LDS holds it as [c][r]; each lane takes a 4 x 4 byte block out
// of it (four words, one per source row), transposes it in registers with byte permutes and
// stores one word into each of four rows of the result.
__global__ __launch_bounds__(256) void to_layer_order_fast_kernel(
    const uint8_t* __restrict__ qin, const int64_t* __restrict__ perm_inv,
    uint8_t* __restrict__ qout, int64_t R, int64_t C, int64_t ldi, int64_t i_stride,
    const int64_t* __restrict__ index) {
    constexpr int TC = 128, TR = 256, PITCH = TR + 4;    // 65 words per row: odd
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];   // (at launch: see above)
    uint8_t (*tile)[PITCH] = reinterpret_cast<uint8_t (*)[PITCH]>(lds_raw);
    run_beside_the_search();
    const int64_t b = blockIdx.z, sb = index ? index[b] : b;
    const int64_t r0 = (int64_t)blockIdx.y * TR, c0 = (int64_t)blockIdx.x * TC;
    const int tid = threadIdx.x;
    {   // 16 lanes x 16 bytes read the 256 bytes of one source row; four loads of a lane are in
        // flight before the first is stored (eight would put the kernel beyond 32 registers)
        const int cw = tid >> 4, r16 = (tid & 15) * 16;
#pragma unroll 1
        for (int h = 0; h < TC / 64; ++h) {
            uint4 v[4];
#pragma unroll
            for (int p = 0; p < 4; ++p)
                v[p] = *reinterpret_cast<const uint4*>(
                    qin + b * i_stride + perm_inv[sb * C + c0 + 64 * h + 16 * p + cw] * ldi + r0 + r16);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[64 * h + 16 * p + cw][r16]);   // rows are 4-aligned
                dst[0] = v[p].x; dst[1] = v[p].y; dst[2] = v[p].z; dst[3] = v[p].w;
            }
        }
    }
    __syncthreads();
    {   // 32 lanes x 4 bytes cover one 128-byte row piece; a lane's block is rows r4 .. r4 + 3
        const int rg = tid >> 5, c4 = (tid & 31) * 4;
#pragma unroll 1
        for (int p = 0; p < TR / 32; ++p) {
            const int r4 = 4 * (8 * p + rg);
            const uint32_t w0 = *reinterpret_cast<const uint32_t*>(&tile[c4 + 0][r4]);
            const uint32_t w1 = *reinterpret_cast<const uint32_t*>(&tile[c4 + 1][r4]);
            const uint32_t w2 = *reinterpret_cast<const uint32_t*>(&tile[c4 + 2][r4]);
            const uint32_t w3 = *reinterpret_cast<const uint32_t*>(&tile[c4 + 3][r4]);
            // perm(hi, lo, sel): result byte i = byte sel[i] of {hi, lo} (0..3 = lo, 4..7 = hi)
            const uint32_t a = __builtin_amdgcn_perm(w1, w0, 0x05010400u);   // w0.0 w1.0 w0.1 w1.1
            const uint32_t bq = __builtin_amdgcn_perm(w3, w2, 0x05010400u);  // w2.0 w3.0 w2.1 w3.1
            const uint32_t cq = __builtin_amdgcn_perm(w1, w0, 0x07030602u);  // w0.2 w1.2 w0.3 w1.3
            const uint32_t d = __builtin_amdgcn_perm(w3, w2, 0x07030602u);   // w2.2 w3.2 w2.3 w3.3
            uint8_t* out = qout + sb * R * C + (r0 + r4) * C + c0 + c4;
            *reinterpret_cast<uint32_t*>(out) = __builtin_amdgcn_perm(bq, a, 0x05040100u);
            *reinterpret_cast<uint32_t*>(out + C) = __builtin_amdgcn_perm(bq, a, 0x07060302u);
            *reinterpret_cast<uint32_t*>(out + 2 * C) = __builtin_amdgcn_perm(d, cq, 0x05040100u);
            *reinterpret_cast<uint32_t*>(out + 3 * C) = __builtin_amdgcn_perm(d, cq, 0x07060302u);
        }
    }
}

// Hp[b][i][j] = H[b][perm[i]][perm[j]], dead rows/columns zeroed with a unit diagonal
// (forge/gptq.py:100-103,117,145-149).  The source row is streamed into LDS with coalesced
// loads, gathered from there in permuted order and written out coalesced, so HBM sees one
// sequential read and one sequential write.
//
// General form: one workgroup per output row, scalar accesses, LDS staging when C fits.
__global__ __launch_bounds__(256) void hessian_permute_kernel(
    const float* __restrict__ H, const int64_t* __restrict__ perm, const uint8_t* __restrict__ dead,
    float* __restrict__ Hp, int64_t C, const int64_t* __restrict__ index) {
    extern __shared__ float srow[];                 // C floats, or nothing when C is too large
    const int64_t b = blockIdx.y, i = blockIdx.x, sb = index ? index[b] : b;
    const int64_t* __restrict__ pb = perm + sb * C;
    const uint8_t* __restrict__ db = dead ? dead + sb * C : nullptr;
    const float* __restrict__ src = H + sb * C * C + pb[i] * C;
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

// Fast form for C % 4 == 0 and C <= 1024 * NCH: a workgroup produces kPermuteRows
// consecutive output rows.  Thread t owns the output columns 4*(t + 256u) .. +3 (u < NCH)
// of every row and keeps their source indices in registers, so the permutation is read
// once per workgroup instead of once per row; rows move as float4 on both sides and the
// two LDS row buffers alternate, which leaves one barrier per row.
constexpr int kPermuteRows = 16;
// lower_blocks: columns beyond the row's own 128-column block are not written (a factorisation
// that works on the lower triangle in 128 x 128 blocks never reads them).
template <int NCH>
__global__ __launch_bounds__(256) void hessian_permute_rows_kernel(
    const float* __restrict__ H, const int64_t* __restrict__ perm, const uint8_t* __restrict__ dead,
    float* __restrict__ Hp, int C, bool lower_blocks, const int64_t* __restrict__ index) {
    extern __shared__ float srow[];                 // 2 * C floats
    const int64_t b = blockIdx.y, sb = index ? index[b] : b;
    const int i0 = blockIdx.x * kPermuteRows;
    const int tid = threadIdx.x;
    const int64_t* __restrict__ pb = perm + sb * C;
    const uint8_t* __restrict__ db = dead ? dead + sb * C : nullptr;
    const float* __restrict__ Hb = H + sb * (int64_t)C * C;
    float* __restrict__ Hpb = Hp + b * (int64_t)C * C;

    // Column chunks past the end are clamped onto the last one: they move the same data a
    // second time and are not written out.  (Guarding the register arrays instead makes
    // the compiler keep them in scratch memory.)
    int col[NCH];
    int src_col[NCH][4];
    unsigned dead_cols = 0;                         // bit 4u+k: output column is dead
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
        const int j = 4 * (tid + 256 * u);
        col[u] = j < C ? j : C - 4;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            src_col[u][k] = (int)pb[col[u] + k];
            if (db && db[col[u] + k]) dead_cols |= 1u << (4 * u + k);
        }
    }
    // the row in flight: named registers (as an array the compiler left it in scratch memory)
    float4 st0, st1, st2, st3, st4, st5, st6, st7;
#define FORGE_CHUNKS(M)                                  \
    M(0, st0) M(1, st1)                                  \
    if constexpr (NCH > 2) { M(2, st2) M(3, st3) }       \
    if constexpr (NCH > 4) { M(4, st4) M(5, st5) M(6, st6) M(7, st7) }
#define FORGE_LOAD(u, reg) reg = *reinterpret_cast<const float4*>(src + col[u]);
#define FORGE_STORE(u, reg) *reinterpret_cast<float4*>(buf + col[u]) = reg;
    static_assert(NCH == 2 || NCH == 4 || NCH == 8, "chunk counts the macro covers");
    const int rows = (C - i0) < kPermuteRows ? (C - i0) : kPermuteRows;
    {
        const float* __restrict__ src = Hb + pb[i0] * C;
        FORGE_CHUNKS(FORGE_LOAD)
    }
    for (int r = 0; r < rows; ++r) {
        float* __restrict__ buf = srow + (r & 1) * C;
        FORGE_CHUNKS(FORGE_STORE)
        __syncthreads();                            // also fences the buffer used two rows ago
        // next source row -> registers while this one is gathered (the last row again at the end)
        const int i_next = i0 + (r + 1 < rows ? r + 1 : r);
        const float* __restrict__ src = Hb + pb[i_next] * C;
        FORGE_CHUNKS(FORGE_LOAD)
        const int i = i0 + r;
        const bool dead_i = db && db[i];
        float* __restrict__ dst = Hpb + (int64_t)i * C;
        const int jmax = lower_blocks ? (i / 128 + 1) * 128 : C;
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            if (4 * (tid + 256 * u) >= jmax) continue;
            float4 v;
            v.x = buf[src_col[u][0]];
            v.y = buf[src_col[u][1]];
            v.z = buf[src_col[u][2]];
            v.w = buf[src_col[u][3]];
            const unsigned dc = dead_i ? 0xFu : (dead_cols >> (4 * u)) & 0xFu;
            if (dc & 1u) v.x = (i == col[u] + 0) ? 1.0f : 0.0f;
            if (dc & 2u) v.y = (i == col[u] + 1) ? 1.0f : 0.0f;
            if (dc & 4u) v.z = (i == col[u] + 2) ? 1.0f : 0.0f;
            if (dc & 8u) v.w = (i == col[u] + 3) ? 1.0f : 0.0f;
            if (4 * (tid + 256 * u) < C) *reinterpret_cast<float4*>(dst + col[u]) = v;
        }
    }
#undef FORGE_CHUNKS
#undef FORGE_LOAD
#undef FORGE_STORE
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

// C and the group size multiples of 8, rows 8-byte aligned: the 8 codes of a word are one
// 8-byte load and share one zero.
__global__ __launch_bounds__(256) void pack_int4_fast_kernel(const uint8_t* __restrict__ codes,
                                                             const float* __restrict__ qzeros,
                                                             int32_t* __restrict__ packed, int64_t R,
                                                             int64_t C, int64_t gs, int64_t G) {
    const int64_t W8 = C / 8;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= R * W8) return;
    const int64_t r = idx / W8, w = idx - r * W8;
    const uint2 cc = *reinterpret_cast<const uint2*>(codes + r * C + w * 8);
    const int z = qzeros ? (int)qzeros[r * G + (w * 8) / gs] : 8;
    const int bias = 8 - z;
    uint32_t word = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        word |= (uint32_t)(((int)((cc.x >> (8 * k)) & 0xFFu) + bias) & 0xF) << (4 * k);
        word |= (uint32_t)(((int)((cc.y >> (8 * k)) & 0xFFu) + bias) & 0xF) << (4 * k + 16);
    }
    packed[idx] = (int32_t)word;
}

// The four codes in the bytes of x, each plus its row's bias modulo 16, as four nibbles.
__device__ __forceinline__ uint32_t four_nibbles(uint32_t x, uint32_t bias4) {
    const uint32_t v = ((x & 0x0F0F0F0Fu) + bias4) & 0x0F0F0F0Fu;
    const uint32_t t = (v | (v >> 4)) & 0x00FF00FFu;
    return (t | (t >> 8)) & 0xFFFFu;
}

// C and the group size multiples of 16, codes 16-byte aligned, fewer than 2^32 pieces: the
// code array is one run of 16-byte pieces, a thread packs one piece into two words.  32-bit
// index arithmetic throughout (with 64-bit divisions per thread the kernel is bound by them,
// not by memory).  EVEN: the groups tile the row exactly, so piece / (gs / 16) numbers the
// zero points.
template <bool EVEN>
__global__ __launch_bounds__(256) void pack_int4_wide_kernel(const uint4* __restrict__ codes,
                                                             const float* __restrict__ qzeros,
                                                             uint2* __restrict__ packed, uint32_t pieces,
                                                             uint32_t per_row, uint32_t gs16, uint32_t G) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= pieces) return;
    const uint4 cc = codes[idx];
    int z = 8;
    if (qzeros) {
        uint32_t zi;
        if constexpr (EVEN) {
            zi = idx / gs16;
        } else {
            const uint32_t r = idx / per_row;
            zi = r * G + (idx - r * per_row) / gs16;
        }
        z = (int)qzeros[zi];
    }
    const uint32_t bias4 = ((uint32_t)(8 - z) & 0xFu) * 0x01010101u;
    packed[idx] = make_uint2(four_nibbles(cc.x, bias4) | (four_nibbles(cc.y, bias4) << 16),
                             four_nibbles(cc.z, bias4) | (four_nibbles(cc.w, bias4) << 16));
}

}  // namespace

static int weight_to_solver_order(const void* W, int w_dtype, int64_t w_stride, int64_t ldw,
                                  const int64_t* index, const int64_t* perm_inv, const uint8_t* dead,
                                  float* Xout, void* W0out, int64_t ldo, int64_t o_stride,
                                  int64_t batch, int64_t R, int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(w_dtype == FORGE_F32 || w_dtype == FORGE_BF16, "w_dtype=%d", w_dtype);
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && R >= 0 && C >= 0 && ldw >= C, "bad shape");
    FORGE_REQUIRE(ldo >= R && o_stride >= (C > 0 ? (C - 1) * ldo + R : 0), "output pitch too small");
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(W && perm_inv && (Xout || W0out), "null pointer");
    dim3 grid((unsigned)forge::ceil_div(C, 64), (unsigned)forge::ceil_div(R, 64), (unsigned)batch);
    FORGE_REQUIRE(grid.y < 65536, "R too large");
    forge::KernelTiming timing("weight_to_solver_order", (hipStream_t)stream,
                               (double)batch * R * C * ((Xout ? 4.0 : 0.0) + (w_dtype == FORGE_F32 ? 4.0 : 2.0) * (W0out ? 2.0 : 1.0)),
                               forge::WORK_BYTES);
    const bool fast = w_dtype == FORGE_BF16 && (R % 256) == 0 && (C % 64) == 0 && (ldw % 4) == 0 &&
                      (w_stride % 4) == 0 && (reinterpret_cast<uintptr_t>(W) % 8) == 0 &&
                      (reinterpret_cast<uintptr_t>(Xout) % 16) == 0 && (ldo % 4) == 0 &&
                      (o_stride % 4) == 0 && R / 256 < 65536 &&
                      (reinterpret_cast<uintptr_t>(W0out) % 8) == 0;
    if (fast) {
        const dim3 tiles((unsigned)(C / 64), (unsigned)(R / 256), (unsigned)batch);
        constexpr size_t kLds = 64 * 260 * sizeof(uint16_t);
#define FORGE_W2S(DEAD, XOUT)                                                                        \
    to_solver_order_bf16_kernel<DEAD, XOUT><<<tiles, dim3(256), kLds, (hipStream_t)stream>>>(       \
        (const uint16_t*)W, w_stride, ldw, perm_inv, dead, Xout, (uint16_t*)W0out, R, C, ldo, o_stride, index)
        if (dead && Xout) FORGE_W2S(true, true);
        else if (dead) FORGE_W2S(true, false);
        else if (Xout) FORGE_W2S(false, true);
        else FORGE_W2S(false, false);
#undef FORGE_W2S
    } else if (w_dtype == FORGE_F32) {
        to_solver_order_kernel<float><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            (const float*)W, w_stride, ldw, perm_inv, dead, Xout, (float*)W0out, R, C, ldo, o_stride, index);
    } else {
        to_solver_order_kernel<__hip_bfloat16><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            (const __hip_bfloat16*)W, w_stride, ldw, perm_inv, dead, Xout, (__hip_bfloat16*)W0out, R, C,
            ldo, o_stride, index);
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_weight_to_solver_order_pair(const void* W, int w_dtype, int64_t w_stride,
                                                 int64_t ldw, const int64_t* perm_inv,
                                                 const uint8_t* dead, float* Xout, void* W0out,
                                                 int64_t ldo, int64_t o_stride, int64_t batch,
                                                 int64_t R, int64_t C, forge_stream_t stream) {
    return weight_to_solver_order(W, w_dtype, w_stride, ldw, nullptr, perm_inv, dead, Xout, W0out, ldo,
                                  o_stride, batch, R, C, stream);
}

extern "C" int forge_weight_to_solver_order_gather(const void* W, int w_dtype, int64_t w_stride,
                                                   int64_t ldw, const int64_t* index,
                                                   const int64_t* perm_inv, const uint8_t* dead,
                                                   float* Xout, void* W0out, int64_t ldo,
                                                   int64_t o_stride, int64_t batch, int64_t R,
                                                   int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(index || batch == 0, "null index");
    return weight_to_solver_order(W, w_dtype, w_stride, ldw, index, perm_inv, dead, Xout, W0out, ldo,
                                  o_stride, batch, R, C, stream);
}

extern "C" int forge_weight_to_solver_order_strided(const void* W, int w_dtype, int64_t w_stride,
                                                    int64_t ldw, const int64_t* perm_inv,
                                                    const uint8_t* dead, float* Xout, int64_t ldo,
                                                    int64_t o_stride, int64_t batch, int64_t R,
                                                    int64_t C, forge_stream_t stream) {
    return forge_weight_to_solver_order_pair(W, w_dtype, w_stride, ldw, perm_inv, dead, Xout, nullptr,
                                             ldo, o_stride, batch, R, C, stream);
}

extern "C" int forge_weight_to_solver_order(const void* W, int w_dtype, int64_t w_stride,
                                            int64_t ldw, const int64_t* perm_inv,
                                            const uint8_t* dead, float* Xout, int64_t batch,
                                            int64_t R, int64_t C, forge_stream_t stream) {
    return forge_weight_to_solver_order_strided(W, w_dtype, w_stride, ldw, perm_inv, dead, Xout, R,
                                                C * R, batch, R, C, stream);
}

static int codes_to_layer_order(const uint8_t* qin, int64_t ldi, int64_t i_stride, const int64_t* index,
                                const int64_t* perm_inv, uint8_t* qout, int64_t batch, int64_t R,
                                int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && R >= 0 && C >= 0, "bad shape");
    FORGE_REQUIRE(ldi >= R && i_stride >= (C > 0 ? (C - 1) * ldi + R : 0), "input pitch too small");
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(qin && perm_inv && qout, "null pointer");
    dim3 grid((unsigned)forge::ceil_div(C, 64), (unsigned)forge::ceil_div(R, 64), (unsigned)batch);
    FORGE_REQUIRE(grid.y < 65536, "R too large");
    forge::KernelTiming timing("codes_to_layer_order", (hipStream_t)stream, 2.0 * batch * R * C,
                               forge::WORK_BYTES);
    const bool fast = (R % 256) == 0 && (C % 128) == 0 && (reinterpret_cast<uintptr_t>(qin) % 16) == 0 &&
                      (reinterpret_cast<uintptr_t>(qout) % 4) == 0 && (ldi % 16) == 0 && (i_stride % 16) == 0;
    if (fast) {
        const dim3 tiles((unsigned)(C / 128), (unsigned)(R / 256), (unsigned)batch);
        to_layer_order_fast_kernel<<<tiles, dim3(256), 128 * 260, (hipStream_t)stream>>>(qin, perm_inv, qout, R, C,
                                                                                 ldi, i_stride, index);
    } else {
        to_layer_order_kernel<<<grid, dim3(256), 0, (hipStream_t)stream>>>(qin, perm_inv, qout, R, C, ldi,
                                                                           i_stride, index);
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_codes_to_layer_order_strided(const uint8_t* qin, int64_t ldi, int64_t i_stride,
                                                  const int64_t* perm_inv, uint8_t* qout,
                                                  int64_t batch, int64_t R, int64_t C,
                                                  forge_stream_t stream) {
    return codes_to_layer_order(qin, ldi, i_stride, nullptr, perm_inv, qout, batch, R, C, stream);
}

extern "C" int forge_codes_to_layer_order_scatter(const uint8_t* qin, int64_t ldi, int64_t i_stride,
                                                  const int64_t* index, const int64_t* perm_inv,
                                                  uint8_t* qout, int64_t batch, int64_t R, int64_t C,
                                                  forge_stream_t stream) {
    FORGE_REQUIRE(index || batch == 0, "null index");
    return codes_to_layer_order(qin, ldi, i_stride, index, perm_inv, qout, batch, R, C, stream);
}

extern "C" int forge_codes_to_layer_order(const uint8_t* qin, const int64_t* perm_inv,
                                          uint8_t* qout, int64_t batch, int64_t R, int64_t C,
                                          forge_stream_t stream) {
    return forge_codes_to_layer_order_strided(qin, R, C * R, perm_inv, qout, batch, R, C, stream);
}

static int hessian_permute(const float* H, const int64_t* index, const int64_t* perm,
                           const uint8_t* dead, float* Hp, float* damp, float rel_damp, int64_t batch,
                           int64_t C, bool lower_blocks, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && batch < 65536 && C >= 1, "bad shape");
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(H && perm && Hp && damp, "null pointer");
    FORGE_REQUIRE(H != Hp, "hessian_permute cannot run in place");
    hipStream_t st = (hipStream_t)stream;
    forge::KernelTiming timing("hessian_permute", st, (lower_blocks ? 6.0 : 8.0) * C * C * (double)batch,
                               forge::WORK_BYTES);
    const bool vec_ok = (C % 4) == 0 && C <= 8192 && (reinterpret_cast<uintptr_t>(H) % 16) == 0 &&
                        (reinterpret_cast<uintptr_t>(Hp) % 16) == 0;
    if (vec_ok) {
        const dim3 grid((unsigned)forge::ceil_div(C, kPermuteRows), (unsigned)batch);
        const size_t lds = 2 * (size_t)C * sizeof(float);   // <= 64 KB
        if (C <= 2048)
            hessian_permute_rows_kernel<2><<<grid, dim3(256), lds, st>>>(H, perm, dead, Hp, (int)C, lower_blocks, index);
        else if (C <= 4096)
            hessian_permute_rows_kernel<4><<<grid, dim3(256), lds, st>>>(H, perm, dead, Hp, (int)C, lower_blocks, index);
        else
            hessian_permute_rows_kernel<8><<<grid, dim3(256), lds, st>>>(H, perm, dead, Hp, (int)C, lower_blocks, index);
    } else {
        const size_t lds = C <= kPermuteLdsFloats ? (size_t)C * sizeof(float) : 0;
        hessian_permute_kernel<<<dim3((unsigned)C, (unsigned)batch), dim3(256), lds, st>>>(
            H, perm, dead, Hp, C, index);
    }
    FORGE_LAUNCH_CHECK();
    damp_kernel<<<dim3((unsigned)batch), dim3(256), 0, st>>>(Hp, damp, rel_damp, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_hessian_permute(const float* H, const int64_t* perm, const uint8_t* dead,
                                     float* Hp, float* damp, float rel_damp, int64_t batch,
                                     int64_t C, forge_stream_t stream) {
    return hessian_permute(H, nullptr, perm, dead, Hp, damp, rel_damp, batch, C, false, stream);
}

extern "C" int forge_hessian_permute_lower(const float* H, const int64_t* perm, const uint8_t* dead,
                                           float* Hp, float* damp, float rel_damp, int64_t batch,
                                           int64_t C, forge_stream_t stream) {
    return hessian_permute(H, nullptr, perm, dead, Hp, damp, rel_damp, batch, C, true, stream);
}

extern "C" int forge_hessian_permute_gather(const float* H, const int64_t* index, const int64_t* perm,
                                            const uint8_t* dead, float* Hp, float* damp,
                                            float rel_damp, int64_t batch, int64_t C, int lower_blocks,
                                            forge_stream_t stream) {
    FORGE_REQUIRE(index || batch == 0, "null index");
    return hessian_permute(H, index, perm, dead, Hp, damp, rel_damp, batch, C, lower_blocks != 0, stream);
}

extern "C" int forge_pack_int4(const uint8_t* codes, const float* qzeros, int32_t* packed,
                               int64_t R, int64_t C, int64_t gs, forge_stream_t stream) {
    FORGE_REQUIRE(R >= 0 && C >= 0 && gs >= 1, "bad shape");
    if (R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(codes && packed, "null pointer");
    const int64_t n = R * ((C + 7) / 8);
    forge::KernelTiming timing("pack_int4", (hipStream_t)stream,
                               1.5 * R * C + 4.0 * R * forge::ceil_div(C, gs), forge::WORK_BYTES);
    if (C % 16 == 0 && gs % 16 == 0 && (reinterpret_cast<uintptr_t>(codes) % 16) == 0 &&
        (reinterpret_cast<uintptr_t>(packed) % 8) == 0 && n / 2 < (1LL << 32) - 256 && gs < (1LL << 32) &&
        R * forge::ceil_div(C, gs) < (1LL << 32)) {
        const uint32_t pieces = (uint32_t)(n / 2), per_row = (uint32_t)(C / 16);
        const dim3 grid((unsigned)forge::ceil_div((int64_t)pieces, 256));
        if (C % gs == 0)
            pack_int4_wide_kernel<true><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
                (const uint4*)codes, qzeros, (uint2*)packed, pieces, per_row, (uint32_t)(gs / 16),
                (uint32_t)(C / gs));
        else
            pack_int4_wide_kernel<false><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
                (const uint4*)codes, qzeros, (uint2*)packed, pieces, per_row, (uint32_t)(gs / 16),
                (uint32_t)forge::ceil_div(C, gs));
        FORGE_LAUNCH_CHECK();
        return FORGE_OK;
    }
    if (C % 8 == 0 && gs % 8 == 0 && (reinterpret_cast<uintptr_t>(codes) % 8) == 0 &&
        forge::ceil_div(n, 256) < (1LL << 31)) {
        pack_int4_fast_kernel<<<dim3((unsigned)forge::ceil_div(n, 256)), dim3(256), 0,
                                (hipStream_t)stream>>>(codes, qzeros, packed, R, C, gs,
                                                       forge::ceil_div(C, gs));
        FORGE_LAUNCH_CHECK();
        return FORGE_OK;
    }
    pack_int4_kernel<<<dim3((unsigned)forge::ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream>>>(
        codes, qzeros, packed, R, C, gs, forge::ceil_div(C, gs));
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

// ---------------------------------------------------------------------------------------------
// Front end of the blocked closed form: its operands straight from the calibration rows.
namespace {

// BT[b][r][j] = Bp[b][j][r] = (float)((double)rows[row0[b] + r][perm[b][j]] * root[b]) for r below
// the matrix's own row count and a column that is not pruned, else 0: the rows of
// sqrt(2/n) X (forge/gptq.py:70-79 sums their products into H) in solver order, once row-major
// (the factor's K-major operand) and once column-major (the sweep's).  32 x 32 tiles: the gather
// along the permuted columns and the row-major store by lanes along j, the transposed store by
// lanes along r.  Every element of both outputs is written (zeros beyond n[b]); BT may be null.
template <typename T>
__global__ __launch_bounds__(256) void rows_operands_kernel(
    const T* __restrict__ rows, const int64_t* __restrict__ row0, const int32_t* __restrict__ n,
    const double* __restrict__ root, const int64_t* __restrict__ perm,
    const uint8_t* __restrict__ dead, float* __restrict__ BT, float* __restrict__ Bp, int64_t C,
    int64_t nmax) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];   // (at launch, as above)
    float (*tile)[33] = reinterpret_cast<float (*)[33]>(lds_raw);
    run_beside_the_search();
    const int64_t b = blockIdx.z;
    const int64_t j0 = (int64_t)blockIdx.x * 32, r0 = (int64_t)blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int64_t j = j0 + tx;
    const int nb = n[b];
    const double sc = root[b];
    const bool live = j < C && !dead[b * C + j];
    const int64_t src = live ? perm[b * C + j] : 0;
    const T* __restrict__ Xb = rows + row0[b] * C;
#pragma unroll
    for (int i = ty; i < 32; i += 8) {
        const int64_t r = r0 + i;
        float v = 0.0f;
        if (live && r < nb) v = (float)((double)ld_as_f32(Xb + r * C + src) * sc);
        tile[i][tx] = v;
        if (BT && j < C && r < nmax) BT[(b * nmax + r) * C + j] = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = ty; i < 32; i += 8) {
        const int64_t jj = j0 + i, r = r0 + tx;
        if (jj < C && r < nmax) Bp[(b * C + jj) * nmax + r] = tile[tx][i];
    }
}

// out[b][c] = (float)(alpha[b] * sum_r (double)x[r][c]^2): the diagonal of (2/n) X^T X summed
// in float64 and rounded once.  One lane per feature, rows in sequence: the loads of a
// wavefront are one contiguous piece of a row.
template <typename T>
__global__ __launch_bounds__(256) void rows_diagonal_kernel(
    const T* __restrict__ rows, const int64_t* __restrict__ row0, const int32_t* __restrict__ n,
    const double* __restrict__ alpha, float* __restrict__ out, int64_t C) {
    run_beside_the_search();
    const int64_t b = blockIdx.y;
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const T* __restrict__ Xb = rows + row0[b] * C + c;
    const int nb = n[b];
    double acc = 0.0;
    for (int r = 0; r < nb; ++r) {
        const double x = (double)ld_as_f32(Xb + (int64_t)r * C);
        acc = __builtin_fma(x, x, acc);
    }
    out[b * C + c] = (float)(acc * alpha[b]);
}

}  // namespace

extern "C" int forge_rows_operands(const void* rows, int x_dtype, const int64_t* row0,
                                   const int32_t* n, const double* root, const int64_t* perm,
                                   const uint8_t* dead, float* BT, float* Bp, int64_t batch,
                                   int64_t C, int64_t nmax, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && C >= 1 && nmax >= 1, "bad shape");
    FORGE_REQUIRE(x_dtype == FORGE_BF16 || x_dtype == FORGE_F32, "rows must be bf16 or f32");
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(rows && row0 && n && root && perm && dead && Bp, "null pointer");
    FORGE_REQUIRE(batch <= 65535 && forge::ceil_div(nmax, 32) <= 65535, "batch or nmax too large for one grid");
    hipStream_t st = (hipStream_t)stream;
    forge::KernelTiming timing("rows_operands", st, (BT ? 8.0 : 4.0) * batch * nmax * C, forge::WORK_BYTES);
    const dim3 grid((unsigned)forge::ceil_div(C, 32), (unsigned)forge::ceil_div(nmax, 32), (unsigned)batch);
    if (x_dtype == FORGE_BF16)
        rows_operands_kernel<__hip_bfloat16><<<grid, dim3(256), 32 * 33 * sizeof(float), st>>>(
            (const __hip_bfloat16*)rows, row0, n, root, perm, dead, BT, Bp, C, nmax);
    else
        rows_operands_kernel<float><<<grid, dim3(256), 32 * 33 * sizeof(float), st>>>((const float*)rows, row0, n, root, perm,
                                                                dead, BT, Bp, C, nmax);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_rows_diagonal(const void* rows, int x_dtype, const int64_t* row0,
                                   const int32_t* n, const double* alpha, float* out, int64_t batch,
                                   int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(batch >= 0 && C >= 1, "bad shape");
    FORGE_REQUIRE(x_dtype == FORGE_BF16 || x_dtype == FORGE_F32, "rows must be bf16 or f32");
    if (batch == 0) return FORGE_OK;
    FORGE_REQUIRE(rows && row0 && n && alpha && out, "null pointer");
    FORGE_REQUIRE(batch <= 65535, "batch too large for one grid");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)forge::ceil_div(C, 256), (unsigned)batch);
    if (x_dtype == FORGE_BF16)
        rows_diagonal_kernel<__hip_bfloat16><<<grid, dim3(256), 0, st>>>(
            (const __hip_bfloat16*)rows, row0, n, alpha, out, C);
    else
        rows_diagonal_kernel<float><<<grid, dim3(256), 0, st>>>((const float*)rows, row0, n, alpha, out, C);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
