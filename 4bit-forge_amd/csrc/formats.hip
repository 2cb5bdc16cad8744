// Data formats either side of the solve: the fp8 block-scaled checkpoint weights that
// come in, the 1:4 sparse int4 words that go out, the dequantised weight written back into
// the layer and the gather of routed rows in front of the Hessian update.  All HBM-bound
// byte movers.
#include "common.h"

namespace {

// OCP float8 e4m3fn (1-4-3, bias 7, no infinities, 0x7f/0xff = NaN) -> f32, exact.
__device__ __forceinline__ float e4m3fn_to_f32(uint32_t b) {
    const uint32_t sign = (b & 0x80u) << 24;
    const uint32_t exp = (b >> 3) & 0xFu, man = b & 0x7u;
    uint32_t bits;
    if (exp == 0xFu && man == 0x7u) {
        bits = 0x7FC00000u;                                   // NaN
    } else if (exp == 0) {
        // subnormal: man * 2^-9  (exact in f32)
        return __uint_as_float(sign | __float_as_uint((float)man * 0.001953125f));
    } else {
        bits = ((exp + 120u) << 23) | (man << 20);            // 127 - 7 = 120
    }
    return __uint_as_float(sign | bits);
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x) {
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);   // quiet NaN
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// w = fp8.to(f32) * scale_inv[row / so][col / si] -> bf16 (or f32); 16 bytes in per thread
// (forge/utils/io.py:533-563, 863-872).
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void fp8_block_dequant_kernel(
    const uint8_t* __restrict__ w, const float* __restrict__ sinv, void* __restrict__ out,
    int64_t O, int64_t I, int64_t so, int64_t si, int64_t nO, int64_t nI, int64_t batch) {
    const int64_t per_row = (I + 15) / 16;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= batch * O * per_row) return;
    const int64_t b = idx / (O * per_row);
    const int64_t rem = idx - b * O * per_row;
    const int64_t r = rem / per_row, c0 = (rem - r * per_row) * 16;
    const uint8_t* src = w + (b * O + r) * I + c0;
    const float* srow = sinv + (b * nO + r / so) * nI;
    const int n = (int)((I - c0) < 16 ? (I - c0) : 16);
    const int64_t o0 = (b * O + r) * I + c0;
    // whole 16-byte piece inside one scale tile, output piece aligned: one load, one scale,
    // 32 (bf16) or 64 (f32) bytes out in 16-byte stores
    const bool out_ok = ((reinterpret_cast<uintptr_t>(out) + (uint64_t)o0 * (OUT_BF16 ? 2 : 4)) & 15u) == 0;
    if (n == 16 && (si & 15) == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0 && out_ok) {
        const uint4 q = *reinterpret_cast<const uint4*>(src);
        const uint32_t wq[4] = {q.x, q.y, q.z, q.w};
        const float sc = srow[c0 / si];
        float f[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) f[i] = e4m3fn_to_f32((wq[i >> 2] >> (8 * (i & 3))) & 0xFFu) * sc;
        if constexpr (OUT_BF16) {
            uint32_t pk[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                pk[k] = (uint32_t)f32_to_bf16_rne(f[2 * k]) | ((uint32_t)f32_to_bf16_rne(f[2 * k + 1]) << 16);
            uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out) + o0);
            dst[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            dst[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
        } else {
            float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + o0);
#pragma unroll
            for (int k = 0; k < 4; ++k) dst[k] = make_float4(f[4 * k], f[4 * k + 1], f[4 * k + 2], f[4 * k + 3]);
        }
        return;
    }
    uint8_t v[16];
    for (int i = 0; i < n; ++i) v[i] = src[i];
    for (int i = 0; i < n; ++i) {
        const float f = e4m3fn_to_f32(v[i]) * srow[(c0 + i) / si];
        const int64_t o = (b * O + r) * I + c0 + i;
        if (OUT_BF16) reinterpret_cast<uint16_t*>(out)[o] = f32_to_bf16_rne(f);
        else reinterpret_cast<float*>(out)[o] = f;
    }
}

// I and the scale tile width multiples of 16, input and output 16-byte aligned: one workgroup
// per row (row, scale row and batch come from the block index once, in scalar registers), one
// 16-byte piece per thread and turn, and the conversions the matrix cores' input formats
// brought along: two fp8 -> two f32 and two f32 -> two bf16 (round to nearest even) in one
// instruction each.  Both are exact restatements of the bit arithmetic above for every input
// that is no NaN; a NaN stays a NaN.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

template <bool OUT_BF16>
__global__ __launch_bounds__(1024) void fp8_block_dequant_rows_kernel(
    const uint4* __restrict__ w, const float* __restrict__ sinv, void* __restrict__ out, uint32_t O,
    uint32_t per_row, uint32_t so, uint32_t si16, uint32_t nO, uint32_t nI) {
    const uint32_t row = blockIdx.x;                  // batch * O + r
    const uint32_t b = row / O, r = row - b * O;
    const float* srow = sinv + ((size_t)b * nO + r / so) * nI;
    const size_t base = (size_t)row * per_row;
    for (uint32_t p = threadIdx.x; p < per_row; p += blockDim.x) {
        const uint4 q = w[base + p];
        const float sc = srow[p / si16];
        const uint32_t wq[4] = {q.x, q.y, q.z, q.w};
        f32x2 f[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            f[2 * k] = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq[k], false) * sc;
            f[2 * k + 1] = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq[k], true) * sc;
        }
        if constexpr (OUT_BF16) {
            uint32_t pk[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const bf16x2 h = __builtin_convertvector(f[k], bf16x2);
                pk[k] = __builtin_bit_cast(uint32_t, h);
            }
            uint4* dst = reinterpret_cast<uint4*>(out) + 2 * (base + p);
            dst[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            dst[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
        } else {
            float4* dst = reinterpret_cast<float4*>(out) + 4 * (base + p);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                dst[k] = make_float4(f[2 * k].x, f[2 * k].y, f[2 * k + 1].x, f[2 * k + 1].y);
        }
    }
}

// 1:4 codes + keep-masks -> the inference layout of bitpacking_sparsegptq14.cu:58-107: for
// every row and every 32-column word one u64
//   bf16(scale) << 48 | idx16 << 32 | qw32
// qw32 = the eight kept 4-bit codes of the word (8, the code of a zero weight, where a group
// of four kept nothing), idx16 = their 2-bit positions inside their groups; words are stored
// in pairs, out[pair][row][2].
//
// The three inputs want different lane orders: the codes are row-major [R, C] (a word's 32
// bytes are contiguous, neighbouring words of one row follow each other), while masks,
// scales and the output are word-major ([word][row]: neighbouring rows are contiguous).  So a
// workgroup takes a tile of 128 rows x 8 words, brings the tile's codes into LDS with lanes
// running along the columns (256 bytes contiguous per row, 16 bytes per lane), and then
// switches to lanes running along the rows for everything else: 512-byte runs of masks and
// scales, 2 KiB runs of output, and 16-byte reads from LDS (row pitch 272 bytes).
constexpr int SP_ROWS = 128, SP_WORDS = 8, SP_COLS = SP_WORDS * 32, SP_PITCH = SP_COLS + 16;
constexpr int SP_PAIRS_PER_TURN = 256 / SP_ROWS;     // word pairs that the 256 threads build at a time

__global__ __launch_bounds__(256) void pack_sparse14_tile_kernel(
    const uint8_t* __restrict__ codes, const uint32_t* __restrict__ keep,
    const float* __restrict__ scales, uint64_t* __restrict__ out, int64_t C, int64_t R,
    int64_t n_words, bool vec_ok) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[SP_ROWS * SP_PITCH];
    const int64_t row0 = (int64_t)blockIdx.y * SP_ROWS;
    const int64_t word0 = (int64_t)blockIdx.x * SP_WORDS;
    const int64_t col0 = word0 * 32;
    const int tid = threadIdx.x;
    // phase 1: lanes along the columns
#pragma unroll
    for (int j = 0; j < SP_ROWS * (SP_COLS / 16) / 256; ++j) {
        const int piece = tid + 256 * j;
        const int lr = piece / (SP_COLS / 16), lc = (piece % (SP_COLS / 16)) * 16;
        const int64_t r = row0 + lr, c = col0 + lc;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (r < R && c < C) {
            const uint8_t* src = codes + r * C + c;
            if (vec_ok && c + 16 <= C) {
                v = *reinterpret_cast<const uint4*>(src);
            } else {
                uint32_t w[4] = {0u, 0u, 0u, 0u};
                for (int k = 0; k < 16 && c + k < C; ++k) w[k >> 2] |= (uint32_t)src[k] << (8 * (k & 3));
                v = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
        *reinterpret_cast<uint4*>(&tile[lr * SP_PITCH + lc]) = v;
    }
    __syncthreads();
    // phase 2: lanes along the rows; a thread builds both words of a pair
    const int lr = tid & (SP_ROWS - 1);
    const int64_t r = row0 + lr;
    if (r >= R) return;
    const uint8_t* trow = &tile[lr * SP_PITCH];
#pragma unroll
    for (int it = 0; it < SP_WORDS / 2 / SP_PAIRS_PER_TURN; ++it) {
        const int lpair = tid / SP_ROWS + SP_PAIRS_PER_TURN * it;   // pair of words inside the tile
        const int64_t pair = word0 / 2 + lpair;
        if (2 * pair >= n_words) break;
        uint64_t both[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int64_t word = 2 * pair + h;
            uint64_t packed = 0ull;
            if (word < n_words) {
                const uint32_t mask = keep[word * R + r];
                // the word's 32 codes as two 16-byte reads, a group of four = one register;
                // no branch below: a data-dependent byte read inside a branch is a branch and
                // an LDS round trip per group, one after the other
                const uint4* tw = reinterpret_cast<const uint4*>(trow + (2 * lpair + h) * 32);
                const uint4 lo4 = tw[0], hi4 = tw[1];
                const uint32_t fours[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
                const int64_t col = word * 32;
                uint32_t where = 0u, kept = 0u;
#pragma unroll
                for (int grp = 0; grp < 8; ++grp) {
                    const uint32_t four = (mask >> (4 * grp)) & 0xFu;
                    // first kept column of the group (0 where it kept nothing)
                    const uint32_t pos = (uint32_t)__builtin_ctz(four | 16u) & 3u;
                    // columns past C hold no code: the slot keeps the code of zero
                    const bool has = four != 0u && col + 4 * grp + pos < C;
                    const uint32_t code = has ? (fours[grp] >> (8 * pos)) & 0xFu : 8u;
                    where |= pos << (2 * grp);
                    kept |= code << (4 * grp);
                }
                packed = ((uint64_t)f32_to_bf16_rne(scales[word * R + r]) << 48) |
                         ((uint64_t)where << 32) | (uint64_t)kept;
            }
            both[h] = packed;
        }
        ulonglong2 o;
        o.x = both[0];
        o.y = both[1];
        *reinterpret_cast<ulonglong2*>(out + (pair * R + r) * 2) = o;
    }
}

// (q - q0) * s per group -> bf16/f32; 16 codes per thread (forge/utils/engine.py:71-97).
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void dequantize_groups_kernel(
    const uint8_t* __restrict__ q, const float* __restrict__ scales,
    const float* __restrict__ qzeros, void* __restrict__ out, int64_t R, int64_t C, int64_t gs,
    int64_t G, int64_t batch) {
    const int64_t per_row = (C + 15) / 16;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= batch * R * per_row) return;
    const int64_t br = idx / per_row;                      // b * R + r
    const int64_t c0 = (idx - br * per_row) * 16;
    const uint8_t* __restrict__ src = q + br * C + c0;
    const float* __restrict__ s = scales + br * G;
    const float* __restrict__ z = qzeros + br * G;
    const bool vec = c0 + 16 <= C && ((reinterpret_cast<uintptr_t>(src) & 15u) == 0);
    uint8_t code[16];
    if (vec) {
        const uint4 v = *reinterpret_cast<const uint4*>(src);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 16; ++k) code[k] = (uint8_t)(w[k >> 2] >> (8 * (k & 3)));
    } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) code[k] = c0 + k < C ? src[k] : (uint8_t)0;
    }
    float val[16];
    if (vec && (gs & 15) == 0) {
        // the 16 columns share a group: one scale, one zero, no per-element division
        const int64_t g = c0 / gs;
        const float zz = z[g], ss = s[g];
#pragma unroll
        for (int k = 0; k < 16; ++k) val[k] = ((float)code[k] - zz) * ss;
    } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int64_t g = (c0 + k < C ? c0 + k : C - 1) / gs;
            val[k] = ((float)code[k] - z[g]) * s[g];
        }
    }
    if constexpr (OUT_BF16) {
        uint16_t* __restrict__ dst = reinterpret_cast<uint16_t*>(out) + br * C + c0;
        if (c0 + 16 <= C && ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0)) {
            uint32_t pk[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                pk[k] = (uint32_t)f32_to_bf16_rne(val[2 * k]) | ((uint32_t)f32_to_bf16_rne(val[2 * k + 1]) << 16);
            reinterpret_cast<uint4*>(dst)[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            reinterpret_cast<uint4*>(dst)[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k)
                if (c0 + k < C) dst[k] = f32_to_bf16_rne(val[k]);
        }
    } else {
        float* __restrict__ dst = reinterpret_cast<float*>(out) + br * C + c0;
#pragma unroll
        for (int k = 0; k < 16; ++k)
            if (c0 + k < C) dst[k] = val[k];
    }
}

// C and the group size multiples of 16, codes and output 16-byte aligned: one workgroup per
// row, a 16-byte piece of codes per thread and turn, 32-bit indices, bf16 rounding (to nearest
// even, as f32_to_bf16_rne) by the hardware's packed conversion.
template <bool OUT_BF16>
__global__ __launch_bounds__(1024) void dequantize_groups_rows_kernel(
    const uint4* __restrict__ q, const float* __restrict__ scales, const float* __restrict__ qzeros,
    void* __restrict__ out, uint32_t per_row, uint32_t gs16, uint32_t G) {
    const size_t row = blockIdx.x;                    // batch * R + r
    const float* __restrict__ s = scales + row * G;
    const float* __restrict__ z = qzeros + row * G;
    const size_t base = row * per_row;
    for (uint32_t p = threadIdx.x; p < per_row; p += blockDim.x) {
        const uint4 v = q[base + p];
        const uint32_t g = p / gs16;
        const float zz = z[g], ss = s[g];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        float val[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) val[k] = ((float)((w[k >> 2] >> (8 * (k & 3))) & 0xFFu) - zz) * ss;
        if constexpr (OUT_BF16) {
            uint32_t pk[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                f32x2 pair;
                pair.x = val[2 * k];
                pair.y = val[2 * k + 1];
                pk[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
            }
            uint4* dst = reinterpret_cast<uint4*>(out) + 2 * (base + p);
            dst[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            dst[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
        } else {
            float4* dst = reinterpret_cast<float4*>(out) + 4 * (base + p);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                dst[k] = make_float4(val[4 * k], val[4 * k + 1], val[4 * k + 2], val[4 * k + 3]);
        }
    }
}

// out[i][:] = X[row_idx[i]][:] * weight[i]; one workgroup per output row, 8 bytes per lane.
template <typename T, bool SCALE>
__global__ __launch_bounds__(256) void gather_scaled_rows_kernel(
    const T* __restrict__ X, int64_t ldx, int64_t C, const int64_t* __restrict__ row_idx,
    const T* __restrict__ weight, T* __restrict__ out) {
    const int64_t i = blockIdx.x;
    const T* __restrict__ src = X + row_idx[i] * ldx;
    T* __restrict__ dst = out + i * C;
    float w = 1.0f;
    if constexpr (SCALE) {
        if constexpr (sizeof(T) == 2) w = __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(weight)[i] << 16);
        else w = reinterpret_cast<const float*>(weight)[i];
    }
    constexpr int PER = 8 / sizeof(T);                      // elements per 8-byte access
    const bool vec = (C % PER) == 0 && ((reinterpret_cast<uintptr_t>(src) & 7u) == 0) &&
                     ((reinterpret_cast<uintptr_t>(dst) & 7u) == 0);
    if (vec) {
        for (int64_t j = threadIdx.x; j < C / PER; j += blockDim.x) {
            uint2 v = reinterpret_cast<const uint2*>(src)[j];
            if constexpr (SCALE) {
                if constexpr (sizeof(T) == 2) {
                    const uint32_t in[2] = {v.x, v.y};
                    uint32_t o[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const float a = __uint_as_float(in[h] << 16) * w;
                        const float b = __uint_as_float(in[h] & 0xFFFF0000u) * w;
                        o[h] = (uint32_t)f32_to_bf16_rne(a) | ((uint32_t)f32_to_bf16_rne(b) << 16);
                    }
                    v = make_uint2(o[0], o[1]);
                } else {
                    v = make_uint2(__float_as_uint(__uint_as_float(v.x) * w),
                                   __float_as_uint(__uint_as_float(v.y) * w));
                }
            }
            reinterpret_cast<uint2*>(dst)[j] = v;
        }
    } else {
        for (int64_t j = threadIdx.x; j < C; j += blockDim.x) {
            if constexpr (sizeof(T) == 2) {
                const uint16_t x = reinterpret_cast<const uint16_t*>(src)[j];
                reinterpret_cast<uint16_t*>(dst)[j] =
                    SCALE ? f32_to_bf16_rne(__uint_as_float((uint32_t)x << 16) * w) : x;
            } else {
                const float x = reinterpret_cast<const float*>(src)[j];
                reinterpret_cast<float*>(dst)[j] = SCALE ? x * w : x;
            }
        }
    }
}

}  // namespace

extern "C" int forge_fp8_e4m3_block_dequant(const uint8_t* w, const float* scale_inv, void* out,
                                            int out_dtype, int64_t batch, int64_t O, int64_t I,
                                            int64_t so, int64_t si, forge_stream_t stream) {
    FORGE_REQUIRE(out_dtype == FORGE_F32 || out_dtype == FORGE_BF16, "out_dtype=%d", out_dtype);
    FORGE_REQUIRE(batch >= 0 && O >= 0 && I >= 0 && so >= 1 && si >= 1, "bad shape");
    if (batch == 0 || O == 0 || I == 0) return FORGE_OK;
    FORGE_REQUIRE(w && scale_inv && out, "null pointer");
    const int64_t nO = forge::ceil_div(O, so), nI = forge::ceil_div(I, si);
    const int64_t n = batch * O * forge::ceil_div(I, 16);
    forge::KernelTiming timing("fp8_block_dequant", (hipStream_t)stream,
                               (double)batch * O * I * (out_dtype == FORGE_BF16 ? 3.0 : 5.0),
                               forge::WORK_BYTES);
    if (I % 16 == 0 && si % 16 == 0 && (reinterpret_cast<uintptr_t>(w) % 16) == 0 &&
        (reinterpret_cast<uintptr_t>(out) % 16) == 0 && batch * O < (1LL << 31) && I < (1LL << 32) &&
        so < (1LL << 32) && si < (1LL << 32) && nO < (1LL << 32)) {
        const uint32_t per_row = (uint32_t)(I / 16);
        const dim3 rows((unsigned)(batch * O));
        const dim3 block((unsigned)std::min<int64_t>(1024, forge::ceil_div((int64_t)per_row, 64) * 64));
        if (out_dtype == FORGE_BF16)
            fp8_block_dequant_rows_kernel<true><<<rows, block, 0, (hipStream_t)stream>>>(
                (const uint4*)w, scale_inv, out, (uint32_t)O, per_row, (uint32_t)so, (uint32_t)(si / 16),
                (uint32_t)nO, (uint32_t)nI);
        else
            fp8_block_dequant_rows_kernel<false><<<rows, block, 0, (hipStream_t)stream>>>(
                (const uint4*)w, scale_inv, out, (uint32_t)O, per_row, (uint32_t)so, (uint32_t)(si / 16),
                (uint32_t)nO, (uint32_t)nI);
        FORGE_LAUNCH_CHECK();
        return FORGE_OK;
    }
    dim3 grid((unsigned)forge::ceil_div(n, 256));
    if (out_dtype == FORGE_BF16)
        fp8_block_dequant_kernel<true><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            w, scale_inv, out, O, I, so, si, nO, nI, batch);
    else
        fp8_block_dequant_kernel<false><<<grid, dim3(256), 0, (hipStream_t)stream>>>(
            w, scale_inv, out, O, I, so, si, nO, nI, batch);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_pack_sparsegptq14_to_u64x2(const uint8_t* qweight_rc, const uint32_t* M,
                                                const float* scales, uint64_t* out, int64_t R,
                                                int64_t C, forge_stream_t stream) {
    FORGE_REQUIRE(R >= 0 && C >= 0, "bad shape");
    if (R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(qweight_rc && M && scales && out, "null pointer");
    const int64_t G32 = forge::ceil_div(C, 32), G2 = (G32 + 1) >> 1;
    forge::KernelTiming timing("pack_sparse14_u64x2", (hipStream_t)stream,
                               (double)R * C + 8.0 * G32 * R + 16.0 * G2 * R, forge::WORK_BYTES);
    const bool vec_ok = (C % 16) == 0 && (reinterpret_cast<uintptr_t>(qweight_rc) % 16) == 0;
    FORGE_REQUIRE(forge::ceil_div(R, SP_ROWS) < 65536, "R=%lld too large", (long long)R);
    pack_sparse14_tile_kernel<<<dim3((unsigned)forge::ceil_div(G32, SP_WORDS),
                                     (unsigned)forge::ceil_div(R, SP_ROWS)),
                                dim3(256), 0, (hipStream_t)stream>>>(qweight_rc, M, scales, out, C, R,
                                                                     G32, vec_ok);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_dequantize_groups(const uint8_t* q, const float* scales, const float* qzeros,
                                       void* out, int out_dtype, int64_t batch, int64_t R,
                                       int64_t C, int64_t gs, forge_stream_t stream) {
    FORGE_REQUIRE(out_dtype == FORGE_F32 || out_dtype == FORGE_BF16, "out_dtype=%d", out_dtype);
    FORGE_REQUIRE(batch >= 0 && R >= 0 && C >= 0 && gs >= 1, "bad shape");
    if (batch == 0 || R == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(q && scales && qzeros && out, "null pointer");
    const int64_t G = forge::ceil_div(C, gs);
    const int64_t n = batch * R * forge::ceil_div(C, 16);
    forge::KernelTiming timing("dequantize_groups", (hipStream_t)stream,
                               (double)batch * R * (C * (out_dtype == FORGE_BF16 ? 3.0 : 5.0) + 8.0 * G),
                               forge::WORK_BYTES);
    if (C % 16 == 0 && gs % 16 == 0 && (reinterpret_cast<uintptr_t>(q) % 16) == 0 &&
        (reinterpret_cast<uintptr_t>(out) % 16) == 0 && batch * R < (1LL << 31) && C < (1LL << 32) &&
        gs < (1LL << 32)) {
        const uint32_t per_row = (uint32_t)(C / 16);
        const dim3 rows((unsigned)(batch * R));
        const dim3 block((unsigned)std::min<int64_t>(1024, forge::ceil_div((int64_t)per_row, 64) * 64));
        if (out_dtype == FORGE_BF16)
            dequantize_groups_rows_kernel<true><<<rows, block, 0, (hipStream_t)stream>>>(
                (const uint4*)q, scales, qzeros, out, per_row, (uint32_t)(gs / 16), (uint32_t)G);
        else
            dequantize_groups_rows_kernel<false><<<rows, block, 0, (hipStream_t)stream>>>(
                (const uint4*)q, scales, qzeros, out, per_row, (uint32_t)(gs / 16), (uint32_t)G);
        FORGE_LAUNCH_CHECK();
        return FORGE_OK;
    }
    const dim3 grid((unsigned)forge::ceil_div(n, 256));
    if (out_dtype == FORGE_BF16)
        dequantize_groups_kernel<true><<<grid, dim3(256), 0, (hipStream_t)stream>>>(q, scales, qzeros, out,
                                                                                  R, C, gs, G, batch);
    else
        dequantize_groups_kernel<false><<<grid, dim3(256), 0, (hipStream_t)stream>>>(q, scales, qzeros, out,
                                                                                   R, C, gs, G, batch);
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}

extern "C" int forge_gather_scaled_rows(const void* X, int x_dtype, int64_t ldx, int64_t T, int64_t C,
                                        const int64_t* row_idx, const void* weight, void* out,
                                        int64_t N, forge_stream_t stream) {
    FORGE_REQUIRE(x_dtype == FORGE_F32 || x_dtype == FORGE_BF16, "x_dtype=%d", x_dtype);
    FORGE_REQUIRE(N >= 0 && N < (1LL << 31) && T >= 0 && C >= 0 && ldx >= C, "bad shape");
    if (N == 0 || C == 0) return FORGE_OK;
    FORGE_REQUIRE(T > 0, "rows requested from an empty matrix");
    FORGE_REQUIRE(X && row_idx && out, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    forge::KernelTiming timing("gather_scaled_rows", st,
                               2.0 * N * C * (x_dtype == FORGE_BF16 ? 2.0 : 4.0), forge::WORK_BYTES);
    const dim3 grid((unsigned)N), block(256);
    if (x_dtype == FORGE_BF16) {
        if (weight)
            gather_scaled_rows_kernel<uint16_t, true><<<grid, block, 0, st>>>(
                (const uint16_t*)X, ldx, C, row_idx, (const uint16_t*)weight, (uint16_t*)out);
        else
            gather_scaled_rows_kernel<uint16_t, false><<<grid, block, 0, st>>>(
                (const uint16_t*)X, ldx, C, row_idx, nullptr, (uint16_t*)out);
    } else {
        if (weight)
            gather_scaled_rows_kernel<float, true><<<grid, block, 0, st>>>(
                (const float*)X, ldx, C, row_idx, (const float*)weight, (float*)out);
        else
            gather_scaled_rows_kernel<float, false><<<grid, block, 0, st>>>(
                (const float*)X, ldx, C, row_idx, nullptr, (float*)out);
    }
    FORGE_LAUNCH_CHECK();
    return FORGE_OK;
}
