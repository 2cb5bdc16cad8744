// Matrix-pipe rate probe: a benchmark helper of its own, built into libforge_probe.so beside
// this file and loaded by bench.py only; not part of libforge_hip.so and of no use to a caller
// of the library.
//
// The split GEMMs of this library run at about half of the published bf16 / fp16 matrix rate
// although their matrix instructions are issued back to back.  This kernel measures what the
// pipe itself sustains on the device at hand: every wavefront issues v_mfma_f32_32x32x16 on
// eight independent accumulators from operands that stay in registers -- no loads, no LDS, no
// other work.  With `random_bits` the operands are pseudo-random numbers in (-1, 1) (every
// mantissa and several exponent bits toggle between consecutive instructions, as with real
// weights); without, every operand is 1.0.  The difference between the two is the device's power
// management, and the random-operand rate is the ceiling that a GEMM on real data can reach.
#include <hip/hip_runtime.h>
#include <cstdint>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeAcc = 8;        // independent accumulators per wavefront
constexpr int kProbeOperands = 4;   // operand registers of each side

template <bool F16>
__global__ __launch_bounds__(256) void mfma_rate_kernel(int iters, int random_bits, float* __restrict__ sink) {
    unsigned lcg = 12345u + 77u * threadIdx.x + 1001u * blockIdx.x;
    auto next = [&]() -> float {
        lcg = lcg * 1664525u + 1013904223u;
        return random_bits ? __uint_as_float((lcg >> 9) | 0x3f800000u) * 2.0f - 3.0f : 1.0f;
    };
    u32x4 a[kProbeOperands], b[kProbeOperands];
#pragma unroll
    for (int i = 0; i < kProbeOperands; ++i)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f32x2 va = {next(), next()}, vb = {next(), next()};
            if (F16) {
                a[i][w] = __builtin_bit_cast(unsigned, __builtin_convertvector(va, f16x2));
                b[i][w] = __builtin_bit_cast(unsigned, __builtin_convertvector(vb, f16x2));
            } else {
                a[i][w] = __builtin_bit_cast(unsigned, __builtin_convertvector(va, bf16x2));
                b[i][w] = __builtin_bit_cast(unsigned, __builtin_convertvector(vb, bf16x2));
            }
        }
    f32x16 acc[kProbeAcc];
#pragma unroll
    for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < kProbeAcc; ++i) {
            if (F16)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    __builtin_bit_cast(f16x8, a[i % kProbeOperands]),
                    __builtin_bit_cast(f16x8, b[(i + it) % kProbeOperands]), acc[i], 0, 0, 0);
            else
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf16x8, a[i % kProbeOperands]),
                    __builtin_bit_cast(bf16x8, b[(i + it) % kProbeOperands]), acc[i], 0, 0, 0);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += acc[i][v];
    sink[(int64_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

// sink: probe_sink_floats(workgroups) floats of device memory.  *flops receives the work of the
// launch; the caller times it with events on `stream`.  Returns 0, or 1 for a bad argument or a
// failed launch.
extern "C" int64_t probe_sink_floats(int workgroups) {
    return workgroups > 0 ? (int64_t)workgroups * 256 : 0;
}

extern "C" int probe_mfma_rate(int f16, int random_bits, int iters, int workgroups, float* sink,
                               double* flops, void* stream) {
    if (iters < 1 || iters > (1 << 24) || workgroups < 1 || workgroups > 65535 || !sink || !flops) return 1;
    hipStream_t st = (hipStream_t)stream;
    *flops = 2.0 * 32 * 32 * 16 * kProbeAcc * (double)iters * 4.0 * (double)workgroups;
    if (f16) mfma_rate_kernel<true><<<dim3((unsigned)workgroups), dim3(256), 0, st>>>(iters, random_bits, sink);
    else mfma_rate_kernel<false><<<dim3((unsigned)workgroups), dim3(256), 0, st>>>(iters, random_bits, sink);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
