// Measurement aid, not part of the operator boundary: what the matrix pipes of the GPU sustain with
// nothing else going on.  A register-only loop of bf16 32x32x16 MFMAs (no LDS, no memory traffic), two
// 256-thread blocks per CU, eight independent accumulators per wave.  With `random_operands` the A and B
// registers are eight pseudo-random sets rotated from instruction to instruction, otherwise constants:
// under MFMA load the chip is power-limited and operands that toggle cost clock, so the two rates differ,
// and the expert-GEMM figures of the benchmark are printed next to the first.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mts_common.h"
#include "mts_probe.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

constexpr int kSets = 8;         // operand register sets and accumulators per wave
constexpr int kThreads = 256;

__device__ __forceinline__ uint32_t lcg(uint32_t& s) {
    s = s * 1664525u + 1013904223u;
    return s;
}

template <bool RANDOM>
__global__ __launch_bounds__(kThreads) void mfma_rate_kernel(float* sink, int rounds) {
    bf16x8 a[kSets], b[kSets];
    uint32_t s = threadIdx.x * 2654435761u + blockIdx.x * 97u + 12345u;
    for (int n = 0; n < kSets; ++n)
        for (int i = 0; i < 8; ++i) {
            const float va = RANDOM ? ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.001f : 0.5f;
            const float vb = RANDOM ? ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.00002f : 0.01f;
            a[n][i] = (__bf16)va;
            b[n][i] = (__bf16)vb;
        }
    f32x16 acc[kSets];
    for (int j = 0; j < kSets; ++j)
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    for (int it = 0; it < rounds; ++it) {   // one round = kSets * kSets MFMAs per wave
#pragma unroll
        for (int r = 0; r < kSets; ++r)
#pragma unroll
            for (int j = 0; j < kSets; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 3 * r) & 7], b[(j + r) & 7], acc[j], 0, 0, 0);
    }
    float total = 0.f;
    for (int j = 0; j < kSets; ++j)
        for (int i = 0; i < 16; ++i) total += acc[j][i];
    sink[(size_t)blockIdx.x * kThreads + threadIdx.x] = total;
}

}  // namespace

extern "C" int64_t mts_probe_mfma_sink_bytes(int blocks) { return blocks > 0 ? (int64_t)blocks * kThreads * 4 : 0; }

extern "C" int mts_probe_mfma_rate(int random_operands, int blocks, int rounds, void* sink, int64_t sink_bytes,
                                   double* flops, void* stream) {
    if (!sink) return MTS_ERR_NULL;
    if (blocks <= 0 || blocks > 65535 || rounds <= 0 || rounds > (1 << 20)) return MTS_ERR_SHAPE;
    if (sink_bytes < mts_probe_mfma_sink_bytes(blocks)) return MTS_ERR_WORKSPACE;
    if (flops) *flops = (double)blocks * (kThreads / 64) * rounds * (kSets * kSets) * (2.0 * 32 * 32 * 16);
    if (random_operands)
        mfma_rate_kernel<true><<<blocks, kThreads, 0, (hipStream_t)stream>>>((float*)sink, rounds);
    else
        mfma_rate_kernel<false><<<blocks, kThreads, 0, (hipStream_t)stream>>>((float*)sink, rounds);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
