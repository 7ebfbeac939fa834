// Measurement aid, not part of the operator boundary: what the matrix pipes of the GPU sustain with
// nothing else going on.  A register-only loop of bf16 32x32x16 MFMAs (no LDS, no memory traffic), two
// 256-thread blocks per CU, eight independent accumulators per wave.  With `random_operands` the A and B
// registers hold pseudo-random values, otherwise constants: operands that toggle cost power, and under
// continuous MFMA load the power governor sets the clock, so the two rates differ; the expert-GEMM figures
// of the benchmark are printed next to the first.
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

// Two blocks per CU (two waves per SIMD), so that the matrix pipe never waits for one wave's issue.  The
// operands are selected at run time, which keeps both variants in vector registers (constants known at
// compile time would be held in scalar registers and spill from there).  Consecutive MFMAs use the
// operands the way a 4x2 register tile of a GEMM does: the A fragment stays for two instructions.
__global__ __launch_bounds__(kThreads, 2) void mfma_rate_kernel(float* sink, int rounds, int random) {
    bf16x8 a[kSets], b[kSets];
    uint32_t s = threadIdx.x * 2654435761u + blockIdx.x * 97u + 12345u;
    for (int n = 0; n < kSets; ++n)
        for (int i = 0; i < 8; ++i) {
            const float ra = ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.001f;
            const float rb = ((int)(lcg(s) >> 8) % 2001 - 1000) * 0.00002f;
            a[n][i] = (__bf16)(random ? ra : 0.5f);
            b[n][i] = (__bf16)(random ? rb : 0.01f);
        }
    f32x16 acc[kSets];
    for (int j = 0; j < kSets; ++j)
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    for (int it = 0; it < rounds; ++it) {   // one round = kSets * kSets MFMAs per wave
#pragma unroll
        for (int r = 0; r < kSets; ++r)
#pragma unroll
            for (int j = 0; j < kSets; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j / 2 + 4 * (r & 1)) & 7], b[(j % 2 + 2 * (r & 3)) & 7],
                                                                 acc[j], 0, 0, 0);
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
    mfma_rate_kernel<<<blocks, kThreads, 0, (hipStream_t)stream>>>((float*)sink, rounds, random_operands != 0);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
