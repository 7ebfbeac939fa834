// Shared device helpers for the gfx950 MoE kernels (wave size 64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mts_moe.h"

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define MTS_WAVE 64

#define MTS_CHECK_LAUNCH()                       \
    do {                                         \
        hipError_t _e = hipGetLastError();       \
        if (_e != hipSuccess) return (int)_e;    \
    } while (0)

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MTS_WAVE);
    return v;
}

__device__ __forceinline__ uint64_t lanemask_lt() {
    return (1ull << (threadIdx.x & 63)) - 1ull;
}

static inline bool mts_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// fp32 GEMM launchers (mts_gemm_f32.hip); epi: 0 plain, 1 SwiGLU, 2 dO*W2 with SwiGLU backward
int mts_f32_rows(int epi, const float* A, int lda, const int32_t* a_gather, const float* B, int b_rows,
                 int N, int Kdim, const int32_t* expert_start, int E, int64_t TK, float* C, float* C2,
                 const float* pre_act, const float* route_w, const int32_t* s_scatter, float* ds_part,
                 int np, hipStream_t s);
int mts_f32_dw(const float* P, const int32_t* p_gather, const float* Q, const int32_t* q_gather, int M,
               int N, const int32_t* expert_start, int E, int grad_dtype, void* C, hipStream_t s);
