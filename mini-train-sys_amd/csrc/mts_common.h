// Shared device helpers for the gfx950 MoE kernels (wave size 64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mts_moe.h"

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef _Float16 mts_f16_t;
typedef __attribute__((ext_vector_type(8))) _Float16 mts_f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 mts_f16x4;
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

// fp16 instantiation of the grouped GEMMs (mts_gemm_f16.hip); the public entry points forward to it
extern "C" {
int mts_moe_fwd_gateup_swiglu_f16(const void* x, const void* w1, const int32_t* x_gather, const int32_t* expert_start,
                                  const void* weights, const int32_t* s_scatter, int64_t T, int K, int E, int H, int I, int act_dtype, void* pre_act, void* post_act,
                                  void* stream);
int mts_moe_fwd_down_f16(const void* post_act, const void* w2, const int32_t* expert_start, int64_t TK, int E, int H,
                         int I, int act_dtype, void* y, void* stream);
int mts_moe_fwd_gateup_down_f16(const void* x, const void* w1, const void* w2, const int32_t* x_gather,
                                const int32_t* expert_start, const void* weights, const int32_t* s_scatter, int64_t T, int K,
                                int E, int H, int I, int act_dtype, void* pre_act, void* post_act, void* y,
                                int32_t* workspace, int64_t workspace_bytes, void* stream);
int mts_moe_bwd_dy1_f16(const void* d_out, const void* w2, int w2_as_stored, const void* pre_act, const void* weights,
                        const int32_t* x_gather, const int32_t* s_scatter, const int32_t* expert_start, int64_t T,
                        int K, int E, int H, int I, int act_dtype, void* d_pre_act, void* weighted_act,
                        float* ds_partial, int32_t* schedule, void* stream);
int mts_moe_bwd_dx_f16(const void* d_pre_act, const void* w1, int w1_as_stored, const int32_t* expert_start,
                       int64_t TK, int E, int H, int I, int act_dtype, void* dx_expanded, void* stream);
int mts_moe_bwd_dw2_f16(const void* d_out, const void* weighted_act, const int32_t* x_gather,
                        const int32_t* expert_start, int64_t T, int K, int E, int H, int I, int act_dtype,
                        int grad_dtype, void* d_w2, void* workspace, int64_t workspace_bytes, void* stream);
int mts_moe_bwd_dw1_f16(const void* d_pre_act, const void* x, const int32_t* x_gather, const int32_t* expert_start,
                        int64_t T, int K, int E, int H, int I, int act_dtype, int grad_dtype, void* d_w1,
                        void* workspace, int64_t workspace_bytes, void* stream);
int mts_moe_bwd_joint_f16(const void* d_out, const void* weighted_act, const void* d_pre_act, const void* x,
                          const void* w1, const int32_t* x_gather, const int32_t* expert_start,
                          const int32_t* s_reverse, const float* ds_partial, int64_t T, int K, int E, int H, int I,
                          int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2, void* d_weights,
                          void* workspace1, int64_t workspace1_bytes, void* workspace2, int64_t workspace2_bytes,
                          const int32_t* schedule, void* stream);
int mts_moe_bwd_joint_router_f16(const void* d_out, const void* weighted_act, const void* d_pre_act, const void* x,
                                 const void* w1, const int32_t* x_gather, const int32_t* expert_start,
                                 const int32_t* s_reverse, const float* ds_partial, int64_t T, int K, int E, int H,
                                 int I, int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2,
                                 void* d_weights, void* workspace1, int64_t workspace1_bytes, void* workspace2,
                                 int64_t workspace2_bytes, const float* w_r, const float* logits,
                                 const float* weights, const int32_t* indices, const int32_t* counts,
                                 const float* g_prob_mean, const float* g_z_loss, const float* g_load_balance,
                                 int normalize, void* dx_router, void* dx, float* d_w_r, void* router_workspace,
                                 int64_t router_workspace_bytes, const int32_t* schedule, void* stream);
}

// fp32 GEMM launchers (mts_gemm_f32.hip); epi: 0 plain, 1 SwiGLU, 2 dO*W2 with SwiGLU backward
int mts_f32_rows(int epi, const float* A, int lda, const int32_t* a_gather, const float* B, int b_rows,
                 int N, int Kdim, const int32_t* expert_start, int E, int64_t TK, float* C, float* C2,
                 const float* pre_act, const float* route_w, const int32_t* s_scatter, float* ds_part,
                 int np, hipStream_t s);
int mts_f32_dw(const float* P, const int32_t* p_gather, const float* Q, const int32_t* q_gather, int M,
               int N, const int32_t* expert_start, int E, int grad_dtype, void* C, hipStream_t s);

// chained router forward (mts_router_linear.hip), launched by mts_moe_head_fwd (mts_route.hip)
#define MTS_HEAD_MAX_CHUNKS 512
// Launch shape of the chained router backward (mts_router_linear.hip): row blocks x column ranges, the threads
// a block needs (groups sets of col_threads) and its dynamic LDS; contract checks of that path; the reduction
// of its per-block dW_r partials.
struct MtsRouterBwdShape {
    int row_blocks, rows_per_block, groups, col_threads, cols_per_block, ranges;
};
int mts_router_bwd_check(const void* x, const float* w_r, int64_t T, int H, int E, int act_dtype);
void mts_router_bwd_shape(int64_t T, int H, int E, MtsRouterBwdShape* shape);
int mts_launch_router_dw_reduce(const float* part, int row_blocks, int64_t EH, float* d_w_r, hipStream_t s);
int mts_router_head_group(int H, int E, int act_dtype);   // rows a wave of the chained forward kernel finishes together
void mts_router_head_geometry(int64_t T, int group, int* blocks, int* rows_per_wave);
int mts_launch_router_head(const void* x, const float* w_r, int64_t T, int H, int E, int K, int normalize, int act_dtype,
                           float* logits, float* weights, int32_t* indices, void* weights_act, float* partial,
                           int32_t* cnt, hipStream_t s);
