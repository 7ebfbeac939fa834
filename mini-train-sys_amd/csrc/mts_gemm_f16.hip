// fp16 instantiation of the grouped expert GEMMs: the source of mts_gemm.hip with fp16 as the
// 16-bit element type (v_mfma_f32_32x32x16_f16, fp32 accumulation) and entry points named
// mts_moe_*_f16, reached through the public entry points when act_dtype is MTS_F16.
#define MTS_GEMM_F16 1
#include "mts_gemm.hip"
