// The per-token sum of expert rows (combine) as the work of one block, shared by the stand-alone kernel
// (mts_combine.hip) and by the launch that holds it behind the partial sums of the backward pass
// (mts_gemm.hip).
#pragma once

#include "mts_common.h"

namespace mts_cb {

constexpr int kCombineThreads = 256;

// One thread produces 8 consecutive columns (16 bytes of a 16-bit type) of one token:
// K row loads of 16 bytes each, fp32 accumulation, one rounding.  A thread works on
// UN outputs at a time (token t, t + T/UN, ...) and issues all their index, weight
// and row loads before the first use, to keep enough bytes in flight per CU.
// A negative s_rev entry is a dropped route: it contributes nothing, whatever its weight.
// ET is the 16-bit element type (bf16 or fp16).
template <typename ET>
struct Vec8;
template <>
struct Vec8<bf16_t> {
    typedef bf16x8 type;
};
template <>
struct Vec8<mts_f16_t> {
    typedef mts_f16x8 type;
};

// the work of block `block` of `nblocks` blocks of kCombineThreads threads
template <typename ET, int KK, int UN>
__device__ __forceinline__ void combine_rows_block(const ET* __restrict__ y, const ET* __restrict__ w,
                                                   const ET* __restrict__ addend, const int32_t* __restrict__ s_rev,
                                                   int64_t T, int K, int H, ET* __restrict__ out, int64_t block,
                                                   int64_t nblocks) {
    typedef typename Vec8<ET>::type vec8;   // 8 elements, 16 bytes
    const int vec_per_row = H / 8;
    const int64_t chunk = (T + UN - 1) / UN;           // tokens per unrolled slice
    const int64_t total = chunk * (int64_t)vec_per_row;
    for (int64_t i = block * kCombineThreads + threadIdx.x; i < total; i += nblocks * kCombineThreads) {
        const int64_t t0 = i / vec_per_row;
        const int c = (int)(i - t0 * vec_per_row);
        vec8 v[UN][KK], add[UN];
        float s[UN][KK];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int64_t t = t0 + u * chunk;
            add[u] = (addend && t < T) ? *reinterpret_cast<const vec8*>(addend + t * H + c * 8) : vec8{};
#pragma unroll
            for (int k = 0; k < KK; ++k) {
                const bool in = t < T && k < K;
                const int32_t r = in ? s_rev[t * K + k] : -1;
                const bool ok = r >= 0;
                const int64_t row = ok ? r : 0;
                const float wt = in ? (w ? (float)w[t * K + k] : 1.0f) : 0.f;
                s[u][k] = ok ? wt : 0.f;
                v[u][k] = *reinterpret_cast<const vec8*>(y + row * H + c * 8);
                if (!ok) v[u][k] = vec8{};   // row 0 may hold anything
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int64_t t = t0 + u * chunk;
            if (t >= T) continue;
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = (float)add[u][j];
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] += s[u][k] * (float)v[u][k][j];
            vec8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (ET)acc[j];
            *reinterpret_cast<vec8*>(out + t * H + c * 8) = o;
        }
    }
}

}  // namespace mts_cb
