// The backward of the router projection as the work of one block, shared by the stand-alone kernels
// (mts_router_linear.hip) and by the launch that holds it next to the expert GEMMs' backward
// (mts_gemm.hip): dx (activation dtype) and a partial dW_r per block; with CHAIN the block first forms
// the logit gradients of its rows from the post-process's saved tensors.
#pragma once

#include "mts_common.h"
#include "mts_router_row.h"

namespace mts_rl {

__device__ __forceinline__ f32x4 load4(const bf16_t* p) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
    f32x4 r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    return r;
}
__device__ __forceinline__ f32x4 load4(const mts_f16_t* p) {
    const mts_f16x4 v = *reinterpret_cast<const mts_f16x4*>(p);
    f32x4 r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    return r;
}
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *reinterpret_cast<bf16x4*>(p) = o;
}
__device__ __forceinline__ void store4(mts_f16_t* p, f32x4 v) {
    mts_f16x4 o = {(mts_f16_t)v[0], (mts_f16_t)v[1], (mts_f16_t)v[2], (mts_f16_t)v[3]};
    *reinterpret_cast<mts_f16x4*>(p) = o;
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }

template <typename XT>
struct RawVec;
template <>
struct RawVec<bf16_t> {
    typedef bf16x4 type;
};
template <>
struct RawVec<mts_f16_t> {
    typedef mts_f16x4 type;
};
template <>
struct RawVec<float> {
    typedef f32x4 type;
};
__device__ __forceinline__ bf16x4 load_raw(const bf16_t* p) { return *reinterpret_cast<const bf16x4*>(p); }
__device__ __forceinline__ mts_f16x4 load_raw(const mts_f16_t* p) { return *reinterpret_cast<const mts_f16x4*>(p); }
__device__ __forceinline__ f32x4 load_raw(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 widen(bf16x4 v) {
    f32x4 r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    return r;
}
__device__ __forceinline__ f32x4 widen(mts_f16x4 v) {
    f32x4 r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    return r;
}
__device__ __forceinline__ f32x4 widen(f32x4 v) { return v; }

constexpr int bwd_max_threads(int EP) { return EP <= 8 ? 768 : 384; }   // 16 experts need twice the registers

// What the backward kernel needs to form the logit gradients itself (CHAIN): the saved outputs of
// the post-process and the gradients that arrived at them (null = zeros).
struct RouterGradIn {
    const float* logits;
    const float* weights;
    const int32_t* indices;
    const int32_t* counts;
    const float* g_w;
    const void* g_w_act;
    const float* g_p;
    const float* g_z;
    const float* g_lb;
    int act_dtype, K, normalize;
    // instead of g_w_act: partial row sums [rows][np] of the routing-weight gradient and the entry -> row map
    const float* ds_part;
    const int32_t* s_reverse;
    int np;
};
constexpr int kChainRows = 256;   // most rows a block of the chained kernel takes (their logit gradients sit in LDS)

// CHAIN: `dl` is not read; the block first computes the logit gradients of its rows from the
// post-process's saved tensors (one thread per row, the arithmetic of the stand-alone
// post-process backward) into LDS, [row][EP] with zeros past E, and the row loop reads them there.
template <typename XT, int EP, bool EXACT, bool CHAIN>
__device__ __forceinline__ void router_logits_bwd_block(const float* __restrict__ dl, const XT* __restrict__ x,
                                                        const float* __restrict__ w, int64_t T, int H, int E,
                                                        int rows_per_block, int groups, int cols_per_block,
                                                        XT* __restrict__ dx, float* __restrict__ part,
                                                        const RouterGradIn& rg, int bx, int by, int col_threads,
                                                        float* set_sum, float* dl_lds) {

    if constexpr (CHAIN) {
        using namespace mts_router;
        const int64_t b0 = (int64_t)bx * rows_per_block;
        const int64_t b1 = b0 + rows_per_block < T ? b0 + rows_per_block : T;
        const float inv_t = 1.0f / (float)T;
        const float gz = rg.g_z ? rg.g_z[0] * 2.0f * inv_t : 0.f;
        float gp[EP];
#pragma unroll
        for (int e = 0; e < EP; ++e) {
            gp[e] = (rg.g_p && e < E) ? rg.g_p[e] * inv_t : 0.f;
            if (rg.g_lb && e < E)
                gp[e] += rg.g_lb[0] * (float)E * ((float)rg.counts[e] / ((float)T * (float)rg.K)) * inv_t;
        }
        for (int64_t row = b0 + threadIdx.x; row < b1; row += blockDim.x) {
            RowState<EP, 1> r;
            load_row<EP, 1>(rg.logits, row, E, 0, r);
            float o[EP];
            auto grad_w = [&](int k) {
                const int64_t i = row * rg.K + k;
                float v = rg.g_w ? rg.g_w[i] : 0.f;
                if (rg.g_w_act)
                    v += rg.act_dtype == MTS_BF16 ? (float)reinterpret_cast<const bf16_t*>(rg.g_w_act)[i]
                                                  : (float)reinterpret_cast<const mts_f16_t*>(rg.g_w_act)[i];
                if (rg.ds_part) {   // the routing-weight gradient straight from the partial row sums of the dO*W2 GEMM
                    const int32_t r = rg.s_reverse[i];
                    float t = 0.f;
                    if (r >= 0) {
                        const float* p = rg.ds_part + (int64_t)r * rg.np;
                        for (int j = 0; j < rg.np; ++j) t += p[j];
                    }
                    v += (float)(XT)t;   // rounded as the operator's dS output is
                }
                return v;
            };
            row_logit_gradient<EP, 1>(r, gp, gz, rg.K, rg.normalize, 0, rg.weights + row * rg.K, rg.indices + row * rg.K,
                                      grad_w, o);
#pragma unroll
            for (int e = 0; e < EP; ++e) dl_lds[(row - b0) * EP + e] = e < E ? o[e] : 0.f;
        }
        __syncthreads();
    }
    const int grp = threadIdx.x / col_threads;
    const int cl = (threadIdx.x % col_threads) * 4;   // column within the block's range (`by` picks the range)
    const int c = by * cols_per_block + cl;
    const bool active = grp < groups && cl < cols_per_block && c < H;   // a block may hold more threads than the sets need
    typedef typename RawVec<XT>::type raw_t;
    f32x4 wv[EP], acc[EP];
#pragma unroll
    for (int e = 0; e < EP; ++e) {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        wv[e] = (active && e < E) ? *reinterpret_cast<const f32x4*>(w + (int64_t)e * H + c) : z;
        acc[e] = z;
    }
    const int64_t block_beg = (int64_t)bx * rows_per_block;
    const int64_t block_end = block_beg + rows_per_block < T ? block_beg + rows_per_block : T;
    const int64_t per_set = (block_end - block_beg + groups - 1) / groups;
    const int64_t row_beg = block_beg + grp * per_set < block_end ? block_beg + grp * per_set : block_end;
    const int64_t row_end = !active ? row_beg : (row_beg + per_set < block_end ? row_beg + per_set : block_end);
    auto one_row = [&](int64_t row, raw_t raw) {
        const f32x4 xv = widen(raw);
        float g[EP];
        if constexpr (CHAIN) {
            const float* src = dl_lds + (row - block_beg) * EP;   // the same address in every lane: a broadcast read
#pragma unroll
            for (int q = 0; q < EP / 4; ++q) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(src + q * 4);
                g[q * 4] = v[0], g[q * 4 + 1] = v[1], g[q * 4 + 2] = v[2], g[q * 4 + 3] = v[3];
            }
        } else if constexpr (EXACT) {
#pragma unroll
            for (int q = 0; q < EP / 4; ++q) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(dl + row * EP + q * 4);
                g[q * 4] = v[0], g[q * 4 + 1] = v[1], g[q * 4 + 2] = v[2], g[q * 4 + 3] = v[3];
            }
        } else {
#pragma unroll
            for (int e = 0; e < EP; ++e) g[e] = e < E ? dl[row * E + e] : 0.f;   // experts past E have zero weights
        }
        f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < EP; ++e) {
            d += g[e] * wv[e];
            acc[e] += g[e] * xv;
        }
        store4(dx + row * H + c, d);
    };
    constexpr int UN = 4;   // rows per group; two groups are in flight, in two register sets that swap roles
    int64_t row = row_beg;
    raw_t ga[UN], gb[UN];
    auto load_group = [&](raw_t (&dst)[UN], int64_t r0) {
#pragma unroll
        for (int u = 0; u < UN; ++u) dst[u] = load_raw(x + (r0 + u) * H + c);
    };
    auto do_group = [&](raw_t (&src)[UN], int64_t r0) {
#pragma unroll
        for (int u = 0; u < UN; ++u) one_row(r0 + u, src[u]);
    };
    bool have_a = row + UN <= row_end;   // every condition here is block-uniform
    if (have_a) load_group(ga, row);
#pragma unroll 1
    while (have_a) {
        const bool have_b = row + 2 * UN <= row_end;
        if (have_b) load_group(gb, row + UN);
        do_group(ga, row);
        row += UN;
        if (!have_b) break;
        have_a = row + 2 * UN <= row_end;
        if (have_a) load_group(ga, row + UN);
        do_group(gb, row);
        row += UN;
    }
#pragma unroll 1
    for (; row < row_end; ++row) one_row(row, load_raw(x + row * H + c));
    for (int r = 1; r < groups; ++r) {   // set 0 collects the others in set order
        if (grp == r && active) {
#pragma unroll
            for (int e = 0; e < EP; ++e)
                if (e < E) *reinterpret_cast<f32x4*>(set_sum + e * cols_per_block + cl) = acc[e];
        }
        __syncthreads();
        if (grp == 0 && active) {
#pragma unroll
            for (int e = 0; e < EP; ++e)
                if (e < E) acc[e] += *reinterpret_cast<const f32x4*>(set_sum + e * cols_per_block + cl);
        }
        __syncthreads();
    }
    if (grp != 0 || !active) return;
    float* out = part + (int64_t)bx * E * H;
#pragma unroll
    for (int e = 0; e < EP; ++e)
        if (e < E) *reinterpret_cast<f32x4*>(out + (int64_t)e * H + c) = acc[e];
}

// dW_r[i] = sum_b part[b][i], the work of block `job` of kReduceThreads threads: kSegs threads share an
// output (4 floats), each sums a contiguous range of blocks in order, and the kSegs sums are added in
// segment order.
constexpr int kSegs = 64, kReduceThreads = 256;
constexpr int kReduceCols = (kReduceThreads / kSegs) * 4;   // outputs per block
__device__ __forceinline__ void router_dw_reduce_block(const float* __restrict__ part, int nblocks, int64_t EH,
                                                       float* __restrict__ d_w, int64_t job) {
    __shared__ f32x4 seg_sum[kSegs][kReduceThreads / kSegs];
    const int col = threadIdx.x % (kReduceThreads / kSegs), seg = threadIdx.x / (kReduceThreads / kSegs);
    const int64_t i = (job * (kReduceThreads / kSegs) + col) * 4;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < EH) {
        const int per = (nblocks + kSegs - 1) / kSegs;
        const int b1 = (seg + 1) * per < nblocks ? (seg + 1) * per : nblocks;
        for (int b = seg * per; b < b1; ++b) s += *reinterpret_cast<const f32x4*>(part + (int64_t)b * EH + i);
    }
    seg_sum[seg][col] = s;
    __syncthreads();
    if (seg == 0 && i < EH) {
        f32x4 t = seg_sum[0][col];
#pragma unroll
        for (int q = 1; q < kSegs; ++q) t += seg_sum[q][col];
        *reinterpret_cast<f32x4*>(d_w + i) = t;
    }
}

}  // namespace mts_rl
