// Router projection around the post-process kernels: logits = float(x) W_r^T in fp32 and its
// backward (dx in the activation dtype, dW_r in fp32).  x is read in its own dtype, so no fp32
// copy of the activations is made; every sum runs in a fixed order (no float atomics).
// All three kernels are VALU/HBM bound: 2*T*H*E FLOP forward, twice that backward.
#include "mts_common.h"

namespace {

constexpr int kRows = 4;         // rows per wave in the forward kernel
constexpr int kFwdThreads = 256;
constexpr int kSegs = 8;         // segments of the partial sums in the reduction kernel

__device__ __forceinline__ f32x4 load4(const bf16_t* p) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
    f32x4 r = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
    return r;
}
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ void store4(bf16_t* p, f32x4 v) {
    bf16x4 o = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
    *reinterpret_cast<bf16x4*>(p) = o;
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }

// One wave computes kRows rows: a lane owns 4 consecutive columns of every 256-column slab,
// the weights of a slab are read once per kRows rows (they stay in L1/L2), and the E partial
// dot products of a row are summed across the wave with a fixed shuffle tree.
template <typename XT, int EP>
__global__ __launch_bounds__(kFwdThreads) void router_logits_fwd_kernel(const XT* __restrict__ x,
                                                                         const float* __restrict__ w, int64_t T,
                                                                         int H, int E, float* __restrict__ logits) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int64_t wave0 = (int64_t)blockIdx.x * (kFwdThreads / MTS_WAVE) + threadIdx.x / MTS_WAVE;
    const int64_t nwaves = (int64_t)gridDim.x * (kFwdThreads / MTS_WAVE);
    for (int64_t r0 = wave0 * kRows; r0 < T; r0 += nwaves * kRows) {
        float acc[kRows][EP];
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int e = 0; e < EP; ++e) acc[r][e] = 0.f;
        for (int c = lane * 4; c < H; c += MTS_WAVE * 4) {
            f32x4 xv[kRows];
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                xv[r] = r0 + r < T ? load4(x + (r0 + r) * H + c) : z;
            }
#pragma unroll
            for (int e = 0; e < EP; ++e) {
                if (e < E) {
                    const f32x4 wv = *reinterpret_cast<const f32x4*>(w + (int64_t)e * H + c);
#pragma unroll
                    for (int r = 0; r < kRows; ++r)
                        acc[r][e] += xv[r][0] * wv[0] + xv[r][1] * wv[1] + xv[r][2] * wv[2] + xv[r][3] * wv[3];
                }
            }
        }
        float mine = 0.f;
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int e = 0; e < EP; ++e) {
                const float v = wave_sum(acc[r][e]);
                if (lane == r * EP + e) mine = v;
            }
        static_assert(kRows * EP <= MTS_WAVE, "one lane per output of the wave");
        const int r = lane / EP, e = lane % EP;
        if (lane < kRows * EP && e < E && r0 + r < T) logits[(r0 + r) * E + e] = mine;
    }
}

// Backward: a thread owns 4 consecutive columns.  Per row it forms dx (in the activation
// dtype) from the row's E logit gradients and its weight columns, and adds the row's
// contribution to its E x 4 block of dW_r; every block writes its partial dW_r to the
// workspace, and the reduction kernel sums the partials in block order.
template <typename XT, int EP>
__global__ __launch_bounds__(256) void router_logits_bwd_kernel(const float* __restrict__ dl,
                                                                 const XT* __restrict__ x,
                                                                 const float* __restrict__ w, int64_t T, int H,
                                                                 int E, int rows_per_block, XT* __restrict__ dx,
                                                                 float* __restrict__ part) {
    const int c = threadIdx.x * 4;
    if (c >= H) return;
    f32x4 wv[EP], acc[EP];
#pragma unroll
    for (int e = 0; e < EP; ++e) {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        wv[e] = e < E ? *reinterpret_cast<const f32x4*>(w + (int64_t)e * H + c) : z;
        acc[e] = z;
    }
    const int64_t row_beg = (int64_t)blockIdx.x * rows_per_block;
    const int64_t row_end = row_beg + rows_per_block < T ? row_beg + rows_per_block : T;
    for (int64_t row = row_beg; row < row_end; ++row) {
        const f32x4 xv = load4(x + row * H + c);
        f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < EP; ++e) {
            if (e < E) {
                const float g = dl[row * E + e];   // the same address for every thread of the block
                d += g * wv[e];
                acc[e] += g * xv;
            }
        }
        store4(dx + row * H + c, d);
    }
    float* out = part + (int64_t)blockIdx.x * E * H;
#pragma unroll
    for (int e = 0; e < EP; ++e)
        if (e < E) *reinterpret_cast<f32x4*>(out + (int64_t)e * H + c) = acc[e];
}

// dW_r[i] = sum_b part[b][i]: kSegs threads share an output (4 floats), each sums a contiguous
// range of blocks in order, and the kSegs sums are added in segment order.
__global__ __launch_bounds__(256) void router_dw_reduce_kernel(const float* __restrict__ part, int nblocks,
                                                               int64_t EH, float* __restrict__ d_w) {
    __shared__ f32x4 seg_sum[kSegs][256 / kSegs];
    const int col = threadIdx.x % (256 / kSegs), seg = threadIdx.x / (256 / kSegs);
    const int64_t i = ((int64_t)blockIdx.x * (256 / kSegs) + col) * 4;
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

constexpr int kMaxE = 16;
constexpr int kBwdBlocks = 512;

int check(const void* x, const float* w, int64_t T, int H, int E, int act_dtype) {
    if (!x || !w) return MTS_ERR_NULL;
    if (T <= 0 || E < 1 || E > kMaxE || H < 4 || H % 4) return MTS_ERR_SHAPE;
    if (act_dtype != MTS_BF16 && act_dtype != MTS_F32) return MTS_ERR_DTYPE;
    if (!mts_aligned16(w) || (reinterpret_cast<uintptr_t>(x) & 15u)) return MTS_ERR_ALIGN;
    return MTS_OK;
}

int bwd_blocks(int64_t T) { return (int)(T < kBwdBlocks ? T : kBwdBlocks); }

}  // namespace

extern "C" int mts_router_logits_fwd(const void* x, const float* w_r, int64_t T, int H, int E, int act_dtype,
                                     float* logits, void* stream) {
    const int rc = check(x, w_r, T, H, E, act_dtype);
    if (rc != MTS_OK) return rc;
    if (!logits) return MTS_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    const int64_t groups = (T + kRows - 1) / kRows;
    int64_t blocks = (groups + 3) / 4;
    if (blocks > 256 * 8) blocks = 256 * 8;
    const dim3 grid((unsigned)blocks);
    if (act_dtype == MTS_BF16) {
        if (E <= 8) router_logits_fwd_kernel<bf16_t, 8><<<grid, kFwdThreads, 0, s>>>((const bf16_t*)x, w_r, T, H, E, logits);
        else router_logits_fwd_kernel<bf16_t, 16><<<grid, kFwdThreads, 0, s>>>((const bf16_t*)x, w_r, T, H, E, logits);
    } else {
        if (E <= 8) router_logits_fwd_kernel<float, 8><<<grid, kFwdThreads, 0, s>>>((const float*)x, w_r, T, H, E, logits);
        else router_logits_fwd_kernel<float, 16><<<grid, kFwdThreads, 0, s>>>((const float*)x, w_r, T, H, E, logits);
    }
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int64_t mts_router_logits_bwd_workspace_bytes(int64_t T, int H, int E) {
    if (T <= 0 || H <= 0 || E <= 0) return 0;
    return (int64_t)bwd_blocks(T) * E * H * (int64_t)sizeof(float);
}

extern "C" int mts_router_logits_bwd(const float* dlogits, const void* x, const float* w_r, int64_t T, int H,
                                     int E, int act_dtype, void* dx, float* d_w_r, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
    const int rc = check(x, w_r, T, H, E, act_dtype);
    if (rc != MTS_OK) return rc;
    if (!dlogits || !dx || !d_w_r || !workspace) return MTS_ERR_NULL;
    if (H > 1024) return MTS_ERR_SHAPE;   // one thread per 4 columns, one block per row
    if (workspace_bytes < mts_router_logits_bwd_workspace_bytes(T, H, E)) return MTS_ERR_WORKSPACE;
    if (!mts_aligned16(workspace) || !mts_aligned16(d_w_r) || (reinterpret_cast<uintptr_t>(dx) & 15u)) return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const int nb = bwd_blocks(T);
    const int rows_per_block = (int)((T + nb - 1) / nb);
    const int threads = ((H / 4 + MTS_WAVE - 1) / MTS_WAVE) * MTS_WAVE;
    float* part = (float*)workspace;
    if (act_dtype == MTS_BF16) {
        if (E <= 8) router_logits_bwd_kernel<bf16_t, 8><<<nb, threads, 0, s>>>(dlogits, (const bf16_t*)x, w_r, T, H, E, rows_per_block, (bf16_t*)dx, part);
        else router_logits_bwd_kernel<bf16_t, 16><<<nb, threads, 0, s>>>(dlogits, (const bf16_t*)x, w_r, T, H, E, rows_per_block, (bf16_t*)dx, part);
    } else {
        if (E <= 8) router_logits_bwd_kernel<float, 8><<<nb, threads, 0, s>>>(dlogits, (const float*)x, w_r, T, H, E, rows_per_block, (float*)dx, part);
        else router_logits_bwd_kernel<float, 16><<<nb, threads, 0, s>>>(dlogits, (const float*)x, w_r, T, H, E, rows_per_block, (float*)dx, part);
    }
    MTS_CHECK_LAUNCH();
    const int64_t EH = (int64_t)E * H;
    const int per_block = (256 / kSegs) * 4;
    // blocks of the backward kernel past the last row do not exist: nb * rows_per_block >= T and
    // every block has at least one row when nb <= T
    const int used = (int)((T + rows_per_block - 1) / rows_per_block);
    router_dw_reduce_kernel<<<(unsigned)((EH + per_block - 1) / per_block), 256, 0, s>>>(part, used, EH, d_w_r);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
