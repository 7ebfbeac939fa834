// Router post-process for fp32 logits: softmax, top-k on the logits with the
// lower expert index winning a tie, selected-weight normalisation, mean
// probability, z-loss and entropy; and its backward.
//
// A row of E logits is held by G adjacent lanes, EP values per lane
// (expert e = j*G + g).  E <= 8 is one thread per row with two 16-byte loads.
// Row statistics are summed per lane over a grid-stride loop, reduced over the
// wave with a fixed shuffle tree, over the block through LDS and over blocks by a
// second one-block kernel, so that results are bit-stable from run to run.
#include "mts_common.h"
#include "mts_router_row.h"

namespace {

using namespace mts_router;

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 256;
template <int EP, int G>
__global__ __launch_bounds__(kThreads) void router_fwd_kernel(
    const float* __restrict__ logits, int64_t T, int E, int K, int normalize,
    float* __restrict__ weights, int32_t* __restrict__ indices, float* __restrict__ partial,
    int32_t* __restrict__ partial_counts, void* __restrict__ weights_act, int act_dtype) {
    constexpr int ROWS = kThreads / G;
    const int g = threadIdx.x % G;
    const int rl = threadIdx.x / G;
    float psum[EP];
    int csum[EP];   // routes to the experts this lane owns (slot j is expert j*G + g)
#pragma unroll
    for (int j = 0; j < EP; ++j) {
        psum[j] = 0.f;
        csum[j] = 0;
    }
    float zsum = 0.f, hsum = 0.f;

    for (int64_t row0 = (int64_t)blockIdx.x * ROWS; row0 < T; row0 += (int64_t)gridDim.x * ROWS) {
        int64_t row = row0 + rl;
        bool live = row < T;
        RowState<EP, G> r;
        load_row<EP, G>(logits, live ? row : 0, E, g, r);

        float sel_p[MTS_MAX_TOP_K];
        int sel_e[MTS_MAX_TOP_K];
        float mass;
        select_top_k<EP, G>(r, E, K, g, sel_p, sel_e, mass);
#pragma unroll
        for (int k = 0; k < MTS_MAX_TOP_K; ++k)
#pragma unroll
            for (int j = 0; j < EP; ++j) csum[j] += (live && k < K && j * G + g == sel_e[k]) ? 1 : 0;
        if (live && g == 0) {
            float inv = normalize ? 1.0f / fmaxf(mass, 1.1920928955078125e-07f) : 1.0f;
#pragma unroll
            for (int k = 0; k < MTS_MAX_TOP_K; ++k) {
                if (k < K) {
                    const float wk = sel_p[k] * inv;
                    weights[row * K + k] = wk;
                    indices[row * K + k] = sel_e[k];
                    // the copy the MoE block hands to fused_moe: rounded once, as tensor.to() rounds
                    if (weights_act) {
                        if (act_dtype == MTS_BF16) reinterpret_cast<bf16_t*>(weights_act)[row * K + k] = (bf16_t)wk;
                        else reinterpret_cast<mts_f16_t*>(weights_act)[row * K + k] = (mts_f16_t)wk;
                    }
                }
            }
        }
        if (live) {
#pragma unroll
            for (int j = 0; j < EP; ++j) {
                psum[j] += r.p[j];
                // p * log(max(p, 1e-9)); p == 0 (padding or underflow) contributes 0
                float lp = fmaxf(r.l[j] - r.L, kLogFloor);
                hsum -= (r.p[j] > 0.f) ? r.p[j] * lp : 0.f;
            }
            if (g == 0) zsum += r.L * r.L;
        }
    }

    // wave: sum lanes that hold the same experts (same g)
#pragma unroll
    for (int j = 0; j < EP; ++j) {
#pragma unroll
        for (int o = 32; o >= G; o >>= 1) psum[j] += __shfl_xor(psum[j], o, MTS_WAVE);
    }
    zsum = wave_sum(zsum);
    hsum = wave_sum(hsum);
#pragma unroll
    for (int j = 0; j < EP; ++j) {
#pragma unroll
        for (int o = 32; o >= G; o >>= 1) csum[j] += __shfl_xor(csum[j], o, MTS_WAVE);
    }

    __shared__ float red[kThreads / MTS_WAVE][EP * G + 2];
    __shared__ int32_t cred[kThreads / MTS_WAVE][EP * G];
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    if (lane < G) {
#pragma unroll
        for (int j = 0; j < EP; ++j) {
            red[wave][j * G + lane] = psum[j];
            cred[wave][j * G + lane] = csum[j];
        }
    }
    if (lane == 0) {
        red[wave][EP * G] = zsum;
        red[wave][EP * G + 1] = hsum;
    }
    __syncthreads();
    float* out = partial + (int64_t)blockIdx.x * (E + 2);
    for (int i = threadIdx.x; i < E + 2; i += kThreads) {
        int src = i < E ? i : EP * G + (i - E);
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kThreads / MTS_WAVE; ++w) v += red[w][src];
        out[i] = v;
    }
    int32_t* cout = partial_counts + (int64_t)blockIdx.x * E;
    for (int i = threadIdx.x; i < E; i += kThreads) {
        int32_t v = 0;
#pragma unroll
        for (int w = 0; w < kThreads / MTS_WAVE; ++w) v += cred[w][i];
        cout[i] = v;
    }
}

__global__ __launch_bounds__(kThreads) void router_stats_kernel(
    const float* __restrict__ partial, const int32_t* __restrict__ partial_counts, int nblocks, int E,
    float inv_t, float inv_routes, float* __restrict__ prob_mean, float* __restrict__ z_loss,
    float* __restrict__ entropy, int32_t* __restrict__ counts, float* __restrict__ load_balance,
    float* __restrict__ load_stats) {
    stats_block<kThreads / MTS_WAVE>(partial, partial_counts, nblocks, E, inv_t, inv_routes, prob_mean, z_loss, entropy,
                                     counts, load_balance, load_stats, threadIdx.x / MTS_WAVE);
}

template <int EP, int G>
__global__ __launch_bounds__(kThreads) void router_bwd_kernel(
    const float* __restrict__ logits, const float* __restrict__ weights,
    const int32_t* __restrict__ indices, const float* __restrict__ g_w, const void* __restrict__ g_w_act, int act_dtype,
    const float* __restrict__ g_p, const float* __restrict__ g_z, const float* __restrict__ g_lb,
    const int32_t* __restrict__ counts, int64_t T, int E, int K,
    int normalize, float* __restrict__ dlogits) {
    // gradient of the routing weights: the fp32 output's and the activation-dtype copy's, either may be absent
    auto grad_w = [&](int64_t i) {
        float v = g_w ? g_w[i] : 0.f;
        if (g_w_act)
            v += act_dtype == MTS_BF16 ? (float)reinterpret_cast<const bf16_t*>(g_w_act)[i]
                                       : (float)reinterpret_cast<const mts_f16_t*>(g_w_act)[i];
        return v;
    };
    constexpr int ROWS = kThreads / G;
    const int g = threadIdx.x % G;
    const int rl = threadIdx.x / G;
    const float inv_t = 1.0f / (float)T;
    const float gz = g_z ? g_z[0] * 2.0f * inv_t : 0.f;   // every gradient input may be absent (null = zeros)
    float gp[EP];
#pragma unroll
    for (int j = 0; j < EP; ++j) {
        int e = j * G + g;
        gp[j] = (g_p && e < E) ? g_p[e] * inv_t : 0.f;
        // load-balancing term: d/d(mean_prob_e) = E * routes_e / routes (the route fractions carry no gradient)
        if (g_lb && e < E) gp[j] += g_lb[0] * (float)E * ((float)counts[e] / ((float)T * (float)K)) * inv_t;
    }
    for (int64_t row0 = (int64_t)blockIdx.x * ROWS; row0 < T; row0 += (int64_t)gridDim.x * ROWS) {
        int64_t row = row0 + rl;
        bool live = row < T;
        int64_t rr = live ? row : 0;
        RowState<EP, G> r;
        load_row<EP, G>(logits, rr, E, g, r);
        float o[EP];
        row_logit_gradient<EP, G>(r, gp, gz, K, normalize, g, weights + rr * K, indices + rr * K,
                                  [&](int k) { return grad_w(rr * K + k); }, o);
        if (live) {
            float* dst = dlogits + row * (int64_t)E;
            if (G == 1 && EP == 8 && E == 8) {
                f32x4* v = reinterpret_cast<f32x4*>(dst);
                v[0] = f32x4{o[0], o[1], o[2], o[3]};
                v[1] = f32x4{o[4 % EP], o[5 % EP], o[6 % EP], o[7 % EP]};
            } else {
#pragma unroll
                for (int j = 0; j < EP; ++j) {
                    int e = j * G + g;
                    if (e < E) dst[e] = o[j];
                }
            }
        }
    }
}

int grid_for(int64_t T, int G) {
    int64_t rows = kThreads / G;
    int64_t b = (T + rows - 1) / rows;
    return (int)(b < kMaxBlocks ? b : kMaxBlocks);
}

// lanes per row: E <= 8 -> 1, then the smallest power of two with 8*G >= E; 16 per lane above 512
int lanes_for(int E) {
    int G = 1;
    while (G < 64 && 8 * G < E) G <<= 1;
    return G;
}

#define MTS_ROUTER_DISPATCH(FN, ...)                                              \
    do {                                                                          \
        if (E > 512) { FN<16, 64> __VA_ARGS__; break; }                           \
        switch (lanes_for(E)) {                                                   \
            case 1: FN<8, 1> __VA_ARGS__; break;                                  \
            case 2: FN<8, 2> __VA_ARGS__; break;                                  \
            case 4: FN<8, 4> __VA_ARGS__; break;                                  \
            case 8: FN<8, 8> __VA_ARGS__; break;                                  \
            case 16: FN<8, 16> __VA_ARGS__; break;                                \
            case 32: FN<8, 32> __VA_ARGS__; break;                                \
            default: FN<8, 64> __VA_ARGS__; break;                                \
        }                                                                         \
    } while (0)

int check_router(const void* logits, int64_t T, int E, int K) {
    if (!logits) return MTS_ERR_NULL;
    if (T <= 0 || T > (int64_t)1 << 40 || E < 1 || E > MTS_MAX_EXPERTS || K < 1 || K > E ||
        K > MTS_MAX_TOP_K)
        return MTS_ERR_SHAPE;
    if (E == 8 && !mts_aligned16(logits)) return MTS_ERR_ALIGN;
    return MTS_OK;
}

}  // namespace

extern "C" int64_t mts_router_workspace_bytes(int64_t T, int E) {
    (void)T;
    return (int64_t)kMaxBlocks * (2 * E + 2) * (int64_t)sizeof(float);   // float partials, then int32 route counts
}

extern "C" int mts_router_fwd(const float* logits, int64_t T, int E, int K, int normalize,
                              float* weights, int32_t* indices, float* prob_mean, float* z_loss,
                              float* entropy, int32_t* counts, float* load_balance, float* load_stats,
                              void* weights_act, int act_dtype, void* workspace, int64_t workspace_bytes,
                              void* stream) {
    int rc = check_router(logits, T, E, K);
    if (rc) return rc;
    if (weights_act && act_dtype != MTS_BF16 && act_dtype != MTS_F16) return MTS_ERR_DTYPE;
    if (!weights || !indices || !prob_mean || !z_loss || !entropy || !workspace) return MTS_ERR_NULL;
    if ((counts || load_balance || load_stats) && T * (int64_t)K > 0x7fffffffLL) return MTS_ERR_SHAPE;   // int32 route counts
    if (workspace_bytes < mts_router_workspace_bytes(T, E)) return MTS_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    float* partial = (float*)workspace;
    int32_t* partial_counts = (int32_t*)(partial + (int64_t)kMaxBlocks * (E + 2));
    int G = E > 512 ? 64 : lanes_for(E);
    int grid = grid_for(T, G);
    MTS_ROUTER_DISPATCH(router_fwd_kernel, <<<grid, kThreads, 0, s>>>(logits, T, E, K, normalize, weights, indices,
                                                                      partial, partial_counts, weights_act, act_dtype));
    MTS_CHECK_LAUNCH();
    router_stats_kernel<<<1, kThreads, 0, s>>>(partial, partial_counts, grid, E, 1.0f / (float)T,
                                               1.0f / ((float)T * (float)K), prob_mean, z_loss, entropy, counts,
                                               load_balance, load_stats);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int mts_router_bwd(const float* logits, const float* weights, const int32_t* indices,
                              const float* g_weights, const void* g_weights_act, int act_dtype, const float* g_prob_mean,
                              const float* g_z_loss, const float* g_load_balance, const int32_t* counts,
                              int64_t T, int E, int K, int normalize, float* dlogits, void* stream) {
    int rc = check_router(logits, T, E, K);
    if (rc) return rc;
    if (!weights || !indices || !dlogits) return MTS_ERR_NULL;
    if (g_load_balance && !counts) return MTS_ERR_NULL;
    if (g_weights_act && act_dtype != MTS_BF16 && act_dtype != MTS_F16) return MTS_ERR_DTYPE;
    if (E == 8 && !mts_aligned16(dlogits)) return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    int G = E > 512 ? 64 : lanes_for(E);
    int grid = grid_for(T, G);
    MTS_ROUTER_DISPATCH(router_bwd_kernel,
                        <<<grid, kThreads, 0, s>>>(logits, weights, indices, g_weights, g_weights_act, act_dtype, g_prob_mean,
                                                   g_z_loss, g_load_balance, counts, T, E, K, normalize,
                                                   dlogits));
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
