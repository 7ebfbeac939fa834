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

#include <math.h>

namespace {

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 256;
constexpr float kLogFloor = -20.72326583694641f;  // log(1e-9): the entropy clamps p at 1e-9

template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, MTS_WAVE);
    return v;
}
template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MTS_WAVE));
    return v;
}

template <int EP, int G>
struct RowState {
    float l[EP];
    float p[EP];
    float m, s, L;
};

template <int EP, int G>
__device__ __forceinline__ void load_row(const float* __restrict__ logits, int64_t row, int E, int g,
                                         RowState<EP, G>& r) {
    const float* src = logits + row * (int64_t)E;
    if (G == 1 && EP == 8 && E == 8) {
        const f32x4* v = reinterpret_cast<const f32x4*>(src);
        f32x4 a = v[0], b = v[1];
        r.l[0] = a[0]; r.l[1] = a[1]; r.l[2] = a[2]; r.l[3] = a[3];
        r.l[4 % EP] = b[0]; r.l[5 % EP] = b[1]; r.l[6 % EP] = b[2]; r.l[7 % EP] = b[3];
    } else {
#pragma unroll
        for (int j = 0; j < EP; ++j) {
            int e = j * G + g;
            r.l[j] = (e < E) ? src[e] : -INFINITY;
        }
    }
    float m = r.l[0];
#pragma unroll
    for (int j = 1; j < EP; ++j) m = fmaxf(m, r.l[j]);
    m = group_max<G>(m);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < EP; ++j) {
        r.p[j] = expf(r.l[j] - m);
        s += r.p[j];
    }
    s = group_sum<G>(s);
    float inv = 1.0f / s;
#pragma unroll
    for (int j = 0; j < EP; ++j) r.p[j] *= inv;
    r.m = m;
    r.s = s;
    r.L = m + logf(s);
}

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

        uint32_t taken = 0;
#pragma unroll
        for (int j = 0; j < EP; ++j)
            if (j * G + g >= E) taken |= 1u << j;

        float sel_p[MTS_MAX_TOP_K];
        int sel_e[MTS_MAX_TOP_K];
        float mass = 0.f;
#pragma unroll
        for (int k = 0; k < MTS_MAX_TOP_K; ++k) {
            sel_p[k] = 0.f;
            sel_e[k] = 0;
            if (k < K) {
                float bv = -INFINITY;
                int be = 0x7fffffff;
#pragma unroll
                for (int j = 0; j < EP; ++j) {
                    int e = j * G + g;
                    bool free_slot = !((taken >> j) & 1u);
                    if (free_slot && (r.l[j] > bv || (r.l[j] == bv && e < be))) {
                        bv = r.l[j];
                        be = e;
                    }
                }
#pragma unroll
                for (int o = G / 2; o > 0; o >>= 1) {
                    float ov = __shfl_xor(bv, o, MTS_WAVE);
                    int oe = __shfl_xor(be, o, MTS_WAVE);
                    if (ov > bv || (ov == bv && oe < be)) {
                        bv = ov;
                        be = oe;
                    }
                }
                if (be % G == g) taken |= 1u << (be / G);
#pragma unroll
                for (int j = 0; j < EP; ++j) csum[j] += (live && j * G + g == be) ? 1 : 0;
                float pk = expf(bv - r.m) / r.s;
                sel_p[k] = pk;
                sel_e[k] = be;
                mass += pk;
            }
        }
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

// One block: wave w reduces columns w, w+4, ...; lanes stride over the per-block
// partials and the lane sums meet in a fixed shuffle tree (bit-stable).  Also the routes per
// expert and, if asked for, the load-balancing term E * sum_e (routes_e / routes) * mean_prob_e.
__global__ __launch_bounds__(kThreads) void router_stats_kernel(
    const float* __restrict__ partial, const int32_t* __restrict__ partial_counts, int nblocks, int E,
    float inv_t, float inv_routes, float* __restrict__ prob_mean, float* __restrict__ z_loss,
    float* __restrict__ entropy, int32_t* __restrict__ counts, float* __restrict__ load_balance,
    float* __restrict__ load_stats) {
    __shared__ float prod[MTS_MAX_EXPERTS];   // fraction of routes x mean probability, per expert
    __shared__ float share[MTS_MAX_EXPERTS];  // fraction of routes, per expert
    __shared__ int routes_of[MTS_MAX_EXPERTS];
    __shared__ float entropy_s;
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    for (int i = wave; i < E + 2; i += kThreads / MTS_WAVE) {
        float v = 0.f;
        for (int b = lane; b < nblocks; b += MTS_WAVE) v += partial[(int64_t)b * (E + 2) + i];
        v = wave_sum(v) * inv_t;
        int c = 0;
        if (i < E) {
            for (int b = lane; b < nblocks; b += MTS_WAVE) c += partial_counts[(int64_t)b * E + i];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, MTS_WAVE);
        }
        if (lane == 0) {
            if (i < E) {
                prob_mean[i] = v;
                prod[i] = (float)c * inv_routes * v;
                share[i] = (float)c * inv_routes;
                routes_of[i] = c;
                if (counts) counts[i] = c;
            } else if (i == E) {
                z_loss[0] = v;
            } else {
                entropy[0] = v;
                entropy_s = v;
            }
        }
    }
    if (!load_balance && !load_stats) return;
    __syncthreads();
    // E * sum_e f_e * pbar_e, summed in a fixed order by one wave
    if (wave == 0 && load_balance) {
        float v = 0.f;
        for (int e = lane; e < E; e += MTS_WAVE) v += prod[e];
        v = wave_sum(v);
        if (lane == 0) load_balance[0] = (float)E * v;
    }
    // load statistics of the router module (minitrain/model/moe_router.py:113-135) from the route
    // fractions: [0,E) the fractions, then the largest and smallest route count, the coefficient
    // of variation (population standard deviation x E), largest fraction x E, the number of
    // experts without a route, a zero (the dropped-route fraction of dropless routing) and the
    // entropy over log E
    if (wave == 1 % (kThreads / MTS_WAVE) && load_stats) {
        float sum = 0.f, hi = 0.f, dead = 0.f;
        int most = 0, fewest = 0x7fffffff;
        for (int e = lane; e < E; e += MTS_WAVE) {
            const float f = share[e];
            load_stats[e] = f;
            sum += f;
            hi = fmaxf(hi, f);
            most = max(most, routes_of[e]);
            fewest = min(fewest, routes_of[e]);
            dead += routes_of[e] == 0 ? 1.f : 0.f;
        }
        sum = wave_sum(sum);
        dead = wave_sum(dead);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            hi = fmaxf(hi, __shfl_xor(hi, o, MTS_WAVE));
            most = max(most, __shfl_xor(most, o, MTS_WAVE));
            fewest = min(fewest, __shfl_xor(fewest, o, MTS_WAVE));
        }
        const float mean = sum / (float)E;
        float var = 0.f;
        for (int e = lane; e < E; e += MTS_WAVE) {
            const float d = share[e] - mean;
            var += d * d;
        }
        var = wave_sum(var) / (float)E;
        if (lane == 0) {
            load_stats[E] = (float)most;
            load_stats[E + 1] = (float)fewest;
            load_stats[E + 2] = sqrtf(var) * (float)E;
            load_stats[E + 3] = hi * (float)E;
            load_stats[E + 4] = dead;
            load_stats[E + 5] = 0.f;
            load_stats[E + 6] = entropy_s / (E > 1 ? logf((float)E) : 1.0f);
        }
    }
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
        float dp[EP], extra[EP];
#pragma unroll
        for (int j = 0; j < EP; ++j) {
            dp[j] = gp[j];
            extra[j] = 0.f;
        }
        float wdot = 0.f;
        if (normalize) {
            for (int k = 0; k < K; ++k) wdot += weights[rr * K + k] * grad_w(rr * K + k);
        }
        for (int k = 0; k < K; ++k) {
            int e = indices[rr * K + k];
            float gw = grad_w(rr * K + k);
            float w = weights[rr * K + k];
#pragma unroll
            for (int j = 0; j < EP; ++j) {
                if (j * G + g == e) {
                    if (normalize) extra[j] += w * (gw - wdot);
                    else dp[j] += gw;
                }
            }
        }
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < EP; ++j) dot += r.p[j] * dp[j];
        dot = group_sum<G>(dot);
        if (live) {
            float* dst = dlogits + row * (int64_t)E;
            float o[EP];
#pragma unroll
            for (int j = 0; j < EP; ++j) o[j] = r.p[j] * (dp[j] - dot) + gz * r.L * r.p[j] + extra[j];
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
