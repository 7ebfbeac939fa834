// Per-row arithmetic of the router post-process (softmax of a row of fp32 logits held by G
// adjacent lanes, top-k on the logits with the lower expert index winning ties, the gradient
// of a row) and the one-block reduction of the routing statistics.  Shared by the stand-alone
// post-process kernels and the kernels that chain the router projection to them.
#pragma once

#include "mts_common.h"

#include <math.h>

namespace mts_router {

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

// softmax of the row whose logits are in r.l (slots past E hold -inf): p, the row maximum, the
// sum of exponentials and the log-partition
template <int EP, int G>
__device__ __forceinline__ void softmax_row(RowState<EP, G>& r) {
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
    softmax_row<EP, G>(r);
}


// K rounds of arg-max over the logits of a row (ties to the lower expert index).  `taken` has a
// bit per slot j of this lane (expert j*G + g); sel_e / sel_p get the expert and its softmax
// probability per rank, mass the sum of the selected probabilities.
template <int EP, int G>
__device__ __forceinline__ void select_top_k(const RowState<EP, G>& r, int E, int K, int g,
                                             float (&sel_p)[MTS_MAX_TOP_K], int (&sel_e)[MTS_MAX_TOP_K], float& mass) {
    uint32_t taken = 0;
#pragma unroll
    for (int j = 0; j < EP; ++j)
        if (j * G + g >= E) taken |= 1u << j;
    mass = 0.f;
#pragma unroll
    for (int k = 0; k < MTS_MAX_TOP_K; ++k) {
        sel_p[k] = 0.f;
        sel_e[k] = -1;
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
            float pk = expf(bv - r.m) / r.s;
            sel_p[k] = pk;
            sel_e[k] = be;
            mass += pk;
        }
    }
}

// Gradient of a row's logits.  dp: gradient that reaches the row's probabilities through the mean
// probability (and the load-balancing term), per slot of this lane; gz: gradient of the z-loss
// times 2/T; weights / indices / grad_w(k): the row's selected weights, experts and weight gradients.
template <int EP, int G, class GradW>
__device__ __forceinline__ void row_logit_gradient(const RowState<EP, G>& r, const float (&gp)[EP], float gz, int K,
                                                   int normalize, int g, const float* __restrict__ weights,
                                                   const int32_t* __restrict__ indices, GradW grad_w, float (&o)[EP]) {
    float dp[EP], extra[EP];
#pragma unroll
    for (int j = 0; j < EP; ++j) {
        dp[j] = gp[j];
        extra[j] = 0.f;
    }
    float wdot = 0.f;
    if (normalize) {
        for (int k = 0; k < K; ++k) wdot += weights[k] * grad_w(k);
    }
    for (int k = 0; k < K; ++k) {
        int e = indices[k];
        float gw = grad_w(k);
        float w = weights[k];
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
#pragma unroll
    for (int j = 0; j < EP; ++j) o[j] = r.p[j] * (dp[j] - dot) + gz * r.L * r.p[j] + extra[j];
}

// ---- reduction of the routing statistics (one block) ----------------------------------------
// Column i < E of the per-block partials is the probability mass of expert i, column E the sum
// of squared log-partitions, column E+1 the entropy sum.  Sums run in a fixed order (bit-stable).
struct StatsShared {
    float prod[MTS_MAX_EXPERTS];    // fraction of routes x mean probability, per expert
    float share[MTS_MAX_EXPERTS];   // fraction of routes, per expert
    int routes_of[MTS_MAX_EXPERTS];
    float entropy_s;
};

// what one thread does with the mean `v` of column i and, for i < E, the routes `c` of expert i
__device__ __forceinline__ void stats_column(StatsShared& sh, int i, float v, int c, int E, float inv_routes,
                                             float* __restrict__ prob_mean, float* __restrict__ z_loss,
                                             float* __restrict__ entropy, int32_t* __restrict__ counts) {
    if (i < E) {
        prob_mean[i] = v;
        sh.prod[i] = (float)c * inv_routes * v;
        sh.share[i] = (float)c * inv_routes;
        sh.routes_of[i] = c;
        if (counts) counts[i] = c;
    } else if (i == E) {
        z_loss[0] = v;
    } else {
        entropy[0] = v;
        sh.entropy_s = v;
    }
}

// After a block barrier behind the stats_column calls: wave `lb_wave` writes the load-balancing term
// E * sum_e (routes_e / routes) * mean_prob_e, wave `ls_wave` the load statistics of the router module
// (minitrain/model/moe_router.py:113-135) from the route fractions: [0,E) the fractions, then the
// largest and smallest route count, the coefficient of variation (population standard deviation x E),
// largest fraction x E, the number of experts without a route, a zero (the dropped-route fraction of
// dropless routing) and the entropy over log E.  Either output may be NULL.
__device__ __forceinline__ void stats_finalize(const StatsShared& sh, int wave, int lb_wave, int ls_wave, int E,
                                               float* __restrict__ load_balance, float* __restrict__ load_stats) {
    const int lane = threadIdx.x % MTS_WAVE;
    if (wave == lb_wave && load_balance) {
        float v = 0.f;
        for (int e = lane; e < E; e += MTS_WAVE) v += sh.prod[e];
        v = wave_sum(v);
        if (lane == 0) load_balance[0] = (float)E * v;
    }
    if (wave == ls_wave && load_stats) {
        float sum = 0.f, hi = 0.f, dead = 0.f;
        int most = 0, fewest = 0x7fffffff;
        for (int e = lane; e < E; e += MTS_WAVE) {
            const float f = sh.share[e];
            load_stats[e] = f;
            sum += f;
            hi = fmaxf(hi, f);
            most = max(most, sh.routes_of[e]);
            fewest = min(fewest, sh.routes_of[e]);
            dead += sh.routes_of[e] == 0 ? 1.f : 0.f;
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
            const float d = sh.share[e] - mean;
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
            load_stats[E + 6] = sh.entropy_s / (E > 1 ? logf((float)E) : 1.0f);
        }
    }
}

// mean of column i of the partials over nblocks blocks: lanes stride over the blocks, the lane sums
// meet in a fixed shuffle tree
__device__ __forceinline__ float stats_column_mean(const float* __restrict__ partial, int nblocks, int E, int i,
                                                   float inv_t) {
    const int lane = threadIdx.x % MTS_WAVE;
    float v = 0.f;
    for (int b = lane; b < nblocks; b += MTS_WAVE) v += partial[(int64_t)b * (E + 2) + i];
    return wave_sum(v) * inv_t;
}

// The whole reduction by one block of NWAVES waves: wave w takes columns w, w + NWAVES, ...
template <int NWAVES>
__device__ __forceinline__ void stats_block(
    const float* __restrict__ partial, const int32_t* __restrict__ partial_counts, int nblocks, int E,
    float inv_t, float inv_routes, float* __restrict__ prob_mean, float* __restrict__ z_loss,
    float* __restrict__ entropy, int32_t* __restrict__ counts, float* __restrict__ load_balance,
    float* __restrict__ load_stats, int wave) {
    __shared__ StatsShared sh;
    const int lane = threadIdx.x % MTS_WAVE;
    for (int i = wave; i < E + 2; i += NWAVES) {
        const float v = stats_column_mean(partial, nblocks, E, i, inv_t);
        int c = 0;
        if (i < E) {
            for (int b = lane; b < nblocks; b += MTS_WAVE) c += partial_counts[(int64_t)b * E + i];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, MTS_WAVE);
        }
        if (lane == 0) stats_column(sh, i, v, c, E, inv_routes, prob_mean, z_loss, entropy, counts);
    }
    if (!load_balance && !load_stats) return;   // block-uniform
    __syncthreads();
    stats_finalize(sh, wave, 0, 1 % NWAVES, E, load_balance, load_stats);
}

}  // namespace mts_router
