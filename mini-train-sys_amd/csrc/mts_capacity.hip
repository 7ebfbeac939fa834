// Capacity-limited routing: of the routes that chose expert e, the `capacity` routes with
// the largest router weights are kept; among equal weights the lower flat entry t*K+k is
// kept first.  Integer and comparison work only: the result is exact.
//
// The stable expert-major permutation of the routing metadata puts the entries of an
// expert into one segment, in ascending entry order.  One block per expert then finds the
// capacity-th largest weight of its segment with a radix select over order-preserving
// 32-bit keys (four passes of 8 bits, histogram in LDS), and a last pass in segment order
// ranks the entries that tie with that weight.
#include "mts_common.h"

namespace {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / MTS_WAVE;
constexpr int kUnroll = 4;
constexpr int kRegKeys = 32;   // segments of up to 32768 routes keep their keys in registers

// float -> unsigned key with the same order; -0 and +0 get the same key
__device__ __forceinline__ uint32_t order_key(float w) {
    uint32_t b = __float_as_uint(w);
    if (w == 0.0f) b = 0u;
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// One pass of the select over the keys of a thread: counts the digit at `shift` of the keys
// whose higher digits equal `prefix`.  Router weights share their leading bits, so most lanes
// of a wave hit the same bin in the first passes: the two most common digits of a wave are
// added once per wave.
__device__ __forceinline__ void count_digit(uint32_t* hist, bool count, uint32_t d, int lane) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint64_t todo = __ballot(count);
        if (!todo) break;
        const int leader = __ffsll((unsigned long long)todo) - 1;
        const uint32_t dl = (uint32_t)__shfl((int)d, leader, MTS_WAVE);
        const uint64_t same = __ballot(count && d == dl);
        if (lane == leader) atomicAdd(&hist[dl], (uint32_t)__popcll(same));
        count = count && d != dl;
    }
    if (count) atomicAdd(&hist[d], 1u);
}

// REGS: the segment has at most kRegKeys keys per thread and they stay in registers; otherwise
// they are written to `kseg` in the first pass and read back in the later ones (the same thread
// touches kseg[i] in every pass).  Position i of the segment belongs to thread i % kSelThreads.
template <bool REGS>
__device__ __forceinline__ void select_segment(const float* __restrict__ w, const int32_t* __restrict__ seg,
                                               uint32_t* __restrict__ kseg, int n, int e, uint32_t capacity,
                                               uint8_t* __restrict__ keep, int32_t* __restrict__ kept_index,
                                               uint32_t* hist, uint32_t* chosen, uint32_t* wave_ties,
                                               uint32_t* tie_table) {
    const int tid = threadIdx.x, lane = tid % MTS_WAVE, wave = tid / MTS_WAVE;
    uint32_t kr[REGS ? kRegKeys : 1];
    if (REGS) {
        int32_t entry[kRegKeys];
#pragma unroll
        for (int u = 0; u < kRegKeys; ++u) {
            const int i = tid + u * kSelThreads;
            entry[u] = i < n ? seg[i] : 0;
        }
#pragma unroll
        for (int u = 0; u < kRegKeys; ++u) {
            const int i = tid + u * kSelThreads;
            kr[u] = i < n ? order_key(w[entry[u]]) : 0u;
        }
    } else {
        for (int i0 = tid; i0 < n; i0 += kUnroll * kSelThreads) {
            int32_t entry[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int i = i0 + u * kSelThreads;
                entry[u] = i < n ? seg[i] : 0;
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int i = i0 + u * kSelThreads;
                if (i < n) kseg[i] = order_key(w[entry[u]]);
            }
        }
    }

    uint32_t prefix = 0;          // the digits chosen so far, right-aligned
    uint32_t need = capacity;     // keys still to take among those that match prefix
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        if (REGS) {
#pragma unroll
            for (int u = 0; u < kRegKeys; ++u) {
                const int i = tid + u * kSelThreads;
                const bool count = i < n && (pass == 0 || (kr[u] >> (shift + 8)) == prefix);
                if (u * kSelThreads < n) count_digit(hist, count, (kr[u] >> shift) & 255u, lane);
            }
        } else {
            for (int i0 = tid; i0 < n; i0 += kUnroll * kSelThreads) {
                uint32_t k[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const int i = i0 + u * kSelThreads;
                    k[u] = i < n ? kseg[i] : 0u;
                }
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const int i = i0 + u * kSelThreads;
                    const bool count = i < n && (pass == 0 || (k[u] >> (shift + 8)) == prefix);
                    count_digit(hist, count, (k[u] >> shift) & 255u, lane);
                }
            }
        }
        __syncthreads();
        if (wave == 0) {
            // lane l owns bins 4l..4l+3; suffix sums over the lanes find the bin in which the
            // need-th largest matching key lies
            const uint32_t h0 = hist[4 * lane], h1 = hist[4 * lane + 1], h2 = hist[4 * lane + 2],
                           h3 = hist[4 * lane + 3];
            const uint32_t mine = h0 + h1 + h2 + h3;
            uint32_t suffix = mine;
#pragma unroll
            for (int o = 1; o < MTS_WAVE; o <<= 1) {
                const uint32_t up = __shfl_down(suffix, o, MTS_WAVE);
                if (lane + o < MTS_WAVE) suffix += up;
            }
            uint32_t above = suffix - mine;   // matching keys in the bins of higher lanes
            if (above < need && need <= suffix) {
                int d;
                if (above + h3 >= need) d = 3;
                else {
                    above += h3;
                    if (above + h2 >= need) d = 2;
                    else {
                        above += h2;
                        if (above + h1 >= need) d = 1;
                        else {
                            above += h1;
                            d = 0;
                        }
                    }
                }
                chosen[0] = (prefix << 8) | (uint32_t)(4 * lane + d);
                chosen[1] = need - above;
            }
        }
        __syncthreads();
        prefix = chosen[0];
        need = chosen[1];
    }

    // prefix is now the key of the capacity-th largest weight; `need` of the entries with
    // exactly that key are kept, the earliest in segment order (= ascending entry)
    const uint64_t lt = lanemask_lt();
    uint32_t carry = 0;
    auto rank_block = [&](int i, uint32_t k) {   // one block-wide slice of kSelThreads positions
        const bool in = i < n;
        const bool tie = in && k == prefix;
        const uint64_t b = __ballot(tie);
        if (lane == 0) wave_ties[wave] = (uint32_t)__popcll(b);
        __syncthreads();
        uint32_t before = carry, total = 0;
#pragma unroll
        for (int j = 0; j < kSelWaves; ++j) {
            const uint32_t c = wave_ties[j];
            if (j < wave) before += c;
            total += c;
        }
        if (in) {
            const uint32_t rank = before + (uint32_t)__popcll(b & lt);
            const bool kp = k > prefix || (tie && rank < need);
            const int32_t entry = seg[i];
            keep[entry] = kp ? 1 : 0;
            if (kept_index) kept_index[entry] = kp ? e : -1;
        }
        carry += total;
        __syncthreads();
    };
    if (REGS) {
        // all slices at once: ties per (slice, wave) to LDS, one exclusive scan over that table in
        // segment order, then every thread ranks and writes its entries with the loads of their
        // entry numbers in flight together (a barrier per slice would expose one L2 round trip each)
#pragma unroll
        for (int u = 0; u < kRegKeys; ++u) {
            const int i = tid + u * kSelThreads;
            const uint64_t b = __ballot(i < n && kr[u] == prefix);
            if (lane == 0) tie_table[u * kSelWaves + wave] = (uint32_t)__popcll(b);
        }
        __syncthreads();
        if (wave == 0) {
            constexpr int PER_LANE = kRegKeys * kSelWaves / MTS_WAVE;
            uint32_t v[PER_LANE], sum = 0;
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j) {
                v[j] = tie_table[lane * PER_LANE + j];
                sum += v[j];
            }
            uint32_t incl = sum;
#pragma unroll
            for (int o = 1; o < MTS_WAVE; o <<= 1) {
                const uint32_t up = __shfl_up(incl, o, MTS_WAVE);
                if (lane >= o) incl += up;
            }
            uint32_t run = incl - sum;
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j) {
                tie_table[lane * PER_LANE + j] = run;
                run += v[j];
            }
        }
        __syncthreads();
        constexpr int BATCH = 8;
#pragma unroll
        for (int u0 = 0; u0 < kRegKeys; u0 += BATCH) {
            if (u0 * kSelThreads >= n) break;   // block-uniform
            int32_t entry[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int i = tid + (u0 + j) * kSelThreads;
                entry[j] = i < n ? seg[i] : 0;
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int u = u0 + j;
                const int i = tid + u * kSelThreads;
                const bool tie = i < n && kr[u] == prefix;
                const uint64_t b = __ballot(tie);
                const uint32_t rank = tie_table[u * kSelWaves + wave] + (uint32_t)__popcll(b & lt);
                if (i < n) {
                    const bool kp = kr[u] > prefix || (tie && rank < need);
                    keep[entry[j]] = kp ? 1 : 0;
                    if (kept_index) kept_index[entry[j]] = kp ? e : -1;
                }
            }
        }
    } else {
        for (int base = 0; base < n; base += kSelThreads) {
            const int i = base + tid;
            rank_block(i, i < n ? kseg[i] : 0u);
        }
    }
}

__global__ __launch_bounds__(kSelThreads) void capacity_select_kernel(
    const float* __restrict__ w, const int32_t* __restrict__ s_scatter,
    const int32_t* __restrict__ counts, const int32_t* __restrict__ expert_start, int64_t capacity,
    uint32_t* __restrict__ keys, uint8_t* __restrict__ keep, int32_t* __restrict__ kept_index,
    int32_t* __restrict__ accepted) {
    __shared__ uint32_t hist[256];
    __shared__ uint32_t chosen[2];          // prefix, number still to take inside it
    __shared__ uint32_t wave_ties[kSelWaves];
    __shared__ uint32_t tie_table[kRegKeys * kSelWaves];   // ties per (slice of kSelThreads positions, wave)
    const int e = blockIdx.x;
    const int tid = threadIdx.x;
    const int n = counts[e];
    const int32_t* seg = s_scatter + expert_start[e];
    const bool all = (int64_t)n <= capacity, none = capacity <= 0;
    if (tid == 0) accepted[e] = none ? 0 : (all ? n : (int32_t)capacity);
    if (all || none) {   // block-uniform
        for (int i = tid; i < n; i += kSelThreads) {
            const int32_t entry = seg[i];
            keep[entry] = none ? 0 : 1;
            if (kept_index) kept_index[entry] = none ? -1 : e;
        }
        return;
    }
    if (n <= kRegKeys * kSelThreads)
        select_segment<true>(w, seg, nullptr, n, e, (uint32_t)capacity, keep, kept_index, hist, chosen, wave_ties, tie_table);
    else
        select_segment<false>(w, seg, keys + expert_start[e], n, e, (uint32_t)capacity, keep, kept_index, hist,
                              chosen, wave_ties, tie_table);
}

// entries whose index is negative on input belong to no segment: they read as dropped
__global__ __launch_bounds__(256) void capacity_init_kernel(int64_t TK, uint8_t* __restrict__ keep,
                                                            int32_t* __restrict__ kept_index) {
    for (int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x; n < TK; n += (int64_t)gridDim.x * 256) {
        keep[n] = 0;
        if (kept_index) kept_index[n] = -1;
    }
}

int64_t align256(int64_t b) { return (b + 255) & ~(int64_t)255; }

}  // namespace

extern "C" int64_t mts_moe_capacity_workspace_bytes(int64_t T, int K, int E) {
    const int64_t TK = T * K;
    // route workspace, counts [E], expert_start [E+1], s_scatter / s_reverse / x_gather [TK], keys [TK]
    return align256(mts_moe_route_workspace_bytes(T, K, E)) + align256((2 * (int64_t)E + 1) * 4) +
           4 * align256(TK * 4);
}

extern "C" int mts_moe_capacity_mask(const int32_t* top_k_index, const float* top_k_weights, int64_t T,
                                     int K, int E, int64_t capacity, uint8_t* keep, int32_t* kept_index,
                                     int32_t* accepted_counts, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
    if (!top_k_index || !top_k_weights || !keep || !accepted_counts || !workspace) return MTS_ERR_NULL;
    if (T <= 0 || K < 1 || E < 1 || E > MTS_MAX_EXPERTS || T * (int64_t)K > 0x7fffffffLL)
        return MTS_ERR_SHAPE;
    if (workspace_bytes < mts_moe_capacity_workspace_bytes(T, K, E)) return MTS_ERR_WORKSPACE;
    const int64_t TK = T * K;
    char* ws = (char*)workspace;
    const int64_t route_bytes = align256(mts_moe_route_workspace_bytes(T, K, E));
    void* route_ws = ws;
    ws += route_bytes;
    int32_t* counts = (int32_t*)ws;
    int32_t* expert_start = counts + E;
    ws += align256((2 * (int64_t)E + 1) * 4);
    int32_t* s_scatter = (int32_t*)ws;
    ws += align256(TK * 4);
    int32_t* s_reverse = (int32_t*)ws;
    ws += align256(TK * 4);
    int32_t* x_gather = (int32_t*)ws;
    ws += align256(TK * 4);
    uint32_t* keys = (uint32_t*)ws;
    int rc = mts_moe_route(top_k_index, T, K, E, 1, counts, expert_start, s_scatter, s_reverse, x_gather,
                           nullptr, nullptr, nullptr, route_ws, route_bytes, stream);
    if (rc != MTS_OK) return rc;
    const int64_t init_blocks = (TK + 255) / 256;
    capacity_init_kernel<<<(int)(init_blocks < 2048 ? init_blocks : 2048), 256, 0, (hipStream_t)stream>>>(
        TK, keep, kept_index);
    MTS_CHECK_LAUNCH();
    capacity_select_kernel<<<E, kSelThreads, 0, (hipStream_t)stream>>>(
        top_k_weights, s_scatter, counts, expert_start, capacity, keys, keep, kept_index, accepted_counts);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
