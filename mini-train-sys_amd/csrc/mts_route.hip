// Routing metadata: per-expert counts, exclusive prefix sums and the stable
// expert-major permutation of the T*K routes.  Integer work only.
//
// The flat entry array is cut into chunks of kChunk entries, one chunk per wave.
//   1. histogram:  cnt[chunk][e]               (LDS atomics, order-free)
//   2. scan:       cnt[chunk][e] <- number of routes of e in earlier chunks;
//                  counts[e], expert_start[e] and the optional tile list
//   3. scatter:    a wave walks its chunk 64 entries at a time; lanes holding the
//                  same expert are found with ballots, rank inside the group is a
//                  popcount of the lower lanes, so entries keep ascending order
//                  inside every expert (a stable sort by expert).
//
// A negative expert id marks a dropped route (capacity-limited dispatch): it is not
// counted, gets no row, and its s_reverse entry is -1.  expert_start[E] is the number
// of routes that were kept.
#include "mts_common.h"
#include "mts_router_row.h"

#include <mutex>

namespace {

typedef __attribute__((ext_vector_type(4))) int32_t i32x4;
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MTS_WAVE;
constexpr int kChunk = 256;   // entries per wave
constexpr int kSteps = kChunk / MTS_WAVE;
constexpr int kFewExperts = 8;   // windows up to this many experts are ranked with one ballot per expert

// Expert ids >= E are a caller error; they are clamped so that no address derived from
// them can leave the output arrays.  Negative ids (dropped routes) stay negative.
__device__ __forceinline__ int clamp_expert(int e, int E) { return e >= E ? E - 1 : e; }

// Experts are handled in windows of at most MTS_MAX_EXPERTS ids, [e0, e0 + EW): one pass of the
// three kernels per window, so that the per-wave counters fit LDS whatever E is.  A pass counts and
// places the routes of its window only; row offsets and the tile list carry on from the pass before
// (expert_start[e0] and tile_count[0] hold what the earlier windows used).  Up to MTS_MAX_EXPERTS
// experts are one window: e0 = 0, EW = E.
__global__ __launch_bounds__(kThreads) void route_hist_kernel(const int32_t* __restrict__ idx,
                                                              int64_t TK, int E, int e0, int EW,
                                                              int32_t* __restrict__ cnt) {
    extern __shared__ int32_t lds[];  // [kWaves][EW]
    for (int i = threadIdx.x; i < kWaves * EW; i += kThreads) lds[i] = 0;
    __syncthreads();
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int64_t chunk = (int64_t)blockIdx.x * kWaves + wave;
    const int64_t base = chunk * kChunk;
    int32_t* mine = lds + wave * EW;
    for (int i = lane; i < kChunk; i += MTS_WAVE) {
        int64_t n = base + i;
        const int e = (n < TK ? clamp_expert(idx[n], E) : -1) - e0;   // a dropped route stays negative
        if (e >= 0 && e < EW) atomicAdd(&mine[e], 1);
    }
    __syncthreads();
    if (base < TK) {
        for (int e = lane; e < EW; e += MTS_WAVE) cnt[chunk * EW + e] = mine[e];
    }
}

// One block.  Wave w owns experts w, w+nw, ...: exclusive scan over chunks in
// groups of 64, then an exclusive scan of the totals over experts.
// E: experts of this window; counts / expert_start point at the window's first expert, whose id is e0.
// For e0 > 0 the rows and tiles used by the earlier windows are read from expert_start[0] (the
// sentinel the pass before wrote) and tile_count[0].
__device__ __forceinline__ void route_scan_block(
    int32_t* __restrict__ cnt, int64_t n_chunks, int E, int block_m,
    int32_t* __restrict__ counts, int32_t* __restrict__ expert_start,
    int32_t* __restrict__ tile_row_start, int32_t* __restrict__ tile_expert,
    int32_t* __restrict__ tile_count, int e0 = 0) {
    __shared__ int32_t total[MTS_MAX_EXPERTS];
    __shared__ int32_t start[MTS_MAX_EXPERTS + 1];
    __shared__ int32_t tile_off[MTS_MAX_EXPERTS + 1];
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int nw = blockDim.x / MTS_WAVE;
    for (int e = wave; e < E; e += nw) {
        int32_t carry = 0;
        for (int64_t c0 = 0; c0 < n_chunks; c0 += MTS_WAVE) {
            int64_t c = c0 + lane;
            int32_t v = (c < n_chunks) ? cnt[c * E + e] : 0;
            int32_t incl = v;
#pragma unroll
            for (int o = 1; o < MTS_WAVE; o <<= 1) {
                int32_t up = __shfl_up(incl, o, MTS_WAVE);
                if (lane >= o) incl += up;
            }
            if (c < n_chunks) cnt[c * E + e] = carry + incl - v;
            carry += __shfl(incl, MTS_WAVE - 1, MTS_WAVE);
        }
        if (lane == 0) total[e] = carry;
    }
    __syncthreads();
    if (wave == 0) {
        int32_t carry = e0 > 0 ? expert_start[0] : 0, tcarry = (e0 > 0 && tile_count) ? tile_count[0] : 0;
        for (int eb = 0; eb < E; eb += MTS_WAVE) {
            int e = eb + lane;
            int32_t v = (e < E) ? total[e] : 0;
            int32_t tv = (v + block_m - 1) / block_m;
            int32_t incl = v, tincl = tv;
#pragma unroll
            for (int o = 1; o < MTS_WAVE; o <<= 1) {
                int32_t up = __shfl_up(incl, o, MTS_WAVE);
                int32_t tup = __shfl_up(tincl, o, MTS_WAVE);
                if (lane >= o) {
                    incl += up;
                    tincl += tup;
                }
            }
            if (e < E) {
                start[e] = carry + incl - v;
                tile_off[e] = tcarry + tincl - tv;
                counts[e] = v;
                expert_start[e] = carry + incl - v;
            }
            carry += __shfl(incl, MTS_WAVE - 1, MTS_WAVE);
            tcarry += __shfl(tincl, MTS_WAVE - 1, MTS_WAVE);
        }
        if (lane == 0) {
            start[E] = carry;
            tile_off[E] = tcarry;
            expert_start[E] = carry;
            if (tile_count) tile_count[0] = tcarry;
        }
    }
    __syncthreads();
    if (tile_row_start && tile_expert) {
        for (int e = wave; e < E; e += nw) {
            int32_t nt = tile_off[e + 1] - tile_off[e];
            for (int j = lane; j < nt; j += MTS_WAVE) {
                tile_row_start[tile_off[e] + j] = start[e] + j * block_m;
                tile_expert[tile_off[e] + j] = e0 + e;
            }
        }
    }
}

__global__ __launch_bounds__(1024) void route_scan_kernel(
    int32_t* __restrict__ cnt, int64_t n_chunks, int E, int64_t TK, int block_m,
    int32_t* __restrict__ counts, int32_t* __restrict__ expert_start,
    int32_t* __restrict__ tile_row_start, int32_t* __restrict__ tile_expert,
    int32_t* __restrict__ tile_count, int e0) {
    (void)TK;
    route_scan_block(cnt, n_chunks, E, block_m, counts, expert_start, tile_row_start, tile_expert, tile_count, e0);
}

// The stable scatter of one chunk (entries [cbeg, cend)) by one wave; next[e] is the next free row
// of window expert e for this chunk (LDS, private to the wave).
// E: all experts; [e0, e0 + EW): the window of this pass.
// scatter_load fetches the window-relative expert ids of kSteps x 64 entries starting at `base`
// (-1: dropped route, whose -1 goes to s_reverse in the first pass; -2: not this pass);
// scatter_place ranks and writes them.
__device__ __forceinline__ void scatter_load(int (&ev)[kSteps], const int32_t* __restrict__ idx, int E, int e0, int EW,
                                             int64_t base, int64_t cend) {
    const int lane = threadIdx.x % MTS_WAVE;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {  // these loads are in flight together
        const int64_t n = base + s * MTS_WAVE + lane;
        const int e = n < cend ? clamp_expert(idx[n], E) : -1;
        ev[s] = e < 0 ? (e0 == 0 && n < cend ? -1 : -2) : (e >= e0 && e < e0 + EW ? e - e0 : -2);
    }
}

__device__ __forceinline__ void scatter_place(const int (&ev)[kSteps], int K, int EW, int64_t base, int64_t cend,
                                              volatile int32_t* next, int32_t* __restrict__ s_scatter,
                                              int32_t* __restrict__ s_reverse, int32_t* __restrict__ x_gather) {
    const int lane = threadIdx.x % MTS_WAVE;
    const uint64_t lt = lanemask_lt();
    if (EW <= kFewExperts) {   // wave-uniform
        // A window of few experts: one ballot per expert ranks the 64 entries of a step, and the next free rows
        // stay in registers from step to step (the same positions as the loop over the experts present below:
        // entries of one expert in lane order).
        int32_t nx[kFewExperts];
#pragma unroll
        for (int x = 0; x < kFewExperts; ++x) nx[x] = x < EW ? next[x] : 0;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int64_t n = base + s * MTS_WAVE + lane;
            if (base + s * MTS_WAVE >= cend) break;   // wave-uniform
            const int e = ev[s];
            int pos = -1;
#pragma unroll
            for (int x = 0; x < kFewExperts; ++x) {
                const uint64_t same = __ballot(e == x);
                if (e == x) pos = nx[x] + __popcll(same & lt);
                nx[x] += __popcll(same);
            }
            if (e >= -1 && n < cend) s_reverse[n] = pos;
            if (e >= 0) {
                s_scatter[pos] = (int32_t)n;
                x_gather[pos] = (int32_t)(n / K);
            }
        }
#pragma unroll
        for (int x = 0; x < kFewExperts; ++x)
            if (lane == x && x < EW) next[x] = nx[x];
        return;
    }
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        const int64_t n = base + s * MTS_WAVE + lane;
        if (base + s * MTS_WAVE >= cend) break;   // wave-uniform
        const int e = ev[s];
        const bool valid = e >= 0;
        int pos = -1;
        uint64_t todo = __ballot(valid);
        while (todo) {
            int leader = __ffsll((unsigned long long)todo) - 1;
            int el = __shfl(e, leader, MTS_WAVE);
            uint64_t same = __ballot(e == el);
            int first = next[el];  // every lane reads before the leader updates
            if (e == el) pos = first + __popcll(same & lt);
            if (lane == leader) next[el] = first + __popcll(same);
            todo &= ~same;
        }
        if (e >= -1 && n < cend) s_reverse[n] = pos;
        if (valid) {
            s_scatter[pos] = (int32_t)n;
            x_gather[pos] = (int32_t)(n / K);
        }
    }
}

// `first` holds the ids of the chunk's first kSteps x 64 entries already (scatter_load at cbeg)
__device__ __forceinline__ void scatter_chunk(int (&first)[kSteps], const int32_t* __restrict__ idx, int K, int E, int e0,
                                              int EW, int64_t cbeg, int64_t cend, volatile int32_t* next,
                                              int32_t* __restrict__ s_scatter, int32_t* __restrict__ s_reverse,
                                              int32_t* __restrict__ x_gather) {
    scatter_place(first, K, EW, cbeg, cend, next, s_scatter, s_reverse, x_gather);
    for (int64_t base = cbeg + kChunk; base < cend; base += kChunk) {
        int ev[kSteps];
        scatter_load(ev, idx, E, e0, EW, base, cend);
        scatter_place(ev, K, EW, base, cend, next, s_scatter, s_reverse, x_gather);
    }
}

// chunk_len entries per wave (a multiple of 64 is not required); the chunks are the ones the
// counters in cnt were taken over
// E: all experts; [e0, e0 + EW): the window of this pass (cnt is [chunk][EW], expert_start points at expert e0)
__global__ __launch_bounds__(kThreads) void route_scatter_kernel(
    const int32_t* __restrict__ idx, int64_t TK, int K, int E, int e0, int EW, int chunk_len,
    const int32_t* __restrict__ cnt, const int32_t* __restrict__ expert_start, int32_t* __restrict__ s_scatter,
    int32_t* __restrict__ s_reverse, int32_t* __restrict__ x_gather) {
    extern __shared__ int32_t lds[];  // [kWaves][E] next free row per expert
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int64_t chunk = (int64_t)blockIdx.x * kWaves + wave;
    const int64_t cbeg = chunk * chunk_len;
    if (cbeg >= TK) return;  // whole wave leaves; no block barrier below
    const int64_t cend = cbeg + chunk_len < TK ? cbeg + chunk_len : TK;
    int first[kSteps];
    scatter_load(first, idx, E, e0, EW, cbeg, cend);   // in flight with the counter loads below
    volatile int32_t* next = lds + wave * EW;
    for (int e = lane; e < EW; e += MTS_WAVE) next[e] = expert_start[e] + cnt[chunk * EW + e];
    scatter_chunk(first, idx, K, E, e0, EW, cbeg, cend, next, s_scatter, s_reverse, x_gather);
}

// The launch behind the kernel that chains the router projection to the post-process.  Its last block
// reduces that kernel's per-block statistics and route counts (expert totals, expert_start, the
// load-balancing term and the load metrics); every other block scatters four chunks, one per wave,
// and does not wait for the last block: the block adds up the route counts of ALL chunks itself (at most
// kFinishChunks x kFinishMaxE counters, read from L2) to get the experts' first rows and the rows the
// chunks before its own take.  One launch and one dependent round trip less than scan-then-scatter.
constexpr int kFinishChunks = MTS_HEAD_MAX_CHUNKS;
constexpr int kFinishMaxE = 16;
__global__ __launch_bounds__(kThreads) void head_scatter_kernel(
    const float* __restrict__ partial, const int32_t* __restrict__ cnt, int n_chunks, int E, float inv_t,
    float inv_routes, float* __restrict__ prob_mean, float* __restrict__ z_loss, float* __restrict__ entropy,
    int32_t* __restrict__ counts, float* __restrict__ load_balance, float* __restrict__ load_stats,
    int32_t* __restrict__ expert_start, const int32_t* __restrict__ idx, int64_t TK, int K, int chunk_len,
    int32_t* __restrict__ s_scatter, int32_t* __restrict__ s_reverse, int32_t* __restrict__ x_gather) {
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    if (blockIdx.x + 1 < gridDim.x) {
        __shared__ int32_t next_rows[kWaves][kFinishMaxE];
        __shared__ int32_t sums[kWaves][2 * kFinishMaxE];
        static_assert(kFinishChunks == 2 * kThreads, "two chunks per thread");
        const int chunk0 = blockIdx.x * kWaves;   // the block's first chunk; wave w scatters chunk0 + w
        const int64_t cbeg = (int64_t)(chunk0 + wave) * chunk_len;
        const int64_t cend = cbeg + chunk_len < TK ? cbeg + chunk_len : TK;
        int first_ids[kSteps];
        if (cbeg < TK) scatter_load(first_ids, idx, E, 0, E, cbeg, cend);   // in flight with the counter loads below
        // routes per expert: over all chunks, and over the chunks before the block's first one
        int32_t total[kFinishMaxE], before[kFinishMaxE];
#pragma unroll
        for (int e = 0; e < kFinishMaxE; ++e) total[e] = before[e] = 0;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int c = q * kThreads + threadIdx.x;
            if (E == 8) {   // a row is two aligned 16-byte loads
                i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
                if (c < n_chunks) {
                    lo = *reinterpret_cast<const i32x4*>(cnt + (int64_t)c * 8);
                    hi = *reinterpret_cast<const i32x4*>(cnt + (int64_t)c * 8 + 4);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    total[e] += lo[e];
                    total[e + 4] += hi[e];
                    before[e] += c < chunk0 ? lo[e] : 0;
                    before[e + 4] += c < chunk0 ? hi[e] : 0;
                }
            } else {
#pragma unroll
                for (int e = 0; e < kFinishMaxE; ++e) {
                    const int32_t v = (c < n_chunks && e < E) ? cnt[(int64_t)c * E + e] : 0;
                    total[e] += v;
                    before[e] += c < chunk0 ? v : 0;
                }
            }
        }
        // the counts of the block's own chunks before this wave's (at most kWaves - 1 rows), one expert per lane
        int32_t own = 0;
        for (int i = 0; i < wave; ++i)
            if (lane < E && chunk0 + i < n_chunks) own += cnt[(int64_t)(chunk0 + i) * E + lane];
#pragma unroll
        for (int e = 0; e < kFinishMaxE; ++e) {
            if (e < E) {   // block-uniform
                int32_t t = total[e], b = before[e];
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    t += __shfl_xor(t, o, MTS_WAVE);
                    b += __shfl_xor(b, o, MTS_WAVE);
                }
                if (lane == 0) {
                    sums[wave][e] = t;
                    sums[wave][kFinishMaxE + e] = b;
                }
            }
        }
        __syncthreads();
        if (cbeg >= TK) return;  // whole wave leaves; no block barrier below
        // lane e: the expert's first row = the totals of the experts before it, + its routes in earlier chunks
        int32_t t = 0, bsum = 0;
        if (lane < E) {
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                t += sums[w][lane];
                bsum += sums[w][kFinishMaxE + lane];
            }
        }
        int32_t incl = t;
#pragma unroll
        for (int o = 1; o < kFinishMaxE; o <<= 1) {
            const int32_t up = __shfl_up(incl, o, MTS_WAVE);
            if (lane >= o) incl += up;
        }
        volatile int32_t* next = next_rows[wave];
        if (lane < E) next[lane] = incl - t + bsum + own;
        scatter_chunk(first_ids, idx, K, E, 0, E, cbeg, cend, next, s_scatter, s_reverse, x_gather);
        return;
    }
    // the last block: wave w sums columns w, w + kWaves, ... of the partials (and, for an expert's column, its
    // route counts); a lane takes chunks lane, lane + 64, ..., all of them requested before the first sum
    __shared__ mts_router::StatsShared sh;
    __shared__ int32_t total_s[kFinishMaxE];
    static_assert(kFinishChunks % MTS_WAVE == 0, "whole rounds of lanes over the chunks");
    constexpr int ROUNDS = kFinishChunks / MTS_WAVE;
    constexpr int COLS = (kFinishMaxE + 2 + kWaves - 1) / kWaves;   // columns per wave, at most
    float colv[COLS][ROUNDS];
    int32_t totv[COLS][ROUNDS];
#pragma unroll
    for (int q = 0; q < COLS; ++q) {
        const int i = wave + q * kWaves;
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u) {
            const int c = lane + u * MTS_WAVE;
            colv[q][u] = (i < E + 2 && c < n_chunks) ? partial[(int64_t)c * (E + 2) + i] : 0.f;
            totv[q][u] = (i < E && c < n_chunks) ? cnt[(int64_t)c * E + i] : 0;
        }
    }
#pragma unroll
    for (int q = 0; q < COLS; ++q) {
        const int i = wave + q * kWaves;
        if (i < E + 2) {   // wave-uniform
            float v = 0.f;
            int32_t c = 0;
#pragma unroll
            for (int u = 0; u < ROUNDS; ++u) {
                v += colv[q][u];
                c += totv[q][u];
            }
            v = wave_sum(v);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, MTS_WAVE);
            if (lane == 0) {
                if (i < E) total_s[i] = c;
                mts_router::stats_column(sh, i, v * inv_t, c, E, inv_routes, prob_mean, z_loss, entropy, counts);
            }
        }
    }
    __syncthreads();
    if (wave == kWaves - 1) {   // exclusive scan of the routes per expert: one lane per expert
        const int32_t v = lane < E ? total_s[lane] : 0;
        int32_t incl = v;
#pragma unroll
        for (int o = 1; o < MTS_WAVE; o <<= 1) {
            const int32_t up = __shfl_up(incl, o, MTS_WAVE);
            if (lane >= o) incl += up;
        }
        if (lane < E) expert_start[lane] = incl - v;
        if (lane == E - 1) expert_start[E] = incl;
    }
    mts_router::stats_finalize(sh, wave, 0, 1, E, load_balance, load_stats);
}

}  // namespace

extern "C" int64_t mts_moe_route_workspace_bytes(int64_t T, int K, int E) {
    int64_t TK = T * K;
    int64_t n_chunks = (TK + kChunk - 1) / kChunk;
    return n_chunks * (E < MTS_MAX_EXPERTS ? E : MTS_MAX_EXPERTS) * (int64_t)sizeof(int32_t);   // one window of experts at a time
}

namespace {

// the three launches; cnt holds n_chunks * E counters, every one of which is written by the
// histogram kernel before the scan reads it (nothing has to start at zero)
int route_launch(const int32_t* top_k_index, int64_t T, int K, int E, int block_m, int32_t* counts,
                 int32_t* expert_start, int32_t* s_scatter, int32_t* s_reverse, int32_t* x_gather,
                 int32_t* tile_row_start, int32_t* tile_expert, int32_t* tile_count, int32_t* cnt,
                 hipStream_t s) {
    const bool permute = s_scatter != nullptr;
    const int64_t TK = T * K;
    const int64_t n_chunks = (TK + kChunk - 1) / kChunk;
    const int grid = (int)((n_chunks + kWaves - 1) / kWaves);
    for (int e0 = 0; e0 < E; e0 += MTS_MAX_EXPERTS) {   // one pass per window of experts
        const int EW = E - e0 < MTS_MAX_EXPERTS ? E - e0 : MTS_MAX_EXPERTS;
        const size_t lds = (size_t)kWaves * EW * sizeof(int32_t);
        route_hist_kernel<<<grid, kThreads, lds, s>>>(top_k_index, TK, E, e0, EW, cnt);
        MTS_CHECK_LAUNCH();
        route_scan_kernel<<<1, 1024, 0, s>>>(cnt, n_chunks, EW, TK, block_m, counts + e0, expert_start + e0,
                                             tile_row_start, tile_expert, tile_count, e0);
        MTS_CHECK_LAUNCH();
        if (!permute) continue;
        route_scatter_kernel<<<grid, kThreads, lds, s>>>(top_k_index, TK, K, E, e0, EW, kChunk, cnt, expert_start + e0,
                                                         s_scatter, s_reverse, x_gather);
        MTS_CHECK_LAUNCH();
    }
    return MTS_OK;
}

// argument checks shared by the two entry points
int route_check(const int32_t* top_k_index, int64_t T, int K, int E, int block_m, const int32_t* counts,
                const int32_t* expert_start, const int32_t* s_scatter, const int32_t* s_reverse,
                const int32_t* x_gather) {
    // the three permutation arrays are optional as a group: without them only the counts,
    // the expert offsets and (if asked for) the tile list are produced
    const bool permute = s_scatter || s_reverse || x_gather;
    if (!top_k_index || !counts || !expert_start) return MTS_ERR_NULL;
    if (permute && (!s_scatter || !s_reverse || !x_gather)) return MTS_ERR_NULL;
    if (T <= 0 || K < 1 || E < 1 || E > MTS_MAX_MOE_EXPERTS || block_m < 1 ||
        T * (int64_t)K > 0x7fffffffLL)
        return MTS_ERR_SHAPE;
    return MTS_OK;
}

// Chunk counters of mts_moe_route_static: one array per GPU the library runs on, held until the
// process ends.  In host code the symbol is only a handle; the device address is looked up once
// per device (with that device current) and kept.
constexpr int kMaxDevices = 64;
static __device__ __align__(256) int32_t scratch[MTS_ROUTE_STATIC_BYTES / sizeof(int32_t)];
std::mutex scratch_lock;
int32_t* scratch_ptr[kMaxDevices] = {};

int scratch_of_current_device(int32_t** out) {
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return (int)err;
    if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_ptr[dev]) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return (int)err;
        if (!ptr) return (int)hipErrorInvalidSymbol;
        scratch_ptr[dev] = (int32_t*)ptr;
    }
    *out = scratch_ptr[dev];
    return MTS_OK;
}

}  // namespace

extern "C" int mts_moe_route(const int32_t* top_k_index, int64_t T, int K, int E, int block_m,
                             int32_t* counts, int32_t* expert_start, int32_t* s_scatter,
                             int32_t* s_reverse, int32_t* x_gather, int32_t* tile_row_start,
                             int32_t* tile_expert, int32_t* tile_count, void* workspace,
                             int64_t workspace_bytes, void* stream) {
    if (!workspace) return MTS_ERR_NULL;
    const int rc = route_check(top_k_index, T, K, E, block_m, counts, expert_start, s_scatter, s_reverse, x_gather);
    if (rc) return rc;
    if (workspace_bytes < mts_moe_route_workspace_bytes(T, K, E)) return MTS_ERR_WORKSPACE;
    return route_launch(top_k_index, T, K, E, block_m, counts, expert_start, s_scatter, s_reverse, x_gather,
                        tile_row_start, tile_expert, tile_count, (int32_t*)workspace, (hipStream_t)stream);
}

extern "C" int mts_moe_route_static(const int32_t* top_k_index, int64_t T, int K, int E, int block_m,
                                    int32_t* counts, int32_t* expert_start, int32_t* s_scatter,
                                    int32_t* s_reverse, int32_t* x_gather, int32_t* tile_row_start,
                                    int32_t* tile_expert, int32_t* tile_count, void* stream) {
    const int rc = route_check(top_k_index, T, K, E, block_m, counts, expert_start, s_scatter, s_reverse, x_gather);
    if (rc) return rc;
    if (mts_moe_route_workspace_bytes(T, K, E) > (int64_t)MTS_ROUTE_STATIC_BYTES) return MTS_ERR_WORKSPACE;
    int32_t* cnt = nullptr;
    const int err = scratch_of_current_device(&cnt);
    if (err) return err;
    return route_launch(top_k_index, T, K, E, block_m, counts, expert_start, s_scatter, s_reverse, x_gather,
                        tile_row_start, tile_expert, tile_count, cnt, (hipStream_t)stream);
}

extern "C" int64_t mts_moe_head_workspace_bytes(int64_t T, int K, int E) {
    (void)T;
    (void)K;
    return (int64_t)MTS_HEAD_MAX_CHUNKS * (2 * E + 2) * (int64_t)sizeof(float);   // statistics partials, then route counts
}

extern "C" int mts_moe_head_fwd(const void* x, const float* w_r, int64_t T, int H, int E, int K, int normalize,
                                int act_dtype, float* logits, float* weights, int32_t* indices, void* weights_act,
                                float* prob_mean, float* z_loss, float* entropy, int32_t* counts, float* load_balance,
                                float* load_stats, int32_t* expert_start, int32_t* s_scatter, int32_t* s_reverse,
                                int32_t* x_gather, void* workspace, int64_t workspace_bytes, void* stream) {
    if (!prob_mean || !z_loss || !entropy || !counts || !expert_start || !s_scatter || !s_reverse || !x_gather || !workspace)
        return MTS_ERR_NULL;
    if (weights_act && act_dtype == MTS_F32) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1 || T * (int64_t)K > 0x7fffffffLL) return MTS_ERR_SHAPE;
    if (workspace_bytes < mts_moe_head_workspace_bytes(T, K, E)) return MTS_ERR_WORKSPACE;
    if (!mts_aligned16(workspace)) return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    float* partial = (float*)workspace;
    int32_t* cnt = (int32_t*)(partial + (int64_t)MTS_HEAD_MAX_CHUNKS * (E + 2));
    const int rc = mts_launch_router_head(x, w_r, T, H, E, K, normalize, act_dtype, logits, weights, indices, weights_act,
                                          partial, cnt, s);
    if (rc) return rc;
    int blocks, rows_per_wave;
    mts_router_head_geometry(T, mts_router_head_group(H, E, act_dtype), &blocks, &rows_per_wave);
    const int64_t rows_per_chunk = (int64_t)rows_per_wave * 4;
    const int64_t n_chunks = (T + rows_per_chunk - 1) / rows_per_chunk;
    if (n_chunks > kFinishChunks || E > kFinishMaxE) return MTS_ERR_SHAPE;   // cannot happen: the geometry caps the chunks, the projection E
    const int grid = (int)((n_chunks + kWaves - 1) / kWaves) + 1;   // scatter blocks, then the block that reduces
    head_scatter_kernel<<<grid, kThreads, 0, s>>>(partial, cnt, (int)n_chunks, E, 1.0f / (float)T,
                                                  1.0f / ((float)T * (float)K), prob_mean, z_loss, entropy, counts,
                                                  load_balance, load_stats, expert_start, indices, T * (int64_t)K, K,
                                                  (int)(rows_per_chunk * K), s_scatter, s_reverse, x_gather);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
