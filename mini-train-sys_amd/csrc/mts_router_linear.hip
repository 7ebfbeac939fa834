// Router projection around the post-process kernels: logits = float(x) W_r^T in fp32 and its
// backward (dx in the activation dtype, dW_r in fp32).  x is read in its own dtype, so no fp32
// copy of the activations is made; every sum runs in a fixed order (no float atomics).
// All three kernels are VALU/HBM bound: 2*T*H*E FLOP forward, twice that backward.
#include "mts_common.h"
#include "mts_router_row.h"
#include "mts_router_bwd_block.h"

namespace {

using namespace mts_rl;

constexpr int kRows = 4;         // rows per wave in the forward kernel
constexpr int kFwdThreads = 256;

// Butterfly reduce-scatter over the 64 lanes of a wave: N values are live in v[0..N), the
// partner is `O` lanes away.  While N > 1 a lane hands one half of its values to the partner
// and adds the partner's copy of the half it keeps; once one value is left the remaining
// steps are plain pairwise sums.  The order of the additions is fixed.
template <int NV, int N, int O>
__device__ __forceinline__ void reduce_scatter(float (&v)[NV], int lane, int& idx) {
    if constexpr (O >= 1) {
        if constexpr (N > 1) {
            const bool up = (lane & O) != 0;
#pragma unroll
            for (int i = 0; i < N / 2; ++i) {
                const float send = up ? v[i] : v[i + N / 2];
                const float keep = up ? v[i + N / 2] : v[i];
                v[i] = keep + __shfl_xor(send, O, MTS_WAVE);
            }
            idx += up ? N / 2 : 0;
            reduce_scatter<NV, N / 2, O / 2>(v, lane, idx);
        } else {
            v[0] += __shfl_xor(v[0], O, MTS_WAVE);
            reduce_scatter<NV, 1, O / 2>(v, lane, idx);
        }
    }
}

// One wave computes kRows rows: a lane owns 4 consecutive columns of every 256-column slab,
// the weights sit in LDS (loaded once per block), and the E partial dot products of a row are
// summed across the wave with a fixed shuffle tree.
// CHUNKED (rows wider than PASSES slabs): the columns are taken in chunks of PASSES slabs, the
// loads of the next chunk (of the same rows, or the first one of the next row group) in flight
// behind the arithmetic of the current one, and the partial dot products stay in registers
// until the last chunk of the row group.
template <typename XT, int PASSES>
struct RowGroupLoader {
    typedef typename RawVec<XT>::type raw_t;
    // rows r0..r0+kRows-1 (those below `end`), columns of chunk `ch`
    static __device__ __forceinline__ void load(raw_t (&dst)[PASSES][kRows], const XT* __restrict__ x, int64_t r0,
                                                int64_t end, int ch, int H, int lane) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int c = lane * 4 + (ch * PASSES + ps) * MTS_WAVE * 4;
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                const bool ok = c < H && r0 + r < end;
                dst[ps][r] = load_raw(x + (ok ? (r0 + r) * H + c : 0));   // a masked lane reads element 0; its weights are skipped
            }
        }
    }
    // acc[r][e] += the chunk's share of <x[r0+r], w[e]>
    template <int EP>
    static __device__ __forceinline__ void accumulate(float (&acc)[kRows][EP], const raw_t (&cur)[PASSES][kRows],
                                                      const float* w_lds, int64_t r0, int64_t end, int ch, int H, int E,
                                                      int lane) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int c = lane * 4 + (ch * PASSES + ps) * MTS_WAVE * 4;
            if (c < H) {
                f32x4 xv[kRows];
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                    xv[r] = r0 + r < end ? widen(cur[ps][r]) : z;
                }
#pragma unroll
                for (int e = 0; e < EP; ++e) {
                    const f32x4 wv = *reinterpret_cast<const f32x4*>(w_lds + (e < E ? e : 0) * H + c);
#pragma unroll
                    for (int r = 0; r < kRows; ++r)
                        acc[r][e] += xv[r][0] * wv[0] + xv[r][1] * wv[1] + xv[r][2] * wv[2] + xv[r][3] * wv[3];
                }
            }
        }
    }
};

template <typename XT, int EP, int PASSES, bool CHUNKED = false>
__global__ __launch_bounds__(kFwdThreads) void router_logits_fwd_kernel(const XT* __restrict__ x,
                                                                         const float* __restrict__ w, int64_t T,
                                                                         int H, int E, int n_chunks,
                                                                         float* __restrict__ logits) {
    extern __shared__ __attribute__((aligned(16))) float w_lds[];   // [E][H]
#pragma unroll 8
    for (int i = threadIdx.x * 4; i < E * H; i += kFwdThreads * 4)
        *reinterpret_cast<f32x4*>(w_lds + i) = *reinterpret_cast<const f32x4*>(w + i);
    const int lane = threadIdx.x % MTS_WAVE;
    const int nch = CHUNKED ? n_chunks : 1;
    const int64_t wave0 = (int64_t)blockIdx.x * (kFwdThreads / MTS_WAVE) + threadIdx.x / MTS_WAVE;
    const int64_t stride = (int64_t)gridDim.x * (kFwdThreads / MTS_WAVE) * kRows;
    typedef RowGroupLoader<XT, PASSES> Loader;
    typename Loader::raw_t cur[PASSES][kRows], nxt[PASSES][kRows];
    int64_t r0 = wave0 * kRows;
    int ch = 0;
    if (r0 < T) Loader::load(cur, x, r0, T, 0, H, lane);
    __syncthreads();
    float acc[kRows][EP];
    while (r0 < T) {
        const bool last = ch + 1 == nch;
        const int64_t nr0 = last ? r0 + stride : r0;
        const int nc = last ? 0 : ch + 1;
        if (nr0 < T) Loader::load(nxt, x, nr0, T, nc, H, lane);
        if (ch == 0) {
#pragma unroll
            for (int r = 0; r < kRows; ++r)
#pragma unroll
                for (int e = 0; e < EP; ++e) acc[r][e] = 0.f;
        }
        Loader::template accumulate<EP>(acc, cur, w_lds, r0, T, ch, H, E, lane);
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
            for (int r = 0; r < kRows; ++r) cur[ps][r] = nxt[ps][r];
        if (last) {
            // Sum over the 64 lanes of kRows*EP values: at every step a lane hands half of its
            // values to the partner lane and adds the partner's copy of the half it keeps, so the
            // count halves with the lane distance (fixed order: bit-stable).  With kRows*EP == 32
            // one value is left after the distance-2 step, shared by a lane pair.
            static_assert(kRows * EP == 32 || kRows * EP == 64, "reduction layout");
            constexpr int NV = kRows * EP;
            float v[NV];
#pragma unroll
            for (int r = 0; r < kRows; ++r)
#pragma unroll
                for (int e = 0; e < EP; ++e) v[r * EP + e] = acc[r][e];
            int idx = 0;   // index of the value this lane ends up with, built from its lane bits
            reduce_scatter<NV, NV, 32>(v, lane, idx);
            const float mine = v[0];
            const int r = idx / EP, e = idx % EP;
            const bool writer = NV == 64 ? true : (lane & 1) == 0;
            if (writer && e < E && r0 + r < T) logits[(r0 + r) * E + e] = mine;
        }
        r0 = nr0;
        ch = nc;
    }
}

// ---------------------------------------------------------------------------
// The router projection chained to the post-process.  The block takes a contiguous range of
// rows, a wave a contiguous part of it; the 4 rows x E logits a wave has just summed sit one per
// lane (pair), so lanes 0..3 collect a row each with cross-lane reads and run the post-process
// on it (softmax, top-k on the logits, weights) without the logits making a round trip through
// memory; the logits are still written, for the backward pass.  Per block: the sums of the
// statistics (fixed order) and the routes per expert, which are at the same time the chunk
// histogram of the routing metadata (chunk = the entries of the block's rows).
// ---------------------------------------------------------------------------
template <typename XT, int EP, int PASSES, bool CHUNKED = false>
__global__ __launch_bounds__(kFwdThreads) void router_head_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, int64_t T, int H, int E, int K, int normalize,
    int rows_per_wave, int n_chunks, float* __restrict__ logits, float* __restrict__ weights, int32_t* __restrict__ indices,
    void* __restrict__ weights_act, int act_dtype, float* __restrict__ partial, int32_t* __restrict__ cnt) {
    using namespace mts_router;
    extern __shared__ __attribute__((aligned(16))) float w_lds[];   // [E][H]
#pragma unroll 8
    for (int i = threadIdx.x * 4; i < E * H; i += kFwdThreads * 4)
        *reinterpret_cast<f32x4*>(w_lds + i) = *reinterpret_cast<const f32x4*>(w + i);
    constexpr int WAVES = kFwdThreads / MTS_WAVE;
    const int lane = threadIdx.x % MTS_WAVE, wave = threadIdx.x / MTS_WAVE;
    const int nch = CHUNKED ? n_chunks : 1;
    const int64_t beg = ((int64_t)blockIdx.x * WAVES + wave) * rows_per_wave;
    const int64_t end = beg + rows_per_wave < T ? beg + rows_per_wave : T;
    typedef RowGroupLoader<XT, PASSES> Loader;
    typename Loader::raw_t cur[PASSES][kRows], nxt[PASSES][kRows];
    if (beg < end) Loader::load(cur, x, beg, end, 0, H, lane);
    __syncthreads();

    // The logits of up to 64 rows are parked in LDS (row stride EP + 1: a lane per row reads without
    // bank conflicts); then lane L runs the post-process of row L, so a wave pays for the post-process
    // once per 64 rows, not once per group of kRows.
    constexpr int LROW = EP + 1;
    __shared__ float parked[WAVES][MTS_WAVE * LROW];
    float* mine_rows = parked[wave];
    float psum[EP], zsum = 0.f, hsum = 0.f;   // statistics of the rows this lane post-processes
    int csum[EP];
#pragma unroll
    for (int e = 0; e < EP; ++e) {
        psum[e] = 0.f;
        csum[e] = 0;
    }
    int64_t pass_base = beg;
    int64_t r0 = beg;
    int ch = 0;
    float acc[kRows][EP];
    while (r0 < end) {
        const bool last = ch + 1 == nch;
        const int64_t nr0 = last ? r0 + kRows : r0;
        const int nc = last ? 0 : ch + 1;
        if (nr0 < end) Loader::load(nxt, x, nr0, end, nc, H, lane);
        if (ch == 0) {
#pragma unroll
            for (int r = 0; r < kRows; ++r)
#pragma unroll
                for (int e = 0; e < EP; ++e) acc[r][e] = 0.f;
        }
        Loader::template accumulate<EP>(acc, cur, w_lds, r0, end, ch, H, E, lane);
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
            for (int r = 0; r < kRows; ++r) cur[ps][r] = nxt[ps][r];
        const int64_t g0 = r0;   // the row group whose dot products are complete when `last`
        r0 = nr0;
        ch = nc;
        if (!last) continue;
        static_assert(kRows * EP == 32 || kRows * EP == 64, "reduction layout");
        constexpr int NV = kRows * EP;
        float v[NV];
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int e = 0; e < EP; ++e) v[r * EP + e] = acc[r][e];
        int idx = 0;
        reduce_scatter<NV, NV, 32>(v, lane, idx);
        const float mine = v[0];   // value `idx` of the group: row g0 + idx / EP, expert idx % EP
        {
            const int r = idx / EP, e = idx % EP;
            const bool writer = NV == 64 ? true : (lane & 1) == 0;
            if (writer && e < E && g0 + r < end) logits[(g0 + r) * E + e] = mine;
            if (writer) mine_rows[(int)(g0 - pass_base + r) * LROW + e] = e < E ? mine : -INFINITY;
        }
        const int64_t parked_to = g0 + kRows < end ? g0 + kRows : end;
        if (parked_to - pass_base < MTS_WAVE && parked_to < end) continue;   // wave-uniform: park more rows first
        __builtin_amdgcn_wave_barrier();
        const int64_t row = pass_base + lane;
        const bool live = row < parked_to;
        RowState<EP, 1> rs;
#pragma unroll
        for (int e = 0; e < EP; ++e) rs.l[e] = live ? mine_rows[lane * LROW + e] : (e == 0 ? 0.f : -INFINITY);
        softmax_row<EP, 1>(rs);
        float sel_p[MTS_MAX_TOP_K], mass;
        int sel_e[MTS_MAX_TOP_K];
        select_top_k<EP, 1>(rs, E, K, 0, sel_p, sel_e, mass);
        if (live) {
            const float inv = normalize ? 1.0f / fmaxf(mass, 1.1920928955078125e-07f) : 1.0f;
#pragma unroll
            for (int k = 0; k < MTS_MAX_TOP_K; ++k) {
                if (k < K) {
                    const float wk = sel_p[k] * inv;
                    weights[row * K + k] = wk;
                    indices[row * K + k] = sel_e[k];
                    if (weights_act) {
                        if (act_dtype == MTS_BF16) reinterpret_cast<bf16_t*>(weights_act)[row * K + k] = (bf16_t)wk;
                        else reinterpret_cast<mts_f16_t*>(weights_act)[row * K + k] = (mts_f16_t)wk;
                    }
#pragma unroll
                    for (int e = 0; e < EP; ++e) csum[e] += e == sel_e[k] ? 1 : 0;
                }
            }
#pragma unroll
            for (int e = 0; e < EP; ++e) {
                psum[e] += rs.p[e];
                const float lp = fmaxf(rs.l[e] - rs.L, kLogFloor);
                hsum -= (rs.p[e] > 0.f) ? rs.p[e] * lp : 0.f;
            }
            zsum += rs.L * rs.L;
        }
        pass_base = parked_to;
        __builtin_amdgcn_wave_barrier();
    }
    // lanes -> lane 0 (fixed shuffle tree), waves -> block through LDS (fixed order)
    __shared__ float red[WAVES][EP + 2];
    __shared__ int32_t cred[WAVES][EP];
#pragma unroll
    for (int e = 0; e < EP; ++e) {
        psum[e] = wave_sum(psum[e]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) csum[e] += __shfl_xor(csum[e], o, MTS_WAVE);
    }
    zsum = wave_sum(zsum);
    hsum = wave_sum(hsum);
    if (lane == 0) {
#pragma unroll
        for (int e = 0; e < EP; ++e) {
            red[wave][e] = psum[e];
            cred[wave][e] = csum[e];
        }
        red[wave][EP] = zsum;
        red[wave][EP + 1] = hsum;
    }
    __syncthreads();
    if ((int64_t)blockIdx.x * WAVES * rows_per_wave >= T) return;   // no rows: not a chunk
    for (int i = threadIdx.x; i < E + 2; i += kFwdThreads) {
        const int src = i < E ? i : EP + (i - E);
        float sum = 0.f;
#pragma unroll
        for (int q = 0; q < WAVES; ++q) sum += red[q][src];
        partial[(int64_t)blockIdx.x * (E + 2) + i] = sum;
    }
    for (int i = threadIdx.x; i < E; i += kFwdThreads) {
        int32_t sum = 0;
#pragma unroll
        for (int q = 0; q < WAVES; ++q) sum += cred[q][i];
        cnt[(int64_t)blockIdx.x * E + i] = sum;
    }
}

// Backward: a thread owns 4 consecutive columns.  Per row it forms dx (in the activation
// dtype) from the row's E logit gradients and its weight columns, and adds the row's
// contribution to its E x 4 block of dW_r; every block writes its partial dW_r to the
// workspace, and the reduction kernel sums the partials in block order.
// The row loop works on groups of UN rows without a bounds test (the raw loads of the next
// group are issued before the arithmetic of the current one); the rows left over are done one
// by one.  EXACT: E == EP, so a row's logit gradients are EP consecutive floats at an address
// every thread of the block shares, which the compiler turns into scalar loads.
// A block holds `groups` sets of column threads; each set takes a contiguous share of the block's
// rows, and the sets' dW_r sums are added through LDS in set order before the block writes its
// one partial: a quarter of the partials for the same number of waves in flight.
// Rows wider than a block has column threads for are cut into column ranges (blockIdx.y); a CHAIN
// block of every range forms the logit gradients of its rows again.
// the stand-alone launch of the block function: one block per row range (x) and column range (y)
template <typename XT, int EP, bool EXACT, bool CHAIN = false>
__global__ __launch_bounds__(bwd_max_threads(EP)) void router_logits_bwd_kernel(const float* __restrict__ dl,
                                                                 const XT* __restrict__ x,
                                                                 const float* __restrict__ w, int64_t T, int H,
                                                                 int E, int rows_per_block, int groups,
                                                                 int cols_per_block, XT* __restrict__ dx,
                                                                 float* __restrict__ part,
                                                                 RouterGradIn rg = RouterGradIn()) {
    extern __shared__ __attribute__((aligned(16))) float set_sum[];   // [E][cols_per_block]
    __shared__ __attribute__((aligned(16))) float dl_lds[CHAIN ? kChainRows * EP : 4];
    router_logits_bwd_block<XT, EP, EXACT, CHAIN>(dl, x, w, T, H, E, rows_per_block, groups, cols_per_block, dx, part, rg,
                                                  blockIdx.x, blockIdx.y, blockDim.x / groups, set_sum, dl_lds);
}

__global__ __launch_bounds__(kReduceThreads) void router_dw_reduce_kernel(const float* __restrict__ part, int nblocks,
                                                                          int64_t EH, float* __restrict__ d_w) {
    router_dw_reduce_block(part, nblocks, EH, d_w, blockIdx.x);
}

constexpr int kMaxE = 16;
constexpr int kMaxH = 4096;
constexpr int kChunkCols = 4 * MTS_WAVE * 4;        // columns a wave of the forward kernels holds in registers at a time
constexpr size_t kMaxWeightLds = 128 * 1024;        // the forward kernels keep all of W_r [E][H] fp32 in LDS
constexpr int kBwdBlocks = 1024;
constexpr int kHeadMaxBlocks = MTS_HEAD_MAX_CHUNKS;   // blocks of the chained forward kernel = chunks of the routing metadata

int check(const void* x, const float* w, int64_t T, int H, int E, int act_dtype) {
    if (!x || !w) return MTS_ERR_NULL;
    if (T <= 0 || E < 1 || E > kMaxE || H < 4 || H % 4 || H > kMaxH) return MTS_ERR_SHAPE;
    if ((size_t)E * H * sizeof(float) > kMaxWeightLds) return MTS_ERR_SHAPE;   // 4096 columns for 8 experts, 2048 for 16
    if (act_dtype != MTS_BF16 && act_dtype != MTS_F16 && act_dtype != MTS_F32) return MTS_ERR_DTYPE;
    if (!mts_aligned16(w) || (reinterpret_cast<uintptr_t>(x) & 15u)) return MTS_ERR_ALIGN;
    return MTS_OK;
}

int bwd_blocks(int64_t T) { return (int)(T < kBwdBlocks ? T : kBwdBlocks); }

// a kernel whose dynamic LDS, together with `fixed` bytes of static LDS, passes the default limit of
// 64 KiB per block has to say so before the launch
template <typename Kernel>
hipError_t allow_lds(Kernel kernel, size_t bytes, size_t fixed = 0) {
    if (bytes + fixed <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// Block shape of the backward kernel: column ranges (grid.y), column threads per range, row sets per block.
struct BwdShape {
    int ranges, cols_per_block, groups, threads;
};
BwdShape bwd_shape(int H, int E) {
    const int max_threads = bwd_max_threads(E <= 8 ? 8 : 16);
    const int all_threads = ((H / 4 + MTS_WAVE - 1) / MTS_WAVE) * MTS_WAVE;   // one thread per 4 columns
    BwdShape b;
    b.ranges = (all_threads + max_threads - 1) / max_threads;
    const int col_threads = ((all_threads / MTS_WAVE + b.ranges - 1) / b.ranges) * MTS_WAVE;
    b.cols_per_block = b.ranges == 1 ? H : col_threads * 4;
    b.groups = max_threads / col_threads < 4 ? max_threads / col_threads : 4;
    b.threads = b.groups * col_threads;
    return b;
}

}  // namespace

extern "C" int mts_router_logits_fwd(const void* x, const float* w_r, int64_t T, int H, int E, int act_dtype,
                                     float* logits, void* stream) {
    const int rc = check(x, w_r, T, H, E, act_dtype);
    if (rc != MTS_OK) return rc;
    if (!logits) return MTS_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    const int64_t groups = (T + kRows - 1) / kRows;
    int64_t blocks = (groups + 3) / 4;
    if (blocks > 256 * 2) blocks = 256 * 2;
    const dim3 grid((unsigned)blocks);
    const size_t lds = (size_t)E * H * sizeof(float);
    const int passes = (H + MTS_WAVE * 4 - 1) / (MTS_WAVE * 4);   // 256-column slabs per row
    const int n_chunks = (H + kChunkCols - 1) / kChunkCols;
#define MTS_FWD(XT, EP, PS, CH)                                                                                       \
    do {                                                                                                              \
        if (allow_lds(router_logits_fwd_kernel<XT, EP, PS, CH>, lds) != hipSuccess) return MTS_ERR_SHAPE;             \
        router_logits_fwd_kernel<XT, EP, PS, CH><<<grid, kFwdThreads, lds, s>>>((const XT*)x, w_r, T, H, E, n_chunks, logits); \
    } while (0)
#define MTS_FWD_PASSES(XT, EP)                          \
    do {                                                \
        if (passes == 1) MTS_FWD(XT, EP, 1, false);     \
        else if (passes == 2) MTS_FWD(XT, EP, 2, false); \
        else if (passes == 3) MTS_FWD(XT, EP, 3, false); \
        else if (passes == 4) MTS_FWD(XT, EP, 4, false); \
        else MTS_FWD(XT, EP, 4, true);                  \
    } while (0)
    if (act_dtype == MTS_BF16) {
        if (E <= 8) MTS_FWD_PASSES(bf16_t, 8);
        else MTS_FWD_PASSES(bf16_t, 16);
    } else if (act_dtype == MTS_F16) {
        if (E <= 8) MTS_FWD_PASSES(mts_f16_t, 8);
        else MTS_FWD_PASSES(mts_f16_t, 16);
    } else {
        if (E <= 8) MTS_FWD_PASSES(float, 8);
        else MTS_FWD_PASSES(float, 16);
    }
#undef MTS_FWD_PASSES
#undef MTS_FWD
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

// Geometry of the chained forward kernel: blocks, rows per wave (a multiple of kRows); a block's
// rows are one chunk of the routing metadata.
void mts_router_head_geometry(int64_t T, int* blocks, int* rows_per_wave) {
    const int64_t groups = (T + kRows - 1) / kRows;
    int64_t b = (groups + 3) / 4;
    if (b > kHeadMaxBlocks) b = kHeadMaxBlocks;
    const int64_t waves = b * (kFwdThreads / MTS_WAVE);
    const int64_t per_wave = ((T + waves - 1) / waves + kRows - 1) / kRows * kRows;
    *blocks = (int)b;
    *rows_per_wave = (int)per_wave;
}

int mts_launch_router_head(const void* x, const float* w_r, int64_t T, int H, int E, int K, int normalize, int act_dtype,
                           float* logits, float* weights, int32_t* indices, void* weights_act, float* partial,
                           int32_t* cnt, hipStream_t s) {
    const int rc = check(x, w_r, T, H, E, act_dtype);
    if (rc != MTS_OK) return rc;
    if (!logits || !weights || !indices || !partial || !cnt) return MTS_ERR_NULL;
    if (K < 1 || K > E || K > MTS_MAX_TOP_K) return MTS_ERR_SHAPE;
    int blocks, rows_per_wave;
    mts_router_head_geometry(T, &blocks, &rows_per_wave);
    const dim3 grid((unsigned)blocks);
    const size_t lds = (size_t)E * H * sizeof(float);
    const int passes = (H + MTS_WAVE * 4 - 1) / (MTS_WAVE * 4);
    const int n_chunks = (H + kChunkCols - 1) / kChunkCols;
    const int wa_dtype = act_dtype == MTS_F16 ? MTS_F16 : MTS_BF16;   // fp32 activations carry no weights_act (checked by the caller)
#define MTS_HEAD(XT, EP, PS, CH)                                                                                      \
    do {                                                                                                              \
        if (allow_lds(router_head_kernel<XT, EP, PS, CH>, lds, 16 * 1024) != hipSuccess) return MTS_ERR_SHAPE;                   \
        router_head_kernel<XT, EP, PS, CH><<<grid, kFwdThreads, lds, s>>>((const XT*)x, w_r, T, H, E, K, normalize,   \
                                                                          rows_per_wave, n_chunks, logits, weights, indices, \
                                                                          weights_act, wa_dtype, partial, cnt);       \
    } while (0)
#define MTS_HEAD_PASSES(XT, EP)                           \
    do {                                                  \
        if (passes == 1) MTS_HEAD(XT, EP, 1, false);      \
        else if (passes == 2) MTS_HEAD(XT, EP, 2, false); \
        else if (passes == 3) MTS_HEAD(XT, EP, 3, false); \
        else if (passes == 4) MTS_HEAD(XT, EP, 4, false); \
        else MTS_HEAD(XT, EP, 4, true);                   \
    } while (0)
    if (act_dtype == MTS_BF16) {
        if (E <= 8) MTS_HEAD_PASSES(bf16_t, 8);
        else MTS_HEAD_PASSES(bf16_t, 16);
    } else if (act_dtype == MTS_F16) {
        if (E <= 8) MTS_HEAD_PASSES(mts_f16_t, 8);
        else MTS_HEAD_PASSES(mts_f16_t, 16);
    } else {
        if (E <= 8) MTS_HEAD_PASSES(float, 8);
        else MTS_HEAD_PASSES(float, 16);
    }
#undef MTS_HEAD_PASSES
#undef MTS_HEAD
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
    if (workspace_bytes < mts_router_logits_bwd_workspace_bytes(T, H, E)) return MTS_ERR_WORKSPACE;
    if (!mts_aligned16(workspace) || !mts_aligned16(d_w_r) || (reinterpret_cast<uintptr_t>(dx) & 15u)) return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const BwdShape shape = bwd_shape(H, E);
    const int groups = shape.groups, threads = shape.threads;
    int nb = (bwd_blocks(T) + groups - 1) / groups;
    const int rows_per_block = (int)((T + nb - 1) / nb);
    nb = (int)((T + rows_per_block - 1) / rows_per_block);   // every block has at least one row
    const dim3 grid((unsigned)nb, (unsigned)shape.ranges);
    const size_t lds = (size_t)E * shape.cols_per_block * sizeof(float);
    float* part = (float*)workspace;
    const bool vec_dl = mts_aligned16(dlogits);
#define MTS_BWD(XT, EP)                                                                                    \
    do {                                                                                                   \
        if (allow_lds(router_logits_bwd_kernel<XT, EP, true>, lds, 1024) != hipSuccess ||                  \
            allow_lds(router_logits_bwd_kernel<XT, EP, false>, lds, 1024) != hipSuccess)                   \
            return MTS_ERR_SHAPE;                                                                          \
        if (E == EP && vec_dl)                                                                             \
            router_logits_bwd_kernel<XT, EP, true><<<grid, threads, lds, s>>>(dlogits, (const XT*)x, w_r, T, H, E, \
                                                                              rows_per_block, groups, shape.cols_per_block, (XT*)dx, part); \
        else                                                                                               \
            router_logits_bwd_kernel<XT, EP, false><<<grid, threads, lds, s>>>(dlogits, (const XT*)x, w_r, T, H, E, \
                                                                               rows_per_block, groups, shape.cols_per_block, (XT*)dx, part); \
    } while (0)
    if (act_dtype == MTS_BF16) {
        if (E <= 8) MTS_BWD(bf16_t, 8);
        else MTS_BWD(bf16_t, 16);
    } else if (act_dtype == MTS_F16) {
        if (E <= 8) MTS_BWD(mts_f16_t, 8);
        else MTS_BWD(mts_f16_t, 16);
    } else {
        if (E <= 8) MTS_BWD(float, 8);
        else MTS_BWD(float, 16);
    }
#undef MTS_BWD
    MTS_CHECK_LAUNCH();
    const int64_t EH = (int64_t)E * H;
    // blocks of the backward kernel past the last row do not exist: nb * rows_per_block >= T and
    // every block has at least one row when nb <= T
    const int used = (int)((T + rows_per_block - 1) / rows_per_block);
    router_dw_reduce_kernel<<<(unsigned)((EH + kReduceCols - 1) / kReduceCols), kReduceThreads, 0, s>>>(part, used, EH, d_w_r);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

namespace {
int64_t chain_blocks(int64_t T, int groups) {
    int64_t nb = (bwd_blocks(T) + groups - 1) / groups;
    const int64_t need = (T + kChainRows - 1) / kChainRows;   // a block's logit gradients sit in LDS
    return nb > need ? nb : need;
}
}  // namespace

int mts_router_bwd_check(const void* x, const float* w_r, int64_t T, int H, int E, int act_dtype) {
    return check(x, w_r, T, H, E, act_dtype);
}

void mts_router_bwd_shape(int64_t T, int H, int E, MtsRouterBwdShape* out) {
    const BwdShape shape = bwd_shape(H, E);
    int nb = (int)chain_blocks(T, shape.groups);
    const int rows_per_block = (int)((T + nb - 1) / nb);
    nb = (int)((T + rows_per_block - 1) / rows_per_block);
    out->row_blocks = nb;
    out->rows_per_block = rows_per_block;
    out->groups = shape.groups;
    out->col_threads = shape.threads / shape.groups;
    out->cols_per_block = shape.cols_per_block;
    out->ranges = shape.ranges;
}

int mts_launch_router_dw_reduce(const float* part, int row_blocks, int64_t EH, float* d_w_r, hipStream_t s) {
    router_dw_reduce_kernel<<<(unsigned)((EH + kReduceCols - 1) / kReduceCols), kReduceThreads, 0, s>>>(part, row_blocks, EH, d_w_r);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int64_t mts_moe_head_bwd_workspace_bytes(int64_t T, int H, int E) {
    if (T <= 0 || H <= 0 || E <= 0) return 0;
    return chain_blocks(T, 1) * E * H * (int64_t)sizeof(float);
}

extern "C" int mts_moe_head_bwd(const void* x, const float* w_r, const float* logits, const float* weights,
                                const int32_t* indices, const int32_t* counts, const float* g_weights,
                                const void* g_weights_act, const float* g_prob_mean, const float* g_z_loss,
                                const float* g_load_balance, int64_t T, int H, int E, int K, int normalize,
                                int act_dtype, void* dx, float* d_w_r, void* workspace, int64_t workspace_bytes,
                                void* stream) {
    const int rc = check(x, w_r, T, H, E, act_dtype);
    if (rc != MTS_OK) return rc;
    if (!logits || !weights || !indices || !dx || !d_w_r || !workspace) return MTS_ERR_NULL;
    if (g_load_balance && !counts) return MTS_ERR_NULL;
    if (g_weights_act && act_dtype == MTS_F32) return MTS_ERR_DTYPE;   // that gradient comes in a 16-bit activation dtype
    if (K < 1 || K > E || K > MTS_MAX_TOP_K) return MTS_ERR_SHAPE;
    if (workspace_bytes < mts_moe_head_bwd_workspace_bytes(T, H, E)) return MTS_ERR_WORKSPACE;
    if (!mts_aligned16(workspace) || !mts_aligned16(d_w_r) || !mts_aligned16(dx) || (E == 8 && !mts_aligned16(logits)))
        return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const BwdShape shape = bwd_shape(H, E);
    const int groups = shape.groups, threads = shape.threads;
    int nb = (int)chain_blocks(T, groups);
    const int rows_per_block = (int)((T + nb - 1) / nb);
    nb = (int)((T + rows_per_block - 1) / rows_per_block);
    const dim3 grid((unsigned)nb, (unsigned)shape.ranges);
    const size_t lds = (size_t)E * shape.cols_per_block * sizeof(float);
    float* part = (float*)workspace;
    RouterGradIn rg = {logits, weights, indices, counts, g_weights, g_weights_act, g_prob_mean, g_z_loss, g_load_balance,
                       act_dtype, K, normalize, nullptr, nullptr, 0};
#define MTS_CHAIN(XT, EP)                                                                                        \
    do {                                                                                                         \
        if (allow_lds(router_logits_bwd_kernel<XT, EP, false, true>, lds, kChainRows * EP * sizeof(float)) != hipSuccess) \
            return MTS_ERR_SHAPE;                                                                                \
        router_logits_bwd_kernel<XT, EP, false, true><<<grid, threads, lds, s>>>(nullptr, (const XT*)x, w_r, T, H, E, \
                                                                                  rows_per_block, groups,          \
                                                                                  shape.cols_per_block, (XT*)dx, part, rg); \
    } while (0)
    if (act_dtype == MTS_BF16) {
        if (E <= 8) MTS_CHAIN(bf16_t, 8);
        else MTS_CHAIN(bf16_t, 16);
    } else if (act_dtype == MTS_F16) {
        if (E <= 8) MTS_CHAIN(mts_f16_t, 8);
        else MTS_CHAIN(mts_f16_t, 16);
    } else {
        if (E <= 8) MTS_CHAIN(float, 8);
        else MTS_CHAIN(float, 16);
    }
#undef MTS_CHAIN
    MTS_CHECK_LAUNCH();
    const int64_t EH = (int64_t)E * H;
    router_dw_reduce_kernel<<<(unsigned)((EH + kReduceCols - 1) / kReduceCols), kReduceThreads, 0, s>>>(part, nb, EH, d_w_r);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
