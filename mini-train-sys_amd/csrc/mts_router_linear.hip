// Router projection around the post-process kernels: logits = float(x) W_r^T in fp32 and its
// backward (dx in the activation dtype, dW_r in fp32).  x is read in its own dtype, so no fp32
// copy of the activations is made; every sum runs in a fixed order (no float atomics).
// 2*T*H*E FLOP forward, twice that backward: the backward kernels and the forward ones for fp16 / fp32 rows
// run them on the vector pipe; bf16 rows with up to 8 experts take the forward product to the matrix pipe.
#include "mts_common.h"
#include "mts_router_row.h"
#include "mts_router_bwd_block.h"
#include "mts_tuning.h"

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

// ---------------------------------------------------------------------------
// The projection on the matrix pipe (bf16 activations, E <= 8).  An fp32 weight is the exact sum
// of three bf16 terms (each takes the next 8 bits of the mantissa), a bf16 x times a bf16 term is
// exact in fp32, so  x . w  =  x . t0 + x . t1 + x . t2  with fp32 accumulation is an fp32 dot
// product in another order of summation.  The block splits W_r once into LDS, [term][expert][H]
// bf16 = 24 rows (and one of zeros); a wave takes 16 rows of x at a time as the N side of 16x16x32 MFMAs, and the 24
// weight rows as the M side of two of them per k-step, ordered so that lane (n, q) of the
// accumulators (row n of x, q = lane / 16) ends up with the three terms of experts 2q and 2q+1:
//   first MFMA,  M rows 4q .. 4q+3:  (2q, t0) (2q, t1) (2q, t2) (2q+1, t0)
//   second MFMA, M rows 4q .. 4q+3:  (2q+1, t1) (2q+1, t2) zero zero
// A lane reads its row of x straight from memory, 16 bytes per k-step: the four lanes of a row
// read a 128-byte line in two k-steps, 768 columns of it in flight at once.
// ---------------------------------------------------------------------------
constexpr int kMmaRows = 16;          // rows of x per wave pass
constexpr int kMmaSteps = 12;         // k-steps (of 32 columns) per register chunk: two chunks are in flight
constexpr int kMmaTerms = 3;          // bf16 terms of an fp32 weight
constexpr int kMmaMaxH = 2048;        // 25 x (H + 32) bf16 of LDS
constexpr int kStageBatch = 6;        // weight quads a thread has in flight while it splits them
constexpr uint32_t kOutOfRange = 0x80000000u;
typedef __attribute__((ext_vector_type(2))) float f32x2;

__host__ __device__ inline int mma_lds_stride(int H) { return H + 32; }   // elements: consecutive rows 16 banks apart when H % 128 == 0
inline size_t mma_lds_bytes(int H) { return (size_t)(kMmaTerms * 8 + 1) * mma_lds_stride(H) * sizeof(bf16_t); }   // + a row of zeros
inline bool mma_projection_ok(int H, int E, int act_dtype) {
    return mts_tuning().mfma_router && act_dtype == MTS_BF16 && E <= 8 && H % 64 == 0 && H <= kMmaMaxH;
}

// Every thread of the block: W_r [E][H] fp32 -> wb [3][8][stride] bf16 (experts past E are zeros), then a row of zeros.  The loads of a
// batch are issued together (`mma_weights_load`), whatever the caller wants in flight behind them next, and the
// split follows (`mma_weights_split`): returns are in order, so the weights must not queue behind rows of x.
template <int NT>
struct MmaWeights {
    f32x4 v[kStageBatch];
    __device__ __forceinline__ void load(const float* __restrict__ w, int H, int E, int batch) {
        const int quads = H / 4;
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
            const int i = threadIdx.x + (batch * kStageBatch + u) * NT;
            const int e = i / quads, k = (i % quads) * 4;
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            v[u] = (i < 8 * quads && e < E) ? *reinterpret_cast<const f32x4*>(w + (int64_t)e * H + k) : z;
        }
    }
    __device__ __forceinline__ void split(bf16_t* wb, int H, int batch) const {
        const int quads = H / 4, stride = mma_lds_stride(H);
        if (batch == 0) {   // the row of zeros that stands in for the M rows no term maps to
            const bf16x4 z = {};
            for (int k = threadIdx.x * 4; k < H; k += NT * 4) *reinterpret_cast<bf16x4*>(wb + kMmaTerms * 8 * stride + k) = z;
        }
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
            const int i = threadIdx.x + (batch * kStageBatch + u) * NT;
            if (i >= 8 * quads) continue;
            const int e = i / quads, k = (i % quads) * 4;
            bf16x4 t0, t1, t2;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float a = v[u][q];
                bf16_t h = (bf16_t)a;
                // A NaN or infinite weight is carried by the first term alone (inf - inf would turn an infinite weight
                // into NaN logits where the fp32 dot product gives inf); a finite weight that rounds up to infinity
                // is truncated instead, and the terms behind it carry the rest as for every other weight.
                const bool finite = __builtin_isfinite(a);
                if (finite && !__builtin_isfinite((float)h)) h = __builtin_bit_cast(bf16_t, (uint16_t)(__float_as_uint(a) >> 16));
                t0[q] = h;
                const float r1 = finite ? a - (float)h : 0.f;   // exact
                t1[q] = (bf16_t)r1;
                const float r2 = r1 - (float)t1[q];  // exact, 8 bits or fewer are left
                t2[q] = (bf16_t)r2;
            }
            *reinterpret_cast<bf16x4*>(wb + (0 * 8 + e) * stride + k) = t0;
            *reinterpret_cast<bf16x4*>(wb + (1 * 8 + e) * stride + k) = t1;
            *reinterpret_cast<bf16x4*>(wb + (2 * 8 + e) * stride + k) = t2;
        }
    }
    static __device__ __forceinline__ int batches(int H) { return (8 * (H / 4) + kStageBatch * NT - 1) / (kStageBatch * NT); }
};

// First column of the 8 that quarter q (= lane / 16) of a row contributes to k-step `step`.  Which 32 columns
// make up a k-step is free as long as both operands agree: two consecutive k-steps share 64 columns and a
// quarter's two pieces are adjacent, so the four lanes of a row ask for a whole 128-byte line in two loads.
__device__ __forceinline__ int mma_col(int step, int q) { return 64 * (step / 2) + 16 * q + 8 * (step % 2); }

struct MmaRows {
    __amdgpu_buffer_rsrc_t rsrc;   // the wave's rows r0 .. min(r0 + 16, end), so that rows past the end read as zeros
    uint32_t row_off;
};
__device__ __forceinline__ MmaRows mma_rows(const bf16_t* x, int64_t r0, int64_t end, int H, int lane) {
    // r0 and end are the same for the whole wave; say so, a descriptor lives in scalar registers
    const int64_t first = ((int64_t)__builtin_amdgcn_readfirstlane((int)(r0 >> 32)) << 32) |
                          (uint32_t)__builtin_amdgcn_readfirstlane((int)r0);
    const int64_t left = end - r0 < kMmaRows ? end - r0 : kMmaRows;
    const int rows = __builtin_amdgcn_readfirstlane((int)(left > 0 ? left : 0));
    MmaRows m;
    m.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(x + first * H), 0, rows * H * 2, 0x00020000);
    m.row_off = (uint32_t)(lane % 16) * (uint32_t)H * 2u;
    return m;
}
// chunk `ch` of the lane's row: k-steps ch*12 .. ch*12 + 11, see mma_col
__device__ __forceinline__ void mma_load_chunk(u32x4 (&dst)[kMmaSteps], const MmaRows& m, int ch, int H, int lane) {
#pragma unroll
    for (int j = 0; j < kMmaSteps; ++j) {
        const int col = mma_col(ch * kMmaSteps + j, lane / 16);
        dst[j] = __builtin_amdgcn_raw_buffer_load_b128(m.rsrc, (int)(col < H ? m.row_off + (uint32_t)col * 2u : kOutOfRange), 0, 0);
    }
}
// the LDS rows this lane reads as M row lane % 16 of the first and of the second MFMA
struct MmaLaneRows {
    const bf16_t* first;
    const bf16_t* second;
};
__device__ __forceinline__ MmaLaneRows mma_lane_rows(const bf16_t* wb, int H, int lane) {
    const int stride = mma_lds_stride(H), m = lane % 16, q = m / 4, i = m % 4, k0 = 16 * (lane / 16);
    MmaLaneRows r;
    const int e1 = i == 3 ? 2 * q + 1 : 2 * q, t1 = i == 3 ? 0 : i;
    r.first = wb + (t1 * 8 + e1) * stride + k0;
    r.second = wb + (i < 2 ? (i + 1) * 8 + 2 * q + 1 : kMmaTerms * 8) * stride + k0;   // row 24 holds zeros
    return r;
}
template <bool WHOLE>   // WHOLE: all k-steps of the chunk lie inside the row, no test per step (the fragment reads can then run ahead)
__device__ __forceinline__ void mma_chunk_steps(f32x4 (&acc)[2][2], const u32x4 (&cur)[kMmaSteps], const MmaLaneRows& rows,
                                                int ch, int H) {
#pragma unroll
    for (int j = 0; j < kMmaSteps; ++j) {
        const int col = mma_col(ch * kMmaSteps + j, 0);   // the lane's quarter is part of its row pointers
        if (WHOLE || col < H) {   // wave-uniform: H is a multiple of 64
            const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(rows.first + col);
            const bf16x8 a2 = *reinterpret_cast<const bf16x8*>(rows.second + col);
            const bf16x8 b = __builtin_bit_cast(bf16x8, cur[j]);
            acc[j & 1][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b, acc[j & 1][0], 0, 0, 0);
            acc[j & 1][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b, acc[j & 1][1], 0, 0, 0);
        }
    }
}
__device__ __forceinline__ void mma_chunk(f32x4 (&acc)[2][2], const u32x4 (&cur)[kMmaSteps], const MmaLaneRows& rows, int ch,
                                          int H) {
    if ((ch + 1) * kMmaSteps * 32 <= H) mma_chunk_steps<true>(acc, cur, rows, ch, H);
    else mma_chunk_steps<false>(acc, cur, rows, ch, H);
}
// Chunk number p of the wave's stream of chunks, counted from chunk 0 of the rows at r0: the wave's row groups lie
// `step` rows apart and have nch chunks each.  Nothing is loaded past `end`.
__device__ __forceinline__ void mma_prefetch(u32x4 (&dst)[kMmaSteps], const bf16_t* x, int64_t r0, int64_t step, int64_t end,
                                             int H, int nch, int p, int lane) {
    const int64_t rb = r0 + (p / nch) * step;
    if (rb < end) mma_load_chunk(dst, mma_rows(x, rb, end, H, lane), p % nch, H, lane);
}
__device__ __forceinline__ int mma_chunks(int H) { return (H + kMmaSteps * 32 - 1) / (kMmaSteps * 32); }
// logits of experts 2 (lane / 16) and 2 (lane / 16) + 1 of row r0 + lane % 16.  On entry `cur` and `nxt` hold chunks
// 0 and 1 of the stream that starts at r0, on return those of the stream that starts at r0 + step.
__device__ __forceinline__ void mma_project(float (&out)[2], u32x4 (&cur)[kMmaSteps], u32x4 (&nxt)[kMmaSteps], const bf16_t* x,
                                            int64_t r0, int64_t step, int64_t end, int H, const bf16_t* wb, int lane) {
    const int nch = mma_chunks(H);
    const MmaLaneRows lrows = mma_lane_rows(wb, H, lane);
    f32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[0][0][i] = acc[0][1][i] = acc[1][0][i] = acc[1][1][i] = 0.f;
    for (int ch = 0; ch < nch; ++ch) {
        mma_chunk(acc, cur, lrows, ch, H);
#pragma unroll
        for (int j = 0; j < kMmaSteps; ++j) cur[j] = nxt[j];
        mma_prefetch(nxt, x, r0, step, end, H, nch, ch + 2, lane);
    }
    // accumulator element i of lane (n, q): M row 4q + i
    const f32x4 one = acc[0][0] + acc[1][0], two = acc[0][1] + acc[1][1];
    out[0] = (one[2] + one[1]) + one[0];   // small terms first
    out[1] = (two[1] + two[0]) + one[3];
}

// logits only: a wave takes every (waves)th group of 16 rows
__global__ __launch_bounds__(kFwdThreads) void router_logits_mma_kernel(const bf16_t* __restrict__ x,
                                                                         const float* __restrict__ w, int64_t T, int H,
                                                                         int E, float* __restrict__ logits) {
    extern __shared__ __attribute__((aligned(16))) float w_lds[];
    bf16_t* wb = reinterpret_cast<bf16_t*>(w_lds);
    const int lane = threadIdx.x % MTS_WAVE;
    const int64_t stride = (int64_t)gridDim.x * (kFwdThreads / MTS_WAVE) * kMmaRows;
    int64_t r0 = ((int64_t)blockIdx.x * (kFwdThreads / MTS_WAVE) + threadIdx.x / MTS_WAVE) * kMmaRows;
    u32x4 cur[kMmaSteps], nxt[kMmaSteps];
    MmaWeights<kFwdThreads> stage;
    stage.load(w, H, E, 0);
    mma_prefetch(cur, x, r0, stride, T, H, mma_chunks(H), 0, lane);
    mma_prefetch(nxt, x, r0, stride, T, H, mma_chunks(H), 1, lane);
    stage.split(wb, H, 0);
    for (int b = 1; b < stage.batches(H); ++b) {
        stage.load(w, H, E, b);
        stage.split(wb, H, b);
    }
    __syncthreads();
    for (; r0 < T; r0 += stride) {
        float lg[2];
        mma_project(lg, cur, nxt, x, r0, stride, T, H, wb, lane);
        const int64_t row = r0 + lane % 16;
        if (row < T) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int e = 2 * (lane / 16) + q;
                if (e < E) logits[row * E + e] = lg[q];
            }
        }
    }
}

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
template <typename XT, int EP, int PASSES, bool CHUNKED = false, bool MMA = false>
__global__ __launch_bounds__(kFwdThreads, MMA ? 2 : 1) void router_head_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, int64_t T, int H, int E, int K, int normalize,
    int rows_per_wave, int n_chunks, float* __restrict__ logits, float* __restrict__ weights, int32_t* __restrict__ indices,
    void* __restrict__ weights_act, int act_dtype, float* __restrict__ partial, int32_t* __restrict__ cnt) {
    using namespace mts_router;
    static_assert(!MMA || (EP == 8 && sizeof(XT) == 2 && !CHUNKED), "the matrix-pipe projection: bf16 rows, up to 8 experts");
    extern __shared__ __attribute__((aligned(16))) float w_lds[];   // [E][H] fp32, or the bf16 terms of the matrix-pipe path
    constexpr int WAVES = kFwdThreads / MTS_WAVE;
    constexpr int GROUP = MMA ? kMmaRows : kRows;   // rows whose logits are complete together
    const int lane = threadIdx.x % MTS_WAVE, wave = threadIdx.x / MTS_WAVE;
    const int nch = CHUNKED ? n_chunks : 1;
    const int64_t beg = ((int64_t)blockIdx.x * WAVES + wave) * rows_per_wave;
    const int64_t end = beg + rows_per_wave < T ? beg + rows_per_wave : T;
    typedef RowGroupLoader<XT, PASSES> Loader;
    typename Loader::raw_t cur[PASSES][kRows], nxt[PASSES][kRows];
    u32x4 mcur[MMA ? kMmaSteps : 1], mnxt[MMA ? kMmaSteps : 1];
    if constexpr (MMA) {
        // the first rows are on their way while the block splits the weights
        MmaWeights<kFwdThreads> stage;
        stage.load(w, H, E, 0);
        mma_prefetch(mcur, reinterpret_cast<const bf16_t*>(x), beg, kMmaRows, end, H, mma_chunks(H), 0, lane);
        mma_prefetch(mnxt, reinterpret_cast<const bf16_t*>(x), beg, kMmaRows, end, H, mma_chunks(H), 1, lane);
        stage.split(reinterpret_cast<bf16_t*>(w_lds), H, 0);
        for (int b = 1; b < stage.batches(H); ++b) {
            stage.load(w, H, E, b);
            stage.split(reinterpret_cast<bf16_t*>(w_lds), H, b);
        }
    } else {
#pragma unroll 8
        for (int i = threadIdx.x * 4; i < E * H; i += kFwdThreads * 4)
            *reinterpret_cast<f32x4*>(w_lds + i) = *reinterpret_cast<const f32x4*>(w + i);
        if (beg < end) Loader::load(cur, x, beg, end, 0, H, lane);
    }
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
        int64_t g0;   // the row group whose dot products are complete
        if constexpr (MMA) {
            float lg[2];
            mma_project(lg, mcur, mnxt, reinterpret_cast<const bf16_t*>(x), r0, kMmaRows, end, H,
                        reinterpret_cast<const bf16_t*>(w_lds), lane);
            g0 = r0;
            r0 += kMmaRows;
            const int r = lane % 16;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int e = 2 * (lane / 16) + q;
                if (e < E && g0 + r < end) logits[(g0 + r) * E + e] = lg[q];
                mine_rows[(int)(g0 - pass_base + r) * LROW + e] = e < E ? lg[q] : -INFINITY;
            }
        } else {
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
        g0 = r0;   // complete when `last`
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
        }
        const int64_t parked_to = g0 + GROUP < end ? g0 + GROUP : end;
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
    if (mma_projection_ok(H, E, act_dtype)) {
        int64_t nb = ((T + kMmaRows - 1) / kMmaRows + 3) / 4;
        if (nb > 256 * 2) nb = 256 * 2;
        const size_t bytes = mma_lds_bytes(H);
        if (allow_lds(router_logits_mma_kernel, bytes) != hipSuccess) return MTS_ERR_SHAPE;
        router_logits_mma_kernel<<<dim3((unsigned)nb), kFwdThreads, bytes, s>>>((const bf16_t*)x, w_r, T, H, E, logits);
        MTS_CHECK_LAUNCH();
        return MTS_OK;
    }
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
int mts_router_head_group(int H, int E, int act_dtype) { return mma_projection_ok(H, E, act_dtype) ? kMmaRows : kRows; }

void mts_router_head_geometry(int64_t T, int group, int* blocks, int* rows_per_wave) {
    const int64_t groups = (T + group - 1) / group;
    int64_t b = (groups + 3) / 4;
    if (b > kHeadMaxBlocks) b = kHeadMaxBlocks;
    const int64_t waves = b * (kFwdThreads / MTS_WAVE);
    const int64_t per_wave = ((T + waves - 1) / waves + group - 1) / group * group;
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
    mts_router_head_geometry(T, mts_router_head_group(H, E, act_dtype), &blocks, &rows_per_wave);
    const dim3 grid((unsigned)blocks);
    if (mma_projection_ok(H, E, act_dtype)) {
        const size_t bytes = mma_lds_bytes(H);
        if (allow_lds(router_head_kernel<bf16_t, 8, 1, false, true>, bytes, 16 * 1024) != hipSuccess) return MTS_ERR_SHAPE;
        router_head_kernel<bf16_t, 8, 1, false, true><<<grid, kFwdThreads, bytes, s>>>(
            (const bf16_t*)x, w_r, T, H, E, K, normalize, rows_per_wave, 1, logits, weights, indices, weights_act, MTS_BF16,
            partial, cnt);
        MTS_CHECK_LAUNCH();
        return MTS_OK;
    }
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
