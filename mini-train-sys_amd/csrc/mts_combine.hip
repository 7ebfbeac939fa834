// HBM-bound helpers around the grouped GEMMs: the per-token weighted sum of
// expert rows (combine), the routing-weight gradient reduction and the staging
// (cast / transpose) of expert weights to bf16.
#include "mts_common.h"
#include "mts_combine_block.h"

namespace {

constexpr int kThreads = 256;

// ---- combine -------------------------------------------------------------
// the stand-alone launch of the block function in mts_combine_block.h
using mts_cb::Vec8;

template <typename ET, int KK, int UN>
__global__ __launch_bounds__(kThreads) void combine_bf16_kernel(
    const ET* __restrict__ y, const ET* __restrict__ w, const ET* __restrict__ addend,
    const int32_t* __restrict__ s_rev, int64_t T, int K, int H, ET* __restrict__ out) {
    static_assert(kThreads == mts_cb::kCombineThreads, "one block shape");
    mts_cb::combine_rows_block<ET, KK, UN>(y, w, addend, s_rev, T, K, H, out, blockIdx.x, gridDim.x);
}

// any K: the routes of a token are visited in a loop
template <typename ET>
__global__ __launch_bounds__(kThreads) void combine_bf16_anyk_kernel(
    const ET* __restrict__ y, const ET* __restrict__ w, const ET* __restrict__ addend,
    const int32_t* __restrict__ s_rev, int64_t T, int K, int H, ET* __restrict__ out) {
    typedef typename Vec8<ET>::type bf16x8;
    const int vec_per_row = H / 8;
    const int64_t total = T * (int64_t)vec_per_row;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * kThreads) {
        const int64_t t = i / vec_per_row;
        const int c = (int)(i - t * vec_per_row);
        float acc[8];
        const bf16x8 add = addend ? *reinterpret_cast<const bf16x8*>(addend + t * H + c * 8) : bf16x8{};
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = (float)add[j];
        for (int k = 0; k < K; ++k) {
            const int64_t row = s_rev[t * K + k];
            if (row < 0) continue;
            const float s = w ? (float)w[t * K + k] : 1.0f;
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(y + row * H + c * 8);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += s * (float)v[j];
        }
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (ET)acc[j];
        *reinterpret_cast<bf16x8*>(out + t * H + c * 8) = o;
    }
}

__global__ __launch_bounds__(kThreads) void combine_f32_kernel(
    const float* __restrict__ y, const float* __restrict__ w, const float* __restrict__ addend,
    const int32_t* __restrict__ s_rev, int64_t T, int K, int H, float* __restrict__ out) {
    const int vec_per_row = H / 4;
    const int64_t total = T * (int64_t)vec_per_row;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * kThreads) {
        const int64_t t = i / vec_per_row;
        const int c = (int)(i - t * vec_per_row);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (addend) acc = *reinterpret_cast<const f32x4*>(addend + t * H + c * 4);
        for (int k = 0; k < K; ++k) {
            const int64_t row = s_rev[t * K + k];
            if (row < 0) continue;
            const float s = w ? w[t * K + k] : 1.0f;
            const f32x4 v = *reinterpret_cast<const f32x4*>(y + row * H + c * 4);
            acc += s * v;
        }
        *reinterpret_cast<f32x4*>(out + t * H + c * 4) = acc;
    }
}

// ---- routing-weight gradient ---------------------------------------------
template <typename OutT>
__global__ __launch_bounds__(kThreads) void ds_reduce_kernel(const float* __restrict__ part,
                                                             const int32_t* __restrict__ s_rev,
                                                             int64_t TK, int np,
                                                             OutT* __restrict__ d_w) {
    for (int64_t n = (int64_t)blockIdx.x * kThreads + threadIdx.x; n < TK;
         n += (int64_t)gridDim.x * kThreads) {
        const int32_t r = s_rev[n];   // negative: dropped route, no gradient
        float v = 0.f;
        if (r >= 0) {
            const float* p = part + (int64_t)r * np;
            for (int j = 0; j < np; ++j) v += p[j];
        }
        d_w[n] = (OutT)v;
    }
}

// ---- weight staging --------------------------------------------------------
// 64x64 tiles through LDS; reads and writes are both row-contiguous.
template <typename SrcT, typename DstT, bool TRANSPOSE>
__global__ __launch_bounds__(kThreads) void stage_weights_kernel(const SrcT* __restrict__ src,
                                                                 DstT* __restrict__ dst,
                                                                 int64_t R, int64_t C) {
    __shared__ DstT tile[64][64 + 2];
    const int64_t e = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const SrcT* s = src + e * R * C;
    DstT* d = dst + e * R * C;
    const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    for (int i = ty; i < 64; i += kThreads / 64) {
        int64_t r = r0 + i, c = c0 + tx;
        if (r < R && c < C) {
            DstT v = (DstT)(float)s[r * C + c];
            if (TRANSPOSE) tile[i][tx] = v;
            else d[r * C + c] = v;
        }
    }
    if (!TRANSPOSE) return;
    __syncthreads();
    for (int i = ty; i < 64; i += kThreads / 64) {
        int64_t c = c0 + i, r = r0 + tx;  // output row = source column
        if (r < R && c < C) d[c * R + r] = tile[tx][i];
    }
}

// bf16 -> bf16 transpose with 16-byte global accesses: a block moves a 64x64 tile; a thread
// reads 8 consecutive source elements of two rows, and writes 8 consecutive elements of two
// output rows (8 consecutive source rows of one column, gathered from LDS).  The tile rows are
// padded to 66 elements so that the column gather spreads over the banks.
__global__ __launch_bounds__(kThreads) void transpose_bf16_kernel(const bf16_t* __restrict__ src,
                                                                  bf16_t* __restrict__ dst, int R, int C) {
    __shared__ bf16_t tile[64][66];
    const int64_t e = blockIdx.z;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const bf16_t* s = src + e * (int64_t)R * C;
    bf16_t* d = dst + e * (int64_t)R * C;
    const int v = threadIdx.x % 8, rr = threadIdx.x / 8;   // 8 vectors per tile row, 32 rows per pass
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int r = rr + 32 * h;
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(s + (int64_t)(r0 + r) * C + c0 + v * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[r][v * 8 + j] = x[j];
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int c = rr + 32 * h;   // source column = output row
        bf16x8 y;
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = tile[v * 8 + j][c];
        *reinterpret_cast<bf16x8*>(d + (int64_t)(c0 + c) * R + r0 + v * 8) = y;
    }
}

int grid_1d(int64_t total) {
    int64_t b = (total + kThreads - 1) / kThreads;
    const int64_t cap = 256 * 32;
    return (int)(b < cap ? (b > 0 ? b : 1) : cap);
}

}  // namespace

extern "C" int mts_moe_combine(const void* y, const void* weights, const void* addend, const int32_t* s_reverse,
                               int64_t T, int K, int H, int act_dtype, void* out, void* stream) {
    if (!y || !s_reverse || !out) return MTS_ERR_NULL;
    if (T <= 0 || K < 1 || H < 1) return MTS_ERR_SHAPE;
    if (!mts_aligned16(y) || !mts_aligned16(out) || !mts_aligned16(addend)) return MTS_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    if (act_dtype == MTS_BF16 || act_dtype == MTS_F16) {
        if (H % 8) return MTS_ERR_SHAPE;
        constexpr int UN = 2;
        const int64_t sliced = ((T + UN - 1) / UN) * (int64_t)(H / 8);
#define MTS_COMBINE16(ET)                                                                                     \
    do {                                                                                                      \
        if (K <= 2)                                                                                           \
            combine_bf16_kernel<ET, 2, UN><<<grid_1d(sliced), kThreads, 0, s>>>(                              \
                (const ET*)y, (const ET*)weights, (const ET*)addend, s_reverse, T, K, H, (ET*)out);                              \
        else if (K <= 4)                                                                                      \
            combine_bf16_kernel<ET, 4, UN><<<grid_1d(sliced), kThreads, 0, s>>>(                              \
                (const ET*)y, (const ET*)weights, (const ET*)addend, s_reverse, T, K, H, (ET*)out);                              \
        else                                                                                                  \
            combine_bf16_anyk_kernel<ET><<<grid_1d(T * (int64_t)(H / 8)), kThreads, 0, s>>>(                  \
                (const ET*)y, (const ET*)weights, (const ET*)addend, s_reverse, T, K, H, (ET*)out);                              \
    } while (0)
        if (act_dtype == MTS_BF16) MTS_COMBINE16(bf16_t);
        else MTS_COMBINE16(mts_f16_t);
#undef MTS_COMBINE16
    } else if (act_dtype == MTS_F32) {
        if (H % 4) return MTS_ERR_SHAPE;
        combine_f32_kernel<<<grid_1d(T * (int64_t)(H / 4)), kThreads, 0, s>>>(
            (const float*)y, (const float*)weights, (const float*)addend, s_reverse, T, K, H, (float*)out);
    } else {
        return MTS_ERR_DTYPE;
    }
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int mts_moe_bwd_ds(const float* ds_partial, const int32_t* s_reverse, int64_t TK, int I,
                              int act_dtype, void* d_weights, void* stream) {
    if (!ds_partial || !s_reverse || !d_weights) return MTS_ERR_NULL;
    if (TK <= 0 || I < 1) return MTS_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const int np = mts_moe_ds_partials(I);
    if (act_dtype == MTS_BF16)
        ds_reduce_kernel<bf16_t><<<grid_1d(TK), kThreads, 0, s>>>(ds_partial, s_reverse, TK, np,
                                                                  (bf16_t*)d_weights);
    else if (act_dtype == MTS_F16)
        ds_reduce_kernel<mts_f16_t><<<grid_1d(TK), kThreads, 0, s>>>(ds_partial, s_reverse, TK, np,
                                                                     (mts_f16_t*)d_weights);
    else if (act_dtype == MTS_F32)
        ds_reduce_kernel<float><<<grid_1d(TK), kThreads, 0, s>>>(ds_partial, s_reverse, TK, np,
                                                                 (float*)d_weights);
    else
        return MTS_ERR_DTYPE;
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

template <typename SrcT, typename DstT>
void launch_stage(const void* src, void* dst, dim3 grid, int64_t R, int64_t C, int transpose, hipStream_t s) {
    if (transpose) stage_weights_kernel<SrcT, DstT, true><<<grid, kThreads, 0, s>>>((const SrcT*)src, (DstT*)dst, R, C);
    else stage_weights_kernel<SrcT, DstT, false><<<grid, kThreads, 0, s>>>((const SrcT*)src, (DstT*)dst, R, C);
}

extern "C" int mts_moe_stage_weights(const void* src, int src_dtype, void* dst, int dst_dtype, int E,
                                     int64_t R, int64_t C, int transpose, void* stream) {
    if (!src || !dst) return MTS_ERR_NULL;
    if (E < 1 || R < 1 || C < 1 || E > 65535) return MTS_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)E);
    if (grid.y > 65535) return MTS_ERR_SHAPE;
    if (src_dtype == dst_dtype && (src_dtype == MTS_BF16 || src_dtype == MTS_F16) && transpose && R % 64 == 0 && C % 64 == 0 &&
        mts_aligned16(src) && mts_aligned16(dst) && R <= 0x7fffffff && C <= 0x7fffffff)
        transpose_bf16_kernel<<<grid, kThreads, 0, s>>>((const bf16_t*)src, (bf16_t*)dst, (int)R, (int)C);
    else if (src_dtype == MTS_F32 && dst_dtype == MTS_BF16) launch_stage<float, bf16_t>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_BF16 && dst_dtype == MTS_BF16) launch_stage<bf16_t, bf16_t>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_F32 && dst_dtype == MTS_F32) launch_stage<float, float>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_BF16 && dst_dtype == MTS_F32) launch_stage<bf16_t, float>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_F32 && dst_dtype == MTS_F16) launch_stage<float, mts_f16_t>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_F16 && dst_dtype == MTS_F16) launch_stage<mts_f16_t, mts_f16_t>(src, dst, grid, R, C, transpose, s);
    else if (src_dtype == MTS_F16 && dst_dtype == MTS_F32) launch_stage<mts_f16_t, float>(src, dst, grid, R, C, transpose, s);
    else return MTS_ERR_DTYPE;
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

// fp32 -> 16-bit casts of both expert weights in one launch: a thread turns eight consecutive fp32 values
// (two 16-byte loads) into one 16-byte store; the first n1 / 8 items belong to the first tensor.
template <typename DstT>
__global__ __launch_bounds__(kThreads) void cast_pair_kernel(const float* __restrict__ a, DstT* __restrict__ da, int64_t n1,
                                                             const float* __restrict__ b, DstT* __restrict__ db, int64_t n2) {
    typedef typename Vec8<DstT>::type vec8;
    const int64_t items1 = n1 / 8, items = items1 + n2 / 8;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < items; i += (int64_t)gridDim.x * kThreads) {
        const bool first = i < items1;
        const float* src = (first ? a : b) + (first ? i : i - items1) * 8;
        DstT* dst = (first ? da : db) + (first ? i : i - items1) * 8;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(src), hi = *reinterpret_cast<const f32x4*>(src + 4);
        vec8 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[j] = (DstT)lo[j];
            v[4 + j] = (DstT)hi[j];
        }
        *reinterpret_cast<vec8*>(dst) = v;
    }
}

extern "C" int mts_moe_cast_weights_pair(const float* w1, void* w1_out, int64_t n1, const float* w2, void* w2_out, int64_t n2,
                                         int dst_dtype, void* stream) {
    if (!w1 || !w1_out || !w2 || !w2_out) return MTS_ERR_NULL;
    if (n1 < 8 || n2 < 8 || n1 % 8 || n2 % 8) return MTS_ERR_SHAPE;
    if (!mts_aligned16(w1) || !mts_aligned16(w1_out) || !mts_aligned16(w2) || !mts_aligned16(w2_out)) return MTS_ERR_ALIGN;
    const int blocks = grid_1d((n1 + n2) / 8);
    hipStream_t s = (hipStream_t)stream;
    if (dst_dtype == MTS_BF16) cast_pair_kernel<bf16_t><<<blocks, kThreads, 0, s>>>(w1, (bf16_t*)w1_out, n1, w2, (bf16_t*)w2_out, n2);
    else if (dst_dtype == MTS_F16) cast_pair_kernel<mts_f16_t><<<blocks, kThreads, 0, s>>>(w1, (mts_f16_t*)w1_out, n1, w2, (mts_f16_t*)w2_out, n2);
    else return MTS_ERR_DTYPE;
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int mts_version(void) { return MTS_VERSION; }

extern "C" const char* mts_error_string(int code) {
    switch (code) {
        case MTS_OK: return "ok";
        case MTS_ERR_NULL: return "a required pointer is NULL";
        case MTS_ERR_SHAPE: return "sizes outside the supported range";
        case MTS_ERR_DTYPE: return "unsupported element type";
        case MTS_ERR_WORKSPACE: return "workspace too small";
        case MTS_ERR_ALIGN: return "pointer or leading dimension not 16-byte aligned";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}
