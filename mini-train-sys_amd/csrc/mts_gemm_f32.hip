// fp32 variant of the grouped expert GEMMs (activations, weights and accumulation
// all in fp32, plain FMA): the small debug configuration of the layer and fp32
// parity checks run through it.  Same contracts and epilogues as the bf16 MFMA
// kernels; throughput is not a goal here.
//
// 64x64 output tile per 256-thread block, 16-wide k-steps through LDS, 4x4 outputs
// per thread.  Row tiles follow the expert segments exactly as in the bf16 path.
#include "mts_common.h"

namespace {

constexpr int TB = 64;   // tile rows and columns
constexpr int TKS = 16;  // k-step
constexpr int kThreads = 256;

enum Epi32 { E32_PLAIN = 0, E32_SWIGLU = 1, E32_DY1 = 2 };

struct Rows32 {
    const float* A;
    int lda;
    const int32_t* a_gather;
    const float* B;      // [E][b_rows][Kdim]
    int b_rows;
    int N, Kdim;
    const int32_t* expert_start;
    int E;
    float* C;
    float* C2;
    const float* pre_act;
    const float* route_w;
    const int32_t* s_scatter;
    float* ds_part;
    int np;
};

__device__ __forceinline__ float sigmoid32(float x) { return 1.0f / (1.0f + expf(-x)); }

template <int EPI>
__global__ __launch_bounds__(kThreads) void rows_gemm_f32_kernel(Rows32 p) {
    constexpr int NB = (EPI == E32_SWIGLU) ? 2 : 1;  // B tiles per block (gate and up)
    __shared__ float As[TKS][TB + 4];
    __shared__ float Bs[NB][TKS][TB + 4];

    int e = 0, row0 = 0, rend = 0;
    {
        int tile = blockIdx.x, seen = 0;
        bool found = false;
        for (e = 0; e < p.E; ++e) {
            const int s0 = p.expert_start[e], s1 = p.expert_start[e + 1];
            const int nt = (s1 - s0 + TB - 1) / TB;
            if (tile < seen + nt) {
                row0 = s0 + (tile - seen) * TB;
                rend = s1;
                found = true;
                break;
            }
            seen += nt;
        }
        if (!found) return;
    }
    const int n0 = blockIdx.y * TB;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;

    // loader: thread -> (tile row lr, four consecutive k)
    const int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
    const float* a_ptr = nullptr;
    if (row0 + lr < rend) {
        const int64_t src = p.a_gather ? p.a_gather[row0 + lr] : row0 + lr;
        a_ptr = p.A + src * p.lda;
    }
    const float* Be = p.B + (int64_t)e * p.b_rows * p.Kdim;
    const float* b_ptr[NB];
#pragma unroll
    for (int h = 0; h < NB; ++h)
        b_ptr[h] = (n0 + lr < p.N) ? Be + (int64_t)(h * p.N + n0 + lr) * p.Kdim : nullptr;

    float acc[NB][4][4];
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[h][i][j] = 0.f;

    for (int k0 = 0; k0 < p.Kdim; k0 += TKS) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int k = k0 + lk + q;
            As[lk + q][lr] = (a_ptr && k < p.Kdim) ? a_ptr[k] : 0.f;
#pragma unroll
            for (int h = 0; h < NB; ++h) Bs[h][lk + q][lr] = (b_ptr[h] && k < p.Kdim) ? b_ptr[h][k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TKS; ++k) {
            float a[4], b[NB][4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int h = 0; h < NB; ++h)
#pragma unroll
                for (int j = 0; j < 4; ++j) b[h][j] = Bs[h][k][tx * 4 + j];
#pragma unroll
            for (int h = 0; h < NB; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[h][i][j] = fmaf(a[i], b[h][j], acc[h][i][j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = row0 + ty * 4 + i;
        const bool rok = row < rend;
        float s = 0.f, dsp = 0.f;
        if (EPI == E32_DY1 && rok) s = p.route_w[p.s_scatter[row]];
        if (EPI == E32_SWIGLU) s = (rok && p.route_w) ? p.route_w[p.s_scatter[row]] : 1.f;   // post_act may carry the routing weight
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (!rok || n >= p.N) continue;
            if (EPI == E32_PLAIN) {
                p.C[(int64_t)row * p.N + n] = acc[0][i][j];
            } else if (EPI == E32_SWIGLU) {
                const float g = acc[0][i][j], u = acc[NB - 1][i][j];
                p.C[(int64_t)row * (2 * p.N) + n] = g;
                p.C[(int64_t)row * (2 * p.N) + p.N + n] = u;
                p.C2[(int64_t)row * p.N + n] = g * sigmoid32(g) * u * s;
            } else {
                const int64_t o = (int64_t)row * (2 * p.N) + n;
                const float g = p.pre_act[o], u = p.pre_act[o + p.N];
                const float a = acc[0][i][j];
                const float sig = sigmoid32(g);
                const float silu = g * sig;
                const float y1 = silu * u;
                dsp += a * y1;
                if (p.C2) p.C2[(int64_t)row * p.N + n] = s * y1;
                const float da = a * s;
                p.C[o] = da * (silu * (1.0f - sig) + sig) * u;
                p.C[o + p.N] = da * silu;
            }
        }
        if (EPI == E32_DY1) {
            // the 16 threads that share `ty` hold the 64 columns of this row
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) dsp += __shfl_xor(dsp, o, MTS_WAVE);
            if (rok && tx == 0) p.ds_part[(int64_t)row * p.np + blockIdx.y] = dsp;
        }
    }
}

struct Dw32 {
    const float* P;
    const int32_t* p_gather;
    const float* Q;
    const int32_t* q_gather;
    int M, N;
    const int32_t* expert_start;
    void* C;
};

template <typename OutT>
__global__ __launch_bounds__(kThreads) void dw_gemm_f32_kernel(Dw32 p) {
    __shared__ float Ps[TKS][TB + 4];
    __shared__ float Qs[TKS][TB + 4];
    const int e = blockIdx.z;
    const int m0 = blockIdx.x * TB, n0 = blockIdx.y * TB;
    const int rbeg = p.expert_start[e], rend = p.expert_start[e + 1];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int lk = threadIdx.x / 16, lc = (threadIdx.x % 16) * 4;  // loader: (k row, four columns)

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int r0 = rbeg; r0 < rend; r0 += TKS) {
        const int r = r0 + lk;
        const bool ok = r < rend;
        const int64_t ps = ok ? (p.p_gather ? p.p_gather[r] : r) : 0;
        const int64_t qs = ok ? (p.q_gather ? p.q_gather[r] : r) : 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            Ps[lk][lc + q] = (ok && m0 + lc + q < p.M) ? p.P[ps * p.M + m0 + lc + q] : 0.f;
            Qs[lk][lc + q] = (ok && n0 + lc + q < p.N) ? p.Q[qs * p.N + n0 + lc + q] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TKS; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = Ps[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Qs[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    OutT* C = reinterpret_cast<OutT*>(p.C) + (int64_t)e * p.M * p.N;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < p.M && n < p.N) C[(int64_t)m * p.N + n] = (OutT)acc[i][j];
        }
}

int64_t m_tiles32(int64_t TK, int E) {
    const int64_t a = (TK + TB - 1) / TB + E - 1;
    return a < TK ? a : TK;
}

}  // namespace

// entry points used by the dispatchers in mts_gemm.hip when act_dtype == MTS_F32
int mts_f32_rows(int epi, const float* A, int lda, const int32_t* a_gather, const float* B, int b_rows,
                 int N, int Kdim, const int32_t* expert_start, int E, int64_t TK, float* C, float* C2,
                 const float* pre_act, const float* route_w, const int32_t* s_scatter, float* ds_part,
                 int np, hipStream_t s) {
    Rows32 p = {A, lda, a_gather, B, b_rows, N, Kdim, expert_start, E, C, C2, pre_act, route_w, s_scatter, ds_part, np};
    dim3 grid((unsigned)m_tiles32(TK, E), (unsigned)((N + TB - 1) / TB));
    if (epi == E32_PLAIN) rows_gemm_f32_kernel<E32_PLAIN><<<grid, kThreads, 0, s>>>(p);
    else if (epi == E32_SWIGLU) rows_gemm_f32_kernel<E32_SWIGLU><<<grid, kThreads, 0, s>>>(p);
    else rows_gemm_f32_kernel<E32_DY1><<<grid, kThreads, 0, s>>>(p);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

int mts_f32_dw(const float* P, const int32_t* p_gather, const float* Q, const int32_t* q_gather, int M,
               int N, const int32_t* expert_start, int E, int grad_dtype, void* C, hipStream_t s) {
    Dw32 p = {P, p_gather, Q, q_gather, M, N, expert_start, C};
    dim3 grid((unsigned)((M + TB - 1) / TB), (unsigned)((N + TB - 1) / TB), (unsigned)E);
    if (grid.y > 65535 || grid.z > 65535) return MTS_ERR_SHAPE;
    if (grad_dtype == MTS_F32) dw_gemm_f32_kernel<float><<<grid, kThreads, 0, s>>>(p);
    else if (grad_dtype == MTS_BF16) dw_gemm_f32_kernel<bf16_t><<<grid, kThreads, 0, s>>>(p);
    else if (grad_dtype == MTS_F16) dw_gemm_f32_kernel<mts_f16_t><<<grid, kThreads, 0, s>>>(p);
    else return MTS_ERR_DTYPE;
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}
