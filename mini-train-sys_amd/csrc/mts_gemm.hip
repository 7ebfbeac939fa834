// Grouped expert GEMMs on CDNA4 bf16 MFMA (v_mfma_f32_32x32x16_bf16), fp32
// accumulation.  Two kernel families share one LDS-tiled main loop:
//
//   rows_gemm  C[r, n] = sum_k A[row(r), k] * B[e][n, k]        (r tiled per expert)
//       used for gate/up + SwiGLU, down, dO*W2 (+ SwiGLU backward) and dX;
//       A rows are read through the token gather where the operand is x or dO,
//       so the permuted activations are never materialised.
//   dw_gemm    C[e][m, n] = sum_{r in e} P[row(r), m] * Q[row(r), n]
//       used for dW1 and dW2; the reduction runs over the expert's rows, so both
//       operands arrive "k-major" and are transposed 8x8 in registers on their
//       way into LDS.
//
// LDS tiles are [rows][BK + 8] bf16 (the 16-byte pad makes the 16-byte MFMA
// fragment reads of 16 consecutive rows hit distinct banks), double buffered:
// the global loads of tile k+1 are issued before the MFMAs of tile k.
//
// MFMA 32x32x16 register layout used below (lane l):
//   A/B fragment: row (l % 32) of the 32-row operand, k = 8*(l/32) .. 8*(l/32)+7
//   C fragment:   element i (0..15) is row 8*(i/4) + 4*(l/32) + (i%4), column l % 32
#include "mts_common.h"

#include <stdlib.h>

namespace {

constexpr int BK = 64;
constexpr int LDS_LD = BK + 8;

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int NT = NWAVES * MTS_WAVE;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MF = WM / 32, NF = WN / 32;
    static constexpr int LDS_ELEMS = 2 * (BM + BN) * LDS_LD;
    static_assert(WM % 32 == 0 && WN % 64 == 0, "wave tile must hold whole 32x32 fragments");
    static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "loader split");
};

enum Epilogue { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_DY1 = 2 };

struct RowsParams {
    const bf16_t* A;           // activations, row-major, leading dimension lda
    int64_t lda;
    const int32_t* a_gather;   // row -> source row of A, or NULL for identity
    const bf16_t* B;           // [E][n_rows_b][Kdim] bf16
    int64_t b_expert_stride;
    int N;                     // output columns (SwiGLU: I, B holds 2I rows)
    int Kdim;
    const int32_t* expert_start;
    int E;
    bf16_t* C;                 // plain: [TK,N]; SwiGLU: pre_act [TK,2N]; DY1: d_pre_act [TK,2N]
    bf16_t* C2;                // SwiGLU: post_act [TK,N]; DY1: weighted_act [TK,N]
    const bf16_t* pre_act;     // DY1: saved [g;u]
    const bf16_t* route_w;     // DY1: routing weights, flat [T*K]
    const int32_t* s_scatter;  // DY1: row -> entry
    float* ds_part;            // DY1: [TK][np]
    int np;
};

// ---------------------------------------------------------------------------
// global -> register -> LDS staging of a [ROWS][BK] tile whose rows are K-contiguous
// ---------------------------------------------------------------------------
template <int ROWS, int NT>
struct KMajorLoader {
    static constexpr int LOADS = ROWS * (BK / 8) / NT;
    const bf16_t* ptr[LOADS];  // row base + this thread's 8-element column, NULL = zero row
    u32x4 reg[LOADS];
    int col;                   // element offset of this thread's vector inside the k-tile

    __device__ __forceinline__ void fetch(int k0, int Kdim) {
#pragma unroll
        for (int p = 0; p < LOADS; ++p) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (ptr[p] != nullptr && k0 + col < Kdim)
                v = *reinterpret_cast<const u32x4*>(ptr[p] + k0);
            reg[p] = v;
        }
    }
    __device__ __forceinline__ void commit(bf16_t* lds) const {
        const int r = threadIdx.x / 8;
#pragma unroll
        for (int p = 0; p < LOADS; ++p)
            *reinterpret_cast<u32x4*>(lds + (p * (NT / 8) + r) * LDS_LD + col) = reg[p];
    }
};

// one MFMA sweep over a staged k-tile
template <class T, bool SWIGLU>
__device__ __forceinline__ void mma_tile(const bf16_t* As, const bf16_t* Bs, int wm, int wn,
                                         f32x16 (&acc)[T::MF][T::NF]) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int frow = lane % 32, fk = (lane / 32) * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 a[T::MF], b[T::NF];
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
            a[mf] = *reinterpret_cast<const bf16x8*>(As + (wm * T::WM + mf * 32 + frow) * LDS_LD +
                                                    ks * 16 + fk);
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf) {
            int brow;
            if (SWIGLU) {
                constexpr int HALF = T::NF / 2;
                brow = (nf / HALF) * (T::BN / 2) + wn * (T::WN / 2) + (nf % HALF) * 32;
            } else {
                brow = wn * T::WN + nf * 32;
            }
            b[nf] = *reinterpret_cast<const bf16x8*>(Bs + (brow + frow) * LDS_LD + ks * 16 + fk);
        }
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
                acc[mf][nf] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mf], b[nf], acc[mf][nf], 0, 0, 0);
    }
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }

// ---------------------------------------------------------------------------
// rows_gemm
// ---------------------------------------------------------------------------
template <class T, int EPI>
__global__ __launch_bounds__(T::NT) void rows_gemm_kernel(RowsParams p) {
    __shared__ __attribute__((aligned(16))) bf16_t smem[T::LDS_ELEMS];
    constexpr bool SWIGLU = (EPI == EPI_SWIGLU);

    // which expert does this m-tile belong to
    int e = 0, row0 = 0, rend = 0;
    {
        int tile = blockIdx.x, seen = 0;
        bool found = false;
        for (e = 0; e < p.E; ++e) {
            int s0 = p.expert_start[e], s1 = p.expert_start[e + 1];
            int nt = (s1 - s0 + T::BM - 1) / T::BM;
            if (tile < seen + nt) {
                row0 = s0 + (tile - seen) * T::BM;
                rend = s1;
                found = true;
                break;
            }
            seen += nt;
        }
        if (!found) return;
    }
    const int ntile = blockIdx.y;
    const int n0 = ntile * (SWIGLU ? T::BN / 2 : T::BN);  // first output column of this block

    KMajorLoader<T::BM, T::NT> la;
    KMajorLoader<T::BN, T::NT> lb;
    la.col = lb.col = (threadIdx.x % 8) * 8;
    {
        const int r = threadIdx.x / 8;
#pragma unroll
        for (int q = 0; q < la.LOADS; ++q) {
            int row = row0 + q * (T::NT / 8) + r;
            const bf16_t* ptr = nullptr;
            if (row < rend) {
                int64_t src = p.a_gather ? (int64_t)p.a_gather[row] : (int64_t)row;
                ptr = p.A + src * p.lda + la.col;
            }
            la.ptr[q] = ptr;
        }
        const bf16_t* Be = p.B + (int64_t)e * p.b_expert_stride;
#pragma unroll
        for (int q = 0; q < lb.LOADS; ++q) {
            int br = q * (T::NT / 8) + r;  // row inside the B tile
            int n, grow;
            if (SWIGLU) {
                int half = br / (T::BN / 2);
                n = n0 + br % (T::BN / 2);
                grow = half * p.N + n;
            } else {
                n = n0 + br;
                grow = n;
            }
            lb.ptr[q] = (n < p.N) ? Be + (int64_t)grow * p.Kdim + lb.col : nullptr;
        }
    }

    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mf][nf][i] = 0.f;

    constexpr int STAGE = (T::BM + T::BN) * LDS_LD;  // one buffer: A tile then B tile
    constexpr int B_OFF = T::BM * LDS_LD;
    const int nk = (p.Kdim + BK - 1) / BK;
    la.fetch(0, p.Kdim);
    lb.fetch(0, p.Kdim);
    la.commit(smem);
    lb.commit(smem + B_OFF);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        bf16_t* cur = smem + (kt & 1) * STAGE;
        bf16_t* nxt = smem + ((kt & 1) ^ 1) * STAGE;
        if (kt + 1 < nk) {
            la.fetch((kt + 1) * BK, p.Kdim);
            lb.fetch((kt + 1) * BK, p.Kdim);
        }
        mma_tile<T, SWIGLU>(cur, cur + B_OFF, wm, wn, acc);
        if (kt + 1 < nk) {
            la.commit(nxt);
            lb.commit(nxt + B_OFF);
        }
        __syncthreads();
    }

    // ---- epilogue ----
    const int fcol = lane % 32, frow4 = (lane / 32) * 4;
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = row0 + wm * T::WM + mf * 32 + 8 * (i / 4) + frow4 + (i % 4);
            const bool rok = row < rend;
            if (EPI == EPI_PLAIN) {
#pragma unroll
                for (int nf = 0; nf < T::NF; ++nf) {
                    int n = n0 + wn * T::WN + nf * 32 + fcol;
                    if (rok && n < p.N) p.C[(int64_t)row * p.N + n] = (bf16_t)acc[mf][nf][i];
                }
            } else if (EPI == EPI_SWIGLU) {
                constexpr int HALF = T::NF / 2;
#pragma unroll
                for (int f = 0; f < HALF; ++f) {
                    int n = n0 + wn * (T::WN / 2) + f * 32 + fcol;
                    float g = acc[mf][f][i], u = acc[mf][f + HALF][i];
                    if (rok && n < p.N) {
                        p.C[(int64_t)row * (2 * p.N) + n] = (bf16_t)g;
                        p.C[(int64_t)row * (2 * p.N) + p.N + n] = (bf16_t)u;
                        p.C2[(int64_t)row * p.N + n] = (bf16_t)(g * sigmoidf_(g) * u);
                    }
                }
            } else {  // EPI_DY1
                float s = 0.f;
                if (rok) s = (float)p.route_w[p.s_scatter[row]];
                float dsp = 0.f;
#pragma unroll
                for (int nf = 0; nf < T::NF; ++nf) {
                    int n = n0 + wn * T::WN + nf * 32 + fcol;
                    if (rok && n < p.N) {
                        const int64_t o = (int64_t)row * (2 * p.N) + n;
                        float g = (float)p.pre_act[o], u = (float)p.pre_act[o + p.N];
                        float a = acc[mf][nf][i];
                        float sig = sigmoidf_(g);
                        float silu = g * sig;
                        float y1 = silu * u;
                        dsp += a * y1;
                        p.C2[(int64_t)row * p.N + n] = (bf16_t)(s * y1);
                        float da = a * s;
                        p.C[o] = (bf16_t)(da * (silu * (1.0f - sig) + sig) * u);
                        p.C[o + p.N] = (bf16_t)(da * silu);
                    }
                }
#pragma unroll
                for (int o = 16; o > 0; o >>= 1) dsp += __shfl_xor(dsp, o, MTS_WAVE);
                if (rok && fcol == 0) p.ds_part[(int64_t)row * p.np + ntile * T::WAVES_N + wn] = dsp;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// dw_gemm
// ---------------------------------------------------------------------------
struct DwParams {
    const bf16_t* P;  // rows -> M side, row-major [*, M]
    int64_t ldp;
    const int32_t* p_gather;
    const bf16_t* Q;  // rows -> N side, row-major [*, N]
    int64_t ldq;
    const int32_t* q_gather;
    int M, N;
    const int32_t* expert_start;
    void* C;  // [E][M][N], bf16 or f32
};

// Stages a [64 k][64 m] block per wave-item: lane = (kgrp = lane%8, mc = lane/8) loads
// rows k = 8*kgrp+i, columns 8*mc..8*mc+7, transposes the 8x8 block in registers
// and writes 8 rows of LDS (m-major, 16 bytes of k each).
template <class T>
struct MMajorLoader {
    static constexpr int ITEMS_A = T::BM / 64, ITEMS_B = T::BN / 64;
    static constexpr int ITEMS = ITEMS_A + ITEMS_B;
    static constexpr int PER_WAVE = (ITEMS + T::NWAVES - 1) / T::NWAVES;
    u32x4 reg[PER_WAVE][8];

    __device__ __forceinline__ void fetch(const DwParams& p, int m0, int n0, int r0, int rend) {
        const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
        const int kgrp = lane % 8, mc = lane / 8;
#pragma unroll
        for (int q = 0; q < PER_WAVE; ++q) {
            const int item = q * T::NWAVES + wave;
            if (item >= ITEMS) break;
            const bool isA = item < ITEMS_A;
            const bf16_t* base = isA ? p.P : p.Q;
            const int64_t ld = isA ? p.ldp : p.ldq;
            const int32_t* gather = isA ? p.p_gather : p.q_gather;
            const int dim = isA ? p.M : p.N;
            const int c = (isA ? m0 + item * 64 : n0 + (item - ITEMS_A) * 64) + mc * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int r = r0 + kgrp * 8 + i;
                u32x4 v = {0u, 0u, 0u, 0u};
                if (r < rend && c < dim) {
                    int64_t src = gather ? (int64_t)gather[r] : (int64_t)r;
                    v = *reinterpret_cast<const u32x4*>(base + src * ld + c);
                }
                reg[q][i] = v;
            }
        }
    }

    __device__ __forceinline__ void commit(bf16_t* As, bf16_t* Bs) const {
        const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
        const int kgrp = lane % 8, mc = lane / 8;
#pragma unroll
        for (int q = 0; q < PER_WAVE; ++q) {
            const int item = q * T::NWAVES + wave;
            if (item >= ITEMS) break;
            const bool isA = item < ITEMS_A;
            bf16_t* dst = (isA ? As + (item * 64) * LDS_LD : Bs + ((item - ITEMS_A) * 64) * LDS_LD) +
                          (mc * 8) * LDS_LD + kgrp * 8;
#pragma unroll
            for (int md = 0; md < 4; ++md) {
                u32x4 lo, hi;  // columns 2*md and 2*md+1 of the 8x8 block, k = 0..7
#pragma unroll
                for (int kp = 0; kp < 4; ++kp) {
                    uint32_t a = reg[q][2 * kp][md], b = reg[q][2 * kp + 1][md];
                    lo[kp] = (a & 0xffffu) | (b << 16);
                    hi[kp] = (a >> 16) | (b & 0xffff0000u);
                }
                *reinterpret_cast<u32x4*>(dst + (2 * md) * LDS_LD) = lo;
                *reinterpret_cast<u32x4*>(dst + (2 * md + 1) * LDS_LD) = hi;
            }
        }
    }
};

template <class T, typename OutT>
__global__ __launch_bounds__(T::NT) void dw_gemm_kernel(DwParams p) {
    __shared__ __attribute__((aligned(16))) bf16_t smem[T::LDS_ELEMS];
    const int e = blockIdx.z;
    const int m0 = blockIdx.x * T::BM, n0 = blockIdx.y * T::BN;
    const int rbeg = p.expert_start[e], rend = p.expert_start[e + 1];

    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mf][nf][i] = 0.f;

    constexpr int STAGE = (T::BM + T::BN) * LDS_LD;
    constexpr int B_OFF = T::BM * LDS_LD;
    const int nk = (rend - rbeg + BK - 1) / BK;
    MMajorLoader<T> ld;
    if (nk > 0) {
        ld.fetch(p, m0, n0, rbeg, rend);
        ld.commit(smem, smem + B_OFF);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        bf16_t* cur = smem + (kt & 1) * STAGE;
        bf16_t* nxt = smem + ((kt & 1) ^ 1) * STAGE;
        if (kt + 1 < nk) ld.fetch(p, m0, n0, rbeg + (kt + 1) * BK, rend);
        mma_tile<T, false>(cur, cur + B_OFF, wm, wn, acc);
        if (kt + 1 < nk) ld.commit(nxt, nxt + B_OFF);
        __syncthreads();
    }

    OutT* C = reinterpret_cast<OutT*>(p.C) + (int64_t)e * p.M * p.N;
    const int fcol = lane % 32, frow4 = (lane / 32) * 4;
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = m0 + wm * T::WM + mf * 32 + 8 * (i / 4) + frow4 + (i % 4);
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf) {
                const int n = n0 + wn * T::WN + nf * 32 + fcol;
                if (m < p.M && n < p.N) C[(int64_t)m * p.N + n] = (OutT)acc[mf][nf][i];
            }
        }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
typedef Tile<128, 128, 2, 2> TileS;
typedef Tile<256, 256, 2, 2> TileL;

int tile_choice() {
    static int choice = -1;
    if (choice < 0) {
        const char* s = getenv("MTS_GEMM_TILE");
        choice = (s && atoi(s) == 256) ? 1 : 0;
    }
    return choice;
}

int check_common(int64_t TK, int E, int H, int I) {
    if (TK <= 0 || TK > 0x7fffffffLL || E < 1 || E > MTS_MAX_EXPERTS || H < 8 || I < 8 || H % 8 ||
        I % 8)
        return MTS_ERR_SHAPE;
    return MTS_OK;
}

template <class T>
int64_t m_tiles(int64_t TK, int E) {
    int64_t a = (TK + T::BM - 1) / T::BM + E - 1;
    return a < TK ? a : TK;
}

template <class T, int EPI>
int launch_rows(const RowsParams& p, int64_t TK, hipStream_t s) {
    const int per_block = (EPI == EPI_SWIGLU) ? T::BN / 2 : T::BN;
    dim3 grid((unsigned)m_tiles<T>(TK, p.E), (unsigned)((p.N + per_block - 1) / per_block));
    rows_gemm_kernel<T, EPI><<<grid, T::NT, 0, s>>>(p);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

template <int EPI>
int launch_rows_any(const RowsParams& p, int64_t TK, hipStream_t s) {
    return tile_choice() ? launch_rows<TileL, EPI>(p, TK, s) : launch_rows<TileS, EPI>(p, TK, s);
}

template <class T>
int launch_dw(const DwParams& p, int E, int grad_dtype, hipStream_t s) {
    dim3 grid((unsigned)((p.M + T::BM - 1) / T::BM), (unsigned)((p.N + T::BN - 1) / T::BN), (unsigned)E);
    if (grad_dtype == MTS_BF16) dw_gemm_kernel<T, bf16_t><<<grid, T::NT, 0, s>>>(p);
    else if (grad_dtype == MTS_F32) dw_gemm_kernel<T, float><<<grid, T::NT, 0, s>>>(p);
    else return MTS_ERR_DTYPE;
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

int launch_dw_any(const DwParams& p, int E, int grad_dtype, hipStream_t s) {
    return tile_choice() ? launch_dw<TileL>(p, E, grad_dtype, s) : launch_dw<TileS>(p, E, grad_dtype, s);
}

}  // namespace

extern "C" int mts_moe_ds_partials(int I) {
    if (tile_choice()) return ((I + TileL::BN - 1) / TileL::BN) * TileL::WAVES_N;
    return ((I + TileS::BN - 1) / TileS::BN) * TileS::WAVES_N;
}

extern "C" int mts_moe_fwd_gateup_swiglu(const void* x, const void* w1, const int32_t* x_gather,
                                         const int32_t* expert_start, int64_t T, int K, int E,
                                         int H, int I, int act_dtype, void* pre_act,
                                         void* post_act, void* stream) {
    if (!x || !w1 || !x_gather || !expert_start || !pre_act || !post_act) return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    int rc = check_common(T * K, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(x) || !mts_aligned16(w1)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)x; p.lda = H; p.a_gather = x_gather;
    p.B = (const bf16_t*)w1; p.b_expert_stride = (int64_t)2 * I * H;
    p.N = I; p.Kdim = H; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)pre_act; p.C2 = (bf16_t*)post_act;
    return launch_rows_any<EPI_SWIGLU>(p, T * K, (hipStream_t)stream);
}

extern "C" int mts_moe_fwd_down(const void* post_act, const void* w2, const int32_t* expert_start,
                                int64_t TK, int E, int H, int I, int act_dtype, void* y,
                                void* stream) {
    if (!post_act || !w2 || !expert_start || !y) return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    int rc = check_common(TK, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(post_act) || !mts_aligned16(w2)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)post_act; p.lda = I; p.a_gather = nullptr;
    p.B = (const bf16_t*)w2; p.b_expert_stride = (int64_t)H * I;
    p.N = H; p.Kdim = I; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)y;
    return launch_rows_any<EPI_PLAIN>(p, TK, (hipStream_t)stream);
}

extern "C" int mts_moe_bwd_dy1(const void* d_out, const void* w2t, const void* pre_act,
                               const void* weights, const int32_t* x_gather,
                               const int32_t* s_scatter, const int32_t* expert_start, int64_t T,
                               int K, int E, int H, int I, int act_dtype, void* d_pre_act,
                               void* weighted_act, float* ds_partial, void* stream) {
    if (!d_out || !w2t || !pre_act || !weights || !x_gather || !s_scatter || !expert_start ||
        !d_pre_act || !weighted_act || !ds_partial)
        return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    int rc = check_common(T * K, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(d_out) || !mts_aligned16(w2t)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)d_out; p.lda = H; p.a_gather = x_gather;
    p.B = (const bf16_t*)w2t; p.b_expert_stride = (int64_t)H * I;
    p.N = I; p.Kdim = H; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)d_pre_act; p.C2 = (bf16_t*)weighted_act;
    p.pre_act = (const bf16_t*)pre_act; p.route_w = (const bf16_t*)weights;
    p.s_scatter = s_scatter; p.ds_part = ds_partial; p.np = mts_moe_ds_partials(I);
    return launch_rows_any<EPI_DY1>(p, T * K, (hipStream_t)stream);
}

extern "C" int mts_moe_bwd_dx(const void* d_pre_act, const void* w1t, const int32_t* expert_start,
                              int64_t TK, int E, int H, int I, int act_dtype, void* dx_expanded,
                              void* stream) {
    if (!d_pre_act || !w1t || !expert_start || !dx_expanded) return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    int rc = check_common(TK, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(d_pre_act) || !mts_aligned16(w1t)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)d_pre_act; p.lda = (int64_t)2 * I; p.a_gather = nullptr;
    p.B = (const bf16_t*)w1t; p.b_expert_stride = (int64_t)2 * I * H;
    p.N = H; p.Kdim = 2 * I; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)dx_expanded;
    return launch_rows_any<EPI_PLAIN>(p, TK, (hipStream_t)stream);
}

extern "C" int mts_moe_bwd_dw2(const void* d_out, const void* weighted_act, const int32_t* x_gather,
                               const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                               int act_dtype, int grad_dtype, void* d_w2, void* stream) {
    if (!d_out || !weighted_act || !x_gather || !expert_start || !d_w2) return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    int rc = check_common(T * K, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(d_out) || !mts_aligned16(weighted_act)) return MTS_ERR_ALIGN;
    DwParams p = {};
    p.P = (const bf16_t*)d_out; p.ldp = H; p.p_gather = x_gather;
    p.Q = (const bf16_t*)weighted_act; p.ldq = I; p.q_gather = nullptr;
    p.M = H; p.N = I; p.expert_start = expert_start; p.C = d_w2;
    return launch_dw_any(p, E, grad_dtype, (hipStream_t)stream);
}

extern "C" int mts_moe_bwd_dw1(const void* d_pre_act, const void* x, const int32_t* x_gather,
                               const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                               int act_dtype, int grad_dtype, void* d_w1, void* stream) {
    if (!d_pre_act || !x || !x_gather || !expert_start || !d_w1) return MTS_ERR_NULL;
    if (act_dtype != MTS_BF16) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    int rc = check_common(T * K, E, H, I);
    if (rc) return rc;
    if (!mts_aligned16(d_pre_act) || !mts_aligned16(x)) return MTS_ERR_ALIGN;
    DwParams p = {};
    p.P = (const bf16_t*)d_pre_act; p.ldp = (int64_t)2 * I; p.p_gather = nullptr;
    p.Q = (const bf16_t*)x; p.ldq = H; p.q_gather = x_gather;
    p.M = 2 * I; p.N = H; p.expert_start = expert_start; p.C = d_w1;
    return launch_dw_any(p, E, grad_dtype, (hipStream_t)stream);
}
