// Grouped expert GEMMs on CDNA4 bf16 MFMA (v_mfma_f32_32x32x16_bf16), fp32
// accumulation.  Two kernel families share one LDS-tiled main loop:
//
//   rows_gemm  C[r, n] = sum_k A[row(r), k] * B[e][n, k]        (r tiled per expert)
//       used for gate/up + SwiGLU, down, dO*W2 (+ SwiGLU backward) and dX;
//       A rows are read through the token gather where the operand is x or dO,
//       so the permuted activations are never materialised.
//   dw_gemm    C[e][m, n] = sum_{r in e} P[row(r), m] * Q[row(r), n]
//       used for dW1 and dW2; the reduction runs over the expert's rows, so both
//       operands arrive "k-major"; the staged pipeline transposes them 8x8 in
//       registers on their way into LDS, the ring pipeline keeps them k-major in
//       LDS and reads fragments with the transposing LDS load.
//
// Global reads are raw buffer loads: a lane that must contribute zeros (row past
// the expert's end, column past N, k past K) is given an offset beyond the buffer
// and the hardware returns 0, so the main loops have no divergent branches.
//
// Pipelines.  "staged": global -> VGPR -> LDS, two stages, any K that is a multiple
// of 8.  "ring": global -> LDS directly (buffer_load ... lds), three or four stages,
// whole k-tiles only, every wave loads and multiplies.  "ws": the same ring with
// specialised waves (producers issue the loads, consumers the MFMAs).  LDS rows are
// XOR-swizzled instead of padded, so fragment reads and tile writes are both
// bank-conflict free.
//
// MFMA 32x32x16 register layout used below (lane l):
//   A/B fragment: row (l % 32) of the 32-row operand, k = 8*(l/32) .. 8*(l/32)+7
//   C fragment:   element i (0..15) is row 8*(i/4) + 4*(l/32) + (i%4), column l % 32
#include "mts_common.h"
#include "mts_router_bwd_block.h"
#include "mts_combine_block.h"
#include "mts_tuning.h"

#include <stdlib.h>

// This source is compiled twice: as it stands for bf16, and from mts_gemm_f16.hip with
// MTS_GEMM_F16 defined for fp16 (same tiles and pipelines, the fp16 MFMA, entry points with an
// _f16 suffix that the bf16 build's entry points forward to).  Below, bf16_t / bf16x8 / bf16x4 are
// the 16-bit element type of the build.
#ifdef MTS_GEMM_F16
#define bf16_t mts_f16_t
#define bf16x8 mts_f16x8
#define bf16x4 mts_f16x4
#define MTS_GEMM_ENTRY(name) name##_f16
#define MTS_GEMM_DTYPE MTS_F16
#define MTS_MFMA_32x32x16 __builtin_amdgcn_mfma_f32_32x32x16_f16
#else
#define MTS_GEMM_ENTRY(name) name
#define MTS_GEMM_DTYPE MTS_BF16
#define MTS_MFMA_32x32x16 __builtin_amdgcn_mfma_f32_32x32x16_bf16
#endif

namespace {

// fp32 value of a 16-bit element given as the low bits of a word
__device__ __forceinline__ float elem_bits_to_f32(uint32_t bits16) {
#ifdef MTS_GEMM_F16
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
#else
    return bf16_bits_to_f32(bits16);
#endif
}

constexpr int BK = 64;                       // k extent of an LDS tile (8 chunks of 8 bf16)
constexpr uint32_t kInvalid = 0x80000000u;   // buffer offset that is out of range for every operand
constexpr int64_t kMaxOperandBytes = 0x7fffffffLL;

// Raw buffer descriptor over `bytes` bytes at p.  Lane offsets are 32-bit and kInvalid (2^31) must stay
// out of range, so a descriptor spans at most 2^31 - 1 bytes: operands that can be larger are addressed
// through a descriptor that starts at the block's own tile (a 64-bit base, small offsets).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
    const int64_t span = bytes < 0 ? 0 : (bytes > kMaxOperandBytes ? kMaxOperandBytes : bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)span, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
}
__device__ __forceinline__ int buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
    return (int)__builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0);
}

// Scalar buffer load of 8 consecutive dwords (read-only, through the scalar cache).  The
// descriptor has the raw-buffer layout make_rsrc builds; offsets past `bytes` return 0.
// The wait is part of the same statement: the compiler does not track the completion of a
// load issued from inline assembly and may copy the result registers at any later point.
typedef __attribute__((ext_vector_type(4))) int i32x4;
__device__ __forceinline__ u32x4 scalar_rsrc(const void* p, int64_t bytes) {
    const uint64_t a = (uint64_t)p;
    u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
    return r;
}
__device__ __forceinline__ void s_buffer_load8(u32x4 rsrc, int byte_off, i32x4& lo, i32x4& hi) {
    asm volatile(
        "s_buffer_load_dwordx4 %0, %2, %3\n\t"
        "s_buffer_load_dwordx4 %1, %2, %4\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(lo), "=&s"(hi)
        : "s"(rsrc), "s"(byte_off), "s"(byte_off + 16));
}

// element offset of 16-byte chunk `chunk` of row `row` inside a swizzled tile
__device__ __forceinline__ int lds_off(int row, int chunk) {
    return row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
}

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int NT = NWAVES * MTS_WAVE;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MF = WM / 32, NF = WN / 32;
    static constexpr int STAGE = (BM + BN) * BK;   // elements per pipeline stage
    static constexpr int LDS_ELEMS = 2 * STAGE;
    static_assert(WM % 32 == 0 && WN % 64 == 0, "wave tile must hold whole 32x32 fragments");
    static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "loader split");
};

// EPI_DY1N: the dO*W2 epilogue without the weighted_act output (the caller kept the forward
// pass's post_act, which already carries the routing weight)
enum Epilogue { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_DY1 = 2, EPI_DY1N = 3 };
constexpr bool epi_is_dy1(int epi) { return epi == EPI_DY1 || epi == EPI_DY1N; }

struct RowsParams {
    const bf16_t* A;           // activations, row-major, leading dimension lda
    int64_t a_rows;            // rows of A (for the buffer range)
    int lda;
    const int32_t* a_gather;   // row -> source row of A, or NULL for identity
    const bf16_t* B;           // [E][b_rows][Kdim] bf16
    int b_rows;
    int N;                     // output columns (SwiGLU: I, B holds 2I rows)
    int Kdim;
    const int32_t* expert_start;
    int E;
    bf16_t* C;                 // plain: [TK,N]; SwiGLU: pre_act [TK,2N]; DY1: d_pre_act [TK,2N]
    bf16_t* C2;                // SwiGLU: post_act [TK,N]; DY1: weighted_act [TK,N]
    const bf16_t* pre_act;     // DY1: saved [g;u]
    const bf16_t* route_w;     // DY1: routing weights, flat [T*K]; SwiGLU: the same, or NULL (post_act unscaled)
    const int32_t* s_scatter;  // DY1, SwiGLU with route_w: row -> entry
    float* ds_part;            // DY1: [TK][np]
    int np;
    int64_t TK;                // rows of every output
    int n_tiles;               // column tiles per m-tile (set by the launcher)
    int xcd_ranges;            // block -> tile mapping: 1 = every XCD takes a contiguous range of m-tiles
    int n_groups;              // with xcd_ranges: the n-tiles are walked in this many groups, all m-tiles of the range per group
    int reverse;               // with xcd_ranges: the range's m-tiles are walked from the last to the first
    int tail_slots;            // with xcd_ranges: blocks an XCD runs at a time; when the tiles behind its last whole round
                               // fill at most half of them, each of those is cut into two tiles of half the height (0: never)
    int tail_tiles;            // with xcd_ranges: this many tiles at the end of every XCD's list are cut in two whatever the rounds
                               // come to (a launch whose blocks start behind another part's: its rounds are not aligned)
    const int32_t* sched;      // with xcd_ranges: the m-tile range of every XCD (first[8], count[8]) from the schedule of the joint
                               // backward launch, or NULL: equal ranges
    int32_t* sched_out;        // dO*W2 launch: one more block writes the schedule of the joint backward launch here (NULL: none)
    int sched_slots, sched_dx_cap;
};

// the schedule of the joint backward launch (defined with the weight-gradient GEMMs below)
__device__ __forceinline__ void joint_schedule_wave(const int32_t* __restrict__ expert_start, int E, int slots, int dx_bm,
                                                    int dx_cap, int32_t* __restrict__ sched);
constexpr int kSchedDxRows = 256;   // rows of a dX tile of that launch (JointDxTile::BM)

// The last block of a dO*W2 launch that was given a table writes the schedule: it needs nothing but expert_start,
// and inside this launch it costs no time of its own.
__device__ __forceinline__ bool schedule_block(const RowsParams& p) {
    if (p.sched_out == nullptr || blockIdx.x != gridDim.x - 1) return false;
    if (threadIdx.x < MTS_WAVE) joint_schedule_wave(p.expert_start, p.E, p.sched_slots, kSchedDxRows, p.sched_dx_cap, p.sched_out);
    return true;
}

// ---------------------------------------------------------------------------
// global -> register -> LDS staging of a [ROWS][BK] tile whose rows are K-contiguous
// ---------------------------------------------------------------------------
template <int ROWS, int NT>
struct KMajorLoader {
    static constexpr int LOADS = ROWS * (BK / 8) / NT;
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t voff[LOADS];  // byte offset of this thread's chunk at k = 0, or kInvalid
    u32x4 reg[LOADS];
    int chunk;             // this thread's 16-byte chunk inside the k-tile

    __device__ __forceinline__ void fetch(int k0, int Kdim) {
        const bool kok = k0 + chunk * 8 < Kdim;
#pragma unroll
        for (int p = 0; p < LOADS; ++p)
            reg[p] = buf_load16(rsrc, kok ? voff[p] + (uint32_t)k0 * 2u : kInvalid);
    }
    __device__ __forceinline__ void commit(bf16_t* lds) const {
        const int r = threadIdx.x / 8;
#pragma unroll
        for (int p = 0; p < LOADS; ++p)
            *reinterpret_cast<u32x4*>(lds + lds_off(p * (NT / 8) + r, chunk)) = reg[p];
    }
};

// one MFMA sweep over a staged k-tile
// (ROWLEN = k extent of the LDS rows: 64 with swizzle (row>>1)&7, 32 with (row>>2)&3)
// 32 x 16 MFMA fragments out of LDS tiles that hold one k per row ("k-major": the operand's
// memory rows are k) are read with the transposing LDS load; the layout is described at the
// weight-gradient GEMMs below.
typedef __attribute__((ext_vector_type(4))) short s16x4;

// 32 (m) x 16 (k) MFMA fragment out of a k-major LDS tile with row length ROWLEN
template <int ROWLEN>
__device__ __forceinline__ bf16x8 read_frag_tr(const bf16_t* tile, int krow0, int col0) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int col = col0 + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
    const int chunk = col / 8, within = col % 8;
    s16x4 h[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int row = krow0 + 8 * (lane / 32) + 4 * q + (lane % 16) / 4;
        const bf16_t* src = tile + row * ROWLEN + ((chunk ^ ((row & 3) << 2)) << 3) + within;
        h[q] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(src));
    }
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    s16x8 v = {h[0][0], h[0][1], h[0][2], h[0][3], h[1][0], h[1][1], h[1][2], h[1][3]};
    return __builtin_bit_cast(bf16x8, v);
}

struct NoHook {
    __device__ __forceinline__ void operator()(int) const {}
};

// `hook(ks)` runs once per 16-wide k-step, between the fragment reads and the MFMAs.
// Fragments are double buffered: the LDS reads of k-step ks+1 are issued before the
// MFMAs of k-step ks, so that their latency is covered by the matrix pipe.
// BKM: the B tile is k-major, [ROWLEN k][T::BN] (weights in their stored layout).
template <class T, bool SWIGLU, int ROWLEN = BK, bool WEIGHT_FIRST = true, bool BKM = false, class Hook = NoHook>
__device__ __forceinline__ void mma_tile(const bf16_t* As, const bf16_t* Bs, int wm, int wn,
                                         f32x16 (&acc)[T::MF][T::NF], Hook hook = Hook()) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int frow = lane % 32, kb = lane / 32;
    const int swz = ROWLEN == 64 ? (frow >> 1) & 7 : (frow >> 2) & 3;
    const bf16_t* a_base = As + (wm * T::WM + frow) * ROWLEN;
    const bf16_t* b_base = Bs + frow * ROWLEN;
    constexpr int KSTEPS = ROWLEN / 16;
    bf16x8 a[2][T::MF], b[2][T::NF];

    auto load_frags = [&](int ks, int buf) {
        const int coff = ((ks * 2 + kb) ^ swz) << 3;
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
            a[buf][mf] = *reinterpret_cast<const bf16x8*>(a_base + mf * 32 * ROWLEN + coff);
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf) {
            int brow;
            if (SWIGLU) {
                constexpr int HALF = T::NF / 2;
                brow = (nf / HALF) * (T::BN / 2) + wn * (T::WN / 2) + (nf % HALF) * 32;
            } else {
                brow = wn * T::WN + nf * 32;
            }
            if constexpr (BKM) b[buf][nf] = read_frag_tr<T::BN>(Bs, ks * 16, brow);
            else b[buf][nf] = *reinterpret_cast<const bf16x8*>(b_base + brow * ROWLEN + coff);
        }
    };

    load_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const int cur = ks & 1;
        if (ks + 1 < KSTEPS) load_frags(ks + 1, cur ^ 1);
        hook(ks);
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
                acc[mf][nf] = WEIGHT_FIRST
                                  ? MTS_MFMA_32x32x16(b[cur][nf], a[cur][mf], acc[mf][nf], 0, 0, 0)
                                  : MTS_MFMA_32x32x16(a[cur][mf], b[cur][nf], acc[mf][nf], 0, 0, 0);
    }
}

// Fragment pipeline of a consumer wave that runs across k-tiles: the LDS reads of the next
// 16-wide k-step (of this tile or of the next one) are in flight while the MFMAs of the
// current step are issued, so the matrix pipe does not idle at the start of a k-tile.
// Weight fragments are double buffered; an activation fragment is reloaded for the next
// k-step right behind the MFMAs that used it.
template <class T, bool SWIGLU, int ROWLEN, bool BKM = false>
struct FragPipe {
    static constexpr int KSTEPS = ROWLEN / 16;
    static_assert(KSTEPS % 2 == 0, "weight fragment buffers alternate with the k-step");
    bf16x8 a[T::MF], b[2][T::NF];
    int a_off, b_off[T::NF], swz, kb;

    __device__ __forceinline__ void init(int wm, int wn) {
        const int lane = threadIdx.x % MTS_WAVE;
        const int frow = lane % 32;
        kb = lane / 32;
        swz = ROWLEN == 64 ? (frow >> 1) & 7 : (frow >> 2) & 3;
        a_off = (wm * T::WM + frow) * ROWLEN;
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf) {
            int brow;
            if (SWIGLU) {
                constexpr int HALF = T::NF / 2;
                brow = (nf / HALF) * (T::BN / 2) + wn * (T::WN / 2) + (nf % HALF) * 32;
            } else {
                brow = wn * T::WN + nf * 32;
            }
            // k-major B: b_off is the fragment's first column; the tile starts behind the A tile
            b_off[nf] = BKM ? brow : T::BM * ROWLEN + (brow + frow) * ROWLEN;
        }
    }
    __device__ __forceinline__ bf16x8 read_b(const bf16_t* tile, int nf, int ks, int coff) const {
        if constexpr (BKM) return read_frag_tr<T::BN>(tile + T::BM * ROWLEN, ks * 16, b_off[nf]);
        else return *reinterpret_cast<const bf16x8*>(tile + b_off[nf] + coff);
    }
    __device__ __forceinline__ int chunk_off(int ks) const { return ((ks * 2 + kb) ^ swz) << 3; }
    // all fragments of k-step 0 of the stage at `tile`
    __device__ __forceinline__ void prime(const bf16_t* tile) { prime(tile, tile); }
    // the same with the two operands in buffers of their own: tile_b is where a stage would start whose weight tile
    // is the buffer (the buffer's address minus the size of an activation tile)
    __device__ __forceinline__ void prime(const bf16_t* tile, const bf16_t* tile_b) {
        const int coff = chunk_off(0);
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
            a[mf] = *reinterpret_cast<const bf16x8*>(tile + a_off + mf * 32 * ROWLEN + coff);
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf) b[0][nf] = read_b(tile_b, nf, 0, coff);
    }
    // MFMAs of k-step `ks` (weight fragment first); behind them, the fragments of k-step `nks`
    // of the stage at `next` are read: the weight fragments up front into the other buffer, each
    // activation fragment as soon as its MFMAs are issued
    // READ = false: the MFMAs only (the last k-step of a buffer whose successor is not visible yet)
    template <bool READ = true>
    __device__ __forceinline__ void step(int ks, f32x16 (&acc)[T::MF][T::NF], const bf16_t* next, int nks) {
        step<READ>(ks, acc, next, next, nks);
    }
    template <bool READ = true>
    __device__ __forceinline__ void step(int ks, f32x16 (&acc)[T::MF][T::NF], const bf16_t* next, const bf16_t* next_b, int nks) {
        const int coff = chunk_off(nks), buf = ks & 1;
        if constexpr (READ) {
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf) b[buf ^ 1][nf] = read_b(next_b, nf, nks, coff);
        }
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf) {
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
                acc[mf][nf] = MTS_MFMA_32x32x16(b[buf][nf], a[mf], acc[mf][nf], 0, 0, 0);
            if constexpr (READ) a[mf] = *reinterpret_cast<const bf16x8*>(next + a_off + mf * 32 * ROWLEN + coff);
        }
    }
};

// v_rcp_f32 (1 ulp) instead of the IEEE division sequence, which costs nine more instructions per
// value; the results are rounded to 16 bits
__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

template <class T>
__device__ __forceinline__ void zero_acc(f32x16 (&acc)[T::MF][T::NF]) {
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mf][nf][i] = 0.f;
}

// ---------------------------------------------------------------------------
// epilogues of rows_gemm (accumulators -> global memory)
//
// The MFMAs of rows_gemm take the weight fragment as the first operand, so a lane
// holds, for ONE activation row (lane % 32), four runs of four consecutive output
// columns: element i of fragment nf is column 32*nf + 8*(i/4) + 4*(lane/32) + i%4.
// Per-row quantities (routing weight, dS) therefore live in one lane pair, and
// the bf16 results are staged through a per-wave LDS tile [32][COLS+8] with 8-byte
// writes and flushed with 16-byte, row-contiguous buffer stores; rows past the
// expert's end and columns past N get an out-of-range offset and are dropped by
// the hardware, so there are no divergent branches.
// ---------------------------------------------------------------------------
template <class T, int EPI>
struct EpiShape {
    static constexpr int COLS = (EPI == EPI_SWIGLU) ? T::WN / 2 : T::WN;  // contiguous columns per staged tile
    static constexpr int NBUF = (EPI == EPI_PLAIN) ? 1 : (EPI == EPI_DY1N ? 2 : 3);
    static constexpr int LDW = COLS + 8;
    static constexpr int ELEMS = T::NWAVES * NBUF * 32 * LDW;
};

__device__ __forceinline__ void stage4(bf16_t* dst, float a, float b, float c, float d) {
    bf16x4 v = {(bf16_t)a, (bf16_t)b, (bf16_t)c, (bf16_t)d};
    *reinterpret_cast<bf16x4*>(dst) = v;
}

// staged [32][COLS] tile -> rows rowg0.. (counted from the start of the descriptor, rend of them exist),
// columns col.. of a matrix with leading dimension ldc
template <int COLS>
__device__ __forceinline__ void flush_tile(const bf16_t* buf, __amdgpu_buffer_rsrc_t rs, uint32_t ldc, uint32_t col,
                                           int rowg0, int rend, int ncol0, int N) {
    constexpr int LPR = COLS / 8, RPI = MTS_WAVE / LPR, LDW = COLS + 8;
    const int lane = threadIdx.x % MTS_WAVE;
    const int c = (lane % LPR) * 8;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
        const int r = it * RPI + lane / LPR;
        const u32x4 v = *reinterpret_cast<const u32x4*>(buf + r * LDW + c);
        const int row = rowg0 + r;
        const bool ok = row < rend && ncol0 + c < N;
        const uint32_t off = ok ? ((uint32_t)row * ldc + col + (uint32_t)c) * 2u : kInvalid;
        __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)off, 0, 0);
    }
}

// PREFETCH (dY1): the pre-activations of slab mf+1 are loaded into registers before the
// arithmetic of slab mf (32 more registers: for the kernels that have them to spare).
template <class T, int EPI, bool PREFETCH = false>
__device__ __forceinline__ void rows_epilogue(const RowsParams& p, f32x16 (&acc)[T::MF][T::NF], bf16_t* smem,
                                              int row0, int rend, int n0, int wm, int wn) {
    typedef EpiShape<T, EPI> ES;
    constexpr int COLS = ES::COLS, LDW = ES::LDW;
    constexpr bool DY1 = epi_is_dy1(EPI), WACT = (EPI == EPI_DY1);
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int ml = lane % 32, nq = (lane / 32) * 4;
    bf16_t* buf0 = smem + wave * ES::NBUF * 32 * LDW;
    bf16_t* buf1 = buf0 + 32 * LDW;
    bf16_t* buf2 = buf1 + 32 * LDW;
    // dY1: staging tiles of the gate and up halves, and of weighted_act where it is written
    bf16_t* bufg = WACT ? buf1 : buf0;
    bf16_t* bufu = WACT ? buf2 : buf1;
    const int ncol0 = n0 + wn * COLS;  // first output column of this wave
    const uint32_t N = (uint32_t)p.N;
    // The [TK, ...] outputs (and the saved pre-activations) may exceed what one descriptor spans: the
    // descriptors start at the tile's first row and end at the expert's last row, and rows are
    // counted from row0 below.
    const int64_t left = rend - row0;
    const int64_t ldc = EPI == EPI_PLAIN ? N : 2 * N;
    const bool has_c2 = EPI == EPI_SWIGLU || EPI == EPI_DY1;
    const __amdgpu_buffer_rsrc_t rs_c = make_rsrc(p.C + (int64_t)row0 * ldc, left * ldc * 2);
    const __amdgpu_buffer_rsrc_t rs_c2 = make_rsrc(has_c2 ? p.C2 + (int64_t)row0 * N : nullptr, has_c2 ? left * (int64_t)N * 2 : 0);
    const __amdgpu_buffer_rsrc_t rs_pre = make_rsrc(DY1 ? p.pre_act + (int64_t)row0 * 2 * N : nullptr, DY1 ? left * (int64_t)N * 4 : 0);
    const int rrel = rend - row0;   // rows of the tile that exist

    // routing weight of each of the lane's rows (dY1; SwiGLU when post_act carries the weight): two
    // dependent loads, issued for all rows up front
    float srow[T::MF];
    // dY1: gate and up pre-activations of one 32 x COLS slab of the wave's tile, row-contiguous
    // 16-byte loads held in registers; the loads of slab mf+1 are issued before the arithmetic of
    // slab mf so that their latency is covered
    constexpr int PRE_LPR = COLS / 8, PRE_RPI = MTS_WAVE / PRE_LPR, PRE_IT = 32 / PRE_RPI;
    u32x4 gv[DY1 ? PRE_IT : 1], uv[DY1 ? PRE_IT : 1];
    auto load_pre = [&](int mf) {
        const int c = (lane % PRE_LPR) * 8;
#pragma unroll
        for (int it = 0; it < PRE_IT; ++it) {
            const int grow = wm * T::WM + mf * 32 + it * PRE_RPI + lane / PRE_LPR;   // row inside the tile
            const bool ok = grow < rrel && ncol0 + c < p.N;
            const uint32_t po = ok ? ((uint32_t)grow * 2u * N + (uint32_t)(ncol0 + c)) * 2u : kInvalid;
            gv[it] = buf_load16(rs_pre, po);
            uv[it] = buf_load16(rs_pre, po == kInvalid ? kInvalid : po + N * 2u);
        }
    };
    if (DY1 || EPI == EPI_SWIGLU) {
        const bool weighted = DY1 || p.route_w != nullptr;
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf) {
            const int row = row0 + wm * T::WM + mf * 32 + ml;
            srow[mf] = !weighted ? 1.f : (row < rend ? (float)p.route_w[p.s_scatter[row]] : 0.f);
        }
        if (DY1 && PREFETCH) load_pre(0);
    }
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf) {
        const int rowg0 = wm * T::WM + mf * 32;   // first row of the slab, counted from row0
        if (EPI == EPI_PLAIN) {
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    stage4(buf0 + ml * LDW + nf * 32 + 8 * j + nq, acc[mf][nf][4 * j], acc[mf][nf][4 * j + 1],
                           acc[mf][nf][4 * j + 2], acc[mf][nf][4 * j + 3]);
            flush_tile<COLS>(buf0, rs_c, N, ncol0, rowg0, rrel, ncol0, p.N);
        } else if (EPI == EPI_SWIGLU) {
            constexpr int HALF = T::NF / 2;
            const float s = srow[mf];
#pragma unroll
            for (int f = 0; f < HALF; ++f)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float g[4], u[4], a[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        g[q] = acc[mf][f][4 * j + q];
                        u[q] = acc[mf][f + HALF][4 * j + q];
                        a[q] = g[q] * sigmoidf_(g[q]) * u[q] * s;
                    }
                    const int o = ml * LDW + f * 32 + 8 * j + nq;
                    stage4(buf0 + o, g[0], g[1], g[2], g[3]);
                    stage4(buf1 + o, u[0], u[1], u[2], u[3]);
                    stage4(buf2 + o, a[0], a[1], a[2], a[3]);
                }
            flush_tile<COLS>(buf0, rs_c, 2 * N, ncol0, rowg0, rrel, ncol0, p.N);
            flush_tile<COLS>(buf1, rs_c, 2 * N, N + ncol0, rowg0, rrel, ncol0, p.N);
            flush_tile<COLS>(buf2, rs_c2, N, ncol0, rowg0, rrel, ncol0, p.N);
        } else {  // dY1
            const int row = row0 + rowg0 + ml;
            const bool rok = row < rend;
            const float s = srow[mf];
            // the slab's pre-activations go to the buffers that take d_gate and d_up afterwards (a
            // lane reads exactly the positions it overwrites), then the next slab's loads start
            {
                const int c = (lane % PRE_LPR) * 8;
#pragma unroll
                for (int it = 0; it < PRE_IT; ++it) {
                    const int r = it * PRE_RPI + lane / PRE_LPR;
                    if (PREFETCH) {
                        *reinterpret_cast<u32x4*>(bufg + r * LDW + c) = gv[it];
                        *reinterpret_cast<u32x4*>(bufu + r * LDW + c) = uv[it];
                    } else {   // load and hand over one row group at a time: few registers live
                        const int grow = rowg0 + r;
                        const bool ok = grow < rrel && ncol0 + c < p.N;
                        const uint32_t po = ok ? ((uint32_t)grow * 2u * N + (uint32_t)(ncol0 + c)) * 2u : kInvalid;
                        const u32x4 g16 = buf_load16(rs_pre, po);
                        const u32x4 u16 = buf_load16(rs_pre, po == kInvalid ? kInvalid : po + N * 2u);
                        *reinterpret_cast<u32x4*>(bufg + r * LDW + c) = g16;
                        *reinterpret_cast<u32x4*>(bufu + r * LDW + c) = u16;
                    }
                }
                if (PREFETCH && mf + 1 < T::MF) load_pre(mf + 1);
            }
            float dsp = 0.f;
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int nl = nf * 32 + 8 * j + nq;   // column inside the wave tile
                    const int o = ml * LDW + nl;
                    const uint2 gr = *reinterpret_cast<const uint2*>(bufg + o);
                    const uint2 ur = *reinterpret_cast<const uint2*>(bufu + o);
                    float wa[4], dg[4], du[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t gw = q < 2 ? gr.x : gr.y, uw = q < 2 ? ur.x : ur.y;
                        const float g = elem_bits_to_f32((q & 1) ? gw >> 16 : gw & 0xffffu);
                        const float u = elem_bits_to_f32((q & 1) ? uw >> 16 : uw & 0xffffu);
                        const float a = acc[mf][nf][4 * j + q];
                        const float sig = sigmoidf_(g);
                        const float silu = g * sig;
                        const float y1 = silu * u;
                        dsp += a * y1;
                        wa[q] = s * y1;
                        const float da = a * s;
                        // d silu/dg * u = (sig + silu (1 - sig)) u = y1 + sig (u - y1)
                        dg[q] = da * __builtin_fmaf(sig, u - y1, y1);
                        du[q] = da * silu;
                    }
                    if (WACT) stage4(buf0 + o, wa[0], wa[1], wa[2], wa[3]);
                    stage4(bufg + o, dg[0], dg[1], dg[2], dg[3]);
                    stage4(bufu + o, du[0], du[1], du[2], du[3]);
                }
            dsp += __shfl_xor(dsp, 32, MTS_WAVE);
            // one partial per 64 output columns, whatever the tile shape: a wave that
            // covers 128 columns writes its sum to the first slot and 0 to the second
            if (rok && lane < 32) {
                const int slot = ncol0 / 64;
#pragma unroll
                for (int q = 0; q < T::WN / 64; ++q)
                    if (slot + q < p.np) p.ds_part[(int64_t)row * p.np + slot + q] = q == 0 ? dsp : 0.f;
            }
            if (WACT) flush_tile<COLS>(buf0, rs_c2, N, ncol0, rowg0, rrel, ncol0, p.N);
            flush_tile<COLS>(bufg, rs_c, 2 * N, ncol0, rowg0, rrel, ncol0, p.N);
            flush_tile<COLS>(bufu, rs_c, 2 * N, N + ncol0, rowg0, rrel, ncol0, p.N);
        }
    }
}

// ---------------------------------------------------------------------------
// block -> tile mapping.  Workgroups are handed to the 8 XCDs round-robin
// (block b runs on XCD b % 8) and every XCD has its own L2.  The m-tiles are in
// expert order, so every XCD is given a contiguous range of them (xcd_ranges = 1):
// it works its way through one expert after the other, the expert's weights are
// fetched into that L2 once and every m-tile of the range finds them there, and the
// j-th block of an XCD computes n-tile j % n_tiles of the range's m-tile j / n_tiles,
// so all column tiles of an m-tile (same activation rows) run side by side.  The
// Two refinements of the range mapping (measured together: 1.5 % of the layer step).  n_groups: where an
// expert's weights take more than half an L2, the n-tiles are walked in groups - all m-tiles of the range for
// the first group of weight columns, then for the next - so that a group's weights stay in the L2 next to the
// activations and outputs that stream through it (gate/up at 768/1024: 280 instead of 350 MB fetched, for
// reading the activations twice).  reverse: a GEMM that reads what the launch before it has just written
// (down after gate/up, dX after dY1) walks its range from the last m-tile to the first, so it starts with the
// rows the caches still hold.
// The older mapping (xcd_ranges = 0) deals the m-tiles round-robin, m-tile
// xcd + 8*(j / n_tiles): all eight L2s then stream the same expert's weights at the
// same time and each of them again for every group of m-tiles.
// ---------------------------------------------------------------------------
constexpr int kXcds = 8;

// The expert that owns m-tile `tile` is found with one vector load: lane l reads
// expert_start[l] and [l+1], a wave scan turns tile counts into tile offsets, and a
// ballot picks the first expert whose offset range contains the tile (63 experts per
// round; more experts take more rounds).
// mtile: the m-tile's index in expert order, -1 where the block has none; a block that has the empty half of a cut tile
// (the tile's rows end in the other half) gets the index and the answer false.
template <int BM>
__device__ __forceinline__ bool find_rows_tile(const RowsParams& p, int b, int& e, int& row0, int& rend, int& ntile, int& parts,
                                               int& mtile) {
    mtile = -1;
    // up to 64 experts: lane l reads expert_start[l] and [l + 1] once, for the count of m-tiles and for the search
    const bool in_regs = p.E <= MTS_WAVE;
    const int lane_ = threadIdx.x % MTS_WAVE;
    const int w0 = in_regs && lane_ < p.E ? p.expert_start[lane_] : 0;
    const int w1 = in_regs && lane_ < p.E ? p.expert_start[lane_ + 1] : 0;
    const int xcd = b % kXcds;
    int j = b / kXcds;
    const int lane = threadIdx.x % MTS_WAVE;
    int tile = xcd + kXcds * (j / p.n_tiles);
    ntile = j % p.n_tiles;
    parts = 1;      // pieces the tile is cut into: this block computes piece `part`
    int part = 0;
    if (p.xcd_ranges && p.sched) {
        // the XCD's range of m-tiles comes from the table (n-tile groups and cut tiles are not combined with it); a block
        // the table leaves without work finds that out with one load
        const int my = p.sched[kXcds + xcd];
        int k = j / p.n_tiles;
        if (k >= my) return false;
        if (p.reverse) k = my - 1 - k;
        tile = p.sched[xcd] + k;
    } else if (p.xcd_ranges) {
        // m-tiles of the launch: the first (total % 8) XCDs take one more than the others
        int mine = 0;
        if (in_regs) mine = (w1 - w0 + BM - 1) / BM;
        else
            for (int le = lane; le < p.E; le += MTS_WAVE) mine += (p.expert_start[le + 1] - p.expert_start[le] + BM - 1) / BM;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, MTS_WAVE);
        const int per = mine / kXcds, rem = mine % kXcds;
        const int my = per + (xcd < rem ? 1 : 0);
        if (p.tail_slots > 0 || p.tail_tiles > 0) {
            // the blocks behind the last whole round of this XCD: two per tile, the upper and the lower half (cutting
            // into four where a quarter of the slots is filled gains another 0.15 % of the layer step: not done)
            const int total = my * p.n_tiles;
            const int whole = p.tail_tiles > 0 ? (total > p.tail_tiles ? total - p.tail_tiles : 0) : total / p.tail_slots * p.tail_slots;
            const int cut = p.tail_tiles > 0 || 2 * (total - whole) <= p.tail_slots ? 2 : 1;
            if (cut > 1 && j >= whole) {
                parts = cut;
                part = (j - whole) % cut;
                j = whole + (j - whole) / cut;
                ntile = j % p.n_tiles;
            }
        }
        int k = j / p.n_tiles;
        if (p.n_groups > 1 && my > 0) {
            const int npg = p.n_tiles / p.n_groups;   // n-tiles per group (n_tiles is a multiple of n_groups)
            const int g = j / (my * npg);
            if (g >= p.n_groups) return false;
            const int r = j - g * my * npg;
            k = r / npg;
            ntile = g * npg + r % npg;
        }
        if (k >= my) return false;
        if (p.reverse) k = my - 1 - k;
        tile = xcd * per + (xcd < rem ? xcd : rem) + k;
    }
    int seen = 0;
    for (int e0 = 0; e0 < p.E; e0 += MTS_WAVE) {
        const int le = e0 + lane;
        const int s0 = in_regs ? w0 : (le < p.E ? p.expert_start[le] : 0);
        const int s1 = in_regs ? w1 : (le < p.E ? p.expert_start[le + 1] : 0);
        const int nt = (s1 - s0 + BM - 1) / BM;
        int incl = nt;
#pragma unroll
        for (int o = 1; o < MTS_WAVE; o <<= 1) {
            const int up = __shfl_up(incl, o, MTS_WAVE);
            if (lane >= o) incl += up;
        }
        const uint64_t hit = __ballot(tile < seen + incl);
        if (hit) {
            const int w = __ffsll((unsigned long long)hit) - 1;
            const int first = seen + __shfl(incl, w, MTS_WAVE) - __shfl(nt, w, MTS_WAVE);
            e = e0 + w;
            row0 = __shfl(s0, w, MTS_WAVE) + (tile - first) * BM;
            rend = __shfl(s1, w, MTS_WAVE);
            mtile = tile;
            if (parts > 1) {
                row0 += part * (BM / parts);
                if (row0 + BM / parts < rend) rend = row0 + BM / parts;
                return row0 < rend;
            }
            return true;
        }
        seen += __shfl(incl, MTS_WAVE - 1, MTS_WAVE);
    }
    return false;
}

// The answer is the same in every lane, and the compiler is told so behind the search loop: descriptors
// and LDS addresses built from these values then stay in scalar registers (a buffer instruction whose
// descriptor sits in vector registers is wrapped in a loop over its distinct values).
template <int BM>
__device__ __forceinline__ bool locate_rows_tile(const RowsParams& p, int b, int& e, int& row0, int& rend, int& ntile, int& parts,
                                                 int& mtile) {
    int fe = 0, frow0 = 0, frend = 0, fn = 0, fh = 1, fm = -1;
    const bool found = find_rows_tile<BM>(p, b, fe, frow0, frend, fn, fh, fm);
    e = __builtin_amdgcn_readfirstlane(fe);
    row0 = __builtin_amdgcn_readfirstlane(frow0);
    rend = __builtin_amdgcn_readfirstlane(frend);
    ntile = __builtin_amdgcn_readfirstlane(fn);
    parts = __builtin_amdgcn_readfirstlane(fh);
    mtile = __builtin_amdgcn_readfirstlane(fm);
    return __builtin_amdgcn_readfirstlane((int)found) != 0;
}
template <int BM>
__device__ __forceinline__ bool locate_rows_tile(const RowsParams& p, int b, int& e, int& row0, int& rend, int& ntile, int& parts) {
    int mtile;
    return locate_rows_tile<BM>(p, b, e, row0, rend, ntile, parts, mtile);
}
template <int BM>
__device__ __forceinline__ bool locate_rows_tile(const RowsParams& p, int b, int& e, int& row0, int& rend, int& ntile) {
    int parts;   // a slice of a tile is a tile with fewer rows to a kernel that does not treat it specially
    return locate_rows_tile<BM>(p, b, e, row0, rend, ntile, parts);
}

// ---------------------------------------------------------------------------
// rows_gemm
// ---------------------------------------------------------------------------
template <class T, int EPI>
__global__ __launch_bounds__(T::NT) void rows_gemm_kernel(RowsParams p) {
    constexpr int LDS_ELEMS = T::LDS_ELEMS > EpiShape<T, EPI>::ELEMS ? T::LDS_ELEMS : EpiShape<T, EPI>::ELEMS;
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
    __shared__ __attribute__((aligned(16))) bf16_t smem[LDS_ELEMS];
    constexpr bool SWIGLU = (EPI == EPI_SWIGLU);

    if constexpr (epi_is_dy1(EPI)) {
        if (schedule_block(p)) return;
    }
    int e, row0, rend, ntile;
    if (!locate_rows_tile<T::BM>(p, blockIdx.x, e, row0, rend, ntile)) return;
    const int n0 = ntile * (SWIGLU ? T::BN / 2 : T::BN);  // first output column of this block

    KMajorLoader<T::BM, T::NT> la;
    KMajorLoader<T::BN, T::NT> lb;
    la.chunk = lb.chunk = threadIdx.x % 8;
    // an operand read in place is addressed from the tile's first row (it may be larger than a descriptor spans)
    la.rsrc = p.a_gather ? make_rsrc(p.A, p.a_rows * p.lda * 2)
                         : make_rsrc(p.A + (int64_t)row0 * p.lda, (int64_t)(rend - row0) * p.lda * 2);
    lb.rsrc = make_rsrc(p.B + (int64_t)e * p.b_rows * p.Kdim, (int64_t)p.b_rows * p.Kdim * 2);
    {
        const int r = threadIdx.x / 8;
#pragma unroll
        for (int q = 0; q < la.LOADS; ++q) {
            int row = row0 + q * (T::NT / 8) + r;
            int lrow = row < rend ? row : rend - 1;          // keep the index load in range
            int src = p.a_gather ? p.a_gather[lrow] : lrow - row0;
            la.voff[q] = row < rend ? ((uint32_t)src * (uint32_t)p.lda + la.chunk * 8) * 2u : kInvalid;
        }
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
            lb.voff[q] = (n < p.N) ? ((uint32_t)grow * (uint32_t)p.Kdim + lb.chunk * 8) * 2u : kInvalid;
        }
    }

    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
    zero_acc<T>(acc);

    constexpr int B_OFF = T::BM * BK;
    const int nk = (p.Kdim + BK - 1) / BK;
    la.fetch(0, p.Kdim);
    lb.fetch(0, p.Kdim);
    la.commit(smem);
    lb.commit(smem + B_OFF);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        bf16_t* cur = smem + (kt & 1) * T::STAGE;
        bf16_t* nxt = smem + ((kt & 1) ^ 1) * T::STAGE;
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

    rows_epilogue<T, EPI>(p, acc, smem, row0, rend, n0, wm, wn);
}

// ---------------------------------------------------------------------------
// rows_gemm, ring pipeline.  Tiles go from global memory straight into LDS with
// `buffer_load_dwordx4 ... lds` (16 bytes per lane, one KiB per wave instruction),
// STAGES deep, so the loads of tiles k+1 .. k+STAGES-1 are in flight during the
// MFMAs of tile k and no VGPRs or ds_write instructions are spent on staging.
// The LDS image of a wave instruction is fixed (lane l lands at byte 16*l), so
// the swizzle is applied on the global side: lane l fetches the chunk that
// belongs at its landing slot.  Requires Kdim % BKS == 0.
// ---------------------------------------------------------------------------
// A_STAGES_ = STAGES_ + 1: the activation tile has a buffer more than the weight tile (two stages only)
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int BKS_, int STAGES_, int WAVES_PER_EU_ = 1, int A_STAGES_ = STAGES_>
struct RingTile {
    static constexpr int A_STAGES = A_STAGES_;
    static constexpr int WAVES_PER_EU = WAVES_PER_EU_;  // register budget: 512 / WAVES_PER_EU per lane
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int BKS = BKS_, STAGES = STAGES_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;
    static constexpr int NT = NWAVES * MTS_WAVE;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MF = WM / 32, NF = WN / 32;
    static constexpr int CHUNKS = BKS / 8;          // 16-byte chunks per LDS row
    static constexpr int RPI = MTS_WAVE / CHUNKS;   // rows covered by one wave instruction
    static constexpr int A_INSTR = BM / RPI / NWAVES, B_INSTR = BN / RPI / NWAVES;
    static constexpr int STAGE = (BM + BN) * BKS;
    static constexpr int LDS_ELEMS = (A_STAGES * BM + STAGES * BN) * BKS;
    static_assert(BKS == 32 || BKS == 64, "LDS rows are 64 or 128 bytes");
    static_assert(WM % 32 == 0 && WN % 64 == 0, "wave tile must hold whole 32x32 fragments");
    static_assert(A_INSTR * RPI * NWAVES == BM && B_INSTR * RPI * NWAVES == BN, "loader split");
    static_assert(STAGES >= 2 && STAGES <= 4 && (A_INSTR + B_INSTR) * (STAGES - 2) <= 63, "vmcnt range");
    static_assert(A_STAGES == STAGES || (A_STAGES == 3 && STAGES == 2 && BKS == 32), "the extra activation buffer goes with two stages");
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
};

#define MTS_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt = simm16[15:14,3:0], expcnt [6:4], lgkmcnt [11:8])
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// BKM: B is read in the weights' stored layout [E][Kdim][N] (a row is one k) instead of the
// transposed copy [E][N][Kdim]; its tiles land in LDS as [BKS k][BN] like the operands of the
// weight-gradient GEMMs.
template <class T, int EPI, bool BKM = false>
__global__ __launch_bounds__(T::NT, T::WAVES_PER_EU) void rows_gemm_ring_kernel(RowsParams p) {
    constexpr int LDS_ELEMS = T::LDS_ELEMS > EpiShape<T, EPI>::ELEMS ? T::LDS_ELEMS : EpiShape<T, EPI>::ELEMS;
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
    __shared__ __attribute__((aligned(1024))) bf16_t smem[LDS_ELEMS];
    constexpr bool SWIGLU = (EPI == EPI_SWIGLU);
    constexpr int S = T::STAGES, L = T::A_INSTR + T::B_INSTR;

    if constexpr (epi_is_dy1(EPI)) {
        if (schedule_block(p)) return;
    }
    int e, row0, rend, ntile;
    if (!locate_rows_tile<T::BM>(p, blockIdx.x, e, row0, rend, ntile)) return;
    const int n0 = ntile * (SWIGLU ? T::BN / 2 : T::BN);
    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;

    constexpr int CPR_B = T::BN / 8, RPI_B = MTS_WAVE / CPR_B;   // k-major B: chunks per tile row, rows per instruction
    static_assert(!BKM || (EPI != EPI_SWIGLU && T::BKS / RPI_B / T::NWAVES == T::B_INSTR), "k-major B loader split");
    // an operand read in place is addressed from the tile's first row (it may be larger than a descriptor spans)
    const __amdgpu_buffer_rsrc_t rs_a = p.a_gather ? make_rsrc(p.A, p.a_rows * p.lda * 2)
                                                   : make_rsrc(p.A + (int64_t)row0 * p.lda, (int64_t)(rend - row0) * p.lda * 2);
    const __amdgpu_buffer_rsrc_t rs_b =
        make_rsrc(p.B + (int64_t)e * p.b_rows * p.Kdim, (int64_t)p.b_rows * p.Kdim * 2);
    uint32_t voff_a[T::A_INSTR], voff_b[T::B_INSTR];
    {
        const int slot = lane % T::CHUNKS, rin = lane / T::CHUNKS;
#pragma unroll
        for (int j = 0; j < T::A_INSTR; ++j) {
            const int tr = (wave * T::A_INSTR + j) * T::RPI + rin;   // row inside the A tile
            const int chunk = slot ^ (T::CHUNKS == 8 ? (tr >> 1) & 7 : (tr >> 2) & 3);
            const int row = row0 + tr;
            const int lrow = row < rend ? row : rend - 1;
            const int src = p.a_gather ? p.a_gather[lrow] : lrow - row0;
            voff_a[j] = row < rend ? ((uint32_t)src * (uint32_t)p.lda + chunk * 8) * 2u : kInvalid;
        }
#pragma unroll
        for (int j = 0; j < T::B_INSTR; ++j) {
            if constexpr (BKM) {
                const int tr = (wave * T::B_INSTR + j) * RPI_B + lane / CPR_B;   // k row inside the B tile
                const int c = n0 + (((lane % CPR_B) ^ ((tr & 3) << 2)) << 3);
                voff_b[j] = c < p.N ? ((uint32_t)tr * (uint32_t)p.N + (uint32_t)c) * 2u : kInvalid;
            } else {
                const int br = (wave * T::B_INSTR + j) * T::RPI + rin;   // row inside the B tile
                const int chunk = slot ^ (T::CHUNKS == 8 ? (br >> 1) & 7 : (br >> 2) & 3);
                int n, grow;
                if (SWIGLU) {
                    n = n0 + br % (T::BN / 2);
                    grow = (br / (T::BN / 2)) * p.N + n;
                } else {
                    n = n0 + br;
                    grow = n;
                }
                voff_b[j] = (n < p.N) ? ((uint32_t)grow * (uint32_t)p.Kdim + chunk * 8) * 2u : kInvalid;
            }
        }
    }

    // loads of one stage; `part` of `parts` selects a slice so that the refill of a
    // stage can be spread over the k-steps of the tile that is being multiplied
    auto issue = [&](int stage, int kt, int part, int parts) {
        bf16_t* sa = smem + stage * T::STAGE + wave * T::A_INSTR * 512;
        bf16_t* sb = smem + stage * T::STAGE + T::BM * T::BKS + wave * T::B_INSTR * 512;
        const int soff = kt * T::BKS * 2;
        const int soff_b = BKM ? kt * T::BKS * p.N * 2 : soff;   // a k-tile of k-major B is BKS memory rows further
#pragma unroll
        for (int j = 0; j < T::A_INSTR; ++j)
            if (j % parts == part)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, MTS_LDS_PTR(sa + j * 512), 16, (int)voff_a[j], soff, 0, 0);
#pragma unroll
        for (int j = 0; j < T::B_INSTR; ++j)
            if ((j + T::A_INSTR) % parts == part)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, MTS_LDS_PTR(sb + j * 512), 16, (int)voff_b[j], soff_b, 0, 0);
    };

    f32x16 acc[T::MF][T::NF];
    zero_acc<T>(acc);

    const int nk = p.Kdim / T::BKS;
    if constexpr (T::A_STAGES == 3 && S == 2) {
        // The activation tile (rows gathered from anywhere) is fetched two k-tiles ahead into three buffers, the
        // weight tile one ahead into two.  The weight loads of tile kt+1 are issued in the first k-step of tile kt,
        // the activation loads of tile kt+2 in the second: the wait in front of a tile then leaves only the youngest
        // activation loads in flight.
        static_assert(T::BKS / 16 == 2, "two k-steps per tile");
        auto issue_a = [&](int buf, int kt) {
            bf16_t* sa = smem + buf * T::BM * T::BKS + wave * T::A_INSTR * 512;
            const int soff = kt * T::BKS * 2;
#pragma unroll
            for (int j = 0; j < T::A_INSTR; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, MTS_LDS_PTR(sa + j * 512), 16, (int)voff_a[j], soff, 0, 0);
        };
        auto issue_b = [&](int buf, int kt) {
            bf16_t* sb = smem + 3 * T::BM * T::BKS + buf * T::BN * T::BKS + wave * T::B_INSTR * 512;
            const int soff_b = BKM ? kt * T::BKS * p.N * 2 : kt * T::BKS * 2;
#pragma unroll
            for (int j = 0; j < T::B_INSTR; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, MTS_LDS_PTR(sb + j * 512), 16, (int)voff_b[j], soff_b, 0, 0);
        };
        issue_a(0, 0);
        issue_b(0, 0);
        if (nk > 1) issue_a(1, 1);
        int abuf = 0;
        for (int kt = 0; kt < nk; ++kt) {
            if (kt + 1 < nk) wait_vmcnt<T::A_INSTR>();
            else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();   // tile kt has landed for every wave, and every wave is past tile kt-1
            const bf16_t* ca = smem + abuf * T::BM * T::BKS;
            const bf16_t* cb = smem + 3 * T::BM * T::BKS + (kt & 1) * T::BN * T::BKS;
            const int a_next = abuf == 0 ? 2 : abuf - 1;   // buffer of tile kt+2 = buffer of tile kt-1
            mma_tile<T, SWIGLU, T::BKS, true, BKM>(ca, cb, wm, wn, acc, [&](int ks) {
                if (ks == 0 && kt + 1 < nk) issue_b((kt + 1) & 1, kt + 1);
                if (ks == 1 && kt + 2 < nk) issue_a(a_next, kt + 2);
            });
            abuf = abuf == 2 ? 0 : abuf + 1;
        }
        __builtin_amdgcn_s_barrier();  // every wave is done reading the buffers before they are reused
        rows_epilogue<T, EPI, true>(p, acc, smem, row0, rend, n0, wm, wn);
        return;
    }
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (s < nk) issue(s, s, 0, 1);
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt) {
        // tile kt must have landed; up to S-2 younger tiles may stay in flight
        const int younger = nk - 1 - kt;
        if (S >= 4 && younger >= 2) wait_vmcnt<L * (S >= 4 ? 2 : 0)>();
        else if (S >= 3 && younger >= 1) wait_vmcnt<L>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        // every wave is past the MFMAs of tile kt-1: its stage can be refilled
        const bool refill = kt + S - 1 < nk;
        const int rstage = stage == 0 ? S - 1 : stage - 1;
        const bf16_t* cur = smem + stage * T::STAGE;
        constexpr int KSTEPS = T::BKS / 16;
        mma_tile<T, SWIGLU, T::BKS, true, BKM>(cur, cur + T::BM * T::BKS, wm, wn, acc, [&](int ks) {
            if (refill && (T::NWAVES < 8 ? true : ks == (wave / 4) % KSTEPS)) {
                if (T::NWAVES < 8) issue(rstage, kt + S - 1, ks, KSTEPS);
                else issue(rstage, kt + S - 1, 0, 1);  // waves w and w+4 share a SIMD and take turns
            }
        });
        stage = stage + 1 == S ? 0 : stage + 1;
    }
    __builtin_amdgcn_s_barrier();  // every wave is done reading the ring before it is reused
    rows_epilogue<T, EPI, true>(p, acc, smem, row0, rend, n0, wm, wn);
}

// ---------------------------------------------------------------------------
// rows_gemm, ring pipeline with specialised waves: consumer waves read fragments,
// issue MFMAs and run the epilogue; producer waves compute the gather offsets and
// issue every tile load, so that a load that cannot be queued stalls a wave that has
// no MFMAs to issue.  Pays off
// for the longer reductions (down, dX).
// ---------------------------------------------------------------------------
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int BKS_, int STAGES_, int PRODUCERS_, int WAVES_PER_EU_>
struct WsTile {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int BKS = BKS_, STAGES = STAGES_, PRODUCERS = PRODUCERS_, WAVES_PER_EU = WAVES_PER_EU_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;   // consumer waves
    static constexpr int NT = (NWAVES + PRODUCERS) * MTS_WAVE;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MF = WM / 32, NF = WN / 32;
    static constexpr int CHUNKS = BKS / 8;
    static constexpr int RPI = MTS_WAVE / CHUNKS;
    static constexpr int A_INSTR = BM / RPI / PRODUCERS, B_INSTR = BN / RPI / PRODUCERS;   // per producer wave
    static constexpr int STAGE = (BM + BN) * BKS;
    // STAGES == 3: three buffers for the activation tile and two for the weight tile (the gathered rows come from
    // further away than the weights, which mostly sit in the XCD's L2)
    static constexpr int LDS_ELEMS = STAGES == 3 ? (3 * BM + 2 * BN) * BKS : STAGES * STAGE;
    static_assert(BKS == 32 || BKS == 64, "LDS rows are 64 or 128 bytes");
    static_assert(WM % 32 == 0 && WN % 64 == 0, "wave tile must hold whole 32x32 fragments");
    static_assert(A_INSTR * RPI * PRODUCERS == BM && B_INSTR * RPI * PRODUCERS == BN, "loader split");
    static_assert((STAGES == 4 || STAGES == 2 || STAGES == 3) && (A_INSTR + B_INSTR) * 2 <= 63, "the producer waits are written for a 4-stage ring, for two buffers and for three plus two");
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
};

template <class T, int EPI>
constexpr int ws_lds_elems() {
    return T::LDS_ELEMS > EpiShape<T, EPI>::ELEMS ? T::LDS_ELEMS : EpiShape<T, EPI>::ELEMS;
}

// one output tile: rows [row0, rend) of expert e (at most T::BM of them), column tile ntile
// `rows_ready` runs in the producer waves of a tile on three activation buffers, behind the first loads of the weights and
// in front of the first loads of the activation rows (a launch whose rows are written by other blocks of the same launch).
template <class T, int EPI, bool BKM, class RowsReady = NoHook>
__device__ __forceinline__ void rows_gemm_ws_tile(const RowsParams& p, bf16_t* smem, int e, int row0, int rend, int ntile,
                                                  RowsReady rows_ready = RowsReady()) {
    constexpr bool SWIGLU = (EPI == EPI_SWIGLU);
    constexpr int S = T::STAGES, L = T::A_INSTR + T::B_INSTR;
    const int n0 = ntile * (SWIGLU ? T::BN / 2 : T::BN);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MTS_WAVE), lane = threadIdx.x % MTS_WAVE;
    const int nk = p.Kdim / T::BKS;

    if (wave >= T::NWAVES) {
        // ------------------------------ producer ------------------------------
        const int pw = wave - T::NWAVES;
        // an operand read in place is addressed from the tile's first row (it may be larger than a descriptor spans)
        const __amdgpu_buffer_rsrc_t rs_a = p.a_gather ? make_rsrc(p.A, p.a_rows * p.lda * 2)
                                                       : make_rsrc(p.A + (int64_t)row0 * p.lda, (int64_t)(rend - row0) * p.lda * 2);
        const __amdgpu_buffer_rsrc_t rs_b =
            make_rsrc(p.B + (int64_t)e * p.b_rows * p.Kdim, (int64_t)p.b_rows * p.Kdim * 2);
        uint32_t voff_a[T::A_INSTR], voff_b[T::B_INSTR];
        const int slot = lane % T::CHUNKS, rin = lane / T::CHUNKS;
        constexpr int CPR_B = T::BN / 8, RPI_B = MTS_WAVE / CPR_B;   // k-major B: chunks per tile row, rows per instruction
        static_assert(!BKM || (EPI != EPI_SWIGLU && T::BKS / RPI_B / T::PRODUCERS == T::B_INSTR), "k-major B loader split");
#pragma unroll
        for (int j = 0; j < T::A_INSTR; ++j) {
            const int tr = (pw * T::A_INSTR + j) * T::RPI + rin;
            const int chunk = slot ^ (T::CHUNKS == 8 ? (tr >> 1) & 7 : (tr >> 2) & 3);
            const int row = row0 + tr;
            const int lrow = row < rend ? row : rend - 1;
            const int src = p.a_gather ? p.a_gather[lrow] : lrow - row0;
            voff_a[j] = row < rend ? ((uint32_t)src * (uint32_t)p.lda + chunk * 8) * 2u : kInvalid;
        }
#pragma unroll
        for (int j = 0; j < T::B_INSTR; ++j) {
            if constexpr (BKM) {
                const int tr = (pw * T::B_INSTR + j) * RPI_B + lane / CPR_B;   // k row inside the B tile
                const int c = n0 + (((lane % CPR_B) ^ ((tr & 3) << 2)) << 3);
                voff_b[j] = c < p.N ? ((uint32_t)tr * (uint32_t)p.N + (uint32_t)c) * 2u : kInvalid;
            } else {
                const int br = (pw * T::B_INSTR + j) * T::RPI + rin;
                const int chunk = slot ^ (T::CHUNKS == 8 ? (br >> 1) & 7 : (br >> 2) & 3);
                int n, grow;
                if (SWIGLU) {
                    n = n0 + br % (T::BN / 2);
                    grow = (br / (T::BN / 2)) * p.N + n;
                } else {
                    n = n0 + br;
                    grow = n;
                }
                voff_b[j] = (n < p.N) ? ((uint32_t)grow * (uint32_t)p.Kdim + chunk * 8) * 2u : kInvalid;
            }
        }
        auto issue = [&](int stage, int kt) {
            bf16_t* sa = smem + stage * T::STAGE + pw * T::A_INSTR * 512;
            bf16_t* sb = smem + stage * T::STAGE + T::BM * T::BKS + pw * T::B_INSTR * 512;
            const int soff = kt * T::BKS * 2;
            const int soff_b = BKM ? kt * T::BKS * p.N * 2 : soff;   // a k-tile of k-major B is BKS memory rows further
#pragma unroll
            for (int j = 0; j < T::A_INSTR; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, MTS_LDS_PTR(sa + j * 512), 16, (int)voff_a[j], soff, 0, 0);
#pragma unroll
            for (int j = 0; j < T::B_INSTR; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, MTS_LDS_PTR(sb + j * 512), 16, (int)voff_b[j], soff_b, 0, 0);
        };
        if constexpr (S == 3) {
            // Three buffers for the activation tile, two for the weight tile.  Barrier kt says that tile kt has landed
            // and that tile kt-1 has been consumed: its weight buffer then takes tile kt+1 and its activation buffer
            // tile kt+2, which has two tiles' time to land.  The activation loads of tile kt+1, the youngest in flight,
            // may still be on their way at barrier kt-1... they are waited for one barrier later.
            auto issue_a = [&](int buf, int kt) {
                bf16_t* sa = smem + buf * T::BM * T::BKS + pw * T::A_INSTR * 512;
#pragma unroll
                for (int j = 0; j < T::A_INSTR; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, MTS_LDS_PTR(sa + j * 512), 16, (int)voff_a[j], kt * T::BKS * 2, 0, 0);
            };
            auto issue_b = [&](int buf, int kt) {
                bf16_t* sb = smem + 3 * T::BM * T::BKS + buf * T::BN * T::BKS + pw * T::B_INSTR * 512;
                const int soff_b = BKM ? kt * T::BKS * p.N * 2 : kt * T::BKS * 2;   // a k-tile of k-major B is BKS memory rows further
#pragma unroll
                for (int j = 0; j < T::B_INSTR; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, MTS_LDS_PTR(sb + j * 512), 16, (int)voff_b[j], soff_b, 0, 0);
            };
            // in this order the loads that the first barrier does not wait for are still the youngest
            issue_b(0, 0);
            rows_ready(0);
            issue_a(0, 0);
            if (nk > 1) issue_a(1, 1);
            int abuf = 2;   // activation buffer of tile kt+2
            for (int kt = 0; kt < nk; ++kt) {
                if (kt + 1 < nk) wait_vmcnt<T::A_INSTR>();   // all but the activation tile kt+1
                else wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
                if (kt + 1 < nk) issue_b((kt + 1) & 1, kt + 1);
                if (kt + 2 < nk) issue_a(abuf, kt + 2);
                abuf = abuf == 2 ? 0 : abuf + 1;
            }
            __builtin_amdgcn_s_barrier();       // matches the consumers' barrier behind the last tile
            return;
        }
        if constexpr (S == 2) {
            // Two buffers of 64-wide k-tiles (a row contributes a whole 128-byte line per load): barrier kt says
            // that tile kt has landed and that tile kt-1 has been consumed, whose buffer then takes tile kt+1.
            issue(0, 0);
            for (int kt = 0; kt < nk; ++kt) {
                wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
                if (kt + 1 < nk) issue((kt + 1) & 1, kt + 1);
            }
            __builtin_amdgcn_s_barrier();       // matches the consumers' barrier behind the last tile
            return;
        }
        // Barrier kt tells the consumers that tiles kt and kt+1 have landed (they read the first
        // fragments of tile kt+1 behind the last MFMAs of tile kt) and tells the producers that
        // every consumer is done with tile kt-1, whose stage then takes tile kt-1+S.
#pragma unroll
        for (int s = 0; s < S; ++s)
            if (s < nk) issue(s, s);
        int stage = S - 1;   // stage of tile kt-1
        for (int kt = 0; kt < nk; ++kt) {
            // tiles up to kt+1 must have landed; tile kt+2 (and, before barrier 0, tile 3) may be in flight
            if (kt == 0 && S >= 4 && nk >= 4) wait_vmcnt<L * (S >= 4 ? 2 : 0)>();
            else if (S >= 3 && kt + 2 < nk) wait_vmcnt<L>();
            else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            if (kt >= 1 && kt - 1 + S < nk) issue(stage, kt - 1 + S);
            stage = stage + 1 == S ? 0 : stage + 1;
        }
        __builtin_amdgcn_s_barrier();       // matches the consumers' barrier behind the last tile
        return;
    }

    // -------------------------------- consumer --------------------------------
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
    zero_acc<T>(acc);
    FragPipe<T, SWIGLU, T::BKS, BKM> pipe;
    pipe.init(wm, wn);
    constexpr int KSTEPS = T::BKS / 16;
    if constexpr (S == 3) {
        int abuf = 0;
        for (int kt = 0; kt < nk; ++kt) {
            __builtin_amdgcn_s_barrier();   // tile kt is visible
            const bf16_t* cur = smem + abuf * T::BM * T::BKS;
            const bf16_t* cur_b = smem + 3 * T::BM * T::BKS + (kt & 1) * T::BN * T::BKS - T::BM * T::BKS;
            abuf = abuf == 2 ? 0 : abuf + 1;
            pipe.prime(cur, cur_b);
#pragma unroll
            for (int ks = 0; ks < KSTEPS - 1; ++ks) pipe.step(ks, acc, cur, cur_b, ks + 1);
            pipe.template step<false>(KSTEPS - 1, acc, cur, cur_b, 0);
        }
        __builtin_amdgcn_s_barrier();       // every wave is done with the buffers before the epilogue reuses them
        rows_epilogue<T, EPI>(p, acc, smem, row0, rend, n0, wm, wn);
        return;
    }
    if constexpr (S == 2) {
        for (int kt = 0; kt < nk; ++kt) {
            __builtin_amdgcn_s_barrier();   // tile kt is visible
            const bf16_t* cur = smem + (kt & 1) * T::STAGE;
            pipe.prime(cur);
#pragma unroll
            for (int ks = 0; ks < KSTEPS - 1; ++ks) pipe.step(ks, acc, cur, ks + 1);
            pipe.template step<false>(KSTEPS - 1, acc, cur, 0);
        }
        __builtin_amdgcn_s_barrier();       // every wave is done with the buffers before the epilogue reuses them
        rows_epilogue<T, EPI>(p, acc, smem, row0, rend, n0, wm, wn);
        return;
    }
    __builtin_amdgcn_s_barrier();   // tiles 0 and 1 are visible
    pipe.prime(smem);
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt) {
        const bf16_t* cur = smem + stage * T::STAGE;
        stage = stage + 1 == S ? 0 : stage + 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS - 1; ++ks) pipe.step(ks, acc, cur, ks + 1);
        // behind the last k-step the first fragments of tile kt+1 are read (after the last tile
        // this reads a stage nobody uses: harmless)
        pipe.step(KSTEPS - 1, acc, smem + stage * T::STAGE, 0);
        // tile kt+2 is visible after this barrier and tile kt may be overwritten; behind the last
        // tile it is the barrier that frees the ring for the epilogue
        __builtin_amdgcn_s_barrier();
    }
    rows_epilogue<T, EPI>(p, acc, smem, row0, rend, n0, wm, wn);
}

// the work of block `block` of a launch; `smem` holds ws_lds_elems<T, EPI>() elements, 1 KiB aligned.
// TH (same block shape and columns, half the rows) runs the halves of the tiles that a launch with tail_slots cuts up.
// a located tile, whole (T) or one of `parts` = 2 halves (TH)
template <class T, int EPI, bool BKM, class TH, class RowsReady = NoHook>
__device__ __forceinline__ void rows_gemm_ws_run(const RowsParams& p, bf16_t* smem, int e, int row0, int rend, int ntile, int parts,
                                                 RowsReady rows_ready = RowsReady()) {
    if constexpr (TH::BM != T::BM) {
        if (parts == 2) return rows_gemm_ws_tile<TH, EPI, BKM>(p, smem, e, row0, rend, ntile, rows_ready);
    }
    rows_gemm_ws_tile<T, EPI, BKM>(p, smem, e, row0, rend, ntile, rows_ready);
}

template <class T, int EPI, bool BKM, class TH = T>
__device__ __forceinline__ void rows_gemm_ws_block(const RowsParams& p, bf16_t* smem, int block) {
    static_assert(TH::NT == T::NT && TH::BN == T::BN && (TH::BM == T::BM || 2 * TH::BM == T::BM), "half tile shape");
    static_assert(ws_lds_elems<TH, EPI>() <= ws_lds_elems<T, EPI>(), "the half tile fits the same LDS");
    int e, row0, rend, ntile, parts;
    if (!locate_rows_tile<T::BM>(p, block, e, row0, rend, ntile, parts)) return;
    rows_gemm_ws_run<T, EPI, BKM, TH>(p, smem, e, row0, rend, ntile, parts);
}

template <class T, int EPI, bool BKM = false, class TH = T>
__global__ __launch_bounds__(T::NT, T::WAVES_PER_EU) void rows_gemm_ws_kernel(RowsParams p) {
    static_assert(ws_lds_elems<T, EPI>() * 2 <= 160 * 1024, "LDS capacity");
    __shared__ __attribute__((aligned(1024))) bf16_t smem[ws_lds_elems<T, EPI>()];
    if constexpr (epi_is_dy1(EPI)) {
        if (schedule_block(p)) return;
    }
    rows_gemm_ws_block<T, EPI, BKM, TH>(p, smem, blockIdx.x);
}

// ---------------------------------------------------------------------------
// dw_gemm
// ---------------------------------------------------------------------------
struct DwParams {
    const bf16_t* P;  // rows -> M side, row-major [p_rows, M]
    int64_t p_rows;
    const int32_t* p_gather;
    const bf16_t* Q;  // rows -> N side, row-major [q_rows, N]
    int64_t q_rows;
    const int32_t* q_gather;
    int M, N;
    int64_t TK;
    const int32_t* expert_start;
    void* C;  // [E][M][N], bf16 or f32
    float* part;   // fp32 tile partials of experts whose rows are split over several blocks, or null
    int E, n_tiles, tiles_per_expert;  // set by the launcher
    const int32_t* sched;   // the unit table of the joint backward launch's schedule (which units an XCD runs), or NULL:
    int sched_slots;        // unit u runs on XCD u % 8; sched_slots: table entries per XCD
};

// ---------------------------------------------------------------------------
// Row chunks of over-full experts.  A weight-gradient tile reduces over all rows of its
// expert, so with skewed routing the tiles of the fullest expert set the kernel's time.
// When the caller supplies a workspace, an expert with more than 1.15 times the balanced
// share of rows (share = ceil(kept routes / E), rounded up to 32) is cut into
// ceil(count / share) chunks of equal length (a multiple of 32 rows).  A (expert, chunk)
// pair is a unit; the units of an expert that was cut write fp32 tiles to the workspace,
// slot by slot, and a second kernel adds the chunks of a tile in chunk order, so the result
// does not depend on the order the blocks ran in.  There are at most 2E units.
// ---------------------------------------------------------------------------
struct DwUnit {
    int e, rbeg, rend;   // expert and the rows of this unit
    int slot;            // index of the unit's partial tiles in the workspace, -1: writes C itself
};

__device__ __forceinline__ int dw_share_of(const int32_t* expert_start, int E) {
    const int total = expert_start[E] - expert_start[0];   // the caller may pass a sub-range of the experts
    return ((total + E - 1) / E + 31) / 32 * 32;
}
__device__ __forceinline__ int dw_share(const DwParams& p) { return dw_share_of(p.expert_start, p.E); }

// 1.15 shares: uniform routing stays far below it (the counts of 24576 tokens scatter by about 1 %), and at the uneven
// routing of a trained router it beats 1.25 by 2-3 % of the layer step where an expert falls between the two
__device__ __forceinline__ int dw_chunks_cut(int count, int share) { return count > share + share * 3 / 20 ? (count + share - 1) / share : 1; }
__device__ __forceinline__ int dw_chunks(const DwParams& p, int count, int share) {
    return p.part != nullptr ? dw_chunks_cut(count, share) : 1;
}

// every lane of the calling wave gets the same answer
__device__ __forceinline__ bool locate_dw_unit(const DwParams& p, int unit, DwUnit& u) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int share = dw_share(p);
    int seen = 0, seen_slots = 0;
    for (int e0 = 0; e0 < p.E; e0 += MTS_WAVE) {
        const int le = e0 + lane;
        const int s0 = le < p.E ? p.expert_start[le] : 0;
        const int s1 = le < p.E ? p.expert_start[le + 1] : 0;
        const int nc = le < p.E ? dw_chunks(p, s1 - s0, share) : 0;
        const int ns = nc > 1 ? nc : 0;
        int incl = nc, sincl = ns;
#pragma unroll
        for (int o = 1; o < MTS_WAVE; o <<= 1) {
            const int up = __shfl_up(incl, o, MTS_WAVE), sup = __shfl_up(sincl, o, MTS_WAVE);
            if (lane >= o) {
                incl += up;
                sincl += sup;
            }
        }
        const uint64_t hit = __ballot(le < p.E && unit < seen + incl);
        if (hit) {
            const int w = __ffsll((unsigned long long)hit) - 1;
            const int ncw = __shfl(nc, w, MTS_WAVE);
            const int c = unit - (seen + __shfl(incl, w, MTS_WAVE) - ncw);
            const int b = __shfl(s0, w, MTS_WAVE), e = __shfl(s1, w, MTS_WAVE);
            const int per = ((e - b + ncw - 1) / ncw + 31) / 32 * 32;
            const int r0 = b + c * per;
            u.e = e0 + w;
            u.rbeg = r0 < e ? r0 : e;
            u.rend = r0 + per < e ? r0 + per : e;
            u.slot = ncw > 1 ? seen_slots + __shfl(sincl, w, MTS_WAVE) - __shfl(ns, w, MTS_WAVE) + c : -1;
            return true;
        }
        seen += __shfl(incl, MTS_WAVE - 1, MTS_WAVE);
        seen_slots += __shfl(sincl, MTS_WAVE - 1, MTS_WAVE);
    }
    return false;
}


// ---------------------------------------------------------------------------
// Schedule of the joint backward launch under uneven routing.  Block b of a launch runs on XCD b % 8, and
// the weight-gradient tiles of a unit (an expert, or a row chunk of an over-full one) all run on one XCD.  With
// the units dealt round-robin an XCD that draws two long units finishes far behind the others (routing in a
// trained model is uneven: the fullest expert of a layer holds 1.1 to 2 times the balanced share).  One wave
// works the deal out before the launch: the units go to the XCDs longest first, each to the XCD with the least
// rows so far (at most `slots` units per XCD, which is what the grid holds), and the dX tiles, which any XCD
// can run, are split so that weight-gradient and dX work together are the same everywhere: a row costs a
// weight-gradient unit 6 H I FLOPs (dW1 and dW2) and a dX tile 4 H I.  Which XCD computes a tile has no
// influence on the tile's value: results are the same as with the round-robin deal, bit for bit.
// Table (int32): [0,8) first dX m-tile of every XCD, [8,16) its number of m-tiles, [16,24) its number of
// units, from kSchedUnits on (e, first row, end row, workspace slot) of unit k of XCD x at (x * slots + k) * 4.
// ---------------------------------------------------------------------------
constexpr int kSchedCounts = 16, kSchedUnits = 32;
constexpr int kSchedMaxExperts = 32;          // one unit per lane: 2 E <= 64
constexpr int64_t kSchedBytes = 4096;         // (32 + 8 * 8 * 4) * 4 bytes are used
// Called by one whole wave (lane = threadIdx.x % 64); E <= kSchedMaxExperts.  Units are cut as locate_dw_unit cuts
// them when it has a workspace for the chunk partials.
__device__ __forceinline__ void joint_schedule_wave(const int32_t* __restrict__ expert_start, int E, int slots, int dx_bm,
                                                    int dx_cap, int32_t* __restrict__ sched) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int share = dw_share_of(expert_start, E);
    const int s0 = lane < E ? expert_start[lane] : 0, s1 = lane < E ? expert_start[lane + 1] : 0;
    const int nc = lane < E ? dw_chunks_cut(s1 - s0, share) : 0;
    const int ns = nc > 1 ? nc : 0;
    const int nt = (s1 - s0 + dx_bm - 1) / dx_bm;
    int uincl = nc, sincl = ns, tincl = nt;
#pragma unroll
    for (int o = 1; o < MTS_WAVE; o <<= 1) {
        const int a = __shfl_up(uincl, o, MTS_WAVE), b = __shfl_up(sincl, o, MTS_WAVE), c = __shfl_up(tincl, o, MTS_WAVE);
        if (lane >= o) {
            uincl += a;
            sincl += b;
            tincl += c;
        }
    }
    const int n_units = __shfl(uincl, MTS_WAVE - 1, MTS_WAVE);
    const int m_tiles = __shfl(tincl, MTS_WAVE - 1, MTS_WAVE);
    // lane u < n_units: unit u in expert order
    int ue = 0, ub = 0, uend = 0, uslot = -1;
    for (int e = 0; e < E; ++e) {
        const int n = __shfl(nc, e, MTS_WAVE), off = __shfl(uincl, e, MTS_WAVE) - n;
        const int b = __shfl(s0, e, MTS_WAVE), en = __shfl(s1, e, MTS_WAVE);
        const int sl = __shfl(sincl, e, MTS_WAVE) - __shfl(ns, e, MTS_WAVE);
        if (lane >= off && lane < off + n) {
            const int c = lane - off;
            const int per = ((en - b + n - 1) / n + 31) / 32 * 32;
            const int r0 = b + c * per;
            ue = e;
            ub = r0 < en ? r0 : en;
            uend = r0 + per < en ? r0 + per : en;
            uslot = n > 1 ? sl + c : -1;
        }
    }
    const int urows = lane < n_units ? uend - ub : 0;
    int rank = 0;   // position in the order longest first (ties: expert order)
    for (int v = 0; v < n_units; ++v) {
        const int rv = __shfl(urows, v, MTS_WAVE);
        rank += (rv > urows || (rv == urows && v < lane)) ? 1 : 0;
    }
    // the rows of the units in that order, one per lane, so that the deal below reads them with a lane index
    int sorted_rows = 0;
    for (int v = 0; v < n_units; ++v) {
        const int rk = __shfl(rank, v, MTS_WAVE), rv = __shfl(urows, v, MTS_WAVE);
        if (rk == lane) sorted_rows = rv;
    }
    int load[kXcds], held[kXcds];
#pragma unroll
    for (int x = 0; x < kXcds; ++x) load[x] = held[x] = 0;
    int my_x = 0, my_k = 0;
    for (int k = 0; k < n_units; ++k) {
        const int r = __builtin_amdgcn_readlane(sorted_rows, k);
        int best = -1, best_load = 0;
#pragma unroll
        for (int x = 0; x < kXcds; ++x)
            if (held[x] < slots && (best < 0 || load[x] < best_load)) {
                best = x;
                best_load = load[x];
            }
#pragma unroll
        for (int x = 0; x < kXcds; ++x)
            if (x == best) {
                if (rank == k) {
                    my_x = x;
                    my_k = held[x];
                }
                load[x] += r;
                held[x] += 1;
            }
    }
    if (lane < n_units) {
        int32_t* u = sched + kSchedUnits + (my_x * slots + my_k) * 4;
        u[0] = ue; u[1] = ub; u[2] = uend; u[3] = uslot;
    }
    if (lane == 0) {
        // dX rows an XCD should take: (5 * total / 8 - 3 * its weight-gradient rows) / 2, not below zero; the
        // m-tiles (in expert order) are cut at the running sums of these wishes, at most dx_cap of them per XCD
        const float total = (float)(expert_start[E] - expert_start[0]);
        float want[kXcds], sum = 0.f;
#pragma unroll
        for (int x = 0; x < kXcds; ++x) {
            const float w = 5.f * total - 24.f * (float)load[x];
            want[x] = w > 0.f ? w : 0.f;
            sum += want[x];
        }
        const float scale = sum > 0.f ? (float)m_tiles * __builtin_amdgcn_rcpf(sum) : 0.f;
        int count[kXcds];
        float run = 0.f;
        int before = 0;
#pragma unroll
        for (int x = 0; x < kXcds; ++x) {
            run += want[x];
            int upto = sum > 0.f ? (int)(run * scale + 0.5f) : (m_tiles * (x + 1)) / kXcds;
            upto = upto < before ? before : (upto > m_tiles ? m_tiles : upto);
            if (x == kXcds - 1) upto = m_tiles;
            count[x] = upto - before;
            before = upto;
        }
        int carry = 0;   // what an XCD cannot hold moves to the next one, and what is left at the end moves back
#pragma unroll
        for (int x = 0; x < kXcds; ++x) {
            const int c = count[x] + carry;
            count[x] = c > dx_cap ? dx_cap : c;
            carry = c - count[x];
        }
#pragma unroll
        for (int x = kXcds - 1; x >= 0; --x) {
            const int c = count[x] + carry;
            count[x] = c > dx_cap ? dx_cap : c;
            carry = c - count[x];
        }
        int first = 0;
#pragma unroll
        for (int x = 0; x < kXcds; ++x) {
            sched[x] = first;
            sched[kXcds + x] = count[x];
            sched[kSchedCounts + x] = held[x];
            first += count[x];
        }
    }
}

// the schedule in a launch of its own (for a caller whose dO*W2 GEMM is not this library's)
__global__ __launch_bounds__(MTS_WAVE) void joint_schedule_kernel(const int32_t* expert_start, int E, int slots, int dx_bm, int dx_cap,
                                                                    int32_t* sched) {
    joint_schedule_wave(expert_start, E, slots, dx_bm, dx_cap, sched);
}

// Adds the chunk partials of the experts that were cut: thread = 4 consecutive columns of a tile row.
template <int BM, int BN, typename OutT>
__device__ __forceinline__ void dw_chunk_sum_expert(const DwParams& p, int e) {
    const int lane = threadIdx.x % MTS_WAVE;
    const int share = dw_share(p);
    const int nc = dw_chunks(p, p.expert_start[e + 1] - p.expert_start[e], share);
    if (nc <= 1) return;
    int before = 0;   // slots of the experts below e
    for (int le = lane; le < e; le += MTS_WAVE) {
        const int c = dw_chunks(p, p.expert_start[le + 1] - p.expert_start[le], share);
        before += c > 1 ? c : 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o, MTS_WAVE);
    constexpr int PER_TILE = BM * BN / 4;
    const int64_t tile_stride = (int64_t)BM * BN;
    const int64_t items = (int64_t)p.tiles_per_expert * PER_TILE;
    for (int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x; item < items; item += (int64_t)gridDim.x * 256) {
        const int tile = (int)(item / PER_TILE), within = (int)(item % PER_TILE);
        const int ml = within / (BN / 4), nl = (within % (BN / 4)) * 4;
        const int m = (tile / p.n_tiles) * BM + ml, n = (tile % p.n_tiles) * BN + nl;
        if (m >= p.M || n >= p.N) continue;
        const float* src = p.part + ((int64_t)before * p.tiles_per_expert + tile) * tile_stride + (int64_t)ml * BN + nl;
        const int64_t chunk_stride = (int64_t)p.tiles_per_expert * tile_stride;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int c0 = 0; c0 < nc; c0 += 4) {   // four loads in flight, added in chunk order
            f32x4 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[j] = c0 + j < nc ? *reinterpret_cast<const f32x4*>(src + (c0 + j) * chunk_stride) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) acc += v[j];
        }
        OutT* C = reinterpret_cast<OutT*>(p.C) + ((int64_t)e * p.M + m) * p.N + n;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (n + j < p.N) C[j] = (OutT)acc[j];
    }
}

template <int BM, int BN, typename OutT>
__global__ __launch_bounds__(256) void dw_chunk_sum_kernel(DwParams p) {
    dw_chunk_sum_expert<BM, BN, OutT>(p, blockIdx.y);
}

// What follows the joint backward launch of the layer node besides the chunk sums: the sum of the router's
// dW_r partials and the dX combine (which adds the router's share of dx), as further rows of blocks.
struct TailJobs {
    const float* r_part;    // [r_blocks][r_EH] partial dW_r (NULL: none)
    int r_blocks;
    int64_t r_EH;
    float* r_dw;
    int r_rows;             // rows of blocks (blockIdx.y) that sum dW_r
    const bf16_t* c_y;      // dx_expanded [T*2, H] (NULL: no combine)
    const bf16_t* c_addend; // [T, H]
    const int32_t* c_srev;
    int64_t c_T;
    int c_H;
    bf16_t* c_out;          // dx [T, H]
    int c_rows;             // rows of blocks that combine
};

// the same for two GEMMs over the same experts in one launch: blockIdx.y < E is the first's expert; the rows of
// blocks past the second's experts take the jobs in `t`
template <int BM, int BN, typename OutT>
__global__ __launch_bounds__(256) void dw_chunk_sum_pair_kernel(DwParams a, DwParams b, TailJobs t) {
    static_assert(mts_rl::kReduceThreads == 256 && mts_cb::kCombineThreads == 256, "one block shape");
    int e = blockIdx.y;
    if (e < a.E) return dw_chunk_sum_expert<BM, BN, OutT>(a, e);
    e -= a.E;
    if (e < b.E) return dw_chunk_sum_expert<BM, BN, OutT>(b, e);
    e -= b.E;
    if (e < t.r_rows) return mts_rl::router_dw_reduce_block(t.r_part, t.r_blocks, t.r_EH, t.r_dw, (int64_t)e * gridDim.x + blockIdx.x);
    e -= t.r_rows;
    // two routes per token: the combine of the layer's dX (plain sum of the two expert rows plus the addend)
    mts_cb::combine_rows_block<bf16_t, 2, 2>(t.c_y, (const bf16_t*)nullptr, t.c_addend, t.c_srev, t.c_T, 2, t.c_H, t.c_out,
                                             (int64_t)e * gridDim.x + blockIdx.x, (int64_t)t.c_rows * gridDim.x);
}

// Stages a [64 k][64 m] block per wave-item: lane = (kgrp = lane%8, mc = lane/8) loads
// rows k = 8*kgrp+i, columns 8*mc..8*mc+7, transposes the 8x8 block in registers
// and writes 8 rows of LDS (m-major, 16 bytes of k each).  Gathered operands take
// their source rows from one index load per k-tile (lane j holds the index of row
// j), fetched one tile ahead and spread with cross-lane reads.
template <class T>
struct MMajorLoader {
    static constexpr int ITEMS_A = T::BM / 64, ITEMS_B = T::BN / 64;
    static constexpr int ITEMS = ITEMS_A + ITEMS_B;
    static constexpr int PER_WAVE = (ITEMS + T::NWAVES - 1) / T::NWAVES;
    __amdgpu_buffer_rsrc_t rs_p, rs_q, rs_gp, rs_gq;
    bool gp, gq;
    int tok_p, tok_q;  // source row of k-row `lane` of the tile that is fetched next
    u32x4 reg[PER_WAVE][8];

    __device__ __forceinline__ void init(const DwParams& p) {
        gp = p.p_gather != nullptr;
        gq = p.q_gather != nullptr;
        rs_p = make_rsrc(p.P, gp ? p.p_rows * p.M * 2 : 0);   // an operand read in place gets its descriptor per k-tile
        rs_q = make_rsrc(p.Q, gq ? p.q_rows * p.N * 2 : 0);
        rs_gp = make_rsrc(p.p_gather, gp ? p.TK * 4 : 0);
        rs_gq = make_rsrc(p.q_gather, gq ? p.TK * 4 : 0);
    }
    // source rows for the tile starting at row r0 (rows past the end read index 0; they are masked later);
    // an operand read in place is addressed from the tile's first row, so its row index is the k-row itself
    __device__ __forceinline__ void fetch_index(int r0) {
        const int lane = threadIdx.x % MTS_WAVE;
        tok_p = gp ? buf_load4(rs_gp, (uint32_t)(r0 + lane) * 4u) : lane;
        tok_q = gq ? buf_load4(rs_gq, (uint32_t)(r0 + lane) * 4u) : lane;
    }
    __device__ __forceinline__ void fetch(const DwParams& p, int m0, int n0, int r0, int rend) {
        const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
        const int kgrp = lane % 8, mc = lane / 8;
        const int left = rend > r0 ? rend - r0 : 0;
        const __amdgpu_buffer_rsrc_t tp = gp ? rs_p : make_rsrc(p.P + (int64_t)r0 * p.M, (int64_t)left * p.M * 2);
        const __amdgpu_buffer_rsrc_t tq = gq ? rs_q : make_rsrc(p.Q + (int64_t)r0 * p.N, (int64_t)left * p.N * 2);
#pragma unroll
        for (int q = 0; q < PER_WAVE; ++q) {
            const int item = q * T::NWAVES + wave;
            if (item >= ITEMS) break;
            const bool isA = item < ITEMS_A;
            const int dim = isA ? p.M : p.N;
            const int c = (isA ? m0 + item * 64 : n0 + (item - ITEMS_A) * 64) + mc * 8;
            const int tok = isA ? tok_p : tok_q;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int kr = kgrp * 8 + i;
                const int src = __shfl(tok, kr, MTS_WAVE);
                const bool ok = (r0 + kr < rend) && (c < dim);
                const uint32_t off = ok ? ((uint32_t)src * (uint32_t)dim + (uint32_t)c) * 2u : kInvalid;
                reg[q][i] = buf_load16(isA ? tp : tq, off);
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
            bf16_t* dst = isA ? As : Bs;
            const int rbase = (isA ? item : item - ITEMS_A) * 64 + mc * 8;
#pragma unroll
            for (int md = 0; md < 4; ++md) {
                u32x4 lo, hi;  // columns 2*md and 2*md+1 of the 8x8 block, k = 0..7
#pragma unroll
                for (int kp = 0; kp < 4; ++kp) {
                    uint32_t a = reg[q][2 * kp][md], b = reg[q][2 * kp + 1][md];
                    lo[kp] = (a & 0xffffu) | (b << 16);
                    hi[kp] = (a >> 16) | (b & 0xffff0000u);
                }
                *reinterpret_cast<u32x4*>(dst + lds_off(rbase + 2 * md, kgrp)) = lo;
                *reinterpret_cast<u32x4*>(dst + lds_off(rbase + 2 * md + 1, kgrp)) = hi;
            }
        }
    }
};

template <class T, typename OutT>
__global__ __launch_bounds__(T::NT) void dw_gemm_kernel(DwParams p) {
    __shared__ __attribute__((aligned(16))) bf16_t smem[T::LDS_ELEMS];
    // all tiles of one expert run on one XCD (block b -> XCD b % 8), so the expert's
    // activation rows stream through that XCD's L2 once and are shared by its tiles
    const int xcd = blockIdx.x % kXcds, j = blockIdx.x / kXcds;
    const int e = xcd + kXcds * (j / p.tiles_per_expert);
    if (e >= p.E) return;
    const int tile = j % p.tiles_per_expert;
    const int m0 = (tile / p.n_tiles) * T::BM, n0 = (tile % p.n_tiles) * T::BN;
    const int rbeg = p.expert_start[e], rend = p.expert_start[e + 1];

    const int wave = threadIdx.x / MTS_WAVE, lane = threadIdx.x % MTS_WAVE;
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
    zero_acc<T>(acc);

    constexpr int B_OFF = T::BM * BK;
    const int nk = (rend - rbeg + BK - 1) / BK;
    MMajorLoader<T> ld;
    ld.init(p);
    if (nk > 0) {
        ld.fetch_index(rbeg);
        ld.fetch(p, m0, n0, rbeg, rend);
        ld.fetch_index(rbeg + BK);
        ld.commit(smem, smem + B_OFF);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        bf16_t* cur = smem + (kt & 1) * T::STAGE;
        bf16_t* nxt = smem + ((kt & 1) ^ 1) * T::STAGE;
        if (kt + 1 < nk) {
            ld.fetch(p, m0, n0, rbeg + (kt + 1) * BK, rend);
            ld.fetch_index(rbeg + (kt + 2) * BK);
        }
        mma_tile<T, false, BK, false>(cur, cur + B_OFF, wm, wn, acc);
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
// dw_gemm, ring pipeline.  Both operands are k-major in memory (a row of the
// operand is one k), so tiles are brought into LDS as they are, [BKS k][BM or BN]
// with `buffer_load ... lds`, and the MFMA fragments (8 consecutive k per lane)
// are read with the transposing LDS load ds_read_b64_tr_b16: within a group of 16
// lanes, lane s addresses 4 consecutive columns of row s/4 and lane l receives the
// 4 rows of column l.  The 16-byte chunk index of a row is XOR-swizzled with
// 4*(row % 4) so that the 4 rows x 2 column halves read by 32 lanes cover all banks.
// Source rows of a gathered operand come from a scalar load of the row indices, one
// k-tile ahead.  Rows past the expert's end are fetched with an out-of-range offset
// and arrive as zeros.
//
// Waves are specialised.  A wave whose tile load cannot be queued stalls at that
// instruction and, issue being in order, its MFMAs wait behind it.  So 8 consumer
// waves (two per SIMD) only read fragments and issue MFMAs, and 4 producer waves (one
// per SIMD) only issue the tile loads and the row-index loads, and a blocked load
// never holds up the matrix pipe.  One barrier per k-tile joins them: producers
// arrive once tiles kt and kt+1 have landed, consumers once they are done reading
// tile kt-1.
// ---------------------------------------------------------------------------
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int BKS_, int STAGES_, int PRODUCERS_>
struct DwWsTile {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int BKS = BKS_, STAGES = STAGES_, PRODUCERS = PRODUCERS_;
    static constexpr int NWAVES = WAVES_M * WAVES_N;              // consumer waves
    static constexpr int NT = (NWAVES + PRODUCERS) * MTS_WAVE;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MF = WM / 32, NF = WN / 32;
    static constexpr int CPR_A = BM / 8, CPR_B = BN / 8;
    static constexpr int RPI_A = MTS_WAVE / CPR_A, RPI_B = MTS_WAVE / CPR_B;
    static constexpr int A_INSTR = BKS / RPI_A / PRODUCERS, B_INSTR = BKS / RPI_B / PRODUCERS;  // per producer wave
    static constexpr int STAGE = BKS * (BM + BN);
    static constexpr int LDS_ELEMS = STAGES * STAGE;
    static_assert(A_INSTR >= 1 && B_INSTR >= 1 && A_INSTR * RPI_A * PRODUCERS == BKS && B_INSTR * RPI_B * PRODUCERS == BKS,
                  "loader split");
    static_assert((STAGES == 4 || STAGES == 2) && (A_INSTR + B_INSTR) * 2 <= 63,
                  "the producer waits are written for a 4-stage ring and for two buffers");
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
};

// the work of block `block` of a launch; `smem` holds T::LDS_ELEMS elements, 1 KiB aligned
template <class T, typename OutT>
__device__ __forceinline__ void dw_gemm_ws_block(const DwParams& p, bf16_t* smem, int block) {
    constexpr int S = T::STAGES, L = T::A_INSTR + T::B_INSTR;
    // all tiles of a unit (an expert, or a row chunk of an over-full one) run on one XCD
    const int xcd = block % kXcds, jb = block / kXcds;
    DwUnit unit;
    if (p.sched) {
        const int k = jb / p.tiles_per_expert;
        if (k >= p.sched[kSchedCounts + xcd]) return;
        const int32_t* u = p.sched + kSchedUnits + (xcd * p.sched_slots + k) * 4;
        unit.e = u[0]; unit.rbeg = u[1]; unit.rend = u[2]; unit.slot = u[3];
    } else if (!locate_dw_unit(p, xcd + kXcds * (jb / p.tiles_per_expert), unit)) {
        return;
    }
    const int e = __builtin_amdgcn_readfirstlane(unit.e);
    const int rbeg = __builtin_amdgcn_readfirstlane(unit.rbeg), rend = __builtin_amdgcn_readfirstlane(unit.rend);
    const int slot = __builtin_amdgcn_readfirstlane(unit.slot);
    const int tile = jb % p.tiles_per_expert;
    const int m0 = (tile / p.n_tiles) * T::BM, n0 = (tile % p.n_tiles) * T::BN;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MTS_WAVE), lane = threadIdx.x % MTS_WAVE;
    const int nk = (rend - rbeg + T::BKS - 1) / T::BKS;

    if (wave >= T::NWAVES) {
        // ------------------------------ producer ------------------------------
        // The producer's own instruction count bounds the fill rate (a wave issues roughly one
        // instruction per 4-8 clocks), so everything that does not change from tile to tile is
        // computed once.  An operand that is read in place gets a descriptor that starts at the
        // tile's first row and ends at the expert's last row, rebuilt with scalar instructions
        // per tile: the per-lane offsets are constants and rows past the expert's end read as
        // zeros.  A gathered operand takes its row indices through the scalar cache, fetched
        // after the tile loads of the iteration were issued (a scalar load is counted by
        // lgkmcnt, so waiting for it does not wait for the tile loads issued before it; vmcnt
        // retires in order and a vector index load would drain the ring once per tile).
        const int pw = wave - T::NWAVES;
        const bool gath_p = p.p_gather != nullptr, gath_q = p.q_gather != nullptr;
        constexpr int ROWS_A = T::A_INSTR * T::RPI_A, ROWS_B = T::B_INSTR * T::RPI_B;
        static_assert(T::RPI_A == 2 && T::RPI_B == 2 && T::CPR_A == T::CPR_B, "two rows per wave instruction");
        static_assert(ROWS_A == ROWS_B && (ROWS_A == 8 || ROWS_A == 16), "index fetch layout: 8 or 16 rows per producer wave");
        const bool upper = lane >= T::CPR_A;
        const uint32_t ld_a = (uint32_t)p.M * 2u, ld_b = (uint32_t)p.N * 2u;   // row pitch in bytes
        uint32_t col_a[T::A_INSTR], col_b[T::B_INSTR], fix_a[T::A_INSTR], fix_b[T::B_INSTR];
        int rin_a[T::A_INSTR], rin_b[T::B_INSTR];
#pragma unroll
        for (int j = 0; j < T::A_INSTR; ++j) {
            const int tr = (pw * T::A_INSTR + j) * T::RPI_A + lane / T::CPR_A;
            const int c = m0 + (((lane % T::CPR_A) ^ ((tr & 3) << 2)) << 3);
            rin_a[j] = tr;
            col_a[j] = c < p.M ? (uint32_t)c * 2u : kInvalid;
            fix_a[j] = c < p.M ? (uint32_t)tr * ld_a + (uint32_t)c * 2u : kInvalid;
        }
#pragma unroll
        for (int j = 0; j < T::B_INSTR; ++j) {
            const int tr = (pw * T::B_INSTR + j) * T::RPI_B + lane / T::CPR_B;
            const int c = n0 + (((lane % T::CPR_B) ^ ((tr & 3) << 2)) << 3);
            rin_b[j] = tr;
            col_b[j] = c < p.N ? (uint32_t)c * 2u : kInvalid;
            fix_b[j] = c < p.N ? (uint32_t)tr * ld_b + (uint32_t)c * 2u : kInvalid;
        }
        const __amdgpu_buffer_rsrc_t rs_p = make_rsrc(p.P, p.p_rows * p.M * 2);
        const __amdgpu_buffer_rsrc_t rs_q = make_rsrc(p.Q, p.q_rows * p.N * 2);
        const u32x4 rs_gp = scalar_rsrc(p.p_gather, gath_p ? p.TK * 4 : 0);
        const u32x4 rs_gq = scalar_rsrc(p.q_gather, gath_q ? p.TK * 4 : 0);
        i32x4 idx_a[ROWS_A / 4] = {}, idx_b[ROWS_B / 4] = {};
        auto fetch_index = [&](int r0) {
#pragma unroll
            for (int h = 0; h < ROWS_A / 8; ++h) {
                if (gath_p) s_buffer_load8(rs_gp, (r0 + pw * ROWS_A + 8 * h) * 4, idx_a[2 * h], idx_a[2 * h + 1]);
                if (gath_q) s_buffer_load8(rs_gq, (r0 + pw * ROWS_B + 8 * h) * 4, idx_b[2 * h], idx_b[2 * h + 1]);
            }
        };
        auto issue = [&](int stage, int r0) {
            bf16_t* sa = smem + stage * T::STAGE + pw * T::A_INSTR * 512;
            bf16_t* sb = smem + stage * T::STAGE + T::BKS * T::BM + pw * T::B_INSTR * 512;
            const int left = rend - r0;   // rows of the expert from this tile on
            if (gath_p) {
#pragma unroll
                for (int j = 0; j < T::A_INSTR; ++j) {
                    const uint32_t lo = (uint32_t)idx_a[(2 * j) / 4][(2 * j) % 4] * ld_a;
                    const uint32_t hi = (uint32_t)idx_a[(2 * j + 1) / 4][(2 * j + 1) % 4] * ld_a;
                    const uint32_t off = rin_a[j] < left ? (upper ? hi : lo) + col_a[j] : kInvalid;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_p, MTS_LDS_PTR(sa + j * 512), 16, (int)off, 0, 0, 0);
                }
            } else {
                const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.P + (int64_t)r0 * p.M, (int64_t)left * p.M * 2);
#pragma unroll
                for (int j = 0; j < T::A_INSTR; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, MTS_LDS_PTR(sa + j * 512), 16, (int)fix_a[j], 0, 0, 0);
            }
            if (gath_q) {
#pragma unroll
                for (int j = 0; j < T::B_INSTR; ++j) {
                    const uint32_t lo = (uint32_t)idx_b[(2 * j) / 4][(2 * j) % 4] * ld_b;
                    const uint32_t hi = (uint32_t)idx_b[(2 * j + 1) / 4][(2 * j + 1) % 4] * ld_b;
                    const uint32_t off = rin_b[j] < left ? (upper ? hi : lo) + col_b[j] : kInvalid;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_q, MTS_LDS_PTR(sb + j * 512), 16, (int)off, 0, 0, 0);
                }
            } else {
                const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.Q + (int64_t)r0 * p.N, (int64_t)left * p.N * 2);
#pragma unroll
                for (int j = 0; j < T::B_INSTR; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, MTS_LDS_PTR(sb + j * 512), 16, (int)fix_b[j], 0, 0, 0);
            }
        };

        if constexpr (S == 2) {
            // Two buffers of wide tiles: barrier kt tells the consumers that tile kt has landed and
            // the producers that tile kt-1 is consumed, whose buffer then takes tile kt+1.
            fetch_index(rbeg);
            issue(0, rbeg);
            if (1 < nk) fetch_index(rbeg + T::BKS);
            for (int kt = 0; kt < nk; ++kt) {
                wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
                if (kt + 1 < nk) {
                    issue((kt + 1) & 1, rbeg + (kt + 1) * T::BKS);
                    if (kt + 2 < nk) fetch_index(rbeg + (kt + 2) * T::BKS);
                }
            }
            return;
        }
        // Barrier kt tells the consumers that tiles kt and kt+1 have landed (they read the first
        // fragments of tile kt+1 behind the last MFMAs of tile kt) and tells the producers that
        // every consumer is done with tile kt-1, whose stage then takes tile kt-1+S.
#pragma unroll
        for (int s = 0; s < S; ++s) {
            if (s < nk) {
                fetch_index(rbeg + s * T::BKS);
                issue(s, rbeg + s * T::BKS);
            }
        }
        if (S < nk) fetch_index(rbeg + S * T::BKS);
        int stage = S - 1;   // stage of tile kt-1
        for (int kt = 0; kt < nk; ++kt) {
            // tiles up to kt+1 must have landed; tile kt+2 (and, before barrier 0, tile 3) may be in flight
            if (kt == 0 && S >= 4 && nk >= 4) wait_vmcnt<L * (S >= 4 ? 2 : 0)>();
            else if (kt + 2 < nk) wait_vmcnt<L>();
            else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            if (kt >= 1 && kt - 1 + S < nk) {
                issue(stage, rbeg + (kt - 1 + S) * T::BKS);
                if (kt + S < nk) fetch_index(rbeg + (kt + S) * T::BKS);
            }
            stage = stage + 1 == S ? 0 : stage + 1;
        }
        __builtin_amdgcn_s_barrier();   // matches the consumers' barrier behind the last tile
        return;
    }

    // -------------------------------- consumer --------------------------------
    // Fragments run one k-step ahead of the MFMAs, across tile boundaries: Q fragments are
    // double buffered, a P fragment is reloaded right behind the MFMAs that used it.
    const int wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;
    f32x16 acc[T::MF][T::NF];
    zero_acc<T>(acc);
    constexpr int KSTEPS = T::BKS / 16;
    static_assert(KSTEPS % 2 == 0, "fragment buffers alternate with the k-step");
    bf16x8 fa[T::MF], fb[2][T::NF];
    auto step = [&](int ks, const bf16_t* next, int nks) {
        const bf16_t* nB = next + T::BKS * T::BM;
        const int buf = ks & 1;
#pragma unroll
        for (int nf = 0; nf < T::NF; ++nf) fb[buf ^ 1][nf] = read_frag_tr<T::BN>(nB, nks * 16, wn * T::WN + nf * 32);
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf) {
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
                acc[mf][nf] = MTS_MFMA_32x32x16(fa[mf], fb[buf][nf], acc[mf][nf], 0, 0, 0);
            fa[mf] = read_frag_tr<T::BM>(next, nks * 16, wm * T::WM + mf * 32);
        }
    };
    if constexpr (S == 2) {
        for (int kt = 0; kt < nk; ++kt) {
            __builtin_amdgcn_s_barrier();   // tile kt is visible, tile kt-1 may be overwritten
            const bf16_t* cur = smem + (kt & 1) * T::STAGE;
#pragma unroll
            for (int mf = 0; mf < T::MF; ++mf) fa[mf] = read_frag_tr<T::BM>(cur, 0, wm * T::WM + mf * 32);
#pragma unroll
            for (int nf = 0; nf < T::NF; ++nf)
                fb[0][nf] = read_frag_tr<T::BN>(cur + T::BKS * T::BM, 0, wn * T::WN + nf * 32);
#pragma unroll
            for (int ks = 0; ks < KSTEPS - 1; ++ks) step(ks, cur, ks + 1);
#pragma unroll
            for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
                for (int nf = 0; nf < T::NF; ++nf)
                    acc[mf][nf] = MTS_MFMA_32x32x16(fa[mf], fb[(KSTEPS - 1) & 1][nf], acc[mf][nf], 0, 0, 0);
        }
    } else {
    __builtin_amdgcn_s_barrier();   // tiles 0 and 1 are visible
#pragma unroll
    for (int mf = 0; mf < T::MF; ++mf) fa[mf] = read_frag_tr<T::BM>(smem, 0, wm * T::WM + mf * 32);
#pragma unroll
    for (int nf = 0; nf < T::NF; ++nf) fb[0][nf] = read_frag_tr<T::BN>(smem + T::BKS * T::BM, 0, wn * T::WN + nf * 32);
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt) {
        const bf16_t* cur = smem + stage * T::STAGE;
        stage = stage + 1 == S ? 0 : stage + 1;
#pragma unroll
        for (int ks = 0; ks < KSTEPS - 1; ++ks) step(ks, cur, ks + 1);
        // behind the last k-step the first fragments of tile kt+1 are read (after the last tile
        // this reads a stage nobody uses: harmless)
        step(KSTEPS - 1, smem + stage * T::STAGE, 0);
        __builtin_amdgcn_s_barrier();   // tile kt+2 is visible, tile kt may be overwritten
    }
    }

    const int fcol = lane % 32, frow4 = (lane / 32) * 4;
    if (slot >= 0) {   // a row chunk: the whole fp32 tile goes to the unit's slot of the workspace
        float* part = p.part + ((int64_t)slot * p.tiles_per_expert + tile) * (int64_t)(T::BM * T::BN);
#pragma unroll
        for (int mf = 0; mf < T::MF; ++mf)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int ml = wm * T::WM + mf * 32 + 8 * (i / 4) + frow4 + (i % 4);
#pragma unroll
                for (int nf = 0; nf < T::NF; ++nf)
                    part[ml * T::BN + wn * T::WN + nf * 32 + fcol] = acc[mf][nf][i];
            }
        return;
    }
    OutT* C = reinterpret_cast<OutT*>(p.C) + (int64_t)e * p.M * p.N;
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

template <class T, typename OutT>
__global__ __launch_bounds__(T::NT) void dw_gemm_ws_kernel(DwParams p) {
    __shared__ __attribute__((aligned(1024))) bf16_t smem[T::LDS_ELEMS];
    dw_gemm_ws_block<T, OutT>(p, smem, blockIdx.x);
}

// the compiled tile shapes
typedef Tile<128, 128, 2, 2> StagedSmall;                 // 4 waves of 64x64, any K that is a multiple of 8
typedef RingTile<256, 128, 2, 2, 32, 3, 2> RingTwoPerCu;  // 4 waves of 128x64, 3 x 24 KiB stages, two blocks per CU
// 4 waves of 96x64, 2 x 20 KiB stages, three blocks per CU (at most 168 registers per lane): while one block
// is in its epilogue two others are in their k-loops, and a block that waits for its one tile in flight
// has two neighbours to cover for it
typedef RingTile<192, 128, 2, 2, 32, 2, 3, 3> RingThreePerCu;   // three activation buffers + two weight buffers: 52 KiB a block
typedef WsTile<256, 256, 2, 4, 32, 4, 4, 3> WsLarge;      // 8 consumer waves of 128x64 + 4 producers, 4 x 32 KiB stages
typedef WsTile<256, 256, 4, 2, 64, 2, 4, 3> WsWideGu;     // gate/up: waves of 64x128, so that a wave stores 64 columns (whole lines) of g, u and a
typedef WsTile<256, 256, 2, 4, 64, 2, 4, 3> WsWide;
typedef WsTile<256, 256, 2, 4, 64, 3, 4, 3> WsDeep;        // three activation buffers and two weight buffers: the down projection, whose
typedef WsTile<128, 256, 2, 4, 64, 3, 4, 3> WsDeepHalf;    // activation rows the launch before it has written (-4 %; nothing for gate/up and dX)
typedef WsTile<128, 256, 2, 4, 64, 2, 4, 3> WsWideHalf;    // half-height tiles of the last round: the same waves take 64x64 each,
typedef WsTile<128, 256, 4, 2, 64, 2, 4, 3> WsWideGuHalf;  // and for gate/up 32x128 each       // the same waves on two buffers of 64-wide k-tiles (whole cache lines per row)
typedef DwWsTile<256, 256, 2, 4, 32, 4, 4> DwWsLarge;     // same shape for the weight-gradient GEMMs
typedef DwWsTile<256, 256, 2, 4, 64, 2, 4> DwWsWide;      // two buffers of 64 rows: half the barriers per row
typedef DwWsWide JointDwTile;                             // the weight-gradient tile of the joint backward launch

// ---------------------------------------------------------------------------
// dW1, dW2, dX and the reduction of the dS partials as one launch.  All four depend on dY1
// only.  As separate launches on separate streams they share the CUs in whatever order the
// hardware queues interleave them, and the long weight-gradient tiles (one tile reduces
// over all rows of an expert) tend to start last and finish last.  Here the block index
// fixes the order: the dW1 tiles first, then dW2, then the dX tiles, which are a third as
// long and fill the CUs as they come free, then a few blocks that add up dS.
// Every part starts at a multiple of the XCD count, so block % 8 is still the part's own
// XCD index.
// ---------------------------------------------------------------------------
constexpr int kJointRouterExperts = 8;   // the router blocks of the joint launch are compiled for up to 8 experts
struct BwdJointParams {
    DwParams dw1, dw2;
    RowsParams dx;
    int n_dw1, n_dw2, n_dx;        // blocks per part, in launch order
    const float* ds_part;          // [entries rows][np]
    const int32_t* s_reverse;      // entry -> row, negative for a dropped route
    bf16_t* d_weights;             // [entries]
    int np;
    int64_t entries;
    int n_ds;                      // blocks that reduce dS
    // The router's backward behind the dS blocks (n_router = 0: not part of this launch): the blocks of the
    // chained projection backward, which form the routing-weight gradient from ds_part themselves.  They
    // depend on nothing this launch writes and take the CUs that the last round of dX tiles leaves idle.
    int n_router, router_row_blocks;
    const bf16_t* rx;              // activations [T, H]
    const float* rw;               // router weight [E, H]
    int64_t rT;
    int rH, rE, r_rows_per_block, r_groups, r_cols_per_block, r_col_threads;
    bf16_t* r_dx;                  // the router's share of dx [T, H]
    float* r_part;                 // [router_row_blocks][E][H] partial dW_r
    float* r_dw;                   // dW_r [E][H]: summed from r_part by the launch that follows (host side only)
    bf16_t* c_out;                 // dx [T][H]: the dX combine in the launch that follows (host side only; NULL: not asked for)
    int c_K;
    mts_rl::RouterGradIn rg;
};

static_assert(WsWide::BM == kSchedDxRows, "the schedule counts dX tiles of this height");
typedef WsWide JointDxTile;   // dX reads d_pre_act row-major: whole lines per row with 64-wide k-tiles (a third buffer gains nothing here)
template <typename OutT>
__global__ __launch_bounds__(WsLarge::NT, WsLarge::WAVES_PER_EU) void bwd_joint_kernel(BwdJointParams q) {
    static_assert(WsLarge::NT == JointDwTile::NT && JointDxTile::NT == WsLarge::NT, "one block shape");
    constexpr int ROWS_LDS = ws_lds_elems<JointDxTile, EPI_PLAIN>();
    constexpr int LDS_ELEMS = ROWS_LDS > JointDwTile::LDS_ELEMS ? ROWS_LDS : JointDwTile::LDS_ELEMS;
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
    __shared__ __attribute__((aligned(1024))) bf16_t smem[LDS_ELEMS];
    int b = blockIdx.x;
    if (b < q.n_dw1) {
        dw_gemm_ws_block<JointDwTile, OutT>(q.dw1, smem, b);
        return;
    }
    b -= q.n_dw1;
    if (b < q.n_dw2) {
        dw_gemm_ws_block<JointDwTile, OutT>(q.dw2, smem, b);
        return;
    }
    b -= q.n_dw2;
    if (b < q.n_dx) {
        rows_gemm_ws_block<JointDxTile, EPI_PLAIN, true>(q.dx, smem, b);   // W1 as stored: [E][2I][H]
        return;
    }
    b -= q.n_dx;
    if (b < q.n_ds) {
        for (int64_t n = (int64_t)b * WsLarge::NT + threadIdx.x; n < q.entries; n += (int64_t)q.n_ds * WsLarge::NT) {
            const int32_t r = q.s_reverse[n];
            float v = 0.f;
            if (r >= 0) {
                const float* part = q.ds_part + (int64_t)r * q.np;
                for (int j = 0; j < q.np; ++j) v += part[j];
            }
            q.d_weights[n] = (bf16_t)v;
        }
        return;
    }
    b -= q.n_ds;
    if (b < q.n_router) {
        constexpr int EP = kJointRouterExperts;
        float* set_sum = reinterpret_cast<float*>(smem);                       // [E][cols_per_block]
        float* dl_lds = set_sum + q.rE * q.r_cols_per_block;                    // [kChainRows][EP]
        mts_rl::router_logits_bwd_block<bf16_t, EP, false, true>(
            nullptr, q.rx, q.rw, q.rT, q.rH, q.rE, q.r_rows_per_block, q.r_groups, q.r_cols_per_block, q.r_dx, q.r_part,
            q.rg, b % q.router_row_blocks, b / q.router_row_blocks, q.r_col_threads, set_sum, dl_lds);
    }
}

// ---------------------------------------------------------------------------
// gate/up and down as one launch.
//
// On their own the two forward GEMMs each end in a round that fills a fraction of the chip (6.1 and 2.3 tiles of
// 256 x 256 per CU at the 24576-token layer: an eighth and a seventh of their CU time idles).  In one launch the
// down tiles take the CUs as the gate/up tiles leave them, and only the end of the down part is ragged.
//
// A down tile reads the post_act rows of its m-tile, which the gate/up tiles of that m-tile (all column tiles)
// write in the same launch.  The m-tiles of both parts are dealt to the XCDs in the same contiguous ranges, so
// the writers and the readers of an m-tile run on the SAME XCD and meet in that XCD's L2:
//   * a consumer wave of a gate/up tile waits until its stores are acknowledged (s_waitcnt vmcnt(0): the
//     vector cache writes through, the acknowledgement comes from the L2) and then adds one to the m-tile's
//     counter with a relaxed device-scope atomic, which the L2 executes;
//   * the producer waves of a down tile poll the counter with loads that bypass the vector cache until it
//     holds (consumer waves x column tiles), invalidate the vector cache (acquire fence) and start loading.
// No L2 is written back for this: the release that device scope formally asks for (it writes the whole L2
// back, for readers on OTHER XCDs) would cost three times the GEMM.  The counter's upper bits carry the sum of
// the writers' XCC_ID; a reader that finds another XCD's id there than its own - a placement this code does
// not expect - raises the status word instead of trusting the data.
// Deadlock: blocks are placed in the order of their index, XCD by XCD; every gate/up block has a smaller index
// than every down block, so the tiles that a waiting down block needs are running or done, whatever else waits.
// The wait is bounded all the same: after spin_ticks of the 100 MHz wall clock a block gives up, raises the
// status word (which ends every other block's wait at once) and computes on what is there; the call's outputs
// are then invalid, and the status word says so.
// Counters: ready[t] as above, done[t] counts the down blocks of m-tile t; the last of them puts both back
// to zero, so a launch that ran through leaves the workspace as it found it (all zeros).
// ---------------------------------------------------------------------------
struct FwdJointParams {
    RowsParams gu, down;
    int n_gu;                  // blocks of the gate/up part (the down part's follow)
    int32_t* ready;            // [max m-tiles]
    int32_t* done;             // [max m-tiles]
    int32_t* status;           // one word, sticky: FWD_JOINT_TIMEOUT | FWD_JOINT_PLACEMENT
    int ready_count;           // consumer waves x column tiles of gate/up
    int64_t spin_ticks;
};
enum { FWD_JOINT_TIMEOUT = 1, FWD_JOINT_PLACEMENT = 2 };
constexpr int kReadyCountBits = 16;   // arrivals below, the sum of the writers' XCC_ID (at most 7 each) above
constexpr int kReadyCountMax = 4096;

__device__ __forceinline__ int xcc_id() { return (int)__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)); }   // HW_REG_XCC_ID[3:0]

__device__ __forceinline__ void wait_rows_ready(const FwdJointParams& q, const int32_t* ctr, int v);
// The wait of a down tile's producer waves.  The counter is read when the object is made (in front of the tile's address
// arithmetic and its first weight loads, which cover the load's latency); the call returns once the counter holds
// all arrivals (or the wait was given up).
struct RowsReadyWait {
    const FwdJointParams& q;
    const int32_t* ctr;
    int first;
    __device__ __forceinline__ RowsReadyWait(const FwdJointParams& q_, int mtile) : q(q_), ctr(q_.ready + mtile) {
        first = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ void operator()(int) const { wait_rows_ready(q, ctr, first); }
};
__device__ __forceinline__ void wait_rows_ready(const FwdJointParams& q, const int32_t* ctr, int v) {
    const int mask = (1 << kReadyCountBits) - 1;
    if ((v & mask) != q.ready_count) {
        const uint64_t t0 = wall_clock64();
        for (;;) {
            __builtin_amdgcn_s_sleep(16);
            v = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((v & mask) == q.ready_count) break;
            if (__hip_atomic_load(q.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;
            if ((int64_t)(wall_clock64() - t0) > q.spin_ticks) {
                __hip_atomic_fetch_or(q.status, FWD_JOINT_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return;
            }
        }
    }
    if ((int)((uint32_t)v >> kReadyCountBits) != q.ready_count * xcc_id())
        __hip_atomic_fetch_or(q.status, FWD_JOINT_PLACEMENT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // This CU's vector cache is invalidated (what an acquire costs between CUs that share an L2; also the compiler's
    // barrier for the loads that follow).  The acquire that device scope formally asks for walks the L2 as well,
    // 3.7 us per tile, for lines that only a writer on another XCD could have made stale.
    asm volatile("buffer_inv sc0" ::: "memory");
}

typedef WsWideGu FwdGuTile;
typedef WsDeep FwdDownTile;
typedef WsDeepHalf FwdDownHalf;
template <class GuTile>
__global__ __launch_bounds__(FwdGuTile::NT, FwdGuTile::WAVES_PER_EU) void fwd_joint_kernel(FwdJointParams q) {
    static_assert(FwdGuTile::NT == FwdDownTile::NT && FwdDownHalf::NT == FwdDownTile::NT, "one block shape");
    static_assert(FwdGuTile::BM == FwdDownTile::BM, "both parts count the same m-tiles");
    constexpr int GU_LDS = ws_lds_elems<FwdGuTile, EPI_SWIGLU>(), DOWN_LDS = ws_lds_elems<FwdDownTile, EPI_PLAIN>();
    constexpr int LDS_ELEMS = GU_LDS > DOWN_LDS ? GU_LDS : DOWN_LDS;
    static_assert(LDS_ELEMS * 2 <= 160 * 1024, "LDS capacity");
    __shared__ __attribute__((aligned(1024))) bf16_t smem[LDS_ELEMS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MTS_WAVE), lane = threadIdx.x % MTS_WAVE;
    int b = blockIdx.x;
    int e, row0, rend, ntile, parts, mtile;
    if (b < q.n_gu) {
        if (!locate_rows_tile<FwdGuTile::BM>(q.gu, b, e, row0, rend, ntile, parts, mtile)) return;   // whole tiles only
        rows_gemm_ws_run<FwdGuTile, EPI_SWIGLU, false, FwdGuTile>(q.gu, smem, e, row0, rend, ntile, 1);
        if (wave < FwdGuTile::NWAVES) {
            wait_vmcnt<0>();   // this wave's rows of pre_act and post_act are in the L2
            if (lane == 0)
                __hip_atomic_fetch_add(q.ready + mtile, 1 + (xcc_id() << kReadyCountBits), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    b -= q.n_gu;
    const bool found = locate_rows_tile<FwdDownTile::BM>(q.down, b, e, row0, rend, ntile, parts, mtile);
    if (mtile < 0) return;
    if (found)
        rows_gemm_ws_run<FwdDownTile, EPI_PLAIN, false, FwdDownHalf>(q.down, smem, e, row0, rend, ntile, parts, RowsReadyWait(q, mtile));
    // the last block of the m-tile (the empty half of a cut tile counts as one) clears its counters; all other readers
    // of ready[mtile] have had their answer by then: they add to done[] behind their loads
    if (wave == FwdDownTile::NWAVES && lane == 0) {
        const int blocks = q.down.n_tiles * parts;
        if (__hip_atomic_fetch_add(q.done + mtile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == blocks) {
            __hip_atomic_store(q.ready + mtile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(q.done + mtile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

typedef MtsGemmKind Kind;
constexpr Kind K_GATEUP = MTS_K_GATEUP, K_DOWN = MTS_K_DOWN, K_DY1 = MTS_K_DY1, K_DX = MTS_K_DX, K_DW2 = MTS_K_DW2, K_DW1 = MTS_K_DW1;
constexpr int K_COUNT = MTS_K_COUNT;
// rows_gemm: 0 StagedSmall, 1 RingTwoPerCu, 2 WsLarge, 3 RingThreePerCu (dY1 without the weighted_act output
// only), 4 WsWide (no SwiGLU backward: gate/up, down and dX; dY1 falls back to 2);
// dw_gemm: 0 StagedSmall, 2 DwWsLarge, 4 DwWsWide (the same output tiles, so one workspace layout).
// Defaults are the choices with the shortest LAYER STEP measured on the 24576-token, 768/1024, 8-expert layer.
// The chip runs this step against its power limit, so a kernel's own duration is not the whole story: what
// it leaves of the power budget shows in the kernels around it.  Gate/up on 256x256 tiles with specialised
// waves moves a third less data from L2 to LDS per FLOP than on two co-resident 256x128 ring blocks and makes
// the step 2-3.5 % shorter, although the kernel alone is at best as fast; dO*W2 with the SwiGLU backward in
// its epilogue is better off with three co-resident 4-wave blocks per CU.  The forward GEMMs take their
// k-tiles 64 wide (two buffers instead of four stages, the same time for a tile to land): a row then contributes
// a whole 128-byte line per load instruction, which the CU's vector cache serves at twice the rate of two
// half lines (gate/up -2.4 %, down -1 %); so does dX, inside the joint backward launch and on its own.
// The weight gradients read whole lines either way (a k-tile is rows of 256 columns); taking 64 rows per
// tile into two buffers halves their barriers (joint launch -1.7 %).
const int kDefaultTile[K_COUNT] = {4, 4, 3, 4, 4, 4};

// a tile family forced for a comparison run (mts_tuning.h), else the default
bool tile_forced(int kind) { return mts_tuning().tile[kind] >= 0; }
int tile_choice(int kind) { return tile_forced(kind) ? mts_tuning().tile[kind] : kDefaultTile[kind]; }

// `gathered_rows`: rows of the [T,H] operand that is read through the token gather (0: none).  Lane
// offsets are 32-bit: one expert's weights and an operand whose rows are gathered from anywhere must
// fit a single descriptor; the [TK, ...] operands are addressed tile by tile and may be larger.
int check_common(int64_t TK, int E, int H, int I, int64_t gathered_rows) {
    if (TK <= 0 || TK > 0x7fffffffLL || E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 8 || I < 8 || H % 8 ||
        I % 8)
        return MTS_ERR_SHAPE;
    if ((int64_t)2 * I * H * 2 > kMaxOperandBytes || gathered_rows * (int64_t)H * 2 > kMaxOperandBytes ||
        TK * 4 > kMaxOperandBytes)   // the index arrays are read through descriptors as well
        return MTS_ERR_SHAPE;
    return MTS_OK;
}

template <class T>
int64_t m_tiles(int64_t TK, int E) {
    int64_t a = (TK + T::BM - 1) / T::BM + E - 1;
    return a < TK ? a : TK;
}

// Contiguous ranges of m-tiles per XCD pay off while one expert's weight matrix stays resident in an
// XCD's 4 MiB L2 next to the streaming operands; larger weights are better streamed by all XCDs at the
// same time (round-robin deal: one fetch from HBM, the other seven from the Infinity Cache).
// A comparison run can force one or the other (mts_tuning.h).
constexpr int64_t kL2Bytes = 4 << 20;   // per XCD
int xcd_ranges_choice(int64_t expert_weight_bytes) {
    const int forced = mts_tuning().xcd_ranges;
    if (forced >= 0) return forced;
    return expert_weight_bytes <= kL2Bytes ? 1 : 0;
}

// the n-tile groups and the reversed walks of the range mapping, which a comparison run can switch off one by one
enum { ORDER_GROUPS = 1, ORDER_DOWN = 2, ORDER_DY1 = 4, ORDER_DX = 8, ORDER_ALL = 15 };
int tile_order_mask() { return mts_tuning().tile_order_mask; }

constexpr int kCusPerXcd = 32;
bool tail_split_on() { return mts_tuning().tail_split; }

template <class T, int EPI>
dim3 rows_grid(RowsParams& p, int64_t TK) {
    const int per_block = (EPI == EPI_SWIGLU) ? T::BN / 2 : T::BN;
    p.n_tiles = (p.N + per_block - 1) / per_block;
    const int64_t weight_bytes = (int64_t)p.b_rows * p.Kdim * (int64_t)sizeof(bf16_t);
    p.xcd_ranges = xcd_ranges_choice(weight_bytes);
    p.n_groups = 1;
    if (p.xcd_ranges && (tile_order_mask() & ORDER_GROUPS))
        while (weight_bytes / p.n_groups > kL2Bytes / 2 && p.n_tiles % (2 * p.n_groups) == 0 && p.n_tiles / (2 * p.n_groups) >= 4)
            p.n_groups *= 2;
    const int64_t m_groups = (m_tiles<T>(TK, p.E) + kXcds - 1) / kXcds;
    if (!p.xcd_ranges) p.tail_slots = 0;
    // tiles that are cut in two add at most tail_slots / 2 blocks per XCD; one more block writes the schedule (dO*W2 only)
    return dim3((unsigned)((m_groups * p.n_tiles + p.tail_slots / 2 + p.tail_tiles) * kXcds + (p.sched_out ? 1 : 0)));
}

// does launch_rows_any take B in the weights' stored layout for this kind and reduction length?
bool rows_kmajor_ok(int kind, int Kdim) { return tile_choice(kind) >= 1 && Kdim % 64 == 0; }

// b_kmajor: B is [E][Kdim][N] (the weights as stored) instead of the transposed copy [E][N][Kdim];
// only the ring and specialised kernels read it that way
template <int EPI>
int launch_rows_any(int kind, RowsParams p, int64_t TK, hipStream_t s, bool b_kmajor = false) {
    p.reverse = ((kind == K_DOWN && (tile_order_mask() & ORDER_DOWN)) || (kind == K_DY1 && (tile_order_mask() & ORDER_DY1)) ||
                 (kind == K_DX && (tile_order_mask() & ORDER_DX))) ? 1 : 0;
    int choice = tile_choice(kind);
    // three blocks per CU hold two stages each: for short reductions, and for the epilogue that fits beside them
    if (choice == 3 && (EPI != EPI_DY1N || !b_kmajor || (!tile_forced(kind) && p.Kdim > 1024))) choice = 1;
    // the 64-wide variant exists for the GEMMs with a plain or SwiGLU epilogue
    if (choice == 4 && epi_is_dy1(EPI)) choice = 2;
    // the ring kernels need whole k-tiles; other shapes use the staged kernel
    if (choice >= 1 && p.Kdim % 64 != 0) choice = 0;
    if (b_kmajor && (choice == 0 || EPI == EPI_SWIGLU)) return MTS_ERR_SHAPE;
    if (choice == 3) {
        if constexpr (EPI == EPI_DY1N) {
            const dim3 grid = rows_grid<RingThreePerCu, EPI>(p, TK);
            rows_gemm_ring_kernel<RingThreePerCu, EPI, true><<<grid, RingThreePerCu::NT, 0, s>>>(p);
        }
    } else if (choice == 1) {
        const dim3 grid = rows_grid<RingTwoPerCu, EPI>(p, TK);
        if constexpr (EPI != EPI_SWIGLU) {
            if (b_kmajor) rows_gemm_ring_kernel<RingTwoPerCu, EPI, true><<<grid, RingTwoPerCu::NT, 0, s>>>(p);
            else rows_gemm_ring_kernel<RingTwoPerCu, EPI><<<grid, RingTwoPerCu::NT, 0, s>>>(p);
        } else {
            rows_gemm_ring_kernel<RingTwoPerCu, EPI><<<grid, RingTwoPerCu::NT, 0, s>>>(p);
        }
    } else if (choice == 4) {
        if constexpr (!epi_is_dy1(EPI)) {
            // The tiles are few and long: 6.25 (gate/up) and 2.34 (down) per CU at the 24576-token layer.  The ones
            // behind the last whole round of an XCD's 32 CUs are cut in two where they would leave more than half
            // of the CUs idle (gate/up -3 %, down -4 %).
            if (!b_kmajor && tail_split_on()) p.tail_slots = kCusPerXcd;
            const dim3 grid = rows_grid<WsWide, EPI>(p, TK);
            if constexpr (EPI != EPI_SWIGLU) {
                if (b_kmajor) rows_gemm_ws_kernel<WsWide, EPI, true><<<grid, WsWide::NT, 0, s>>>(p);
                else rows_gemm_ws_kernel<WsDeep, EPI, false, WsDeepHalf><<<grid, WsWide::NT, 0, s>>>(p);
            } else {
                // same tile, waves of 64x128: a wave's 32-row slab of g, u and a is 64 columns wide, i.e. whole 128-byte
                // lines per row and store (with 128x64 waves it is 32 columns: gate/up +2.5 %)
                static_assert(WsWideGu::BM == WsWide::BM && WsWideGu::BN == WsWide::BN && WsWideGu::NT == WsWide::NT, "same grid");
                rows_gemm_ws_kernel<WsWideGu, EPI, false, WsWideGuHalf><<<grid, WsWideGu::NT, 0, s>>>(p);
            }
        }
    } else if (choice == 2) {
        const dim3 grid = rows_grid<WsLarge, EPI>(p, TK);
        if constexpr (EPI != EPI_SWIGLU) {
            if (b_kmajor) rows_gemm_ws_kernel<WsLarge, EPI, true><<<grid, WsLarge::NT, 0, s>>>(p);
            else rows_gemm_ws_kernel<WsLarge, EPI><<<grid, WsLarge::NT, 0, s>>>(p);
        } else {
            rows_gemm_ws_kernel<WsLarge, EPI><<<grid, WsLarge::NT, 0, s>>>(p);
        }
    } else {
        const dim3 grid = rows_grid<StagedSmall, EPI>(p, TK);
        rows_gemm_kernel<StagedSmall, EPI><<<grid, StagedSmall::NT, 0, s>>>(p);
    }
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

template <class T>
dim3 dw_grid(DwParams& p, int E, int units) {
    p.E = E;
    p.n_tiles = (p.N + T::BN - 1) / T::BN;
    p.tiles_per_expert = ((p.M + T::BM - 1) / T::BM) * p.n_tiles;
    return dim3((unsigned)(((units + kXcds - 1) / kXcds) * kXcds * p.tiles_per_expert));
}

// fp32 tile partials of up to 2E row-chunk units (see DwUnit)
int64_t dw_chunk_workspace_bytes(int E, int M, int N) {
    typedef DwWsLarge T;
    const int64_t tiles = (int64_t)((M + T::BM - 1) / T::BM) * ((N + T::BN - 1) / T::BN);
    return 2 * (int64_t)E * tiles * T::BM * T::BN * (int64_t)sizeof(float);
}

// adds the row-chunk partials of the experts that dw_gemm_ws cut (p.part set, grid values filled in)
void launch_dw_chunk_sum(const DwParams& p, int E, int grad_dtype, hipStream_t s) {
    typedef DwWsLarge T;
    const int64_t items = (int64_t)p.tiles_per_expert * (T::BM * T::BN / 4);
    const int64_t want = (items + 255) / 256;   // experts that were not cut leave at once
    const dim3 sum_grid((unsigned)(want < 256 ? want : 256), (unsigned)E);
    if (grad_dtype == MTS_GEMM_DTYPE) dw_chunk_sum_kernel<T::BM, T::BN, bf16_t><<<sum_grid, 256, 0, s>>>(p);
    else dw_chunk_sum_kernel<T::BM, T::BN, float><<<sum_grid, 256, 0, s>>>(p);
}

int launch_dw_any(int kind, DwParams p, int E, int grad_dtype, void* workspace, int64_t workspace_bytes,
                  hipStream_t s) {
    if (grad_dtype != MTS_GEMM_DTYPE && grad_dtype != MTS_F32) return MTS_ERR_DTYPE;
    const int choice = tile_choice(kind);
    if (choice == 2 || choice == 4) {
        typedef DwWsLarge T;   // DwWsWide has the same output tile, grid and block
        static_assert(DwWsWide::BM == T::BM && DwWsWide::BN == T::BN && DwWsWide::NT == T::NT, "one grid for both");
        if (workspace) {
            if (workspace_bytes < dw_chunk_workspace_bytes(E, p.M, p.N)) return MTS_ERR_WORKSPACE;
            if (!mts_aligned16(workspace)) return MTS_ERR_ALIGN;
            p.part = (float*)workspace;
        }
        const dim3 grid = dw_grid<T>(p, E, p.part ? 2 * E : E);
        if (choice == 4) {
            if (grad_dtype == MTS_GEMM_DTYPE) dw_gemm_ws_kernel<DwWsWide, bf16_t><<<grid, T::NT, 0, s>>>(p);
            else dw_gemm_ws_kernel<DwWsWide, float><<<grid, T::NT, 0, s>>>(p);
        } else {
            if (grad_dtype == MTS_GEMM_DTYPE) dw_gemm_ws_kernel<T, bf16_t><<<grid, T::NT, 0, s>>>(p);
            else dw_gemm_ws_kernel<T, float><<<grid, T::NT, 0, s>>>(p);
        }
        if (p.part) {
            MTS_CHECK_LAUNCH();
            launch_dw_chunk_sum(p, E, grad_dtype, s);
        }
    } else {
        const dim3 grid = dw_grid<StagedSmall>(p, E, E);
        if (grad_dtype == MTS_GEMM_DTYPE) dw_gemm_kernel<StagedSmall, bf16_t><<<grid, StagedSmall::NT, 0, s>>>(p);
        else dw_gemm_kernel<StagedSmall, float><<<grid, StagedSmall::NT, 0, s>>>(p);
    }
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

// gate/up + down as one launch: both on the 256 x 256 tiles with specialised waves, both dealt to the XCDs in
// contiguous ranges of the same m-tiles (an expert's W1 fits an L2)
bool fwd_joint_ok(int H, int I) {
    const int n_tiles_gu = (I + FwdGuTile::BN / 2 - 1) / (FwdGuTile::BN / 2);
    return tile_choice(K_GATEUP) == 4 && tile_choice(K_DOWN) == 4 && H % 64 == 0 && I % 64 == 0 &&
           xcd_ranges_choice((int64_t)2 * I * H * (int64_t)sizeof(bf16_t)) == 1 &&
           xcd_ranges_choice((int64_t)I * H * (int64_t)sizeof(bf16_t)) == 1 && FwdGuTile::NWAVES * n_tiles_gu <= kReadyCountMax;
}
int64_t fwd_joint_counters(int64_t TK, int E) { return m_tiles<FwdGuTile>(TK, E); }

int launch_fwd_joint(RowsParams gu, RowsParams down, int64_t TK, int32_t* workspace, hipStream_t s) {
    FwdJointParams q = {};
    gu.reverse = down.reverse = 0;   // the down part follows the gate/up part through the range, oldest rows first
    gu.tail_slots = down.tail_slots = 0;
    q.n_gu = (int)rows_grid<FwdGuTile, EPI_SWIGLU>(gu, TK).x;
    // Only the end of the down part is ragged: its last m-tiles (per XCD) are cut into tiles of half the height, as many
    // as make about 3/8 of a round of whole tiles (measured at 768/1024: 2, 4 and 6 m-tiles of 3 tiles each give 276, 272
    // and 281 us; none 277).
    down.n_tiles = (down.N + FwdDownTile::BN - 1) / FwdDownTile::BN;
    const int forced = mts_tuning().fwd_joint_tail;
    const int by_rule = (kCusPerXcd * 3 / 8 + down.n_tiles / 2) / down.n_tiles;
    const int tail_mtiles = forced >= 0 ? forced : (by_rule > 1 ? by_rule : 1);
    down.tail_tiles = tail_mtiles * down.n_tiles;
    const int n_down = (int)rows_grid<FwdDownTile, EPI_PLAIN>(down, TK).x;
    if (!gu.xcd_ranges || !down.xcd_ranges || down.n_groups != 1) return MTS_ERR_SHAPE;
    q.gu = gu;
    q.down = down;
    const int64_t n = fwd_joint_counters(TK, gu.E);
    q.status = workspace;           // word 0; the counters start 16 bytes in
    q.ready = workspace + 4;
    q.done = q.ready + n;
    q.ready_count = FwdGuTile::NWAVES * gu.n_tiles;
    q.spin_ticks = mts_tuning().fwd_joint_spin_us * 100;   // the wall clock counts at 100 MHz
    fwd_joint_kernel<FwdGuTile><<<dim3((unsigned)(q.n_gu + n_down)), FwdGuTile::NT, 0, s>>>(q);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

int dy1_partials(int I) { return (I + 63) / 64; }

// can dW1, dW2, dX and the dS reduction go out as one launch for these shapes?
bool bwd_joint_ok(int H, int I) {
    return tile_choice(K_DX) >= 2 && tile_choice(K_DW1) == 4 && tile_choice(K_DW2) == 4 && rows_kmajor_ok(K_DX, 2 * I) &&
           H % 8 == 0;
}

// the dX combine rides in the launch of the partial sums when the layer has two routes per token (the block
// function is compiled for that) and whole 16-byte chunks per row
bool combine_in_tail(const BwdJointParams& q) { return q.c_out && q.n_router && q.c_K == 2 && q.rH % 8 == 0; }

// Table entries per XCD and the most dX m-tiles one XCD is given: the dO*W2 launch that writes the table and the joint
// launch that sizes its grid by it must agree.  One and a half even shares: the routing of a trained router asks for up
// to 1.3; every block beyond an XCD's tiles costs the launch a microsecond of one CU in front of the router's blocks
// (twice the even share: 640 such blocks at the 24576-token layer, 2.7 us of the whole chip).
void schedule_shape(int64_t TK, int E, int& slots, int& cap) {
    slots = (2 * E + kXcds - 1) / kXcds;
    const int64_t upper = m_tiles<WsWide>(TK, E);
    const int64_t even = (upper + kXcds - 1) / kXcds;
    const int64_t most = even + (even / 2 > 2 ? even / 2 : 2);
    cap = (int)(most < upper ? most : upper);
}

int launch_bwd_joint(BwdJointParams q, int E, int grad_dtype, void* ws1, int64_t ws1_bytes, void* ws2, int64_t ws2_bytes,
                     const int32_t* schedule, hipStream_t s) {
    typedef DwWsLarge T;
    if (grad_dtype != MTS_GEMM_DTYPE && grad_dtype != MTS_F32) return MTS_ERR_DTYPE;
    if (ws1) {
        if (ws1_bytes < dw_chunk_workspace_bytes(E, q.dw1.M, q.dw1.N)) return MTS_ERR_WORKSPACE;
        if (!mts_aligned16(ws1)) return MTS_ERR_ALIGN;
        q.dw1.part = (float*)ws1;
    }
    if (ws2) {
        if (ws2_bytes < dw_chunk_workspace_bytes(E, q.dw2.M, q.dw2.N)) return MTS_ERR_WORKSPACE;
        if (!mts_aligned16(ws2)) return MTS_ERR_ALIGN;
        q.dw2.part = (float*)ws2;
    }
    q.n_dw1 = (int)dw_grid<T>(q.dw1, E, q.dw1.part ? 2 * E : E).x;
    q.n_dw2 = (int)dw_grid<T>(q.dw2, E, q.dw2.part ? 2 * E : E).x;
    const bool own_dw2 = q.dw2.C != nullptr;
    if (!own_dw2) {
        q.n_dw2 = 0;
        q.dw2.E = 0;
        q.dw2.part = nullptr;
    }
    q.dx.reverse = (tile_order_mask() & ORDER_DX) ? 1 : 0;
    q.n_dx = (int)rows_grid<JointDxTile, EPI_PLAIN>(q.dx, q.dx.TK).x;
    // With both workspaces (row chunks on) and a schedule from the caller (written by the dO*W2 launch), units and dX
    // tiles go to the XCDs as the table says.
    if (schedule && own_dw2 && q.dw1.part && q.dw2.part && E <= kSchedMaxExperts && mts_tuning().joint_schedule) {
        if (!mts_aligned16(schedule)) return MTS_ERR_ALIGN;
        int slots, cap;
        schedule_shape(q.dx.TK, E, slots, cap);
        q.dw1.sched = q.dw2.sched = schedule;
        q.dw1.sched_slots = q.dw2.sched_slots = slots;
        if (q.dx.xcd_ranges) {
            q.dx.sched = schedule;
            q.dx.n_groups = 1;
            q.n_dx = cap * q.dx.n_tiles * kXcds;
        }
    }
    const int64_t want = (q.entries + WsLarge::NT * 4 - 1) / (WsLarge::NT * 4);
    q.n_ds = (int)(want < 64 ? want : 64);
    const dim3 grid((unsigned)(q.n_dw1 + q.n_dw2 + q.n_dx + q.n_ds + q.n_router));
    if (grad_dtype == MTS_GEMM_DTYPE) bwd_joint_kernel<bf16_t><<<grid, WsLarge::NT, 0, s>>>(q);
    else bwd_joint_kernel<float><<<grid, WsLarge::NT, 0, s>>>(q);
    MTS_CHECK_LAUNCH();
    if (q.dw1.part && (q.dw2.part || !own_dw2) && 2 * E <= 65535) {
        const int t = q.dw1.tiles_per_expert > q.dw2.tiles_per_expert ? q.dw1.tiles_per_expert : q.dw2.tiles_per_expert;
        const int64_t want = ((int64_t)t * (T::BM * T::BN / 4) + 255) / 256;
        const unsigned gx = (unsigned)(want < 256 ? want : 256);
        // the sum of the router's dW_r partials and the dX combine ride along as extra rows of blocks
        TailJobs jobs = {};
        if (q.n_router) {
            jobs.r_part = q.r_part; jobs.r_blocks = q.router_row_blocks; jobs.r_EH = (int64_t)q.rE * q.rH; jobs.r_dw = q.r_dw;
            jobs.r_rows = (int)(((jobs.r_EH + mts_rl::kReduceCols - 1) / mts_rl::kReduceCols + gx - 1) / gx);
        }
        const bool combined = combine_in_tail(q);
        if (combined) {
            jobs.c_y = q.dx.C; jobs.c_addend = q.r_dx; jobs.c_srev = q.s_reverse; jobs.c_T = q.rT; jobs.c_H = q.rH;
            jobs.c_out = q.c_out;
            const int64_t items = ((q.rT + 1) / 2) * (int64_t)(q.rH / 8);   // 16 bytes of output for two tokens each
            const int64_t rows = ((items + 255) / 256 + gx - 1) / gx;
            jobs.c_rows = (int)(rows < 32 ? rows : 32);
        }
        const dim3 sum_grid(gx, (unsigned)(q.dw1.E + q.dw2.E + jobs.r_rows + jobs.c_rows));
        if (grad_dtype == MTS_GEMM_DTYPE) dw_chunk_sum_pair_kernel<T::BM, T::BN, bf16_t><<<sum_grid, 256, 0, s>>>(q.dw1, q.dw2, jobs);
        else dw_chunk_sum_pair_kernel<T::BM, T::BN, float><<<sum_grid, 256, 0, s>>>(q.dw1, q.dw2, jobs);
        MTS_CHECK_LAUNCH();
        if (combined) return MTS_OK;
    } else {   // one of the two, or more experts than a grid holds in y twice over
        if (q.dw1.part) launch_dw_chunk_sum(q.dw1, E, grad_dtype, s);
        if (q.dw2.part) launch_dw_chunk_sum(q.dw2, E, grad_dtype, s);
        MTS_CHECK_LAUNCH();
        if (q.n_router) {
            const int rc = mts_launch_router_dw_reduce(q.r_part, q.router_row_blocks, (int64_t)q.rE * q.rH, q.r_dw, s);
            if (rc) return rc;
        }
    }
    // the dX combine, where it was asked for and did not ride in the launch above
    if (q.c_out)
        return mts_moe_combine(q.dx.C, nullptr, q.r_dx, q.s_reverse, q.rT, q.c_K, q.rH, MTS_GEMM_DTYPE, q.c_out, (void*)s);
    return MTS_OK;
}

}  // namespace

#ifndef MTS_GEMM_F16
extern "C" int mts_moe_ds_partials(int I) { return dy1_partials(I); }
#endif

extern "C" int MTS_GEMM_ENTRY(mts_moe_fwd_gateup_swiglu)(const void* x, const void* w1, const int32_t* x_gather,
                                         const int32_t* expert_start, const void* weights,
                                         const int32_t* s_scatter, int64_t T, int K, int E,
                                         int H, int I, int act_dtype, void* pre_act,
                                         void* post_act, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_fwd_gateup_swiglu_f16(x, w1, x_gather, expert_start, weights, s_scatter, T, K, E, H, I, act_dtype, pre_act, post_act, stream);
#endif
    if (!x || !w1 || !x_gather || !expert_start || !pre_act || !post_act) return MTS_ERR_NULL;
    if ((weights != nullptr) != (s_scatter != nullptr)) return MTS_ERR_NULL;   // the routing weight needs the row -> entry map
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    if (act_dtype == MTS_F32) {
        if (E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1 || T * K > 0x7fffffffLL) return MTS_ERR_SHAPE;
        return mts_f32_rows(1, (const float*)x, H, x_gather, (const float*)w1, 2 * I, I, H, expert_start, E, T * K,
                            (float*)pre_act, (float*)post_act, nullptr, (const float*)weights, s_scatter, nullptr, 0,
                            (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(T * K, E, H, I, T);
    if (rc) return rc;
    if (!mts_aligned16(x) || !mts_aligned16(w1) || !mts_aligned16(pre_act) || !mts_aligned16(post_act)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)x; p.a_rows = T; p.lda = H; p.a_gather = x_gather;
    p.B = (const bf16_t*)w1; p.b_rows = 2 * I;
    p.N = I; p.Kdim = H; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)pre_act; p.C2 = (bf16_t*)post_act; p.TK = T * K;
    p.route_w = (const bf16_t*)weights; p.s_scatter = s_scatter;
    return launch_rows_any<EPI_SWIGLU>(K_GATEUP, p, T * K, (hipStream_t)stream);
}

extern "C" int MTS_GEMM_ENTRY(mts_moe_fwd_down)(const void* post_act, const void* w2, const int32_t* expert_start,
                                int64_t TK, int E, int H, int I, int act_dtype, void* y,
                                void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_fwd_down_f16(post_act, w2, expert_start, TK, E, H, I, act_dtype, y, stream);
#endif
    if (!post_act || !w2 || !expert_start || !y) return MTS_ERR_NULL;
    if (act_dtype == MTS_F32) {
        if (TK <= 0 || TK > 0x7fffffffLL || E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1) return MTS_ERR_SHAPE;
        return mts_f32_rows(0, (const float*)post_act, I, nullptr, (const float*)w2, H, H, I, expert_start, E, TK,
                            (float*)y, nullptr, nullptr, nullptr, nullptr, nullptr, 0, (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(TK, E, H, I, 0);
    if (rc) return rc;
    if (!mts_aligned16(post_act) || !mts_aligned16(w2) || !mts_aligned16(y)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)post_act; p.a_rows = TK; p.lda = I; p.a_gather = nullptr;
    p.B = (const bf16_t*)w2; p.b_rows = H;
    p.N = H; p.Kdim = I; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)y; p.TK = TK;
    return launch_rows_any<EPI_PLAIN>(K_DOWN, p, TK, (hipStream_t)stream);
}

#ifndef MTS_GEMM_F16
extern "C" int mts_moe_fwd_joint_supported(int act_dtype, int H, int I) {
    return (act_dtype == MTS_BF16 || act_dtype == MTS_F16) && H >= 64 && I >= 64 && fwd_joint_ok(H, I) ? 1 : 0;
}
extern "C" int64_t mts_moe_fwd_joint_workspace_bytes(int64_t TK, int E) {
    if (TK <= 0 || E < 1) return 0;
    return ((2 * fwd_joint_counters(TK, E) + 4) * (int64_t)sizeof(int32_t) + 15) / 16 * 16;
}
#endif

extern "C" int MTS_GEMM_ENTRY(mts_moe_fwd_gateup_down)(const void* x, const void* w1, const void* w2, const int32_t* x_gather,
                                       const int32_t* expert_start, const void* weights, const int32_t* s_scatter,
                                       int64_t T, int K, int E, int H, int I, int act_dtype, void* pre_act, void* post_act,
                                       void* y, int32_t* workspace, int64_t workspace_bytes, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_fwd_gateup_down_f16(x, w1, w2, x_gather, expert_start, weights, s_scatter, T, K, E, H, I, act_dtype, pre_act, post_act, y, workspace, workspace_bytes, stream);
#endif
    if (!x || !w1 || !w2 || !x_gather || !expert_start || !pre_act || !post_act || !y || !workspace) return MTS_ERR_NULL;
    if ((weights != nullptr) != (s_scatter != nullptr)) return MTS_ERR_NULL;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(T * K, E, H, I, T);
    if (rc) return rc;
    if (!fwd_joint_ok(H, I)) return MTS_ERR_SHAPE;
    if (!mts_aligned16(x) || !mts_aligned16(w1) || !mts_aligned16(w2) || !mts_aligned16(pre_act) || !mts_aligned16(post_act) ||
        !mts_aligned16(y) || !mts_aligned16(workspace))
        return MTS_ERR_ALIGN;
    if (workspace_bytes < (2 * fwd_joint_counters(T * K, E) + 4) * (int64_t)sizeof(int32_t)) return MTS_ERR_WORKSPACE;
    RowsParams g = {};
    g.A = (const bf16_t*)x; g.a_rows = T; g.lda = H; g.a_gather = x_gather;
    g.B = (const bf16_t*)w1; g.b_rows = 2 * I;
    g.N = I; g.Kdim = H; g.expert_start = expert_start; g.E = E;
    g.C = (bf16_t*)pre_act; g.C2 = (bf16_t*)post_act; g.TK = T * K;
    g.route_w = (const bf16_t*)weights; g.s_scatter = s_scatter;
    RowsParams d = {};
    d.A = (const bf16_t*)post_act; d.a_rows = T * K; d.lda = I; d.a_gather = nullptr;
    d.B = (const bf16_t*)w2; d.b_rows = H;
    d.N = H; d.Kdim = I; d.expert_start = expert_start; d.E = E;
    d.C = (bf16_t*)y; d.TK = T * K;
    return launch_fwd_joint(g, d, T * K, workspace, (hipStream_t)stream);
}

#ifndef MTS_GEMM_F16
extern "C" int mts_moe_bwd_weights_as_stored(int act_dtype, int H, int I) {
    return (act_dtype == MTS_BF16 || act_dtype == MTS_F16) && rows_kmajor_ok(K_DY1, H) && rows_kmajor_ok(K_DX, 2 * I) ? 1 : 0;
}
#endif

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_dy1)(const void* d_out, const void* w2t, int w2_as_stored, const void* pre_act,
                               const void* weights, const int32_t* x_gather,
                               const int32_t* s_scatter, const int32_t* expert_start, int64_t T,
                               int K, int E, int H, int I, int act_dtype, void* d_pre_act,
                               void* weighted_act, float* ds_partial, int32_t* schedule, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_bwd_dy1_f16(d_out, w2t, w2_as_stored, pre_act, weights, x_gather, s_scatter, expert_start, T, K, E, H, I, act_dtype, d_pre_act, weighted_act, ds_partial, schedule, stream);
#endif
    if (!d_out || !w2t || !pre_act || !weights || !x_gather || !s_scatter || !expert_start ||
        !d_pre_act || !ds_partial)
        return MTS_ERR_NULL;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    if (schedule && (E > kSchedMaxExperts || act_dtype == MTS_F32)) return MTS_ERR_SHAPE;   // see mts_moe_bwd_schedule_bytes
    if (act_dtype == MTS_F32) {
        if (E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1 || T * K > 0x7fffffffLL || w2_as_stored) return MTS_ERR_SHAPE;
        return mts_f32_rows(2, (const float*)d_out, H, x_gather, (const float*)w2t, I, I, H, expert_start, E, T * K,
                            (float*)d_pre_act, (float*)weighted_act, (const float*)pre_act, (const float*)weights,
                            s_scatter, ds_partial, mts_moe_ds_partials(I), (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(T * K, E, H, I, T);
    if (rc) return rc;
    if (!mts_aligned16(d_out) || !mts_aligned16(w2t) || !mts_aligned16(pre_act) || !mts_aligned16(d_pre_act) ||
        !mts_aligned16(weighted_act))
        return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)d_out; p.a_rows = T; p.lda = H; p.a_gather = x_gather;
    p.B = (const bf16_t*)w2t; p.b_rows = I;
    p.N = I; p.Kdim = H; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)d_pre_act; p.C2 = (bf16_t*)weighted_act;
    p.pre_act = (const bf16_t*)pre_act; p.route_w = (const bf16_t*)weights;
    p.s_scatter = s_scatter; p.ds_part = ds_partial; p.np = mts_moe_ds_partials(I); p.TK = T * K;
    if (schedule) {
        if (!mts_aligned16(schedule)) return MTS_ERR_ALIGN;
        p.sched_out = schedule;
        schedule_shape(T * K, E, p.sched_slots, p.sched_dx_cap);
    }
    if (!weighted_act) return launch_rows_any<EPI_DY1N>(K_DY1, p, T * K, (hipStream_t)stream, w2_as_stored != 0);
    return launch_rows_any<EPI_DY1>(K_DY1, p, T * K, (hipStream_t)stream, w2_as_stored != 0);
}

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_dx)(const void* d_pre_act, const void* w1t, int w1_as_stored,
                              const int32_t* expert_start, int64_t TK, int E, int H, int I, int act_dtype,
                              void* dx_expanded, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_bwd_dx_f16(d_pre_act, w1t, w1_as_stored, expert_start, TK, E, H, I, act_dtype, dx_expanded, stream);
#endif
    if (!d_pre_act || !w1t || !expert_start || !dx_expanded) return MTS_ERR_NULL;
    if (act_dtype == MTS_F32) {
        if (TK <= 0 || TK > 0x7fffffffLL || E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1 || w1_as_stored) return MTS_ERR_SHAPE;
        return mts_f32_rows(0, (const float*)d_pre_act, 2 * I, nullptr, (const float*)w1t, H, H, 2 * I, expert_start, E,
                            TK, (float*)dx_expanded, nullptr, nullptr, nullptr, nullptr, nullptr, 0,
                            (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(TK, E, H, I, 0);
    if (rc) return rc;
    if (!mts_aligned16(d_pre_act) || !mts_aligned16(w1t) || !mts_aligned16(dx_expanded)) return MTS_ERR_ALIGN;
    RowsParams p = {};
    p.A = (const bf16_t*)d_pre_act; p.a_rows = TK; p.lda = 2 * I; p.a_gather = nullptr;
    p.B = (const bf16_t*)w1t; p.b_rows = H;
    p.N = H; p.Kdim = 2 * I; p.expert_start = expert_start; p.E = E;
    p.C = (bf16_t*)dx_expanded; p.TK = TK;
    return launch_rows_any<EPI_PLAIN>(K_DX, p, TK, (hipStream_t)stream, w1_as_stored != 0);
}

#ifndef MTS_GEMM_F16
extern "C" int64_t mts_moe_bwd_dw_workspace_bytes(int which, int E, int H, int I) {
    if (E < 1 || H < 1 || I < 1 || (which != 1 && which != 2)) return 0;
    return which == 1 ? dw_chunk_workspace_bytes(E, 2 * I, H) : dw_chunk_workspace_bytes(E, H, I);
}
#endif

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_dw2)(const void* d_out, const void* weighted_act, const int32_t* x_gather,
                               const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                               int act_dtype, int grad_dtype, void* d_w2, void* workspace,
                               int64_t workspace_bytes, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_bwd_dw2_f16(d_out, weighted_act, x_gather, expert_start, T, K, E, H, I, act_dtype, grad_dtype, d_w2, workspace, workspace_bytes, stream);
#endif
    if (!d_out || !weighted_act || !x_gather || !expert_start || !d_w2) return MTS_ERR_NULL;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    if (act_dtype == MTS_F32) {
        if (E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1) return MTS_ERR_SHAPE;
        return mts_f32_dw((const float*)d_out, x_gather, (const float*)weighted_act, nullptr, H, I, expert_start, E,
                          grad_dtype, d_w2, (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(T * K, E, H, I, T);
    if (rc) return rc;
    if (!mts_aligned16(d_out) || !mts_aligned16(weighted_act) || !mts_aligned16(d_w2)) return MTS_ERR_ALIGN;
    DwParams p = {};
    p.P = (const bf16_t*)d_out; p.p_rows = T; p.p_gather = x_gather;
    p.Q = (const bf16_t*)weighted_act; p.q_rows = T * K; p.q_gather = nullptr;
    p.M = H; p.N = I; p.TK = T * K; p.expert_start = expert_start; p.C = d_w2;
    return launch_dw_any(K_DW2, p, E, grad_dtype, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_dw1)(const void* d_pre_act, const void* x, const int32_t* x_gather,
                               const int32_t* expert_start, int64_t T, int K, int E, int H, int I,
                               int act_dtype, int grad_dtype, void* d_w1, void* workspace,
                               int64_t workspace_bytes, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16) return mts_moe_bwd_dw1_f16(d_pre_act, x, x_gather, expert_start, T, K, E, H, I, act_dtype, grad_dtype, d_w1, workspace, workspace_bytes, stream);
#endif
    if (!d_pre_act || !x || !x_gather || !expert_start || !d_w1) return MTS_ERR_NULL;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    if (act_dtype == MTS_F32) {
        if (E < 1 || E > MTS_MAX_MOE_EXPERTS || H < 1 || I < 1) return MTS_ERR_SHAPE;
        return mts_f32_dw((const float*)d_pre_act, nullptr, (const float*)x, x_gather, 2 * I, H, expert_start, E,
                          grad_dtype, d_w1, (hipStream_t)stream);
    }
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    int rc = check_common(T * K, E, H, I, T);
    if (rc) return rc;
    if (!mts_aligned16(d_pre_act) || !mts_aligned16(x) || !mts_aligned16(d_w1)) return MTS_ERR_ALIGN;
    DwParams p = {};
    p.P = (const bf16_t*)d_pre_act; p.p_rows = T * K; p.p_gather = nullptr;
    p.Q = (const bf16_t*)x; p.q_rows = T; p.q_gather = x_gather;
    p.M = 2 * I; p.N = H; p.TK = T * K; p.expert_start = expert_start; p.C = d_w1;
    return launch_dw_any(K_DW1, p, E, grad_dtype, workspace, workspace_bytes, (hipStream_t)stream);
}

#ifndef MTS_GEMM_F16
extern "C" int mts_moe_bwd_joint_supported(int act_dtype, int H, int I) {
    return (act_dtype == MTS_BF16 || act_dtype == MTS_F16) && bwd_joint_ok(H, I) ? 1 : 0;
}
#endif

namespace {
// argument checks of the joint launch and its parameter block (without the router's part)
int fill_bwd_joint(BwdJointParams& q, const void* d_out, const void* weighted_act, const void* d_pre_act, const void* x,
                   const void* w1, const int32_t* x_gather, const int32_t* expert_start, const int32_t* s_reverse,
                   const float* ds_partial, int64_t T, int K, int E, int H, int I, int act_dtype, void* dx_expanded,
                   void* d_w1, void* d_w2, void* d_weights) {
    // d_w2 == NULL: the caller runs dW2 in a launch of its own (next to dO*W2, which it does not depend on)
    if (!d_out || !d_pre_act || !x || !w1 || !x_gather || !expert_start || !s_reverse || !ds_partial ||
        !dx_expanded || !d_w1 || !d_weights || (d_w2 && !weighted_act))
        return MTS_ERR_NULL;
    if (act_dtype != MTS_GEMM_DTYPE) return MTS_ERR_DTYPE;
    if (T <= 0 || K < 1) return MTS_ERR_SHAPE;
    const int64_t TK = T * K;
    int rc = check_common(TK, E, H, I, T);
    if (rc) return rc;
    if (!bwd_joint_ok(H, I)) return MTS_ERR_SHAPE;
    if (!mts_aligned16(d_out) || !mts_aligned16(weighted_act) || !mts_aligned16(d_pre_act) || !mts_aligned16(x) ||
        !mts_aligned16(w1) || !mts_aligned16(dx_expanded) || !mts_aligned16(d_w1) || !mts_aligned16(d_w2))
        return MTS_ERR_ALIGN;
    q.dw1.P = (const bf16_t*)d_pre_act; q.dw1.p_rows = TK; q.dw1.p_gather = nullptr;
    q.dw1.Q = (const bf16_t*)x; q.dw1.q_rows = T; q.dw1.q_gather = x_gather;
    q.dw1.M = 2 * I; q.dw1.N = H; q.dw1.TK = TK; q.dw1.expert_start = expert_start; q.dw1.C = d_w1;
    q.dw2.P = (const bf16_t*)d_out; q.dw2.p_rows = T; q.dw2.p_gather = x_gather;
    q.dw2.Q = (const bf16_t*)weighted_act; q.dw2.q_rows = TK; q.dw2.q_gather = nullptr;
    q.dw2.M = H; q.dw2.N = I; q.dw2.TK = TK; q.dw2.expert_start = expert_start; q.dw2.C = d_w2;
    q.dx.A = (const bf16_t*)d_pre_act; q.dx.a_rows = TK; q.dx.lda = 2 * I; q.dx.a_gather = nullptr;
    q.dx.B = (const bf16_t*)w1; q.dx.b_rows = H;
    q.dx.N = H; q.dx.Kdim = 2 * I; q.dx.expert_start = expert_start; q.dx.E = E;
    q.dx.C = (bf16_t*)dx_expanded; q.dx.TK = TK;
    q.ds_part = ds_partial; q.s_reverse = s_reverse; q.d_weights = (bf16_t*)d_weights; q.np = dy1_partials(I); q.entries = TK;
    return MTS_OK;
}

// can the router's backward ride in the joint launch?  Its blocks are compiled for up to kJointRouterExperts
// experts, need no more threads than a block of the launch has, and keep E x cols floats of dW_r sums and the
// logit gradients of their rows in the block's LDS
bool joint_router_ok(int H, int E, const MtsRouterBwdShape& g) {
    constexpr size_t lds_bytes = (size_t)ws_lds_elems<JointDxTile, EPI_PLAIN>() * sizeof(bf16_t);
    const size_t need = ((size_t)E * g.cols_per_block + (size_t)mts_rl::kChainRows * kJointRouterExperts) * sizeof(float);
    return E <= kJointRouterExperts && g.groups * g.col_threads <= WsLarge::NT && need <= lds_bytes && H % 4 == 0;
}
}  // namespace

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_joint)(const void* d_out, const void* weighted_act, const void* d_pre_act,
                                                 const void* x, const void* w1, const int32_t* x_gather,
                                                 const int32_t* expert_start, const int32_t* s_reverse,
                                                 const float* ds_partial, int64_t T, int K, int E, int H, int I,
                                                 int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2,
                                                 void* d_weights, void* workspace1, int64_t workspace1_bytes,
                                                 void* workspace2, int64_t workspace2_bytes, const int32_t* schedule,
                                                 void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16)
        return mts_moe_bwd_joint_f16(d_out, weighted_act, d_pre_act, x, w1, x_gather, expert_start, s_reverse,
                                     ds_partial, T, K, E, H, I, act_dtype, grad_dtype, dx_expanded, d_w1, d_w2, d_weights,
                                     workspace1, workspace1_bytes, workspace2, workspace2_bytes, schedule, stream);
#endif
    BwdJointParams q = {};
    const int rc = fill_bwd_joint(q, d_out, weighted_act, d_pre_act, x, w1, x_gather, expert_start, s_reverse, ds_partial, T,
                                  K, E, H, I, act_dtype, dx_expanded, d_w1, d_w2, d_weights);
    if (rc) return rc;
    return launch_bwd_joint(q, E, grad_dtype, workspace1, workspace1_bytes, workspace2, workspace2_bytes, schedule, (hipStream_t)stream);
}

#ifndef MTS_GEMM_F16
extern "C" int64_t mts_moe_bwd_schedule_bytes(int E) { return E >= 1 && E <= kSchedMaxExperts ? kSchedBytes : 0; }

extern "C" int mts_moe_bwd_schedule(const int32_t* expert_start, int64_t TK, int E, int32_t* schedule, void* stream) {
    if (!expert_start || !schedule) return MTS_ERR_NULL;
    if (TK <= 0 || TK > 0x7fffffffLL || E < 1 || E > kSchedMaxExperts) return MTS_ERR_SHAPE;
    if (!mts_aligned16(schedule)) return MTS_ERR_ALIGN;
    int slots, cap;
    schedule_shape(TK, E, slots, cap);
    joint_schedule_kernel<<<1, MTS_WAVE, 0, (hipStream_t)stream>>>(expert_start, E, slots, kSchedDxRows, cap, schedule);
    MTS_CHECK_LAUNCH();
    return MTS_OK;
}

extern "C" int mts_moe_bwd_joint_router_supported(int act_dtype, int64_t T, int H, int I, int E) {
    if (!mts_moe_bwd_joint_supported(act_dtype, H, I) || T <= 0 || H < 4 || H % 4 || E < 1 || E > kJointRouterExperts) return 0;
    MtsRouterBwdShape g;
    mts_router_bwd_shape(T, H, E, &g);
    return joint_router_ok(H, E, g) ? 1 : 0;
}
#endif

extern "C" int MTS_GEMM_ENTRY(mts_moe_bwd_joint_router)(
    const void* d_out, const void* weighted_act, const void* d_pre_act, const void* x, const void* w1,
    const int32_t* x_gather, const int32_t* expert_start, const int32_t* s_reverse, const float* ds_partial, int64_t T,
    int K, int E, int H, int I, int act_dtype, int grad_dtype, void* dx_expanded, void* d_w1, void* d_w2, void* d_weights,
    void* workspace1, int64_t workspace1_bytes, void* workspace2, int64_t workspace2_bytes, const float* w_r,
    const float* logits, const float* weights, const int32_t* indices, const int32_t* counts, const float* g_prob_mean,
    const float* g_z_loss, const float* g_load_balance, int normalize, void* dx_router, void* dx, float* d_w_r,
    void* router_workspace, int64_t router_workspace_bytes, const int32_t* schedule, void* stream) {
#ifndef MTS_GEMM_F16
    if (act_dtype == MTS_F16)
        return mts_moe_bwd_joint_router_f16(d_out, weighted_act, d_pre_act, x, w1, x_gather, expert_start, s_reverse,
                                            ds_partial, T, K, E, H, I, act_dtype, grad_dtype, dx_expanded, d_w1, d_w2,
                                            d_weights, workspace1, workspace1_bytes, workspace2, workspace2_bytes, w_r, logits,
                                            weights, indices, counts, g_prob_mean, g_z_loss, g_load_balance, normalize,
                                            dx_router, dx, d_w_r, router_workspace, router_workspace_bytes, schedule, stream);
#endif
    BwdJointParams q = {};
    int rc = fill_bwd_joint(q, d_out, weighted_act, d_pre_act, x, w1, x_gather, expert_start, s_reverse, ds_partial, T, K, E,
                            H, I, act_dtype, dx_expanded, d_w1, d_w2, d_weights);
    if (rc) return rc;
    rc = mts_router_bwd_check(x, w_r, T, H, E, act_dtype);
    if (rc) return rc;
    if (!logits || !weights || !indices || !dx_router || !d_w_r || !router_workspace) return MTS_ERR_NULL;
    if (g_load_balance && !counts) return MTS_ERR_NULL;
    if (K > E || K > MTS_MAX_TOP_K) return MTS_ERR_SHAPE;
    MtsRouterBwdShape g;
    mts_router_bwd_shape(T, H, E, &g);
    if (!joint_router_ok(H, E, g)) return MTS_ERR_SHAPE;
    if (router_workspace_bytes < (int64_t)g.row_blocks * E * H * (int64_t)sizeof(float)) return MTS_ERR_WORKSPACE;
    if (!mts_aligned16(router_workspace) || !mts_aligned16(d_w_r) || !mts_aligned16(dx_router) || !mts_aligned16(dx) ||
        (E == 8 && !mts_aligned16(logits)))
        return MTS_ERR_ALIGN;
    q.n_router = g.row_blocks * g.ranges;
    q.router_row_blocks = g.row_blocks;
    q.rx = (const bf16_t*)x; q.rw = w_r; q.rT = T; q.rH = H; q.rE = E;
    q.r_rows_per_block = g.rows_per_block; q.r_groups = g.groups; q.r_cols_per_block = g.cols_per_block;
    q.r_col_threads = g.col_threads;
    q.r_dx = (bf16_t*)dx_router; q.r_part = (float*)router_workspace; q.r_dw = d_w_r;
    q.c_out = (bf16_t*)dx; q.c_K = K;
    q.rg = {logits, weights, indices, counts, nullptr, nullptr, g_prob_mean, g_z_loss, g_load_balance, act_dtype, K, normalize,
            ds_partial, s_reverse, q.np};
    return launch_bwd_joint(q, E, grad_dtype, workspace1, workspace1_bytes, workspace2, workspace2_bytes, schedule, (hipStream_t)stream);
}
