// Ragged (per-expert) GEMM for gfx950 with MFMA and fp32 accumulation.
//
// One kernel body serves the three operand layouts of the MoE layer; they differ only in how a
// tile is fetched from HBM:
//   TN  C[p, n] = sum_k A[row(p), k] * W[e][n, k]     forward projections (optional row gather on A)
//   NN  C[p, n] = sum_k A[p, k]      * W[e][k, n]     input gradients
//   MT  C[e][i, j] = sum_p A[p, i] * B[row(p), j]     weight gradients (reduction over routed rows)
// Inside LDS both operands always look the same: [tile rows][BK] with the reduction index
// contiguous, 128 bytes per row, the eight 16-byte chunks of a row XOR-swizzled by the row
// number.  Operands whose reduction index is strided in HBM (W in NN, both in MT) are fetched as
// PV x PV element blocks (PV = elements per 16 bytes), transposed in registers, and written to
// LDS as whole chunks.  The MFMA loop reads 16-byte fragments, multiplies 32x32 sub-tiles, and
// the epilogue stages the tile in LDS again so that HBM sees full 16-byte row-wise stores
// (optionally fused with SwiGLU forward / backward, row scatter).
//
// Work-group -> tile mapping: a prologue kernel expands the expert offsets into a list of row
// tiles (expert, first row), so ragged and empty groups cost nothing; the main kernel renumbers
// work-groups so that each of the 8 XCDs (private L2 each) owns a contiguous range of tiles, and
// walks tiles in bands of 4 row tiles x all column tiles to reuse both panels from L2.
#include <cstddef>
#include <cstring>

#include "grouped_gemm_common.h"

namespace xma {

// ---- per-dtype tile configuration -----------------------------------------------------------
template <typename T>
struct TileCfg {  // 16-bit element types
    static constexpr int BM = 256, BN = 256, BK = 64, THREADS = 512, WAVES_M = 2, WAVES_N = 4;
};
template <>
struct TileCfg<float> {
    static constexpr int BM = 128, BN = 128, BK = 32, THREADS = 256, WAVES_M = 2, WAVES_N = 2;
};

constexpr int kLdsRowBytes = 128;  // BK * sizeof(T) for every configuration
constexpr int kChunksPerRow = 8;

__device__ __forceinline__ int swizzle_of_row(int row) { return ((row >> 1) ^ (row >> 4)) & 7; }
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
    return row * kLdsRowBytes + ((chunk ^ swizzle_of_row(row)) << 4);
}

// ---- register transposes of a PV x PV block ---------------------------------------------------
// in[r] = PV consecutive elements of block row r; out[c] = the PV elements of block column c.
__device__ __forceinline__ uint32_t pack_lo(uint32_t a, uint32_t b) { return (a & 0xffffu) | (b << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xffff0000u); }

template <int PV>
__device__ __forceinline__ void transpose_block(const uint4 (&in)[PV], uint4 (&out)[PV]);

template <>
__device__ __forceinline__ void transpose_block<8>(const uint4 (&in)[8], uint4 (&out)[8]) {
#define XMA_T16(J, D)                                                                                       \
    out[2 * J] = make_uint4(pack_lo(in[0].D, in[1].D), pack_lo(in[2].D, in[3].D), pack_lo(in[4].D, in[5].D), \
                            pack_lo(in[6].D, in[7].D));                                                     \
    out[2 * J + 1] = make_uint4(pack_hi(in[0].D, in[1].D), pack_hi(in[2].D, in[3].D), pack_hi(in[4].D, in[5].D), \
                                pack_hi(in[6].D, in[7].D));
    XMA_T16(0, x)
    XMA_T16(1, y)
    XMA_T16(2, z)
    XMA_T16(3, w)
#undef XMA_T16
}

template <>
__device__ __forceinline__ void transpose_block<4>(const uint4 (&in)[4], uint4 (&out)[4]) {
    out[0] = make_uint4(in[0].x, in[1].x, in[2].x, in[3].x);
    out[1] = make_uint4(in[0].y, in[1].y, in[2].y, in[3].y);
    out[2] = make_uint4(in[0].z, in[1].z, in[2].z, in[3].z);
    out[3] = make_uint4(in[0].w, in[1].w, in[2].w, in[3].w);
}

__device__ __forceinline__ uint4 load16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }

// Element-wise forms of a 16-byte access for operands whose sizes are not multiples of the vector width or whose
// rows are not 16-byte aligned (the reference's kernels mask such tails,
// xma/layers/moe/triton_implementation/scatter_kernel.py:39-45,91-95): the first `count` elements are moved one by
// one, the rest of the vector reads as zero / is not written.
template <typename T>
__device__ __forceinline__ uint4 load_elems(const T* p, int count) {
    constexpr int PV = 16 / (int)sizeof(T);
    union {
        uint4 v;
        T e[PV];
    } u;
    u.v = zero16();
#pragma unroll
    for (int q = 0; q < PV; ++q)
        if (q < count) u.e[q] = p[q];
    return u.v;
}
template <typename T>
__device__ __forceinline__ void store_elems(T* p, const uint4& v, int count) {
    constexpr int PV = 16 / (int)sizeof(T);
    union {
        uint4 v;
        T e[PV];
    } u;
    u.v = v;
#pragma unroll
    for (int q = 0; q < PV; ++q)
        if (q < count) p[q] = u.e[q];
}
// number of the PV elements starting at index `first` that lie below `limit`
__device__ __forceinline__ int elems_below(int64_t first, int64_t limit, int pv) {
    const int64_t left = limit - first;
    return left <= 0 ? 0 : left >= pv ? pv : (int)left;
}
// RAGGED: element-wise, `count` valid elements; otherwise one vector access (count is 0 or PV)
template <bool RAGGED, typename T>
__device__ __forceinline__ uint4 load_vec(const T* p, int count) {
    if constexpr (RAGGED) return load_elems(p, count);
    else return count > 0 ? load16(p) : zero16();
}
template <bool RAGGED, typename T>
__device__ __forceinline__ void store_vec(T* p, const uint4& v, int count) {
    if constexpr (RAGGED) store_elems(p, v, count);
    else if (count > 0) *reinterpret_cast<uint4*>(p) = v;
}

// ---- tile loaders -----------------------------------------------------------------------------
// DirectLoader: the operand's reduction index is contiguous in HBM.  NT threads starting at
// thread T0 copy R rows x 8 chunks per stage; each thread keeps its chunk column and walks rows.
template <typename T, int R, int NT, int T0>
struct DirectLoader {
    static constexpr int PV = Elem<T>::kPerVec;
    static constexpr int ITEMS = R * kChunksPerRow / NT;
    static constexpr int ROW_STEP = NT / kChunksPerRow;
    const T* row_ptr[ITEMS];  // points at the thread's chunk in reduction step 0; nullptr = masked row
    int chunk;
    int row0;
    bool active;

    template <typename RowFn>
    __device__ __forceinline__ void init(int tid, RowFn row_fn) {
        const int lt = tid - T0;
        active = lt >= 0 && lt < NT;
        chunk = lt & (kChunksPerRow - 1);
        row0 = lt / kChunksPerRow;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const T* p = active ? row_fn(row0 + i * ROW_STEP) : nullptr;
            row_ptr[i] = p ? p + chunk * PV : nullptr;
        }
    }
    // k0: first reduction index of the stage, klen: total reduction length
    template <bool RAGGED, int NV>
    __device__ __forceinline__ void load(uint4 (&v)[NV], int64_t k0, int64_t klen) const {
        static_assert(NV >= ITEMS, "staging registers");
        if (!active) return;
        const int count = elems_below(k0 + chunk * PV, klen, PV);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) v[i] = row_ptr[i] ? load_vec<RAGGED>(row_ptr[i] + k0, count) : zero16();
    }
    template <int NV>
    __device__ __forceinline__ void store(const uint4 (&v)[NV], char* lds) const {
        if (!active) return;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int row = row0 + i * ROW_STEP;
            *reinterpret_cast<uint4*>(lds + lds_chunk_offset(row, chunk)) = v[i];
        }
    }
};

// TransLoader: the operand's tile-row index is contiguous in HBM and the reduction index walks
// HBM rows.  Each of NT = 8 * R / PV threads fetches PV reduction rows x PV tile rows, transposes
// the block in registers and writes PV chunks.
template <typename T, int R, int NT, int T0>
struct TransLoader {
    static constexpr int PV = Elem<T>::kPerVec;
    static constexpr int TCOLS = R / PV;
    static_assert(NT == kChunksPerRow * TCOLS, "one PV x PV block per thread");
    int tcol, tk;
    bool active;

    __device__ __forceinline__ void init(int tid) {
        const int lt = tid - T0;
        active = lt >= 0 && lt < NT;
        tcol = lt % TCOLS;
        tk = lt / TCOLS;
    }
    // ptr_fn(r, col, count) returns the HBM address of reduction row (tk*PV + r) of this stage at this thread's
    // PV tile rows and sets `count` to how many of them exist, or returns nullptr when that row is out of range
    template <bool RAGGED, int NV, typename PtrFn>
    __device__ __forceinline__ void load(uint4 (&v)[NV], PtrFn ptr_fn) const {
        static_assert(NV >= PV, "staging registers");
        if (!active) return;
#pragma unroll
        for (int r = 0; r < PV; ++r) {
            int count = 0;
            const T* p = ptr_fn(tk * PV + r, tcol * PV, count);
            v[r] = p ? load_vec<RAGGED>(p, count) : zero16();
        }
    }
    template <int NV>
    __device__ __forceinline__ void store(const uint4 (&v)[NV], char* lds) const {
        if (!active) return;
        uint4 in[PV], o[PV];
#pragma unroll
        for (int r = 0; r < PV; ++r) in[r] = v[r];
        transpose_block<PV>(in, o);
#pragma unroll
        for (int c = 0; c < PV; ++c) *reinterpret_cast<uint4*>(lds + lds_chunk_offset(tcol * PV + c, tk)) = o[c];
    }
};

// RAGGED: column counts and reduction lengths may be any number and rows may start at any element: every access to
// HBM is element-wise with per-element bounds (slow, for the shapes the vector forms cannot take).
template <typename T, int KIND, int EPI, bool RAGGED>
__global__ __launch_bounds__(TileCfg<T>::THREADS) void grouped_gemm_kernel(const GemmParams P) {
    using Cfg = TileCfg<T>;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, THREADS = Cfg::THREADS;
    constexpr int PV = Elem<T>::kPerVec;
    constexpr int WM = BM / Cfg::WAVES_M, WN = BN / Cfg::WAVES_N;
    constexpr int MI = WM / 32, NI = WN / 32;
    constexpr int STAGE_BYTES = (BM + BN) * kLdsRowBytes;
    constexpr int C_ROW_BYTES = BN * (int)sizeof(T) + 16;
    // column tile width in units of output columns: the SwiGLU epilogue packs BN/2 `up` and BN/2
    // `gate` columns into one tile
    constexpr int BN_OUT = EPI == EPI_PAIRED ? BN / 2 : BN;
    static_assert(BK * sizeof(T) == kLdsRowBytes, "LDS rows are 128 bytes");

    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm0 = (wave / Cfg::WAVES_N) * WM;
    const int wn0 = (wave % Cfg::WAVES_N) * WN;

    // ---- which tile ----
    const int row_tiles = KIND == XMA_GEMM_MT ? P.row_tiles_max * P.num_experts : P.tile_count[0];
    int row_tile, col_tile;
    if (!locate_tile<KIND == XMA_GEMM_MT>(row_tiles, P.col_tiles, row_tile, col_tile)) return;

    const T* A = reinterpret_cast<const T*>(P.a);
    const T* B = reinterpret_cast<const T*>(P.b);

    int expert;
    int64_t m_begin, m_end;      // grouped rows covered by this tile (TN/NN) or reduced over (MT)
    int64_t tile_i0 = 0;         // MT: first row of C[e] in this tile
    int64_t n0;                  // first output column (TN/NN) / first column of C[e] (MT)
    int64_t red_len;             // reduction length
    if constexpr (KIND == XMA_GEMM_MT) {
        expert = row_tile / P.row_tiles_max;
        tile_i0 = (int64_t)(row_tile % P.row_tiles_max) * BM;
        m_begin = P.offsets[expert];
        m_end = P.offsets[expert + 1];
        red_len = m_end - m_begin;
        n0 = (int64_t)col_tile * BN;
    } else {
        expert = P.tile_expert[row_tile];
        m_begin = P.tile_row0[row_tile];
        const int64_t e_end = P.offsets[expert + 1];
        m_end = m_begin + BM < e_end ? m_begin + BM : e_end;
        red_len = P.k;
        n0 = (int64_t)col_tile * BN_OUT;
    }

    // ---- loaders ----
    constexpr bool A_TRANS = KIND == XMA_GEMM_MT;
    constexpr bool B_TRANS = KIND != XMA_GEMM_TN;
    constexpr bool SPLIT = sizeof(T) == 2 && (A_TRANS || B_TRANS);  // halves of the block serve one operand each
    constexpr int NT_HALF = THREADS / 2;
    // thread ranges: (count, first thread) per operand
    constexpr int A_NT = SPLIT ? NT_HALF : THREADS;
    constexpr int A_T0 = (SPLIT && KIND == XMA_GEMM_NN) ? NT_HALF : 0;
    constexpr int B_NT = SPLIT ? NT_HALF : THREADS;
    constexpr int B_T0 = (SPLIT && KIND == XMA_GEMM_MT) ? NT_HALF : 0;

    DirectLoader<T, BM, A_NT, A_T0> a_direct;
    TransLoader<T, BM, kChunksPerRow * BM / PV, A_T0> a_trans;
    DirectLoader<T, BN, B_NT, B_T0> b_direct;
    TransLoader<T, BN, kChunksPerRow * BN / PV, B_T0> b_trans;
    // Staging registers between HBM and LDS.  When the block is split, a thread serves one operand
    // only, so both loaders share one register set.
    constexpr int A_REGS = A_TRANS ? PV : BM * kChunksPerRow / A_NT;
    constexpr int B_REGS = B_TRANS ? PV : BN * kChunksPerRow / B_NT;
    uint4 st_a[A_REGS > B_REGS || !SPLIT ? A_REGS : B_REGS];
    uint4 st_b_own[SPLIT ? 1 : B_REGS];
    auto& st_b = [&]() -> auto& {
        if constexpr (SPLIT)
            return st_a;
        else
            return st_b_own;
    }();
    static_assert(!A_TRANS || kChunksPerRow * BM / PV == A_NT, "A transposing loader thread count");
    static_assert(!B_TRANS || kChunksPerRow * BN / PV == B_NT, "B transposing loader thread count");

    const T* Wexp = B + (KIND == XMA_GEMM_MT ? 0 : (int64_t)expert * P.b_expert_stride);

    if constexpr (!A_TRANS) {
        a_direct.init(tid, [&](int r) -> const T* {
            const int64_t p = m_begin + r;
            if (p >= m_end) return nullptr;
            const int64_t src = P.in_index ? source_row(P, p) : p;
            return A + src * P.lda;
        });
    } else {
        a_trans.init(tid);
    }
    if constexpr (!B_TRANS) {
        b_direct.init(tid, [&](int r) -> const T* {
            int64_t n;
            if constexpr (EPI == EPI_PAIRED) {
                const int64_t half = P.n / 2;
                const int64_t j = n0 + (r % BN_OUT);
                if (j >= half) return nullptr;
                n = r < BN_OUT ? j : half + j;
            } else {
                n = n0 + r;
                if (n >= P.n) return nullptr;
            }
            return Wexp + n * P.ldb;
        });
    } else {
        b_trans.init(tid);
    }

    auto load_stage = [&](int64_t k0) {
        if constexpr (!A_TRANS) {
            a_direct.template load<RAGGED>(st_a, k0, red_len);
        } else {
            a_trans.template load<RAGGED>(st_a, [&](int r, int col, int& count) -> const T* {
                const int64_t p = m_begin + k0 + r;
                const int64_t i = tile_i0 + col;
                count = elems_below(i, P.n, PV);
                return (p < m_end && count > 0) ? A + p * P.lda + i : nullptr;
            });
        }
        if constexpr (!B_TRANS) {
            b_direct.template load<RAGGED>(st_b, k0, red_len);
        } else if constexpr (KIND == XMA_GEMM_NN) {
            b_trans.template load<RAGGED>(st_b, [&](int r, int col, int& count) -> const T* {
                const int64_t kk = k0 + r;
                const int64_t n = n0 + col;
                count = elems_below(n, P.n, PV);
                return (kk < P.k && count > 0) ? Wexp + kk * P.ldb + n : nullptr;
            });
        } else {
            b_trans.template load<RAGGED>(st_b, [&](int r, int col, int& count) -> const T* {
                const int64_t p = m_begin + k0 + r;
                const int64_t j = n0 + col;
                count = elems_below(j, P.k, PV);
                if (p >= m_end || count == 0) return nullptr;
                const int64_t src = P.in_index ? source_row(P, p) : p;
                return B + src * P.ldb + j;
            });
        }
    };
    auto store_stage = [&](int buf) {
        char* base = lds + buf * STAGE_BYTES;
        if constexpr (!A_TRANS)
            a_direct.store(st_a, base);
        else
            a_trans.store(st_a, base);
        if constexpr (!B_TRANS)
            b_direct.store(st_b, base + BM * kLdsRowBytes);
        else
            b_trans.store(st_b, base + BM * kLdsRowBytes);
    };

    // ---- accumulators and fragment addressing ----
    f32x16_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    const int frag_row = lane & 31;
    const int frag_half = lane >> 5;
    int a_off[MI], a_sw[MI], b_off[NI], b_sw[NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const int row = wm0 + mi * 32 + frag_row;
        a_off[mi] = row * kLdsRowBytes;
        a_sw[mi] = swizzle_of_row(row);
    }
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int row = wn0 + ni * 32 + frag_row;
        b_off[ni] = BM * kLdsRowBytes + row * kLdsRowBytes;
        b_sw[ni] = swizzle_of_row(row);
    }

    const int64_t num_stages = (red_len + BK - 1) / BK;
    if (num_stages > 0) {
        load_stage(0);
        store_stage(0);
    }
    __syncthreads();
    for (int64_t s = 0; s < num_stages; ++s) {
        const bool more = s + 1 < num_stages;
        if (more) load_stage((s + 1) * BK);
        const char* base = lds + (int)(s & 1) * STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < kChunksPerRow / 2; ++kk) {
            const int chunk = 2 * kk + frag_half;
            uint4 af[MI], bfr[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                af[mi] = *reinterpret_cast<const uint4*>(base + a_off[mi] + ((chunk ^ a_sw[mi]) << 4));
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
                bfr[ni] = *reinterpret_cast<const uint4*>(base + b_off[ni] + ((chunk ^ b_sw[ni]) << 4));
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) Mma<T>::run(bfr[ni], af[mi], acc[mi][ni]);
        }
        if (more) store_stage((int)((s + 1) & 1));
        __syncthreads();
    }

    // ---- epilogue: registers -> LDS tile [BM][BN] -> HBM ----
    // MFMA result element r of lane l: tile column = 8*(r/4) + 4*(l/32) + r%4 (+32*ni), tile row = l%32 (+32*mi)
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        const int row = wm0 + mi * 32 + frag_row;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = wn0 + ni * 32 + 8 * g + 4 * frag_half;
                char* dst = lds + row * C_ROW_BYTES + col * (int)sizeof(T);
                float f[4] = {acc[mi][ni][4 * g], acc[mi][ni][4 * g + 1], acc[mi][ni][4 * g + 2], acc[mi][ni][4 * g + 3]};
                if constexpr (KIND == XMA_GEMM_TN) {
                    // the expert's bias, added to the fp32 sums before they are rounded; tile column `col` is
                    // weight row n0 + col, or for a gated tile n0 + col (first half) and N/2 + n0 + col - BN_OUT
                    if (P.bias != nullptr) {
                        int64_t n;
                        bool exists;
                        if constexpr (EPI == EPI_PAIRED) {
                            const int64_t half_n = P.n / 2;
                            n = n0 + (col % BN_OUT) + (col >= BN_OUT ? half_n : 0);
                            exists = n0 + (col % BN_OUT) < half_n;
                        } else {
                            n = n0 + col;
                            exists = n < P.n;
                        }
                        if (exists) {
                            const T* b = reinterpret_cast<const T*>(P.bias) + (int64_t)expert * P.ld_bias + n;
                            const int64_t limit = EPI == EPI_PAIRED ? (col >= BN_OUT ? P.n : P.n / 2) : P.n;
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                                if (!RAGGED || n + q < limit) f[q] += Elem<T>::load(b + q);
                        }
                    }
                }
                if constexpr (sizeof(T) == 4) {
                    *reinterpret_cast<uint4*>(dst) = Elem<float>::pack(f);
                } else {
                    *reinterpret_cast<uint2*>(dst) = make_uint2(Elem<T>::pack2(f[0], f[1]), Elem<T>::pack2(f[2], f[3]));
                }
            }
        }
    }
    __syncthreads();

    constexpr int C_CHUNKS = BN / PV;          // 16-byte chunks per tile row
    constexpr int ROWS_PER_PASS = THREADS / C_CHUNKS;
    const int cc = tid % C_CHUNKS;
    T* C = reinterpret_cast<T*>(P.c);
#pragma unroll 1
    for (int r = tid / C_CHUNKS; r < BM; r += ROWS_PER_PASS) {
        const char* src = lds + r * C_ROW_BYTES;
        if constexpr (KIND == XMA_GEMM_MT) {
            const int64_t i = tile_i0 + r, j = n0 + cc * PV;
            if (i < P.n)
                store_vec<RAGGED>(C + (int64_t)expert * P.c_expert_stride + i * P.ldc + j,
                                  *reinterpret_cast<const uint4*>(src + cc * 16), elems_below(j, P.k, PV));
        } else {
            const int64_t p = m_begin + r;
            if (p >= m_end) break;
            const int64_t orow = P.out_index ? load_index(P.out_index, P.idx_is_i64, p) : p;
            if constexpr (EPI == EPI_PLAIN) {
                const int64_t n = n0 + cc * PV;
                const int count = elems_below(n, P.n, PV);
                if (count > 0) {
                    const uint4 v = *reinterpret_cast<const uint4*>(src + cc * 16);
                    if (KIND == XMA_GEMM_TN && P.act == ACT_GELU_TANH) {
                        if (P.aux) store_vec<RAGGED>(reinterpret_cast<T*>(P.aux) + p * P.ld_aux + n, v, count);
                        float h[PV], o[PV];
                        Elem<T>::unpack(v, h);
#pragma unroll
                        for (int q = 0; q < PV; ++q) o[q] = gelu_tanh_forward<false>(h[q]);
                        store_vec<RAGGED>(C + orow * P.ldc + n, Elem<T>::pack(o), count);
                    } else {
                        store_vec<RAGGED>(C + orow * P.ldc + n, v, count);
                    }
                }
            } else if constexpr (EPI == EPI_PAIRED) {
                constexpr int HALF_CHUNKS = C_CHUNKS / 2;
                const int64_t half = P.n / 2;
                const int64_t j = n0 + (cc % HALF_CHUNKS) * PV;
                const int count = elems_below(j, half, PV);
                if (count > 0) {
                    if (P.aux) {
                        T* h = reinterpret_cast<T*>(P.aux) + p * P.ld_aux;
                        store_vec<RAGGED>(h + (cc < HALF_CHUNKS ? j : half + j),
                                          *reinterpret_cast<const uint4*>(src + cc * 16), count);
                    }
                    if (cc < HALF_CHUNKS) {
                        float u[PV], g[PV], o[PV];
                        Elem<T>::unpack(*reinterpret_cast<const uint4*>(src + cc * 16), u);
                        Elem<T>::unpack(*reinterpret_cast<const uint4*>(src + (cc + HALF_CHUNKS) * 16), g);
#pragma unroll
                        for (int q = 0; q < PV; ++q) o[q] = gated_forward<false>(P.act, u[q], g[q]);
                        store_vec<RAGGED>(C + orow * P.ldc + j, Elem<T>::pack(o), count);
                    }
                }
            } else {  // EPI_BACKWARD: the product is the activation's upstream gradient
                const int64_t n = n0 + cc * PV;
                const int count = elems_below(n, P.n, PV);
                if (count > 0) {
                    const T* h = reinterpret_cast<const T*>(P.aux) + p * P.ld_aux;
                    float u[PV], g[PV], d[PV], du[PV], dg[PV];
                    Elem<T>::unpack(load_vec<RAGGED>(h + n, count), u);
                    Elem<T>::unpack(*reinterpret_cast<const uint4*>(src + cc * 16), d);
                    if (P.act == ACT_GELU_TANH) {
#pragma unroll
                        for (int q = 0; q < PV; ++q) du[q] = gelu_tanh_backward<false>(u[q], d[q]);
                        store_vec<RAGGED>(C + orow * P.ldc + n, Elem<T>::pack(du), count);
                    } else {
                        Elem<T>::unpack(load_vec<RAGGED>(h + P.n + n, count), g);
#pragma unroll
                        for (int q = 0; q < PV; ++q) gated_backward<false>(P.act, u[q], g[q], d[q], du[q], dg[q]);
                        store_vec<RAGGED>(C + orow * P.ldc + n, Elem<T>::pack(du), count);
                        store_vec<RAGGED>(C + orow * P.ldc + P.n + n, Elem<T>::pack(dg), count);
                    }
                }
            }
        }
    }
}

template <typename T>
constexpr int lds_bytes() {
    using Cfg = TileCfg<T>;
    constexpr int stages = 2 * (Cfg::BM + Cfg::BN) * kLdsRowBytes;
    constexpr int ctile = Cfg::BM * (Cfg::BN * (int)sizeof(T) + 16);
    return stages > ctile ? stages : ctile;
}

template <typename T, int KIND, int EPI, bool RAGGED>
static int launch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    using Cfg = TileCfg<T>;
    constexpr int PV = Elem<T>::kPerVec;
    GemmParams P;
    fill_params(a, P);

    int64_t grid;
    if (KIND == XMA_GEMM_MT) {
        P.row_tiles_max = (int32_t)ceil_div(a.n, Cfg::BM);
        P.col_tiles = (int32_t)ceil_div(a.k, Cfg::BN);
        grid = grid_for_tiles((int64_t)P.row_tiles_max * a.num_experts, P.col_tiles);
    } else {
        const int64_t rt = max_row_tiles(a.rows, a.num_experts, Cfg::BM);
        int32_t* ws = reinterpret_cast<int32_t*>(a.workspace);
        P.tile_count = ws;
        P.tile_expert = ws + 4;
        P.tile_row0 = ws + 4 + rt;
        P.row_tiles_max = (int32_t)rt;
        const int bn_out = EPI == EPI_PAIRED ? Cfg::BN / 2 : Cfg::BN;
        const int64_t n_out = EPI == EPI_PAIRED ? a.n / 2 : a.n;
        P.col_tiles = (int32_t)ceil_div(n_out, bn_out);
        grid = grid_for_tiles(rt, P.col_tiles);
        hipLaunchKernelGGL(build_row_tiles_kernel, dim3(1), dim3(1024), 0, stream, a.expert_offsets, a.num_experts,
                           Cfg::BM, ws + 4, ws + 4 + rt, ws, nullptr);
    }
    XMA_REQUIRE(grid < ((int64_t)1 << 31), "xma_grouped_gemm: %lld tiles exceed the grid limit", (long long)grid);
    (void)PV;
    auto kernel = grouped_gemm_kernel<T, KIND, EPI, RAGGED>;
    // set on every launch: the attribute belongs to the (function, device) pair, and the call is a cheap host-side
    // update that needs no shared flag between threads
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes<T>());
    if (err != hipSuccess) {
        set_error("xma_grouped_gemm: cannot reserve %d bytes of LDS: %s", lds_bytes<T>(), hipGetErrorString(err));
        return 2;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(Cfg::THREADS), lds_bytes<T>(), stream, P);
    return check_launch("xma_grouped_gemm");
}

void fill_params(const xma_grouped_gemm_args& a, GemmParams& P) {
    P.a = a.a;
    P.b = a.b;
    P.c = a.c;
    P.aux = a.aux;
    P.offsets = a.expert_offsets;
    P.expert_order = nullptr;
    P.bias = a.bias;
    P.ld_bias = a.ld_bias;
    int shape = 0;
    split_epilogue(a.epilogue, shape, P.act);
    P.in_index = a.in_index;
    P.out_index = a.out_index;
    P.lda = a.lda;
    P.ldb = a.ldb;
    P.ldc = a.ldc;
    P.ld_aux = a.ld_aux;
    P.b_expert_stride = a.b_expert_stride;
    P.c_expert_stride = a.c_expert_stride;
    P.n = a.n;
    P.k = a.k;
    P.num_experts = a.num_experts;
    P.in_fan_out = a.in_fan_out > 0 ? a.in_fan_out : 1;
    P.idx_is_i64 = a.idx_is_i64;
    P.tile_expert = nullptr;
    P.tile_row0 = nullptr;
    P.tile_count = nullptr;
    P.row_tiles_max = 0;
    P.col_tiles = 0;
}

template <typename T, bool RAGGED>
static int dispatch_kind(const xma_grouped_gemm_args& a, hipStream_t stream) {
    int shape = EPI_PLAIN, act = ACT_NONE;
    split_epilogue(a.epilogue, shape, act);
    switch (a.kind) {
        case XMA_GEMM_TN:
            if (shape == EPI_PAIRED) return launch<T, XMA_GEMM_TN, EPI_PAIRED, RAGGED>(a, stream);
            return launch<T, XMA_GEMM_TN, EPI_PLAIN, RAGGED>(a, stream);
        case XMA_GEMM_NN:
            if (shape == EPI_BACKWARD) return launch<T, XMA_GEMM_NN, EPI_BACKWARD, RAGGED>(a, stream);
            return launch<T, XMA_GEMM_NN, EPI_PLAIN, RAGGED>(a, stream);
        default:
            return launch<T, XMA_GEMM_MT, EPI_PLAIN, RAGGED>(a, stream);
    }
}
template <typename T>
static int dispatch_kind(const xma_grouped_gemm_args& a, bool ragged, hipStream_t stream) {
    return ragged ? dispatch_kind<T, true>(a, stream) : dispatch_kind<T, false>(a, stream);
}

static int largest_bm() { return TileCfg<bf16_t>::BM > TileCfg<float>::BM ? TileCfg<bf16_t>::BM : TileCfg<float>::BM; }
static int smallest_bm() { return TileCfg<bf16_t>::BM < TileCfg<float>::BM ? TileCfg<bf16_t>::BM : TileCfg<float>::BM; }

}  // namespace xma

using namespace xma;

extern "C" {

int64_t xma_grouped_gemm_workspace_bytes(int32_t num_experts, int64_t rows) {
    if (num_experts < 1 || rows < 0) return -1;
    (void)largest_bm();
    // tile tables (sized for the smallest tile height of any kernel), then the split-K counters and partials
    const int64_t rt = max_row_tiles(rows, num_experts, smallest_bm());
    return tile_table_bytes(rt) + split_region_bytes();
}

int xma_grouped_gemm(const xma_grouped_gemm_args* args, void* stream_) {
    XMA_REQUIRE(args != nullptr, "xma_grouped_gemm: null args");
    // The caller says how long its revision of the struct is; fields it does not know are zero / NULL.
    XMA_REQUIRE(args->struct_size >= offsetof(xma_grouped_gemm_args, workspace_bytes) + sizeof(int64_t) &&
                    args->struct_size <= sizeof(xma_grouped_gemm_args),
                "xma_grouped_gemm: struct_size=%u is not a revision of xma_grouped_gemm_args this library knows "
                "(%zu bytes at ABI version %d)",
                args->struct_size, sizeof(xma_grouped_gemm_args), XMA_ABI_VERSION);
    xma_grouped_gemm_args copy;
    memset(&copy, 0, sizeof(copy));
    memcpy(&copy, args, args->struct_size);
    const xma_grouped_gemm_args& a = copy;
    XMA_REQUIRE(a.reserved == 0, "xma_grouped_gemm: reserved field must be 0");
    XMA_REQUIRE(valid_dtype(a.dtype), "xma_grouped_gemm: bad dtype %d", a.dtype);
    XMA_REQUIRE(a.kind >= XMA_GEMM_TN && a.kind <= XMA_GEMM_MT, "xma_grouped_gemm: bad kind %d", a.kind);
    XMA_REQUIRE(a.num_experts >= 1 && a.num_experts <= 16384, "xma_grouped_gemm: num_experts=%d outside [1, 16384]",
                a.num_experts);
    XMA_REQUIRE(a.rows >= 0 && a.rows < ((int64_t)1 << 31) && a.n >= 0 && a.k >= 0, "xma_grouped_gemm: bad sizes");
    XMA_REQUIRE(a.expert_offsets != nullptr, "xma_grouped_gemm: expert_offsets is null");
    // Sizes that are multiples of the vector width (8 elements of a 16-bit type, 4 of fp32) and 16-byte aligned rows
    // take the vector kernels.  Anything else takes the element-wise form of the register-staged kernel: correct for
    // every size and alignment, at a fraction of the speed.
    const int pv = a.dtype == XMA_F32 ? 4 : 8;
    const int64_t elem = a.dtype == XMA_F32 ? 4 : 2;
    auto elem_aligned = [&](const void* p) { return (reinterpret_cast<uintptr_t>(p) % elem) == 0; };
    XMA_REQUIRE(elem_aligned(a.a) && elem_aligned(a.b) && elem_aligned(a.c) && elem_aligned(a.aux) && elem_aligned(a.bias),
                "xma_grouped_gemm: operands must be aligned to their element size");
    const bool ragged = a.n % pv != 0 || a.k % pv != 0 || a.lda % pv != 0 || a.ldb % pv != 0 || a.ldc % pv != 0 ||
                        a.b_expert_stride % pv != 0 || a.c_expert_stride % pv != 0 || a.ld_aux % pv != 0 ||
                        (a.bias != nullptr && a.ld_bias % pv != 0) || !aligned16(a.a) || !aligned16(a.b) ||
                        !aligned16(a.c) || !aligned16(a.aux) || !aligned16(a.bias);
    const bool mt = a.kind == XMA_GEMM_MT;
    if (mt) {
        XMA_REQUIRE(a.epilogue == XMA_EPI_NONE && a.bias == nullptr, "xma_grouped_gemm: MT takes no epilogue and no bias");
        XMA_REQUIRE(a.lda >= a.n && a.ldb >= a.k && a.ldc >= a.k, "xma_grouped_gemm: MT row strides too small");
        XMA_REQUIRE(a.out_index == nullptr, "xma_grouped_gemm: MT takes no out_index");
        XMA_REQUIRE(a.workspace == nullptr || a.workspace_bytes >= expert_order_bytes(a.num_experts),
                    "xma_grouped_gemm: MT workspace too small (%lld < %lld)", (long long)a.workspace_bytes,
                    (long long)expert_order_bytes(a.num_experts));
        if (a.n == 0 || a.k == 0) return 0;
    } else {
        int shape = EPI_PLAIN, act = ACT_NONE;
        split_epilogue(a.epilogue, shape, act);
        const bool forward_epi = a.epilogue == XMA_EPI_SWIGLU || a.epilogue == XMA_EPI_GLU || a.epilogue == XMA_EPI_GELU_TANH;
        const bool backward_epi =
            a.epilogue == XMA_EPI_SWIGLU_BWD || a.epilogue == XMA_EPI_GLU_BWD || a.epilogue == XMA_EPI_GELU_TANH_BWD;
        XMA_REQUIRE(a.epilogue == XMA_EPI_NONE || (a.kind == XMA_GEMM_TN && forward_epi) ||
                        (a.kind == XMA_GEMM_NN && backward_epi),
                    "xma_grouped_gemm: epilogue %d not available for kind %d", a.epilogue, a.kind);
        // nothing to do, and nothing to hold the views of empty tensors to (their pointers may be null and their
        // strides anything)
        if (a.rows == 0 || a.n == 0) return 0;
        XMA_REQUIRE(a.lda >= a.k, "xma_grouped_gemm: lda too small");
        XMA_REQUIRE(a.ldb >= (a.kind == XMA_GEMM_TN ? a.k : a.n), "xma_grouped_gemm: ldb too small");
        if (shape == EPI_PAIRED) {
            XMA_REQUIRE(a.n % 2 == 0, "xma_grouped_gemm: gated epilogue needs an even n");
            XMA_REQUIRE(a.ldc >= a.n / 2, "xma_grouped_gemm: ldc too small");
            XMA_REQUIRE(a.aux == nullptr || a.ld_aux >= a.n, "xma_grouped_gemm: ld_aux too small");
        } else if (shape == EPI_BACKWARD) {
            const int64_t saved = act == ACT_GELU_TANH ? a.n : 2 * a.n;  // columns of the saved pre-activation
            XMA_REQUIRE(a.aux != nullptr && a.ld_aux >= saved && a.ldc >= saved,
                        "xma_grouped_gemm: activation backward epilogue needs aux/ldc of %lld columns", (long long)saved);
            XMA_REQUIRE(a.out_index == nullptr, "xma_grouped_gemm: activation backward epilogue writes grouped rows");
        } else {
            XMA_REQUIRE(a.ldc >= a.n, "xma_grouped_gemm: ldc too small");
            XMA_REQUIRE(act == ACT_NONE || a.aux == nullptr || a.ld_aux >= a.n, "xma_grouped_gemm: ld_aux too small");
            XMA_REQUIRE(act == ACT_NONE || a.out_index == nullptr || a.aux == nullptr,
                        "xma_grouped_gemm: the pre-activation is kept for grouped outputs only");
        }
        XMA_REQUIRE(a.bias == nullptr || (a.kind == XMA_GEMM_TN && a.ld_bias >= a.n),
                    "xma_grouped_gemm: bias needs a forward (TN) kind and ld_bias >= n");
        XMA_REQUIRE(a.workspace != nullptr &&
                        a.workspace_bytes >= xma_grouped_gemm_workspace_bytes(a.num_experts, a.rows),
                    "xma_grouped_gemm: workspace too small (%lld < %lld)", (long long)a.workspace_bytes,
                    (long long)xma_grouped_gemm_workspace_bytes(a.num_experts, a.rows));
    }
    // (without rows the weight-gradient kind still writes its zeros; its operands, which may then be null, are never read)
    XMA_REQUIRE(a.c && (a.rows == 0 || (a.a && a.b)), "xma_grouped_gemm: null operand");
    hipStream_t stream = (hipStream_t)stream_;
    // a gated tile of the vector kernels pairs whole 16-byte chunks of the two halves
    const bool paired_tail = (a.epilogue == XMA_EPI_SWIGLU || a.epilogue == XMA_EPI_GLU) && a.n % (2 * pv) != 0;
    const bool elementwise = ragged || paired_tail;
    if (!elementwise && dma_gemm_supports(a)) return launch_dma_gemm(a, stream);
    switch (a.dtype) {
        case XMA_F32:
            return dispatch_kind<float>(a, elementwise, stream);
        case XMA_F16:
            return dispatch_kind<f16_t>(a, elementwise, stream);
        default:
            return dispatch_kind<bf16_t>(a, elementwise, stream);
    }
}

}  // extern "C"
