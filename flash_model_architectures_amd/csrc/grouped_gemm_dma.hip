// Ragged (per-expert) GEMM for 16-bit element types on gfx950, built around the LDS-DMA load path
// (global_load_lds_dwordx4): tiles travel HBM -> LDS without passing through registers, four
// 32-deep stages are kept in LDS so that three stages of loads are always in flight while the
// fourth is multiplied, and operands whose reduction index is strided in HBM are fetched in their
// HBM layout and transposed by the LDS read itself (ds_read_b64_tr_b16).
//
// Tile 256 x 256 per work-group, 8 waves as 2 x 4, each wave 128 x 64 (4 x 2 MFMA 32x32x16 tiles).
//
// LDS layouts (one 32 KiB array per stage: 16 KiB per operand):
//   K-contiguous operand (A in TN/NN, W in TN): [256 tile rows][32 k], 64 bytes per row; the four
//     16-byte chunks of row r sit at chunk ^ ((r >> 2) & 3), so that the 16 rows a quarter-wave reads
//     in one ds_read_b128 cover all 64 banks.
//   K-strided operand (W in NN, both operands in MT): [32 k][256 tile rows], 512 bytes per k row; chunk c
//     of k row r sits at c ^ ((r & 3) << 2), so that the four k rows one transposing read touches fall
//     into different bank groups.
// A DMA load writes lane l's 16 bytes at (wave-uniform LDS base) + 16*l, so the swizzles are applied
// by choosing which HBM chunk each lane fetches.  Masked rows / reduction tails are fetched from a
// 16-byte page of zeros, which keeps every lane active and the outstanding-load count uniform.
#include "grouped_gemm_common.h"

namespace xma {
namespace dma {

constexpr int BM = 256, BN = 256, BK = 32, NS = 4, THREADS = 512;
constexpr int WAVES_N = 4, WM = 128, WN = 64, MI = WM / 32, NI = WN / 32;
constexpr int OPERAND_BYTES = BM * BK * 2;  // 16 KiB, same for both layouts and both operands
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;
constexpr int LOADS_PER_STAGE = 4;          // DMA instructions per wave per stage (2 per operand)
static_assert(BM == BN, "both operands use the same tile height");

__shared__ __attribute__((aligned(1024))) char stage0[STAGE_BYTES];
__shared__ __attribute__((aligned(1024))) char stage1[STAGE_BYTES];
__shared__ __attribute__((aligned(1024))) char stage2[STAGE_BYTES];
__shared__ __attribute__((aligned(1024))) char stage3[STAGE_BYTES];

// The stages are distinct arrays on purpose: the compiler can then prove that a fragment read of
// one stage does not alias the DMA writes still in flight to the others, and does not drain them.
template <int S>
__device__ __forceinline__ char* stage_ptr() {
    static_assert(S >= 0 && S < NS, "stage index");
    if constexpr (S == 0) return stage0;
    if constexpr (S == 1) return stage1;
    if constexpr (S == 2) return stage2;
    return stage3;
}

__device__ __attribute__((aligned(16))) uint32_t g_zero_page[4];  // zero-initialised

typedef __attribute__((ext_vector_type(4))) short short4_t;
#define XMA_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define XMA_LDS_S4(p) ((__attribute__((address_space(3))) short4_t*)(p))

__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// s_waitcnt with only the vector-memory counter constrained (lgkmcnt = 15, expcnt = 7)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    compiler_fence();
    __builtin_amdgcn_s_waitcnt((N & 0xF) | (7 << 4) | (0xF << 8) | ((N >> 4) << 14));
    compiler_fence();
}

__device__ __forceinline__ void block_barrier() {
    compiler_fence();
    __builtin_amdgcn_s_barrier();
    compiler_fence();
}

// Per-thread state of one operand's DMA loads: two loads per stage.
template <typename T>
struct OperandLoads {
    const T* ptr[2];    // HBM address of this lane's chunk in stage 0 (or the zero page)
    int64_t step;       // elements to advance per stage
    int32_t red[2];     // reduction index covered by the lane in stage 0 (chunk start or k row)
    bool valid[2];      // false: always the zero page (row / column outside the operand)
    int lds_off[2];     // byte offset of the wave's 1 KiB destination inside the operand's LDS tile
};

// K-contiguous layout: wave w fills tile rows [16w, 16w+16) and [128 + 16w, ...): lane l -> row + l/4,
// physical chunk l%4.  row_fn(tile row) returns the HBM row base or nullptr.
template <typename T, typename RowFn>
__device__ __forceinline__ void setup_kcontig(OperandLoads<T>& L, int wave, int lane, RowFn row_fn) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = i * 128 + wave * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);  // logical chunk stored at physical position lane&3
        const T* base = row_fn(row);
        L.valid[i] = base != nullptr;
        L.ptr[i] = L.valid[i] ? base + chunk * 8 : reinterpret_cast<const T*>(g_zero_page);
        L.red[i] = chunk * 8;
        L.lds_off[i] = (i * 128 + wave * 16) * (BK * 2);
    }
    L.step = BK;
}

// K-strided layout: wave w fills k rows {2w, 2w+1} and {16 + 2w, 16 + 2w + 1}: lane l -> k row + l/32,
// physical chunk l%32.  `base` points at (reduction row 0, first tile column); `cols_left` = number of
// valid columns from there; ld = row stride.
template <typename T>
__device__ __forceinline__ void setup_kstrided(OperandLoads<T>& L, int wave, int lane, const T* base, int64_t ld,
                                               int64_t cols_left) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int krow = i * 16 + wave * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2);
        L.valid[i] = chunk * 8 < cols_left;
        L.ptr[i] = L.valid[i] ? base + (int64_t)krow * ld + chunk * 8 : reinterpret_cast<const T*>(g_zero_page);
        L.red[i] = krow;
        L.lds_off[i] = (i * 16 + wave * 2) * (BN * 2);
    }
    L.step = (int64_t)BK * ld;
}

// Issue this wave's two loads of one operand for the stage starting at reduction index k0.
template <typename T>
__device__ __forceinline__ void issue_operand(const OperandLoads<T>& L, char* lds_stage, int operand_off, int64_t stage,
                                              int64_t k0, int64_t red_len) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const bool ok = L.valid[i] && (k0 + L.red[i] < red_len);
        const T* src = ok ? L.ptr[i] + stage * L.step : reinterpret_cast<const T*>(g_zero_page);
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(src),
                                         XMA_LDS(lds_stage + (operand_off + L.lds_off[i])), 16, 0, 0);
    }
}

// LDS accesses below add ONE integer byte offset to the stage array, and the offset is passed through
// opaque() so that the optimiser cannot split it into a chain of partial sums: the compiler attaches the
// "this access belongs to stage array X" information it needs to keep DMA loads to the other arrays in
// flight only to accesses whose address is a short derivation from the array.
__device__ __forceinline__ int opaque(int v) {
    asm("" : "+v"(v));
    return v;
}

// Fragment of a K-contiguous tile: row `row`, reduction elements kk*16 + 8*half .. +7.
__device__ __forceinline__ int kcontig_offset(int row, int kk, int half) {
    const int chunk = (2 * kk + half) ^ ((row >> 2) & 3);
    return row * (BK * 2) + (chunk << 4);
}

// Same fragment out of a K-strided tile, transposed by the LDS read.  Within each 16-lane group the
// instruction hands lane i the i-th 16-bit element of four 16-element rows, where row j is assembled from
// the 8-byte pieces addressed by lanes 4j..4j+3.  So lane i addresses (k row 4*j' + i/4, columns 4*(i%4)..+3)
// and receives four consecutive k of column i; a second read four k rows further down completes the
// eight reduction elements of the MFMA operand.
__device__ __forceinline__ int kstrided_offset(int col0, int kk, int lane) {
    const int i = lane & 15, group = lane >> 4;
    const int col = col0 + 16 * (group & 1) + 4 * (i & 3);
    const int krow0 = kk * 16 + 8 * (group >> 1) + (i >> 2);
    const int chunk = (col >> 3) ^ ((krow0 & 3) << 2);  // (krow0 + 4) & 3 == krow0 & 3
    return krow0 * (BN * 2) + (chunk << 4) + ((col & 4) << 1);
}

typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

template <bool STRIDED>
__device__ __forceinline__ u32x4_t read_fragment(const char* stage, int offset) {
    if constexpr (STRIDED) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(stage + offset));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(stage + (offset + 4 * (BN * 2))));
        const u32x2_t a = __builtin_bit_cast(u32x2_t, lo), b = __builtin_bit_cast(u32x2_t, hi);
        return u32x4_t{a.x, a.y, b.x, b.y};
    } else {
        return *reinterpret_cast<const u32x4_t*>(stage + offset);
    }
}

template <typename T, int KIND, int EPI>
struct Kernel {
    static constexpr bool A_STRIDED = KIND == XMA_GEMM_MT;
    static constexpr bool B_STRIDED = KIND != XMA_GEMM_TN;
    static constexpr int BN_OUT = EPI == XMA_EPI_SWIGLU ? BN / 2 : BN;

    OperandLoads<T> la, lb;
    int64_t red_len;
    int wave, lane;

    template <int S>
    __device__ __forceinline__ void issue(int64_t stage) {
        issue_operand(la, stage_ptr<S>(), 0, stage, stage * BK, red_len);
        issue_operand(lb, stage_ptr<S>(), OPERAND_BYTES, stage, stage * BK, red_len);
    }

    template <int S>
    __device__ __forceinline__ void compute(f32x16_t (&acc)[MI][NI]) {
        const char* stage = stage_ptr<S>();
        const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
        const int frow = lane & 31, half = lane >> 5;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4_t af[MI], bf[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const int off = A_STRIDED ? kstrided_offset(wm0 + mi * 32, kk, lane)
                                          : kcontig_offset(wm0 + mi * 32 + frow, kk, half);
                af[mi] = read_fragment<A_STRIDED>(stage, opaque(off));
            }
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int off = B_STRIDED ? kstrided_offset(wn0 + ni * 32, kk, lane)
                                          : kcontig_offset(wn0 + ni * 32 + frow, kk, half);
                bf[ni] = read_fragment<B_STRIDED>(stage, opaque(OPERAND_BYTES + off));
            }
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) Mma<T>::run(bf[ni], af[mi], acc[mi][ni]);
        }
    }

    // One pipeline step on stage s (S = s % NS): wait until at most the two younger stages are in
    // flight, meet the other waves (stage s has landed for everybody and the buffer of stage s-1 is no longer
    // read), refill that buffer with stage s+3, multiply.  The step is branch-free: stages past the end of
    // the reduction fetch the zero page, which keeps the count of loads in flight the same at every step and
    // lets the compiler see that the loop needs no other wait on vector memory.
    template <int S>
    __device__ __forceinline__ void step(int64_t s, f32x16_t (&acc)[MI][NI]) {
        wait_vmcnt<2 * LOADS_PER_STAGE>();
        block_barrier();
        issue<(S + NS - 1) % NS>(s + NS - 1);
        compute<S>(acc);
    }
};

template <typename T, int KIND, int EPI>
__global__ __launch_bounds__(THREADS) void grouped_gemm_dma_kernel(const GemmParams P) {
    using K = Kernel<T, KIND, EPI>;
    constexpr int PV = 8;
    constexpr int BN_OUT = K::BN_OUT;

    const int tid = threadIdx.x;
    K k;
    k.lane = tid & 63;
    k.wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const int row_tiles = KIND == XMA_GEMM_MT ? P.row_tiles_max * P.num_experts : P.tile_count[0];
    int row_tile, col_tile;
    if (!locate_tile(row_tiles, P.col_tiles, row_tile, col_tile)) return;

    const T* A = reinterpret_cast<const T*>(P.a);
    const T* B = reinterpret_cast<const T*>(P.b);

    int expert;
    int64_t m_begin, m_end, tile_i0 = 0, n0;
    if constexpr (KIND == XMA_GEMM_MT) {
        expert = row_tile / P.row_tiles_max;
        tile_i0 = (int64_t)(row_tile % P.row_tiles_max) * BM;
        m_begin = P.offsets[expert];
        m_end = P.offsets[expert + 1];
        k.red_len = m_end - m_begin;
        n0 = (int64_t)col_tile * BN;
    } else {
        expert = P.tile_expert[row_tile];
        m_begin = P.tile_row0[row_tile];
        const int64_t e_end = P.offsets[expert + 1];
        m_end = m_begin + BM < e_end ? m_begin + BM : e_end;
        k.red_len = P.k;
        n0 = (int64_t)col_tile * BN_OUT;
    }

    // ---- operand load plans ----
    if constexpr (KIND == XMA_GEMM_MT) {
        setup_kstrided(k.la, k.wave, k.lane, A + m_begin * P.lda + tile_i0, P.lda, P.n - tile_i0);
        setup_kstrided(k.lb, k.wave, k.lane, B + m_begin * P.ldb + n0, P.ldb, P.k - n0);
    } else {
        setup_kcontig(k.la, k.wave, k.lane, [&](int r) -> const T* {
            const int64_t p = m_begin + r;
            if (p >= m_end) return nullptr;
            const int64_t src = P.in_index ? source_row(P, p) : p;
            return A + src * P.lda;
        });
        const T* W = B + (int64_t)expert * P.b_expert_stride;
        if constexpr (KIND == XMA_GEMM_TN) {
            setup_kcontig(k.lb, k.wave, k.lane, [&](int r) -> const T* {
                int64_t n;
                if constexpr (EPI == XMA_EPI_SWIGLU) {
                    const int64_t half = P.n / 2;
                    const int64_t j = n0 + (r % BN_OUT);
                    if (j >= half) return nullptr;
                    n = r < BN_OUT ? j : half + j;
                } else {
                    n = n0 + r;
                    if (n >= P.n) return nullptr;
                }
                return W + n * P.ldb;
            });
        } else {
            setup_kstrided(k.lb, k.wave, k.lane, W + n0, P.ldb, P.n - n0);
        }
    }

    f32x16_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    // ---- pipelined main loop: the stage count is rounded up to a multiple of NS with all-zero stages ----
    const int64_t num_stages = (k.red_len + BK - 1) / BK;
    if (num_stages > 0) {
        k.template issue<0>(0);
        k.template issue<1>(1);
        k.template issue<2>(2);
        for (int64_t s = 0; s < num_stages; s += NS) {
            k.template step<0>(s, acc);
            k.template step<1>(s + 1, acc);
            k.template step<2>(s + 2, acc);
            k.template step<3>(s + 3, acc);
        }
        wait_vmcnt<0>();  // the trailing zero-page loads
    }
    block_barrier();  // every wave is done reading the stages; no load is in flight any more

    // ---- epilogue: accumulators -> LDS (stage array mi holds the 64 tile rows {wr*128 + mi*32 + 0..31}) -> HBM ----
    // MFMA result element r of lane l: tile column 8*(r/4) + 4*(l/32) + r%4 (+32*ni), tile row l%32 (+32*mi).
    // A 512-byte LDS row holds 32 chunks of 8 columns; chunk c of buffer row br sits at c ^ (br & 31).
    {
        const int wn0 = (k.wave % WAVES_N) * WN;
        const int br = (k.wave / WAVES_N) * 32 + (k.lane & 31);
        const int half = k.lane >> 5;
        auto write_rows = [&](char* buf, const f32x16_t (&a)[NI]) {
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int chunk = ((wn0 + ni * 32 + 8 * g) >> 3) ^ (br & 31);
                    *reinterpret_cast<uint2*>(buf + br * (BN * 2) + (chunk << 4) + half * 8) =
                        make_uint2(Elem<T>::pack2(a[ni][4 * g], a[ni][4 * g + 1]),
                                   Elem<T>::pack2(a[ni][4 * g + 2], a[ni][4 * g + 3]));
                }
            }
        };
        write_rows(stage_ptr<0>(), acc[0]);
        write_rows(stage_ptr<1>(), acc[1]);
        write_rows(stage_ptr<2>(), acc[2]);
        write_rows(stage_ptr<3>(), acc[3]);
    }
    __syncthreads();

    T* C = reinterpret_cast<T*>(P.c);
    constexpr int C_CHUNKS = BN / PV;  // 32
    const int cc = tid % C_CHUNKS;
    auto store_rows = [&](const char* buf, int mi) {
#pragma unroll 1
        for (int br = tid / C_CHUNKS; br < 64; br += THREADS / C_CHUNKS) {
            const int r = (br >> 5) * 128 + mi * 32 + (br & 31);
            const char* src = buf + br * (BN * 2);
            auto chunk_at = [&](int c) { return *reinterpret_cast<const uint4*>(src + ((c ^ (br & 31)) << 4)); };
            if constexpr (KIND == XMA_GEMM_MT) {
                const int64_t i = tile_i0 + r, j = n0 + cc * PV;
                if (i < P.n && j < P.k)
                    *reinterpret_cast<uint4*>(C + (int64_t)expert * P.c_expert_stride + i * P.ldc + j) = chunk_at(cc);
            } else {
                const int64_t p = m_begin + r;
                if (p >= m_end) continue;
                const int64_t orow = P.out_index ? load_index(P.out_index, P.idx_is_i64, p) : p;
                if constexpr (EPI == XMA_EPI_NONE) {
                    const int64_t n = n0 + cc * PV;
                    if (n < P.n) *reinterpret_cast<uint4*>(C + orow * P.ldc + n) = chunk_at(cc);
                } else if constexpr (EPI == XMA_EPI_SWIGLU) {
                    constexpr int HALF_CHUNKS = C_CHUNKS / 2;
                    const int64_t half_n = P.n / 2;
                    const int64_t j = n0 + (cc % HALF_CHUNKS) * PV;
                    if (j < half_n) {
                        if (P.aux) {
                            T* h = reinterpret_cast<T*>(P.aux) + p * P.ld_aux;
                            *reinterpret_cast<uint4*>(h + (cc < HALF_CHUNKS ? j : half_n + j)) = chunk_at(cc);
                        }
                        if (cc < HALF_CHUNKS) {
                            float u[PV], g[PV], o[PV];
                            Elem<T>::unpack(chunk_at(cc), u);
                            Elem<T>::unpack(chunk_at(cc + HALF_CHUNKS), g);
#pragma unroll
                            for (int q = 0; q < PV; ++q) o[q] = u[q] * (g[q] * sigmoid_f32(g[q]));
                            *reinterpret_cast<uint4*>(C + orow * P.ldc + j) = Elem<T>::pack(o);
                        }
                    }
                } else {  // XMA_EPI_SWIGLU_BWD
                    const int64_t n = n0 + cc * PV;
                    if (n < P.n) {
                        const T* h = reinterpret_cast<const T*>(P.aux) + p * P.ld_aux;
                        float u[PV], g[PV], d[PV], du[PV], dg[PV];
                        Elem<T>::unpack(*reinterpret_cast<const uint4*>(h + n), u);
                        Elem<T>::unpack(*reinterpret_cast<const uint4*>(h + P.n + n), g);
                        Elem<T>::unpack(chunk_at(cc), d);
#pragma unroll
                        for (int q = 0; q < PV; ++q) {
                            const float sg = sigmoid_f32(g[q]);
                            dg[q] = d[q] * u[q] * (sg + g[q] * sg * (1.0f - sg));
                            du[q] = d[q] * g[q] * sg;
                        }
                        *reinterpret_cast<uint4*>(C + orow * P.ldc + n) = Elem<T>::pack(du);
                        *reinterpret_cast<uint4*>(C + orow * P.ldc + P.n + n) = Elem<T>::pack(dg);
                    }
                }
            }
        }
    };
    store_rows(stage_ptr<0>(), 0);
    store_rows(stage_ptr<1>(), 1);
    store_rows(stage_ptr<2>(), 2);
    store_rows(stage_ptr<3>(), 3);
}

template <typename T, int KIND, int EPI>
static int launch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    GemmParams P;
    fill_params(a, P);
    int64_t grid;
    if (KIND == XMA_GEMM_MT) {
        P.row_tiles_max = (int32_t)ceil_div(a.n, BM);
        P.col_tiles = (int32_t)ceil_div(a.k, BN);
        grid = grid_for_tiles((int64_t)P.row_tiles_max * a.num_experts, P.col_tiles);
    } else {
        const int64_t rt = max_row_tiles(a.rows, a.num_experts, BM);
        int32_t* ws = reinterpret_cast<int32_t*>(a.workspace);
        P.tile_count = ws;
        P.tile_expert = ws + 4;
        P.tile_row0 = ws + 4 + rt;
        P.row_tiles_max = (int32_t)rt;
        const int bn_out = EPI == XMA_EPI_SWIGLU ? BN / 2 : BN;
        const int64_t n_out = EPI == XMA_EPI_SWIGLU ? a.n / 2 : a.n;
        P.col_tiles = (int32_t)ceil_div(n_out, bn_out);
        grid = grid_for_tiles(rt, P.col_tiles);
        hipLaunchKernelGGL(build_row_tiles_kernel, dim3(1), dim3(1024), 0, stream, a.expert_offsets, a.num_experts, BM,
                           ws + 4, ws + 4 + rt, ws);
    }
    XMA_REQUIRE(grid < ((int64_t)1 << 31), "xma_grouped_gemm: %lld tiles exceed the grid limit", (long long)grid);
    hipLaunchKernelGGL((grouped_gemm_dma_kernel<T, KIND, EPI>), dim3((unsigned)grid), dim3(THREADS), 0, stream, P);
    return check_launch("xma_grouped_gemm");
}

template <typename T>
static int dispatch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    switch (a.kind) {
        case XMA_GEMM_TN:
            if (a.epilogue == XMA_EPI_SWIGLU) return launch<T, XMA_GEMM_TN, XMA_EPI_SWIGLU>(a, stream);
            return launch<T, XMA_GEMM_TN, XMA_EPI_NONE>(a, stream);
        case XMA_GEMM_NN:
            if (a.epilogue == XMA_EPI_SWIGLU_BWD) return launch<T, XMA_GEMM_NN, XMA_EPI_SWIGLU_BWD>(a, stream);
            return launch<T, XMA_GEMM_NN, XMA_EPI_NONE>(a, stream);
        default:
            return launch<T, XMA_GEMM_MT, XMA_EPI_NONE>(a, stream);
    }
}

}  // namespace dma

// 16-bit element types; the weight-gradient layout only without a fused row gather (its reduction rows
// would need an index lookup per stage).
bool dma_gemm_supports(const xma_grouped_gemm_args& a) {
    if (a.dtype != XMA_BF16 && a.dtype != XMA_F16) return false;
    if (a.kind == XMA_GEMM_MT && a.in_index != nullptr) return false;
    return true;
}

int launch_dma_gemm(const xma_grouped_gemm_args& a, hipStream_t stream) {
    return a.dtype == XMA_BF16 ? dma::dispatch<bf16_t>(a, stream) : dma::dispatch<f16_t>(a, stream);
}

}  // namespace xma
