// Ragged (per-expert) GEMM for 16-bit element types on gfx950, built around the LDS-DMA load path
// (global_load_lds_dwordx4): tiles travel L2 -> LDS without passing through registers, several
// stages are kept in LDS so that loads stay in flight while a stage is multiplied, and operands whose
// reduction index is strided in HBM are fetched in their HBM layout and transposed by the LDS read
// itself (ds_read_b64_tr_b16).
//
// Tile 256 x 256 per work-group, 8 waves as 2 x 4, each wave 128 x 64 (4 x 2 MFMA 32x32x16 tiles).
//
// LDS is a pool of four 32 KiB slabs; the pipeline policy Pipe32x4 keeps four stages of 32 reduction
// elements in them, one slab each (A tile | B tile), with three stages of loads in flight.  (A variant
// with 64-deep blocks rotating through five slabs, so that every DMA instruction asks for whole 128-byte
// lines, measured the same or slower on the layer's shapes and was dropped.)
// Tile layouts inside a slab:
//   K-contiguous operand (A in TN/NN, W in TN): [256 tile rows][BK k]; the 16-byte chunks of a row are
//     XOR-swizzled by the row number so that the 16 rows a quarter-wave reads in one ds_read_b128 cover all
//     64 banks.
//   K-strided operand (W in NN, both operands in MT): [BK k][256 tile rows], 512 bytes per k row; chunk c
//     of k row r sits at c ^ ((r & 3) << 2), so that the four k rows one transposing read touches fall
//     into different bank groups.
// A DMA load writes lane l's 16 bytes at (wave-uniform LDS base) + 16*l, so the swizzles are applied
// by choosing which HBM chunk each lane fetches.  Masked rows / reduction tails are fetched from a
// 16-byte page of zeros, which keeps every lane active and the outstanding-load count uniform.
#include "grouped_gemm_common.h"

namespace xma {
namespace dma {

constexpr int BM = 256, BN = 256, THREADS = 512;
constexpr int WAVES_N = 4, WM = 128, WN = 64, MI = WM / 32, NI = WN / 32;
constexpr int SLAB_BYTES = 32768;
static_assert(BM == BN, "both operands use the same tile height");

__shared__ __attribute__((aligned(1024))) char slab0[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab1[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab2[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab3[SLAB_BYTES];

// The slabs are distinct arrays on purpose: the compiler can then prove that a fragment read of
// one slab does not alias the DMA writes still in flight to the others, and does not drain them.
template <int I>
__device__ __forceinline__ char* slab() {
    static_assert(I >= 0 && I < 4, "slab index");
    if constexpr (I == 0) return slab0;
    if constexpr (I == 1) return slab1;
    if constexpr (I == 2) return slab2;
    return slab3;
}

__device__ __attribute__((aligned(16))) uint32_t g_zero_page[4];  // zero-initialised

typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
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

// LDS accesses add ONE integer byte offset to a slab, and the variable part of the offset is passed
// through opaque() so that the optimiser cannot split it into a chain of partial sums: the compiler
// attaches the "this access belongs to slab X" information it needs to keep DMA loads to the other
// slabs in flight only to accesses whose address is a short derivation from the array.
__device__ __forceinline__ int opaque(int v) {
    asm("" : "+v"(v));
    return v;
}

// ---- tile geometry for a stage depth of BK reduction elements ---------------------------------------
template <int BK>
struct Geometry {
    static constexpr int CPR = BK / 8;            // 16-byte chunks per K-contiguous row
    static constexpr int ROW_BYTES = BK * 2;
    static constexpr int ROWS_PER_LOAD = 64 / CPR;  // tile rows one DMA instruction covers
    static constexpr int LOADS = BK / 16;         // DMA instructions per wave, operand and stage
    static constexpr int TILE_BYTES = BM * BK * 2;
    static_assert(BK == 32 || BK == 64, "stage depth");

    __device__ static __forceinline__ int swizzle(int row) { return BK == 32 ? (row >> 2) & 3 : (row >> 1) & 7; }

    // K-contiguous tile: byte offset of the fragment (row, reduction elements kk*16 + 8*half .. +7)
    __device__ static __forceinline__ int kcontig_offset(int row, int kk, int half) {
        return row * ROW_BYTES + (((2 * kk + half) ^ swizzle(row)) << 4);
    }
    // K-strided tile: byte offset of the first of the two transposing reads of the fragment
    // (tile rows col0..col0+31, reduction elements kk*16 .. +15).  Within each 16-lane group the
    // instruction hands lane i the i-th 16-bit element of four 16-element rows, where row j is assembled
    // from the 8-byte pieces addressed by lanes 4j..4j+3.  So lane i addresses (k row i/4, columns
    // 4*(i%4)..+3) and receives four consecutive k of column i; a second read four k rows further down
    // completes the eight reduction elements of the MFMA operand.
    __device__ static __forceinline__ int kstrided_offset(int col0, int kk, int lane) {
        const int i = lane & 15, group = lane >> 4;
        const int col = col0 + 16 * (group & 1) + 4 * (i & 3);
        const int krow0 = kk * 16 + 8 * (group >> 1) + (i >> 2);
        const int chunk = (col >> 3) ^ ((krow0 & 3) << 2);  // (krow0 + 4) & 3 == krow0 & 3
        return krow0 * (BN * 2) + (chunk << 4) + ((col & 4) << 1);
    }
};

template <bool STRIDED>
__device__ __forceinline__ u32x4_t read_fragment(const char* slab_base, int offset) {
    if constexpr (STRIDED) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(slab_base + offset));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(slab_base + (offset + 4 * (BN * 2))));
        const u32x2_t a = __builtin_bit_cast(u32x2_t, lo), b = __builtin_bit_cast(u32x2_t, hi);
        return u32x4_t{a.x, a.y, b.x, b.y};
    } else {
        return *reinterpret_cast<const u32x4_t*>(slab_base + offset);
    }
}

// ---- per-thread DMA plan of one operand ---------------------------------------------------------------
template <typename T, int BK>
struct OperandLoads {
    static constexpr int LOADS = Geometry<BK>::LOADS;
    const T* ptr[LOADS];  // HBM address of this lane's chunk in stage 0 (or the zero page)
    int64_t step;         // elements to advance per stage
    int32_t red[LOADS];   // reduction index covered by the lane in stage 0 (chunk start or k row)
    bool valid[LOADS];    // false: always the zero page (row / column outside the operand)
    int lds_off[LOADS];   // byte offset of the wave's 1 KiB destination inside the operand's LDS tile

    // K-contiguous layout: DMA instruction i of wave w fills tile rows [R*(8i + w), +R), R = ROWS_PER_LOAD:
    // lane l -> row + l/CPR, physical chunk l%CPR.  row_fn(tile row) returns the HBM row base or nullptr.
    template <typename RowFn>
    __device__ __forceinline__ void setup_kcontig(int wave, int lane, RowFn row_fn) {
        using G = Geometry<BK>;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int row0 = (i * 8 + wave) * G::ROWS_PER_LOAD;
            const int row = row0 + lane / G::CPR;
            const int chunk = (lane % G::CPR) ^ G::swizzle(row);  // logical chunk stored at physical position
            const T* base = row_fn(row);
            valid[i] = base != nullptr;
            ptr[i] = valid[i] ? base + chunk * 8 : reinterpret_cast<const T*>(g_zero_page);
            red[i] = chunk * 8;
            lds_off[i] = row0 * G::ROW_BYTES;
        }
        step = BK;
    }

    // K-strided layout: DMA instruction i of wave w fills k rows {2*(8i + w), +1}: lane l -> k row + l/32,
    // physical chunk l%32.  `base` points at (reduction row 0, first tile column); `cols_left` = number of
    // valid columns from there; ld = row stride.
    __device__ __forceinline__ void setup_kstrided(int wave, int lane, const T* base, int64_t ld, int64_t cols_left) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int krow0 = (i * 8 + wave) * 2;
            const int krow = krow0 + (lane >> 5);
            const int chunk = (lane & 31) ^ ((krow & 3) << 2);
            valid[i] = chunk * 8 < cols_left;
            ptr[i] = valid[i] ? base + (int64_t)krow * ld + chunk * 8 : reinterpret_cast<const T*>(g_zero_page);
            red[i] = krow;
            lds_off[i] = krow0 * (BN * 2);
        }
        step = (int64_t)BK * ld;
    }

    // Issue this wave's loads for the stage `stage` into the tile at slab_base + tile_off.
    __device__ __forceinline__ void issue(char* slab_base, int tile_off, int64_t stage, int64_t red_len) const {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const bool ok = valid[i] && (stage * BK + red[i] < red_len);
            const T* src = ok ? ptr[i] + stage * step : reinterpret_cast<const T*>(g_zero_page);
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(src),
                                             XMA_LDS(slab_base + (tile_off + lds_off[i])), 16, 0, 0);
        }
    }
};

// ---- pipeline policies --------------------------------------------------------------------------------------
// A policy names, for every position P of its unrolled cycle, the slab and offset of the A and B tiles
// that step P multiplies, what the step loads, and how many younger DMA instructions may stay in flight
// when the step starts.
struct Pipe32x4 {
    static constexpr int BK = 32, CYCLE = 4;
    static constexpr int WAIT = 2 * 2 * Geometry<BK>::LOADS;  // two younger stages, two operands each
    template <int P> struct At {
        static constexpr int A_SLAB = P, A_OFF = 0, B_SLAB = P, B_OFF = Geometry<BK>::TILE_BYTES;
    };
    template <typename K> __device__ static __forceinline__ void prologue(K& k) {
        k.template issue_a<0>(0); k.template issue_b<0>(0);
        k.template issue_a<1>(1); k.template issue_b<1>(1);
        k.template issue_a<2>(2); k.template issue_b<2>(2);
    }
    // step s refills the slab that step s-1 released with stage s+3
    template <int P, typename K> __device__ static __forceinline__ void refill(K& k, int64_t s) {
        k.template issue_a<(P + 3) % CYCLE>(s + 3);
        k.template issue_b<(P + 3) % CYCLE>(s + 3);
    }
};

template <typename T, int KIND, int EPI, typename Pipe>
struct Kernel {
    static constexpr int BK = Pipe::BK;
    using G = Geometry<BK>;
    static constexpr bool A_STRIDED = KIND == XMA_GEMM_MT;
    static constexpr bool B_STRIDED = KIND != XMA_GEMM_TN;
    static constexpr int BN_OUT = EPI == XMA_EPI_SWIGLU ? BN / 2 : BN;

    OperandLoads<T, BK> la, lb;
    int64_t red_len;
    int wave, lane;
    int a_off[4], b_off[4];  // variable parts of the fragment offsets (see fragment_offsets)

    template <int P> __device__ __forceinline__ void issue_a(int64_t stage) {
        la.issue(slab<Pipe::template At<P>::A_SLAB>(), Pipe::template At<P>::A_OFF, stage, red_len);
    }
    template <int P> __device__ __forceinline__ void issue_b(int64_t stage) {
        lb.issue(slab<Pipe::template At<P>::B_SLAB>(), Pipe::template At<P>::B_OFF, stage, red_len);
    }

    // Byte offsets of this lane's fragments inside an operand tile.  Only the part that is not a
    // compile-time constant goes through opaque(): for the K-contiguous layout the tile-row block adds a
    // constant (32 rows, same swizzle), for the K-strided layout the k16 step does (16 k rows = 8 KiB).
    template <bool STRIDED, int BLOCKS>
    __device__ __forceinline__ void fragment_offsets(int row0, int (&var)[4]) const {
        if constexpr (STRIDED) {
#pragma unroll
            for (int b = 0; b < BLOCKS; ++b) var[b] = opaque(G::kstrided_offset(row0 + b * 32, 0, lane));
        } else {
#pragma unroll
            for (int kk = 0; kk < BK / 16; ++kk) var[kk] = opaque(G::kcontig_offset(row0 + (lane & 31), kk, lane >> 5));
        }
    }
    template <bool STRIDED>
    __device__ static __forceinline__ int fragment_offset(const int (&var)[4], int block, int kk) {
        return STRIDED ? var[block] + kk * (16 * BN * 2) : var[kk] + block * (32 * G::ROW_BYTES);
    }
    __device__ __forceinline__ void init_fragments() {
        fragment_offsets<A_STRIDED, MI>((wave / WAVES_N) * WM, a_off);
        fragment_offsets<B_STRIDED, NI>((wave % WAVES_N) * WN, b_off);
    }

    template <int P>
    __device__ __forceinline__ void compute(f32x16_t (&acc)[MI][NI]) {
        using At = typename Pipe::template At<P>;
        const char* ta = slab<At::A_SLAB>();
        const char* tb = slab<At::B_SLAB>();
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4_t af[MI], bf[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                af[mi] = read_fragment<A_STRIDED>(ta, At::A_OFF + fragment_offset<A_STRIDED>(a_off, mi, kk));
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
                bf[ni] = read_fragment<B_STRIDED>(tb, At::B_OFF + fragment_offset<B_STRIDED>(b_off, ni, kk));
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) Mma<T>::run(bf[ni], af[mi], acc[mi][ni]);
        }
    }

    // One pipeline step at cycle position P on stage s: wait until only the younger loads named by the
    // policy are in flight, meet the other waves (stage s has landed for everybody and the slabs of stage
    // s-1 are no longer read), refill the released slabs, multiply.  A step is branch-free: stages past the
    // end of the reduction fetch the zero page, which keeps the count of loads in flight the same at every
    // step and lets the compiler see that the loop needs no other wait on vector memory.
    template <int P>
    __device__ __forceinline__ void step(int64_t s, f32x16_t (&acc)[MI][NI]) {
        wait_vmcnt<Pipe::WAIT>();
        block_barrier();
        Pipe::template refill<P>(*this, s);
        compute<P>(acc);
    }

    template <int P>
    __device__ __forceinline__ void steps_from(int64_t s, int64_t count, f32x16_t (&acc)[MI][NI]) {
        if constexpr (P < Pipe::CYCLE) {
            if (P < count) {
                step<P>(s + P, acc);
                steps_from<P + 1>(s, count, acc);
            }
        }
    }
    template <int P>
    __device__ __forceinline__ void full_cycle(int64_t s, f32x16_t (&acc)[MI][NI]) {
        if constexpr (P < Pipe::CYCLE) {
            step<P>(s + P, acc);
            full_cycle<P + 1>(s, acc);
        }
    }

    __device__ __forceinline__ void run(f32x16_t (&acc)[MI][NI]) {
        const int64_t num_stages = (red_len + BK - 1) / BK;
        if (num_stages > 0) {
            Pipe::prologue(*this);
            int64_t s = 0;
            for (; s + Pipe::CYCLE <= num_stages; s += Pipe::CYCLE) full_cycle<0>(s, acc);
            steps_from<0>(s, num_stages - s, acc);  // fewer than CYCLE steps remain
            wait_vmcnt<0>();                         // the trailing zero-page loads
        }
        block_barrier();  // every wave is done reading the slabs; no load is in flight any more
    }
};

template <typename T, int KIND, int EPI, typename Pipe>
__global__ __launch_bounds__(THREADS) void grouped_gemm_dma_kernel(const GemmParams P) {
    using K = Kernel<T, KIND, EPI, Pipe>;
    constexpr int PV = 8;
    constexpr int BN_OUT = K::BN_OUT;

    const int tid = threadIdx.x;
    K k;
    k.lane = tid & 63;
    k.wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const int row_tiles = KIND == XMA_GEMM_MT ? P.row_tiles_max * P.num_experts : P.tile_count[0];
    int row_tile, col_tile;
    if (!locate_tile<XMA_SPREAD(KIND)>(row_tiles, P.col_tiles, row_tile, col_tile)) return;

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
        k.la.setup_kstrided(k.wave, k.lane, A + m_begin * P.lda + tile_i0, P.lda, P.n - tile_i0);
        k.lb.setup_kstrided(k.wave, k.lane, B + m_begin * P.ldb + n0, P.ldb, P.k - n0);
    } else {
        k.la.setup_kcontig(k.wave, k.lane, [&](int r) -> const T* {
            const int64_t p = m_begin + r;
            if (p >= m_end) return nullptr;
            const int64_t src = P.in_index ? source_row(P, p) : p;
            return A + src * P.lda;
        });
        const T* W = B + (int64_t)expert * P.b_expert_stride;
        if constexpr (KIND == XMA_GEMM_TN) {
            k.lb.setup_kcontig(k.wave, k.lane, [&](int r) -> const T* {
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
            k.lb.setup_kstrided(k.wave, k.lane, W + n0, P.ldb, P.n - n0);
        }
    }
    k.init_fragments();

    f32x16_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    k.run(acc);

    // ---- epilogue: accumulators -> LDS (slab mi holds the 64 tile rows {wr*128 + mi*32 + 0..31}) -> HBM ----
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
        write_rows(slab<0>(), acc[0]);
        write_rows(slab<1>(), acc[1]);
        write_rows(slab<2>(), acc[2]);
        write_rows(slab<3>(), acc[3]);
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
                            for (int q = 0; q < PV; ++q) o[q] = u[q] * (g[q] * sigmoid_fast(g[q]));
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
                            const float sg = sigmoid_fast(g[q]);
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
    store_rows(slab<0>(), 0);
    store_rows(slab<1>(), 1);
    store_rows(slab<2>(), 2);
    store_rows(slab<3>(), 3);
}

template <typename T, int KIND, int EPI, typename Pipe>
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
    hipLaunchKernelGGL((grouped_gemm_dma_kernel<T, KIND, EPI, Pipe>), dim3((unsigned)grid), dim3(THREADS), 0, stream, P);
    return check_launch("xma_grouped_gemm");
}

template <typename T>
static int dispatch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    using Pipe = Pipe32x4;
    switch (a.kind) {
        case XMA_GEMM_TN:
            if (a.epilogue == XMA_EPI_SWIGLU) return launch<T, XMA_GEMM_TN, XMA_EPI_SWIGLU, Pipe>(a, stream);
            return launch<T, XMA_GEMM_TN, XMA_EPI_NONE, Pipe>(a, stream);
        case XMA_GEMM_NN:
            if (a.epilogue == XMA_EPI_SWIGLU_BWD) return launch<T, XMA_GEMM_NN, XMA_EPI_SWIGLU_BWD, Pipe>(a, stream);
            return launch<T, XMA_GEMM_NN, XMA_EPI_NONE, Pipe>(a, stream);
        default:
            return launch<T, XMA_GEMM_MT, XMA_EPI_NONE, Pipe>(a, stream);
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
