// Pieces shared by the grouped-GEMM kernels: kernel arguments, the row-tile list that maps
// work-groups to (expert, rows) without host synchronisation, and the XCD-aware tile walk.
#pragma once

#include "common.h"

namespace xma {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;  // 16 bytes moved as ONE vector access

constexpr int kNumXcd = 8;     // accelerator complex dies, each with a private L2
constexpr int kBandTiles = 4;  // row tiles per band of the tile walk (2, 8 and 16 measured slower)

// ---- kernel arguments -----------------------------------------------------------------------------
struct GemmParams {
    const void* a;
    const void* b;
    void* c;
    void* aux;
    const int32_t* offsets;
    const void* in_index;
    const void* out_index;
    const int32_t* tile_expert;  // [row tiles] expert of each row tile (TN/NN)
    const int32_t* tile_row0;    // [row tiles] first grouped row of each row tile
    const int32_t* tile_count;   // [1] number of row tiles actually present
    int64_t lda, ldb, ldc, ld_aux, b_expert_stride, c_expert_stride;
    int64_t n, k;
    int32_t num_experts, in_fan_out, idx_is_i64;
    int32_t row_tiles_max;  // upper bound used for the grid (TN/NN); MT: row tiles per expert
    int32_t col_tiles;
    // split-K of the last, partly filled round of tiles (16-bit TN/NN kernels)
    int32_t* split_counters;  // [kSplitSlots] arrivals per split tile, zero at launch
    float* split_partials;    // [kSplitSlots][tile] fp32 accumulators of the parts
    int32_t num_cu;
    // MT: experts in descending order of their row counts, one record {expert, first row, end row, 0} per slot;
    // nullptr: slot e is expert e
    const int32_t* expert_order;
    // fused activation of the epilogue (enum Activation) and the optional per-expert bias of the forward kinds
    const void* bias;
    int64_t ld_bias;
    int32_t act;
};

// The kernels are instantiated for three epilogue shapes; the activation inside a shape is a run-time value
// (GemmParams::act), so SwiGLU and GLU, or the two backward forms, share one instantiation.
//   EPI_PLAIN     store the product (optionally through tanh-GELU, keeping the pre-activation)
//   EPI_PAIRED    TN: tile columns [0, 128) and [128, 256) are the two halves of a gated pre-activation
//   EPI_BACKWARD  NN: the product is the activation's upstream gradient; the saved pre-activation is read back
constexpr int EPI_PLAIN = 0, EPI_PAIRED = 1, EPI_BACKWARD = 2;
inline void split_epilogue(int epilogue, int& shape, int& act) {
    switch (epilogue) {
        case XMA_EPI_SWIGLU: shape = EPI_PAIRED; act = ACT_SWIGLU; break;
        case XMA_EPI_GLU: shape = EPI_PAIRED; act = ACT_GLU; break;
        case XMA_EPI_SWIGLU_BWD: shape = EPI_BACKWARD; act = ACT_SWIGLU; break;
        case XMA_EPI_GLU_BWD: shape = EPI_BACKWARD; act = ACT_GLU; break;
        case XMA_EPI_GELU_TANH: shape = EPI_PLAIN; act = ACT_GELU_TANH; break;
        case XMA_EPI_GELU_TANH_BWD: shape = EPI_BACKWARD; act = ACT_GELU_TANH; break;
        default: shape = EPI_PLAIN; act = ACT_NONE; break;
    }
}

// At most kSplitSlots (tile, part) pairs exist at a time: the split tiles are those of one round of the device.
constexpr int kSplitSlots = 256;
constexpr int kMaxSplit = 4;
constexpr int kSplitMaxRounds = 8;
constexpr int kSplitMinStages = 32;  // a part must keep this many 64-deep stages of the reduction
constexpr int64_t kSplitTileFloats = 256 * 256;
inline int64_t tile_table_bytes(int64_t row_tiles) { return ((4 + 2 * row_tiles) * (int64_t)sizeof(int32_t) + 255) / 256 * 256; }
inline int64_t split_region_bytes() {
    return kSplitSlots * (int64_t)sizeof(int32_t) + kSplitSlots * kSplitTileFloats * (int64_t)sizeof(float);
}

// The weight-gradient kind walks the experts in descending order of their row counts (ties: lower expert first), so
// that the cost of consecutive bands of tiles falls monotonically and dealing them to the XCDs forwards and backwards
// in turn (locate_tile<true>) gives every XCD about the same work however skewed the routing is.  One block;
// rank sort for up to kMaxOrderedExperts experts, natural order beyond.
constexpr int kMaxOrderedExperts = 1024;
inline int64_t expert_order_bytes(int64_t E) { return 4 * E * (int64_t)sizeof(int32_t); }
static __global__ __launch_bounds__(1024) void build_expert_order_kernel(const int32_t* __restrict__ offsets, int E,
                                                                         int32_t* __restrict__ records) {
    __shared__ int32_t count[kMaxOrderedExperts];
    if (E > kMaxOrderedExperts) {
        for (int e = threadIdx.x; e < E; e += blockDim.x) {
            records[4 * e] = e;
            records[4 * e + 1] = offsets[e];
            records[4 * e + 2] = offsets[e + 1];
            records[4 * e + 3] = 0;
        }
        return;
    }
    const int e = threadIdx.x;
    int32_t begin = 0, end = 0;
    if (e < E) {
        begin = offsets[e];
        end = offsets[e + 1];
        count[e] = end - begin;
    }
    __syncthreads();
    if (e < E) {
        const int32_t mine = end - begin;
        int slot = 0;
        for (int o = 0; o < E; ++o) slot += (count[o] > mine || (count[o] == mine && o < e)) ? 1 : 0;
        records[4 * slot] = e;
        records[4 * slot + 1] = begin;
        records[4 * slot + 2] = end;
        records[4 * slot + 3] = 0;
    }
}

// routed row p -> source row of the gathered operand (indices are < 2^31, so divide in 32 bits)
__device__ __forceinline__ int64_t source_row(const GemmParams& P, int64_t p) {
    return (int64_t)((uint32_t)load_index(P.in_index, P.idx_is_i64, p) / (uint32_t)P.in_fan_out);
}

// Row-tile list for the row-grouped kinds: expert e owns ceil(count_e / BM) consecutive tiles.
static __global__ __launch_bounds__(1024) void build_row_tiles_kernel(const int32_t* __restrict__ offsets, int E, int BM,
                                                                int32_t* __restrict__ tile_expert,
                                                                int32_t* __restrict__ tile_row0,
                                                                int32_t* __restrict__ tile_count,
                                                                int32_t* __restrict__ split_counters) {
    __shared__ int32_t part[1024];
    if (split_counters != nullptr && threadIdx.x < kSplitSlots) split_counters[threadIdx.x] = 0;
    const int per = (E + 1023) / 1024;
    const int e0 = threadIdx.x * per;
    int32_t s = 0;
    for (int i = 0; i < per; ++i) {
        const int e = e0 + i;
        if (e < E) s += (offsets[e + 1] - offsets[e] + BM - 1) / BM;
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int32_t v = threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    int32_t t = part[threadIdx.x] - s;
    for (int i = 0; i < per; ++i) {
        const int e = e0 + i;
        if (e < E) {
            const int32_t begin = offsets[e], end = offsets[e + 1];
            for (int32_t r = begin; r < end; r += BM) {
                tile_expert[t] = e;
                tile_row0[t] = r;
                ++t;
            }
        }
    }
    if (threadIdx.x == 1023) tile_count[0] = part[1023];
}


// Work-group -> (row tile, column tile).  Tiles are numbered in bands of kBandTiles row tiles x all column
// tiles, row tile fastest, so that work-groups running at the same time share A row panels and B column
// panels.  The hardware deals work-groups round-robin to the XCDs (block b runs on XCD b % 8, as that XCD's
// b / 8-th block; checked on the device), and each XCD has a private L2, so neighbouring tiles must go to
// the same XCD.  Two ways to deal the tiles:
//   SPREAD = false: XCD x takes the x-th of eight equal contiguous ranges of the tile sequence (ranges may
//     cut a band).  Balanced to one tile when every tile costs the same (row-grouped kinds).
//   SPREAD = true: every group of eight consecutive bands is dealt one band per XCD, forwards and backwards in
//     turn; spreads a run of expensive bands (the weight-gradient tiles of an overloaded expert) over all XCDs and,
//     when band costs fall monotonically, balances them.
// `row_tiles` is the number of row tiles actually present.  Returns false when this work-group has no tile.
template <bool SPREAD>
__device__ __forceinline__ bool locate_tile(int row_tiles, int col_tiles, int& row_tile, int& col_tile) {
    const int xcd = blockIdx.x % kNumXcd;
    const int local = blockIdx.x / kNumXcd;
    const int per_band = kBandTiles * col_tiles;
    int band, in_band;
    if constexpr (SPREAD) {
        // forwards over the XCDs for even groups of eight bands, backwards for odd ones
        const int group = local / per_band;
        band = group * kNumXcd + ((group & 1) ? kNumXcd - 1 - xcd : xcd);
        in_band = local % per_band;
    } else {
        const int total = row_tiles * col_tiles;
        const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
        const int tile = xcd * per_xcd + local;
        if (local >= per_xcd || tile >= total) return false;
        band = tile / per_band;
        in_band = tile - band * per_band;
    }
    const int band_first = band * kBandTiles;
    if (band_first >= row_tiles) return false;
    const int band_rows = row_tiles - band_first < kBandTiles ? row_tiles - band_first : kBandTiles;
    row_tile = band_first + in_band % band_rows;
    col_tile = in_band / band_rows;
    return col_tile < col_tiles;
}

// Row-grouped kinds with split-K of the remainder.  With T tiles on a device of C compute units the first
// floor(T / C) * C tiles fill whole rounds; the R = T mod C tiles of the last round would leave C - R units idle
// for a whole tile time, so each of them is cut along the reduction into S = min(kMaxSplit, C / R,
// stages / kSplitMinStages) parts that run side by side.  Only when the launch has fewer than kSplitMaxRounds
// rounds (the idle units of a last round matter less the more rounds there are), and only while a part keeps
// kSplitMinStages stages: every part parks a 256 KiB tile of fp32 sums in memory and the last one reads them all
// back, 40-50 k cycles or about 17 stages of the main loop (measured; reductions of 14336 and 28672 split in three
// gain 7 % and 5 % of their launches).  Work-groups are dealt per XCD as in
// locate_tile<false>: XCD x takes the x-th eighth of the whole tiles, then the x-th eighth of the parts
// (part-major, so neighbours share panels).
struct TileWork {
    int row_tile, col_tile;
    int part, parts;  // this work-group reduces stages [part * n / parts, (part + 1) * n / parts)
    int split_tile;   // index of the tile among the split ones
    int split_tiles;
};
__device__ __forceinline__ bool locate_work(int row_tiles, int col_tiles, int num_cu, int64_t stages, TileWork& w) {
    const int xcd = blockIdx.x % kNumXcd;
    const int local = blockIdx.x / kNumXcd;
    const int total = row_tiles * col_tiles;
    const int whole = total / num_cu * num_cu;  // num_cu is a multiple of kNumXcd
    const int rem = total - whole;
    int parts = rem > 0 && total < kSplitMaxRounds * num_cu ? num_cu / rem : 1;
    parts = parts > kMaxSplit ? kMaxSplit : parts;
    parts = parts > stages / kSplitMinStages ? (int)(stages / kSplitMinStages) : parts;
    parts = parts < 1 ? 1 : parts;
    const int whole_per_xcd = whole / kNumXcd;
    int tile;
    if (local < whole_per_xcd) {
        tile = xcd * whole_per_xcd + local;
        w.part = 0;
        w.parts = 1;
        w.split_tile = 0;
    } else {
        const int items = rem * parts;
        const int per_xcd = (items + kNumXcd - 1) / kNumXcd;
        const int l = local - whole_per_xcd;
        const int q = xcd * per_xcd + l;
        if (l >= per_xcd || q >= items) return false;
        w.part = q / rem;
        w.split_tile = q - w.part * rem;
        w.parts = parts;
        tile = whole + w.split_tile;
    }
    w.split_tiles = rem;
    const int per_band = kBandTiles * col_tiles;
    const int band = tile / per_band, in_band = tile - band * per_band;
    const int band_first = band * kBandTiles;
    const int band_rows = row_tiles - band_first < kBandTiles ? row_tiles - band_first : kBandTiles;
    w.row_tile = band_first + in_band % band_rows;
    w.col_tile = in_band / band_rows;
    return true;
}
// number of work-groups that covers every case of locate_work() for up to `tiles` tiles
inline int64_t grid_for_work(int64_t tiles) { return (ceil_div(tiles, kNumXcd) + kSplitSlots / kNumXcd + 1) * kNumXcd; }

// number of work-groups that covers up to `row_tiles` x `col_tiles` under either dealing of locate_tile()
inline int64_t grid_for_tiles(int64_t row_tiles, int64_t col_tiles) {
    const int64_t bands = ceil_div(row_tiles, kBandTiles);
    return ceil_div(bands, kNumXcd) * kNumXcd * kBandTiles * col_tiles;
}

inline int64_t max_row_tiles(int64_t rows, int E, int BM) { return rows / BM + E; }

// The MFMA instruction of the register-staged kernel for 16-bit types: acc(32x32) += X(32 x 16) * Y(32 x 16)^T,
// lane l supplies row l%32 and the 8 reduction elements 8*(l/32)..8*(l/32)+7 of both operands.
template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
    template <typename V>
    __device__ static __forceinline__ void run(const V& x, const V& y, f32x16_t& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, x), __builtin_bit_cast(bf16x8_t, y),
                                                      acc, 0, 0, 0);
    }
};
// The 16x16x32 form, which the LDS-DMA kernel is built on: acc(16x16) += X(16 x 32) * Y(16 x 32)^T; lane l supplies row l%16 and the 8 reduction
// elements 8*(l/16)..+7 of both operands; result register r of lane l is D[4*(l/16) + r][l%16] (rows from X).  Half the
// accumulator traffic per FLOP of the 32x32x16 form: under the device's power cap it sustains a higher clock.  Written
// as inline assembly with the accumulator tied in place: the compiler's builtin has no tied form for a four-register
// result and copies accumulators once all 256 are live.
template <typename T>
struct Mma16;
template <>
struct Mma16<bf16_t> {
    template <typename V>
    __device__ static __forceinline__ void run(const V& x, const V& y, f32x4_t& acc) {
        asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }
};
template <>
struct Mma16<f16_t> {
    template <typename V>
    __device__ static __forceinline__ void run(const V& x, const V& y, f32x4_t& acc) {
        asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }
};
template <>
struct Mma<f16_t> {
    template <typename V>
    __device__ static __forceinline__ void run(const V& x, const V& y, f32x16_t& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, x), __builtin_bit_cast(f16x8_t, y),
                                                     acc, 0, 0, 0);
    }
};
template <>
struct Mma<float> {
    // a 16-byte fragment holds 4 reduction steps per lane half; one 32x32x2 MFMA per component
    __device__ static __forceinline__ void run(const uint4& x, const uint4& y, f32x16_t& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(x.x), __uint_as_float(y.x), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(x.y), __uint_as_float(y.y), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(x.z), __uint_as_float(y.z), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(x.w), __uint_as_float(y.w), acc, 0, 0, 0);
    }
};

// Fills the fields of GemmParams that do not depend on the tile shape.
void fill_params(const xma_grouped_gemm_args& a, GemmParams& P);

// The LDS-DMA pipelined kernel for 16-bit element types (grouped_gemm_dma.hip).
bool dma_gemm_supports(const xma_grouped_gemm_args& a);
int launch_dma_gemm(const xma_grouped_gemm_args& a, hipStream_t stream);

}  // namespace xma
