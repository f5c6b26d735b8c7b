// HBM-bound row kernels of the MoE layer on gfx950: token gather (permute) with optional
// per-row coefficient, row scatter (unpermute), top-k weighted combine / fold, and the gate
// gradient.  Rows are moved as 16-byte vectors, kRowsPerIter rows per block and iteration (one measured
// fastest on 4-8 KiB rows: many small blocks keep more requests in flight than fewer, longer ones).
#include "common.h"

namespace xma {

constexpr int kRowsPerIter = 1;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

enum RowMode { kGather = 0, kScatter = 1 };

constexpr int64_t kInfinityCacheBytes = (int64_t)256 << 20;

// 16-byte path: cols is a multiple of Elem<T>::kPerVec, strides keep rows 16-byte aligned.
template <typename T, int MODE, bool COEFF>
__global__ __launch_bounds__(256) void move_rows_vec_kernel(const T* __restrict__ src, int64_t ld_src,
                                                             T* __restrict__ dst, int64_t ld_dst,
                                                             const void* __restrict__ index, int idx_is_i64,
                                                             int64_t rows, int chunks, int fan_out,
                                                             const T* __restrict__ coeff) {
    constexpr int PV = Elem<T>::kPerVec;
    for (int64_t r0 = (int64_t)blockIdx.x * kRowsPerIter; r0 < rows; r0 += (int64_t)gridDim.x * kRowsPerIter) {
        int64_t srow[kRowsPerIter], drow[kRowsPerIter];
        float scale[kRowsPerIter];
        bool live[kRowsPerIter];  // a gathered row whose index is negative has no source and is left as it is
#pragma unroll
        for (int j = 0; j < kRowsPerIter; ++j) {
            const int64_t p = r0 + j < rows ? r0 + j : rows - 1;
            int64_t ix = index ? load_index(index, idx_is_i64, p) : p;
            live[j] = r0 + j < rows && (MODE != kGather || ix >= 0);
            if (MODE == kGather && ix < 0) ix = 0;
            srow[j] = MODE == kGather ? ix / fan_out : p;
            drow[j] = MODE == kGather ? p : ix;
            scale[j] = 1.0f;
            if constexpr (COEFF) scale[j] = Elem<T>::load(coeff + ix);
        }
        // kChunksInFlight chunks of each row requested before the first is stored
        constexpr int kChunksInFlight = 2;
        auto move = [&](int c0, int count) {
            uint4 v[kChunksInFlight][kRowsPerIter];
#pragma unroll
            for (int i = 0; i < kChunksInFlight; ++i)
#pragma unroll
                for (int j = 0; j < kRowsPerIter; ++j)
                    if (i < count) v[i][j] = load_stream(src + srow[j] * ld_src + (int64_t)(c0 + i * (int)blockDim.x) * PV);
#pragma unroll
            for (int i = 0; i < kChunksInFlight; ++i)
#pragma unroll
                for (int j = 0; j < kRowsPerIter; ++j) {
                    if (i >= count) continue;
                    if constexpr (COEFF) {
                        float f[PV];
                        Elem<T>::unpack(v[i][j], f);
#pragma unroll
                        for (int q = 0; q < PV; ++q) f[q] *= scale[j];
                        v[i][j] = Elem<T>::pack(f);
                    }
                    if (live[j]) store_stream(dst + drow[j] * ld_dst + (int64_t)(c0 + i * (int)blockDim.x) * PV, v[i][j]);
                }
        };
        int c = threadIdx.x;
        for (; c + (kChunksInFlight - 1) * (int)blockDim.x < chunks; c += kChunksInFlight * (int)blockDim.x)
            move(c, kChunksInFlight);
        for (; c < chunks; c += blockDim.x) move(c, 1);
    }
}

// element-wise path for odd widths or unaligned views
template <typename T, int MODE, bool COEFF>
__global__ __launch_bounds__(256) void move_rows_scalar_kernel(const T* __restrict__ src, int64_t ld_src,
                                                                T* __restrict__ dst, int64_t ld_dst,
                                                                const void* __restrict__ index, int idx_is_i64,
                                                                int64_t rows, int64_t cols, int fan_out,
                                                                const T* __restrict__ coeff) {
    for (int64_t p = blockIdx.x; p < rows; p += gridDim.x) {
        const int64_t ix = index ? load_index(index, idx_is_i64, p) : p;
        if (MODE == kGather && ix < 0) continue;
        const int64_t srow = MODE == kGather ? ix / fan_out : p;
        const int64_t drow = MODE == kGather ? p : ix;
        float scale = 1.0f;
        if constexpr (COEFF) scale = Elem<T>::load(coeff + ix);
        for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
            if constexpr (COEFF)
                Elem<T>::store(dst + drow * ld_dst + c, Elem<T>::load(src + srow * ld_src + c) * scale);
            else
                dst[drow * ld_dst + c] = src[srow * ld_src + c];
        }
    }
}

// inverse[index[p]] = p: who writes each destination row of a scatter (any one writer when several name the row;
// -1, set beforehand, when nobody does).  Entries outside [0, dst_rows) are ignored.
__global__ __launch_bounds__(256) void fill_minus_one_kernel(int32_t* __restrict__ inverse, int64_t dst_rows) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < dst_rows) inverse[i] = -1;
}
__global__ __launch_bounds__(256) void invert_index_kernel(const void* __restrict__ index, int idx_is_i64, int64_t rows,
                                                           int64_t dst_rows, int32_t* __restrict__ inverse) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= rows) return;
    const int64_t d = load_index(index, idx_is_i64, p);
    if (d >= 0 && d < dst_rows) inverse[d] = (int32_t)p;
}

// y[t, :] = sum_j gates[t, j] * y_exp[t*k + j, :]   (GATED) or the plain sum over j.
// STREAM: the expanded rows are read with streaming loads.  That is the faster way when they come from HBM; rows that
// the previous kernel has just written and that fit the 256 MiB Infinity Cache are served from there, and plain
// loads are faster (measured: 34 vs 37 us on 128 MiB of rows).
template <typename T, bool GATED, bool VEC, bool STREAM>
__global__ __launch_bounds__(256) void combine_kernel(const T* __restrict__ y_exp, int64_t ld_exp,
                                                       const T* __restrict__ gates, T* __restrict__ y, int64_t ld_y,
                                                       int64_t Tn, int k, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    const int64_t chunks = cols / PV;
    auto load_row_chunk = [](const T* p) {
        if constexpr (STREAM) return load_stream(p);
        else return *reinterpret_cast<const uint4*>(p);
    };
    for (int64_t t = blockIdx.x; t < Tn; t += gridDim.x) {
        const T* base = y_exp + t * k * ld_exp;
        for (int64_t c = threadIdx.x; c < chunks; c += blockDim.x) {
            float acc[PV];
#pragma unroll
            for (int q = 0; q < PV; ++q) acc[q] = 0.0f;
            int j = 0;
            if constexpr (VEC) {
                // four rows in flight per thread while there are four, then two: the walk over a token's k rows
                // is otherwise a chain of load latencies
                for (; j + 4 <= k; j += 4) {
                    uint4 v[4];
                    float g[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        v[r] = load_row_chunk(base + (int64_t)(j + r) * ld_exp + c * PV);
                        g[r] = GATED ? Elem<T>::load(gates + t * k + j + r) : 1.0f;
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float f[PV];
                        Elem<T>::unpack(v[r], f);
#pragma unroll
                        for (int q = 0; q < PV; ++q) acc[q] = fmaf(g[r], f[q], acc[q]);
                    }
                }
                for (; j + 2 <= k; j += 2) {
                    const uint4 v0 = load_row_chunk(base + (int64_t)j * ld_exp + c * PV);
                    const uint4 v1 = load_row_chunk(base + (int64_t)(j + 1) * ld_exp + c * PV);
                    float f0[PV], f1[PV];
                    Elem<T>::unpack(v0, f0);
                    Elem<T>::unpack(v1, f1);
                    const float g0 = GATED ? Elem<T>::load(gates + t * k + j) : 1.0f;
                    const float g1 = GATED ? Elem<T>::load(gates + t * k + j + 1) : 1.0f;
#pragma unroll
                    for (int q = 0; q < PV; ++q) acc[q] = fmaf(g0, f0[q], acc[q]);
#pragma unroll
                    for (int q = 0; q < PV; ++q) acc[q] = fmaf(g1, f1[q], acc[q]);
                }
            }
            for (; j < k; ++j) {
                const float g = GATED ? Elem<T>::load(gates + t * k + j) : 1.0f;
                if constexpr (VEC) {
                    const uint4 v = load_row_chunk(base + (int64_t)j * ld_exp + c * PV);
                    float f[PV];
                    Elem<T>::unpack(v, f);
#pragma unroll
                    for (int q = 0; q < PV; ++q) acc[q] = fmaf(g, f[q], acc[q]);
                } else {
                    acc[0] = fmaf(g, Elem<T>::load(base + (int64_t)j * ld_exp + c), acc[0]);
                }
            }
            if constexpr (VEC)
                *reinterpret_cast<uint4*>(y + t * ld_y + c * PV) = Elem<T>::pack(acc);
            else
                Elem<T>::store(y + t * ld_y + c, acc[0]);
        }
    }
}

// d_gates[t, j] = <y_exp[t*k + j, :], dy[t, :]>; block per token, wave per slot j.
template <typename T, bool VEC>
__global__ __launch_bounds__(1024) void gate_grad_kernel(const T* __restrict__ y_exp, int64_t ld_exp,
                                                         const T* __restrict__ dy, int64_t ld_dy,
                                                         T* __restrict__ d_gates, int64_t Tn, int k, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    const int64_t chunks = cols / PV;
    const int wave = threadIdx.x / kWaveSize;
    const int nwaves = blockDim.x / kWaveSize;
    const int lane = lane_id();
    for (int64_t t = blockIdx.x; t < Tn; t += gridDim.x) {
        for (int j = wave; j < k; j += nwaves) {
            const T* row = y_exp + (t * k + j) * ld_exp;
            const T* g = dy + t * ld_dy;
            float acc = 0.0f;
            int64_t c = lane;
            if constexpr (VEC) {
                // four chunk pairs in flight per lane
                for (; c + 3 * kWaveSize < chunks; c += 4 * kWaveSize) {
                    uint4 ra[4], rb[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        ra[r] = load_stream(row + (c + r * kWaveSize) * PV);
                        rb[r] = *reinterpret_cast<const uint4*>(g + (c + r * kWaveSize) * PV);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float a[PV], b[PV];
                        Elem<T>::unpack(ra[r], a);
                        Elem<T>::unpack(rb[r], b);
#pragma unroll
                        for (int q = 0; q < PV; ++q) acc = fmaf(a[q], b[q], acc);
                    }
                }
            }
            for (; c < chunks; c += kWaveSize) {
                if constexpr (VEC) {
                    float a[PV], b[PV];
                    Elem<T>::unpack(load_stream(row + c * PV), a);
                    Elem<T>::unpack(*reinterpret_cast<const uint4*>(g + c * PV), b);
#pragma unroll
                    for (int q = 0; q < PV; ++q) acc = fmaf(a[q], b[q], acc);
                } else {
                    acc = fmaf(Elem<T>::load(row + c), Elem<T>::load(g + c), acc);
                }
            }
            acc = wave_sum(acc);
            if (lane == 0) Elem<T>::store(d_gates + t * k + j, acc);
        }
    }
}

// One work item per block: many short blocks keep HBM busier than a capped grid of long-running ones
// (measured on the 16 GiB gather: 71 % of peak instead of 65 %); the kernels' stride loops only matter
// beyond 2^31 - 1 work items.
static unsigned row_grid(int64_t work_items) {
    const int64_t cap = 0x7fffffff;
    int64_t g = work_items < cap ? work_items : cap;
    return (unsigned)(g < 1 ? 1 : g);
}

static unsigned row_block(int64_t chunks) {
    int64_t b = ((chunks + kWaveSize - 1) / kWaveSize) * kWaveSize;
    if (b > 256) b = 256;
    if (b < kWaveSize) b = kWaveSize;
    return (unsigned)b;
}

template <typename T>
static bool vec_ok(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t cols) {
    constexpr int PV = Elem<T>::kPerVec;
    return aligned16(a) && aligned16(b) && lda % PV == 0 && ldb % PV == 0 && cols % PV == 0;
}

template <typename T, int MODE>
static void launch_move(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* index,
                        int idx_is_i64, int64_t rows, int64_t cols, int fan_out, const void* coeff,
                        hipStream_t stream) {
    constexpr int PV = Elem<T>::kPerVec;
    if (vec_ok<T>(src, ld_src, dst, ld_dst, cols)) {
        const int chunks = (int)(cols / PV);
        const dim3 grid(row_grid(ceil_div(rows, kRowsPerIter))), block(row_block(chunks));
        if (coeff)
            hipLaunchKernelGGL((move_rows_vec_kernel<T, MODE, true>), grid, block, 0, stream, (const T*)src, ld_src,
                               (T*)dst, ld_dst, index, idx_is_i64, rows, chunks, fan_out, (const T*)coeff);
        else
            hipLaunchKernelGGL((move_rows_vec_kernel<T, MODE, false>), grid, block, 0, stream, (const T*)src, ld_src,
                               (T*)dst, ld_dst, index, idx_is_i64, rows, chunks, fan_out, (const T*)nullptr);
    } else {
        const dim3 grid(row_grid(rows)), block(row_block(cols));
        if (coeff)
            hipLaunchKernelGGL((move_rows_scalar_kernel<T, MODE, true>), grid, block, 0, stream, (const T*)src, ld_src,
                               (T*)dst, ld_dst, index, idx_is_i64, rows, cols, fan_out, (const T*)coeff);
        else
            hipLaunchKernelGGL((move_rows_scalar_kernel<T, MODE, false>), grid, block, 0, stream, (const T*)src,
                               ld_src, (T*)dst, ld_dst, index, idx_is_i64, rows, cols, fan_out, (const T*)nullptr);
    }
}

}  // namespace xma

using namespace xma;

extern "C" {

int xma_gather_rows(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* index, int idx_is_i64,
                    int64_t rows, int64_t cols, int dtype, int32_t fan_out, const void* coeff, void* stream_) {
    XMA_REQUIRE(valid_dtype(dtype), "xma_gather_rows: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 0 && ld_src >= cols && ld_dst >= cols, "xma_gather_rows: bad shape");
    XMA_REQUIRE(fan_out >= 1, "xma_gather_rows: fan_out=%d must be >= 1", fan_out);
    XMA_REQUIRE(coeff == nullptr || index != nullptr, "xma_gather_rows: coeff needs an index");
    if (rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(src && dst, "xma_gather_rows: null pointer");
    XMA_DISPATCH_DTYPE(dtype, T, (launch_move<T, kGather>(src, ld_src, dst, ld_dst, index, idx_is_i64, rows, cols,
                                                          fan_out, coeff, (hipStream_t)stream_)))
    return check_launch("xma_gather_rows");
}

int xma_scatter_rows(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* index, int idx_is_i64,
                     int64_t rows, int64_t cols, int dtype, void* stream_) {
    XMA_REQUIRE(valid_dtype(dtype), "xma_scatter_rows: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 0 && ld_src >= cols && ld_dst >= cols, "xma_scatter_rows: bad shape");
    if (rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(src && dst, "xma_scatter_rows: null pointer");
    XMA_DISPATCH_DTYPE(dtype, T, (launch_move<T, kScatter>(src, ld_src, dst, ld_dst, index, idx_is_i64, rows, cols, 1,
                                                           nullptr, (hipStream_t)stream_)))
    return check_launch("xma_scatter_rows");
}

int xma_scatter_rows_ordered(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* index,
                             int idx_is_i64, int64_t rows, int64_t dst_rows, int64_t cols, int dtype, void* inverse,
                             void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_scatter_rows_ordered: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && dst_rows >= 0 && cols >= 0 && ld_src >= cols && ld_dst >= cols,
                "xma_scatter_rows_ordered: bad shape");
    XMA_REQUIRE(rows <= 0x7fffffff && dst_rows <= 0x7fffffff, "xma_scatter_rows_ordered: more than 2^31 - 1 rows");
    if (rows == 0 || dst_rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(src && dst && index && inverse, "xma_scatter_rows_ordered: null pointer");
    int32_t* inv = reinterpret_cast<int32_t*>(inverse);
    hipLaunchKernelGGL(fill_minus_one_kernel, dim3((unsigned)ceil_div(dst_rows, 256)), dim3(256), 0, stream, inv,
                       dst_rows);
    hipLaunchKernelGGL(invert_index_kernel, dim3((unsigned)ceil_div(rows, 256)), dim3(256), 0, stream, index, idx_is_i64,
                       rows, dst_rows, inv);
    XMA_DISPATCH_DTYPE(dtype, T, (launch_move<T, kGather>(src, ld_src, dst, ld_dst, inv, 0, dst_rows, cols, 1, nullptr,
                                                          stream)))
    return check_launch("xma_scatter_rows_ordered");
}

int xma_combine_topk(const void* y_exp, int64_t ld_exp, const void* gates, void* y, int64_t ld_y, int64_t T,
                     int32_t k, int64_t cols, int dtype, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_combine_topk: bad dtype %d", dtype);
    XMA_REQUIRE(T >= 0 && k >= 1 && cols >= 0 && ld_exp >= cols && ld_y >= cols, "xma_combine_topk: bad shape");
    if (T == 0 || cols == 0) return 0;
    XMA_REQUIRE(y_exp && y, "xma_combine_topk: null pointer");
#define XMA_COMBINE(G, V)                                                                                         \
    do {                                                                                                          \
        if (from_hbm)                                                                                             \
            hipLaunchKernelGGL((combine_kernel<T_, G, V, true>), grid, block, 0, stream, (const T_*)y_exp, ld_exp, \
                               (const T_*)gates, (T_*)y, ld_y, T, (int)k, cols);                                   \
        else                                                                                                      \
            hipLaunchKernelGGL((combine_kernel<T_, G, V, false>), grid, block, 0, stream, (const T_*)y_exp,       \
                               ld_exp, (const T_*)gates, (T_*)y, ld_y, T, (int)k, cols);                           \
    } while (0)
    XMA_DISPATCH_DTYPE(
        dtype, T_, const bool vec = vec_ok<T_>(y_exp, ld_exp, y, ld_y, cols);
        const bool from_hbm = T * k * cols * (int64_t)sizeof(T_) > kInfinityCacheBytes;
        const int64_t chunks = vec ? cols / Elem<T_>::kPerVec : cols;
        const dim3 grid(row_grid(T)), block(row_block(chunks));
        if (gates) {
            if (vec)
                XMA_COMBINE(true, true);
            else
                XMA_COMBINE(true, false);
        } else {
            if (vec)
                XMA_COMBINE(false, true);
            else
                XMA_COMBINE(false, false);
        })
#undef XMA_COMBINE
    return check_launch("xma_combine_topk");
}

int xma_gate_grad(const void* y_exp, int64_t ld_exp, const void* dy, int64_t ld_dy, void* d_gates, int64_t T,
                  int32_t k, int64_t cols, int dtype, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_gate_grad: bad dtype %d", dtype);
    XMA_REQUIRE(T >= 0 && k >= 1 && cols >= 0 && ld_exp >= cols && ld_dy >= cols, "xma_gate_grad: bad shape");
    if (T == 0) return 0;
    XMA_REQUIRE(y_exp && dy && d_gates, "xma_gate_grad: null pointer");
    XMA_DISPATCH_DTYPE(
        dtype, T_, const bool vec = vec_ok<T_>(y_exp, ld_exp, dy, ld_dy, cols);
        // one wave per slot of the token's k, so that no wave of the block idles
        const dim3 grid(row_grid(T)), block((unsigned)(kWaveSize * (k < 16 ? k : 16)));
        if (vec) hipLaunchKernelGGL((gate_grad_kernel<T_, true>), grid, block, 0, stream, (const T_*)y_exp, ld_exp,
                                    (const T_*)dy, ld_dy, (T_*)d_gates, T, (int)k, cols);
        else hipLaunchKernelGGL((gate_grad_kernel<T_, false>), grid, block, 0, stream, (const T_*)y_exp, ld_exp,
                                (const T_*)dy, ld_dy, (T_*)d_gates, T, (int)k, cols))
    return check_launch("xma_gate_grad");
}

}  // extern "C"
