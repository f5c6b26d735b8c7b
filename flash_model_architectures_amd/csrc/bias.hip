// Per-expert bias of the expert projections: y[row, :] += bias[expert(row), :] after a projection, and
// its gradient d_bias[e, :] = sum of the grouped gradient rows of expert e.  The reference supports
// biases only on its torch path (F.linear(x, W[e], bias[e]), xma/layers/moe/__init__.py:103-106) and
// asserts them away on its kernel path (:54,79).  Both kernels are plain HBM streams.
#include "common.h"

namespace xma {

constexpr int kBiasRowsPerBlock = 8;

// Block = 8 rows x up to 32 column chunks per pass; row p is routed row p, written at out_index[p] (or p).
template <typename T, bool VEC, typename SeT>
__global__ __launch_bounds__(256) void add_expert_bias_kernel(T* __restrict__ y, int64_t ld_y,
                                                               const T* __restrict__ bias, int64_t ld_bias,
                                                               const SeT* __restrict__ expert_of_row,
                                                               const void* __restrict__ out_index, int idx_is_i64,
                                                               int64_t rows, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    const int64_t chunks = cols / PV;
    const int cl = threadIdx.x % 32, rl = threadIdx.x / 32;
    for (int64_t p0 = (int64_t)blockIdx.x * kBiasRowsPerBlock; p0 < rows; p0 += (int64_t)gridDim.x * kBiasRowsPerBlock) {
        const int64_t p = p0 + rl;
        if (p >= rows) continue;
        const int64_t e = (int64_t)expert_of_row[p];
        const int64_t r = out_index ? load_index(out_index, idx_is_i64, p) : p;
        T* row = y + r * ld_y;
        const T* b = bias + e * ld_bias;
        for (int64_t c = cl; c < chunks; c += 32) {
            if constexpr (VEC) {
                float a[PV], v[PV];
                Elem<T>::unpack(load_stream(row + c * PV), a);
                Elem<T>::unpack(*reinterpret_cast<const uint4*>(b + c * PV), v);
#pragma unroll
                for (int q = 0; q < PV; ++q) a[q] += v[q];
                store_stream(row + c * PV, Elem<T>::pack(a));
            } else {
                Elem<T>::store(row + c, Elem<T>::load(row + c) + Elem<T>::load(b + c));
            }
        }
    }
}

// Block (x = column block of 32 chunks, y = expert): 32 row lanes walk the expert's rows in order, each
// keeps fp32 partial sums of its chunk, the lanes are added in lane order through LDS.  The order of the
// additions is fixed, so the result is reproducible.
template <typename T, bool VEC>
__global__ __launch_bounds__(1024) void expert_colsum_kernel(const T* __restrict__ src, int64_t ld,
                                                              const int32_t* __restrict__ offsets,
                                                              T* __restrict__ out, int64_t ld_out, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    __shared__ float part[32][32 * PV + 1];
    const int cl = threadIdx.x % 32, rl = threadIdx.x / 32;
    const int e = blockIdx.y;
    const int64_t chunk = (int64_t)blockIdx.x * 32 + cl;
    const int64_t chunks = cols / PV;
    const int64_t begin = offsets[e], end = offsets[e + 1];
    float acc[PV];
#pragma unroll
    for (int q = 0; q < PV; ++q) acc[q] = 0.0f;
    if (chunk < chunks) {
        for (int64_t r = begin + rl; r < end; r += 32) {
            if constexpr (VEC) {
                float a[PV];
                Elem<T>::unpack(load_stream(src + r * ld + chunk * PV), a);
#pragma unroll
                for (int q = 0; q < PV; ++q) acc[q] += a[q];
            } else {
                acc[0] += Elem<T>::load(src + r * ld + chunk);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < PV; ++q) part[rl][cl * PV + q] = acc[q];
    __syncthreads();
    if (rl == 0 && chunk < chunks) {
        float total[PV];
#pragma unroll
        for (int q = 0; q < PV; ++q) total[q] = 0.0f;
        for (int i = 0; i < 32; ++i)
#pragma unroll
            for (int q = 0; q < PV; ++q) total[q] += part[i][cl * PV + q];
        T* dst = out + (int64_t)e * ld_out + chunk * PV;
        if constexpr (VEC) {
            *reinterpret_cast<uint4*>(dst) = Elem<T>::pack(total);
        } else {
            Elem<T>::store(dst, total[0]);
        }
    }
}

}  // namespace xma

using namespace xma;

extern "C" {

int xma_add_expert_bias(void* y, int64_t ld_y, const void* bias, int64_t ld_bias, const void* expert_of_row,
                        int se_is_i64, const void* out_index, int idx_is_i64, int64_t rows, int64_t cols, int dtype,
                        void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_add_expert_bias: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 0 && ld_y >= cols && ld_bias >= cols, "xma_add_expert_bias: bad shape");
    if (rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(y && bias && expert_of_row, "xma_add_expert_bias: null pointer");
    const int64_t blocks = ceil_div(rows, kBiasRowsPerBlock);
    const dim3 grid((unsigned)(blocks < 256 * 16 ? blocks : 256 * 16)), block(256);
#define XMA_BIAS_LAUNCH(VEC, SeT)                                                                                     \
    hipLaunchKernelGGL((add_expert_bias_kernel<T_, VEC, SeT>), grid, block, 0, stream, (T_*)y, ld_y, (const T_*)bias, \
                       ld_bias, (const SeT*)expert_of_row, out_index, idx_is_i64, rows, cols)
    XMA_DISPATCH_DTYPE(
        dtype, T_,
        const bool vec = aligned16(y) && aligned16(bias) && ld_y % Elem<T_>::kPerVec == 0 &&
                         ld_bias % Elem<T_>::kPerVec == 0 && cols % Elem<T_>::kPerVec == 0;
        if (vec) {
            if (se_is_i64) XMA_BIAS_LAUNCH(true, int64_t);
            else XMA_BIAS_LAUNCH(true, int32_t);
        } else {
            if (se_is_i64) XMA_BIAS_LAUNCH(false, int64_t);
            else XMA_BIAS_LAUNCH(false, int32_t);
        })
#undef XMA_BIAS_LAUNCH
    return check_launch("xma_add_expert_bias");
}

int xma_expert_colsum(const void* src, int64_t ld, const int32_t* expert_offsets, int32_t num_experts, int64_t cols,
                      void* out, int64_t ld_out, int dtype, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_expert_colsum: bad dtype %d", dtype);
    XMA_REQUIRE(num_experts >= 1 && num_experts <= 65535 && cols >= 0 && ld >= cols && ld_out >= cols,
                "xma_expert_colsum: bad shape");
    if (cols == 0) return 0;
    XMA_REQUIRE(src && expert_offsets && out, "xma_expert_colsum: null pointer");
    XMA_DISPATCH_DTYPE(
        dtype, T_,
        const bool vec = aligned16(src) && aligned16(out) && ld % Elem<T_>::kPerVec == 0 &&
                         ld_out % Elem<T_>::kPerVec == 0 && cols % Elem<T_>::kPerVec == 0;
        const int64_t chunks = vec ? cols / Elem<T_>::kPerVec : cols;
        const dim3 grid((unsigned)ceil_div(chunks, 32), (unsigned)num_experts), block(1024);
        if (vec) hipLaunchKernelGGL((expert_colsum_kernel<T_, true>), grid, block, 0, stream, (const T_*)src, ld,
                                    expert_offsets, (T_*)out, ld_out, cols);
        else hipLaunchKernelGGL((expert_colsum_kernel<T_, false>), grid, block, 0, stream, (const T_*)src, ld,
                                expert_offsets, (T_*)out, ld_out, cols))
    return check_launch("xma_expert_colsum");
}

}  // extern "C"
