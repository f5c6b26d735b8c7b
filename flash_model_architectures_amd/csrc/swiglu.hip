// SwiGLU forward / backward on gfx950: y = up * gate * sigmoid(gate), evaluated in fp32.
// Operands are 2-D with independent row strides so that the halves of a packed [rows, 2*cols]
// tensor can be passed as views.  16-byte vectors along the row, a 64x4 thread block covering
// 64 vectors of 4 rows, two row groups in flight per thread.
#include "common.h"

namespace xma {

__device__ __forceinline__ float swiglu_f(float g, float u) { return u * (g * sigmoid_f32(g)); }

__device__ __forceinline__ void swiglu_b(float g, float u, float dy, float& dg, float& du) {
    const float s = sigmoid_f32(g);
    dg = dy * u * (s + g * s * (1.0f - s));
    du = dy * g * s;
}

constexpr int kRowUnroll = 2;

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ gate, int64_t ld_g,
                                                          const T* __restrict__ up, int64_t ld_u, T* __restrict__ y,
                                                          int64_t ld_y, int64_t rows, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    const int64_t chunks = cols / PV;
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= chunks) return;
    const int64_t row_step = (int64_t)gridDim.y * blockDim.y;
    for (int64_t r0 = (int64_t)blockIdx.y * blockDim.y + threadIdx.y; r0 < rows; r0 += row_step * kRowUnroll) {
        if constexpr (VEC) {
            uint4 gv[kRowUnroll], uv[kRowUnroll];
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step < rows ? r0 + j * row_step : r0;
                gv[j] = load_stream(gate + r * ld_g + c * PV);
                uv[j] = load_stream(up + r * ld_u + c * PV);
            }
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step;
                if (r >= rows) break;
                float g[PV], u[PV], o[PV];
                Elem<T>::unpack(gv[j], g);
                Elem<T>::unpack(uv[j], u);
#pragma unroll
                for (int q = 0; q < PV; ++q) o[q] = swiglu_f(g[q], u[q]);
                store_stream(y + r * ld_y + c * PV, Elem<T>::pack(o));
            }
        } else {
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step;
                if (r >= rows) break;
                Elem<T>::store(y + r * ld_y + c, swiglu_f(Elem<T>::load(gate + r * ld_g + c), Elem<T>::load(up + r * ld_u + c)));
            }
        }
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ gate, int64_t ld_g,
                                                          const T* __restrict__ up, int64_t ld_u,
                                                          const T* __restrict__ dy, int64_t ld_dy, T* __restrict__ dgate,
                                                          int64_t ld_dg, T* __restrict__ dup, int64_t ld_du,
                                                          int64_t rows, int64_t cols) {
    constexpr int PV = VEC ? Elem<T>::kPerVec : 1;
    const int64_t chunks = cols / PV;
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= chunks) return;
    const int64_t row_step = (int64_t)gridDim.y * blockDim.y;
    for (int64_t r0 = (int64_t)blockIdx.y * blockDim.y + threadIdx.y; r0 < rows; r0 += row_step * kRowUnroll) {
        if constexpr (VEC) {
            uint4 gv[kRowUnroll], uv[kRowUnroll], dv[kRowUnroll];
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step < rows ? r0 + j * row_step : r0;
                gv[j] = load_stream(gate + r * ld_g + c * PV);
                uv[j] = load_stream(up + r * ld_u + c * PV);
                dv[j] = load_stream(dy + r * ld_dy + c * PV);
            }
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step;
                if (r >= rows) break;
                float g[PV], u[PV], d[PV], og[PV], ou[PV];
                Elem<T>::unpack(gv[j], g);
                Elem<T>::unpack(uv[j], u);
                Elem<T>::unpack(dv[j], d);
#pragma unroll
                for (int q = 0; q < PV; ++q) swiglu_b(g[q], u[q], d[q], og[q], ou[q]);
                store_stream(dgate + r * ld_dg + c * PV, Elem<T>::pack(og));
                store_stream(dup + r * ld_du + c * PV, Elem<T>::pack(ou));
            }
        } else {
#pragma unroll
            for (int j = 0; j < kRowUnroll; ++j) {
                const int64_t r = r0 + j * row_step;
                if (r >= rows) break;
                float og, ou;
                swiglu_b(Elem<T>::load(gate + r * ld_g + c), Elem<T>::load(up + r * ld_u + c),
                         Elem<T>::load(dy + r * ld_dy + c), og, ou);
                Elem<T>::store(dgate + r * ld_dg + c, og);
                Elem<T>::store(dup + r * ld_du + c, ou);
            }
        }
    }
}

template <typename T>
static bool all_vec(int64_t cols, std::initializer_list<const void*> ptrs, std::initializer_list<int64_t> lds) {
    constexpr int PV = Elem<T>::kPerVec;
    if (cols % PV) return false;
    for (const void* p : ptrs)
        if (!aligned16(p)) return false;
    for (int64_t ld : lds)
        if (ld % PV) return false;
    return true;
}

static void swiglu_grid(int64_t rows, int64_t chunks, dim3& grid, dim3& block) {
    block = dim3(64, 4);
    int64_t gy = ceil_div(rows, 4 * kRowUnroll);
    if (gy > 16384) gy = 16384;
    grid = dim3((unsigned)ceil_div(chunks, 64), (unsigned)(gy < 1 ? 1 : gy));
}

}  // namespace xma

using namespace xma;

extern "C" {

int xma_swiglu_forward(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y, int64_t ld_y,
                       int64_t rows, int64_t cols, int dtype, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_swiglu_forward: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 0 && ld_gate >= cols && ld_up >= cols && ld_y >= cols,
                "xma_swiglu_forward: bad shape");
    if (rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(gate && up && y, "xma_swiglu_forward: null pointer");
    XMA_DISPATCH_DTYPE(
        dtype, T, const bool vec = all_vec<T>(cols, {gate, up, y}, {ld_gate, ld_up, ld_y}); dim3 grid, block;
        swiglu_grid(rows, vec ? cols / Elem<T>::kPerVec : cols, grid, block);
        if (vec) hipLaunchKernelGGL((swiglu_fwd_kernel<T, true>), grid, block, 0, stream, (const T*)gate, ld_gate,
                                    (const T*)up, ld_up, (T*)y, ld_y, rows, cols);
        else hipLaunchKernelGGL((swiglu_fwd_kernel<T, false>), grid, block, 0, stream, (const T*)gate, ld_gate,
                                (const T*)up, ld_up, (T*)y, ld_y, rows, cols))
    return check_launch("xma_swiglu_forward");
}

int xma_swiglu_backward(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, const void* dy,
                        int64_t ld_dy, void* d_gate, int64_t ld_dgate, void* d_up, int64_t ld_dup, int64_t rows,
                        int64_t cols, int dtype, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_swiglu_backward: bad dtype %d", dtype);
    XMA_REQUIRE(rows >= 0 && cols >= 0 && ld_gate >= cols && ld_up >= cols && ld_dy >= cols && ld_dgate >= cols &&
                    ld_dup >= cols,
                "xma_swiglu_backward: bad shape");
    if (rows == 0 || cols == 0) return 0;
    XMA_REQUIRE(gate && up && dy && d_gate && d_up, "xma_swiglu_backward: null pointer");
    XMA_DISPATCH_DTYPE(
        dtype, T,
        const bool vec = all_vec<T>(cols, {gate, up, dy, d_gate, d_up}, {ld_gate, ld_up, ld_dy, ld_dgate, ld_dup});
        dim3 grid, block; swiglu_grid(rows, vec ? cols / Elem<T>::kPerVec : cols, grid, block);
        if (vec) hipLaunchKernelGGL((swiglu_bwd_kernel<T, true>), grid, block, 0, stream, (const T*)gate, ld_gate,
                                    (const T*)up, ld_up, (const T*)dy, ld_dy, (T*)d_gate, ld_dgate, (T*)d_up, ld_dup,
                                    rows, cols);
        else hipLaunchKernelGGL((swiglu_bwd_kernel<T, false>), grid, block, 0, stream, (const T*)gate, ld_gate,
                                (const T*)up, ld_up, (const T*)dy, ld_dy, (T*)d_gate, ld_dgate, (T*)d_up, ld_dup, rows,
                                cols))
    return check_launch("xma_swiglu_backward");
}

}  // extern "C"
