// Weight gradient of the router's linear layer: dW[E, H] = d_logits[T, E]^T x[T, H], fp32 accumulation.
// A short, wide output (E <= 256 rows) reduced over every token: a library GEMM gives this shape one tile per
// 64 x 64 outputs and walks all T tokens in each (140-170 us at 16384 tokens x 2048 x 64..128), although the
// operands are a single pass over x (67 MB).  Here the token range is split over many blocks, every block reduces
// its share on the matrix cores into an fp32 partial, and a second kernel adds the partials in a fixed order
// (so the result is reproducible).  The reference leaves this product to autograd's F.linear backward
// (xma/layers/moe/__init__.py:148,192).
//
// Both operands have the reduction index (the token) as their strided dimension, so they are staged in LDS in their
// HBM layout ([token][column]) and the matrix-instruction fragments are read with the transposing LDS read
// (ds_read_b64_tr_b16), as the grouped weight-gradient kernel does.
#include "grouped_gemm_common.h"

namespace xma {
namespace router {

typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
#define XMA_ROUTER_LDS_S4(p) ((__attribute__((address_space(3))) short4_t*)(p))

constexpr int BT = 128;     // tokens per stage
constexpr int BH = 64;      // output columns per block: 4 waves x 16
constexpr int THREADS = 256;
constexpr int X_PITCH = BH * 2 + 16;  // bytes per token row of the x tile (padded: rows four apart fall into different banks)

// Fragment of the 16x16x32 matrix instruction for columns col0 .. col0+15, tokens k0 .. k0+31 of an LDS tile stored
// [token][column]: within each 16-lane group the transposing read hands lane i the i-th 16-bit element of four
// 16-element rows, row j being assembled from the 8-byte pieces addressed by lanes 4j .. 4j+3.  Lane i of group g
// therefore addresses (token 8g + i/4, columns 4*(i%4) .. +3) and receives four consecutive tokens of column i; a
// second read four tokens further down completes the eight reduction elements 8g .. 8g+7 of the operand.
__device__ __forceinline__ u32x4_t read_fragment(const char* tile, int pitch, int col0, int k0, int lane) {
    const int i = lane & 15, g = lane >> 4;
    const char* p = tile + (k0 + 8 * g + (i >> 2)) * pitch + (col0 + 4 * (i & 3)) * 2;
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_ROUTER_LDS_S4(p));
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_ROUTER_LDS_S4(p + 4 * pitch));
    const u32x2_t a = __builtin_bit_cast(u32x2_t, lo), b = __builtin_bit_cast(u32x2_t, hi);
    return u32x4_t{a.x, a.y, b.x, b.y};
}

// Block (x = 64-column tile of H, y = split s of the tokens): partial[s][e][h] = sum over the split's tokens.
// EB = number of 16-row blocks of the output (E <= 16 * EB).  Wave w owns columns 16w .. 16w+15 of the tile.
template <typename T, int EB>
__global__ __launch_bounds__(THREADS) void router_wgrad_partial_kernel(const T* __restrict__ x, int64_t ldx,
                                                                       const T* __restrict__ dl, int64_t ldd, int64_t Tn,
                                                                       int E, int64_t H, int64_t tokens_per_split,
                                                                       float* __restrict__ partial) {
    constexpr int EP = EB * 16;            // padded number of experts
    constexpr int D_PITCH = EP * 2 + 16;   // bytes per token row of the d_logits tile
    constexpr int D_CHUNKS = EP / 8;       // 16-byte chunks per token row
    constexpr int D_LOADS = (BT * D_CHUNKS + THREADS - 1) / THREADS;
    constexpr int X_LOADS = BT * (BH / 8) / THREADS;  // 2
    __shared__ __attribute__((aligned(16))) char x_tile[BT * X_PITCH];
    __shared__ __attribute__((aligned(16))) char d_tile[BT * D_PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t h0 = (int64_t)blockIdx.x * BH;
    const int64_t t_begin = (int64_t)blockIdx.y * tokens_per_split;
    const int64_t t_end = t_begin + tokens_per_split < Tn ? t_begin + tokens_per_split : Tn;

    f32x4_t acc[EB];
#pragma unroll
    for (int eb = 0; eb < EB; ++eb) acc[eb] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    uint4 xr[X_LOADS], dr[D_LOADS];
    auto fetch = [&](int64_t t0) {
#pragma unroll
        for (int p = 0; p < X_LOADS; ++p) {
            const int c = tid + p * THREADS, row = c / (BH / 8), chunk = c % (BH / 8);
            const int64_t t = t0 + row, h = h0 + chunk * 8;
            xr[p] = t < t_end && h < H ? *reinterpret_cast<const uint4*>(x + t * ldx + h) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < D_LOADS; ++p) {
            const int c = tid + p * THREADS, row = c / D_CHUNKS, chunk = c % D_CHUNKS;
            const int64_t t = t0 + row;
            dr[p] = row < BT && t < t_end && chunk * 8 < E ? *reinterpret_cast<const uint4*>(dl + t * ldd + chunk * 8)
                                                            : make_uint4(0, 0, 0, 0);
        }
    };
    auto stage_to_lds = [&]() {
#pragma unroll
        for (int p = 0; p < X_LOADS; ++p) {
            const int c = tid + p * THREADS, row = c / (BH / 8), chunk = c % (BH / 8);
            *reinterpret_cast<uint4*>(x_tile + row * X_PITCH + chunk * 16) = xr[p];
        }
#pragma unroll
        for (int p = 0; p < D_LOADS; ++p) {
            const int c = tid + p * THREADS, row = c / D_CHUNKS, chunk = c % D_CHUNKS;
            if (row < BT) *reinterpret_cast<uint4*>(d_tile + row * D_PITCH + chunk * 16) = dr[p];
        }
    };

    fetch(t_begin);
    for (int64_t t0 = t_begin; t0 < t_end; t0 += BT) {
        __syncthreads();  // the previous stage has been read
        stage_to_lds();
        __syncthreads();
        if (t0 + BT < t_end) fetch(t0 + BT);  // on its way while this stage is multiplied
#pragma unroll
        for (int ks = 0; ks < BT / 32; ++ks) {
            const u32x4_t xf = read_fragment(x_tile, X_PITCH, 16 * wave, 32 * ks, lane);
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) {
                const u32x4_t df = read_fragment(d_tile, D_PITCH, 16 * eb, 32 * ks, lane);
                Mma16<T>::run(df, xf, acc[eb]);
            }
        }
    }
    // The matrix instructions are inline assembly: the compiler does not keep the distance the hardware needs between
    // the last of them and a read of its result.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // result register r of lane l in block eb: expert 16*eb + 4*(l/16) + r, column 16*wave + l%16
    float* out = partial + (int64_t)blockIdx.y * E * H;
    const int64_t h = h0 + 16 * wave + (lane & 15);
    if (h < H) {
#pragma unroll
        for (int eb = 0; eb < EB; ++eb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = 16 * eb + 4 * (lane >> 4) + r;
                if (e < E) out[(int64_t)e * H + h] = acc[eb][r];
            }
    }
}

// dW[e][h] = sum over the splits, in split order.  A thread adds up four adjacent columns (H is a multiple of 8) and
// requests four splits at a time.
template <typename T>
__global__ __launch_bounds__(256) void router_wgrad_reduce_kernel(const float* __restrict__ partial, int splits, int E,
                                                                  int64_t H, T* __restrict__ dw, int64_t ldw) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const int64_t plane = (int64_t)E * H;
    if (i >= plane) return;
    float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    int s = 0;
    for (; s + 4 <= splits; s += 4) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = *reinterpret_cast<const float4*>(partial + (s + j) * plane + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sum.x += v[j].x;
            sum.y += v[j].y;
            sum.z += v[j].z;
            sum.w += v[j].w;
        }
    }
    for (; s < splits; ++s) {
        const float4 v = *reinterpret_cast<const float4*>(partial + s * plane + i);
        sum.x += v.x;
        sum.y += v.y;
        sum.z += v.z;
        sum.w += v.w;
    }
    T* out = dw + (i / H) * ldw + i % H;
    Elem<T>::store(out, sum.x);
    Elem<T>::store(out + 1, sum.y);
    Elem<T>::store(out + 2, sum.z);
    Elem<T>::store(out + 3, sum.w);
}

// Tokens per split (a multiple of the stage) and the number of splits: about 512 blocks, at least two stages each.
static void plan(int64_t Tn, int64_t H, int64_t& tokens_per_split, int& splits) {
    const int64_t col_tiles = ceil_div(H, BH);
    int64_t want = ceil_div((int64_t)512, col_tiles);
    const int64_t most = ceil_div(Tn, (int64_t)2 * BT);
    if (want > most) want = most;
    if (want < 1) want = 1;
    tokens_per_split = ceil_div(ceil_div(Tn, want), (int64_t)BT) * BT;
    splits = (int)ceil_div(Tn, tokens_per_split);
}

}  // namespace router
}  // namespace xma

using namespace xma;

extern "C" {

int64_t xma_router_weight_grad_workspace_bytes(int64_t T, int32_t E, int64_t H) {
    if (T < 0 || E < 1 || H < 1) return -1;
    if (T == 0) return 0;
    int64_t tokens_per_split = 0;
    int splits = 1;
    router::plan(T, H, tokens_per_split, splits);
    return (int64_t)splits * E * H * (int64_t)sizeof(float);
}

int xma_router_weight_grad(const void* x, int64_t ldx, const void* d_logits, int64_t ldd, int dtype, int64_t T,
                           int32_t E, int64_t H, void* dw, int64_t ldw, void* workspace, int64_t workspace_bytes,
                           void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(dtype == XMA_BF16 || dtype == XMA_F16, "xma_router_weight_grad: 16-bit element types only (dtype %d)", dtype);
    XMA_REQUIRE(E >= 1 && E <= 256 && E % 8 == 0, "xma_router_weight_grad: E=%d must be a multiple of 8, at most 256", E);
    XMA_REQUIRE(T >= 0 && H >= 1 && H % 8 == 0, "xma_router_weight_grad: bad T=%lld or H=%lld (H must be a multiple of 8)",
                (long long)T, (long long)H);
    XMA_REQUIRE(dw != nullptr && ldw >= H, "xma_router_weight_grad: null output or row stride %lld < H", (long long)ldw);
    XMA_REQUIRE(T == 0 || (x && d_logits && workspace), "xma_router_weight_grad: null pointer");
    XMA_REQUIRE(T == 0 || (ldx >= H && ldd >= E && ldx % 8 == 0 && ldd % 8 == 0 && aligned16(x) && aligned16(d_logits)),
                "xma_router_weight_grad: operand rows must be 16-byte aligned (ldx=%lld, ldd=%lld)", (long long)ldx,
                (long long)ldd);
    XMA_REQUIRE(workspace_bytes >= xma_router_weight_grad_workspace_bytes(T, E, H),
                "xma_router_weight_grad: workspace too small (%lld < %lld)", (long long)workspace_bytes,
                (long long)xma_router_weight_grad_workspace_bytes(T, E, H));
    int64_t tokens_per_split = 0;
    int splits = 0;
    if (T > 0) router::plan(T, H, tokens_per_split, splits);
    float* partial = (float*)workspace;
    if (T > 0) {
        const dim3 grid((unsigned)ceil_div(H, (int64_t)router::BH), (unsigned)splits);
#define XMA_ROUTER_PARTIAL(T_, EB)                                                                                    \
    hipLaunchKernelGGL((router::router_wgrad_partial_kernel<T_, EB>), grid, dim3(router::THREADS), 0, stream,         \
                       (const T_*)x, ldx, (const T_*)d_logits, ldd, T, (int)E, H, tokens_per_split, partial)
#define XMA_ROUTER_PARTIAL_E(T_)                                                                                      \
    if (E <= 16)                                                                                                      \
        XMA_ROUTER_PARTIAL(T_, 1);                                                                                    \
    else if (E <= 32)                                                                                                 \
        XMA_ROUTER_PARTIAL(T_, 2);                                                                                    \
    else if (E <= 64)                                                                                                 \
        XMA_ROUTER_PARTIAL(T_, 4);                                                                                    \
    else if (E <= 128)                                                                                                \
        XMA_ROUTER_PARTIAL(T_, 8);                                                                                    \
    else                                                                                                              \
        XMA_ROUTER_PARTIAL(T_, 16)
        if (dtype == XMA_BF16) {
            XMA_ROUTER_PARTIAL_E(bf16_t);
        } else {
            XMA_ROUTER_PARTIAL_E(f16_t);
        }
#undef XMA_ROUTER_PARTIAL_E
#undef XMA_ROUTER_PARTIAL
    }
    const unsigned blocks = (unsigned)ceil_div((int64_t)E * H, (int64_t)1024);
    if (dtype == XMA_BF16)
        hipLaunchKernelGGL(router::router_wgrad_reduce_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                           (const float*)partial, splits, (int)E, H, (bf16_t*)dw, ldw);
    else
        hipLaunchKernelGGL(router::router_wgrad_reduce_kernel<f16_t>, dim3(blocks), dim3(256), 0, stream,
                           (const float*)partial, splits, (int)E, H, (f16_t*)dw, ldw);
    return check_launch("xma_router_weight_grad");
}

}  // extern "C"
