// Shared host/device helpers for the gfx950 MoE kernels: error reporting, 16-byte vector
// types, dtype conversion and wave64 primitives.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/xma_hip.h"

namespace xma {

constexpr int kWaveSize = 64;  // CDNA wavefront width

// ---- host-side error channel --------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);  // reads hipGetLastError(), 0 if clean

#define XMA_REQUIRE(cond, ...)            \
    do {                                  \
        if (!(cond)) {                    \
            ::xma::set_error(__VA_ARGS__); \
            return 1;                     \
        }                                 \
    } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int dtype_size(int dtype) { return dtype == XMA_F32 ? 4 : 2; }
inline bool valid_dtype(int dtype) { return dtype == XMA_F32 || dtype == XMA_F16 || dtype == XMA_BF16; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device-side scalar conversion -----------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    _Float16 v;
};

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

template <typename T>
struct Elem;

template <>
struct Elem<float> {
    static constexpr int kDtype = XMA_F32;
    static constexpr int kPerVec = 4;  // elements in 16 bytes
    __device__ static __forceinline__ float load(const float* p) { return *p; }
    __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
    __device__ static __forceinline__ void unpack(const uint4& v, float* out) {
        out[0] = __uint_as_float(v.x);
        out[1] = __uint_as_float(v.y);
        out[2] = __uint_as_float(v.z);
        out[3] = __uint_as_float(v.w);
    }
    __device__ static __forceinline__ uint4 pack(const float* in) {
        return make_uint4(__float_as_uint(in[0]), __float_as_uint(in[1]), __float_as_uint(in[2]),
                          __float_as_uint(in[3]));
    }
};

template <>
struct Elem<bf16_t> {
    static constexpr int kDtype = XMA_BF16;
    static constexpr int kPerVec = 8;
    __device__ static __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
    __device__ static __forceinline__ void store(bf16_t* p, float v) { p->bits = (uint16_t)float_to_bf16_bits(v); }
    __device__ static __forceinline__ void unpack(const uint4& v, float* out) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    // two floats -> packed bf16 pair, round to nearest even: one v_cvt_pk_bf16_f32 on gfx950
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        typedef __attribute__((ext_vector_type(2))) float f32x2_t;
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t));
    }
    __device__ static __forceinline__ uint4 pack(const float* in) {
        return make_uint4(pack2(in[0], in[1]), pack2(in[2], in[3]), pack2(in[4], in[5]), pack2(in[6], in[7]));
    }
};

template <>
struct Elem<f16_t> {
    static constexpr int kDtype = XMA_F16;
    static constexpr int kPerVec = 8;
    __device__ static __forceinline__ float load(const f16_t* p) { return (float)p->v; }
    __device__ static __forceinline__ void store(f16_t* p, float v) { p->v = (_Float16)v; }
    __device__ static __forceinline__ void unpack(const uint4& v, float* out) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            union {
                uint32_t u;
                _Float16 h[2];
            } cvt;
            cvt.u = w[i];
            out[2 * i] = (float)cvt.h[0];
            out[2 * i + 1] = (float)cvt.h[1];
        }
    }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        union {
            uint32_t u;
            _Float16 h[2];
        } cvt;
        cvt.h[0] = (_Float16)a;
        cvt.h[1] = (_Float16)b;
        return cvt.u;
    }
    __device__ static __forceinline__ uint4 pack(const float* in) {
        return make_uint4(pack2(in[0], in[1]), pack2(in[2], in[3]), pack2(in[4], in[5]), pack2(in[6], in[7]));
    }
};

// sigmoid in fp32 with an accurate exponential
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// sigmoid from the hardware exp2 and reciprocal (a few ulp in fp32): for results that are rounded to a
// 16-bit type anyway
__device__ __forceinline__ float sigmoid_fast(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// The activations the grouped GEMM epilogues fuse, forward and backward, on fp32 values.  FAST selects the hardware
// exp2 / reciprocal (a few ulp in fp32) for results that are rounded to a 16-bit type anyway.
enum Activation { ACT_NONE = 0, ACT_SWIGLU = 1, ACT_GLU = 2, ACT_GELU_TANH = 3 };

template <bool FAST>
__device__ __forceinline__ float sigmoid_any(float x) {
    if constexpr (FAST) return sigmoid_fast(x);
    else return sigmoid_f32(x);
}

// act(a, b) of the two halves of a gated pre-activation: SwiGLU a * b * sigmoid(b) (a = up, b = gate,
// xma/functional/swiglu/__init__.py:34-43); GLU a * sigmoid(b) (torch.nn.GLU)
template <bool FAST>
__device__ __forceinline__ float gated_forward(int act, float a, float b) {
    const float s = sigmoid_any<FAST>(b);
    return act == ACT_SWIGLU ? a * (b * s) : a * s;
}
// gradients with respect to a and b for an upstream gradient d
template <bool FAST>
__device__ __forceinline__ void gated_backward(int act, float a, float b, float d, float& da, float& db) {
    const float s = sigmoid_any<FAST>(b);
    if (act == ACT_SWIGLU) {  // xma/functional/swiglu/triton_implementation/backward.py:45-56
        const float t = b * s;
        da = d * t;
        db = d * a * (s + t * (1.0f - s));
    } else {
        da = d * s;
        db = d * a * (s * (1.0f - s));
    }
}

// tanh-approximated GELU and its derivative; tanh(u) = 2 sigmoid(2u) - 1
template <bool FAST>
__device__ __forceinline__ float gelu_tanh_forward(float x) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x * sigmoid_any<FAST>(2.0f * u);  // 0.5 x (1 + tanh u)
}
template <bool FAST>
__device__ __forceinline__ float gelu_tanh_backward(float x, float d) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float s = sigmoid_any<FAST>(2.0f * u);  // (1 + tanh u) / 2
    const float du = 0.7978845608028654f * (1.0f + 3.0f * 0.044715f * x * x);
    // d/dx [x s(2u)] = s + x * 2 s (1 - s) du
    return d * (s + 2.0f * x * s * (1.0f - s) * du);
}

// Streaming accesses for data that is touched once: kept from displacing reusable lines in the caches (measured on
// the element-wise kernels: 80 % of the HBM peak instead of 71 %).
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_stream_t;
__device__ __forceinline__ uint4 load_stream(const void* p) {
    const u32x4_stream_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_stream_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_stream(void* p, const uint4& v) {
    __builtin_nontemporal_store(u32x4_stream_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_stream_t*>(p));
}

// ---- wave64 primitives ------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (kWaveSize - 1)); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWaveSize);
    return v;
}

// index loads that accept int32 or int64 tables
__device__ __forceinline__ int64_t load_index(const void* table, int is_i64, int64_t i) {
    return is_i64 ? reinterpret_cast<const int64_t*>(table)[i]
                  : (int64_t) reinterpret_cast<const int32_t*>(table)[i];
}

// dispatch a templated launch over the three element types
#define XMA_DISPATCH_DTYPE(dtype, T, ...)       \
    switch (dtype) {                            \
        case XMA_F32: {                         \
            using T = float;                    \
            __VA_ARGS__;                        \
        } break;                                \
        case XMA_F16: {                         \
            using T = ::xma::f16_t;             \
            __VA_ARGS__;                        \
        } break;                                \
        default: {                              \
            using T = ::xma::bf16_t;            \
            __VA_ARGS__;                        \
        } break;                                \
    }

}  // namespace xma
