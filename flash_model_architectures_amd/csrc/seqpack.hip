// Sequence packing on gfx950: padded [B, S, row] <-> packed [total_tokens, row], driven by the cumulative
// sequence lengths (xma/functional/sequence_packing/cuda_implementation/kernel.cu:45-137).  Pure byte moves,
// so rows are handled as bytes whatever the element type.  Differences in shape from the reference kernel,
// which launches one block per padded position and relies on a separate zero fill of the unpacked tensor:
//   pack    walks the packed tokens (padding is never read) and finds each token's sequence by a binary
//           search of cu_seqlens;
//   unpack  walks the padded positions and writes the zeros of the padding itself, so the output is written
//           exactly once.
// Both keep kPackRows independent 16-byte loads in flight per lane before the first store.
#include "common.h"

namespace xma {

constexpr int kPackRows = 2;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

__device__ __forceinline__ int64_t cu_at(const void* cu, int is_i64, int64_t i) {
    return is_i64 ? reinterpret_cast<const int64_t*>(cu)[i] : (int64_t)reinterpret_cast<const uint32_t*>(cu)[i];
}

// largest b in [0, B) with cu[b] <= t, skipping empty sequences that start at t's position
__device__ __forceinline__ int64_t sequence_of(const void* cu, int is_i64, int64_t B, int64_t t) {
    int64_t lo = 0, hi = B;  // invariant: cu[lo] <= t < cu[hi] (cu[B] = total > t)
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (cu_at(cu, is_i64, mid) <= t) lo = mid;
        else hi = mid;
    }
    return lo;
}

// Padded row of packed token t (or -1 when the sequence is longer than S and the token has no place).
__device__ __forceinline__ int64_t padded_row_of(const void* cu, int is_i64, int64_t B, int64_t S, int left, int64_t t) {
    const int64_t b = sequence_of(cu, is_i64, B, t);
    const int64_t start = cu_at(cu, is_i64, b), len = cu_at(cu, is_i64, b + 1) - start;
    const int64_t s = left ? S - len + (t - start) : t - start;
    return s >= 0 && s < S ? b * S + s : -1;
}

// Packed token held by padded row r (or -1 for padding).
__device__ __forceinline__ int64_t packed_row_of(const void* cu, int is_i64, int64_t S, int left, int64_t total,
                                                 int64_t r) {
    const int64_t b = r / S, s = r - b * S;
    const int64_t start = cu_at(cu, is_i64, b), len = cu_at(cu, is_i64, b + 1) - start;
    const int64_t j = left ? s - (S - len) : s;
    const int64_t t = start + j;
    return j >= 0 && j < len && t < total ? t : -1;
}

// One kernel for both directions.  PACK: destination rows are packed tokens, sources are padded rows.
// UNPACK: destination rows are padded positions, sources are packed tokens or nothing (zeros).
// VEC = bytes moved per access (16, 4 or 1).
template <bool PACK, int VEC>
__global__ __launch_bounds__(256) void pack_unpack_kernel(const char* __restrict__ src, char* __restrict__ dst,
                                                          const void* __restrict__ cu, int cu_is_i64, int64_t B,
                                                          int64_t S, int64_t total, int64_t row_bytes, int left) {
    const int64_t dst_rows = PACK ? total : B * S;
    const int64_t chunks = row_bytes / VEC;
    for (int64_t r0 = (int64_t)blockIdx.x * kPackRows; r0 < dst_rows; r0 += (int64_t)gridDim.x * kPackRows) {
        int64_t from[kPackRows];
#pragma unroll
        for (int j = 0; j < kPackRows; ++j) {
            const int64_t r = r0 + j < dst_rows ? r0 + j : dst_rows - 1;
            from[j] = PACK ? padded_row_of(cu, cu_is_i64, B, S, left, r) : packed_row_of(cu, cu_is_i64, S, left, total, r);
        }
        for (int64_t c = threadIdx.x; c < chunks; c += blockDim.x) {
            if constexpr (VEC == 16) {
                u32x4_t v[kPackRows];
#pragma unroll
                for (int j = 0; j < kPackRows; ++j)
                    v[j] = from[j] >= 0 ? __builtin_nontemporal_load(
                                              reinterpret_cast<const u32x4_t*>(src + from[j] * row_bytes + c * 16))
                                        : u32x4_t{0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < kPackRows; ++j)
                    if (r0 + j < dst_rows)
                        __builtin_nontemporal_store(v[j], reinterpret_cast<u32x4_t*>(dst + (r0 + j) * row_bytes + c * 16));
            } else if constexpr (VEC == 4) {
#pragma unroll
                for (int j = 0; j < kPackRows; ++j)
                    if (r0 + j < dst_rows)
                        reinterpret_cast<uint32_t*>(dst + (r0 + j) * row_bytes)[c] =
                            from[j] >= 0 ? reinterpret_cast<const uint32_t*>(src + from[j] * row_bytes)[c] : 0u;
            } else {
#pragma unroll
                for (int j = 0; j < kPackRows; ++j)
                    if (r0 + j < dst_rows) dst[(r0 + j) * row_bytes + c] = from[j] >= 0 ? src[from[j] * row_bytes + c] : (char)0;
            }
        }
    }
}

template <bool PACK>
static int launch_pack_unpack(const void* src, void* dst, const void* cu, int cu_is_i64, int64_t B, int64_t S,
                              int64_t total, int64_t row_bytes, int left, hipStream_t stream, const char* what) {
    const int64_t dst_rows = PACK ? total : B * S;
    if (dst_rows == 0 || row_bytes == 0) return 0;
    const int64_t groups = ceil_div(dst_rows, kPackRows);
    // one small group of rows per block (measured faster than a capped grid of long-running blocks: 74-78 % of HBM
    // peak instead of 65-68 %); the stride loop in the kernel only matters beyond 2^31 groups
    const dim3 grid((unsigned)(groups < 0x7fffffff ? groups : 0x7fffffff));
    const auto both = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t)row_bytes;
#define XMA_PACK_LAUNCH(VEC, THREADS)                                                                            \
    hipLaunchKernelGGL((pack_unpack_kernel<PACK, VEC>), grid, dim3(THREADS), 0, stream, (const char*)src, (char*)dst, \
                       cu, cu_is_i64, B, S, total, row_bytes, left)
    if (both % 16 == 0) {
        const int64_t chunks = row_bytes / 16;
        if (chunks <= 64) XMA_PACK_LAUNCH(16, 64);
        else if (chunks <= 128) XMA_PACK_LAUNCH(16, 128);
        else XMA_PACK_LAUNCH(16, 256);
    } else if (both % 4 == 0) {
        XMA_PACK_LAUNCH(4, 256);
    } else {
        XMA_PACK_LAUNCH(1, 256);
    }
#undef XMA_PACK_LAUNCH
    return check_launch(what);
}

}  // namespace xma

using namespace xma;

extern "C" {

int xma_pack_sequence(const void* x, void* out, const void* cu_seqlens, int cu_is_i64, int64_t batch, int64_t seq_len,
                      int64_t total_tokens, int64_t row_bytes, int left_padding, void* stream) {
    XMA_REQUIRE(batch >= 0 && seq_len >= 0 && total_tokens >= 0 && row_bytes >= 0, "xma_pack_sequence: bad shape");
    XMA_REQUIRE(batch * seq_len < ((int64_t)1 << 40), "xma_pack_sequence: too many padded positions");
    if (total_tokens == 0 || row_bytes == 0) return 0;
    XMA_REQUIRE(batch >= 1 && seq_len >= 1, "xma_pack_sequence: tokens without sequences");
    XMA_REQUIRE(x && out && cu_seqlens, "xma_pack_sequence: null pointer");
    return launch_pack_unpack<true>(x, out, cu_seqlens, cu_is_i64, batch, seq_len, total_tokens, row_bytes,
                                    left_padding != 0, (hipStream_t)stream, "xma_pack_sequence");
}

int xma_unpack_sequence(const void* x, void* out, const void* cu_seqlens, int cu_is_i64, int64_t batch,
                        int64_t seq_len, int64_t total_tokens, int64_t row_bytes, int left_padding, void* stream) {
    XMA_REQUIRE(batch >= 0 && seq_len >= 0 && total_tokens >= 0 && row_bytes >= 0, "xma_unpack_sequence: bad shape");
    XMA_REQUIRE(batch * seq_len < ((int64_t)1 << 40), "xma_unpack_sequence: too many padded positions");
    if (batch * seq_len == 0 || row_bytes == 0) return 0;
    XMA_REQUIRE(out && cu_seqlens && (x || total_tokens == 0), "xma_unpack_sequence: null pointer");
    return launch_pack_unpack<false>(x, out, cu_seqlens, cu_is_i64, batch, seq_len, total_tokens, row_bytes,
                                     left_padding != 0, (hipStream_t)stream, "xma_unpack_sequence");
}

}  // extern "C"
