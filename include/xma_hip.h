/*
 * xma_hip.h — C ABI of libxma_hip.so: the MI355X (gfx950) kernels behind the XMA
 * Mixture-of-Experts hot path.
 *
 * Every entry point takes raw device pointers, sizes, strides (in elements), a dtype
 * code and a HIP stream handle passed as `void*` (a `hipStream_t`; NULL = the null
 * stream).  Nothing here allocates or frees device memory: the caller owns every
 * buffer, including the workspaces whose sizes the `*_workspace_bytes` helpers
 * return.  All launches are asynchronous on the given stream.  Return value: 0 on
 * success, non-zero on a rejected argument or a failed launch; `xma_last_error()`
 * then returns a thread-local, NUL-terminated description.
 *
 * Reference interfaces are cited as file:line of open-lm-engine/flash-model-architectures.
 */
#ifndef XMA_HIP_H
#define XMA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activation / weight buffers */
enum xma_dtype { XMA_F32 = 0, XMA_F16 = 1, XMA_BF16 = 2 };

/* operand layouts of xma_grouped_gemm */
enum xma_gemm_kind {
    /* C[p, n] = sum_k A[row(p), k] * B[e(p)][n, k]      (B stored [E, N, K], K contiguous).
       Forward projections: xma/layers/moe/__init__.py:58,83 pass weight.permute(0,2,1). */
    XMA_GEMM_TN = 0,
    /* C[p, n] = sum_k A[row(p), k] * B[e(p)][k, n]      (B stored [E, K, N], N contiguous).
       Input gradients: xma/layers/moe/triton_implementation/__init__.py:131-140. */
    XMA_GEMM_NN = 1,
    /* C[e][i, j] = sum_{p in expert e} A[p, i] * B[row(p), j]   (reduction over the routed rows).
       Weight gradients: xma/layers/moe/triton_implementation/group_backward_kernel.py:13-125. */
    XMA_GEMM_MT = 2
};

/* epilogues of xma_grouped_gemm: the activation between the two projections, fused into the up-projection
   (TN kinds) and, for backward, into the input gradient of the down-projection (NN kinds) */
enum xma_gemm_epilogue {
    XMA_EPI_NONE = 0,
    /* TN only.  B rows [0, N/2) are `up`, rows [N/2, N) are `gate` (xma/functional/swiglu_packed.py:36).
       Writes act[p, j] = up * gate * sigmoid(gate) for j < N/2 into `C` (ldc >= N/2) and, when
       `aux` is non-NULL, the pre-activation row [p, 0..N) into `aux` (ld_aux >= N). */
    XMA_EPI_SWIGLU = 1,
    /* NN only.  The product is dAct[p, j], j < N.  `aux` holds the pre-activation [p, 0..2N)
       (up | gate).  Writes d_up into C[p, j] and d_gate into C[p, N + j] (ldc >= 2N), following
       xma/functional/swiglu/triton_implementation/backward.py:45-56. */
    XMA_EPI_SWIGLU_BWD = 2,
    /* TN only.  torch.nn.GLU over the last dimension, the activation of the reference's own MoE test
       (tests/test_commons.py:93): act[p, j] = h[p, j] * sigmoid(h[p, N/2 + j]).  Operands as XMA_EPI_SWIGLU. */
    XMA_EPI_GLU = 3,
    /* NN only.  Backward of XMA_EPI_GLU, operands as XMA_EPI_SWIGLU_BWD: with a = h[p, j], b = h[p, N + j],
       s = sigmoid(b): C[p, j] = d * s, C[p, N + j] = d * a * s * (1 - s). */
    XMA_EPI_GLU_BWD = 4,
    /* TN only.  tanh-approximated GELU (torch.nn.GELU(approximate="tanh"), tests/test_commons.py:94):
       act[p, j] = 0.5 h (1 + tanh(sqrt(2/pi) (h + 0.044715 h^3))), j < N, into `C` (ldc >= N); the
       pre-activation [p, 0..N) into `aux` when non-NULL (ld_aux >= N). */
    XMA_EPI_GELU_TANH = 5,
    /* NN only.  Backward of XMA_EPI_GELU_TANH: `aux` holds the pre-activation [p, 0..N); writes
       C[p, j] = d * gelu'(h[p, j]), j < N (ldc >= N). */
    XMA_EPI_GELU_TANH_BWD = 6
};

/* ABI revision of this header: bumped whenever a struct gains a field or an enum a value.  A caller may compare it
   with xma_abi_version() of the library it loaded. */
#define XMA_ABI_VERSION 3

typedef struct xma_grouped_gemm_args {
    uint32_t struct_size; /* sizeof(xma_grouped_gemm_args) as the CALLER was compiled: fields beyond it are taken as
                             zero / NULL, so a caller built against a shorter revision of the struct keeps working;
                             0 or a size larger than the library's is rejected */
    int32_t kind;      /* enum xma_gemm_kind */
    int32_t dtype;     /* enum xma_dtype of A, B, C, aux */
    int32_t epilogue;  /* enum xma_gemm_epilogue */
    int32_t num_experts;
    int32_t reserved;  /* 0 */
    int64_t rows;      /* routed rows M = T * top_k (the ragged dimension) */
    int64_t n;         /* TN/NN: output columns.  MT: columns of A (rows of each C[e]) */
    int64_t k;         /* TN/NN: reduction length.  MT: columns of B (columns of each C[e]) */
    const void* a;
    int64_t lda;
    const void* b;
    int64_t ldb;           /* row stride of B; MT: row stride of the activation operand B */
    int64_t b_expert_stride; /* TN/NN: elements between B[e] and B[e+1] */
    void* c;
    int64_t ldc;
    int64_t c_expert_stride; /* MT: elements between C[e] and C[e+1] */
    void* aux;
    int64_t ld_aux;
    const int32_t* expert_offsets; /* [num_experts + 1], exclusive prefix sums of the histogram */
    /* Optional row maps over the grouped position p (either int32 or int64, see idx_is_i64):
       in_index : TN/NN: A row = in_index[p] / in_fan_out.  MT: B row = in_index[p] / in_fan_out.
       out_index: TN/NN: C row = out_index[p].  NULL means the identity. */
    const void* in_index;
    const void* out_index;
    int32_t idx_is_i64;
    int32_t in_fan_out;
    void* workspace;         /* TN/NN: xma_grouped_gemm_workspace_bytes(num_experts, rows) bytes.  MT: optional,
                                16 * num_experts bytes; with it the 16-bit kernel walks the experts in descending
                                order of their row counts, which balances the chip under skewed routing */
    int64_t workspace_bytes;
    /* TN only, optional: per-expert bias [num_experts, N] (row stride ld_bias) added to the fp32 product before the
       epilogue's activation and rounding: F.linear(x, W[e], bias[e]) of xma/layers/moe/__init__.py:103-106. */
    const void* bias;
    int64_t ld_bias;
} xma_grouped_gemm_args;

/* Description of the last failure on the calling thread ("" if none). */
const char* xma_last_error(void);

/* Library version and the GPU architecture the code objects were built for ("gfx950"). */
const char* xma_version(void);
const char* xma_target_arch(void);
/* XMA_ABI_VERSION of the header the library was built from. */
int xma_abi_version(void);

/*
 * Histogram of ids in [0, bins) into counts[bins] (uint32).  ids: int32 or int64, n < 2^32.
 * Out-of-range ids are ignored.  Replaces continuous_count_cuda
 * (xma/functional/continuous_count/cuda_implementation/forward.cu:115-167, called from
 * xma/functional/continuous_count/__init__.py:42-43).
 */
int xma_continuous_count(const void* ids, int ids_is_i64, int64_t n, int32_t bins,
                         uint32_t* counts, void* stream);

/*
 * Routing metadata from the UNSORTED expert choice of every (token, slot) pair:
 *   counts[e]      = #{p : ids[p] == e}                                       (uint32[E])
 *   offsets[0..E]  = exclusive prefix sums of counts, offsets[E] = n          (int32[E+1])
 *   perm           = the stable sort permutation of ids (ties keep position order)
 *   sorted_ids[q]  = ids[perm[q]]
 * perm and sorted_ids are int32 or int64 (out_is_i64).  Replaces the sort / continuous_count /
 * cumsum sequence at xma/layers/moe/__init__.py:218-225 with one stable counting sort.
 * E <= 16384, n < 2^31.  workspace: xma_route_workspace_bytes(n, E) bytes.
 */
int64_t xma_route_workspace_bytes(int64_t n, int32_t num_experts);
int xma_route_build(const void* ids, int ids_is_i64, int64_t n, int32_t num_experts,
                    uint32_t* counts, int32_t* offsets, void* sorted_ids, void* perm,
                    int out_is_i64, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * offsets[e] = first position of sorted_ids (int32 or int64, non-decreasing, values in [0, num_experts)) whose
 * value is >= e, for e in [0, num_experts]: the int32[num_experts + 1] exclusive prefix sums that xma_grouped_gemm
 * takes, recovered from the sorted expert ids.  For callers that hold what the reference's scatter2scatter is given
 * (xma/layers/moe/triton_implementation/scatter_kernel.py:137-147: the sorted ids, no offsets).
 */
int xma_offsets_from_sorted(const void* sorted_ids, int ids_is_i64, int64_t n, int32_t num_experts,
                            int32_t* offsets, void* stream);

/*
 * xma_route_build without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same inputs, outputs and results as xma_route_build; the per-chunk histograms live in a 1 MiB array inside the
 * library (xma_route_build_static_max_bytes(), one copy per GPU, held until the process ends), so the call is
 * rejected when xma_route_workspace_bytes(n, num_experts) exceeds that.  It calls no hipMalloc / hipFree.  All
 * calls on one GPU share the array: calls that may overlap on one GPU (two streams, two threads) race, and must
 * use xma_route_build with a workspace each instead.
 */
int64_t xma_route_build_static_max_bytes(void);
int xma_route_build_static(const void* ids, int ids_is_i64, int64_t n, int32_t num_experts,
                           uint32_t* counts, int32_t* offsets, void* sorted_ids, void* perm,
                           int out_is_i64, void* stream);

/*
 * Router selection: for each of T rows of logits[T, E] (row stride ld) pick the k largest
 * (ties: lower expert index first; output ordered by descending value, then ascending index;
 * NaN ranks above +inf), and softmax over the k selected values in fp32
 * (xma/layers/moe/__init__.py:190-203,268-274).  weights[T, k] has the logits' dtype,
 * idx[T, k] is int32 or int64.  k <= 64, k <= E <= 16384.
 */
int xma_topk_softmax(const void* logits, int dtype, int64_t T, int32_t E, int32_t k, int64_t ld,
                     void* weights, void* idx, int idx_is_i64, void* stream);

/*
 * Backward of xma_topk_softmax: d_logits[T, E] (row stride ld, fully overwritten) is zero except
 * d_logits[t, idx[t, j]] = w_j * (d_weights[t, j] - sum_i w_i * d_weights[t, i]), where
 * w = softmax(logits[t, idx[t, :]]) is recomputed in fp32.  This is what autograd derives for
 * xma/layers/moe/__init__.py:196-201 (top-k gather, fp32 softmax, cast back).
 */
int xma_topk_softmax_bwd(const void* logits, int64_t ld_logits, const void* d_weights, const void* idx,
                         int idx_is_i64, int dtype, int64_t T, int32_t E, int32_t k, void* d_logits,
                         int64_t ld, void* stream);

/*
 * dst[p, :] = src[index[p] / fan_out, :] * (coeff ? coeff[index[p]] : 1) for p < rows.
 * Replaces `group` (xma/layers/moe/triton_implementation/group_kernel.py:12-100).
 * index NULL means the identity; a row whose index is negative is left as it is.  coeff has the rows' dtype.
 */
int xma_gather_rows(const void* src, int64_t ld_src, void* dst, int64_t ld_dst,
                    const void* index, int idx_is_i64, int64_t rows, int64_t cols, int dtype,
                    int32_t fan_out, const void* coeff, void* stream);

/* dst[index[p], :] = src[p, :] for p < rows (index must be a permutation for a defined result). */
int xma_scatter_rows(const void* src, int64_t ld_src, void* dst, int64_t ld_dst,
                     const void* index, int idx_is_i64, int64_t rows, int64_t cols, int dtype,
                     void* stream);

/*
 * The same scatter, done in the order of the destination: the index is inverted first (inverse[index[p]] = p,
 * int32[dst_rows], the caller's scratch memory), then every destination row fetches its source row, so that HBM
 * is written front to back and read at random rather than the reverse (measured 5-7 % faster on 8 KiB rows).
 * Destination rows that no index names are left as they are; a row that several name receives one of them,
 * whole; index entries outside [0, dst_rows) are ignored.  The inverse of the reference's `group`
 * (xma/layers/moe/triton_implementation/group_kernel.py:12-100), which the reference expresses as a second
 * `group` through the inverse permutation.
 */
int xma_scatter_rows_ordered(const void* src, int64_t ld_src, void* dst, int64_t ld_dst,
                             const void* index, int idx_is_i64, int64_t rows, int64_t dst_rows, int64_t cols,
                             int dtype, void* inverse, void* stream);

/*
 * y[t, :] = sum_{j<k} (gates ? gates[t, j] : 1) * y_exp[t*k + j, :], fp32 accumulation.
 * Replaces the bmm at xma/layers/moe/triton_implementation/__init__.py:42-43 and the
 * top-k fold at :145.
 */
int xma_combine_topk(const void* y_exp, int64_t ld_exp, const void* gates, void* y, int64_t ld_y,
                     int64_t T, int32_t k, int64_t cols, int dtype, void* stream);

/*
 * d_gates[t, j] = <y_exp[t*k + j, :], dy[t, :]>, fp32 accumulation
 * (xma/layers/moe/triton_implementation/__init__.py:83).
 */
int xma_gate_grad(const void* y_exp, int64_t ld_exp, const void* dy, int64_t ld_dy, void* d_gates,
                  int64_t T, int32_t k, int64_t cols, int dtype, void* stream);

/*
 * Weight gradient of the router's linear layer: dw[E, H] = d_logits[T, E]^T x[T, H], fp32 accumulation in a
 * fixed order (the token range is split over many blocks; the partial sums are added in split order).
 * XMA_BF16 / XMA_F16 only; E a multiple of 8, at most 256; H a multiple of 8; ldx, ldd multiples of 8 and
 * x, d_logits 16-byte aligned; ldw >= H.  T = 0 writes zeros.  The workspace holds the fp32 partial sums;
 * launches that may run concurrently need a workspace each.
 * Replaces autograd's F.linear backward for the gate's weight (xma/layers/moe/__init__.py:148,192).
 */
int64_t xma_router_weight_grad_workspace_bytes(int64_t T, int32_t E, int64_t H);
int xma_router_weight_grad(const void* x, int64_t ldx, const void* d_logits, int64_t ldd, int dtype, int64_t T,
                           int32_t E, int64_t H, void* dw, int64_t ldw, void* workspace, int64_t workspace_bytes,
                           void* stream);

/*
 * y = up * gate * sigmoid(gate), computed in fp32 (xma/functional/swiglu/__init__.py:34-43);
 * all operands [rows, cols] with independent row strides, so the two halves of a packed
 * tensor can be passed as views (xma/functional/swiglu_packed.py:48).
 */
int xma_swiglu_forward(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y,
                       int64_t ld_y, int64_t rows, int64_t cols, int dtype, void* stream);

/*
 * d_gate = dy * up * (s + gate * s * (1 - s)), d_up = dy * gate * s, s = sigmoid(gate)
 * (xma/functional/swiglu/triton_implementation/backward.py:45-56).
 */
int xma_swiglu_backward(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                        const void* dy, int64_t ld_dy, void* d_gate, int64_t ld_dgate, void* d_up,
                        int64_t ld_dup, int64_t rows, int64_t cols, int dtype, void* stream);

/*
 * Sequence packing: padded x[batch, seq_len, row] -> packed out[total_tokens, row] and back.  Sequence b
 * holds cu_seqlens[b+1] - cu_seqlens[b] tokens (uint32 / int32, or int64 when cu_is_i64), placed at the end of
 * its padded row block when left_padding is non-zero, at the start otherwise.  Rows are moved as bytes
 * (row_bytes = elements per token x element size).  xma_unpack_sequence writes zeros into the padding, so
 * the output needs no prior clearing.  Tokens of a sequence longer than seq_len have no padded position:
 * they pack as zeros and are dropped by unpack.
 * Replaces pack_unpack_sequence_cuda (xma/functional/sequence_packing/cuda_implementation/kernel.cu:64-137,
 * stub cuda_implementation/__init__.py:11-20) and the zero fill that precedes its unpack calls
 * (xma/functional/sequence_packing/__init__.py:76,139).
 */
int xma_pack_sequence(const void* x, void* out, const void* cu_seqlens, int cu_is_i64, int64_t batch,
                      int64_t seq_len, int64_t total_tokens, int64_t row_bytes, int left_padding, void* stream);
int xma_unpack_sequence(const void* x, void* out, const void* cu_seqlens, int cu_is_i64, int64_t batch,
                        int64_t seq_len, int64_t total_tokens, int64_t row_bytes, int left_padding, void* stream);

/*
 * Per-expert bias of a projection: y[r, :] += bias[expert_of_row[p], :] for every routed row p, where
 * r = out_index[p] (the row's place in a scattered buffer) or p when out_index is NULL.  In place.
 * Replaces the bias operand of F.linear on the reference's torch path
 * (xma/layers/moe/__init__.py:103-106); the reference's kernel path has no bias (:54,79).
 */
int xma_add_expert_bias(void* y, int64_t ld_y, const void* bias, int64_t ld_bias, const void* expert_of_row,
                        int expert_is_i64, const void* out_index, int idx_is_i64, int64_t rows, int64_t cols,
                        int dtype, void* stream);

/*
 * Bias gradient: out[e, :] = sum over the grouped rows expert_offsets[e] .. expert_offsets[e+1]-1 of src,
 * accumulated in fp32 in a fixed order.  expert_offsets: int32[num_experts + 1].  Replaces autograd's
 * reduction for the bias of F.linear on the reference's torch path (same lines).
 */
int xma_expert_colsum(const void* src, int64_t ld, const int32_t* expert_offsets, int32_t num_experts,
                      int64_t cols, void* out, int64_t ld_out, int dtype, void* stream);

/*
 * Ragged batched GEMM over the experts' row groups with fp32 accumulation; see the enums
 * above for layouts and fused epilogues.  Empty groups are legal; XMA_GEMM_MT writes zeros
 * for them (the reference pre-zeroes DW, xma/layers/moe/triton_implementation/__init__.py:121).
 * Replaces scatter2scatter (scatter_kernel.py:137-183) and group_bwd_W
 * (group_backward_kernel.py:102-125).
 * The workspace (TN/NN) holds the row-tile tables and a fixed 64 MiB region for the fp32
 * partial sums of tiles whose reduction is split; launches that may run concurrently need
 * a workspace each.  The kernel initialises what it uses.
 */
int64_t xma_grouped_gemm_workspace_bytes(int32_t num_experts, int64_t rows);
int xma_grouped_gemm(const xma_grouped_gemm_args* args, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XMA_HIP_H */
