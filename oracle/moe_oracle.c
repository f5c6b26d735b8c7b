/*
 * CPU oracle for the XMA MoE hot path — TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement, in scalar loops with double accumulation, of what the reference's torch
 * path computes.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this; the product package never does.
 *
 * Each function cites the file:line of open-lm-engine/flash-model-architectures it follows.  The
 * reference leaves two orders to the library (torch.sort is called unstably at
 * xma/layers/moe/__init__.py:218, torch.topk's tie order at :272); this oracle fixes them the way
 * the product does: stable sort by position, top-k ties to the lower expert index.
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC -> oracle/_build/libmoe_oracle.so)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* counts[e] = #{i : ids[i] == e}; ids outside [0, bins) ignored.
 * xma/functional/continuous_count/__init__.py:28-40 (bincount(minlength=bins)). */
void xo_count(const int64_t* ids, int64_t n, int32_t bins, uint32_t* counts) {
    memset(counts, 0, sizeof(uint32_t) * (size_t)bins);
    for (int64_t i = 0; i < n; ++i)
        if (ids[i] >= 0 && ids[i] < bins) counts[ids[i]]++;
}

/* Stable sort of ids by value: xma/layers/moe/__init__.py:218 (sort) + :219 (count) + :225 (cumsum).
 * offsets has bins+1 entries (exclusive; offsets[1..] is the reference's inclusive cumsum). */
void xo_route(const int64_t* ids, int64_t n, int32_t bins, uint32_t* counts, int32_t* offsets,
              int64_t* sorted_ids, int64_t* perm) {
    xo_count(ids, n, bins, counts);
    offsets[0] = 0;
    for (int32_t e = 0; e < bins; ++e) offsets[e + 1] = offsets[e] + (int32_t)counts[e];
    int64_t* next = (int64_t*)malloc(sizeof(int64_t) * (size_t)bins);
    for (int32_t e = 0; e < bins; ++e) next[e] = offsets[e];
    for (int64_t i = 0; i < n; ++i) { /* increasing i => ties keep position order */
        int64_t pos = next[ids[i]]++;
        perm[pos] = i;
        sorted_ids[pos] = ids[i];
    }
    free(next);
}

/* Top-k by selection: largest value first, ties to the lower index; then softmax over the k
 * selected values.  xma/layers/moe/__init__.py:190-203 (softmax of the selected logits in fp32)
 * and :268-274 (k == 1 uses max, which returns the first maximal index). */
void xo_topk_softmax(const float* logits, int64_t T, int32_t E, int32_t k, double* weights, int64_t* idx) {
    char* taken = (char*)malloc((size_t)E);
    for (int64_t t = 0; t < T; ++t) {
        const float* row = logits + t * E;
        memset(taken, 0, (size_t)E);
        for (int32_t s = 0; s < k; ++s) {
            int32_t best = -1;
            for (int32_t e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || row[e] > row[best]) best = e; /* strict > keeps the lowest index */
            }
            taken[best] = 1;
            idx[t * k + s] = best;
        }
        double vmax = row[idx[t * k]], denom = 0.0;
        for (int32_t s = 0; s < k; ++s) denom += exp((double)row[idx[t * k + s]] - vmax);
        for (int32_t s = 0; s < k; ++s) weights[t * k + s] = exp((double)row[idx[t * k + s]] - vmax) / denom;
    }
    free(taken);
}

/* y = up * gate * sigmoid(gate): xma/functional/swiglu/__init__.py:34-43. */
void xo_swiglu(const double* gate, const double* up, int64_t n, double* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = up[i] * gate[i] / (1.0 + exp(-gate[i]));
}

/* d_gate = dy*up*(s + gate*s*(1-s)), d_up = dy*gate*s:
 * xma/functional/swiglu/triton_implementation/backward.py:45-56. */
void xo_swiglu_bwd(const double* gate, const double* up, const double* dy, int64_t n, double* d_gate, double* d_up) {
    for (int64_t i = 0; i < n; ++i) {
        const double s = 1.0 / (1.0 + exp(-gate[i]));
        d_gate[i] = dy[i] * up[i] * (s + gate[i] * s * (1.0 - s));
        d_up[i] = dy[i] * gate[i] * s;
    }
}

/*
 * Whole layer forward for a SwiGLU MoE, token by token (no grouping at all, so it shares no
 * indexing logic with the grouped implementations):
 *   y[t] = sum_s w[t,s] * W2[e] * swiglu_packed(W1[e] * x[t]),  e = idx[t,s]
 * W1: [E, 2I, H] (rows [0,I) = up, [I,2I) = gate: xma/functional/swiglu_packed.py:36),
 * W2: [E, H, I] (F.linear(x, W[e]): xma/layers/moe/__init__.py:103-106).
 * Algebraically equal to the torch branch at xma/layers/moe/__init__.py:243-262.
 */
void xo_moe_forward(const double* x, const double* w1, const double* w2, const double* weights, const int64_t* idx,
                    int64_t T, int32_t H, int32_t I, int32_t k, double* y) {
    double* h = (double*)malloc(sizeof(double) * 2 * (size_t)I);
    double* a = (double*)malloc(sizeof(double) * (size_t)I);
    for (int64_t t = 0; t < T; ++t) {
        double* yt = y + t * H;
        for (int32_t c = 0; c < H; ++c) yt[c] = 0.0;
        for (int32_t s = 0; s < k; ++s) {
            const int64_t e = idx[t * k + s];
            const double* W1 = w1 + e * 2 * (int64_t)I * H;
            const double* W2 = w2 + e * (int64_t)H * I;
            for (int32_t j = 0; j < 2 * I; ++j) {
                double acc = 0.0;
                for (int32_t c = 0; c < H; ++c) acc += W1[(int64_t)j * H + c] * x[t * H + c];
                h[j] = acc;
            }
            for (int32_t j = 0; j < I; ++j) a[j] = h[j] * h[I + j] / (1.0 + exp(-h[I + j]));
            for (int32_t c = 0; c < H; ++c) {
                double acc = 0.0;
                for (int32_t j = 0; j < I; ++j) acc += W2[(int64_t)c * I + j] * a[j];
                yt[c] += weights[t * k + s] * acc;
            }
        }
    }
    free(h);
    free(a);
}
