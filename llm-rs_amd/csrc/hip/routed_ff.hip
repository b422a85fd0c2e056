// Feed-forwards whose activation runs on a product's 32-bit sums, act(x Wup^T) Wdown^T without a gate projection or
// act(x Wgate^T, x Wup^T) Wdown^T with one, dense or as a mixture of experts.
//
// The router: scores = softmax over all experts of the 32-bit logits; the `top` largest are chosen (of equal scores the
// lower index first); an expert's weight is its score, as it is or divided by the chosen scores' sum.  Or (score kind
// 1) scores = sigmoid(logit) for each expert by itself, chosen by score + correction[e], weighed by the score without
// it (divided by the chosen scores' sum + 1e-20 with `renormalize`), times `scale`.  The experts' up
// matrices lie one under the other and their down matrices side by side, so that the experts of a token are a dense
// feed-forward of experts * ff hidden units whose activations are multiplied by the expert's weight, zero for the
// experts that were not chosen: the activation kernel below applies act and that weight in one pass.
#include "common.h"

#define ROUTE_MAX_EXPERTS 1024

// One wave a token.  weights [T, E] 32-bit: the chosen experts' weights, zero elsewhere.
__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ logits, int ld, float* __restrict__ weights, int ldw,
                                                         int E, int top, int renormalize) {
    int t = blockIdx.x, lane = threadIdx.x;
    constexpr int PER = ROUTE_MAX_EXPERTS / 64;
    float z[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        z[i] = e < E ? logits[(size_t)t * ld + e] : -INFINITY;
        mx = fmaxf(mx, z[i]);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        z[i] = (lane + 64 * i) < E ? expf(z[i] - mx) : -1.0f;       // (scores are >= 0: -1 marks what is not there or taken)
        sum += fmaxf(z[i], 0.0f);
    }
    float inv = 1.0f / wave_sum(sum);
    float keep[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) keep[i] = 0.0f;
    float chosen_sum = 0.0f;
    for (int r = 0; r < top; ++r) {
        float best = -1.0f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (z[i] > best) { best = z[i]; at = lane + 64 * i; }      // ascending index within a lane: the first of equals stays
        // the wave's best: the largest score, of equal scores the lowest index
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            float ob = __shfl_xor(best, d, 64);
            int oa = __shfl_xor(at, d, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (best < 0.0f) break;
        chosen_sum += best * inv;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + 64 * i == at) { keep[i] = z[i] * inv; z[i] = -1.0f; }
    }
    float norm = renormalize ? 1.0f / chosen_sum : 1.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        if (e < E) weights[(size_t)t * ldw + e] = keep[i] * norm;
    }
}

// Score kind 1.  One wave a token; the chosen experts' weights into weights [T, E], zero elsewhere.
__global__ __launch_bounds__(64) void route_topk_sigmoid_kernel(const float* __restrict__ logits, int ld, float* __restrict__ weights, int ldw,
                                                                 int E, int top, int renormalize, const float* __restrict__ correction,
                                                                 float scale) {
    int t = blockIdx.x, lane = threadIdx.x;
    constexpr int PER = ROUTE_MAX_EXPERTS / 64;
    float s[PER], c[PER], keep[PER];        // score, what the choice goes by (-inf: not there or taken), the weight kept
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        bool in = e < E;
        s[i] = in ? 1.0f / (1.0f + expf(-logits[(size_t)t * ld + e])) : 0.0f;
        c[i] = in ? s[i] + (correction ? correction[e] : 0.0f) : -INFINITY;
        keep[i] = 0.0f;
    }
    float chosen_sum = 0.0f;
    for (int r = 0; r < top; ++r) {
        float best = -INFINITY, best_s = 0.0f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (c[i] > best) { best = c[i]; best_s = s[i]; at = lane + 64 * i; }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            float ob = __shfl_xor(best, d, 64), os = __shfl_xor(best_s, d, 64);
            int oa = __shfl_xor(at, d, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; best_s = os; at = oa; }
        }
        if (at == 0x7fffffff) break;
        chosen_sum += best_s;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + 64 * i == at) { keep[i] = s[i]; c[i] = -INFINITY; }
    }
    float norm = (renormalize ? 1.0f / (chosen_sum + 1e-20f) : 1.0f) * scale;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        if (e < E) weights[(size_t)t * ldw + e] = keep[i] * norm;
    }
}

// score_kind 0: softmax over the experts (correction and scale are not used: null and 1); 1: a sigmoid for each expert,
// chosen by score + correction [E] (null: none), weights times scale.
extern "C" int llmrs_route_topk(hipStream_t stream, const float* logits, int ld, float* weights, int ldw, int n_tokens, int E, int top,
                                int renormalize, int score_kind, const float* correction, float scale) {
    LLMRS_REQUIRE(logits && weights && E > 0 && top > 0 && top <= E && ld >= E && ldw >= E, "route_topk: bad arguments");
    LLMRS_REQUIRE(E <= ROUTE_MAX_EXPERTS, "route_topk: %d experts exceed %d", E, ROUTE_MAX_EXPERTS);
    LLMRS_REQUIRE(score_kind == 0 || score_kind == 1, "route_topk: unknown score kind %d (0: softmax, 1: sigmoid)", score_kind);
    LLMRS_REQUIRE(score_kind == 1 || (correction == nullptr && scale == 1.0f), "route_topk: a correction or a scale goes with sigmoid scores");
    if (n_tokens <= 0) return 0;
    if (score_kind == 1) route_topk_sigmoid_kernel<<<n_tokens, 64, 0, stream>>>(logits, ld, weights, ldw, E, top, renormalize, correction, scale);
    else route_topk_kernel<<<n_tokens, 64, 0, stream>>>(logits, ld, weights, ldw, E, top, renormalize);
    LLMRS_LAUNCH_CHECK("route_topk");
    return 0;
}

// out[t, c] = act * (weights ? weights[t, c / ff] : 1); up 32-bit sums, out in the activation type (one rounding).
// kind 0: act = relu(up[t, c])^2.  kind 1, a gated activation on sums whose columns are (gate_0, up_0, gate_1, up_1, ...):
// g = min(up[t, 2c], limit), u = clamp(up[t, 2c + 1], -limit, limit), act = g * sigmoid(alpha * g) * (u + 1).
template <class T, int KIND>
__global__ void act_weight_kernel(const float* __restrict__ up, int ldu, const float* __restrict__ weights, int ldw, int ff, int n,
                                  long total, T* __restrict__ out, int ldo, float limit, float alpha) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    long t = i / n;
    int c = (int)(i - t * n);
    float y;
    if constexpr (KIND == 0) {
        float x = fmaxf(up[(size_t)t * ldu + c], 0.0f);
        y = x * x;
    } else {
        float2 gu = *(const float2*)(up + (size_t)t * ldu + 2 * c);
        float g = fminf(gu.x, limit), u = fminf(fmaxf(gu.y, -limit), limit);
        y = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    }
    if (weights) y *= weights[(size_t)t * ldw + c / ff];
    out[(size_t)t * ldo + c] = from_f32<T>(y);
}

// n: columns of out; up has n columns (kind 0) or 2 n (kind 1, then ldu even and up 8-byte aligned).
extern "C" int llmrs_act_weight(hipStream_t stream, int dtype, const float* up, int ldu, const float* weights, int ldw, int ff,
                                int n_tokens, int n, int kind, void* out, int ldo, float limit, float alpha) {
    LLMRS_REQUIRE(up && out && n > 0 && ldo >= n && ff > 0 && n % ff == 0, "act_weight: bad arguments");
    LLMRS_REQUIRE(kind == 0 || kind == 1, "act_weight: unknown activation %d (0: squared relu, 1: clamped gated sigmoid)", kind);
    LLMRS_REQUIRE(ldu >= (kind == 1 ? 2 * n : n), "act_weight: the sums' rows are too short");
    LLMRS_REQUIRE(kind == 0 || (ldu % 2 == 0 && ((uintptr_t)up & 7) == 0 && limit > 0.0f), "act_weight: gate and up side by side in 8-byte pairs, and a positive limit");
    LLMRS_REQUIRE(!weights || ldw >= n / ff, "act_weight: the weights' rows are too short");
    long total = (long)n_tokens * n;
    if (total <= 0) return 0;
    LLMRS_REQUIRE(ceil_div(total, 256) <= 0x7fffffff, "act_weight: too many elements for one launch");
    int blocks = ceil_div(total, 256);
#define ACT(TT, KK) act_weight_kernel<TT, KK><<<blocks, 256, 0, stream>>>(up, ldu, weights, ldw, ff, n, total, (TT*)out, ldo, limit, alpha)
    if (dtype == LLMRS_F32) { if (kind == 0) ACT(float, 0); else ACT(float, 1); }
    else if (dtype == LLMRS_BF16) { if (kind == 0) ACT(bf16, 0); else ACT(bf16, 1); }
    else return llmrs_fail("act_weight: unknown dtype %d", dtype);
#undef ACT
    LLMRS_LAUNCH_CHECK("act_weight");
    return 0;
}

// ---- the experts' rows one after the other --------------------------------------------------------------------------
// For steps of many tokens the chosen (token, expert) pairs are laid out expert by expert, each expert's rows in the
// order of their tokens, so that an expert's tokens are a dense product of their own.  counts[e]: how many tokens chose
// expert e (a wave an expert).  With the counts known: row_token[row], row_weight[row] for every row, and
// row_of[t, e] = the row of token t with expert e, or -1 (a wave an expert; an expert's first row is the sum of the
// counts before it).
__global__ __launch_bounds__(64) void route_counts_kernel(const float* __restrict__ weights, int ldw, int T, int* __restrict__ counts) {
    int e = blockIdx.x, lane = threadIdx.x, n = 0;
    for (int t = lane; t < T; t += 64) n += weights[(size_t)t * ldw + e] > 0.0f;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) n += __shfl_xor(n, d, 64);
    if (lane == 0) counts[e] = n;
}

__global__ __launch_bounds__(64) void route_rows_kernel(const float* __restrict__ weights, int ldw, int T, int E, const int* __restrict__ counts,
                                                         int* __restrict__ row_token, float* __restrict__ row_weight, int* __restrict__ row_of) {
    int e = blockIdx.x, lane = threadIdx.x, first = 0;
    for (int i = lane; i < e; i += 64) first += counts[i];
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) first += __shfl_xor(first, d, 64);
    for (int t0 = 0; t0 < T; t0 += 64) {
        int t = t0 + lane;
        float w = t < T ? weights[(size_t)t * ldw + e] : 0.0f;
        unsigned long long chosen = __ballot(w > 0.0f);
        int row = first + __popcll(chosen & ((1ull << lane) - 1ull));
        if (t < T) row_of[(size_t)t * E + e] = w > 0.0f ? row : -1;
        if (w > 0.0f) { row_token[row] = t; row_weight[row] = w; }
        first += __popcll(chosen);
    }
}

extern "C" int llmrs_route_counts(hipStream_t stream, const float* weights, int ldw, int n_tokens, int E, int* counts) {
    LLMRS_REQUIRE(weights && counts && E > 0 && ldw >= E && n_tokens >= 0 && E <= 65535, "route_counts: bad arguments");
    route_counts_kernel<<<E, 64, 0, stream>>>(weights, ldw, n_tokens, counts);
    LLMRS_LAUNCH_CHECK("route_counts");
    return 0;
}

extern "C" int llmrs_route_rows(hipStream_t stream, const float* weights, int ldw, int n_tokens, int E, const int* counts, int* row_token,
                                float* row_weight, int* row_of) {
    LLMRS_REQUIRE(weights && counts && row_token && row_weight && row_of && E > 0 && ldw >= E && n_tokens >= 0 && E <= 65535, "route_rows: bad arguments");
    route_rows_kernel<<<E, 64, 0, stream>>>(weights, ldw, n_tokens, E, counts, row_token, row_weight, row_of);
    LLMRS_LAUNCH_CHECK("route_rows");
    return 0;
}

// out[r, :] = x[rows[r], :] (rows of the activation type)
template <class T>
__global__ void gather_rows_kernel(T* __restrict__ out, int ldo, const T* __restrict__ x, int ldx, const int* __restrict__ rows, int D) {
    int r = blockIdx.x, src = rows[r];
    for (int d = threadIdx.x; d < D; d += blockDim.x) out[(size_t)r * ldo + d] = x[(size_t)src * ldx + d];
}

extern "C" int llmrs_gather_rows(hipStream_t stream, int dtype, void* out, int ldo, const void* x, int ldx, const int* rows, int n_rows, int D) {
    LLMRS_REQUIRE(out && x && rows && D > 0 && ldo >= D && ldx >= D && n_rows >= 0, "gather_rows: bad arguments");
    if (n_rows == 0) return 0;
    if (dtype == LLMRS_F32) gather_rows_kernel<float><<<n_rows, 256, 0, stream>>>((float*)out, ldo, (const float*)x, ldx, rows, D);
    else if (dtype == LLMRS_BF16) gather_rows_kernel<bf16><<<n_rows, 256, 0, stream>>>((bf16*)out, ldo, (const bf16*)x, ldx, rows, D);
    else return llmrs_fail("gather_rows: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("gather_rows");
    return 0;
}

// h[t, :] += sum over the experts e that token t chose, in ascending e, of y[row_of[t, e], :]; 32-bit.
__global__ void combine_rows_kernel(float* __restrict__ h, int ldh, const float* __restrict__ y, int ldy, const int* __restrict__ row_of, int E, int D) {
    int t = blockIdx.x;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float acc = 0.0f;
        for (int e = 0; e < E; ++e) {
            int row = row_of[(size_t)t * E + e];
            if (row >= 0) acc += y[(size_t)row * ldy + d];
        }
        h[(size_t)t * ldh + d] += acc;
    }
}

extern "C" int llmrs_combine_rows(hipStream_t stream, float* h, int ldh, const float* y, int ldy, const int* row_of, int n_tokens, int E, int D) {
    LLMRS_REQUIRE(h && y && row_of && D > 0 && ldh >= D && ldy >= D && E > 0 && n_tokens >= 0, "combine_rows: bad arguments");
    if (n_tokens == 0) return 0;
    combine_rows_kernel<<<n_tokens, 256, 0, stream>>>(h, ldh, y, ldy, row_of, E, D);
    LLMRS_LAUNCH_CHECK("combine_rows");
    return 0;
}
