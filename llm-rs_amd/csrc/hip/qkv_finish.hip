// What lies between a q/k/v projection and attention for mixers that do more to q and k than rotate them:
// a short causal convolution over time, biases, a norm of q and k to unit root mean square per head (with or without a
// weight), a rotation by position, and the write of k and v into the paged cache, in one pass over the projection's
// 32-bit sums.
//
//   u[t, c] = sum_j taps[c, j] * sums[t - (K - 1 - j), c]     (with taps; rows before an entry's first token come from
//             the request's state, [K - 1][columns] 32-bit, whose last row is the token before the entry)
//   q[t, h, :] = rot(unit(u_q[t, h, :] + bias_q[h, :]) * w_q)   unit(x) = x / sqrt(mean(x^2) + eps) over the head (eps 0: x)
//   rot: features (2i, 2i + 1), i < rotary_dim / 2, turned by the angle position * inv_freq[i], cosine and sine both
//        times `gain`; the others pass
//   k likewise (weight w_k), into its page; v[t, g, :] = u_v + bias_v, into its page (values lie transposed, cache_layout.h).
// Everything is computed in 32-bit and rounded once to the activation type on the way out.
#include "cache_layout.h"
#include "common.h"

struct QkvFinishArgs {
    int n_tokens, n_heads, n_kv_heads, head_dim, v_dim;
    int in_stride, q_stride;       // elements between tokens in the sums and in q
    int page_size, num_pages, write_kv;
    float eps;                     // of the unit norm; 0: q and k are not normed
    int rotary_dim;                // 0: no rotation
    float gain;                    // cosine and sine are multiplied by this
    const float* q_weight;         // [head_dim] each, or null: what the normed q and k are multiplied by
    const float* k_weight;
    // the convolution (taps null: none): taps [columns][n_taps]; state [slots][n_taps - 1][columns] at state_stride a slot
    const float* taps;
    int n_taps, columns;
    const float* state;
    long state_stride;
    const int* q_starts;
    const int* slots;
    const int* token_entry;
};

// One wave for each (token, head of q, k or v); a block's four waves take four neighbouring tokens of the same head
// (a quarter of the blocks to hand out, and the rows that a convolution reads again lie in the same block's reach).
// NI: how many features a lane holds (heads of up to 64 NI features), so that narrow heads pay for no empty turns.
template <class T, int NI>
__global__ __launch_bounds__(256) void qkv_finish_kernel(const float* __restrict__ sums, const float* __restrict__ bias,
                                                         T* __restrict__ q, const int* __restrict__ slot_map,
                                                         T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                         const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                                         QkvFinishArgs a) {
    int t = blockIdx.x * 4 + (threadIdx.x >> 6), head = blockIdx.y, lane = threadIdx.x & 63;
    if (t >= a.n_tokens) return;
    bool is_q = head < a.n_heads, is_k = !is_q && head < a.n_heads + a.n_kv_heads;
    if (!is_q && !a.write_kv) return;
    int width = (is_q || is_k) ? a.head_dim : a.v_dim;
    int col = is_q ? head * a.head_dim
                   : is_k ? a.n_heads * a.head_dim + (head - a.n_heads) * a.head_dim
                          : (a.n_heads + a.n_kv_heads) * a.head_dim + (head - a.n_heads - a.n_kv_heads) * a.v_dim;
    const float* src = sums + (size_t)t * a.in_stride + col;
    float x[NI];           // features lane, lane + 64, ... (heads of up to 512)
    float ss = 0.0f;
    // what the later stages read from memory is asked for now, beside the rows: a step of few tokens is a chain of
    // trips to memory, and these do not depend on one another
    const bool normed = (is_q || is_k) && a.eps > 0.0f, turned = (is_q || is_k) && a.rotary_dim > 0;
    const float* nw = is_q ? a.q_weight : a.k_weight;
    float nwv[NI], freq[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        int d = lane + 64 * i;
        nwv[i] = (normed && nw && d < width) ? nw[d] : 1.0f;
        freq[i] = (turned && d < a.rotary_dim) ? inv_freq[d >> 1] : 0.0f;
    }
    const float pos = turned ? (float)positions[t] : 0.0f;
    const int slot = is_q ? 0 : slot_map[t];
    if (a.taps) {
        int e = a.token_entry[t];
        int place = t - a.q_starts[e];                     // the token's place in its entry
        const float* sp = a.n_taps > 1 ? a.state + (size_t)a.slots[e] * a.state_stride + col : nullptr;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int d = lane + 64 * i;
            float acc = 0.0f;
            if (d < width) {
                const float* w = a.taps + (size_t)(col + d) * a.n_taps;
                for (int j = 0; j < a.n_taps; ++j) {
                    int back = a.n_taps - 1 - j;           // how many tokens before this one
                    float in = place - back >= 0 ? src[d - (long)back * a.in_stride]
                                                 : sp[(size_t)(a.n_taps - 1 + place - back) * a.columns + d];
                    acc = fmaf(w[j], in, acc);
                }
            }
            x[i] = acc;
            ss = fmaf(acc, acc, ss);
        }
    } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int d = lane + 64 * i;
            x[i] = d < width ? src[d] + (bias ? bias[col + d] : 0.0f) : 0.0f;
            ss = fmaf(x[i], x[i], ss);
        }
    }
    float inv = 1.0f;
    if (normed) {
        inv = 1.0f / sqrtf(wave_sum(ss) / (float)width + a.eps);
        if (nw) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                int d = lane + 64 * i;
                x[i] = d < width ? x[i] * inv * nwv[i] : 0.0f;
            }
            inv = 1.0f;
        }
    }
    if (turned) {
        // feature d's partner d ^ 1 lies in the neighbouring lane; angles and the turn in 32-bit
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int d = lane + 64 * i;
            x[i] *= inv;
            float other = __shfl_xor(x[i], 1, 64);
            if (d < a.rotary_dim) {
                float s, c;
                sincosf(pos * freq[i], &s, &c);
                s *= a.gain;
                c *= a.gain;
                x[i] = (d & 1) ? fmaf(x[i], c, other * s) : fmaf(x[i], c, -other * s);
            }
        }
        inv = 1.0f;
    }
    if (is_q) {
        T* dst = q + (size_t)t * a.q_stride + col;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int d = lane + 64 * i;
            if (d < width) dst[d] = from_f32<T>(x[i] * inv);
        }
        return;
    }
    if (slot < 0 || slot >= a.num_pages * a.page_size) return;  // never write outside the cache
    int page = slot / a.page_size, off = slot % a.page_size;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        int d = lane + 64 * i;
        if (d >= width) continue;
        if (is_k)
            k_cache[k_cache_index(page, head - a.n_heads, off, d, a.n_kv_heads, a.page_size, a.head_dim)] = from_f32<T>(x[i] * inv);
        else
            v_cache[v_cache_index(page, head - a.n_heads - a.n_kv_heads, off, d, a.n_kv_heads, a.page_size, a.v_dim)] = from_f32<T>(x[i]);
    }
}

// The same with four neighbouring columns a lane, for heads whose width is a power of two from 8 to 256 and rows of whole
// 16-byte pieces: a wave takes 256 columns of a token (several heads, whatever they are heads of) and four tokens one after
// the other, a block sixteen tokens, whose rows a convolution finds in LDS; every load is 16 bytes; a head's sum of squares is added up within its own head_dim / 4 lanes; the two
// partners of a rotation lie in the same lane.  Which of the two kernels runs depends on the sizes and the rows'
// alignment alone, never on what a step holds.
template <class T>
__device__ __forceinline__ void qkv_store4(T* dst, const float (&v)[4]);
template <>
__device__ __forceinline__ void qkv_store4<float>(float* dst, const float (&v)[4]) {
    *(float4*)dst = float4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void qkv_store4<bf16>(bf16* dst, const float (&v)[4]) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    *(bf16x4_t*)dst = bf16x4_t{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

// TPW: tokens a wave takes, one after the other (a block takes 4 TPW): four over many rows, one in steps of few rows,
// which are a chain of trips to memory; the sums are the same bits either way.
template <class T, int TPW>
__global__ __launch_bounds__(256) void qkv_finish_wide_kernel(const float* __restrict__ sums, const float* __restrict__ bias,
                                                              T* __restrict__ q, const int* __restrict__ slot_map,
                                                              T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                              const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                                              QkvFinishArgs a) {
    // With taps: the block's rows of its 256 columns, and the n_taps - 1 rows before them, once through LDS (a row is
    // read by up to n_taps tokens): [4 TPW + n_taps - 1][64 lanes] pieces of four columns.
    extern __shared__ float4 staged[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int QKV_WIDE_TOKENS = 4 * TPW;
    const int t0 = blockIdx.x * QKV_WIDE_TOKENS;
    const int c = blockIdx.y * 256 + 4 * lane;                 // this lane's first column
    const int q_cols = a.n_heads * a.head_dim, qk_cols = q_cols + a.n_kv_heads * a.head_dim;
    const bool inside = c < a.columns, is_q = c < q_cols, is_k = !is_q && c < qk_cols, is_v = inside && !is_q && !is_k;
    const bool works = inside && (is_q || a.write_kv);
    const int d = (is_q || is_k) ? c % a.head_dim : 0;          // the first of the lane's four features within its head
    const bool normed = (is_q || is_k) && a.eps > 0.0f, turned = (is_q || is_k) && a.rotary_dim > 0 && d < a.rotary_dim;
    const int K = a.taps ? a.n_taps : 1;
    const int first = t0 - (K - 1);                            // the row that staged[0 ..] holds (rows before 0 are not there)
    if (TPW > 1 && a.taps) {      // (a wave with one token reads its few rows from memory itself: no wait for the block)
        int n_rows = min(t0 + QKV_WIDE_TOKENS, a.n_tokens) - first;
        for (int i = wave; i < n_rows; i += 4) {
            int r = first + i;
            if (r >= 0 && works) staged[i * 64 + lane] = *(const float4*)(sums + (size_t)r * a.in_stride + c);
        }
        __syncthreads();
    }
    // what does not depend on the token
    float nwv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    const float* nw = is_q ? a.q_weight : a.k_weight;
    if (works && normed && nw) load4(nw + d, nwv);
    float f0 = 0.0f, f1 = 0.0f;
    if (works && turned) {
        f0 = inv_freq[d >> 1];
        f1 = d + 2 < a.rotary_dim ? inv_freq[(d >> 1) + 1] : 0.0f;
    }
    float tw[4][4] = {};                                       // the taps of the lane's four columns, where there are at most four
    const float* w = a.taps ? a.taps + (size_t)c * K : nullptr;      // column c + f's taps at w[f * K ..]
    if (works && a.taps && K <= 4) {
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (j < K) tw[f][j] = w[f * K + j];
    }
    float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (works && !a.taps && bias) load4(bias + c, bv);

    for (int tt = 0; tt < QKV_WIDE_TOKENS / 4; ++tt) {
        const int t = t0 + wave * (QKV_WIDE_TOKENS / 4) + tt;
        if (t >= a.n_tokens) break;                            // (the whole wave: t is the wave's)
        float x[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const float pos = (works && turned) ? (float)positions[t] : 0.0f;
        const int slot = (works && !is_q) ? slot_map[t] : -1;
        if (works) {
            if (a.taps) {
                int e = a.token_entry[t];
                int place = t - a.q_starts[e];
                const float* sp = K > 1 ? a.state + (size_t)a.slots[e] * a.state_stride + c : nullptr;
                auto row = [&](int back, float (&in)[4]) {       // the row `back` tokens before this one
                    if (place - back >= 0) {
                        float4 v = TPW > 1 ? staged[(t - back - first) * 64 + lane]
                                           : *(const float4*)(sums + (size_t)(t - back) * a.in_stride + c);
                        in[0] = v.x; in[1] = v.y; in[2] = v.z; in[3] = v.w;
                    } else {
                        load4(sp + (size_t)(K - 1 + place - back) * a.columns, in);
                    }
                };
                if (K <= 4) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (j < K) {
                            float in[4];
                            row(K - 1 - j, in);
#pragma unroll
                            for (int f = 0; f < 4; ++f) x[f] = fmaf(tw[f][j], in[f], x[f]);
                        }
                } else {
                    for (int j = 0; j < K; ++j) {
                        float in[4];
                        row(K - 1 - j, in);
#pragma unroll
                        for (int f = 0; f < 4; ++f) x[f] = fmaf(w[f * K + j], in[f], x[f]);
                    }
                }
            } else {
                load4(sums + (size_t)t * a.in_stride + c, x);
#pragma unroll
                for (int f = 0; f < 4; ++f) x[f] += bv[f];
            }
        }
        // every lane takes part in the sums across lanes; a head's lanes are head_dim / 4 neighbours
        if (a.eps > 0.0f) {
            float ss = fmaf(x[0], x[0], fmaf(x[1], x[1], fmaf(x[2], x[2], x[3] * x[3])));
            for (int off = 1; off < a.head_dim / 4; off <<= 1) ss += __shfl_xor(ss, off, 64);
            if (normed) {
                float inv = 1.0f / sqrtf(ss / (float)a.head_dim + a.eps);
#pragma unroll
                for (int f = 0; f < 4; ++f) x[f] = x[f] * inv * nwv[f];
            }
        }
        if (!works) continue;
        if (turned) {
            float s, co;
            sincosf(pos * f0, &s, &co);
            s *= a.gain;
            co *= a.gain;
            float u = x[0], v = x[1];
            x[0] = fmaf(u, co, -v * s);
            x[1] = fmaf(v, co, u * s);
            if (d + 2 < a.rotary_dim) {
                sincosf(pos * f1, &s, &co);
                s *= a.gain;
                co *= a.gain;
                u = x[2];
                v = x[3];
                x[2] = fmaf(u, co, -v * s);
                x[3] = fmaf(v, co, u * s);
            }
        }
        if (is_q) {
            qkv_store4<T>(q + (size_t)t * a.q_stride + c, x);
            continue;
        }
        if (slot < 0 || slot >= a.num_pages * a.page_size) continue;  // never write outside the cache
        int page = slot / a.page_size, off = slot % a.page_size;
        if (is_k) {
            int head = (c - q_cols) / a.head_dim;
            qkv_store4<T>(k_cache + k_cache_index(page, head, off, d, a.n_kv_heads, a.page_size, a.head_dim), x);
        } else if (is_v) {
            int idx = c - qk_cols, head = idx / a.v_dim, dv = idx % a.v_dim;
#pragma unroll
            for (int f = 0; f < 4; ++f)
                v_cache[v_cache_index(page, head, off, dv + f, a.n_kv_heads, a.page_size, a.v_dim)] = from_f32<T>(x[f]);
        }
    }
}

// sums: [n_tokens, in_stride] 32-bit, a token's q heads, then its k heads, then its v heads; bias: the same columns
// (or null); q: [n_tokens, q_stride] in `dtype`; the caches in `dtype`; slot_map: [n_tokens] page * page_size + slot.
// n_kv_heads 0: the projection has no k and v (a mixer that reads another's cache).
// positions: [n_tokens], inv_freq: [rotary_dim / 2] 32-bit, for the rotation (rotary_dim 0: none); gain: see above.
// q_weight, k_weight: [head_dim] 32-bit or null.  taps: [columns of q | k | v][n_taps] 32-bit or null; then state (null when
// n_taps == 1), q_starts [n_entries + 1], slots [n_entries], token_entry [n_tokens] say where a token's earlier rows lie.
// The state is only read here: llmrs_conv_state_update brings it up to date afterwards.
extern "C" int llmrs_qkv_finish(hipStream_t stream, int dtype, const float* sums, int in_stride, const float* bias, void* q,
                                int q_stride, const int* slot_map, void* k_cache, void* v_cache, int n_tokens, int n_heads,
                                int n_kv_heads, int head_dim, int v_dim, int page_size, int num_pages, int write_kv, float eps,
                                const int* positions, const float* inv_freq, int rotary_dim, const float* q_weight,
                                const float* k_weight, float gain, const float* taps, int n_taps, const float* state,
                                long state_stride, const int* q_starts, const int* slots, const int* token_entry, int n_entries) {
    LLMRS_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0 && v_dim > 0, "qkv_finish: bad sizes");
    LLMRS_REQUIRE(head_dim <= 512 && v_dim <= 512, "qkv_finish: heads of %d / %d features exceed 512", head_dim, v_dim);
    LLMRS_REQUIRE(in_stride >= (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_dim && q_stride >= n_heads * head_dim,
                  "qkv_finish: row stride too short");
    LLMRS_REQUIRE(eps >= 0.0f, "qkv_finish: negative eps");
    LLMRS_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= head_dim, "qkv_finish: a rotation of %d features does not fit heads of %d", rotary_dim, head_dim);
    LLMRS_REQUIRE(rotary_dim == 0 || (positions && inv_freq), "qkv_finish: a rotation needs positions and frequencies");
    LLMRS_REQUIRE(!write_kv || (page_size > 0 && num_pages > 0 && slot_map && k_cache && v_cache), "qkv_finish: no cache to write");
    LLMRS_REQUIRE(n_heads + 2 * n_kv_heads <= 65535, "qkv_finish: too many heads for one launch");
    LLMRS_REQUIRE((q_weight == nullptr && k_weight == nullptr) || eps > 0.0f, "qkv_finish: a norm's weight without the norm");
    int columns = (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_dim;
    if (taps) {
        LLMRS_REQUIRE(n_taps >= 1 && bias == nullptr, "qkv_finish: a convolution needs at least one tap and goes without biases");
        LLMRS_REQUIRE(q_starts && slots && token_entry && n_entries > 0, "qkv_finish: a convolution needs the step's entries");
        LLMRS_REQUIRE(n_taps == 1 || (state && state_stride >= (long)(n_taps - 1) * columns), "qkv_finish: the convolution's state is too small");
    }
    if (n_tokens == 0) return 0;
    QkvFinishArgs a{n_tokens, n_heads, n_kv_heads, head_dim, v_dim, in_stride, q_stride, page_size, num_pages, write_kv, eps, rotary_dim,
                    gain, q_weight, k_weight, taps, n_taps, columns, state, state_stride, q_starts, slots, token_entry};
    // four columns a lane where the heads and the rows allow it
    auto pieces = [](const void* p) { return p == nullptr || ((uintptr_t)p & 15) == 0; };
    bool pow2 = head_dim >= 8 && head_dim <= 256 && (head_dim & (head_dim - 1)) == 0;
    size_t out_piece = dtype == LLMRS_F32 ? 15 : 7;
    bool wide = pow2 && v_dim % 4 == 0 && in_stride % 4 == 0 && q_stride % 4 == 0 && rotary_dim % 2 == 0 && pieces(sums) && pieces(bias) &&
                pieces(q_weight) && pieces(k_weight) && ((uintptr_t)q & out_piece) == 0 && (!write_kv || ((uintptr_t)k_cache & out_piece) == 0) &&
                (n_taps <= 1 || taps == nullptr || (pieces(state) && state_stride % 4 == 0)) && (taps == nullptr || n_taps <= 33) && (dtype == LLMRS_F32 || dtype == LLMRS_BF16);
    if (wide) {
        const int tpw = n_tokens > 256 ? 4 : 1;
        dim3 wgrid(ceil_div(n_tokens, 4 * tpw), ceil_div(columns, 256));
        size_t lds = (taps && tpw > 1) ? (size_t)(4 * tpw + n_taps - 1) * 64 * sizeof(float4) : 0;
#define QKV_WIDE(T, TPW) qkv_finish_wide_kernel<T, TPW><<<wgrid, 256, lds, stream>>>(sums, bias, (T*)q, slot_map, (T*)k_cache, (T*)v_cache, positions, inv_freq, a)
        if (dtype == LLMRS_F32) { if (tpw == 4) QKV_WIDE(float, 4); else QKV_WIDE(float, 1); }
        else { if (tpw == 4) QKV_WIDE(bf16, 4); else QKV_WIDE(bf16, 1); }
#undef QKV_WIDE
        LLMRS_LAUNCH_CHECK("qkv_finish");
        return 0;
    }
    dim3 grid(ceil_div(n_tokens, 4), n_heads + 2 * n_kv_heads);
    int widest = head_dim > v_dim ? head_dim : v_dim;
    if (dtype != LLMRS_F32 && dtype != LLMRS_BF16) return llmrs_fail("qkv_finish: unknown dtype %d", dtype);
#define QKV_FINISH(T, NI) qkv_finish_kernel<T, NI><<<grid, 256, 0, stream>>>(sums, bias, (T*)q, slot_map, (T*)k_cache, (T*)v_cache, positions, inv_freq, a)
#define QKV_FINISH_BY_WIDTH(T) do { if (widest <= 64) QKV_FINISH(T, 1); else if (widest <= 128) QKV_FINISH(T, 2); \
                                     else if (widest <= 256) QKV_FINISH(T, 4); else QKV_FINISH(T, 8); } while (0)
    if (dtype == LLMRS_F32) QKV_FINISH_BY_WIDTH(float); else QKV_FINISH_BY_WIDTH(bf16);
#undef QKV_FINISH_BY_WIDTH
#undef QKV_FINISH
    LLMRS_LAUNCH_CHECK("qkv_finish");
    return 0;
}

// ---- what some designs do to a q/k/v projection's 32-bit sums before the per-head stages above ----------------------
// In place on sums [T, q | k | v], one block for each (token, part):
//   q (and k) RMS-normed over the whole projection, all heads at once, and multiplied by a weight of that width
//     (q_weight [q_cols], k_weight [k_cols]; null: the part stays as it is);
//   v mixed with the values that an earlier layer made of the same token: v <- (1 - lambda) v + lambda first
//     (first [T, v_cols] 32-bit, lambda one number on the device), or (keep given, first null) copied out for later
//     layers to mix with.
__global__ __launch_bounds__(256) void qkv_whole_kernel(float* __restrict__ sums, int ld, int q_cols, int k_cols, int v_cols,
                                                        const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
                                                        const float* __restrict__ first, int ld_first, const float* __restrict__ lambda,
                                                        float* __restrict__ keep, int ld_keep) {
    __shared__ float partial[4];
    const int t = blockIdx.x, part = blockIdx.y;
    if (part == 2) {
        float* v = sums + (size_t)t * ld + q_cols + k_cols;
        if (first) {
            const float lam = *lambda;
            const float* f = first + (size_t)t * ld_first;
            for (int d = threadIdx.x; d < v_cols; d += 256) v[d] = (1.0f - lam) * v[d] + lam * f[d];
        } else if (keep) {
            float* o = keep + (size_t)t * ld_keep;
            for (int d = threadIdx.x; d < v_cols; d += 256) o[d] = v[d];
        }
        return;
    }
    const float* w = part == 0 ? q_weight : k_weight;
    if (!w) return;
    const int n = part == 0 ? q_cols : k_cols;
    float* x = sums + (size_t)t * ld + (part == 0 ? 0 : q_cols);
    float ss = 0.0f;
    for (int d = threadIdx.x; d < n; d += 256) ss = fmaf(x[d], x[d], ss);
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)n + eps);
    for (int d = threadIdx.x; d < n; d += 256) x[d] = x[d] * inv * w[d];
}

extern "C" int llmrs_qkv_whole(hipStream_t stream, float* sums, int ld, int n_tokens, int q_cols, int k_cols, int v_cols,
                               const float* q_weight, const float* k_weight, float eps, const float* first, int ld_first,
                               const float* lambda, float* keep, int ld_keep) {
    LLMRS_REQUIRE(sums && n_tokens >= 0 && q_cols > 0 && k_cols >= 0 && v_cols >= 0 && ld >= q_cols + k_cols + v_cols, "qkv_whole: bad sizes");
    LLMRS_REQUIRE((!q_weight && !k_weight) || eps > 0.0f, "qkv_whole: the norm needs a positive eps");
    LLMRS_REQUIRE(!k_weight || k_cols > 0, "qkv_whole: a weight for keys that are not there");
    LLMRS_REQUIRE(!first || (lambda && ld_first >= v_cols && !keep), "qkv_whole: mixing needs the first values' rows and lambda, and keeps nothing");
    LLMRS_REQUIRE(!keep || ld_keep >= v_cols, "qkv_whole: the kept values' rows are too short");
    if (n_tokens == 0) return 0;
    qkv_whole_kernel<<<dim3(n_tokens, (first || keep) ? 3 : 2), 256, 0, stream>>>(sums, ld, q_cols, k_cols, v_cols, q_weight, k_weight, eps,
                                                                                    first, ld_first, lambda, keep, ld_keep);
    LLMRS_LAUNCH_CHECK("qkv_whole");
    return 0;
}
