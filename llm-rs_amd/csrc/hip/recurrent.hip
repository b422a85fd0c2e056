// Recurrent mixers: a gated recurrence whose gates read only the current token (minGRU), and a selective
// state-space scan with its short causal convolution.  Each request's state lives in 32-bit in the row of its slot
// and is carried from step to step; an entry's tokens are walked in order from the state the step before left.
// Everything that enters a recurrence is 32-bit: gates, decays, step sizes, exponentials and the state itself.
//
// A step's entries are given as on every kernel of the engine: q_starts [n_entries + 1] (where each entry's tokens
// start among the step's rows) and slots [n_entries] (the state row of each entry's request).
//
// Both recurrences are linear in the state, s_t = a_t s_{t-1} + b_t, so a long portion is cut into chunks of
// SCAN_CHUNK tokens that run side by side, in three launches:
//   local:  every chunk but an entry's last runs from a zero state and leaves (prod a_t, its end state);
//   carry:  one thread per (entry, channel) folds these in order, from the request's state, into the state each
//           chunk starts from;
//   final:  every chunk runs again from its true start and writes its tokens; the last one leaves the state.
// A chunk's place in the carry buffer is q_start / chunk length + entry + chunk: distinct for distinct chunks and
// below n_tokens / chunk length + n_entries.  Steps whose entries are all short (decoding) take the final launch
// alone, straight from and to the request's state.  Cut or not, the sums differ in rounding only.
#include "common.h"

#define SCAN_CHUNK 64                      // tokens of a chunk, and of the B and C rows that wait in LDS together
#define SCAN_CHUNK_SHORT 32                // chunks of a step with too few long ones to fill the device
#define SCAN_LOADS 8                       // tokens whose inputs a thread fetches together
#define LOG2_E 1.44269504088896341f

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ---- minGRU ---------------------------------------------------------------------------------------------------
// sums: [T, ld] 32-bit, per token the projections' sums (gate | candidate | output gate), each W wide.
//   z = sigmoid(sums_z + bias_z);  u = sums_c + bias_c;  c = u + 1/2 where u >= 0, sigmoid(u) elsewhere
//   s <- (1 - z) s + z c;  out = s * silu(sums_g)
// One thread for each (entry, chunk, channel).  chunk == 0: an entry is one chunk, from and to the request's state.
// carry: [places][2][W], the state a chunk starts from (LOCAL: ends with, from zero) and the product of its 1 - z.
template <class T, bool LOCAL>
__global__ __launch_bounds__(64) void mingru_scan_kernel(const float* __restrict__ sums, int ld, const float* __restrict__ bias_z,
                                                         const float* __restrict__ bias_c, float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ q_starts, const int* __restrict__ slots, int W,
                                                         T* __restrict__ out, int ldo, float* __restrict__ carry, int chunk) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.z;
    if (c >= W) return;
    int q0 = q_starts[e], q1 = q_starts[e + 1];
    int t0 = q0, t1 = q1;
    size_t place = 0;
    if (chunk > 0) {
        t0 = q0 + (int)blockIdx.y * chunk;
        if (t0 >= q1) return;
        t1 = min(t0 + chunk, q1);
        place = (size_t)(q0 / chunk + e + (int)blockIdx.y);
    }
    bool last_chunk = t1 == q1;
    if (LOCAL && last_chunk) return;
    float* sp = state + (size_t)slots[e] * state_stride + c;
    float s = LOCAL ? 0.0f : (chunk > 0 ? carry[place * 2 * W + c] : *sp), keep = 1.0f;
    float bz = bias_z ? bias_z[c] : 0.0f, bc = bias_c ? bias_c[c] : 0.0f;
    auto one = [&](int t, float vz, float vc, float vg) {
        float z = sigmoid_f32(vz + bz);
        float u = vc + bc;
        float cand = u >= 0.0f ? u + 0.5f : sigmoid_f32(u);
        s = (1.0f - z) * s + z * cand;
        if (LOCAL) keep *= 1.0f - z;
        else out[(size_t)t * ldo + c] = from_f32<T>(s * silu_f32(vg));
    };
    int t = t0;
    for (; t + SCAN_LOADS <= t1; t += SCAN_LOADS) {
        float vz[SCAN_LOADS], vc[SCAN_LOADS], vg[SCAN_LOADS];
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) {
            const float* row = sums + (size_t)(t + i) * ld;
            vz[i] = row[c]; vc[i] = row[W + c]; vg[i] = LOCAL ? 0.0f : row[2 * W + c];
        }
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) one(t + i, vz[i], vc[i], vg[i]);
    }
    for (; t < t1; ++t) {
        const float* row = sums + (size_t)t * ld;
        one(t, row[c], row[W + c], LOCAL ? 0.0f : row[2 * W + c]);
    }
    if (LOCAL) {
        carry[place * 2 * W + c] = s;
        carry[(place * 2 + 1) * W + c] = keep;
    } else if (last_chunk) {
        *sp = s;
    }
}

// One thread for each (entry, channel): what the chunks left becomes what each starts from.
__global__ void mingru_carry_kernel(const float* __restrict__ state, long state_stride, const int* __restrict__ q_starts,
                                    const int* __restrict__ slots, int W, float* __restrict__ carry, int chunk) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.y;
    if (c >= W) return;
    int q0 = q_starts[e], n = q_starts[e + 1] - q0;
    int chunks = (n + chunk - 1) / chunk;
    if (chunks <= 0) return;
    size_t place = (size_t)(q0 / chunk + e);
    float s = state[(size_t)slots[e] * state_stride + c];
    int k = 0;
    for (; k + SCAN_LOADS < chunks; k += SCAN_LOADS, place += SCAN_LOADS) {     // (what SCAN_LOADS chunks left, fetched together)
        float end[SCAN_LOADS], keep[SCAN_LOADS];
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) {
            end[i] = carry[(place + i) * 2 * W + c];
            keep[i] = carry[((place + i) * 2 + 1) * W + c];
        }
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) {
            carry[(place + i) * 2 * W + c] = s;
            s = fmaf(keep[i], s, end[i]);
        }
    }
    for (; k + 1 < chunks; ++k, ++place) {
        float* p = carry + place * 2 * W + c;
        float end = p[0], keep = p[W];
        p[0] = s;
        s = fmaf(keep, s, end);
    }
    carry[place * 2 * W + c] = s;
}

// ---- short causal convolution -------------------------------------------------------------------------------------
// y[t, c] = silu(bias[c] + sum_j taps[c, j] * x[t - (K - 1 - j), c]): the last tap weighs the current token.  Inputs
// from before the step's first token come from the request's state (its last K - 1 inputs, oldest first), which is
// zero at the start of a sequence.  x: the first C columns of `sums` [T, ld], 32-bit.
// A block takes `per_block` neighbouring tokens, one after the other (their inputs overlap).  KMAX: a bound of K
// that the loops over taps are unrolled to, so that a token's inputs are fetched together (0: any K, one by one).
template <class T, int KMAX>
__global__ void causal_conv_silu_kernel(const float* __restrict__ sums, int ld, const float* __restrict__ taps,
                                        const float* __restrict__ bias, const float* __restrict__ state, long state_stride,
                                        const int* __restrict__ q_starts, const int* __restrict__ slots,
                                        const int* __restrict__ token_entry, int n_tokens, int per_block, int C, int K,
                                        T* __restrict__ out, int ldo) {
    int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float b = bias ? bias[c] : 0.0f;
    float w[KMAX > 0 ? KMAX : 1];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) w[j] = j < K ? taps[(size_t)c * K + j] : 0.0f;
    int t_end = min(((int)blockIdx.y + 1) * per_block, n_tokens);
    for (int t = blockIdx.y * per_block; t < t_end; ++t) {
        int e = token_entry[t];
        int i = t - q_starts[e];                    // the token's place in its entry
        const float* sp = state + (size_t)slots[e] * state_stride;
        float acc = b;
        if (KMAX > 0) {
            float x[KMAX > 0 ? KMAX : 1];
#pragma unroll
            for (int j = 0; j < KMAX; ++j) {
                int back = K - 1 - j;               // how many tokens before this one
                x[j] = j >= K ? 0.0f : i - back >= 0 ? sums[(size_t)(t - back) * ld + c] : sp[(size_t)(K - 1 + i - back) * C + c];
            }
#pragma unroll
            for (int j = 0; j < KMAX; ++j)
                if (j < K) acc = fmaf(w[j], x[j], acc);
        } else {
            for (int j = 0; j < K; ++j) {
                int back = K - 1 - j;
                float x = i - back >= 0 ? sums[(size_t)(t - back) * ld + c] : sp[(size_t)(K - 1 + i - back) * C + c];
                acc = fmaf(taps[(size_t)c * K + j], x, acc);
            }
        }
        out[(size_t)t * ldo + c] = from_f32<T>(silu_f32(acc));
    }
}

// After the convolution: the state becomes the last K - 1 inputs of (old state, this step's inputs).
__global__ void causal_conv_state_kernel(const float* __restrict__ sums, int ld, float* __restrict__ state, long state_stride,
                                         const int* __restrict__ q_starts, const int* __restrict__ slots, int C, int K) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.y;
    if (c >= C) return;
    int t0 = q_starts[e], n = q_starts[e + 1] - t0;
    float* sp = state + (size_t)slots[e] * state_stride;
    for (int m = 0; m < K - 1; ++m) {           // ascending: a row is read before a lower one overwrites nothing it needs
        int i = n - (K - 1) + m;                // place in the entry of what row m holds afterwards
        sp[(size_t)m * C + c] = i >= 0 ? sums[(size_t)(t0 + i) * ld + c] : sp[(size_t)(m + n) * C + c];
    }
}

// ---- selective scan -----------------------------------------------------------------------------------------------
// Per channel c and state n, with step = softplus(dt[t, c] + dt_bias[c]) and A[c, n] < 0 (given state by channel):
//   S[c, n] <- exp(step A[c, n]) S[c, n] + step x[t, c] B[t, n];   y = sum_n S[c, n] C[t, n] + D[c] x[t, c]
//   out[t, c] = y * silu(gate[t, c])
// One thread for each (entry, chunk, channel) holds NS states in registers; a channel with more states is walked in
// passes of NS, the partial y of earlier passes waiting in `ypart` [T, C] 32-bit.  A block is one wave of 64 channels;
// the B and C rows of up to SCAN_CHUNK tokens, the same for every channel, wait in LDS as 32-bit values.
// chunk == 0: an entry is one chunk, from and to the request's state.
struct ScanArgs {
    const float* dt; int ld_dt;          // [T, C] sums of the step projection, 32-bit
    const float* dt_bias;                // [C]
    const float* A;                      // [N, C] (state by channel), negative
    const float* D;                      // [C]
    const float* gate; int ld_gate;      // [T, C] 32-bit (the projection's second half)
    float* state; long state_stride;     // [slots][N][C]: a wave's 64 channels read a state's values side by side
    float* ypart;                        // [T, C], needed when N > NS
    float* carry;                        // [places][N][C]: the state a chunk starts from (local launch: ends with, from zero)
    float* steps;                        // [places][C]: the sum of a chunk's step sizes
    int chunk;
    int C, N;
};

template <class T, int NS, bool LOCAL>
__global__ __launch_bounds__(64) void selective_scan_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ bc, int ldbc, int off_b,
                                                            int off_c, const int* __restrict__ q_starts, const int* __restrict__ slots,
                                                            T* __restrict__ out, int ldo, ScanArgs a) {
    __shared__ float rows_bc[SCAN_CHUNK][2 * NS];
    int c = blockIdx.x * 64 + threadIdx.x, e = blockIdx.z;
    bool live = c < a.C;
    int cc = live ? c : a.C - 1;               // (a lane past the last channel follows that channel and writes nothing)
    int q0 = q_starts[e], q1 = q_starts[e + 1];
    int t0 = q0, t1 = q1;
    size_t place = 0;
    if (a.chunk > 0) {
        t0 = q0 + (int)blockIdx.y * a.chunk;
        if (t0 >= q1) return;
        t1 = min(t0 + a.chunk, q1);
        place = (size_t)(q0 / a.chunk + e + (int)blockIdx.y);
    }
    bool last_chunk = t1 == q1;
    if (LOCAL && last_chunk) return;
    float* sp = a.state + (size_t)slots[e] * a.state_stride + cc;          // state n of this channel: sp[n * C]
    float bias = a.dt_bias ? a.dt_bias[cc] : 0.0f, Dc = a.D[cc];
    for (int n0 = 0; n0 < a.N; n0 += NS) {
        bool first = n0 == 0, last = n0 + NS >= a.N;
        float S[NS], Ac[NS];
#pragma unroll
        for (int n = 0; n < NS; ++n) {             // (states past the last stay zero: their B is zero)
            bool in = n0 + n < a.N;
            S[n] = LOCAL || !in ? 0.0f : (a.chunk > 0 ? a.carry[(place * a.N + n0 + n) * a.C + cc] : sp[(size_t)(n0 + n) * a.C]);
            Ac[n] = in ? a.A[(size_t)(n0 + n) * a.C + cc] * LOG2_E : 0.0f;     // exp(step A) as 2^(step A log2 e)
        }
        float step_sum = 0.0f;
        auto one = [&](int t, int r, float vdt, float xv, float vg) {
            float step = softplus_f32(vdt + bias);
            float sx = step * xv;
            float y = 0.0f;
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                S[n] = fmaf(__builtin_amdgcn_exp2f(step * Ac[n]), S[n], sx * rows_bc[r][n]);
                if (!LOCAL) y = fmaf(S[n], rows_bc[r][NS + n], y);
            }
            if (LOCAL) { step_sum += step; return; }
            if (!first) y += a.ypart[(size_t)t * a.C + cc];
            if (!last) { if (live) a.ypart[(size_t)t * a.C + cc] = y; return; }
            y = fmaf(Dc, xv, y);
            if (live) out[(size_t)t * ldo + c] = from_f32<T>(y * silu_f32(vg));
        };
        for (int tb = t0; tb < t1; tb += SCAN_CHUNK) {
            int rows = min(SCAN_CHUNK, t1 - tb);
            __syncthreads();
            for (int i = threadIdx.x; i < rows * NS; i += 64) {
                int r = i / NS, n = i % NS;
                bool in = n0 + n < a.N;
                const T* row = bc + (size_t)(tb + r) * ldbc + n0 + n;
                rows_bc[r][n] = in ? to_f32(row[off_b]) : 0.0f;
                if (!LOCAL) rows_bc[r][NS + n] = in ? to_f32(row[off_c]) : 0.0f;
            }
            __syncthreads();
            int r = 0;
            for (; r + SCAN_LOADS <= rows; r += SCAN_LOADS) {
                float vdt[SCAN_LOADS], vx[SCAN_LOADS], vg[SCAN_LOADS];
#pragma unroll
                for (int i = 0; i < SCAN_LOADS; ++i) {
                    size_t t = (size_t)(tb + r + i);
                    vdt[i] = a.dt[t * a.ld_dt + cc];
                    vx[i] = to_f32(x[t * ldx + cc]);
                    vg[i] = LOCAL || !last ? 0.0f : a.gate[t * a.ld_gate + cc];
                }
#pragma unroll
                for (int i = 0; i < SCAN_LOADS; ++i) one(tb + r + i, r + i, vdt[i], vx[i], vg[i]);
            }
            for (; r < rows; ++r) {
                size_t t = (size_t)(tb + r);
                one(tb + r, r, a.dt[t * a.ld_dt + cc], to_f32(x[t * ldx + cc]), LOCAL || !last ? 0.0f : a.gate[t * a.ld_gate + cc]);
            }
        }
        if (LOCAL) {
#pragma unroll
            for (int n = 0; n < NS; ++n)
                if (live && n0 + n < a.N) a.carry[(place * a.N + n0 + n) * a.C + c] = S[n];
            if (live && first) a.steps[place * a.C + c] = step_sum;
        } else if (last_chunk && live) {
#pragma unroll
            for (int n = 0; n < NS; ++n)
                if (n0 + n < a.N) sp[(size_t)(n0 + n) * a.C] = S[n];
        }
    }
}

// One thread for each (entry, state, channel): what the chunks left becomes what each starts from.  Over a chunk
// the decays multiply to exp(A[c, n] * the sum of its step sizes).  What SCAN_LOADS chunks left is fetched together.
__global__ void selective_scan_carry_kernel(const int* __restrict__ q_starts, const int* __restrict__ slots, ScanArgs a) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, n = blockIdx.y, e = blockIdx.z;
    if (c >= a.C) return;
    int q0 = q_starts[e], count = q_starts[e + 1] - q0;
    int chunks = (count + a.chunk - 1) / a.chunk;
    if (chunks <= 0) return;
    size_t place = (size_t)(q0 / a.chunk + e);
    float s = a.state[(size_t)slots[e] * a.state_stride + (size_t)n * a.C + c], An = a.A[(size_t)n * a.C + c];
    int k = 0;
    for (; k + SCAN_LOADS < chunks; k += SCAN_LOADS, place += SCAN_LOADS) {
        float end[SCAN_LOADS], sum[SCAN_LOADS];
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) {
            end[i] = a.carry[((place + i) * a.N + n) * a.C + c];
            sum[i] = a.steps[(place + i) * a.C + c];
        }
#pragma unroll
        for (int i = 0; i < SCAN_LOADS; ++i) {
            a.carry[((place + i) * a.N + n) * a.C + c] = s;
            s = fmaf(expf(An * sum[i]), s, end[i]);
        }
    }
    for (; k + 1 < chunks; ++k, ++place) {
        float* p = a.carry + (place * a.N + n) * a.C + c;
        float end = *p;
        *p = s;
        s = fmaf(expf(An * a.steps[place * a.C + c]), s, end);
    }
    a.carry[(place * a.N + n) * a.C + c] = s;
}

static bool entries_ok(const int* q_starts, const int* slots, int n_entries) { return q_starts && slots && n_entries >= 0 && n_entries <= 65535; }

// How many chunk places a step of n_tokens in n_entries can need; the carry buffers are sized with it.
extern "C" long llmrs_scan_places(long n_tokens, long n_entries) { return n_tokens / SCAN_CHUNK_SHORT + n_entries + 1; }
extern "C" int llmrs_scan_chunk() { return SCAN_CHUNK; }

static bool cut_in_chunks(int longest, const float* carry) { return longest > SCAN_CHUNK && carry != nullptr; }
// Chunks as long as leave every SIMD of the device several waves (a block is one wave of 64 channels); or the
// length that was asked for (tests run both).
static int g_chunk_asked = 0;
extern "C" int llmrs_scan_set_chunk(int tokens) {
    LLMRS_REQUIRE(tokens == 0 || tokens == SCAN_CHUNK || tokens == SCAN_CHUNK_SHORT, "scan_set_chunk: %d is not a chunk length", tokens);
    g_chunk_asked = tokens;
    return 0;
}
static int chunk_tokens(int longest, int channels) {
    if (g_chunk_asked) return g_chunk_asked;
    return (long)ceil_div(longest, SCAN_CHUNK) * ceil_div(channels, 64) >= 16L * llmrs_compute_units() ? SCAN_CHUNK : SCAN_CHUNK_SHORT;
}

// longest: the most tokens any entry brings (an upper bound will do).  carry: [llmrs_scan_places][2][W] floats, or
// null; with it, entries longer than a chunk run in chunks.
extern "C" int llmrs_mingru_scan(hipStream_t stream, int dtype, const float* sums, int ld, const float* bias_z,
                                 const float* bias_c, float* state, long state_stride, const int* q_starts, const int* slots,
                                 int n_entries, int W, void* out, int ldo, int longest, float* carry) {
    LLMRS_REQUIRE(W > 0 && ld >= 3 * W && ldo >= W && state_stride >= W, "mingru_scan: bad sizes");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries), "mingru_scan: bad entries");
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "mingru_scan: unknown dtype %d", dtype);
    if (n_entries == 0) return 0;
    bool cut = cut_in_chunks(longest, carry);
    int chunk = cut ? chunk_tokens(longest, W) : 0, chunks = cut ? ceil_div(longest, chunk) : 1;
    LLMRS_REQUIRE(chunks <= 65535, "mingru_scan: %d tokens in one entry are too many for one launch", longest);
    dim3 grid(ceil_div(W, 64), chunks, n_entries);
#define MINGRU(T, LOCAL) mingru_scan_kernel<T, LOCAL><<<grid, 64, 0, stream>>>(sums, ld, bias_z, bias_c, state, state_stride, q_starts, slots, W, (T*)out, ldo, carry, chunk)
    if (cut) {
        if (dtype == LLMRS_F32) MINGRU(float, true); else MINGRU(bf16, true);
        mingru_carry_kernel<<<dim3(ceil_div(W, 64), n_entries), 64, 0, stream>>>(state, state_stride, q_starts, slots, W, carry, chunk);
    }
    if (dtype == LLMRS_F32) MINGRU(float, false); else MINGRU(bf16, false);
#undef MINGRU
    LLMRS_LAUNCH_CHECK("mingru_scan");
    return 0;
}

// The convolution of a step's tokens and then the new state.  state: [slots][K - 1][C] at state_stride floats a slot.
extern "C" int llmrs_causal_conv_silu(hipStream_t stream, int dtype, const float* sums, int ld, const float* taps,
                                      const float* bias, float* state, long state_stride, const int* q_starts,
                                      const int* slots, const int* token_entry, int n_entries, int n_tokens, int C, int K,
                                      void* out, int ldo) {
    LLMRS_REQUIRE(C > 0 && K >= 1 && ld >= C && ldo >= C && state_stride >= (long)(K - 1) * C, "causal_conv: bad sizes");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries) && token_entry && n_tokens >= 0 && n_tokens <= 65535 * 32, "causal_conv: bad entries");
    if (n_tokens == 0) return 0;
    int per_block = n_tokens >= 1024 ? 8 : 1, threads = n_tokens >= 1024 && C >= 256 ? 256 : 64;
    LLMRS_REQUIRE(ceil_div(n_tokens, per_block) <= 65535, "causal_conv: %d tokens are too many for one launch", n_tokens);
    dim3 grid(ceil_div(C, threads), ceil_div(n_tokens, per_block));
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "causal_conv: unknown dtype %d", dtype);
#define CONV(T, KMAX) causal_conv_silu_kernel<T, KMAX><<<grid, threads, 0, stream>>>(sums, ld, taps, bias, state, state_stride, q_starts, slots, token_entry, n_tokens, per_block, C, K, (T*)out, ldo)
#define BY_TAPS(T) do { if (K <= 4) CONV(T, 4); else if (K <= 8) CONV(T, 8); else CONV(T, 0); } while (0)
    if (dtype == LLMRS_F32) BY_TAPS(float); else BY_TAPS(bf16);
#undef BY_TAPS
#undef CONV
    if (K > 1)
        causal_conv_state_kernel<<<dim3(ceil_div(C, 64), n_entries), 64, 0, stream>>>(sums, ld, state, state_stride, q_starts, slots, C, K);
    LLMRS_LAUNCH_CHECK("causal_conv");
    return 0;
}

// The state of a causal convolution alone (for a caller that convolves in a kernel of its own): the last K - 1 rows of
// (old state, this step's rows of sums) for every entry.  Launch it after whatever still reads the old state.
extern "C" int llmrs_conv_state_update(hipStream_t stream, const float* sums, int ld, float* state, long state_stride,
                                       const int* q_starts, const int* slots, int n_entries, int C, int K) {
    LLMRS_REQUIRE(C > 0 && K >= 1 && ld >= C && state_stride >= (long)(K - 1) * C, "conv_state_update: bad sizes");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries) && n_entries <= 65535, "conv_state_update: bad entries");
    if (K == 1 || n_entries == 0) return 0;
    causal_conv_state_kernel<<<dim3(ceil_div(C, 64), n_entries), 64, 0, stream>>>(sums, ld, state, state_stride, q_starts, slots, C, K);
    LLMRS_LAUNCH_CHECK("conv_state_update");
    return 0;
}

// x: [T, ldx] the convolution's output; bc: [T, ldbc] with B at column off_b and C at off_c, N wide each; both and
// `out` in `dtype`.  ypart: [T, C] 32-bit, needed only when N > 64.  longest: the most tokens any entry brings (an
// upper bound will do).  carry: [llmrs_scan_places][N + 1][C] floats, or null; with it, entries longer than a chunk
// run in chunks.
extern "C" int llmrs_selective_scan(hipStream_t stream, int dtype, const void* x, int ldx, const void* bc, int ldbc, int off_b,
                                    int off_c, const float* dt, int ld_dt, const float* dt_bias, const float* A, const float* D,
                                    const float* gate, int ld_gate, float* state, long state_stride, float* ypart,
                                    const int* q_starts, const int* slots, int n_entries, int n_tokens, int C, int N, void* out, int ldo,
                                    int longest, float* carry) {
    LLMRS_REQUIRE(C > 0 && N > 0 && ldx >= C && ld_dt >= C && ld_gate >= C && ldo >= C && state_stride >= (long)C * N, "selective_scan: bad sizes");
    LLMRS_REQUIRE(off_b >= 0 && off_c >= 0 && ldbc >= off_b + N && ldbc >= off_c + N, "selective_scan: B and C do not fit their rows");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries) && n_tokens >= 0, "selective_scan: bad entries");
    LLMRS_REQUIRE(N <= 64 || ypart != nullptr, "selective_scan: %d states a channel need room for partial sums", N);
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "selective_scan: unknown dtype %d", dtype);
    if (n_entries == 0) return 0;
    bool cut = cut_in_chunks(longest, carry);
    int chunk = cut ? chunk_tokens(longest, C) : 0, chunks = cut ? ceil_div(longest, chunk) : 1;
    LLMRS_REQUIRE(chunks <= 65535 && N <= 65535, "selective_scan: %d tokens in one entry are too many for one launch", longest);
    // (the sums of the step sizes lie behind the states the chunks carry)
    ScanArgs a{dt, ld_dt, dt_bias, A, D, gate, ld_gate, state, state_stride, ypart, carry,
               cut ? carry + (size_t)llmrs_scan_places(n_tokens, n_entries) * N * C : nullptr, chunk, C, N};
    dim3 grid(ceil_div(C, 64), chunks, n_entries);
#define SCAN(T, NS, LOCAL) selective_scan_kernel<T, NS, LOCAL><<<grid, 64, 0, stream>>>((const T*)x, ldx, (const T*)bc, ldbc, off_b, off_c, q_starts, slots, (T*)out, ldo, a)
#define BY_STATES(T, LOCAL) do { if (N <= 8) SCAN(T, 8, LOCAL); else if (N <= 16) SCAN(T, 16, LOCAL); else if (N <= 32) SCAN(T, 32, LOCAL); else SCAN(T, 64, LOCAL); } while (0)
    if (cut) {
        if (dtype == LLMRS_F32) BY_STATES(float, true); else BY_STATES(bf16, true);
        selective_scan_carry_kernel<<<dim3(ceil_div(C, 64), N, n_entries), 64, 0, stream>>>(q_starts, slots, a);
    }
    if (dtype == LLMRS_F32) BY_STATES(float, false); else BY_STATES(bf16, false);
#undef BY_STATES
#undef SCAN
    LLMRS_LAUNCH_CHECK("selective_scan");
    return 0;
}
