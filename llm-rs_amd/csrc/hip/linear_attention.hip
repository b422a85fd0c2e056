// Mixers whose memory is a matrix per head, S [key channel][value channel], carried from token to token in 32-bit:
//
//   S <- decay * S                      decay: one number per head, or one per (token, head, key channel), or one per
//                                       (token, head) together with a strength per (token, head) that the write is
//                                       multiplied by: gates that move with the token
//   u  = beta (v - S^T k)               with a write strength beta per (token, head): the delta rule;
//   u  = v                              without: plain linear attention
//   S <- S + k u^T;    o = S^T q        (the read-out sees the current token's write)
//
// and what stands around them: the activation of q, k and v where a projection leaves them raw, unit norms of q and k
// with the decay and the write strength of a gated delta rule, the RMS norm of the read-out under a sigmoid gate.
// Every column of S (one value channel) evolves by itself, so the columns are shared out over lanes; a column's rows
// are shared out over 8 to 32 lanes that add their partial dot products up by cross-lane moves.  A step's
// entries (prompt portions and single tokens alike) each start from their request's state and leave it.
#include "common.h"

#define SCAN_THREADS 256
#define SCAN_WAVES (SCAN_THREADS / 64)

struct LinearScanArgs {
    const float* q; int ldq;            // [T, qk_heads * dk]
    const float* k; int ldk;            // [T, qk_heads * dk]
    const float* v; int ldv;            // [T, heads * dv]
    const float* g; int ldg;            // [T, heads * dk] decay per key channel, or null
    const float* decay;                 // [heads] decay per head, or null (both null: none)
    const float* beta; int ldb;         // [T, heads] write strength of the delta rule, or null: plain linear attention
    const float* tdecay;                // [T, heads] decay per (token, head) and
    const float* ttake; int ldt;        // [T, heads] what the token's write is multiplied by, or both null
    int v_cols;                         // columns that v holds per head; the state's columns past them (dv > v_cols) are
                                        // written with the value 1: S's extra column is then the sum of the keys themselves
    float* state; long state_stride;    // [slots][heads][dv][dk]: a column's rows side by side, as a lane reads and leaves them
    int state_vec;                      // rows of the state may be read four at a time (dk % 4 == 0, 16-byte aligned slots)
    float* out; int ldo;                // [T, heads * dv]
    int heads, qk_heads, dk, dv;
};

// The sum of a value over the P neighbouring lanes that share a column, left in all of them.  The moves between lanes
// are the vector unit's own (quads, half rows and rows of 16 lanes mirrored; for 32 lanes the register swap between
// neighbouring rows of 16): a few cycles each, where a move through the LDS crossbar costs a trip there, and a token's
// two sums stand in the chain from token to token.
template <int CTRL>
__device__ __forceinline__ float lanes_moved(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float neighbouring_row(float x) {
    unsigned u = __float_as_uint(x);
    auto sw = __builtin_amdgcn_permlane16_swap(u, u, false, false);      // {rows 0, 0, 2, 2 of x; rows 1, 1, 3, 3 of x}
    return __uint_as_float((threadIdx.x & 16) ? sw[0] : sw[1]);
}
template <int P>
__device__ __forceinline__ float column_sum(float x) {
    static_assert(P == 8 || P == 16 || P == 32, "8, 16 or 32 lanes to a column");
    x += lanes_moved<0xB1>(x);                   // quad_perm [1, 0, 3, 2]: the neighbour
    x += lanes_moved<0x4E>(x);                   // quad_perm [2, 3, 0, 1]: the other pair of the quad
    x += lanes_moved<0x141>(x);                  // row_half_mirror: the other quad of the eight
    if constexpr (P >= 16) x += lanes_moved<0x140>(x);       // row_mirror: the other eight of the sixteen
    if constexpr (P >= 32) x += neighbouring_row(x);
    return x;
}

// P lanes share a column, each holding R of its rows (rows part * R .. part * R + R - 1; those past dk are idle: their
// keys and queries read as zero).  A block is four waves on 4 * 64 / P neighbouring columns of one head and one entry.
// A token's operands are the same for all of them: the block brings the q, k (and decay) rows of the next CHUNK tokens
// into LDS, through registers, while it folds the current CHUNK in, so that the walk from token to token waits for LDS
// and arithmetic only, never for memory.
template <int P, int R, bool DELTA, bool CHANNEL_DECAY, bool TOKEN_GATES = false>
__global__ __launch_bounds__(SCAN_THREADS) void linear_scan_kernel(const int* __restrict__ q_starts, const int* __restrict__ slots,
                                                                    LinearScanArgs a) {
    constexpr int DKP = P * R;                              // rows with the idle ones
    constexpr int CPW = 64 / P, CPB = SCAN_WAVES * CPW;     // columns of a wave, of a block
    constexpr int CHUNK = 2048 / DKP < 16 ? 2048 / DKP : 16;
    constexpr int NROW = CHUNK * DKP / SCAN_THREADS;        // elements of an operand's chunk that a thread brings
    static_assert(R % 4 == 0 && CHUNK >= 1 && CHUNK * DKP % SCAN_THREADS == 0, "rows are read four at a time");
    __shared__ __attribute__((aligned(16))) float sk[2][CHUNK][DKP];
    __shared__ __attribute__((aligned(16))) float sq[2][CHUNK][DKP];
    __shared__ __attribute__((aligned(16))) float sg[CHANNEL_DECAY ? 2 : 1][CHANNEL_DECAY ? CHUNK : 1][CHANNEL_DECAY ? DKP : 4];
    __shared__ float sv[2][CHUNK][CPB];
    __shared__ float sb[2][CHUNK];
    __shared__ float sd[TOKEN_GATES ? 2 : 1][CHUNK], st[TOKEN_GATES ? 2 : 1][CHUNK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int part = lane & (P - 1);
    const int cb = wave * CPW + lane / P;                   // this lane's column within the block
    const int col = blockIdx.x * CPB + cb;
    const int h = blockIdx.y, e = blockIdx.z;
    const int kh = h / (a.heads / a.qk_heads);
    const bool live = col < a.dv;
    const int j = live ? col : a.dv - 1;
    const int r0 = part * R;
    const int t0 = q_starts[e], t1 = q_starts[e + 1];
    if (t0 >= t1) return;
    float* sp = a.state + (size_t)slots[e] * a.state_stride + ((size_t)h * a.dv + j) * a.dk + r0;
    float s[R];
    if (a.state_vec) {
#pragma unroll
        for (int i = 0; i < R; i += 4) {
            float4 x = r0 + i < a.dk ? *(const float4*)(sp + i) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            s[i] = x.x; s[i + 1] = x.y; s[i + 2] = x.z; s[i + 3] = x.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < R; ++i) s[i] = (r0 + i < a.dk) ? sp[i] : 0.0f;
    }
    const float head_decay = (!CHANNEL_DECAY && a.decay) ? a.decay[h] : 1.0f;

    // what this thread brings of a chunk: elements tid, tid + 256, ... of [CHUNK][DKP], and one value or write strength
    constexpr int NV = (CHUNK * CPB + SCAN_THREADS - 1) / SCAN_THREADS;     // values of a chunk that a thread brings
    float rk[NROW], rq[NROW], rg[CHANNEL_DECAY ? NROW : 1], rv[NV], rb = 1.0f, rd = 1.0f, rt = 0.0f;
    auto fetch = [&](int tc) {
#pragma unroll
        for (int n = 0; n < NROW; ++n) {
            int idx = tid + n * SCAN_THREADS, i = idx / DKP, r = idx - i * DKP;
            int t = tc + i;
            bool in = t < t1 && r < a.dk;
            rk[n] = in ? a.k[(size_t)t * a.ldk + (size_t)kh * a.dk + r] : 0.0f;
            rq[n] = in ? a.q[(size_t)t * a.ldq + (size_t)kh * a.dk + r] : 0.0f;
            if constexpr (CHANNEL_DECAY) rg[n] = in ? a.g[(size_t)t * a.ldg + (size_t)h * a.dk + r] : 1.0f;
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            int idx = tid + n * SCAN_THREADS, i = idx / CPB, c = idx - i * CPB, t = tc + i, cc = blockIdx.x * CPB + c;
            rv[n] = (idx < CHUNK * CPB && t < t1 && cc < a.dv) ? (cc < a.v_cols ? a.v[(size_t)t * a.ldv + (size_t)h * a.v_cols + cc] : 1.0f) : 0.0f;
        }
        if (DELTA && tid < CHUNK) rb = tc + tid < t1 ? a.beta[(size_t)(tc + tid) * a.ldb + h] : 0.0f;
        if (TOKEN_GATES && tid < CHUNK) {
            bool in = tc + tid < t1;
            rd = in ? a.tdecay[(size_t)(tc + tid) * a.ldt + h] : 1.0f;
            rt = in ? a.ttake[(size_t)(tc + tid) * a.ldt + h] : 0.0f;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int n = 0; n < NROW; ++n) {
            int idx = tid + n * SCAN_THREADS, i = idx / DKP, r = idx - i * DKP;
            sk[buf][i][r] = rk[n];
            sq[buf][i][r] = rq[n];
            if constexpr (CHANNEL_DECAY) sg[buf][i][r] = rg[n];
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            int idx = tid + n * SCAN_THREADS;
            if (idx < CHUNK * CPB) sv[buf][idx / CPB][idx % CPB] = rv[n];
        }
        if (DELTA && tid < CHUNK) sb[buf][tid] = rb;
        if (TOKEN_GATES && tid < CHUNK) { sd[buf][tid] = rd; st[buf][tid] = rt; }
    };
    fetch(t0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int tc = t0; tc < t1; tc += CHUNK, buf ^= 1) {
        const bool more = tc + CHUNK < t1;
        if (more) fetch(tc + CHUNK);                    // on its way while this chunk is folded in
        const int n_here = min(CHUNK, t1 - tc);
#pragma unroll 4
        for (int i = 0; i < n_here; ++i) {
            float kc[R], qc[R], gc[CHANNEL_DECAY ? R : 1];
#pragma unroll
            for (int x = 0; x < R; x += 4) {
                float4 kk = *(const float4*)&sk[buf][i][r0 + x];
                float4 qq = *(const float4*)&sq[buf][i][r0 + x];
                kc[x] = kk.x; kc[x + 1] = kk.y; kc[x + 2] = kk.z; kc[x + 3] = kk.w;
                qc[x] = qq.x; qc[x + 1] = qq.y; qc[x + 2] = qq.z; qc[x + 3] = qq.w;
                if constexpr (CHANNEL_DECAY) {
                    float4 gg = *(const float4*)&sg[buf][i][r0 + x];
                    gc[x] = gg.x; gc[x + 1] = gg.y; gc[x + 2] = gg.z; gc[x + 3] = gg.w;
                }
            }
            float u = sv[buf][i][cb];
            const float now_decay = TOKEN_GATES ? sd[TOKEN_GATES ? buf : 0][i] : head_decay;
            if constexpr (TOKEN_GATES) u *= st[TOKEN_GATES ? buf : 0][i];
            if constexpr (DELTA) {
                float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
                for (int x = 0; x < R; x += 2) {
                    s[x] *= CHANNEL_DECAY ? gc[x] : now_decay;
                    s[x + 1] *= CHANNEL_DECAY ? gc[x + 1] : now_decay;
                    d0 = fmaf(kc[x], s[x], d0);
                    d1 = fmaf(kc[x + 1], s[x + 1], d1);
                }
                u = sb[buf][i] * (u - column_sum<P>(d0 + d1));
            } else {
#pragma unroll
                for (int x = 0; x < R; ++x) s[x] *= CHANNEL_DECAY ? gc[x] : now_decay;
            }
            float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
            for (int x = 0; x < R; x += 2) {
                s[x] = fmaf(kc[x], u, s[x]);
                s[x + 1] = fmaf(kc[x + 1], u, s[x + 1]);
                o0 = fmaf(qc[x], s[x], o0);
                o1 = fmaf(qc[x + 1], s[x + 1], o1);
            }
            float o = column_sum<P>(o0 + o1);
            if (live && part == 0) a.out[(size_t)(tc + i) * a.ldo + (size_t)h * a.dv + j] = o;
        }
        if (more) stash(buf ^ 1);                       // (the other buffer: nobody reads it during this chunk)
        __syncthreads();
    }
    if (live) {
        if (a.state_vec) {
#pragma unroll
            for (int i = 0; i < R; i += 4)
                if (r0 + i < a.dk) *(float4*)(sp + i) = make_float4(s[i], s[i + 1], s[i + 2], s[i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < R; ++i)
                if (r0 + i < a.dk) sp[i] = s[i];
        }
    }
}

static bool entries_given(const int* q_starts, const int* slots, int n_entries) { return q_starts && slots && n_entries > 0 && n_entries <= 65535; }

// q, k: [T, qk_heads * dk]; v: [T, heads * dv]; g: [T, heads * dk] or null; decay: [heads] or null; beta: [T, heads] or
// null (no delta correction); state: [slots][heads][dv][dk] at state_stride floats a slot, read at an entry's first
// token and left at its last; out: [T, heads * dv].  All 32-bit.  Head h reads the q and k of head h / (heads / qk_heads).
// tdecay, ttake: [T, heads] each or both null: S <- tdecay S + ttake k v^T.  v: [T, heads * v_cols]; with v_cols < dv the
// columns past v_cols are written with 1 in v's place.
extern "C" int llmrs_linear_scan(hipStream_t stream, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                 const float* g, int ldg, const float* decay, const float* beta, int ldb, float* state,
                                 long state_stride, const int* q_starts, const int* slots, int n_entries, int n_tokens,
                                 int heads, int qk_heads, int dk, int dv, float* out, int ldo, const float* tdecay, const float* ttake,
                                 int ldt, int v_cols) {
    LLMRS_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && dk > 0 && dv > 0, "linear_scan: bad sizes");
    LLMRS_REQUIRE(v_cols > 0 && v_cols <= dv, "linear_scan: v holds 1 to dv columns a head, not %d", v_cols);
    LLMRS_REQUIRE((tdecay == nullptr) == (ttake == nullptr) && (!tdecay || ldt >= heads), "linear_scan: gates per token come as a pair of [T, heads]");
    LLMRS_REQUIRE(!tdecay || (!g && !decay && !beta), "linear_scan: gates per token go with no other decay and no delta correction");
    LLMRS_REQUIRE(dk <= 512, "linear_scan: %d key channels exceed 512", dk);
    LLMRS_REQUIRE(ldq >= qk_heads * dk && ldk >= qk_heads * dk && ldv >= heads * v_cols && ldo >= heads * dv, "linear_scan: row stride too short");
    LLMRS_REQUIRE(!g || ldg >= heads * dk, "linear_scan: the decays' rows are too short");
    LLMRS_REQUIRE(!(g && decay), "linear_scan: a decay per head or per channel, not both");
    LLMRS_REQUIRE(!beta || ldb >= heads, "linear_scan: the write strengths' rows are too short");
    LLMRS_REQUIRE(state_stride >= (long)heads * dk * dv && heads <= 65535, "linear_scan: the state does not fit its slot");
    LLMRS_REQUIRE(entries_given(q_starts, slots, n_entries), "linear_scan: bad entries");
    if (n_tokens == 0) return 0;
    int state_vec = dk % 4 == 0 && state_stride % 4 == 0 && ((uintptr_t)state & 15) == 0;
    LinearScanArgs a{q, ldq, k, ldk, v, ldv, g, ldg, decay, beta, ldb, tdecay, ttake, ldt, v_cols, state, state_stride, state_vec, out, ldo, heads, qk_heads, dk, dv};
    // lanes to a column and rows to a lane by the number of key channels: eight rows a lane where that fills the lanes
#define SCAN(PP, RR, D, C, ...) linear_scan_kernel<PP, RR, D, C, ##__VA_ARGS__><<<dim3(ceil_div(dv, SCAN_WAVES * 64 / PP), heads, n_entries), SCAN_THREADS, 0, stream>>>(q_starts, slots, a)
#define BY_SIZE(D, C, ...) do { if (dk <= 32) SCAN(8, 4, D, C, ##__VA_ARGS__); else if (dk <= 64) SCAN(8, 8, D, C, ##__VA_ARGS__); \
                                else if (dk <= 128) SCAN(16, 8, D, C, ##__VA_ARGS__); else if (dk <= 256) SCAN(32, 8, D, C, ##__VA_ARGS__); \
                                else SCAN(32, 16, D, C, ##__VA_ARGS__); } while (0)
    if (tdecay) BY_SIZE(false, false, true); else if (beta && g) BY_SIZE(true, true); else if (beta) BY_SIZE(true, false); else if (g) BY_SIZE(false, true); else BY_SIZE(false, false);
#undef BY_SIZE
#undef SCAN
    LLMRS_LAUNCH_CHECK("linear_scan");
    return 0;
}

// ---- x <- silu(x) on the columns [col0, col0 + n) of 32-bit rows --------------------------------------------------
__global__ void silu_columns_kernel(float* __restrict__ x, int ld, int col0, int n, long total) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    long t = i / n;
    int c = (int)(i - t * n);
    float* p = x + (size_t)t * ld + col0 + c;
    *p = silu_f32(*p);
}

extern "C" int llmrs_silu_columns(hipStream_t stream, float* x, int ld, int n_rows, int col0, int n) {
    LLMRS_REQUIRE(x && ld >= col0 + n && col0 >= 0 && n > 0 && n_rows >= 0, "silu_columns: bad sizes");
    long total = (long)n_rows * n;
    if (total == 0) return 0;
    LLMRS_REQUIRE(ceil_div(total, 256) <= 0x7fffffff, "silu_columns: too many elements for one launch");
    silu_columns_kernel<<<ceil_div(total, 256), 256, 0, stream>>>(x, ld, col0, n, total);
    LLMRS_LAUNCH_CHECK("silu_columns");
    return 0;
}

// ---- what a gated delta rule needs between its convolutions and its recurrence ------------------------------------
// In place, all 32-bit.  One wave for each (token, unit), the units being the q heads, the k heads and the heads:
//   q head: x <- x / sqrt(sum(x^2) + unit_eps) * dk^(-1/2)          k head: x <- x / sqrt(sum(x^2) + unit_eps)
//   head h: a[t, h, :] <- exp(-exp(A_log[h]) * softplus(a[t, h, :] + dt_bias[h, :])),  b[t, h] <- sigmoid(b[t, h])
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

__global__ __launch_bounds__(64) void delta_prepare_kernel(float* __restrict__ q, int ldq, float* __restrict__ k, int ldk,
                                                            float* __restrict__ a, int lda, float* __restrict__ b, int ldb,
                                                            const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                            int heads, int qk_heads, int dk, float unit_eps) {
    int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    if (unit < 2 * qk_heads) {
        bool is_q = unit < qk_heads;
        float* row = is_q ? q + (size_t)t * ldq + (size_t)unit * dk : k + (size_t)t * ldk + (size_t)(unit - qk_heads) * dk;
        float ss = 0.0f;
        for (int d = lane; d < dk; d += 64) ss = fmaf(row[d], row[d], ss);
        float inv = 1.0f / sqrtf(wave_sum(ss) + unit_eps);
        if (is_q) inv *= 1.0f / sqrtf((float)dk);
        for (int d = lane; d < dk; d += 64) row[d] *= inv;
        return;
    }
    int h = unit - 2 * qk_heads;
    float rate = expf(A_log[h]);
    float* row = a + (size_t)t * lda + (size_t)h * dk;
    for (int d = lane; d < dk; d += 64) row[d] = expf(-rate * softplus_f32(row[d] + dt_bias[(size_t)h * dk + d]));
    if (lane == 0) {
        float* bp = b + (size_t)t * ldb + h;
        *bp = 1.0f / (1.0f + expf(-*bp));
    }
}

extern "C" int llmrs_delta_prepare(hipStream_t stream, float* q, int ldq, float* k, int ldk, float* a, int lda, float* b, int ldb,
                                   const float* A_log, const float* dt_bias, int n_tokens, int heads, int qk_heads, int dk,
                                   float unit_eps) {
    LLMRS_REQUIRE(q && k && a && b && A_log && dt_bias && heads > 0 && qk_heads > 0 && dk > 0 && n_tokens >= 0, "delta_prepare: bad arguments");
    LLMRS_REQUIRE(ldq >= qk_heads * dk && ldk >= qk_heads * dk && lda >= heads * dk && ldb >= heads, "delta_prepare: row stride too short");
    LLMRS_REQUIRE(heads + 2 * qk_heads <= 65535, "delta_prepare: too many heads for one launch");
    if (n_tokens == 0) return 0;
    delta_prepare_kernel<<<dim3(n_tokens, heads + 2 * qk_heads), 64, 0, stream>>>(q, ldq, k, ldk, a, lda, b, ldb, A_log, dt_bias,
                                                                                 heads, qk_heads, dk, unit_eps);
    LLMRS_LAUNCH_CHECK("delta_prepare");
    return 0;
}

// ---- the gates of a matrix memory with exponential gates, kept in range by a running maximum -----------------------
// Per (token, head), from the raw gate projections gi, gf (32-bit sums) and their biases:
//   i = cap tanh((gi + bi) / cap)                  the input gate's logarithm, bent into (-cap, cap)
//   f = log sigmoid(cap tanh((gf + bf) / cap))     the forget gate's logarithm
//   m_t = max(f + m_(t-1), i)                      the running maximum, carried in the request's state (it starts at 0)
//   decay = exp(f + m_(t-1) - m_t),  take = exp(i - m_t),  floor = exp(-m_t)
// One block of four waves for each (entry, head), 256 tokens a round, a token a thread: the gates' logarithms (two tanh,
// a log sigmoid) side by side in all four waves; then the first wave walks the maximum over the round's tokens in order,
// one addition and one comparison a token, exactly as token-by-token steps would, so a prompt cut anywhere gives the
// same bits; then all four waves finish their tokens' three exponentials.
__device__ __forceinline__ float log_sigmoid_f32(float z) { return z >= 0.0f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

#define GATES_THREADS 256
__global__ __launch_bounds__(GATES_THREADS) void exp_gates_kernel(const float* __restrict__ gi, const float* __restrict__ gf, int ldg,
                                                                   const float* __restrict__ bi, const float* __restrict__ bf, float cap,
                                                                   float* __restrict__ m_state, long state_stride,
                                                                   const int* __restrict__ q_starts, const int* __restrict__ slots,
                                                                   float* __restrict__ decay, float* __restrict__ take,
                                                                   float* __restrict__ floor_, int ldo) {
    __shared__ float si[GATES_THREADS], sf[GATES_THREADS], s_before[GATES_THREADS], s_mine[GATES_THREADS];
    const int h = blockIdx.x, e = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const int t0 = q_starts[e], t1 = q_starts[e + 1];
    if (t0 >= t1) return;
    float* mp = m_state + (size_t)slots[e] * state_stride + h;
    float m = *mp;                          // (every thread carries it; only the first wave's is kept up to date)
    const float b_i = bi ? bi[h] : 0.0f, b_f = bf ? bf[h] : 0.0f, inv_cap = 1.0f / cap;
    for (int tc = t0; tc < t1; tc += GATES_THREADS) {
        const int t = tc + tid, n_here = min(GATES_THREADS, t1 - tc);
        const bool in = t < t1;
        // (a place past the entry's end holds gates that leave the maximum as it is, bit for bit: m + 0 against minus
        // infinity; the walk then needs no count)
        float i = -INFINITY, f = 0.0f;
        if (in) {
            i = cap * tanhf((gi[(size_t)t * ldg + h] + b_i) * inv_cap);
            f = log_sigmoid_f32(cap * tanhf((gf[(size_t)t * ldg + h] + b_f) * inv_cap));
        }
        si[tid] = i;
        sf[tid] = f;
        __syncthreads();
        if (tid < 64) {
            for (int sub = 0; sub < n_here; sub += 64) {
                const float fi = si[sub + lane], ff = sf[sub + lane];
                // (lane j's gates by a read of that lane with j known at compile time: the walk's chain is then an
                // addition and a maximum a token, and the 128 reads do not stand in it)
                float before = 0.0f, mine = 0.0f;
#pragma unroll
                for (int j = 0; j < 64; ++j) {
                    float fj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ff), j));
                    float ij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fi), j));
                    float m_new = fmaxf(fj + m, ij);
                    if (lane == j) { before = m; mine = m_new; }
                    m = m_new;
                }
                s_before[sub + lane] = before;
                s_mine[sub + lane] = mine;
            }
        }
        __syncthreads();
        if (in) {
            const float before = s_before[tid], mine = s_mine[tid];
            decay[(size_t)t * ldo + h] = expf(f + before - mine);
            take[(size_t)t * ldo + h] = expf(i - mine);
            floor_[(size_t)t * ldo + h] = expf(-mine);
        }
    }
    if (tid == 0) *mp = m;
}

// gi, gf: [T, ldg] 32-bit, head h's raw gate at column h; bi, bf: [heads] or null; m_state: a request's maxima at
// m_state + slot * state_stride + h; decay, take, floor: [T, ldo] 32-bit.
extern "C" int llmrs_exp_gates(hipStream_t stream, const float* gi, const float* gf, int ldg, const float* bi, const float* bf, float cap,
                               float* m_state, long state_stride, const int* q_starts, const int* slots, int n_entries, int n_tokens,
                               int heads, float* decay, float* take, float* floor_, int ldo) {
    LLMRS_REQUIRE(gi && gf && m_state && decay && take && floor_ && heads > 0 && ldg >= heads && ldo >= heads, "exp_gates: bad arguments");
    LLMRS_REQUIRE(cap > 0.0f, "exp_gates: the gates' cap must be positive, got %g", cap);
    LLMRS_REQUIRE(q_starts && slots && n_entries > 0 && n_entries <= 65535, "exp_gates: bad entries");
    if (n_tokens == 0) return 0;
    exp_gates_kernel<<<dim3(heads, n_entries), GATES_THREADS, 0, stream>>>(gi, gf, ldg, bi, bf, cap, m_state, state_stride, q_starts, slots, decay, take, floor_, ldo);
    LLMRS_LAUNCH_CHECK("exp_gates");
    return 0;
}

// ---- RMS norm in groups under a sigmoid gate ------------------------------------------------------------------------
// out[t, c] = y[t, c] / sqrt(mean over c's group of y^2 + eps) * weight[c % weight_len] * sigmoid(gate[t, c]);
// groups of `group` consecutive columns; x and gate 32-bit, out in the activation type.  One block a (token, group).
// y = x, whose groups lie `group_stride` columns apart.  With `floor` [T, groups]: a group of x has one more column, n,
// behind its `group`, and y = x_scale x / (max(x_scale |n|, floor[t, group]) + den_add): a read-out divided by the
// larger of its normaliser and a floor, before the norm.
template <class T>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ gate, int ldg,
                                                             const float* __restrict__ weight, int weight_len, int group, float eps,
                                                             T* __restrict__ out, int ldo, int group_stride, const float* __restrict__ floor_,
                                                             int ldf, float x_scale, float den_add) {
    __shared__ float partial[4];
    int t = blockIdx.x, c0 = blockIdx.y * group, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* xr = x + (size_t)t * ldx + (size_t)blockIdx.y * group_stride;
    float mul = 1.0f;
    if (floor_) mul = x_scale / (fmaxf(fabsf(xr[group]) * x_scale, floor_[(size_t)t * ldf + blockIdx.y]) + den_add);
    float ss = 0.0f;
    for (int d = threadIdx.x; d < group; d += 256) {
        float y = xr[d] * mul;
        ss = fmaf(y, y, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) partial[wave] = ss;
    __syncthreads();
    float inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)group + eps);
    const float* gr = gate + (size_t)t * ldg + c0;
    T* orow = out + (size_t)t * ldo + c0;
    for (int d = threadIdx.x; d < group; d += 256) {
        float sig = 1.0f / (1.0f + expf(-gr[d]));
        orow[d] = from_f32<T>(xr[d] * mul * inv * weight[(c0 + d) % weight_len] * sig);
    }
}

extern "C" int llmrs_gated_rmsnorm(hipStream_t stream, int dtype, const float* x, int ldx, const float* gate, int ldg,
                                   const float* weight, int weight_len, int n_tokens, int n_groups, int group, float eps,
                                   void* out, int ldo, int group_stride, const float* floor_, int ldf, float x_scale, float den_add) {
    LLMRS_REQUIRE(x && gate && weight && out && n_groups > 0 && group > 0 && weight_len > 0, "gated_rmsnorm: bad arguments");
    long width = (long)n_groups * group;
    LLMRS_REQUIRE(group_stride >= group + (floor_ ? 1 : 0), "gated_rmsnorm: the groups of x overlap");
    LLMRS_REQUIRE(ldx >= (long)(n_groups - 1) * group_stride + group + (floor_ ? 1 : 0) && ldg >= width && ldo >= width && n_groups <= 65535,
                  "gated_rmsnorm: row stride too short");
    LLMRS_REQUIRE(!floor_ || ldf >= n_groups, "gated_rmsnorm: the floors' rows are too short");
    LLMRS_REQUIRE(weight_len == group || weight_len == width, "gated_rmsnorm: a weight per column of the row or of a group");
    if (n_tokens == 0) return 0;
    dim3 grid(n_tokens, n_groups);
    if (dtype == LLMRS_F32)
        gated_rmsnorm_kernel<float><<<grid, 256, 0, stream>>>(x, ldx, gate, ldg, weight, weight_len, group, eps, (float*)out, ldo, group_stride, floor_, ldf, x_scale, den_add);
    else if (dtype == LLMRS_BF16)
        gated_rmsnorm_kernel<bf16><<<grid, 256, 0, stream>>>(x, ldx, gate, ldg, weight, weight_len, group, eps, (bf16*)out, ldo, group_stride, floor_, ldf, x_scale, den_add);
    else
        return llmrs_fail("gated_rmsnorm: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("gated_rmsnorm");
    return 0;
}

// ---- sums of normed rows added into the stream ---------------------------------------------------------------------
// out[t, :] += coef * sum_i rmsnorm(x_i[t, :] + bias_i) * w_i,   i < n_in (1 or 2), all 32-bit, rows of D.
// The norm after a sublayer (n_in = 1, coef = 1), and the mean of two mixers' normed outputs (n_in = 2, coef = 1/2).
// HELD > 0: rows of up to 256 * HELD columns, which a thread keeps in registers between the two passes (everything a
// row needs from memory is then asked for at once); HELD == 0: any length, the rows read twice.
template <int HELD>
__global__ __launch_bounds__(256) void rmsnorm_sum_kernel(float* __restrict__ out, const float* __restrict__ x0, const float* __restrict__ b0,
                                                           const float* __restrict__ w0, const float* __restrict__ x1,
                                                           const float* __restrict__ b1, const float* __restrict__ w1, int D,
                                                           float coef, float eps) {
    __shared__ float partial[2][4];
    int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* r0 = x0 + (size_t)t * D;
    const float* r1 = x1 ? x1 + (size_t)t * D : nullptr;
    float* orow = out + (size_t)t * D;
    constexpr int N = HELD > 0 ? HELD : 1;
    float a[N], b[N], wa[N], wb[N], o[N];
    float s0 = 0.0f, s1 = 0.0f;
    if constexpr (HELD > 0) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int d = threadIdx.x + 256 * i;
            bool in = d < D;
            a[i] = in ? r0[d] + (b0 ? b0[d] : 0.0f) : 0.0f;
            b[i] = in && r1 ? r1[d] + (b1 ? b1[d] : 0.0f) : 0.0f;
            wa[i] = in ? w0[d] : 0.0f;
            wb[i] = in && r1 ? w1[d] : 0.0f;
            o[i] = in ? orow[d] : 0.0f;
            s0 = fmaf(a[i], a[i], s0);
            s1 = fmaf(b[i], b[i], s1);
        }
    } else {
        for (int d = threadIdx.x; d < D; d += 256) {
            float u = r0[d] + (b0 ? b0[d] : 0.0f);
            s0 = fmaf(u, u, s0);
            if (r1) {
                float v = r1[d] + (b1 ? b1[d] : 0.0f);
                s1 = fmaf(v, v, s1);
            }
        }
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    if (lane == 0) { partial[0][wave] = s0; partial[1][wave] = s1; }
    __syncthreads();
    float inv0 = 1.0f / sqrtf((partial[0][0] + partial[0][1] + partial[0][2] + partial[0][3]) / (float)D + eps);
    float inv1 = 1.0f / sqrtf((partial[1][0] + partial[1][1] + partial[1][2] + partial[1][3]) / (float)D + eps);
    if constexpr (HELD > 0) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int d = threadIdx.x + 256 * i;
            float y = a[i] * inv0 * wa[i];
            if (r1) y += b[i] * inv1 * wb[i];
            if (d < D) orow[d] = o[i] + coef * y;
        }
    } else {
        for (int d = threadIdx.x; d < D; d += 256) {
            float y = (r0[d] + (b0 ? b0[d] : 0.0f)) * inv0 * w0[d];
            if (r1) y += (r1[d] + (b1 ? b1[d] : 0.0f)) * inv1 * w1[d];
            orow[d] += coef * y;
        }
    }
}

extern "C" int llmrs_rmsnorm_sum(hipStream_t stream, float* out, const float* x0, const float* b0, const float* w0, const float* x1,
                                 const float* b1, const float* w1, int n_rows, int D, float coef, float eps) {
    LLMRS_REQUIRE(out && x0 && w0 && D > 0 && n_rows >= 0, "rmsnorm_sum: bad arguments");
    LLMRS_REQUIRE((x1 == nullptr) == (w1 == nullptr) && (x1 || !b1), "rmsnorm_sum: the second input needs rows and a weight");
    if (n_rows == 0) return 0;
    // few rows: one trip to memory for everything a row needs (8 rows of 2048: 5.3 against 7.1 us); many rows: the
    // second read comes from the cache and more waves fit a unit (2048 rows of 2048: 18 against 21 us)
    if (n_rows < 256 && D <= 256 * 4) rmsnorm_sum_kernel<4><<<n_rows, 256, 0, stream>>>(out, x0, b0, w0, x1, b1, w1, D, coef, eps);
    else if (n_rows < 256 && D <= 256 * 16) rmsnorm_sum_kernel<16><<<n_rows, 256, 0, stream>>>(out, x0, b0, w0, x1, b1, w1, D, coef, eps);
    else rmsnorm_sum_kernel<0><<<n_rows, 256, 0, stream>>>(out, x0, b0, w0, x1, b1, w1, D, coef, eps);
    LLMRS_LAUNCH_CHECK("rmsnorm_sum");
    return 0;
}
