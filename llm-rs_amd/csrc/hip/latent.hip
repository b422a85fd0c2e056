// Kernels of latent attention: keys and values of all heads are matrices times one small vector c per token, and only
// c is cached.  Attention then runs in the latent space (attention*.hip, one key head of width `rank` whose values are
// its keys), between two products that carry every head's query into that space and its result out of it.
//
//   latent_finish: the input product's 32-bit sums -> q in the activation type (as it is, or RMS-normed with a weight
//                  where the queries pass a latent vector of their own); c = rmsnorm(sums_c) * weight into its page
//                  twice: as a row of the keys [page][slot][width], as a column of the values [page][width][slot];
//                  behind c, where the design has one, a key part rotated by position that all heads share
//                  (width = rank + its columns)
//   head_product:  out[t, h, :] = W[h] a[t, h, :], every head by its own small matrix, optionally times
//                  sigmoid(gate[t, h]) computed on the 32-bit sums
#include "cache_layout.h"
#include "common.h"
#include "gemm.h"

template <class T>
__global__ __launch_bounds__(256) void latent_finish_kernel(const float* __restrict__ sums, int ld, T* __restrict__ q, int ldq,
                                                            int q_size, int rank, const float* __restrict__ weight, float eps,
                                                            const int* __restrict__ slot_map, T* __restrict__ k_cache,
                                                            T* __restrict__ v_cache, int page_size, int num_pages, int write,
                                                            const float* __restrict__ q_weight, int rot,
                                                            const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                                            float gain) {
    __shared__ float partial[4];
    int t = blockIdx.x;
    const float* src = sums + (size_t)t * ld;
    float q_inv = 1.0f;
    if (q_weight) {                 // the q part is a latent vector of its own: normed over its whole width
        float ss = 0.0f;
        for (int d = threadIdx.x; d < q_size; d += 256) ss = fmaf(src[d], src[d], ss);
        ss = wave_sum(ss);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
        __syncthreads();
        q_inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)q_size + eps);
    }
    for (int d = threadIdx.x; d < q_size; d += 256) q[(size_t)t * ldq + d] = from_f32<T>(q_weight ? src[d] * q_inv * q_weight[d] : src[d]);
    if (threadIdx.x >= 128 || !write) return;
    int slot = slot_map[t];
    if (slot < 0 || slot >= num_pages * page_size) return;  // never write outside the cache
    int page = slot / page_size, off = slot % page_size;
    const int lane = threadIdx.x & 63, width = rank + rot;
    float x[8];            // features lane, lane + 64, ... (up to 512)
    if (threadIdx.x >= 64) {        // the second wave: the rotated part behind c, pairs (2i, 2i + 1) by position * inv_freq[i]
        if (rot == 0) return;
        const float pos = (float)positions[t];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int d = lane + 64 * i;
            x[i] = d < rot ? src[q_size + rank + d] : 0.0f;
            float other = __shfl_xor(x[i], 1, 64);
            if (d < rot) {
                float sn, cs;
                sincosf(pos * inv_freq[d >> 1], &sn, &cs);
                sn *= gain;
                cs *= gain;
                T y = from_f32<T>((d & 1) ? fmaf(x[i], cs, other * sn) : fmaf(x[i], cs, -other * sn));
                k_cache[k_cache_index(page, 0, off, rank + d, 1, page_size, width)] = y;
                v_cache[v_cache_index(page, 0, off, rank + d, 1, page_size, width)] = y;
            }
        }
        return;
    }
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int d = lane + 64 * i;
        x[i] = d < rank ? src[q_size + d] : 0.0f;
        ss = fmaf(x[i], x[i], ss);
    }
    float inv = 1.0f / sqrtf(wave_sum(ss) / (float)rank + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int d = lane + 64 * i;
        if (d >= rank) continue;
        T c = from_f32<T>(x[i] * inv * weight[d]);
        k_cache[k_cache_index(page, 0, off, d, 1, page_size, width)] = c;
        v_cache[v_cache_index(page, 0, off, d, 1, page_size, width)] = c;
    }
}

// sums: [n_tokens, ld] 32-bit, a token's q part (q_size columns), then its c (rank columns), then `rot` columns of a
// key part that is rotated by position and shared by all heads; q: [n_tokens, ldq] in `dtype`: the q part as it is, or
// (q_weight [q_size] given) RMS-normed over its width and multiplied by q_weight; weight: [rank] 32-bit; the caches in
// `dtype`, one key head of width rank + rot: c, then the rotated part; slot_map: [n_tokens] page * page_size + slot.
extern "C" int llmrs_latent_finish(hipStream_t stream, int dtype, const float* sums, int ld, void* q, int ldq, int n_tokens,
                                   int q_size, int rank, const float* weight, float eps, const int* slot_map, void* k_cache,
                                   void* v_cache, int page_size, int num_pages, int write, const float* q_weight, int rot,
                                   const int* positions, const float* inv_freq, float gain) {
    LLMRS_REQUIRE(n_tokens >= 0 && q_size > 0 && rank > 0 && rot >= 0 && ld >= q_size + rank + rot && ldq >= q_size, "latent_finish: bad sizes");
    LLMRS_REQUIRE(rank <= 512 && rot <= 512, "latent_finish: a latent vector of %d numbers or a rotated part of %d exceeds 512", rank, rot);
    LLMRS_REQUIRE(eps > 0.0f && weight, "latent_finish: the norm needs its weight and a positive eps");
    LLMRS_REQUIRE(rot == 0 || (rot % 2 == 0 && positions && inv_freq), "latent_finish: a rotated part has an even width, positions and frequencies");
    LLMRS_REQUIRE(!write || (page_size > 0 && num_pages > 0 && slot_map && k_cache && v_cache), "latent_finish: no cache to write");
    if (n_tokens == 0) return 0;
    if (dtype == LLMRS_F32)
        latent_finish_kernel<float><<<n_tokens, 256, 0, stream>>>(sums, ld, (float*)q, ldq, q_size, rank, weight, eps, slot_map,
                                                                   (float*)k_cache, (float*)v_cache, page_size, num_pages, write,
                                                                   q_weight, rot, positions, inv_freq, gain);
    else if (dtype == LLMRS_BF16)
        latent_finish_kernel<bf16><<<n_tokens, 256, 0, stream>>>(sums, ld, (bf16*)q, ldq, q_size, rank, weight, eps, slot_map,
                                                                  (bf16*)k_cache, (bf16*)v_cache, page_size, num_pages, write,
                                                                  q_weight, rot, positions, inv_freq, gain);
    else
        return llmrs_fail("latent_finish: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("latent_finish");
    return 0;
}

// ---- every head by its own matrix -----------------------------------------------------------------------------------
// A block of 256 threads makes 64 tokens x 64 outputs of one head: 16 inputs at a time through LDS, every thread a
// 4 x 4 corner in 32-bit multiply-adds (any sizes, any type; what 32-bit runs use, and bfloat16 at sizes the matrix-core
// kernel below does not take).
#define HP_TILE 64
#define HP_K 16
template <class T>
__global__ __launch_bounds__(256) void head_product_kernel(const T* __restrict__ a, int lda, const T* __restrict__ w,
                                                           T* __restrict__ out, int ldo, int n_tokens, int n_in, int n_out,
                                                           const float* __restrict__ gate, int ldg) {
    __shared__ float As[HP_K][HP_TILE + 4], Ws[HP_K][HP_TILE + 4];
    int h = blockIdx.z, m0 = blockIdx.y * HP_TILE, n0 = blockIdx.x * HP_TILE, tid = threadIdx.x;
    const T* ah = a + (size_t)h * n_in;
    const T* wh = w + (size_t)h * n_out * n_in;
    int tm = (tid >> 4) * 4, tn = (tid & 15) * 4;
    int lr = tid >> 2, lk = (tid & 3) * 4;          // this thread's share of a tile's loads: row lr, inputs lk .. lk + 3
    float acc[4][4] = {};
    for (int k0 = 0; k0 < n_in; k0 += HP_K) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int k = k0 + lk + j;
            As[lk + j][lr] = (m0 + lr < n_tokens && k < n_in) ? to_f32(ah[(size_t)(m0 + lr) * lda + k]) : 0.0f;
            Ws[lk + j][lr] = (n0 + lr < n_out && k < n_in) ? to_f32(wh[(size_t)(n0 + lr) * n_in + k]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < HP_K; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][tm + i]; wv[i] = Ws[k][tn + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int m = m0 + tm + i;
        if (m >= n_tokens) continue;
        float g = gate ? 1.0f / (1.0f + expf(-gate[(size_t)m * ldg + h])) : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int n = n0 + tn + j;
            if (n < n_out) out[(size_t)m * ldo + (size_t)h * n_out + n] = from_f32<T>(acc[i][j] * g);
        }
    }
}

// The same on the matrix cores, for bfloat16 with rows of whole 16-byte pieces: a wave makes MT x NT tiles of 16 tokens
// x 16 outputs with v_mfma_f32_16x16x32_bf16, its operands straight from memory (a head's matrix and a tile's rows are
// small and stay in the caches; 32 inputs a turn, lane (row, g) brings inputs 8g .. 8g + 7 of its row).  The four waves
// of a block lie along the tokens, or (ALONG_N, steps of few rows) along the outputs.  Every output's sum runs over
// the inputs in the same order whatever the tiling, so a row's result does not depend on what else is in the step.
typedef __bf16 hp_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 hp_bf16x4 __attribute__((ext_vector_type(4)));
typedef float hp_f32x4 __attribute__((ext_vector_type(4)));

template <int MT, int NT, bool ALONG_N>
__global__ __launch_bounds__(256) void head_product_mfma_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w,
                                                                bf16* __restrict__ out, int ldo, int n_tokens, int n_in, int n_out,
                                                                const float* __restrict__ gate, int ldg, int wide_stores) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, row = lane & 15, g = lane >> 4;
    const int h = blockIdx.z;
    const int m0 = (ALONG_N ? blockIdx.y : blockIdx.y * 4 + wave) * (MT * 16);
    const int n0 = (ALONG_N ? blockIdx.x * 4 + wave : blockIdx.x) * (NT * 16);
    if (m0 >= n_tokens || n0 >= n_out) return;
    const bf16* xp[MT];
    const bf16* wp[NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = a + (size_t)min(m0 + mt * 16 + row, n_tokens - 1) * lda + (size_t)h * n_in;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wp[nt] = w + ((size_t)h * n_out + min(n0 + nt * 16 + row, n_out - 1)) * n_in;
    hp_f32x4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = hp_f32x4{0.f, 0.f, 0.f, 0.f};
    const hp_bf16x8 zero = {};
#pragma unroll 2
    for (int k0 = 0; k0 < n_in; k0 += 32) {
        int k = k0 + 8 * g;
        bool in = k < n_in;                     // (rows are whole pieces of 8: a piece is inside or outside)
        hp_bf16x8 x[MT], ww[NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) x[mt] = in ? *(const hp_bf16x8*)(xp[mt] + k) : zero;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) ww[nt] = in ? *(const hp_bf16x8*)(wp[nt] + k) : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ww[nt], x[mt], acc[mt][nt], 0, 0, 0);
    }
    // the lane holds, of tile (mt, nt), token m0 + 16 mt + row and outputs n0 + 16 nt + 4 g .. + 3
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int m = m0 + mt * 16 + row;
        if (m >= n_tokens) continue;
        float gm = gate ? 1.0f / (1.0f + expf(-gate[(size_t)m * ldg + h])) : 1.0f;
        bf16* dst = out + (size_t)m * ldo + (size_t)h * n_out;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            int n = n0 + nt * 16 + 4 * g;
            if (wide_stores && n + 3 < n_out) {
                *(hp_bf16x4*)(dst + n) = hp_bf16x4{(bf16)(acc[mt][nt][0] * gm), (bf16)(acc[mt][nt][1] * gm),
                                                   (bf16)(acc[mt][nt][2] * gm), (bf16)(acc[mt][nt][3] * gm)};
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < n_out) dst[n + r] = (bf16)(acc[mt][nt][r] * gm);
            }
        }
    }
}

template <int MT, int NT, bool ALONG_N>
static void launch_head_product_mfma(hipStream_t stream, const bf16* a, int lda, const bf16* w, bf16* out, int ldo, int n_tokens,
                                     int heads, int n_in, int n_out, const float* gate, int ldg, int wide_stores) {
    dim3 grid(ceil_div(n_out, NT * 16 * (ALONG_N ? 4 : 1)), ceil_div(n_tokens, MT * 16 * (ALONG_N ? 1 : 4)), heads);
    head_product_mfma_kernel<MT, NT, ALONG_N><<<grid, 256, 0, stream>>>(a, lda, w, out, ldo, n_tokens, n_in, n_out, gate, ldg, wide_stores);
}

// a: [n_tokens, lda], head h's inputs at columns h * n_in ..; w: [heads][n_out][n_in]; out: [n_tokens, ldo], head h's
// outputs at columns h * n_out ..; all in `dtype`, sums in 32-bit.  gate: [n_tokens, ldg] 32-bit, a column a head, or null.
extern "C" int llmrs_head_product(hipStream_t stream, int dtype, const void* a, int lda, const void* w, void* out, int ldo,
                                  int n_tokens, int heads, int n_in, int n_out, int allow_mfma, const float* gate, int ldg) {
    LLMRS_REQUIRE(n_tokens >= 0 && heads > 0 && n_in > 0 && n_out > 0, "head_product: bad sizes");
    LLMRS_REQUIRE(lda >= heads * n_in && ldo >= heads * n_out && (gate == nullptr || ldg >= heads), "head_product: row stride too short");
    LLMRS_REQUIRE(heads <= 65535 && ceil_div(n_tokens, HP_TILE) <= 65535, "head_product: too many heads or tokens for one launch");
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "head_product: unknown dtype %d", dtype);
    if (n_tokens == 0) return 0;
    auto pieces = [](const void* p, int ld) { return ((uintptr_t)p & 15) == 0 && ld % 8 == 0; };
    if (dtype == LLMRS_BF16 && allow_mfma && n_in % 8 == 0 && pieces(a, lda) && pieces(w, n_in) &&
        ceil_div(n_tokens, 16) <= 65535) {
        int wide = ((uintptr_t)out & 7) == 0 && ldo % 4 == 0 && n_out % 4 == 0;
        const bf16 *ab = (const bf16*)a, *wb = (const bf16*)w;
        bf16* ob = (bf16*)out;
        if (n_tokens <= 16) launch_head_product_mfma<1, 1, true>(stream, ab, lda, wb, ob, ldo, n_tokens, heads, n_in, n_out, gate, ldg, wide);
        else if (n_tokens <= 512) launch_head_product_mfma<1, 4, false>(stream, ab, lda, wb, ob, ldo, n_tokens, heads, n_in, n_out, gate, ldg, wide);
        else launch_head_product_mfma<4, 4, false>(stream, ab, lda, wb, ob, ldo, n_tokens, heads, n_in, n_out, gate, ldg, wide);
        LLMRS_LAUNCH_CHECK("head_product");
        return 0;
    }
    dim3 grid(ceil_div(n_out, HP_TILE), ceil_div(n_tokens, HP_TILE), heads);
    if (dtype == LLMRS_F32)
        head_product_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, lda, (const float*)w, (float*)out, ldo, n_tokens, n_in, n_out, gate, ldg);
    else
        head_product_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)a, lda, (const bf16*)w, (bf16*)out, ldo, n_tokens, n_in, n_out, gate, ldg);
    LLMRS_LAUNCH_CHECK("head_product");
    return 0;
}
