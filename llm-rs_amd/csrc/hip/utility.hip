// Small device utilities around the model: seeded normal fill (random-weights
// mode), dtype casts of whole tensors (weights on their way in), and the
// transform some architectures apply to their logits.
#include "../shared/normal_stream.h"
#include "common.h"

// out[i] = mean + std * normal_at(seed, first + i): the same bits as the host's
// llmrs_fill_normal_host for the same (seed, first + i).
template <class T>
__global__ void fill_normal_kernel(T* __restrict__ out, size_t n, uint64_t seed, uint64_t first, float mean, float std) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v = llmrs::normal_value(seed, first + i, mean, std);
        if constexpr (sizeof(T) == 2) ((uint16_t*)out)[i] = llmrs::ns_bf16_bits(v);
        else out[i] = v;
    }
}

extern "C" int llmrs_fill_normal(hipStream_t stream, int dtype, void* out, size_t n, uint64_t seed, uint64_t first,
                                 float mean, float std) {
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "fill_normal: unknown dtype %d", dtype);
    if (n == 0) return 0;
    LLMRS_REQUIRE(out != nullptr, "fill_normal: null output");
    int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (dtype == LLMRS_F32) fill_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, seed, first, mean, std);
    else fill_normal_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)out, n, seed, first, mean, std);
    LLMRS_LAUNCH_CHECK("fill_normal");
    return 0;
}

// dst[i] = (D)src[i]; float16 and bfloat16 widen exactly, float32 -> bfloat16 rounds to nearest even.
enum { CAST_F32 = 0, CAST_BF16 = 1, CAST_F16 = 2 };

template <class S, class D>
__global__ void cast_kernel(D* __restrict__ dst, const S* __restrict__ src, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = (D)(float)src[i];
}

extern "C" int llmrs_cast(hipStream_t stream, void* dst, int dst_dtype, const void* src, int src_dtype, size_t n) {
    if (n == 0) return 0;
    LLMRS_REQUIRE(dst != nullptr && src != nullptr, "cast: null tensor");
    int blocks = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
#define CAST(S, D) cast_kernel<S, D><<<blocks, 256, 0, stream>>>((D*)dst, (const S*)src, n)
    if (src_dtype == CAST_F32 && dst_dtype == CAST_BF16) CAST(float, bf16);
    else if (src_dtype == CAST_F32 && dst_dtype == CAST_F32) CAST(float, float);
    else if (src_dtype == CAST_BF16 && dst_dtype == CAST_F32) CAST(bf16, float);
    else if (src_dtype == CAST_BF16 && dst_dtype == CAST_BF16) CAST(bf16, bf16);
    else if (src_dtype == CAST_F16 && dst_dtype == CAST_F32) CAST(_Float16, float);
    else if (src_dtype == CAST_F16 && dst_dtype == CAST_BF16) CAST(_Float16, bf16);
    else return llmrs_fail("cast: from dtype %d to dtype %d is not offered", src_dtype, dst_dtype);
#undef CAST
    LLMRS_LAUNCH_CHECK("cast");
    return 0;
}

// logits[r, v] <- logits[r, v] * scale, then, if cap > 0, cap * tanh(that / cap), in place and in 32-bit.
__global__ void scale_softcap_kernel(float* __restrict__ logits, int ld, int V, float scale, float cap) {
    float* row = logits + (size_t)blockIdx.y * ld;
    for (int v = blockIdx.x * blockDim.x + threadIdx.x; v < V; v += gridDim.x * blockDim.x) {
        float x = row[v] * scale;
        row[v] = cap > 0.0f ? cap * tanhf(x / cap) : x;
    }
}

extern "C" int llmrs_scale_softcap_rows(hipStream_t stream, float* logits, int ld, int n_rows, int V, float scale, float cap) {
    LLMRS_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "scale_softcap_rows: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    LLMRS_REQUIRE(cap >= 0.0f, "scale_softcap_rows: the cap must not be negative, got %g", cap);
    if (n_rows == 0) return 0;
    LLMRS_REQUIRE(n_rows <= 65535, "scale_softcap_rows: %d rows in one call (at most 65535)", n_rows);
    int bx = (V + 255) / 256 < 64 ? (V + 255) / 256 : 64;
    scale_softcap_kernel<<<dim3(bx, n_rows), 256, 0, stream>>>(logits, ld, V, scale, cap);
    LLMRS_LAUNCH_CHECK("scale_softcap_rows");
    return 0;
}

// rows[t, c] += bias[c], in 32-bit: the bias of a projection whose product was added into 32-bit rows.
__global__ void add_bias_rows_kernel(float* __restrict__ rows, int ld, const float* __restrict__ bias, int n, long total) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    long t = i / n;
    int c = (int)(i - t * n);
    rows[(size_t)t * ld + c] += bias[c];
}

extern "C" int llmrs_add_bias_rows(hipStream_t stream, float* rows, int ld, const float* bias, int n_rows, int n) {
    LLMRS_REQUIRE(rows && bias && n > 0 && ld >= n && n_rows >= 0, "add_bias_rows: bad arguments");
    long total = (long)n_rows * n;
    if (total == 0) return 0;
    LLMRS_REQUIRE((total + 255) / 256 <= 0x7fffffffL, "add_bias_rows: too many elements for one launch");
    add_bias_rows_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(rows, ld, bias, n, total);
    LLMRS_LAUNCH_CHECK("add_bias_rows");
    return 0;
}

// o[t, j] *= sigmoid(gate[t, j / per]) in place: an output gate on a mixer's heads, one gate for every feature (per 1)
// or one for each group of `per` features (a head).  The gate is a product's 32-bit sums; sigmoid and product are 32-bit.
template <class T>
__global__ void sigmoid_gate_kernel(T* __restrict__ o, int ldo, const float* __restrict__ gate, int ldg, int n, int per, long total) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    long t = i / n;
    int c = (int)(i - t * n);
    float g = gate[(size_t)t * ldg + c / per];
    T* p = o + (size_t)t * ldo + c;
    *p = from_f32<T>(to_f32(*p) / (1.0f + expf(-g)));
}

extern "C" int llmrs_sigmoid_gate(hipStream_t stream, int dtype, void* o, int ldo, const float* gate, int ldg, int n_rows, int n, int per) {
    LLMRS_REQUIRE(o && gate && n > 0 && per > 0 && n % per == 0 && ldo >= n && ldg >= n / per && n_rows >= 0, "sigmoid_gate: bad arguments");
    long total = (long)n_rows * n;
    if (total == 0) return 0;
    LLMRS_REQUIRE((total + 255) / 256 <= 0x7fffffffL, "sigmoid_gate: too many elements for one launch");
    int blocks = (int)((total + 255) / 256);
    if (dtype == LLMRS_F32) sigmoid_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)o, ldo, gate, ldg, n, per, total);
    else if (dtype == LLMRS_BF16) sigmoid_gate_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)o, ldo, gate, ldg, n, per, total);
    else return llmrs_fail("sigmoid_gate: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("sigmoid_gate");
    return 0;
}
