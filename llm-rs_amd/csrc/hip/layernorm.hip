// Layer norm with weight and bias: out[i, :] = (x[r, :] - mean) / sqrt(var + eps) * w + b, r = rows ? rows[i] : i,
// var the mean of the squared deviations from the mean (two passes over the row, not E[x^2] - E[x]^2), 32-bit
// throughout, one rounding on the way out.  One block a row.  HELD > 0: rows of up to 256 * HELD features, which a
// thread keeps in registers between the passes (one trip to memory for everything a row needs); HELD == 0: any length,
// the row read three times.  The sums' order depends on D alone.
#include "common.h"

__device__ __forceinline__ float block_sum_256(float v, float* partial) {
    v = wave_sum(v);
    __syncthreads();                                   // (whoever still reads the last sum's partials)
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = v;
    __syncthreads();
    return partial[0] + partial[1] + partial[2] + partial[3];
}

template <class T, int HELD>
__global__ __launch_bounds__(256) void layernorm_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, const int* __restrict__ rows, int D, float eps) {
    __shared__ float partial[4];
    const int r = rows ? rows[blockIdx.x] : blockIdx.x;
    const float* src = x + (size_t)r * D;
    T* dst = out + (size_t)blockIdx.x * D;
    if constexpr (HELD > 0) {
        float v[HELD], ww[HELD], bb[HELD];
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            int d = threadIdx.x + 256 * i;
            bool in = d < D;
            v[i] = in ? src[d] : 0.0f;
            ww[i] = in ? w[d] : 0.0f;
            bb[i] = in ? b[d] : 0.0f;
            s += v[i];
        }
        const float mean = block_sum_256(s, partial) / (float)D;
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            int d = threadIdx.x + 256 * i;
            v[i] = d < D ? v[i] - mean : 0.0f;
            ss = fmaf(v[i], v[i], ss);
        }
        const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)D + eps);
#pragma unroll
        for (int i = 0; i < HELD; ++i) {
            int d = threadIdx.x + 256 * i;
            if (d < D) dst[d] = from_f32<T>(fmaf(v[i] * inv, ww[i], bb[i]));
        }
    } else {
        float s = 0.0f;
        for (int d = threadIdx.x; d < D; d += 256) s += src[d];
        const float mean = block_sum_256(s, partial) / (float)D;
        float ss = 0.0f;
        for (int d = threadIdx.x; d < D; d += 256) {
            float u = src[d] - mean;
            ss = fmaf(u, u, ss);
        }
        const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)D + eps);
        for (int d = threadIdx.x; d < D; d += 256) dst[d] = from_f32<T>(fmaf((src[d] - mean) * inv, w[d], b[d]));
    }
}

template <class T>
static void launch_layernorm(hipStream_t stream, T* out, const float* x, const float* w, const float* b, const int* rows, int n_rows,
                             int D, float eps) {
    if (D <= 256 * 4) layernorm_kernel<T, 4><<<n_rows, 256, 0, stream>>>(out, x, w, b, rows, D, eps);
    else if (D <= 256 * 16) layernorm_kernel<T, 16><<<n_rows, 256, 0, stream>>>(out, x, w, b, rows, D, eps);
    else if (D <= 256 * 32) layernorm_kernel<T, 32><<<n_rows, 256, 0, stream>>>(out, x, w, b, rows, D, eps);
    else layernorm_kernel<T, 0><<<n_rows, 256, 0, stream>>>(out, x, w, b, rows, D, eps);
}

// x: [*, D] 32-bit; weight, bias: [D] 32-bit; out: [n_rows, D] in `dtype`; rows: [n_rows] or null.
extern "C" int llmrs_layernorm(hipStream_t stream, int dtype, void* out, const float* x, const float* weight, const float* bias,
                               const int* rows, int n_rows, int D, float eps) {
    LLMRS_REQUIRE(out && x && weight && bias && n_rows >= 0 && D > 0, "layernorm: bad arguments rows=%d D=%d", n_rows, D);
    LLMRS_REQUIRE(eps > 0.0f, "layernorm: eps must be positive, got %g", eps);
    if (n_rows == 0) return 0;
    if (dtype == LLMRS_F32) launch_layernorm<float>(stream, (float*)out, x, weight, bias, rows, n_rows, D, eps);
    else if (dtype == LLMRS_BF16) launch_layernorm<bf16>(stream, (bf16*)out, x, weight, bias, rows, n_rows, D, eps);
    else return llmrs_fail("layernorm: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("layernorm");
    return 0;
}
