// Dynamic tanh, a norm that sums nothing over the row:  y[d] = tanh(alpha * x[d]) * weight[d] + bias[d],
// with one scalar alpha (read from device memory), a weight and a bias per feature; 32-bit, one rounding on the way
// out.  Two such norms of the same rows (a layer whose two halves read the same stream through norms of their own) run
// in one launch that reads the rows once.
//
// tanh is the device library's (within a couple of units in the last place over the whole range; the kernel moves
// six to eight bytes a feature and has the arithmetic to spare).
#include "common.h"

typedef float dyt_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float tanh_f32(float z) { return tanhf(z); }

template <class T>
__device__ __forceinline__ void store4(T* dst, const float (&v)[4]);
template <>
__device__ __forceinline__ void store4<float>(float* dst, const float (&v)[4]) {
    *(dyt_f32x4*)dst = dyt_f32x4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* dst, const float (&v)[4]) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    *(bf16x4_t*)dst = bf16x4_t{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

// grid (ceil(D / (4 * 256)), rows); every thread four neighbouring features.  TWO: a second norm's output as well.
template <class T, bool TWO, bool VEC>
__global__ __launch_bounds__(256) void dyt_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                                                  const float* __restrict__ b, const float* __restrict__ alpha,
                                                  const int* __restrict__ rows, int D, T* __restrict__ out2,
                                                  const float* __restrict__ w2, const float* __restrict__ b2,
                                                  const float* __restrict__ alpha2) {
    int r = rows ? rows[blockIdx.y] : blockIdx.y;
    int d = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (d >= D) return;
    const float* src = x + (size_t)r * D + d;
    size_t at = (size_t)blockIdx.y * D + d;
    float a1 = alpha[0], a2 = TWO ? alpha2[0] : 0.0f;
    if constexpr (VEC) {
        float v[4], ww[4], bb[4], y[4];
        load4(src, v);
        load4(w + d, ww);
        load4(b + d, bb);
#pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = fmaf(tanh_f32(a1 * v[j]), ww[j], bb[j]);
        store4<T>(out + at, y);
        if constexpr (TWO) {
            load4(w2 + d, ww);
            load4(b2 + d, bb);
#pragma unroll
            for (int j = 0; j < 4; ++j) y[j] = fmaf(tanh_f32(a2 * v[j]), ww[j], bb[j]);
            store4<T>(out2 + at, y);
        }
    } else {
        for (int j = 0; j < 4 && d + j < D; ++j) {
            float v = src[j];
            out[at + j] = from_f32<T>(fmaf(tanh_f32(a1 * v), w[d + j], b[d + j]));
            if constexpr (TWO) out2[at + j] = from_f32<T>(fmaf(tanh_f32(a2 * v), w2[d + j], b2[d + j]));
        }
    }
}

// out[i, :] = tanh(alpha[0] * x[rows[i] or i, :]) * weight + bias in `dtype`; x, weight, bias, alpha 32-bit.
// out2 (with weight2, bias2, alpha2) non-null: the second norm of the same rows.
extern "C" int llmrs_dyt(hipStream_t stream, int dtype, void* out, const float* x, const float* weight, const float* bias,
                         const float* alpha, const int* rows, int n_rows, int D, void* out2, const float* weight2,
                         const float* bias2, const float* alpha2) {
    LLMRS_REQUIRE(n_rows >= 0 && D > 0 && out && x && weight && bias && alpha, "dyt: bad arguments");
    LLMRS_REQUIRE(out2 == nullptr || (weight2 && bias2 && alpha2), "dyt: the second norm needs its weight, bias and alpha");
    LLMRS_REQUIRE(dtype == LLMRS_F32 || dtype == LLMRS_BF16, "dyt: unknown dtype %d", dtype);
    if (n_rows == 0) return 0;
    LLMRS_REQUIRE(n_rows <= 65535 * 32, "dyt: %d rows are too many for one launch", n_rows);
    auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    bool vec = D % 4 == 0 && aligned(x) && aligned(weight) && aligned(bias) && aligned(out) &&
               (out2 == nullptr || (aligned(out2) && aligned(weight2) && aligned(bias2)));
    // rows go to the grid's second dimension, in launches of at most 65535
    for (int r0 = 0; r0 < n_rows; r0 += 65535) {
        int n = n_rows - r0 < 65535 ? n_rows - r0 : 65535;
        dim3 grid(ceil_div(D, 1024), n);
        const float* xs = rows ? x : x + (size_t)r0 * D;
        const int* rs = rows ? rows + r0 : nullptr;
#define DYT(T, TWO, VEC) dyt_kernel<T, TWO, VEC><<<grid, 256, 0, stream>>>((T*)out + (size_t)r0 * D, xs, weight, bias, alpha, rs, D, \
                                                                             out2 ? (T*)out2 + (size_t)r0 * D : nullptr, weight2, bias2, alpha2)
#define BY(T) do { if (out2) { if (vec) DYT(T, true, true); else DYT(T, true, false); } else { if (vec) DYT(T, false, true); else DYT(T, false, false); } } while (0)
        if (dtype == LLMRS_F32) BY(float); else BY(bf16);
#undef BY
#undef DYT
    }
    LLMRS_LAUNCH_CHECK("dyt");
    return 0;
}
