// layernorm.hip — fp32 residual stream operators: embedding with learned positions, LayerNorm (weight + bias), and the
// fused "normalised sublayer output into the residual, then the next sublayer's input norm" step of sandwich-norm
// models. The residual x is fp32 [tokens, width]; sublayer inputs/outputs are the compute dtype (bf16 / f16 / f32);
// every statistic (mean, mean of squared deviations) is taken in fp32 with two passes over the row.
#include "swl_common.h"

namespace swl {

constexpr int kLnThreads = 256;

// Sum over the workgroup; every thread gets the total. `red` holds kLnThreads / 64 floats.
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_allreduce_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();    // (red may still be read from the previous reduction)
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kLnThreads / 64; ++w) t += red[w];
    return t;
}

// Mean and 1/sqrt(var + eps) of row[0..n) held in LDS (fp32).
__device__ __forceinline__ void row_stats(const float *row, int n, float eps, float *red, float &mean, float &rstd) {
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += kLnThreads) s += row[i];
    mean = block_sum(s, red) / static_cast<float>(n);
    float q = 0.f;
    for (int i = threadIdx.x; i < n; i += kLnThreads) {
        const float d = row[i] - mean;
        q += d * d;
    }
    const float var = block_sum(q, red) / static_cast<float>(n);
    rstd = 1.0f / sqrtf(var + eps);
}

// x[t] = embed[token[t]] * scale + pos[position[t]]  (fp32); x0 (optional) receives a copy. pos NULL: no learned positions.
template <typename T>
__global__ __launch_bounds__(kLnThreads) void embed_pos_kernel(float *x, float *x0, const T *embed, const T *pos,
                                                               const int32_t *tokens, const int32_t *positions,
                                                               float scale, int width) {
    const int64_t t = blockIdx.x;
    const T *e = embed + static_cast<int64_t>(tokens[t]) * width;
    const T *p = pos ? pos + static_cast<int64_t>(positions[t]) * width : nullptr;
    for (int i = threadIdx.x; i < width; i += kLnThreads) {
        const float v = p ? to_f(e[i]) * scale + to_f(p[i]) : to_f(e[i]) * scale;
        x[t * width + i] = v;
        if (x0) x0[t * width + i] = v;
    }
}

// out[r] = LN(x[row_idx ? row_idx[r] : r]) * w + b
template <typename T>
__global__ __launch_bounds__(kLnThreads) void layernorm_kernel(T *out, const float *x, const int32_t *row_idx,
                                                               const float *w, const float *b, float eps, int width) {
    extern __shared__ float lds[];
    float *row = lds, *red = lds + width;
    const int64_t r = blockIdx.x;
    const int64_t src = row_idx ? row_idx[r] : r;
    for (int i = threadIdx.x; i < width; i += kLnThreads) row[i] = x[src * width + i];
    __syncthreads();
    float mean, rstd;
    row_stats(row, width, eps, red, mean, rstd);
    for (int i = threadIdx.x; i < width; i += kLnThreads)
        out[r * width + i] = to_t<T>((row[i] - mean) * rstd * w[i] + b[i]);
}

// x <- x + mult * (LN(y) * w1 + b1)   [if y]
//        + x0                          [if x0]
//        + step                        [if step]
// out <- LN(x) * w2 + b2               [if out]
template <typename T>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(float *x, const T *y, float mult, const float *w1,
                                                                   const float *b1, const float *x0, const float *step,
                                                                   T *out, const float *w2, const float *b2, float eps,
                                                                   int width) {
    extern __shared__ float lds[];
    float *row = lds, *red = lds + width;
    const int64_t t = blockIdx.x;
    float mean, rstd;
    if (y) {
        for (int i = threadIdx.x; i < width; i += kLnThreads) row[i] = to_f(y[t * width + i]);
        __syncthreads();
        row_stats(row, width, eps, red, mean, rstd);
    }
    for (int i = threadIdx.x; i < width; i += kLnThreads) {     // (each thread touches only its own columns of row[])
        float v = x[t * width + i];
        if (y) v += mult * ((row[i] - mean) * rstd * w1[i] + b1[i]);
        if (x0) v += x0[t * width + i];
        if (step) v += step[i];
        x[t * width + i] = v;
        row[i] = v;
    }
    if (!out) return;
    __syncthreads();
    row_stats(row, width, eps, red, mean, rstd);
    for (int i = threadIdx.x; i < width; i += kLnThreads)
        out[t * width + i] = to_t<T>((row[i] - mean) * rstd * w2[i] + b2[i]);
}

inline size_t ln_lds_bytes(int width) { return (static_cast<size_t>(width) + kLnThreads / 64) * sizeof(float); }

} // namespace swl

extern "C" int swl_embed_pos(float *x, float *x0, const void *embed, const void *pos, const int32_t *tokens,
                             const int32_t *positions, float scale, int64_t num_tokens, int32_t width, int32_t dtype,
                             swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!x || !embed || !tokens || (pos && !positions)) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::embed_pos_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kLnThreads), 0,
                           static_cast<hipStream_t>(stream), x, x0, static_cast<const T *>(embed),
                           static_cast<const T *>(pos), tokens, positions, scale, width);
    });
    return swl::check_launch();
}

extern "C" int swl_layernorm(void *out, const float *x, const int32_t *row_idx, const float *w, const float *b, float eps,
                             int64_t num_rows, int32_t width, int32_t dtype, swl_stream_t stream) {
    if (num_rows < 0 || width <= 0) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!out || !x || !w || !b) return SWL_ERR_BAD_ARG;
    if (num_rows > 0x7fffffffLL || swl::ln_lds_bytes(width) > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::layernorm_kernel<T>), dim3(static_cast<unsigned>(num_rows)), dim3(swl::kLnThreads),
                           swl::ln_lds_bytes(width), static_cast<hipStream_t>(stream), static_cast<T *>(out), x, row_idx,
                           w, b, eps, width);
    });
    return swl::check_launch();
}

extern "C" int swl_add_layernorm(float *x, const void *y, float mult, const float *w1, const float *b1, const float *x0,
                                 const float *step, void *out, const float *w2, const float *b2, float eps,
                                 int64_t num_tokens, int32_t width, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!x || (y && (!w1 || !b1)) || (out && (!w2 || !b2))) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL || swl::ln_lds_bytes(width) > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::add_layernorm_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kLnThreads),
                           swl::ln_lds_bytes(width), static_cast<hipStream_t>(stream), x, static_cast<const T *>(y), mult,
                           w1, b1, x0, step, static_cast<T *>(out), w2, b2, eps, width);
    });
    return swl::check_launch();
}
