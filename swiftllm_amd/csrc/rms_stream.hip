// rms_stream.hip — fp32 residual stream of models with RMS norms around every sublayer, a gate on every sublayer result and
// a short causal convolution in front of every sublayer.
//
//   swl_gated_add_rmsnorm: the step between two sublayers in one launch, one workgroup per token:
//       y   = m (+ sigmoid(s) * m2)            sublayer result (+ a second addend scaled by a per-token gate)
//       y  *= sigmoid(r + r_bias)              element-wise gate on the result
//       x  += y / rms(y) * w1                  into the fp32 stream
//       out = x / rms(x) * w2                  the next sublayer's input (or, with row_idx, the norm of selected rows only)
//     Statistics, gates and the sum are fp32; m, m2, s, r and out are the compute dtype. Weights arrive as the factor itself
//     (a loader that stores "weight around zero" adds the one).
//   swl_post_norm_add: the same step for models whose sublayers read the stream itself (norm on the sublayer's RESULT only):
//       y   = c * (a' + b')      a' = a / rms(a) * wa when wa is given, else a; b' likewise (b optional)
//       x  += y / rms(y) * w1
//       out = x in the compute dtype, or x / rms(x) * w2 when w2 is given
//     Two results normed separately and averaged (mixers side by side: c = 0.5), or two addends summed as they are (routed
//     experts + a shared expert: c = 1), or one result alone.
//   swl_causal_conv_state: out[t] = (h[t] if add_input) + sum_j w[j][c] * h[t - taps + 1 + j] per channel (w tap-major) over the tokens of
//     one sequence, for any cut of the sequence into steps: inputs of earlier steps come from the sequence's state slot,
//     which keeps the last taps - 1 inputs. The tail is double-buffered: a step reads buffer `parity` and the workgroup of
//     a portion's last token writes the other one, so no launch reads what it writes.
#include "swl_common.h"
#include "conv_tail.h"

namespace swl {

constexpr int kRsThreads = 256;

__device__ __forceinline__ float rs_block_sum(float v, float *red) {
    v = wave_allreduce_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kRsThreads / 64; ++w) t += red[w];
    return t;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(kRsThreads) void gated_add_rmsnorm_kernel(
    float *x, const T *m, const T *m2, const T *m2_gate, int64_t m2_gate_stride, const T *r, int64_t r_stride,
    const float *r_bias, const float *w1, T *out, const float *w2, const int32_t *row_idx, float eps, int width) {
    extern __shared__ float lds[];
    float *row = lds, *red = lds + width;
    const int64_t o = blockIdx.x;
    const int64_t t = row_idx ? row_idx[o] : o;
    float *xr = x + t * width;
    if (m) {
        const float s2 = m2 ? sigmoidf_(to_f(m2_gate[t * m2_gate_stride])) : 0.f;
        float ss = 0.f;
        for (int i = threadIdx.x; i < width; i += kRsThreads) {
            float y = to_f(m[t * width + i]);
            if (m2) y += s2 * to_f(m2[t * width + i]);
            if (r) y *= sigmoidf_(to_f(r[t * r_stride + i]) + r_bias[i]);
            row[i] = y;
            ss += y * y;
        }
        const float rstd = 1.0f / sqrtf(rs_block_sum(ss, red) / static_cast<float>(width) + eps);
        for (int i = threadIdx.x; i < width; i += kRsThreads) {     // (each thread touches only its own columns of row[])
            const float v = xr[i] + row[i] * rstd * w1[i];
            xr[i] = v;
            row[i] = v;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += kRsThreads) row[i] = xr[i];
    }
    if (!out) return;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kRsThreads) ss += row[i] * row[i];
    const float rstd = 1.0f / sqrtf(rs_block_sum(ss, red) / static_cast<float>(width) + eps);
    for (int i = threadIdx.x; i < width; i += kRsThreads) out[o * width + i] = to_t<T>(row[i] * rstd * w2[i]);
}

template <typename T>
__global__ __launch_bounds__(kRsThreads) void post_norm_add_kernel(float *x, const T *a, const float *wa, const T *b,
                                                                   const float *wb, float coef, const float *w1, T *out,
                                                                   const float *w2, float eps, int width) {
    extern __shared__ float lds[];
    float *ra = lds, *rb = lds + width, *red = lds + 2 * width;
    const int64_t t = blockIdx.x;
    float *xr = x + t * width;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < width; i += kRsThreads) {
        const float va = to_f(a[t * width + i]);
        ra[i] = va;
        sa += va * va;
        if (b) {
            const float vb = to_f(b[t * width + i]);
            rb[i] = vb;
            sb += vb * vb;
        }
    }
    float na = 1.f, nb = 1.f;
    if (wa) na = 1.0f / sqrtf(rs_block_sum(sa, red) / static_cast<float>(width) + eps);
    if (b && wb) nb = 1.0f / sqrtf(rs_block_sum(sb, red) / static_cast<float>(width) + eps);
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kRsThreads) {     // (each thread touches only its own columns of the rows)
        float y = wa ? ra[i] * na * wa[i] : ra[i];
        if (b) y += wb ? rb[i] * nb * wb[i] : rb[i];
        y *= coef;
        ra[i] = y;
        ss += y * y;
    }
    const float rstd = 1.0f / sqrtf(rs_block_sum(ss, red) / static_cast<float>(width) + eps);
    float sx = 0.f;
    for (int i = threadIdx.x; i < width; i += kRsThreads) {
        const float v = xr[i] + ra[i] * rstd * w1[i];
        xr[i] = v;
        ra[i] = v;
        sx += v * v;
    }
    if (!out) return;
    if (!w2) {
        for (int i = threadIdx.x; i < width; i += kRsThreads) out[t * width + i] = to_t<T>(ra[i]);
        return;
    }
    const float rx = 1.0f / sqrtf(rs_block_sum(sx, red) / static_cast<float>(width) + eps);
    for (int i = threadIdx.x; i < width; i += kRsThreads) out[t * width + i] = to_t<T>(ra[i] * rx * w2[i]);
}

template <typename T>
__global__ __launch_bounds__(kRsThreads) void causal_conv_state_kernel(
    T *out, int64_t out_stride, const T *h, int64_t h_stride, const float *w, float *state, int64_t slot_stride,
    int64_t tail_off, const int32_t *tok_pos, const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq,
    int64_t num_tokens, int C, int taps, int add_input) {
    const int64_t t = blockIdx.x;
    const ConvTail tail(state, slot_stride, tail_off, tok_pos, tok_start, tok_state, tok_seq, num_tokens, C, taps, t);
    if constexpr (sizeof(T) == 2) {
        if (ConvTail::wide_ok(h, h_stride, w, state, slot_stride, tail_off, C) && (out_stride & 7) == 0 &&
            (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
            for (int c = threadIdx.x * 8; c < C; c += kRsThreads * 8) {
                const vec8_t<T> x = load8(h + t * h_stride + c);
                float cur[8], a[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) cur[j] = to_f(x[j]);
                tail.conv8(h, h_stride, w, c, cur, a);
                vec8_t<T> o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = to_t<T>(add_input ? a[j] + cur[j] : a[j]);
                store8(out + t * out_stride + c, o);
                tail.save8(h, h_stride, c, cur);
            }
            return;
        }
    }
    for (int c = threadIdx.x; c < C; c += kRsThreads) {
        const float cur = to_f(h[t * h_stride + c]);
        float a = tail.conv(h, h_stride, w, c, cur);
        if (add_input) a += cur;
        out[t * out_stride + c] = to_t<T>(a);
        tail.save(h, h_stride, c, cur);
    }
}

inline size_t rs_lds_bytes(int width) { return (static_cast<size_t>(width) + kRsThreads / 64) * sizeof(float); }

} // namespace swl

extern "C" int swl_gated_add_rmsnorm(float *x, const void *m, const void *m2, const void *m2_gate, int64_t m2_gate_stride,
                                     const void *r, int64_t r_stride, const float *r_bias, const float *w1, void *out,
                                     const float *w2, const int32_t *row_idx, float eps, int64_t num_rows, int32_t width,
                                     int32_t dtype, swl_stream_t stream) {
    if (num_rows < 0 || width <= 0) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!x || (m && !w1) || (m2 && (!m || !m2_gate)) || (r && (!m || !r_bias)) || (out && !w2) || (row_idx && m))
        return SWL_ERR_BAD_ARG;
    if (!m && !out) return SWL_OK;
    if (num_rows > 0x7fffffffLL || swl::rs_lds_bytes(width) > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::gated_add_rmsnorm_kernel<T>), dim3(static_cast<unsigned>(num_rows)), dim3(swl::kRsThreads),
                           swl::rs_lds_bytes(width), static_cast<hipStream_t>(stream), x, static_cast<const T *>(m),
                           static_cast<const T *>(m2), static_cast<const T *>(m2_gate), m2_gate_stride,
                           static_cast<const T *>(r), r_stride, r_bias, w1, static_cast<T *>(out), w2, row_idx, eps, width);
    });
    return swl::check_launch();
}

extern "C" int swl_causal_conv_state(void *out, int64_t out_stride, const void *h, int64_t h_stride, const float *w,
                                     float *state, int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos,
                                     const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq,
                                     int64_t num_tokens, int32_t channels, int32_t taps, int32_t add_input, int32_t dtype,
                                     swl_stream_t stream) {
    if (num_tokens < 0 || channels <= 0 || taps < 1 || h_stride < channels || out_stride < channels) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !h || !w || !tok_pos || !tok_start || !tok_seq) return SWL_ERR_BAD_ARG;
    if (taps > 1 && (!state || !tok_state)) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::causal_conv_state_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kRsThreads), 0, static_cast<hipStream_t>(stream), static_cast<T *>(out), out_stride,
                           static_cast<const T *>(h), h_stride, w, state, slot_stride, tail_off, tok_pos, tok_start,
                           tok_state, tok_seq, num_tokens, channels, taps, add_input);
    });
    return swl::check_launch();
}

extern "C" int swl_post_norm_add(float *x, const void *a, const float *wa, const void *b, const float *wb, float coef,
                                 const float *w1, void *out, const float *w2, float eps, int64_t num_rows, int32_t width,
                                 int32_t dtype, swl_stream_t stream) {
    if (num_rows < 0 || width <= 0) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!x || !a || !w1 || (wb && !b) || (w2 && !out)) return SWL_ERR_BAD_ARG;
    const size_t lds = (2 * static_cast<size_t>(width) + swl::kRsThreads / 64) * sizeof(float);
    if (num_rows > 0x7fffffffLL || lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::post_norm_add_kernel<T>), dim3(static_cast<unsigned>(num_rows)), dim3(swl::kRsThreads), lds,
                           static_cast<hipStream_t>(stream), x, static_cast<const T *>(a), wa, static_cast<const T *>(b), wb,
                           coef, w1, static_cast<T *>(out), w2, eps, width);
    });
    return swl::check_launch();
}
