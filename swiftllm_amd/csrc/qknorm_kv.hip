// qknorm_kv.hip — per-head RMS norm of queries and keys fused with the paged KV store.
//
// One workgroup per token of the step (prompt portions and decoded tokens alike: every token carries its own sequence
// row and position). The query heads are normalised in place inside the fused qkv projection output; the key heads are
// normalised on their way into the K pool; the value heads are copied into the V pool. Norm statistics are fp32; the
// norm weight is shared by all heads (plain weight, not one-plus).
//
// Pool layout: block b of a layer run's keys starts at k_cache + b * block_stride and holds [kv_heads, 16, dim]; its values
// start at v_cache + b * block_stride and hold [kv_heads, vdim, 16] — TRANSPOSED, the 16 tokens of a column contiguous, which is
// how the matrix-core attention wants its value operand (block_stride in elements: a block of the pool may hold the
// keys and values of several layer runs side by side, so that swapping moves one contiguous piece per block).
#include "swl_common.h"

namespace swl {

constexpr int kQkThreads = 256;
constexpr int kQkBlock = 16;    // tokens per KV block

template <typename T>
__global__ __launch_bounds__(kQkThreads) void qknorm_store_kv_kernel(
    T *qkv, const float *q_w, const float *k_w, T *k_cache, T *v_cache, const int32_t *block_table,
    const int32_t *tok_seq, const int32_t *tok_pos, int H, int G, int d, int dv, int64_t tok_stride,
    int max_blocks_per_seq, int64_t block_stride, float eps, int store) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    T *row = qkv + t * tok_stride;
    const int pos = tok_pos[t];
    int64_t blk = 0;
    if (store) blk = block_table[static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq + pos / kQkBlock];
    const int off = pos % kQkBlock;
    // heads 0..H-1: queries (in place); H..H+G-1: keys (into the pool)
    bool wide = false;
    if constexpr (sizeof(T) == 2) {
        // 16-bit heads of 32 / 64 / 128 elements on 16-byte-aligned rows: d / 8 lanes per head move 16 bytes each and several
        // heads share a wave (the group reduction stays inside d / 8 aligned lanes)
        wide = (d == 32 || d == 64 || d == 128) && (tok_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
               (!store || ((reinterpret_cast<uintptr_t>(k_cache) & 15) == 0 && (block_stride & 7) == 0));
        if (wide) {
            const int lph = d >> 3;                 // lanes per head: 4, 8 or 16
            const int hpw = 64 / lph;               // heads per wave and pass
            const int slot = lane / lph, el = lane - slot * lph;
            for (int hb = wave * hpw; hb < H + G; hb += (kQkThreads / 64) * hpw) {
                const int h = hb + slot;
                const bool live = h < H + G;
                T *src = row + static_cast<int64_t>(live ? h : 0) * d + el * 8;
                vec8_t<T> v = vec8_t<T>{};
                if (live) v = load8(src);
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) ss += to_f(v[j]) * to_f(v[j]);
                ss = lph == 4 ? group_allreduce_sum<4>(ss) : lph == 8 ? group_allreduce_sum<8>(ss) : group_allreduce_sum<16>(ss);
                const float r = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
                if (!live) continue;
                const bool is_q = h < H;
                if (!is_q && !store) continue;
                const float *wn = (is_q ? q_w : k_w) + el * 8;
                vec8_t<T> o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = to_t<T>(to_f(v[j]) * r * wn[j]);
                if (is_q) store8(src, o);
                else store8(k_cache + blk * block_stride + (static_cast<int64_t>(h - H) * kQkBlock + off) * d + el * 8, o);
            }
        }
    }
    for (int h = wave; h < H + G && !wide; h += kQkThreads / 64) {
        const bool is_q = h < H;
        const T *src = row + static_cast<int64_t>(h) * d;       // k heads follow the q heads: same formula
        float ss = 0.f;
        for (int e = lane; e < d; e += 64) {
            const float v = to_f(src[e]);
            ss += v * v;
        }
        ss = wave_allreduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
        if (is_q) {
            T *dst = row + static_cast<int64_t>(h) * d;
            for (int e = lane; e < d; e += 64) dst[e] = to_t<T>(to_f(src[e]) * r * q_w[e]);
        } else if (store) {
            const int g = h - H;
            T *dst = k_cache + blk * block_stride + (static_cast<int64_t>(g) * kQkBlock + off) * d;
            for (int e = lane; e < d; e += 64) dst[e] = to_t<T>(to_f(src[e]) * r * k_w[e]);
        }
    }
    if (store) {
        const T *vsrc = row + static_cast<int64_t>(H + G) * d;
        for (int i = threadIdx.x; i < G * dv; i += kQkThreads) {
            const int g = i / dv, c = i - g * dv;
            v_cache[blk * block_stride + (static_cast<int64_t>(g) * dv + c) * kQkBlock + off] = vsrc[i];    // transposed page
        }
    }
}


// The same store with ONE norm over the whole query projection and one over the whole key projection (all heads at once,
// a weight per element), and a query multiplier that grows with the logarithm of the position:
//   q <- q / rms(q) * q_w * (1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1)).
// store = 0: the row holds queries only (a layer that attends over another layer's keys and values).
template <typename T>
__global__ __launch_bounds__(kQkThreads) void qknorm_full_store_kv_kernel(
    T *qkv, const float *q_w, const float *k_w, T *k_cache, T *v_cache, const int32_t *block_table,
    const int32_t *tok_seq, const int32_t *tok_pos, int H, int G, int d, int dv, int64_t tok_stride,
    int max_blocks_per_seq, int64_t block_stride, float eps, float temp_coef, int temp_every, int store) {
    __shared__ float red[2][kQkThreads / 64];
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    T *row = qkv + t * tok_stride;
    const int pos = tok_pos[t];
    const int nq = H * d, nk = G * d;
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += kQkThreads) {
        const float v = to_f(row[i]);
        sq += v * v;
    }
    if (store) {
        for (int i = threadIdx.x; i < nk; i += kQkThreads) {
            const float v = to_f(row[nq + i]);
            sk += v * v;
        }
    }
    sq = wave_allreduce_sum(sq);
    sk = wave_allreduce_sum(sk);
    if (lane == 0) {
        red[0][wave] = sq;
        red[1][wave] = sk;
    }
    __syncthreads();
    sq = sk = 0.f;
#pragma unroll
    for (int w = 0; w < kQkThreads / 64; ++w) {
        sq += red[0][w];
        sk += red[1][w];
    }
    float rq = 1.0f / sqrtf(sq / static_cast<float>(nq) + eps);
    if (temp_coef != 0.f) rq *= 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every + 1));
    for (int i = threadIdx.x; i < nq; i += kQkThreads) row[i] = to_t<T>(to_f(row[i]) * q_w[i] * rq);
    if (!store) return;
    const float rk = 1.0f / sqrtf(sk / static_cast<float>(nk) + eps);
    const int64_t blk = block_table[static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq + pos / kQkBlock];
    const int off = pos % kQkBlock;
    for (int i = threadIdx.x; i < nk; i += kQkThreads) {
        const int g = i / d, e = i - g * d;
        k_cache[blk * block_stride + (static_cast<int64_t>(g) * kQkBlock + off) * d + e] = to_t<T>(to_f(row[nq + i]) * k_w[i] * rk);
    }
    const T *vsrc = row + nq + nk;
    for (int i = threadIdx.x; i < G * dv; i += kQkThreads) {
        const int g = i / dv, c = i - g * dv;
        v_cache[blk * block_stride + (static_cast<int64_t>(g) * dv + c) * kQkBlock + off] = vsrc[i];    // transposed page
    }
}


// The same store for projections WITH biases and values that may be blended with the values another layer made for the same
// token. Per token:
//   q_h <- (q_h + b_q) / rms(q_h + b_q) * w_q     in place, per head (w_q NULL: no weight)
//   k_g <- (k_g + b_k) / rms(k_g + b_k) * w_k     into the pool
//   v   <- v + b_v;  v <- (1 - mix) v + mix v_other[t]  (v_other given)   written back into the row AND into the pool
// so that the row's value columns can serve as v_other of a later layer. Biases and weights are fp32, all sums fp32.
template <typename T>
__global__ __launch_bounds__(kQkThreads) void qkv_bias_norm_store_kernel(
    T *qkv, const float *q_b, const float *k_b, const float *v_b, const float *q_w, const float *k_w, const T *v_other,
    int64_t v_other_stride, float mix, T *k_cache, T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, int H, int G, int d, int dv, int64_t tok_stride, int max_blocks_per_seq, int64_t block_stride,
    float eps, int store) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    T *row = qkv + t * tok_stride;
    const int pos = tok_pos[t];
    int64_t blk = 0;
    if (store) blk = block_table[static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq + pos / kQkBlock];
    const int off = pos % kQkBlock;
    bool wide = false;
    if constexpr (sizeof(T) == 2) {
        // 16-bit heads of 32 / 64 / 128 elements on 16-byte-aligned rows: d / 8 lanes per head move 16 bytes each and several
        // heads share a wave (the group reduction stays inside d / 8 aligned lanes)
        wide = (d == 32 || d == 64 || d == 128) && (tok_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
               (!store || ((reinterpret_cast<uintptr_t>(k_cache) & 15) == 0 && (block_stride & 7) == 0)) &&
               ((reinterpret_cast<uintptr_t>(q_b) | reinterpret_cast<uintptr_t>(k_b)) & 15) == 0;
        if (wide) {
            const int lph = d >> 3;                 // lanes per head: 4, 8 or 16
            const int hpw = 64 / lph;               // heads per wave and pass
            const int slot = lane / lph, el = lane - slot * lph;
            for (int hb = wave * hpw; hb < H + G; hb += (kQkThreads / 64) * hpw) {
                const int h = hb + slot;
                const bool live = h < H + G;
                const bool is_q = h < H;
                T *src = row + static_cast<int64_t>(live ? h : 0) * d + el * 8;
                const float *bias = is_q ? q_b : k_b;
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = 0.f;
                if (live) {
                    const vec8_t<T> x = load8(src);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = to_f(x[j]);
                    if (bias) {     // (fp32 tensors start 16-byte aligned and h * d + 8 el is a multiple of 8)
                        const float *bp = bias + static_cast<int64_t>(is_q ? h : h - H) * d + el * 8;
                        const float4_t b0 = *reinterpret_cast<const float4_t *>(bp), b1 = *reinterpret_cast<const float4_t *>(bp + 4);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            v[j] += b0[j];
                            v[4 + j] += b1[j];
                        }
                    }
                }
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
                ss = lph == 4 ? group_allreduce_sum<4>(ss) : lph == 8 ? group_allreduce_sum<8>(ss) : group_allreduce_sum<16>(ss);
                const float r = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
                if (!live || (!is_q && !store)) continue;
                const float *wn = is_q ? q_w : k_w;
                vec8_t<T> o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = to_t<T>(wn ? v[j] * r * wn[el * 8 + j] : v[j] * r);
                if (is_q) store8(src, o);
                else store8(k_cache + blk * block_stride + (static_cast<int64_t>(h - H) * kQkBlock + off) * d + el * 8, o);
            }
        }
    }
    for (int h = wave; h < H + G && !wide; h += kQkThreads / 64) {
        const bool is_q = h < H;
        if (!is_q && !store) continue;
        T *src = row + static_cast<int64_t>(h) * d;         // k heads follow the q heads
        const float *bias = is_q ? (q_b ? q_b + static_cast<int64_t>(h) * d : nullptr)
                                 : (k_b ? k_b + static_cast<int64_t>(h - H) * d : nullptr);
        const float *wn = is_q ? q_w : k_w;
        float ss = 0.f;
        for (int e = lane; e < d; e += 64) {
            const float v = to_f(src[e]) + (bias ? bias[e] : 0.f);
            ss += v * v;
        }
        ss = wave_allreduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
        T *dst = is_q ? src : k_cache + blk * block_stride + (static_cast<int64_t>(h - H) * kQkBlock + off) * d;
        for (int e = lane; e < d; e += 64) {
            const float v = (to_f(src[e]) + (bias ? bias[e] : 0.f)) * r;
            dst[e] = to_t<T>(wn ? v * wn[e] : v);
        }
    }
    T *vsrc = row + static_cast<int64_t>(H + G) * d;
    const T *vo = v_other ? v_other + t * v_other_stride : nullptr;
    if constexpr (sizeof(T) == 2) {
        // value heads whose size is a multiple of 8, on 16-byte-aligned rows: 8 columns per lane (the same sums as below)
        const bool vwide = wide && (dv & 7) == 0 && ((static_cast<int64_t>(H + G) * d) & 7) == 0 &&
                           (!v_b || (reinterpret_cast<uintptr_t>(v_b) & 15) == 0) &&
                           (!vo || ((v_other_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(v_other) & 15) == 0));
        if (vwide) {
            for (int i = threadIdx.x * 8; i < G * dv; i += kQkThreads * 8) {
                const vec8_t<T> x = load8(vsrc + i);
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = to_f(x[j]);
                if (v_b) {
                    const float4_t b0 = *reinterpret_cast<const float4_t *>(v_b + i), b1 = *reinterpret_cast<const float4_t *>(v_b + i + 4);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        v[j] += b0[j];
                        v[4 + j] += b1[j];
                    }
                }
                if (vo) {
                    const vec8_t<T> y = load8(vo + i);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = (1.0f - mix) * v[j] + mix * to_f(y[j]);
                }
                vec8_t<T> o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = to_t<T>(v[j]);
                store8(vsrc + i, o);
                if (store) {
                    const int g = i / dv, c = i - g * dv;       // (8 consecutive columns of one head)
                    T *dst = v_cache + blk * block_stride + (static_cast<int64_t>(g) * dv + c) * kQkBlock + off;
#pragma unroll
                    for (int j = 0; j < 8; ++j) dst[j * kQkBlock] = o[j];       // transposed page
                }
            }
            return;
        }
    }
    for (int i = threadIdx.x; i < G * dv; i += kQkThreads) {
        float v = to_f(vsrc[i]) + (v_b ? v_b[i] : 0.f);
        if (vo) v = (1.0f - mix) * v + mix * to_f(vo[i]);
        const T vt = to_t<T>(v);
        vsrc[i] = vt;
        if (store) {
            const int g = i / dv, c = i - g * dv;
            v_cache[blk * block_stride + (static_cast<int64_t>(g) * dv + c) * kQkBlock + off] = vt;     // transposed page
        }
    }
}

} // namespace swl

extern "C" int swl_qknorm_store_kv(void *qkv, const float *q_w, const float *k_w, void *k_cache, void *v_cache,
                                   const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                                   int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim,
                                   int32_t vdim, int64_t tok_stride, int32_t max_blocks_per_seq, int64_t block_stride,
                                   float eps, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || dim <= 0 || vdim <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!qkv || !q_w || !k_w || !tok_pos) return SWL_ERR_BAD_ARG;
    const int store = k_cache != nullptr;
    if (store && (!v_cache || !block_table || !tok_seq)) return SWL_ERR_BAD_ARG;
    if (tok_stride < static_cast<int64_t>(num_q_heads + num_kv_heads) * dim + static_cast<int64_t>(num_kv_heads) * vdim)
        return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::qknorm_store_kv_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kQkThreads), 0, static_cast<hipStream_t>(stream), static_cast<T *>(qkv), q_w, k_w,
                           static_cast<T *>(k_cache), static_cast<T *>(v_cache), block_table, tok_seq, tok_pos,
                           num_q_heads, num_kv_heads, dim, vdim, tok_stride, max_blocks_per_seq, block_stride, eps, store);
    });
    return swl::check_launch();
}

extern "C" int swl_qknorm_full_store_kv(void *qkv, const float *q_w, const float *k_w, void *k_cache, void *v_cache,
                                        const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                                        int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim,
                                        int32_t vdim, int64_t tok_stride, int32_t max_blocks_per_seq,
                                        int64_t block_stride, float eps, float temp_coef, int32_t temp_every,
                                        int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || dim <= 0 || vdim <= 0 || temp_every < 1)
        return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!qkv || !q_w || !tok_pos) return SWL_ERR_BAD_ARG;
    const int store = k_cache != nullptr;
    if (store && (!k_w || !v_cache || !block_table || !tok_seq)) return SWL_ERR_BAD_ARG;
    const int64_t need = static_cast<int64_t>(num_q_heads) * dim +
                         (store ? static_cast<int64_t>(num_kv_heads) * (dim + vdim) : 0);
    if (tok_stride < need) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::qknorm_full_store_kv_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kQkThreads), 0, static_cast<hipStream_t>(stream), static_cast<T *>(qkv), q_w, k_w,
                           static_cast<T *>(k_cache), static_cast<T *>(v_cache), block_table, tok_seq, tok_pos,
                           num_q_heads, num_kv_heads, dim, vdim, tok_stride, max_blocks_per_seq, block_stride, eps,
                           temp_coef, temp_every, store);
    });
    return swl::check_launch();
}

extern "C" int swl_qkv_bias_norm_store(void *qkv, const float *q_b, const float *k_b, const float *v_b, const float *q_w,
                                       const float *k_w, const void *v_other, int64_t v_other_stride, float mix,
                                       void *k_cache, void *v_cache, const int32_t *block_table, const int32_t *tok_seq,
                                       const int32_t *tok_pos, int64_t num_tokens, int32_t num_q_heads,
                                       int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t tok_stride,
                                       int32_t max_blocks_per_seq, int64_t block_stride, float eps, int32_t dtype,
                                       swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || dim <= 0 || vdim <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!qkv || !tok_pos) return SWL_ERR_BAD_ARG;
    const int store = k_cache != nullptr;
    if (store && (!v_cache || !block_table || !tok_seq)) return SWL_ERR_BAD_ARG;
    if (tok_stride < static_cast<int64_t>(num_q_heads + num_kv_heads) * dim + static_cast<int64_t>(num_kv_heads) * vdim)
        return SWL_ERR_BAD_ARG;
    if (v_other && v_other_stride < static_cast<int64_t>(num_kv_heads) * vdim) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::qkv_bias_norm_store_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kQkThreads), 0, static_cast<hipStream_t>(stream), static_cast<T *>(qkv), q_b, k_b, v_b,
                           q_w, k_w, static_cast<const T *>(v_other), v_other_stride, mix, static_cast<T *>(k_cache),
                           static_cast<T *>(v_cache), block_table, tok_seq, tok_pos, num_q_heads, num_kv_heads, dim, vdim,
                           tok_stride, max_blocks_per_seq, block_stride, eps, store);
    });
    return swl::check_launch();
}
