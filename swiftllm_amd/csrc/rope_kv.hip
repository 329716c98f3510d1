// rope_kv.hip — rotary positions on interleaved pairs fused with the paged KV store, and what attention heads need after the
// softmax when they are gated or combined.
//
// Rotation: inside a head, dimension 2i is paired with dimension 2i + 1 for i < rot_dims / 2; the pair (u, v) of a token at
// position p becomes (u cos a - v sin a, v cos a + u sin a), a = p * freq[i]. The frequencies come from the host as a
// float64 table (base^(-2i / rot_dims), evaluated once per model); the angle and its sine and cosine are evaluated in
// float64 per (token, i) into LDS and used in fp32 by every head of the token — exact to fp32 rounding at any position.
// Dimensions from rot_dims on pass unchanged.
//
//   swl_rope_store_kv         rows [q: nq heads of d | k: nk heads of d | v: nv heads of dv]: q rotated in place, k rotated
//                             into the K pool, v copied into the V pool.
//   swl_latent_rope_store_kv  latent attention. Rows hold H query heads [d unrotated | dr rotated] and (optionally) the
//                             compressed key/value row [r latent | dr shared rotated key part]. The rotated query parts go
//                             to qa[t][h][r : r + dr] (the caller fills qa[t][h][0 : r] with the queries folded through
//                             the key up-projection); the latent is RMS-normed (fp32 statistics, weight) and stored
//                             together with the rotated key part as ONE key head of r + dr, and once more, transposed, as
//                             the value head of r: attention over the pool then IS the latent attention with the
//                             up-projections applied outside (queries before, outputs after).
//   swl_diff_head_combine     out = unit_rms(a1 - lambda a2) * mult * sigmoid(gate) per head, a1 / a2 the fp32 results of two
//                             score maps over the same values.
//   swl_head_gate             y[t][h][:] *= sigmoid(gate[t][h]).
//
// Pool layout as in qknorm_kv.hip: keys of a page [heads, 16, d], values transposed [heads, dv, 16].
#include "swl_common.h"

namespace swl {

constexpr int kRkThreads = 256;
constexpr int kRkBlock = 16;        // tokens per KV block
constexpr int kRkMaxPairs = 256;    // rot_dims <= 512

__device__ __forceinline__ void rk_angles(float *cs, float *sn, const double *freq, int pos, int pairs) {
    for (int i = threadIdx.x; i < pairs; i += kRkThreads) {
        const double a = static_cast<double>(pos) * freq[i];
        cs[i] = static_cast<float>(cos(a));
        sn[i] = static_cast<float>(sin(a));
    }
}

__device__ __forceinline__ float rk_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(kRkThreads) void rope_store_kv_kernel(
    T *qkv, const double *freq, T *k_cache, T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, int nq, int nk, int nv, int d, int dv, int rot_dims, int64_t tok_stride, int max_blocks_per_seq,
    int64_t block_stride) {
    __shared__ float cs[kRkMaxPairs], sn[kRkMaxPairs];
    const int64_t t = blockIdx.x;
    const int pos = tok_pos[t];
    const int pairs = rot_dims >> 1;
    rk_angles(cs, sn, freq, pos, pairs);
    __syncthreads();
    T *row = qkv + t * tok_stride;
    const bool store = k_cache != nullptr;
    int64_t blk = 0;
    if (store) blk = block_table[static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq + pos / kRkBlock];
    const int off = pos % kRkBlock;
    // queries: only the rotated pairs change
    for (int i = threadIdx.x; i < nq * pairs; i += kRkThreads) {
        const int h = i / pairs, j = i - h * pairs;
        T *p = row + static_cast<int64_t>(h) * d + 2 * j;
        const float u = to_f(p[0]), v = to_f(p[1]);
        p[0] = to_t<T>(u * cs[j] - v * sn[j]);
        p[1] = to_t<T>(v * cs[j] + u * sn[j]);
    }
    if (!store) return;
    // keys: every element goes to the pool, the first rot_dims of each head rotated
    const T *krow = row + static_cast<int64_t>(nq) * d;
    for (int i = threadIdx.x; i < nk * d; i += kRkThreads) {
        const int g = i / d, e = i - g * d;
        float x = to_f(krow[i]);
        if (e < rot_dims) {
            const int j = e >> 1;
            const float other = to_f(krow[i ^ 1]);      // (d is even: the partner is inside the head)
            x = (e & 1) ? x * cs[j] + other * sn[j] : x * cs[j] - other * sn[j];
        }
        k_cache[blk * block_stride + (static_cast<int64_t>(g) * kRkBlock + off) * d + e] = to_t<T>(x);
    }
    const T *vrow = krow + static_cast<int64_t>(nk) * d;
    for (int i = threadIdx.x; i < nv * dv; i += kRkThreads)
        v_cache[blk * block_stride + static_cast<int64_t>(i) * kRkBlock + off] = vrow[i];       // transposed page
}

template <typename T>
__global__ __launch_bounds__(kRkThreads) void latent_rope_store_kv_kernel(
    const T *proj, T *qa, const double *freq, const float *c_w, T *k_cache, T *v_cache, const int32_t *block_table,
    const int32_t *tok_seq, const int32_t *tok_pos, int H, int d, int dr, int r, int64_t proj_stride, int64_t dkv_col,
    int64_t qa_stride, int max_blocks_per_seq, int64_t block_stride, float eps) {
    __shared__ float cs[kRkMaxPairs], sn[kRkMaxPairs];
    __shared__ float red[kRkThreads / 64];
    const int64_t t = blockIdx.x;
    const int pos = tok_pos[t];
    const int pairs = dr >> 1;
    rk_angles(cs, sn, freq, pos, pairs);
    __syncthreads();
    const T *row = proj + t * proj_stride;
    T *qrow = qa + t * qa_stride;
    for (int i = threadIdx.x; i < H * pairs; i += kRkThreads) {
        const int h = i / pairs, j = i - h * pairs;
        const T *p = row + static_cast<int64_t>(h) * (d + dr) + d + 2 * j;
        T *o = qrow + static_cast<int64_t>(h) * (r + dr) + r + 2 * j;
        const float u = to_f(p[0]), v = to_f(p[1]);
        o[0] = to_t<T>(u * cs[j] - v * sn[j]);
        o[1] = to_t<T>(v * cs[j] + u * sn[j]);
    }
    if (dkv_col < 0 || k_cache == nullptr) return;
    const T *z = row + dkv_col;
    float ss = 0.f;
    for (int i = threadIdx.x; i < r; i += kRkThreads) {
        const float x = to_f(z[i]);
        ss += x * x;
    }
    ss = wave_allreduce_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int w = 0; w < kRkThreads / 64; ++w) ss += red[w];
    const float rinv = 1.0f / sqrtf(ss / static_cast<float>(r) + eps);
    const int64_t blk = block_table[static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq + pos / kRkBlock];
    const int off = pos % kRkBlock;
    T *kdst = k_cache + blk * block_stride + static_cast<int64_t>(off) * (r + dr);
    T *vdst = v_cache + blk * block_stride + off;
    for (int i = threadIdx.x; i < r; i += kRkThreads) {
        const T c = to_t<T>(to_f(z[i]) * rinv * c_w[i]);
        kdst[i] = c;
        vdst[static_cast<int64_t>(i) * kRkBlock] = c;
    }
    for (int j = threadIdx.x; j < pairs; j += kRkThreads) {
        const float u = to_f(z[r + 2 * j]), v = to_f(z[r + 2 * j + 1]);
        kdst[r + 2 * j] = to_t<T>(u * cs[j] - v * sn[j]);
        kdst[r + 2 * j + 1] = to_t<T>(v * cs[j] + u * sn[j]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void diff_head_combine_kernel(T *out, const float *a, const T *gate, int64_t gate_stride,
                                                                float lambda, float mult, float eps, int H, int dv) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int h = wave; h < H; h += 4) {
        const float *a1 = a + ((t * 2) * H + h) * dv, *a2 = a + ((t * 2 + 1) * H + h) * dv;
        float ss = 0.f;
        for (int e = lane; e < dv; e += 64) {
            const float o = a1[e] - lambda * a2[e];
            ss += o * o;
        }
        ss = wave_allreduce_sum(ss);
        const float g = gate ? rk_sigmoid(to_f(gate[t * gate_stride + h])) : 1.0f;
        const float f = mult * g / sqrtf(ss / static_cast<float>(dv) + eps);
        for (int e = lane; e < dv; e += 64) out[(t * H + h) * dv + e] = to_t<T>((a1[e] - lambda * a2[e]) * f);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T *y, const T *gate, int64_t gate_stride, int H, int dv) {
    const int64_t t = blockIdx.x;
    for (int i = threadIdx.x; i < H * dv; i += 256) {
        const float g = rk_sigmoid(to_f(gate[t * gate_stride + i / dv]));
        y[t * H * dv + i] = to_t<T>(to_f(y[t * H * dv + i]) * g);
    }
}

} // namespace swl

extern "C" int swl_rope_store_kv(void *qkv, const double *freq, void *k_cache, void *v_cache, const int32_t *block_table,
                                 const int32_t *tok_seq, const int32_t *tok_pos, int64_t num_tokens, int32_t num_q_heads,
                                 int32_t num_k_heads, int32_t num_v_heads, int32_t dim, int32_t vdim, int32_t rot_dims,
                                 int64_t tok_stride, int32_t max_blocks_per_seq, int64_t block_stride, int32_t dtype,
                                 swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_k_heads < 0 || num_v_heads < 0 || dim <= 0 || vdim <= 0) return SWL_ERR_BAD_ARG;
    if (rot_dims < 0 || (rot_dims & 1) || rot_dims > dim || (dim & 1)) return SWL_ERR_BAD_ARG;
    if (tok_stride < static_cast<int64_t>(num_q_heads + num_k_heads) * dim + static_cast<int64_t>(num_v_heads) * vdim)
        return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!qkv || !tok_pos || (rot_dims > 0 && !freq)) return SWL_ERR_BAD_ARG;
    if (k_cache && (!v_cache || !block_table || !tok_seq || max_blocks_per_seq <= 0)) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL || rot_dims > 2 * swl::kRkMaxPairs) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::rope_store_kv_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kRkThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(qkv), freq, static_cast<T *>(k_cache),
                           static_cast<T *>(v_cache), block_table, tok_seq, tok_pos, num_q_heads, num_k_heads, num_v_heads,
                           dim, vdim, rot_dims, tok_stride, max_blocks_per_seq, block_stride);
    });
    return swl::check_launch();
}

extern "C" int swl_latent_rope_store_kv(const void *proj, void *qa, const double *freq, const float *c_norm, void *k_cache,
                                        void *v_cache, const int32_t *block_table, const int32_t *tok_seq,
                                        const int32_t *tok_pos, int64_t num_tokens, int32_t num_heads, int32_t dim,
                                        int32_t rot_dim, int32_t kv_rank, int64_t proj_stride, int64_t dkv_col,
                                        int64_t qa_stride, int32_t max_blocks_per_seq, int64_t block_stride, float eps,
                                        int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || dim <= 0 || rot_dim <= 0 || (rot_dim & 1) || kv_rank <= 0) return SWL_ERR_BAD_ARG;
    if (proj_stride < static_cast<int64_t>(num_heads) * (dim + rot_dim) ||
        qa_stride < static_cast<int64_t>(num_heads) * (kv_rank + rot_dim))
        return SWL_ERR_BAD_ARG;
    if (dkv_col >= 0 && dkv_col + kv_rank + rot_dim > proj_stride) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!proj || !qa || !freq || !tok_pos) return SWL_ERR_BAD_ARG;
    if (dkv_col >= 0 && k_cache && (!v_cache || !c_norm || !block_table || !tok_seq || max_blocks_per_seq <= 0))
        return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL || rot_dim > 2 * swl::kRkMaxPairs) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::latent_rope_store_kv_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kRkThreads), 0, static_cast<hipStream_t>(stream), static_cast<const T *>(proj),
                           static_cast<T *>(qa), freq, c_norm, static_cast<T *>(k_cache), static_cast<T *>(v_cache),
                           block_table, tok_seq, tok_pos, num_heads, dim, rot_dim, kv_rank, proj_stride, dkv_col, qa_stride,
                           max_blocks_per_seq, block_stride, eps);
    });
    return swl::check_launch();
}

extern "C" int swl_diff_head_combine(void *out, const float *maps, const void *gate, int64_t gate_stride, float lambda,
                                     float mult, float eps, int64_t num_tokens, int32_t num_heads, int32_t vdim,
                                     int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || vdim <= 0 || (gate && gate_stride < num_heads)) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !maps) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::diff_head_combine_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(out), maps, static_cast<const T *>(gate),
                           gate_stride, lambda, mult, eps, num_heads, vdim);
    });
    return swl::check_launch();
}

extern "C" int swl_head_gate(void *y, const void *gate, int64_t gate_stride, int64_t num_tokens, int32_t num_heads,
                             int32_t vdim, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || vdim <= 0 || gate_stride < num_heads) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!y || !gate) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::head_gate_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(gate), gate_stride,
                           num_heads, vdim);
    });
    return swl::check_launch();
}
