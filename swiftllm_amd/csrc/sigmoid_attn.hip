// sigmoid_attn.hip — attention over the paged KV pool whose weights are sigmoids instead of a softmax: every visible key gets
//     a[g] = sigmoid(scale q_g . k - r1[g] ln(1 + r2[g] (i - j)) + pb[g])        (query position i, key position j <= i)
// on its own, nothing is normalised over the keys, and the heads' weights are then mixed by an [H, H] matrix AFTER the
// sigmoid: a'[h] = sum_g talk[h][g] a[g]; head h applies a'[h] to the values of its own key/value head. The distance term
// (r1, r2: a logarithmic penalty per head), the per-head offset pb and the mixing matrix are each optional (NULL).
//
// Every query token carries its sequence row and position and its own key/value are already in the pool, so a prompt
// portion that continues a cached prefix, a whole prompt and a decoded token are the same case. Pool layout as in
// qknorm_kv.hip: keys [kv_heads, 16, dim], values transposed [kv_heads, vdim, 16] per 16-token block.
//
//   swl_sigmoid_attn:        one workgroup per query token, keys in chunks of 64, everything after the loads in fp32 and
//                            any storage dtype (fp32 included): the reference-grade kernel.
//   swl_sigmoid_attn_tiles:  the matrix-core form for 16-bit storage: tiles of up to 16 consecutive queries of one sequence
//                            against 16-key pages (see below).
// Without a running maximum or denominator the sum over keys is a plain sum: key shares of one query (a split over
// workgroups) are added up, no rescaling.
#include "swl_common.h"

namespace swl {

constexpr int kSgThreads = 256;
constexpr int kSgChunk = 64;        // keys per chunk
constexpr int kSgBlock = 16;        // tokens per KV block
constexpr int kSgMaxAcc = 32;       // (head, value column) accumulators per thread: H * vdim <= 8192

__host__ __device__ inline size_t sg_float_count(int H, int d, int mixed) {
    size_t n = static_cast<size_t>(H) * d + (mixed ? static_cast<size_t>(H) * H : 0) +
               (mixed ? 2 : 1) * static_cast<size_t>(H) * kSgChunk;
    return n + (n & 1);
}

__device__ __forceinline__ float sg_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(kSgThreads) void sigmoid_attn_kernel(
    T *out, const T *q, const T *k_cache, const T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, const float *talk, const float *r1, const float *r2, const float *pb, int H, int G, int d, int dv,
    int64_t q_tok_stride, int window, float scale, int max_blocks_per_seq, int64_t block_stride, int Hall) {
    // H: heads of this workgroup, starting at head hb of the token's Hall heads (all of them when the heads are mixed)
    extern __shared__ float lds[];
    float *qf = lds;                                    // [H * d]
    float *tk = qf + H * d;                             // [H * H] (mixed only)
    float *a = tk + (talk ? H * H : 0);                 // [H][64] weights
    float *p = talk ? a + H * kSgChunk : a;             // [H][64] mixed weights (the weights themselves without a matrix)
    int64_t *kbase = reinterpret_cast<int64_t *>(lds + sg_float_count(H, d, talk != nullptr));   // [64] block of each key
    int *koff = reinterpret_cast<int *>(kbase + kSgChunk);                                        // [64] slot in its block

    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    const int pos = tok_pos[t];
    const int32_t *bt = block_table + static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq;
    const int lo = window <= 0 ? 0 : (pos - window + 1 > 0 ? pos - window + 1 : 0);
    const int nkeys = pos - lo + 1;
    const int rep = Hall / G;
    const int hb = static_cast<int>(blockIdx.y) * H;
    if (hb + H > Hall) H = Hall - hb;

    const T *qrow = q + t * q_tok_stride + static_cast<int64_t>(hb) * d;
    for (int i = tid; i < H * d; i += kSgThreads) qf[i] = to_f(qrow[i]);
    if (talk)
        for (int i = tid; i < H * H; i += kSgThreads) tk[i] = talk[i];

    float acc[kSgMaxAcc];
#pragma unroll
    for (int i = 0; i < kSgMaxAcc; ++i) acc[i] = 0.f;
    const int nacc = (H * dv + kSgThreads - 1) / kSgThreads;

    for (int c0 = 0; c0 < nkeys; c0 += kSgChunk) {
        const int cn = min(kSgChunk, nkeys - c0);
        __syncthreads();    // the previous chunk's weights are consumed (and qf / tk written, the first time)
        if (tid < cn) {
            const int kp = lo + c0 + tid;
            kbase[tid] = bt[kp / kSgBlock];
            koff[tid] = kp % kSgBlock;
        }
        __syncthreads();
        // 1. weights of every head of this workgroup
        for (int idx = tid; idx < H * kSgChunk; idx += kSgThreads) {
            const int g = idx / kSgChunk, j = idx - g * kSgChunk;
            float w = 0.f;
            if (j < cn) {
                const T *kr = k_cache + kbase[j] * block_stride + (static_cast<int64_t>((hb + g) / rep) * kSgBlock + koff[j]) * d;
                const float *qh = qf + g * d;
                float s = 0.f;
                for (int e = 0; e < d; ++e) s += qh[e] * to_f(kr[e]);
                s *= scale;
                if (r1) s -= r1[hb + g] * logf(1.0f + r2[hb + g] * static_cast<float>(pos - (lo + c0 + j)));
                if (pb) s += pb[hb + g];
                w = sg_sigmoid(s);
            }
            a[idx] = w;
        }
        __syncthreads();
        // 2. mix the heads
        if (talk) {
            for (int idx = tid; idx < H * kSgChunk; idx += kSgThreads) {
                const int h = idx / kSgChunk, j = idx - h * kSgChunk;
                float m = 0.f;
                for (int g = 0; g < H; ++g) m += tk[h * H + g] * a[g * kSgChunk + j];
                p[idx] = m;
            }
            __syncthreads();
        }
        // 3. weighted values
#pragma unroll
        for (int i = 0; i < kSgMaxAcc; ++i) {
            if (i >= nacc) break;
            const int idx = tid + i * kSgThreads;
            if (idx < H * dv) {
                const int h = idx / dv, col = idx - h * dv;
                const int g = (hb + h) / rep;
                float s = acc[i];
                const float *ph = p + h * kSgChunk;
                for (int j = 0; j < cn; ++j) {
                    const T *vr = v_cache + kbase[j] * block_stride + (static_cast<int64_t>(g) * dv + col) * kSgBlock;
                    s += ph[j] * to_f(vr[koff[j]]);
                }
                acc[i] = s;
            }
        }
    }
    const int64_t obase = (t * static_cast<int64_t>(Hall) + hb) * dv;
#pragma unroll
    for (int i = 0; i < kSgMaxAcc; ++i) {
        if (i >= nacc) break;
        const int idx = tid + i * kSgThreads;
        if (idx < H * dv) out[obase + idx] = to_t<T>(acc[i]);
    }
}

inline size_t sg_lds_bytes(int H, int d, int mixed) { return sg_float_count(H, d, mixed) * 4 + kSgChunk * (8 + 4); }

} // namespace swl

extern "C" int swl_sigmoid_attn(void *out, const void *q, const void *k_cache, const void *v_cache,
                                const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos, const float *talk,
                                const float *r1, const float *r2, const float *pb, int64_t num_tokens, int32_t num_q_heads,
                                int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride, int32_t window,
                                float scale, int32_t max_blocks_per_seq, int64_t block_stride, int32_t dtype,
                                swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || dim <= 0 || vdim <= 0 || window < 0) return SWL_ERR_BAD_ARG;
    if (num_q_heads % num_kv_heads || (r1 == nullptr) != (r2 == nullptr)) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !q || !k_cache || !v_cache || !block_table || !tok_seq || !tok_pos) return SWL_ERR_BAD_ARG;
    // heads per workgroup: all of them when they are mixed, else as many as its accumulators and LDS hold
    int hpg = num_q_heads;
    if (!talk)
        while (hpg > 1 && (static_cast<int64_t>(hpg) * vdim > swl::kSgMaxAcc * swl::kSgThreads ||
                           swl::sg_lds_bytes(hpg, dim, 0) > 64 * 1024))
            --hpg;
    const size_t lds = swl::sg_lds_bytes(hpg, dim, talk != nullptr);
    if (num_tokens > 0x7fffffffLL || static_cast<int64_t>(hpg) * vdim > swl::kSgMaxAcc * swl::kSgThreads || lds > 64 * 1024)
        return SWL_ERR_UNSUPPORTED;
    const unsigned groups = static_cast<unsigned>((num_q_heads + hpg - 1) / hpg);
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::sigmoid_attn_kernel<T>), dim3(static_cast<unsigned>(num_tokens), groups),
                           dim3(swl::kSgThreads), lds, static_cast<hipStream_t>(stream), static_cast<T *>(out),
                           static_cast<const T *>(q), static_cast<const T *>(k_cache), static_cast<const T *>(v_cache),
                           block_table, tok_seq, tok_pos, talk, r1, r2, pb, hpg, num_kv_heads, dim, vdim, q_tok_stride, window,
                           scale, max_blocks_per_seq, block_stride, num_q_heads);
    });
    return swl::check_launch();
}
