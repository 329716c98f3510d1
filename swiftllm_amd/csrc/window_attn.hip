// window_attn.hip — attention over the paged KV pool with a sliding window, tanh soft-capping and pre-softmax head
// mixing ("talking heads": the capped scores of all query heads at one (query, key) pair are mixed by an [H, H] matrix
// before the softmax; without a matrix every head keeps its own) and an optional learned bias per (distance, head) added to
// the mixed scores, for any mixture of prompt portions and single decoded tokens.
//
// Every query token carries its sequence row and position; its own key/value are already in the pool (qknorm_kv.hip ran
// first), so a prompt portion that continues a cached prefix, a whole prompt and a decoded token are the same case:
// keys [max(0, p - window + 1), p] of the token's sequence, read through the block table.
//
// Because the mix couples the heads, one workgroup owns ALL heads of its query token. Keys are taken in chunks of 64:
//   1. capped scores s[g][j] for every head g (fp32 dot products, fp32 tanh),
//   2. mixed scores  m[h][j] = sum_g talk[h][g] s[g][j], online softmax per mixed head h (fp32, full-precision exp),
//   3. acc[h][:] = acc[h][:] * alpha[h] + sum_j p[h][j] v[kv(h)][j][:]   (fp32 weights, fp32 accumulation).
// This is the reference-grade kernel: everything after the loads is fp32 whatever the storage dtype.
//
// The general entry point (swl_masked_attn) adds what other designs need of the same loop:
//   * mask_kind 1: chunked visibility — keys [floor(p / window) * window, p], chunks counted from position 0;
//   * sink[H]: a learned logit per head that joins the softmax denominator only (no key, no value, not scaled);
//   * num_v_heads < num_kv_heads: several key heads share one value head (value head = key head % num_v_heads) — two
//     score maps over the same values, laid out map-major, are 2 G key heads over G value heads;
//   * out_f32: the result leaves in fp32 (for a combination of maps that cancels);
//   * without a mixing matrix the heads are independent: more than 32 of them (or more than the accumulators and the LDS of
//     one workgroup hold) are shared out over blockIdx.y, every workgroup taking a group of consecutive heads.
#include "swl_common.h"

namespace swl {

constexpr int kWaThreads = 256;
constexpr int kWaChunk = 64;        // keys per chunk = one key per lane in the softmax phase
constexpr int kWaBlock = 16;        // tokens per KV block
constexpr int kWaMaxAcc = 32;       // (head, value column) accumulators per thread: H * vdim <= 8192

// fp32 words ahead of the 8-byte-aligned key tables
__host__ __device__ inline size_t wa_float_count(int H, int d) {
    size_t n = static_cast<size_t>(H) * d + static_cast<size_t>(H) * H + 2 * static_cast<size_t>(H) * kWaChunk +
               2 * static_cast<size_t>(H);
    return n + (n & 1);
}

template <typename T>
__global__ __launch_bounds__(kWaThreads) void window_attn_kernel(
    T *out, const T *q, const T *k_cache, const T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, const float *talk, const float *rel, int rel_len, int H, int G, int d, int dv,
    int64_t q_tok_stride, int window, float scale, float softcap, int max_blocks_per_seq, int64_t block_stride,
    int mask_kind, const float *sink, int GV, int out_f32, int Hall) {
    // H: heads of this workgroup, starting at head hb of the token's Hall heads (G: key heads per Hall query heads)
    extern __shared__ float lds[];
    float *qf = lds;                        // [H * d]
    float *tk = qf + H * d;                 // [H * H]
    float *s = tk + H * H;                  // [H][64] capped scores
    float *p = s + H * kWaChunk;            // [H][64] softmax numerators
    float *alpha = p + H * kWaChunk;        // [H]
    int64_t *kbase = reinterpret_cast<int64_t *>(lds + wa_float_count(H, d));   // [64] block id of each key (8-byte aligned)
    int *koff = reinterpret_cast<int *>(kbase + kWaChunk);                          // [64] slot inside the block

    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int pos = tok_pos[t];
    const int32_t *bt = block_table + static_cast<int64_t>(tok_seq[t]) * max_blocks_per_seq;
    const int lo = window <= 0 ? 0 : mask_kind == 1 ? (pos / window) * window : (pos - window + 1 > 0 ? pos - window + 1 : 0);
    const int nkeys = pos - lo + 1;
    const int rep = Hall / G;
    const int hb = static_cast<int>(blockIdx.y) * H;
    if (hb + H > Hall) H = Hall - hb;
    if (sink) sink += hb;
    if (rel) rel += static_cast<int64_t>(hb) * rel_len;

    const T *qrow = q + t * q_tok_stride + static_cast<int64_t>(hb) * d;
    for (int i = tid; i < H * d; i += kWaThreads) qf[i] = to_f(qrow[i]);
    // (no mixing matrix: every head keeps its own scores)
    for (int i = tid; i < H * H; i += kWaThreads) tk[i] = talk ? talk[i] : (i / H == i % H ? 1.f : 0.f);

    float acc[kWaMaxAcc];
#pragma unroll
    for (int i = 0; i < kWaMaxAcc; ++i) acc[i] = 0.f;
    // running maximum and sum of mixed head h live in the lanes of the wave that owns h (wave = h % 4): replicated
    float mrun[8], lrun[8];     // heads per wave <= 8 -> H <= 32 ... generalised below through LDS when H > 32
#pragma unroll
    for (int i = 0; i < 8; ++i) { mrun[i] = kNegBig; lrun[i] = 0.f; }
    const int hpw = (H + 3) / 4;     // heads per wave (host guarantees <= 8)
    const int nacc = (H * dv + kWaThreads - 1) / kWaThreads;

    for (int c0 = 0; c0 < nkeys; c0 += kWaChunk) {
        const int cn = min(kWaChunk, nkeys - c0);
        __syncthreads();    // previous chunk's p / alpha / kbase fully consumed (and qf / tk written, first time)
        if (tid < kWaChunk) {
            const int kp = lo + c0 + tid;
            if (tid < cn) {
                kbase[tid] = bt[kp / kWaBlock];
                koff[tid] = kp % kWaBlock;
            }
        }
        __syncthreads();
        // 1. capped scores
        for (int idx = tid; idx < H * kWaChunk; idx += kWaThreads) {
            const int g = idx / kWaChunk, j = idx - g * kWaChunk;
            float v = 0.f;
            if (j < cn) {
                const T *kr = k_cache + kbase[j] * block_stride + (static_cast<int64_t>((hb + g) / rep) * kWaBlock + koff[j]) * d;
                const float *qh = qf + g * d;
                float a = 0.f;
                for (int e = 0; e < d; ++e) a += qh[e] * to_f(kr[e]);
                a *= scale;
                v = softcap > 0.f ? softcap * tanhf(a / softcap) : a;
            }
            s[idx] = v;
        }
        __syncthreads();
        // 2. mix the heads, online softmax per mixed head (wave `wave` owns heads wave, wave + 4, ...)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int h = wave + 4 * i;
            if (i >= hpw || h >= H) break;
            float mixed = kNegBig;
            if (lane < cn) {
                float a = 0.f;
                if (talk) {
                    for (int g = 0; g < H; ++g) a += tk[h * H + g] * s[g * kWaChunk + lane];
                } else {
                    a = s[h * kWaChunk + lane];
                }
                // learned bias by distance (query position - key position), one row of the table per head
                if (rel) a += rel[static_cast<int64_t>(h) * rel_len + min(nkeys - 1 - (c0 + lane), rel_len - 1)];
                mixed = a;
            }
            const float cmax = wave_allreduce_max(mixed);
            const float mnew = fmaxf(mrun[i], cmax);
            const float pj = lane < cn ? expf(mixed - mnew) : 0.f;
            const float csum = wave_allreduce_sum(pj);
            const float al = expf(mrun[i] - mnew);      // first chunk: exp(-1e30 - m) = 0
            lrun[i] = lrun[i] * al + csum;
            mrun[i] = mnew;
            p[h * kWaChunk + lane] = pj;
            if (lane == 0) alpha[h] = al;
        }
        __syncthreads();
        // 3. weighted values
#pragma unroll
        for (int i = 0; i < kWaMaxAcc; ++i) {
            if (i >= nacc) break;
            const int idx = tid + i * kWaThreads;
            if (idx < H * dv) {
                const int h = idx / dv, col = idx - h * dv;
                const int g = ((hb + h) / rep) % GV;
                float a = acc[i] * alpha[h];
                const float *ph = p + h * kWaChunk;
                for (int j = 0; j < cn; ++j) {
                    // (a page keeps its values transposed: [kv head][column][16 tokens])
                    const T *vr = v_cache + kbase[j] * block_stride + (static_cast<int64_t>(g) * dv + col) * kWaBlock;
                    a += ph[j] * to_f(vr[koff[j]]);
                }
                acc[i] = a;
            }
        }
    }
    __syncthreads();
    // final scale of every head: 1 / sum, or with a sink e^(m - M) / (sum e^(m - M) + e^(sink - M)), M = max(m, sink)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int h = wave + 4 * i;
        if (i >= hpw || h >= H) break;
        float al = 1.f, l = lrun[i];
        if (sink) {
            const float sk = sink[h], big = fmaxf(mrun[i], sk);
            al = expf(mrun[i] - big);
            l = l * al + expf(sk - big);
        }
        if (lane == 0) alpha[h] = al / l;
    }
    __syncthreads();
    const int64_t obase = (t * static_cast<int64_t>(Hall) + hb) * dv;
#pragma unroll
    for (int i = 0; i < kWaMaxAcc; ++i) {
        if (i >= nacc) break;
        const int idx = tid + i * kWaThreads;
        if (idx < H * dv) {
            const float o = acc[i] * alpha[idx / dv];
            if (out_f32) reinterpret_cast<float *>(out)[obase + idx] = o;
            else out[obase + idx] = to_t<T>(o);
        }
    }
}

inline size_t wa_lds_bytes(int H, int d) {
    return wa_float_count(H, d) * 4 + kWaChunk * (8 + 4);
}

} // namespace swl

extern "C" int swl_masked_attn(void *out, const void *q, const void *k_cache, const void *v_cache,
                               const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                               const float *talk, const float *rel, int32_t rel_len, int64_t num_tokens,
                               int32_t num_q_heads, int32_t num_kv_heads,
                               int32_t dim, int32_t vdim, int64_t q_tok_stride, int32_t window, float scale,
                               float softcap, int32_t max_blocks_per_seq, int64_t block_stride, int32_t mask_kind,
                               const float *sink, int32_t num_v_heads, int32_t out_f32, int32_t dtype,
                               swl_stream_t stream) {
    if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || dim <= 0 || vdim <= 0 || window < 0)
        return SWL_ERR_BAD_ARG;
    if (num_q_heads % num_kv_heads) return SWL_ERR_BAD_ARG;
    if (mask_kind < 0 || mask_kind > 1 || num_v_heads <= 0 || num_kv_heads % num_v_heads) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !q || !k_cache || !v_cache || !block_table || !tok_seq || !tok_pos || (rel && rel_len <= 0))
        return SWL_ERR_BAD_ARG;
    // heads per workgroup: all of them when they are mixed, else as many as its accumulators and LDS hold
    int hpg = num_q_heads;
    if (!talk) {
        if (hpg > 32) hpg = 32;
        while (hpg > 1 && (static_cast<int64_t>(hpg) * vdim > swl::kWaMaxAcc * swl::kWaThreads ||
                           swl::wa_lds_bytes(hpg, dim) > 64 * 1024))
            --hpg;
    }
    const size_t lds = swl::wa_lds_bytes(hpg, dim);
    if (num_tokens > 0x7fffffffLL || hpg > 32 ||
        static_cast<int64_t>(hpg) * vdim > swl::kWaMaxAcc * swl::kWaThreads || lds > 64 * 1024)
        return SWL_ERR_UNSUPPORTED;
    const unsigned groups = static_cast<unsigned>((num_q_heads + hpg - 1) / hpg);
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::window_attn_kernel<T>), dim3(static_cast<unsigned>(num_tokens), groups),
                           dim3(swl::kWaThreads),
                           lds, static_cast<hipStream_t>(stream), static_cast<T *>(out), static_cast<const T *>(q),
                           static_cast<const T *>(k_cache), static_cast<const T *>(v_cache), block_table, tok_seq,
                           tok_pos, talk, rel, rel_len, hpg, num_kv_heads, dim, vdim, q_tok_stride, window, scale,
                           softcap,
                           max_blocks_per_seq, block_stride, mask_kind, sink, num_v_heads, out_f32, num_q_heads);
    });
    return swl::check_launch();
}

extern "C" int swl_window_attn(void *out, const void *q, const void *k_cache, const void *v_cache,
                               const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                               const float *talk, const float *rel, int32_t rel_len, int64_t num_tokens,
                               int32_t num_q_heads, int32_t num_kv_heads,
                               int32_t dim, int32_t vdim, int64_t q_tok_stride, int32_t window, float scale,
                               float softcap, int32_t max_blocks_per_seq, int64_t block_stride, int32_t dtype,
                               swl_stream_t stream) {
    return swl_masked_attn(out, q, k_cache, v_cache, block_table, tok_seq, tok_pos, talk, rel, rel_len, num_tokens,
                           num_q_heads, num_kv_heads, dim, vdim, q_tok_stride, window, scale, softcap, max_blocks_per_seq,
                           block_stride, 0, nullptr, num_kv_heads > 0 ? num_kv_heads : 1, 0, dtype, stream);
}
