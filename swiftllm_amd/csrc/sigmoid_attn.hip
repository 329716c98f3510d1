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

// ---- the matrix-core form ----------------------------------------------------------------------------------------------------
// One workgroup (4 waves; 8 for more than 16 heads) per tile of up to 16 consecutive queries of one sequence and per share of
// the tile's pages. The head mix couples all heads of a (query, key) pair, so the heads are split over the waves: wave w owns
// heads [w * HPW, (w + 1) * HPW) for the score products AND for the outputs, and the weights of all heads meet in LDS in
// between. Per 16-key page:
//   1. S^T_g = K_kv(g) Q_g^T  (16 keys x 16 queries, MFMA 16x16x16, fp32 accumulate); a_g = sigmoid(scale S - r1_g ln(1 + r2_g
//      dist) + pb_g) with the logarithm and the exponential on the transcendental unit, zero outside the mask -> LDS [H][256]
//   2. a'_h = sum_g talk[h][g] a_g  (fp32 VALU, talk as LDS broadcasts)
//   3. O^T_h += V^T_kv(h) a'^T_h   with the fp32 weights split into two 16-bit terms (hi + lo): the product keeps ~16 bits of
//      every weight although the matrix core takes 16-bit operands.
// The query fragments stay in registers for the whole walk; a page's value fragments are requested before its score
// products. Key shares write fp32 partial sums that a second launch adds up (plain sums: nothing to rescale).
constexpr int kSmTile = 16;

template <typename T, int D, int DV, int HPW, int NW, bool MIX>
__global__ __launch_bounds__(NW * 64) void sigmoid_attn_mfma_kernel(
    T *out, const T *q, const T *k_cache, const T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, const int32_t *tile_row0, const int32_t *tile_cnt, const float *__restrict__ talk,
    const float *__restrict__ r1, const float *__restrict__ r2, const float *__restrict__ pb, int H, int G,
    int64_t q_tok_stride, int window, float scale, int max_blocks_per_seq, int64_t block_stride, float *part_o,
    int64_t num_tokens, int nbuf) {
    extern __shared__ float s_all[];        // [nbuf][H][64 lanes][4] weights of a page, then [H][H] the mixing matrix
    float *tk = s_all + nbuf * H * 256;
    constexpr int CT = DV / 16, KS = D / 16;
    constexpr float kLog2e = 1.4426950408889634f;
    const int tile = blockIdx.x;
    const int row0 = __builtin_amdgcn_readfirstlane(tile_row0[tile]), cnt = __builtin_amdgcn_readfirstlane(tile_cnt[tile]);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;       // query (or operand row) index; quarter
    if constexpr (MIX) {
        for (int i = tid; i < H * H; i += NW * 64) tk[i] = talk[i];
        __syncthreads();
    }
    const int p0 = __builtin_amdgcn_readfirstlane(tok_pos[row0]);
    const int32_t *bt = block_table + static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tok_seq[row0])) * max_blocks_per_seq;
    const int rep = H / G;
    const int h0 = wave * HPW;
    const int qpos = p0 + li;
    const bool qok = li < cnt;
    const int qlo = window <= 0 ? 0 : qpos - window + 1;
    const int lo_first = window <= 0 ? 0 : (p0 - window + 1 > 0 ? p0 - window + 1 : 0);
    int kb0 = lo_first / kSmTile, kb1 = (p0 + cnt - 1) / kSmTile;
    if (gridDim.y > 1) {    // key split: this workgroup takes a contiguous share of the tile's pages (possibly none)
        const int per = (kb1 - kb0 + static_cast<int>(gridDim.y)) / static_cast<int>(gridDim.y);
        kb0 += per * static_cast<int>(blockIdx.y);
        kb1 = min(kb1, kb0 + per - 1);
    }
    float4_t acc[HPW][CT];
    float hr1[HPW], hr2[HPW], hpb[HPW];
    int koff[HPW], voff[HPW];
    vec4_t<T> qf[HPW][KS];
    const T *qrow = q + static_cast<int64_t>(row0 + (qok ? li : cnt - 1)) * q_tok_stride;     // rows past cnt: the last row
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int g = __builtin_amdgcn_readfirstlane(min(h0 + hh, H - 1));
        hr1[hh] = r1 ? r1[g] : 0.f;
        hr2[hh] = r2 ? r2[g] : 0.f;
        hpb[hh] = (pb ? pb[g] : 0.f) * kLog2e;
        koff[hh] = (g / rep) * kSmTile * D;
        voff[hh] = (g / rep) * DV * kSmTile;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[hh][ct] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < KS; ++e) load4(qf[hh][e], qrow + g * D + 4 * lq + e * 16);     // B operand: query li
    }
    const int lane_k = li * D + 4 * lq;             // A operand of S^T: key li, dims 4 lq ..
    const int lane_v = li * kSmTile + 4 * lq;       // A operand of O^T: column li of a 16-column tile, keys 4 lq ..
    const float c_scale = scale * kLog2e;
    int blk_next = kb0 <= kb1 ? __builtin_amdgcn_readfirstlane(bt[kb0]) : 0;

    for (int kb = kb0; kb <= kb1; ++kb) {
        float *s_lds = s_all + (nbuf == 2 && ((kb - kb0) & 1) ? H * 256 : 0);
        const int64_t blk = blk_next;
        const int nxt = kb < kb1 ? bt[kb + 1] : 0;
        const T *kblk = k_cache + blk * block_stride;
        const T *vblk = v_cache + blk * block_stride;
        vec4_t<T> vfrag[HPW][CT];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) load4(vfrag[hh][ct], vblk + voff[hh] + ct * 16 * kSmTile + lane_v);
        const int kpos0 = kb * kSmTile + 4 * lq;     // position of this lane's key r = 0
        float dist[4];
        bool ok[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int kp = kpos0 + r;
            ok[r] = qok && kp <= qpos && kp >= qlo;
            dist[r] = static_cast<float>(max(qpos - kp, 0));
        }
        float mixed[HPW][4];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            const int g = h0 + hh;
#pragma unroll
            for (int r = 0; r < 4; ++r) mixed[hh][r] = 0.f;
            if (g < H) {
                float4_t st = {0.f, 0.f, 0.f, 0.f};
                const T *kr = kblk + koff[hh] + lane_k;
#pragma unroll
                for (int e = 0; e < KS; ++e) {
                    vec4_t<T> a;
                    load4(a, kr + e * 16);
                    st = mfma16(a, qf[hh][e], st);
                }
                mfma_results_ready<4>(st);
                // st[r] = S^T[key 4 lq + r][query li]; the weight in base-2 exponent units: 1 / (1 + 2^-z)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float z = fmaf(st[r], c_scale, hpb[hh]);
                    if (r1) z -= hr1[hh] * fast_log2(fmaf(hr2[hh], dist[r], 1.0f));      // r1 ln(..) log2(e) = r1 log2(..)
                    st[r] = ok[r] ? __builtin_amdgcn_rcpf(1.0f + fast_exp2(-z)) : 0.f;
                }
                if constexpr (MIX) {
                    *reinterpret_cast<float4_t *>(&s_lds[(g * 64 + lane) * 4]) = st;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) mixed[hh][r] = st[r];
                }
            }
        }
        if constexpr (MIX) __syncthreads();
        blk_next = __builtin_amdgcn_readfirstlane(nxt);
        for (int g = 0; MIX && g < H; ++g) {
            const float4_t sv = *reinterpret_cast<const float4_t *>(&s_lds[(g * 64 + lane) * 4]);
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const float tw = tk[min(h0 + hh, H - 1) * H + g];       // wave-uniform address: an LDS broadcast
#pragma unroll
                for (int r = 0; r < 4; ++r) mixed[hh][r] = fmaf(tw, sv[r], mixed[hh][r]);
            }
        }
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            if (h0 + hh < H) {
                vec4_t<T> phi, plo;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    phi[r] = to_t<T>(mixed[hh][r]);
                    plo[r] = to_t<T>(mixed[hh][r] - to_f(phi[r]));
                }
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    float4_t o = acc[hh][ct];
                    o = mfma16(vfrag[hh][ct], phi, o);
                    o = mfma16(vfrag[hh][ct], plo, o);
                    acc[hh][ct] = o;
                }
            }
        }
        if constexpr (MIX) {
            if (nbuf == 1) __syncthreads();     // every wave is done with this page's weights before the next page's overwrite them
        }
    }
    // ---- epilogue: O[query li][h][ct * 16 + 4 lq + r] ----------------------------------------------------------------------------
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = h0 + hh;
        if (h < H) {
            const int orow = row0 + li;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                float4_t o = acc[hh][ct];
                mfma_results_ready<4>(o);
                if (!qok) continue;
                if (gridDim.y > 1) {
                    const int64_t slot = (static_cast<int64_t>(blockIdx.y) * num_tokens + orow) * H + h;
                    *reinterpret_cast<float4_t *>(part_o + slot * DV + ct * 16 + 4 * lq) = o;
                } else {
                    typedef T vec4 __attribute__((ext_vector_type(4)));
                    vec4 w;
#pragma unroll
                    for (int r = 0; r < 4; ++r) w[r] = to_t<T>(o[r]);
                    *reinterpret_cast<vec4 *>(out + (static_cast<int64_t>(orow) * H + h) * DV + ct * 16 + 4 * lq) = w;
                }
            }
        }
    }
}

// out[i] = sum over the key shares s of part[s][i]
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attn_sum_kernel(T *out, const float *part, int64_t total, int nsplit) {
    const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    float4_t a = *reinterpret_cast<const float4_t *>(part + i);
    for (int s = 1; s < nsplit; ++s) a += *reinterpret_cast<const float4_t *>(part + s * total + i);
    typedef T vec4 __attribute__((ext_vector_type(4)));
    vec4 w;
#pragma unroll
    for (int r = 0; r < 4; ++r) w[r] = to_t<T>(a[r]);
    *reinterpret_cast<vec4 *>(out + i) = w;
}

template <typename T, int D, int DV>
int launch_sm(int hpw, dim3 grid, size_t lds, hipStream_t s, T *out, const T *q, const T *kc, const T *vc, const int32_t *bt,
              const int32_t *ts, const int32_t *tp, const int32_t *r0, const int32_t *cn, const float *talk, const float *r1,
              const float *r2, const float *pb, int H, int G, int64_t qs, int window, float scale, int mb, int64_t bs, float *po,
              int64_t nt, int nbuf) {
#define SWL_SM_LAUNCH1(HPW, NW, MIX)                                                                                          \
    hipLaunchKernelGGL((sigmoid_attn_mfma_kernel<T, D, DV, HPW, NW, MIX>), grid, dim3(NW * 64), MIX ? lds : 0, s, out, q, kc, \
                       vc, bt, ts, tp, r0, cn, talk, r1, r2, pb, H, G, qs, window, scale, mb, bs, po, nt, nbuf)
#define SWL_SM_LAUNCH(HPW, NW)                   \
    if (talk) SWL_SM_LAUNCH1(HPW, NW, true);     \
    else SWL_SM_LAUNCH1(HPW, NW, false)
    switch (hpw) {
    case 1: SWL_SM_LAUNCH(1, 4); break;
    case 2: SWL_SM_LAUNCH(2, 4); break;
    case 4:
        if constexpr (DV <= 128) { SWL_SM_LAUNCH(4, 4); break; }
        else return SWL_ERR_UNSUPPORTED;
    case 8:
        if constexpr (DV <= 128) { SWL_SM_LAUNCH(4, 8); break; }
        else return SWL_ERR_UNSUPPORTED;
    default: return SWL_ERR_UNSUPPORTED;
    }
#undef SWL_SM_LAUNCH
#undef SWL_SM_LAUNCH1
    if (grid.y > 1) {
        const int64_t total = nt * H * DV;
        hipLaunchKernelGGL((sigmoid_attn_sum_kernel<T>), dim3(static_cast<unsigned>((total / 4 + 255) / 256)), dim3(256), 0, s,
                           out, po, total, static_cast<int>(grid.y));
    }
    return check_launch();
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

// (dim, vdim) pairs with a compiled matrix-core kernel
#define SWL_SM_SHAPES(X) \
    X(32, 32) X(32, 64) X(48, 48) X(64, 32) X(64, 64) X(64, 96) X(64, 128) X(96, 64) X(96, 96) X(128, 64) X(128, 128)

/* 1 when swl_sigmoid_attn_tiles serves this shape (else the caller uses swl_sigmoid_attn). */
extern "C" int swl_sigmoid_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim,
                                                int32_t dtype) {
    if (dtype != SWL_F16 && dtype != SWL_BF16) return 0;
    if (num_q_heads <= 0 || num_q_heads > 32 || num_kv_heads <= 0 || num_q_heads % num_kv_heads) return 0;
#define SWL_SM_IS(DD, DDV) if (dim == DD && vdim == DDV) return 1;
    SWL_SM_SHAPES(SWL_SM_IS)
#undef SWL_SM_IS
    return 0;
}

extern "C" int swl_sigmoid_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache,
                                      const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                                      const int32_t *tile_row0, const int32_t *tile_cnt, const float *talk, const float *r1,
                                      const float *r2, const float *pb, int32_t num_tiles, int32_t num_q_heads,
                                      int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride, int32_t window,
                                      float scale, int32_t max_blocks_per_seq, int64_t block_stride, int32_t key_splits,
                                      float *scratch, int64_t num_tokens, int32_t dtype, swl_stream_t stream) {
    if (num_tiles < 0 || window < 0 || key_splits < 1 || key_splits > 64 || (r1 == nullptr) != (r2 == nullptr))
        return SWL_ERR_BAD_ARG;
    if (key_splits > 1 && (!scratch || num_tokens <= 0 || (reinterpret_cast<uintptr_t>(scratch) & 15))) return SWL_ERR_BAD_ARG;
    if (!swl_sigmoid_attn_tiles_supported(num_q_heads, num_kv_heads, dim, vdim, dtype)) return SWL_ERR_UNSUPPORTED;
    if (num_tiles == 0) return SWL_OK;
    if (!out || !q || !k_cache || !v_cache || !block_table || !tok_seq || !tok_pos || !tile_row0 || !tile_cnt)
        return SWL_ERR_BAD_ARG;
    if ((q_tok_stride & 3) || (block_stride & 3) || (reinterpret_cast<uintptr_t>(q) & 7) ||
        (reinterpret_cast<uintptr_t>(k_cache) & 7) || (reinterpret_cast<uintptr_t>(v_cache) & 7) ||
        (reinterpret_cast<uintptr_t>(out) & 7))
        return SWL_ERR_BAD_ARG;     // 8-byte operand loads
    int hpw = (num_q_heads + 3) / 4;
    hpw = hpw <= 1 ? 1 : hpw <= 2 ? 2 : hpw <= 4 ? 4 : 8;
    const size_t one = static_cast<size_t>(num_q_heads) * 256, mixw = static_cast<size_t>(num_q_heads) * num_q_heads;
    const int nbuf = (2 * one + mixw) * sizeof(float) <= 64 * 1024 ? 2 : 1;
    const size_t lds = (nbuf * one + mixw) * sizeof(float);
    if (lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(num_tiles), static_cast<unsigned>(key_splits));
    hipStream_t s = static_cast<hipStream_t>(stream);
#define SWL_SM_SHAPE(DD, DDV)                                                                                                  \
    if (dim == DD && vdim == DDV)                                                                                              \
        return swl::launch_sm<T, DD, DDV>(hpw, grid, lds, s, static_cast<T *>(out), static_cast<const T *>(q),                \
                                          static_cast<const T *>(k_cache), static_cast<const T *>(v_cache), block_table,      \
                                          tok_seq, tok_pos, tile_row0, tile_cnt, talk, r1, r2, pb, num_q_heads, num_kv_heads, \
                                          q_tok_stride, window, scale, max_blocks_per_seq, block_stride, scratch, num_tokens, \
                                          nbuf);
    SWL_DISPATCH_DTYPE(dtype, T, { SWL_SM_SHAPES(SWL_SM_SHAPE) });
#undef SWL_SM_SHAPE
    return SWL_ERR_UNSUPPORTED;
}
