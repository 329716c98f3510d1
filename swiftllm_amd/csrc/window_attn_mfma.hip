// window_attn_mfma.hip — the matrix-core form of window_attn.hip for 16-bit storage: tiles of up to 16 consecutive query
// tokens of one sequence against 16-key pages of the pool.
//
// One workgroup (4 waves; 8 for more than 16 heads) per query tile. The head mix couples all heads of a (query, key) pair, so the heads are split
// over the waves: wave w owns heads [w * HPW, (w + 1) * HPW) for the score products AND for the outputs, and the capped
// scores of all heads meet in LDS in between. Per 16-key page:
//   1. S^T_g = K_kv(g) Q_g^T      (16 keys x 16 queries, MFMA 16x16x16, fp32 accumulate), scale, tanh cap -> LDS [H][256] fp32
//   2. mixed_h = sum_g talk[h][g] S^T_g   (fp32 VALU, talk as LDS broadcasts), window mask, online softmax per (h, query)
//      with a lazy running maximum, everything in base-2 exponent units
//   3. O^T_h += V^T_kv(h) P^T_h   with the fp32 weights split into two 16-bit terms (hi + lo): the product keeps ~16 bits of
//      every weight although the matrix core takes 16-bit operands.
// The transposed products keep the query index on the lanes' low four bits in every stage, so the softmax statistics of a
// query never move between lanes. Keys outside [pos - window + 1, pos] get weight zero; pages wholly outside are skipped.
//
// The general entry point (swl_masked_attn_tiles) adds: mask_kind 1 (chunked visibility: keys [floor(p / window) * window, p]),
// sink[H] (a logit per head that joins the denominator only), num_v_heads (value head = key head % num_v_heads: score maps
// that share their values), out_f32 (fp32 result), and a split of the heads over blockIdx.z (head_groups: every group of
// heads_per_group heads is a workgroup of its own — many heads over one shared key head, wide value heads).
//
// HEADS mode (decode steps of a layer whose heads all read ONE key head, e.g. latent attention): a tile is one token and the
// sixteen rows of the matrix-core tile are sixteen HEADS of that token instead of sixteen tokens of one head. The page's key
// and value fragments are then loaded once for sixteen heads and every product row is a real one, where the token-row form
// spends fifteen of sixteen rows on padding and repeats the page for every head. One wave per workgroup, grid (tokens, key
// shares, groups of sixteen heads); the softmax statistics stay per row as before.
#include "swl_common.h"

namespace swl {

constexpr int kWmThreads = 256;
constexpr int kWmWaves = 4;
constexpr int kWmTile = 16;     // queries per tile = keys per page = MFMA edge

template <typename T, int D, int DV, int HPW, int NW, bool MIX, bool HEADS = false>
__global__ __launch_bounds__(NW * 64, (HPW <= 2 && NW == 4 && HPW * (D + DV) <= 512) ? 2 : 1) void window_attn_mfma_kernel(
    T *out, const T *q, const T *k_cache, const T *v_cache, const int32_t *block_table, const int32_t *tok_seq,
    const int32_t *tok_pos, const int32_t *tile_row0, const int32_t *tile_cnt, const float *__restrict__ talk,
    const float *__restrict__ rel, int rel_len, int H, int G,
    int64_t q_tok_stride, int window, float scale, float softcap, int max_blocks_per_seq, int64_t block_stride,
    float *part_o, float *part_ml, int64_t num_tokens, int nbuf, int mask_kind, const float *__restrict__ sink, int GV,
    int out_f32, int hpg) {
    // [nbuf][H][64 lanes][4] capped scores of a page, then [H][H] the mixing matrix. nbuf = 2: pages alternate between two
    // score buffers and ONE barrier per page suffices (a wave that is a page ahead writes the other buffer)
    extern __shared__ float s_all[];
    float *tk = s_all + nbuf * H * 256;
    constexpr int CT = DV / 16;         // 16-column tiles of the value head
    constexpr float kLog2e = 1.4426950408889634f;
    constexpr float kLazy = 8.0f;       // (base-2 units: weights stay below 2^8)
    const int tile = blockIdx.x;
    const int row0 = __builtin_amdgcn_readfirstlane(tile_row0[tile]), cnt = __builtin_amdgcn_readfirstlane(tile_cnt[tile]);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // (tells the compiler that it is wave-uniform)
    const int li = lane & 15, lq = lane >> 4;       // query (or operand row) index; quarter
    // mixed scores come out in base-2 exponent units. MIX = false (no matrix): every head keeps its own scores, which then
    // never leave the registers of the wave that made them — no LDS, no barriers
    if constexpr (MIX) {
        for (int i = tid; i < H * H; i += NW * 64) tk[i] = talk[i] * kLog2e;
        __syncthreads();
    }
    const int p0 = __builtin_amdgcn_readfirstlane(tok_pos[row0]);
    const int32_t *bt = block_table + static_cast<int64_t>(__builtin_amdgcn_readfirstlane(tok_seq[row0])) * max_blocks_per_seq;
    const int rep = H / G;
    // heads of this workgroup: [hbase, hend); wave w owns HPW of them
    // (HEADS: row li is head hbase + li of the tile's one token; the wave's "head" h0 stands for the group)
    const int hbase = HEADS ? (static_cast<int>(blockIdx.z) * NW + wave) * kWmTile : static_cast<int>(blockIdx.z) * hpg;
    const int hend = min(H, hbase + (HEADS ? kWmTile : hpg));
    const int h0 = HEADS ? hbase : hbase + wave * HPW;
    const int qpos = HEADS ? p0 : p0 + li;           // this lane's query position (meaningful when li < cnt)
    const bool qok = HEADS ? hbase + li < H : li < cnt;
    // first visible key of this lane's query, and of the tile's first query
    const int qlo = window <= 0 ? 0 : mask_kind == 1 ? (qpos / window) * window : qpos - window + 1;
    const int lo_first = window <= 0 ? 0 : mask_kind == 1 ? (p0 / window) * window : (p0 - window + 1 > 0 ? p0 - window + 1 : 0);
    int kb0 = lo_first / kWmTile, kb1 = (p0 + cnt - 1) / kWmTile;
    if (gridDim.y > 1) {    // key split: this workgroup takes a contiguous share of the tile's pages (possibly none)
        const int per = (kb1 - kb0 + static_cast<int>(gridDim.y)) / static_cast<int>(gridDim.y);
        kb0 += per * static_cast<int>(blockIdx.y);
        kb1 = min(kb1, kb0 + per - 1);
    }
    // cap * tanh(s * scale / cap) = cap - 2 cap / (2^(s * c1) + 1) with c1 = 2 log2(e) scale / cap: five operations per score
    const float c1 = softcap > 0.f ? 2.0f * kLog2e * scale / softcap : 0.f, cap2 = -2.0f * softcap;

    float4_t acc[HPW][CT];
    float mrun[HPW], lrun[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        mrun[hh] = kNegBig;
        lrun[hh] = 0.f;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc[hh][ct] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    // the query row this lane feeds as B operand of S^T = K Q^T: row li of the tile (rows past cnt: the tile's last row)
    const T *qrow = HEADS ? q + static_cast<int64_t>(row0) * q_tok_stride + static_cast<int64_t>(qok ? hbase + li : hbase) * D
                          : q + static_cast<int64_t>(row0 + (qok ? li : cnt - 1)) * q_tok_stride;
    // Registers allowing (PIPE), the query fragments stay resident and the next page's key fragments are fetched while this
    // page's mix / softmax / value products run; the value fragments of a page are requested before its score products.
    constexpr int KS = D / 16;
    constexpr bool PIPE = HPW * D <= 576 && HPW * DV <= 512 && (NW <= 4 || HPW * (D + DV) <= 512);   // (eight waves: 256 registers each)
    vec4_t<T> qf[PIPE ? HPW : 1][KS], kf[PIPE ? HPW : 1][KS];
    // element offsets inside a page: of each head's key / value slice (wave-uniform, divided once) and of this lane's fragment
    int koff[HPW], voff[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int kv = __builtin_amdgcn_readfirstlane(min(h0 + hh, H - 1) / rep);
        koff[hh] = kv * kWmTile * D;
        voff[hh] = (kv % GV) * DV * kWmTile;
    }
    const int lane_k = li * D + 4 * lq;             // A operand of S^T: key li, dims 4 lq ..
    const int lane_v = li * kWmTile + 4 * lq;       // A operand of O^T: column li of a 16-column tile, keys 4 lq ..
    auto fetch_k = [&](int64_t blk) {
        const T *kblk = k_cache + blk * block_stride;
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
            for (int e = 0; e < KS; ++e) load4(kf[PIPE ? hh : 0][e], kblk + koff[hh] + lane_k + e * 16);
        }
    };
    if constexpr (PIPE) {
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            const int g = min(h0 + hh, H - 1);
#pragma unroll
            for (int e = 0; e < KS; ++e) load4(qf[hh][e], qrow + (HEADS ? 0 : g * D) + 4 * lq + e * 16);     // B: query li
        }
    }
    int blk_next = kb0 <= kb1 ? __builtin_amdgcn_readfirstlane(bt[kb0]) : 0;
    if constexpr (PIPE) {
        if (kb0 <= kb1) fetch_k(blk_next);
    }

    for (int kb = kb0; kb <= kb1; ++kb) {
        float *s_lds = s_all + (nbuf == 2 && ((kb - kb0) & 1) ? H * 256 : 0);
        const int64_t blk = blk_next;
        const int nxt = kb < kb1 ? bt[kb + 1] : 0;      // the next page's block id, requested a page ahead of its use
        const T *kblk = k_cache + blk * block_stride;
        const T *vblk = v_cache + blk * block_stride;
        // value fragments of this page, A operand of O^T += V^T P^T: V^T[col ct * 16 + li][keys 4 lq .. 4 lq + 3] — the pool keeps
        // a page's values transposed ([kv head][column][16 keys]), so this is one 8-byte load
        vec4_t<T> vfrag[PIPE ? HPW : 1][CT];
        auto fetch_v = [&](int hh) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) load4(vfrag[PIPE ? hh : 0][ct], vblk + voff[hh] + ct * 16 * kWmTile + lane_v);
        };
        if constexpr (PIPE) {
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) fetch_v(hh);
        }
        // ---- 1. capped scores of this wave's heads -> LDS -------------------------------------------------------------------
        float mixed[HPW][4];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
            for (int r = 0; r < 4; ++r) mixed[hh][r] = 0.f;
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            const int g = h0 + hh;
            if (g < hend) {
                float4_t st = {0.f, 0.f, 0.f, 0.f};
                if constexpr (PIPE) {
#pragma unroll
                    for (int e = 0; e < KS; ++e) st = mfma16(kf[hh][e], qf[hh][e], st);
                } else {
                    const T *kr = kblk + koff[hh] + lane_k;
                    const T *qr = qrow + (HEADS ? 0 : g * D) + 4 * lq;
#pragma unroll
                    for (int e = 0; e < KS; ++e) {
                        vec4_t<T> a, b;
                        load4(a, kr + e * 16);
                        load4(b, qr + e * 16);
                        st = mfma16(a, b, st);
                    }
                }
                mfma_results_ready<4>(st);
                // st[r] = S^T[key 4 lq + r][query li]
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (softcap > 0.f)      // (2^x overflowing to inf gives exactly cap, underflowing to 0 exactly -cap)
                        st[r] = fmaf(cap2, __builtin_amdgcn_rcpf(fast_exp2(st[r] * c1) + 1.0f), softcap);
                    else
                        st[r] *= scale;
                }
                if constexpr (MIX) {
                    *reinterpret_cast<float4_t *>(&s_lds[(g * 64 + lane) * 4]) = st;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) mixed[hh][r] = st[r] * kLog2e;
                }
            }
        }
        if constexpr (MIX) __syncthreads();
        blk_next = __builtin_amdgcn_readfirstlane(nxt);
        if constexpr (PIPE) {
            if (kb < kb1) fetch_k(blk_next);
        }
        // ---- 2. mix, mask, online softmax; 3. O^T += V^T P^T for this wave's heads ------------------------------------------
        const int kpos0 = kb * kWmTile + 4 * lq;     // position of this lane's key r = 0
        bool ok[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int kp = kpos0 + r;
            ok[r] = qok && kp <= qpos && kp >= qlo;
        }
        for (int g = 0; MIX && g < H; ++g) {
            const float4_t sv = *reinterpret_cast<const float4_t *>(&s_lds[(g * 64 + lane) * 4]);
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const int h = min(h0 + hh, H - 1);
                const float tw = tk[h * H + g];         // wave-uniform address: an LDS broadcast
#pragma unroll
                for (int r = 0; r < 4; ++r) mixed[hh][r] += tw * sv[r];
            }
        }
        if (rel) {      // learned bias by distance (query position - key position), one row of the table per head
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const float *rh = rel + static_cast<int64_t>(min(h0 + hh, H - 1)) * rel_len;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    mixed[hh][r] += rh[min(max(qpos - (kpos0 + r), 0), rel_len - 1)] * kLog2e;
            }
        }
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            const int h = h0 + hh;
            if (h < hend) {
                float cmax = kNegBig;
#pragma unroll
                for (int r = 0; r < 4; ++r) cmax = fmaxf(cmax, ok[r] ? mixed[hh][r] : kNegBig);
                cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
                cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
                // lazy running maximum: a row moves its reference only when a page raises it by more than kLazy, so the weights
                // stay below e^kLazy instead of below 1 (fp32 sums; the hi + lo split keeps their relative precision at either
                // scale) and alpha is exactly 1 on most pages: the accumulator rescale below is then skipped for the wave
                const float mnew = cmax - mrun[hh] > kLazy ? cmax : mrun[hh];
                const float alpha = fast_exp2(mrun[hh] - mnew);
                mrun[hh] = mnew;
                vec4_t<T> phi, plo;
                float psum = 0.f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float pv = ok[r] ? fast_exp2(mixed[hh][r] - mnew) : 0.f;
                    psum += pv;
                    phi[r] = to_t<T>(pv);
                    plo[r] = to_t<T>(pv - to_f(phi[r]));
                }
                lrun[hh] = lrun[hh] * alpha + psum;
                const bool rescale = !__all(alpha == 1.0f);     // (wave-uniform) most pages after the first leave the maxima alone
                if constexpr (!PIPE) fetch_v(hh);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    float4_t o = acc[hh][ct];
                    if (rescale) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[r] *= alpha;
                    }
                    o = mfma16(vfrag[PIPE ? hh : 0][ct], phi, o);
                    o = mfma16(vfrag[PIPE ? hh : 0][ct], plo, o);
                    acc[hh][ct] = o;
                }
            }
        }
        if constexpr (MIX) {
            if (nbuf == 1) __syncthreads();     // every wave is done with this page's scores before the next page overwrites them
        }
    }
    // ---- epilogue: O[query li][h][ct * 16 + 4 lq + r] = O^T / l -------------------------------------------------------------------
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = h0 + hh;
        if (h < hend) {
            float l = lrun[hh];
            l += __shfl_xor(l, 16, 64);
            l += __shfl_xor(l, 32, 64);
            const int orow = HEADS ? row0 : row0 + li, ohead = HEADS ? (qok ? hbase + li : hbase) : h;
            if (gridDim.y > 1) {    // partial result of this key share: unnormalised O, running maximum, sum
                const int64_t slot = (static_cast<int64_t>(blockIdx.y) * num_tokens + orow) * H + ohead;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    float4_t o = acc[hh][ct];
                    mfma_results_ready<4>(o);
                    if (qok) *reinterpret_cast<float4_t *>(part_o + slot * DV + ct * 16 + 4 * lq) = o;
                }
                if (qok && lq == 0) {
                    part_ml[slot * 2] = mrun[hh];
                    part_ml[slot * 2 + 1] = l;
                }
                continue;
            }
            float inv = 1.0f / l;
            if (sink) {     // the sink joins the denominator: rebase the row on max(m, sink) (base-2 units)
                const float sk = sink[ohead] * kLog2e, big = fmaxf(mrun[hh], sk);
                const float a = fast_exp2(mrun[hh] - big);
                inv = a / (l * a + fast_exp2(sk - big));
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                float4_t o = acc[hh][ct];
                mfma_results_ready<4>(o);
                if (qok) {
                    const int64_t at = (static_cast<int64_t>(orow) * H + ohead) * DV + ct * 16 + 4 * lq;
                    if (out_f32) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[r] *= inv;
                        *reinterpret_cast<float4_t *>(reinterpret_cast<float *>(out) + at) = o;
                    } else {
                        typedef T vec4 __attribute__((ext_vector_type(4)));
                        vec4 w;
#pragma unroll
                        for (int r = 0; r < 4; ++r) w[r] = to_t<T>(o[r] * inv);
                        *reinterpret_cast<vec4 *>(out + at) = w;
                    }
                }
            }
        }
    }
}

// out[t][h][:] = sum_s e^{m_s - M} O_s / sum_s e^{m_s - M} l_s over the key shares s (a share without keys has l = 0).
// The first wave evaluates the shares' weights once (one share per lane, at most 64) and leaves them in LDS.
template <typename T>
__global__ __launch_bounds__(256) void window_attn_combine_kernel(T *out, const float *part_o, const float *part_ml,
                                                                  int64_t rows, int dv, int nsplit, const float *sink, int H,
                                                                  int out_f32) {
    __shared__ float wgt[64];
    __shared__ float inv_den;
    const int64_t row = blockIdx.x;     // (token, head)
    if (threadIdx.x < 64) {
        const int sp = threadIdx.x;
        const bool live = sp < nsplit;
        const float m = live ? part_ml[(sp * rows + row) * 2] : kNegBig;     // (the maxima are in base-2 exponent units)
        const float l = live ? part_ml[(sp * rows + row) * 2 + 1] : 0.f;
        float mx = wave_allreduce_max(m);
        float extra = 0.f;
        if (sink) {
            const float sk = sink[row % H] * 1.4426950408889634f;
            mx = fmaxf(mx, sk);
            extra = exp2f(sk - mx);
        }
        const float w = live ? exp2f(m - mx) : 0.f;
        const float den = wave_allreduce_sum(w * l) + extra;
        wgt[sp] = w;
        if (sp == 0) inv_den = 1.0f / den;
    }
    __syncthreads();
    const float inv = inv_den;
    for (int c = threadIdx.x; c < dv; c += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) a += wgt[s] * part_o[(s * rows + row) * dv + c];
        if (out_f32) reinterpret_cast<float *>(out)[row * dv + c] = a * inv;
        else out[row * dv + c] = to_t<T>(a * inv);
    }
}

template <typename T, int D, int DV, bool MIXOK>
int launch_wm(int hpw, dim3 grid, size_t lds, hipStream_t s, T *out, const T *q, const T *kc, const T *vc,
              const int32_t *bt, const int32_t *ts, const int32_t *tp, const int32_t *r0, const int32_t *cn,
              const float *talk, const float *rel, int rel_len, int H, int G, int64_t qs, int window, float scale,
              float softcap, int mb, int64_t bs,
              float *po, float *pml, int64_t nt, int nbuf, int mask_kind, const float *sink, int GV, int out_f32, int hpg,
              bool heads_mode) {
    if (heads_mode) {       // rows are heads: one wave per workgroup, grid.z = groups of sixteen heads
        hipLaunchKernelGGL((window_attn_mfma_kernel<T, D, DV, 1, 1, false, true>), grid, dim3(64), 0, s, out, q, kc, vc, bt, ts,
                           tp, r0, cn, nullptr, nullptr, 0, H, G, qs, window, scale, softcap, mb, bs, po, pml, nt, nbuf,
                           mask_kind, sink, GV, out_f32, hpg);
        if (grid.y > 1) {
            const int64_t rows = nt * H;
            hipLaunchKernelGGL((window_attn_combine_kernel<T>), dim3(static_cast<unsigned>(rows)), dim3(DV < 256 ? 64 : 256), 0,
                               s, out, po, pml, rows, DV, static_cast<int>(grid.y), sink, H, out_f32);
        }
        return check_launch();
    }
#define SWL_WM_LAUNCH1(HPW, NW, MIX)                                                                                         \
    hipLaunchKernelGGL((window_attn_mfma_kernel<T, D, DV, HPW, NW, MIX>), grid, dim3(NW * 64), MIX ? lds : 0, s, out, q, kc, \
                       vc, bt, ts, tp, r0, cn, talk, rel, rel_len, H, G, qs, window, scale, softcap, mb, bs, po, pml, nt, nbuf, mask_kind,  \
                       sink, GV, out_f32, hpg)
    // (a wave's accumulators: HPW * DV / 4 registers — variants beyond 128 of them are not compiled for the wide shapes)
#define SWL_WM_LAUNCH(HPW, NW)                                 \
    if constexpr (!MIXOK && HPW * DV > 512) {                  \
        return SWL_ERR_UNSUPPORTED;                            \
    } else if (talk) {                                         \
        if constexpr (MIXOK) SWL_WM_LAUNCH1(HPW, NW, true);    \
        else return SWL_ERR_UNSUPPORTED;                       \
    } else SWL_WM_LAUNCH1(HPW, NW, false)
    // heads per wave x waves: up to 16 heads on four waves, more on eight (four heads per wave at most: the accumulators of
    // eight 128-wide heads do not fit a wave's registers)
    switch (hpw) {
    case 1: SWL_WM_LAUNCH(1, 4); break;
    case 2: SWL_WM_LAUNCH(2, 4); break;
    case 4: SWL_WM_LAUNCH(4, 4); break;
    case 8: SWL_WM_LAUNCH(4, 8); break;
    default: return SWL_ERR_UNSUPPORTED;
    }
#undef SWL_WM_LAUNCH
#undef SWL_WM_LAUNCH1
    if (grid.y > 1) {
        const int64_t rows = nt * H;
        hipLaunchKernelGGL((window_attn_combine_kernel<T>), dim3(static_cast<unsigned>(rows)), dim3(DV < 256 ? 64 : 256), 0, s,
                           out, po, pml, rows, DV, static_cast<int>(grid.y), sink, H, out_f32);
    }
    return check_launch();
}

} // namespace swl

// (dim, vdim) pairs with a compiled kernel; the first four also with the head-mixing matrix
#define SWL_WM_SHAPES_MIX(X) X(64, 64) X(128, 128) X(128, 64) X(64, 128)
#define SWL_WM_SHAPES_PLAIN(X) \
    X(32, 32) X(32, 64) X(48, 48) X(48, 96) X(64, 32) X(64, 96) X(96, 64) X(96, 96) X(128, 96) X(96, 128) X(160, 128) X(192, 128) \
    X(288, 256) X(320, 256) X(576, 512)

static int wm_shape_kind(int dim, int vdim) {      // 2: with or without mixing, 1: without only, 0: none
#define SWL_WM_IS(DD, DDV) if (dim == DD && vdim == DDV) return 2;
    SWL_WM_SHAPES_MIX(SWL_WM_IS)
#undef SWL_WM_IS
#define SWL_WM_IS(DD, DDV) if (dim == DD && vdim == DDV) return 1;
    SWL_WM_SHAPES_PLAIN(SWL_WM_IS)
#undef SWL_WM_IS
    return 0;
}

/* 1 when swl_window_attn_tiles serves this shape (else the caller uses swl_window_attn). */
extern "C" int swl_window_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim,
                                               int32_t dtype) {
    if (dtype != SWL_F16 && dtype != SWL_BF16) return 0;
    if (num_q_heads <= 0 || num_q_heads > 32 || num_kv_heads <= 0 || num_q_heads % num_kv_heads) return 0;
    return wm_shape_kind(dim, vdim) == 2;
}

/* 1 when swl_masked_attn_tiles serves this shape without a head-mixing matrix. More than 32 heads are served when the
 * heads can be split into groups (no mixing), 32 at most per workgroup. */
extern "C" int swl_masked_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t num_v_heads, int32_t dim,
                                               int32_t vdim, int32_t dtype) {
    if (dtype != SWL_F16 && dtype != SWL_BF16) return 0;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads) return 0;
    if (num_v_heads <= 0 || num_kv_heads % num_v_heads) return 0;
    return wm_shape_kind(dim, vdim) > 0;
}

extern "C" int swl_masked_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache,
                                     const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                                     const int32_t *tile_row0, const int32_t *tile_cnt, const float *talk,
                                     const float *rel, int32_t rel_len, int32_t num_tiles, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim,
                                     int32_t vdim, int64_t q_tok_stride, int32_t window, float scale, float softcap,
                                     int32_t max_blocks_per_seq, int64_t block_stride, int32_t key_splits,
                                     float *scratch, int64_t num_tokens, int32_t mask_kind, const float *sink,
                                     int32_t num_v_heads, int32_t out_f32, int32_t heads_per_group, int32_t dtype,
                                     swl_stream_t stream) {
    if (num_tiles < 0 || window < 0 || key_splits < 1 || key_splits > 64) return SWL_ERR_BAD_ARG;
    if (key_splits > 1 && (!scratch || num_tokens <= 0 || (reinterpret_cast<uintptr_t>(scratch) & 15)))
        return SWL_ERR_BAD_ARG;
    if (mask_kind < 0 || mask_kind > 1 || heads_per_group < -1) return SWL_ERR_BAD_ARG;
    // heads_per_group -1: the rows of a tile are heads (every tile is ONE token, all heads read one key head, no mix, no bias)
    const bool heads_mode = heads_per_group == -1;
    if (heads_mode && (talk || rel || num_kv_heads != 1 || num_tiles != num_tokens)) return SWL_ERR_BAD_ARG;
    if (!swl_masked_attn_tiles_supported(num_q_heads, num_kv_heads, num_v_heads, dim, vdim, dtype)) return SWL_ERR_UNSUPPORTED;
    // heads per workgroup: all of them when they are mixed (the mix couples them), else the caller's choice (0: all)
    int hpg = (talk || heads_per_group <= 0) ? num_q_heads : (heads_per_group < num_q_heads ? heads_per_group : num_q_heads);
    if (heads_mode) hpg = 16;
    if (hpg > 32 && !heads_mode) {
        if (talk) return SWL_ERR_UNSUPPORTED;
        hpg = 32;
    }
    // a group asked for by the caller never needs more accumulators than a wave has registers for: wide value heads go to
    // more, smaller groups
    if (!talk && heads_per_group > 0) {
        const int per_wave = vdim >= 512 ? 1 : vdim >= 256 ? 2 : vdim > 64 ? 4 : 8;
        if (hpg > 4 * per_wave) hpg = 4 * per_wave;
    }
    if (num_tiles == 0) return SWL_OK;
    if (!out || !q || !k_cache || !v_cache || !block_table || !tok_seq || !tok_pos || !tile_row0 || !tile_cnt ||
        (rel && rel_len <= 0))
        return SWL_ERR_BAD_ARG;
    if ((q_tok_stride & 3) || (block_stride & 3) || (reinterpret_cast<uintptr_t>(q) & 7) ||
        (reinterpret_cast<uintptr_t>(k_cache) & 7) || (reinterpret_cast<uintptr_t>(v_cache) & 7) ||
        (reinterpret_cast<uintptr_t>(out) & (out_f32 ? 15 : 7)))
        return SWL_ERR_BAD_ARG;     // 8-byte operand loads
    int hpw = (hpg + swl::kWmWaves - 1) / swl::kWmWaves;
    hpw = hpw <= 1 ? 1 : hpw <= 2 ? 2 : hpw <= 4 ? 4 : 8;
    const int groups = (num_q_heads + hpg - 1) / hpg;
    const size_t one = static_cast<size_t>(num_q_heads) * 256, mixw = static_cast<size_t>(num_q_heads) * num_q_heads;
    const int nbuf = (2 * one + mixw) * sizeof(float) <= 64 * 1024 ? 2 : 1;
    const size_t lds = (nbuf * one + mixw) * sizeof(float);
    const dim3 grid(static_cast<unsigned>(num_tiles), static_cast<unsigned>(key_splits), static_cast<unsigned>(groups));
    hipStream_t s = static_cast<hipStream_t>(stream);
    // scratch: [splits][tokens][H][vdim] fp32 partial outputs, then [splits][tokens][H][2] (maximum, sum)
    float *part_o = scratch;
    float *part_ml = scratch ? scratch + static_cast<int64_t>(key_splits) * num_tokens * num_q_heads * vdim : nullptr;
#define SWL_WM_SHAPE_(DD, DDV, MIXOK)                                                                                     \
    if (dim == DD && vdim == DDV)                                                                                         \
        return swl::launch_wm<T, DD, DDV, MIXOK>(hpw, grid, lds, s, static_cast<T *>(out), static_cast<const T *>(q),    \
                                          static_cast<const T *>(k_cache), static_cast<const T *>(v_cache), block_table, \
                                          tok_seq, tok_pos, tile_row0, tile_cnt, talk, rel, rel_len, num_q_heads, num_kv_heads, \
                                          q_tok_stride, window, scale, softcap, max_blocks_per_seq, block_stride, part_o, \
                                          part_ml, num_tokens, nbuf, mask_kind, sink, num_v_heads, out_f32, hpg, heads_mode);
#define SWL_WM_SHAPE_MIX(DD, DDV) SWL_WM_SHAPE_(DD, DDV, true)
#define SWL_WM_SHAPE_PLAIN(DD, DDV) SWL_WM_SHAPE_(DD, DDV, false)
    SWL_DISPATCH_DTYPE(dtype, T, {
        SWL_WM_SHAPES_MIX(SWL_WM_SHAPE_MIX)
        SWL_WM_SHAPES_PLAIN(SWL_WM_SHAPE_PLAIN)
    });
#undef SWL_WM_SHAPE_
#undef SWL_WM_SHAPE_MIX
#undef SWL_WM_SHAPE_PLAIN
    return SWL_ERR_UNSUPPORTED;
}

extern "C" int swl_window_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache,
                                     const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                                     const int32_t *tile_row0, const int32_t *tile_cnt, const float *talk,
                                     const float *rel, int32_t rel_len, int32_t num_tiles, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim,
                                     int32_t vdim, int64_t q_tok_stride, int32_t window, float scale, float softcap,
                                     int32_t max_blocks_per_seq, int64_t block_stride, int32_t key_splits,
                                     float *scratch, int64_t num_tokens, int32_t dtype, swl_stream_t stream) {
    if (!swl_window_attn_tiles_supported(num_q_heads, num_kv_heads, dim, vdim, dtype)) return SWL_ERR_UNSUPPORTED;
    return swl_masked_attn_tiles(out, q, k_cache, v_cache, block_table, tok_seq, tok_pos, tile_row0, tile_cnt, talk, rel,
                                 rel_len, num_tiles, num_q_heads, num_kv_heads, dim, vdim, q_tok_stride, window, scale,
                                 softcap, max_blocks_per_seq, block_stride, key_splits, scratch, num_tokens, 0, nullptr,
                                 num_kv_heads, 0, 0, dtype, stream);
}
