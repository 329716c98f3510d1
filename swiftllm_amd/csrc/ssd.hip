// ssd.hip — a selective state-space recurrence with a scalar decay per head (the "state-space duality" form) as a recurrent
// mixer with per-sequence state slots, for any mixture of prompt portions and decoded tokens.
//
// Per head a state S [state, vdim] (fp32, in the sequence's slot) is carried from token to token:
//     S <- exp(-exp(A_log) dt) S + dt B x^T;     y = S^T C + D x
// with x [vdim] the head's input, B and C [state] shared by the heads of a group, dt = softplus(raw + dt_bias) > 0.
//
//   swl_ssd_prep:  one workgroup per token. The input projection row [z | x | B | C | dt] -> short causal convolution with
//                  bias + SiLU on the x | B | C channels (carried inputs: conv_tail.h) -> fp32 rows [x | B | C]; dt and the
//                  decay per head. Everything after the loads is fp32.
//   swl_ssd_scan:  one workgroup per (portion, head, share of the columns). The columns of S are independent recurrences:
//                  a column belongs to L adjacent lanes, each holding state / L of its elements in registers; per token the
//                  lanes exchange one partial dot product (S^T C) through DPP. B, C, x, dt and the decay of 16 tokens at a
//                  time are staged in LDS; a wave of loaders stages the next 16 tokens into a second buffer while the others
//                  walk the current ones. The token loop is sequential whatever the cut of the sequence into steps: the same
//                  operations in the same order.
//   swl_gated_group_rmsnorm: out = g / rms(g over a group of columns) * w with g = y * silu(z): gated first, normed
//                  afterwards, the row in `groups` equal parts.
#include "swl_common.h"
#include "conv_tail.h"

namespace swl {

constexpr int kSsThreads = 256;
constexpr int kSsChunk = 16;        // tokens staged at a time

__device__ __forceinline__ float ss_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(kSsThreads) void ssd_prep_kernel(
    float *xbc, float *dt_out, float *decay, const T *proj, int64_t proj_stride, const float *conv_w, const float *conv_b,
    const float *a_log, const float *dt_bias, float *state, int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos,
    const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq, int64_t num_tokens, int heads, int inner,
    int C, int taps) {
    const int64_t t = blockIdx.x;
    const T *conv_in = proj + inner;        // the convolved channels follow the gate columns
    const T *row = conv_in + t * proj_stride;
    const ConvTail tail(state, slot_stride, tail_off, tok_pos, tok_start, tok_state, tok_seq, num_tokens, C, taps, t);
    bool wide = false;
    if constexpr (sizeof(T) == 2) wide = ConvTail::wide_ok(conv_in, proj_stride, conv_w, state, slot_stride, tail_off, C);
    if (wide) {
        if constexpr (sizeof(T) == 2) {
            for (int c = threadIdx.x * 8; c < C; c += kSsThreads * 8) {
                const vec8_t<T> x = load8(row + c);
                float cur[8], a[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) cur[j] = to_f(x[j]);
                tail.conv8(conv_in, proj_stride, conv_w, c, cur, a);
                float o[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float v = a[j] + conv_b[c + j];
                    o[j] = v * ss_sigmoid(v);
                }
                float *dst = xbc + t * C + c;       // (C and c are multiples of 8: 32-byte aligned)
                *reinterpret_cast<float4_t *>(dst) = float4_t{o[0], o[1], o[2], o[3]};
                *reinterpret_cast<float4_t *>(dst + 4) = float4_t{o[4], o[5], o[6], o[7]};
                tail.save8(conv_in, proj_stride, c, cur);
            }
        }
    } else {
        for (int c = threadIdx.x; c < C; c += kSsThreads) {
            const float cur = to_f(row[c]);
            const float v = tail.conv(conv_in, proj_stride, conv_w, c, cur) + conv_b[c];
            xbc[t * C + c] = v * ss_sigmoid(v);
            tail.save(conv_in, proj_stride, c, cur);
        }
    }
    for (int h = threadIdx.x; h < heads; h += kSsThreads) {
        const float z = to_f(row[C + h]) + dt_bias[h];
        const float sp = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));      // softplus, no clamp of the step
        dt_out[t * heads + h] = sp;
        decay[t * heads + h] = expf(-expf(a_log[h]) * sp);
    }
}

// LDS rows of B and C are padded by 4 floats per lane slice: the L lanes of a column read L different 16-byte pieces at once,
// and without the padding slices of 8 / 16 / 32 floats start in the same banks.
__host__ __device__ inline int ss_row_floats(int N, int L, int ds) { return L * (ds + 4); }

template <int MAXDS, int L, bool EXACT>
__global__ __launch_bounds__(1024) void ssd_scan_kernel(float *y, const float *xbc, const float *dt, const float *decay,
                                                        const float *dskip, float *state, int64_t slot_stride, int64_t s_off,
                                                        const int32_t *seq_row0, const int32_t *seq_cnt,
                                                        const int32_t *tok_pos, const int32_t *tok_state, int heads, int groups,
                                                        int N, int P, int cpw, int ds, int nload) {
    // nload > 0: the last nload threads of the workgroup only LOAD — they stage chunk c + 1 into the other LDS buffer while
    // the first threads walk the tokens of chunk c, one barrier per chunk. nload = 0: everybody stages, then walks.
    // EXACT: ds == MAXDS and L * ds == N (no predicates in the walk).
    extern __shared__ float lds[];
    const int dp = ss_row_floats(N, L, ds);
    const int buf_floats = kSsChunk * (2 * dp + cpw + 2);
    const int seq = blockIdx.x, h = blockIdx.y;
    const int col0 = blockIdx.z * cpw;
    const int row0 = seq_row0[seq], cnt = seq_cnt[seq];
    const int g = h / (heads / groups);
    const int inner = heads * P, C = inner + 2 * groups * N;
    const int ncomp = static_cast<int>(blockDim.x) - nload;
    const bool computes = static_cast<int>(threadIdx.x) < ncomp;
    const int lc = computes ? threadIdx.x / L : 0, l = threadIdx.x % L;
    const int col = col0 + lc;
    const bool live = computes && lc < cpw && col < P;     // (threads that pad the workgroup to whole waves own no column)
    const int i0 = l * ds;
    float *S = state + static_cast<int64_t>(tok_state[row0] >> 1) * slot_stride + s_off + static_cast<int64_t>(h) * N * P;
    const bool fresh = tok_pos[row0] == 0;      // a sequence starts from the zero state whatever the slot held
    float s[MAXDS];
#pragma unroll
    for (int i = 0; i < MAXDS; ++i)
        s[i] = (live && !fresh && i < ds && i0 + i < N) ? S[static_cast<int64_t>(i0 + i) * P + col] : 0.f;
    const float dh = dskip[h];
    const bool quads = EXACT || (ds & 3) == 0;  // 16-byte LDS reads

    // Stage the chunk at c0 into `buf` with threads sid, sid + sn, ...: all of a thread's loads are issued before the first
    // one is waited for — one memory round trip per chunk.
    auto stage = [&](int c0, float *buf, int sid, int sn) {
        const int cn = min(kSsChunk, cnt - c0);
        float *Bs = buf, *Cs = Bs + kSsChunk * dp, *xs = Cs + kSsChunk * dp, *dts = xs + kSsChunk * cpw, *das = dts + kSsChunk;
        for (int n = sid; n < N; n += sn) {
            float tb[kSsChunk], tc[kSsChunk];
            const float *src = xbc + static_cast<int64_t>(row0 + c0) * C + inner + g * N + n;
#pragma unroll
            for (int j = 0; j < kSsChunk; ++j) {
                const int64_t jj = min(j, cn - 1);      // (rows past the chunk's end re-read its last row: never used)
                tb[j] = src[jj * C];
                tc[j] = src[jj * C + groups * N];
            }
            const int at = n + 4 * (n / ds);
#pragma unroll
            for (int j = 0; j < kSsChunk; ++j) {
                Bs[j * dp + at] = tb[j];
                Cs[j * dp + at] = tc[j];
            }
        }
        for (int e = sid; e < cpw; e += sn) {
            float tv[kSsChunk];
            const float *src = xbc + static_cast<int64_t>(row0 + c0) * C + h * P + min(col0 + e, P - 1);
#pragma unroll
            for (int j = 0; j < kSsChunk; ++j) tv[j] = src[static_cast<int64_t>(min(j, cn - 1)) * C];
#pragma unroll
            for (int j = 0; j < kSsChunk; ++j) xs[j * cpw + e] = tv[j];
        }
        for (int j = sid; j < cn; j += sn) {
            dts[j] = dt[static_cast<int64_t>(row0 + c0 + j) * heads + h];
            das[j] = decay[static_cast<int64_t>(row0 + c0 + j) * heads + h];
        }
    };

    // Walk the tokens of the chunk at c0 (staged in `buf`): the sequential part.
    auto walk = [&](int c0, const float *buf) {
        const int cn = min(kSsChunk, cnt - c0);
        const float *Bs = buf, *Cs = Bs + kSsChunk * dp, *xs = Cs + kSsChunk * dp, *dts = xs + kSsChunk * cpw;
        const float *das = dts + kSsChunk;
#pragma unroll 2
        for (int j = 0; j < cn; ++j) {
            const float xv = xs[j * cpw + (lc < cpw ? lc : 0)];
            const float dA = das[j], dtx = dts[j] * xv;
            const float *bj = Bs + j * dp + l * (ds + 4), *cj = Cs + j * dp + l * (ds + 4);
            float br[MAXDS], cr[MAXDS];
            if (quads) {
#pragma unroll
                for (int i = 0; i < MAXDS; i += 4) {
                    if (EXACT || i < ds) {
                        const float4_t b4 = *reinterpret_cast<const float4_t *>(bj + i);
                        const float4_t c4 = *reinterpret_cast<const float4_t *>(cj + i);
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            br[i + c] = b4[c];
                            cr[i + c] = c4[c];
                        }
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < MAXDS; ++i) {
                    br[i] = i < ds ? bj[i] : 0.f;
                    cr[i] = i < ds ? cj[i] : 0.f;
                }
            }
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < MAXDS; ++i) {
                if (EXACT || (i < ds && i0 + i < N)) {
                    s[i] = fmaf(br[i], dtx, s[i] * dA);
                    acc = fmaf(s[i], cr[i], acc);
                }
            }
            acc = group_allreduce_sum<L>(acc);
            if (l == 0 && live) y[static_cast<int64_t>(row0 + c0 + j) * inner + h * P + col] = fmaf(dh, xv, acc);
        }
    };

    if (nload > 0) {
        if (!computes) stage(0, lds, static_cast<int>(threadIdx.x) - ncomp, nload);
        __syncthreads();
        int c = 0;
        for (int c0 = 0; c0 < cnt; c0 += kSsChunk, ++c) {
            if (computes) walk(c0, lds + (c & 1) * buf_floats);
            else if (c0 + kSsChunk < cnt) stage(c0 + kSsChunk, lds + ((c + 1) & 1) * buf_floats, static_cast<int>(threadIdx.x) - ncomp, nload);
            __syncthreads();    // chunk c has been walked and chunk c + 1 is in place
        }
    } else {
        for (int c0 = 0; c0 < cnt; c0 += kSsChunk) {
            __syncthreads();    // the previous chunk has been consumed
            stage(c0, lds, threadIdx.x, blockDim.x);
            __syncthreads();
            walk(c0, lds);
        }
    }
    if (!live) return;
#pragma unroll
    for (int i = 0; i < MAXDS; ++i)
        if (i < ds && i0 + i < N) S[static_cast<int64_t>(i0 + i) * P + col] = s[i];
}

template <typename T>
__global__ __launch_bounds__(kSsThreads) void gated_group_rmsnorm_kernel(T *out, const float *y, const T *gate,
                                                                         int64_t gate_stride, const float *w, float eps,
                                                                         int cols, int part) {
    __shared__ float red[kSsThreads / 64];
    const int64_t t = blockIdx.x;
    const int c0 = blockIdx.y * part;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float ss = 0.f;
    for (int c = threadIdx.x; c < part; c += kSsThreads) {
        const float z = to_f(gate[t * gate_stride + c0 + c]);
        const float v = y[t * cols + c0 + c] * (z * ss_sigmoid(z));
        ss += v * v;
    }
    ss = wave_allreduce_sum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < kSsThreads / 64; ++i) ss += red[i];
    const float r = 1.0f / sqrtf(ss / static_cast<float>(part) + eps);
    for (int c = threadIdx.x; c < part; c += kSsThreads) {
        const float z = to_f(gate[t * gate_stride + c0 + c]);
        const float v = y[t * cols + c0 + c] * (z * ss_sigmoid(z));
        out[t * cols + c0 + c] = to_t<T>(v * r * w[c0 + c]);
    }
}

template <int L>
int launch_ssd(int ds, dim3 grid, dim3 block, size_t lds, hipStream_t s, float *y, const float *xbc, const float *dt,
               const float *decay, const float *dskip, float *state, int64_t slot_stride, int64_t s_off,
               const int32_t *seq_row0, const int32_t *seq_cnt, const int32_t *tok_pos, const int32_t *tok_state, int heads,
               int groups, int N, int P, int cpw, int nload) {
#define SWL_SS_LAUNCH1(M, X)                                                                                                  \
    hipLaunchKernelGGL((ssd_scan_kernel<M, L, X>), grid, block, lds, s, y, xbc, dt, decay, dskip, state, slot_stride, s_off, \
                       seq_row0, seq_cnt, tok_pos, tok_state, heads, groups, N, P, cpw, ds, nload)
#define SWL_SS_LAUNCH(M)                                    \
    if (ds == M && L * ds == N) SWL_SS_LAUNCH1(M, true);    \
    else SWL_SS_LAUNCH1(M, false)
    if (ds <= 8) { SWL_SS_LAUNCH(8); }
    else if (ds <= 16) { SWL_SS_LAUNCH(16); }
    else if (ds <= 32) { SWL_SS_LAUNCH(32); }
    else if (ds <= 64) { SWL_SS_LAUNCH(64); }
    else return SWL_ERR_UNSUPPORTED;
#undef SWL_SS_LAUNCH
#undef SWL_SS_LAUNCH1
    return check_launch();
}

} // namespace swl

extern "C" int swl_ssd_prep(float *xbc, float *dt, float *decay, const void *proj, int64_t proj_stride, const float *conv_w,
                            const float *conv_b, const float *a_log, const float *dt_bias, float *state, int64_t slot_stride,
                            int64_t tail_off, const int32_t *tok_pos, const int32_t *tok_start, const int32_t *tok_state,
                            const int32_t *tok_seq, int64_t num_tokens, int32_t num_heads, int32_t vdim, int32_t state_dim,
                            int32_t groups, int32_t taps, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || vdim <= 0 || state_dim <= 0 || groups <= 0 || taps < 1 || num_heads % groups)
        return SWL_ERR_BAD_ARG;
    const int64_t inner = static_cast<int64_t>(num_heads) * vdim, C = inner + 2LL * groups * state_dim;
    if (proj_stride < inner + C + num_heads || C > 0x7fffffffLL) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!xbc || !dt || !decay || !proj || !conv_w || !conv_b || !a_log || !dt_bias || !tok_pos || !tok_start || !tok_seq)
        return SWL_ERR_BAD_ARG;
    if (taps > 1 && (!state || !tok_state)) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::ssd_prep_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kSsThreads), 0,
                           static_cast<hipStream_t>(stream), xbc, dt, decay, static_cast<const T *>(proj), proj_stride,
                           conv_w, conv_b, a_log, dt_bias, state, slot_stride, tail_off, tok_pos, tok_start, tok_state,
                           tok_seq, num_tokens, num_heads, static_cast<int>(inner), static_cast<int>(C), taps);
    });
    return swl::check_launch();
}

extern "C" int swl_ssd_scan(float *y, const float *xbc, const float *dt, const float *decay, const float *dskip, float *state,
                            int64_t slot_stride, int64_t s_off, const int32_t *seq_row0, const int32_t *seq_cnt,
                            const int32_t *tok_pos, const int32_t *tok_state, int32_t num_seqs, int32_t num_heads,
                            int32_t vdim, int32_t state_dim, int32_t groups, swl_stream_t stream) {
    if (num_seqs < 0 || num_heads <= 0 || vdim <= 0 || state_dim <= 0 || groups <= 0 || num_heads % groups)
        return SWL_ERR_BAD_ARG;
    if (num_seqs == 0) return SWL_OK;
    if (!y || !xbc || !dt || !decay || !dskip || !state || !seq_row0 || !seq_cnt || !tok_pos || !tok_state)
        return SWL_ERR_BAD_ARG;
    if (num_heads > 65535) return SWL_ERR_UNSUPPORTED;
    // lanes per column: as many (a power of two, at most 16) as keep at least 16 state elements per lane
    int L = 16;
    while (L > 1 && (state_dim + L - 1) / L < 16) L >>= 1;
    const int ds = (state_dim + L - 1) / L;
    // columns per workgroup: all of them when there are (portion, head) pairs enough to fill the chip; a long prompt alone
    // is a sequential walk, so its columns are shared out over more workgroups (down to 16 columns each)
    int cpw = vdim < 960 / L ? vdim : 960 / L;
    while (static_cast<int64_t>(num_seqs) * num_heads * ((vdim + cpw - 1) / cpw) < 512 && cpw % 2 == 0 && cpw > 16) cpw /= 2;
    const unsigned shares = static_cast<unsigned>((vdim + cpw - 1) / cpw);
    const size_t one = (static_cast<size_t>(swl::kSsChunk) * (2 * swl::ss_row_floats(state_dim, L, ds) + cpw + 2)) * sizeof(float);
    if (one > 64 * 1024 || shares > 65535) return SWL_ERR_UNSUPPORTED;
    const int ncomp = ((cpw * L + 63) / 64) * 64;
    // a wave of loaders and a second LDS buffer when both fit
    const int nload = (ncomp + 64 <= 1024 && 2 * one <= 64 * 1024) ? 64 : 0;
    const size_t lds = nload ? 2 * one : one;
    const dim3 grid(static_cast<unsigned>(num_seqs), static_cast<unsigned>(num_heads), shares);
    const dim3 block(static_cast<unsigned>(ncomp + nload));
    hipStream_t s = static_cast<hipStream_t>(stream);
#define SWL_SS_L(LL)                                                                                                          \
    case LL: return swl::launch_ssd<LL>(ds, grid, block, lds, s, y, xbc, dt, decay, dskip, state, slot_stride, s_off, seq_row0, \
                                        seq_cnt, tok_pos, tok_state, num_heads, groups, state_dim, vdim, cpw, nload)
    switch (L) {
        SWL_SS_L(1);
        SWL_SS_L(2);
        SWL_SS_L(4);
        SWL_SS_L(8);
        SWL_SS_L(16);
    }
#undef SWL_SS_L
    return SWL_ERR_UNSUPPORTED;
}

extern "C" int swl_gated_group_rmsnorm(void *out, const float *y, const void *gate, int64_t gate_stride, const float *w,
                                       float eps, int64_t num_tokens, int32_t cols, int32_t groups, int32_t dtype,
                                       swl_stream_t stream) {
    if (num_tokens < 0 || cols <= 0 || groups <= 0 || cols % groups || gate_stride < cols) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !y || !gate || !w) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL || groups > 65535) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::gated_group_rmsnorm_kernel<T>), dim3(static_cast<unsigned>(num_tokens), groups),
                           dim3(swl::kSsThreads), 0, static_cast<hipStream_t>(stream), static_cast<T *>(out), y,
                           static_cast<const T *>(gate), gate_stride, w, eps, cols, cols / groups);
    });
    return swl::check_launch();
}
