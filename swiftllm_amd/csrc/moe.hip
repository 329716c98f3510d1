// moe.hip — mixture-of-experts feed-forward: fp32 router with top-k selection, and the expert products for the
// token counts where an expert's weights are streamed once per assignment (decode and short portions).
//
//   swl_moe_route:        logits = router h + bias in fp32; the `top` largest (ties: lowest expert id); weights =
//                         softmax over the chosen logits only.
//   swl_moe_gate_up:      for every (token, chosen expert): g = min(W_gate h, limit), u = clamp(W_up h, +-limit),
//                         y = g * sigmoid(1.702 g) * (u + 1); fp32 accumulation, y rounded to the compute dtype.
//   swl_moe_down_combine: out[t] = sum_j weight[t][j] * (W_down[e_j] y[t][j]) with fp32 accumulation through the weighted
//                         sum (fixed order j = 0, 1, ...: the result does not depend on what else is in the batch).
//
//   swl_moe_route_grouped: scores s = sigmoid(router h); experts are CHOSEN by s + correction, inside the `keep` best of
//                         `count` equal groups of neighbouring experts (a group's score: the sum of its two largest choice
//                         scores); the weights are the chosen experts' s divided by their sum.
//   act (swl_moe_gate_up, swl_glu_clamp; glu = 3 of swl_moe_expert_stationary): 0 the clamped unit above, 1 the plain gated
//                         unit y = silu(g) * u.
//
// Expert weights are stacked: gate_up [experts, 2 ff, width] (gate rows, then up rows), down [experts, width, ff].
#include "swl_common.h"

namespace swl {

__device__ __forceinline__ bool aligned16_dev(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kMoeThreads = 256;
constexpr int kMoeWaves = kMoeThreads / 64;

// Per-lane share of sum_i x[i] * w[i] over a row of n elements (x fp32 in LDS, w in global memory); the caller reduces
// over the wave. 16-bit rows whose length is a multiple of 8 are read 16 bytes per lane.
template <typename T>
__device__ __forceinline__ float lane_dot(const float *x, const T *w, int n, int lane) {
    float a = 0.f;
    if constexpr (sizeof(T) == 2) {
        if ((n & 7) == 0 && aligned16_dev(w)) {
            for (int i = lane * 8; i < n; i += 64 * 8) {
                const vec8_t<T> v = load8(w + i);
#pragma unroll
                for (int j = 0; j < 8; ++j) a += x[i + j] * to_f(v[j]);
            }
            return a;
        }
    }
    for (int i = lane; i < n; i += 64) a += x[i] * to_f(w[i]);
    return a;
}
// The same with both rows in global memory.
template <typename T>
__device__ __forceinline__ float lane_dot2(const T *x, const T *w, int n, int lane) {
    float a = 0.f;
    if constexpr (sizeof(T) == 2) {
        if ((n & 7) == 0 && aligned16_dev(w) && aligned16_dev(x)) {
            for (int i = lane * 8; i < n; i += 64 * 8) {
                const vec8_t<T> v = load8(w + i), u = load8(x + i);
#pragma unroll
                for (int j = 0; j < 8; ++j) a += to_f(u[j]) * to_f(v[j]);
            }
            return a;
        }
    }
    for (int i = lane; i < n; i += 64) a += to_f(x[i]) * to_f(w[i]);
    return a;
}

// act 0: g' = min(g, limit), u' = clamp(u, +-limit), g' sigmoid(1.702 g') (u' + 1); act 1: silu(g) u
__device__ __forceinline__ float gated_unit(float g, float u, float limit, int act) {
    if (act == 1) return g / (1.0f + expf(-g)) * u;
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * (1.0f / (1.0f + expf(-1.702f * g))) * (u + 1.0f);
}

template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_route_kernel(int32_t *idx_out, float *w_out, const T *h,
                                                                const float *router, const float *bias, int width,
                                                                int experts, int top, int all_scores, float scale) {
    extern __shared__ float lds[];
    float *hf = lds;                // [width]
    float *logit = lds + width;     // [experts]
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < width; i += kMoeThreads) hf[i] = to_f(h[t * width + i]);
    __syncthreads();
    for (int e = wave; e < experts; e += kMoeWaves) {
        const float *wr = router + static_cast<int64_t>(e) * width;
        float a = 0.f;
        for (int i = lane; i < width; i += 64) a += hf[i] * wr[i];
        a = wave_allreduce_sum(a);
        if (lane == 0) logit[e] = a + (bias ? bias[e] : 0.f);
    }
    __syncthreads();
    if (wave != 0) return;
    // all_scores: the weights are scale * softmax over ALL experts (not renormalised over the chosen ones)
    float all_max = -INFINITY, all_den = 0.f;
    if (all_scores) {
        for (int e = lane; e < experts; e += 64) all_max = fmaxf(all_max, logit[e]);
        all_max = wave_allreduce_max(all_max);
        for (int e = lane; e < experts; e += 64) all_den += expf(logit[e] - all_max);
        all_den = wave_allreduce_sum(all_den);
    }
    // top-k by repeated arg-max over the wave (each lane scans experts lane, lane + 64, ...)
    float chosen_max = 0.f, denom = 0.f;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY;
        int besti = 0x7fffffff;
        for (int e = lane; e < experts; e += 64) {
            const float v = logit[e];
            if (v > best) {     // strict: keeps the lowest id among a lane's equals (NaN / taken entries never win)
                best = v;
                besti = e;
            }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const float ob = __shfl_xor(best, m, 64);
            const int oi = __shfl_xor(besti, m, 64);
            if (ob > best || (ob == best && oi < besti)) {
                best = ob;
                besti = oi;
            }
        }
        if (j == 0) chosen_max = all_scores ? all_max : best;
        const float pj = expf(best - chosen_max);
        denom += pj;
        if (lane == 0) {
            idx_out[t * top + j] = besti;
            w_out[t * top + j] = pj;
            logit[besti] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (lane == 0) {
        const float mult = all_scores ? scale / all_den : 1.0f / denom;
        for (int j = 0; j < top; ++j) w_out[t * top + j] *= mult;
    }
}

// Sigmoid scores with group-limited choice. One workgroup per token; the first wave chooses.
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_route_grouped_kernel(int32_t *idx_out, float *w_out, const T *h,
                                                                        const float *router, const float *correction,
                                                                        int width, int experts, int top, int count,
                                                                        int keep) {
    extern __shared__ float lds[];
    float *hf = lds;                    // [width]
    float *score = hf + width;          // [experts] s = sigmoid(logit)
    float *choice = score + experts;    // [experts] s + correction; -inf once taken or outside the kept groups
    float *gscore = choice + experts;   // [count]
    float *gkeep = gscore + count;      // [count] 1 for the groups whose experts may be chosen
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < width; i += kMoeThreads) hf[i] = to_f(h[t * width + i]);
    __syncthreads();
    for (int e = wave; e < experts; e += kMoeWaves) {
        const float *wr = router + static_cast<int64_t>(e) * width;
        float a = 0.f;
        for (int i = lane; i < width; i += 64) a += hf[i] * wr[i];
        a = wave_allreduce_sum(a);
        if (lane == 0) {
            const float sc = 1.0f / (1.0f + expf(-a));
            score[e] = sc;
            choice[e] = sc + (correction ? correction[e] : 0.f);
        }
    }
    __syncthreads();
    if (wave != 0) return;
    // arg-max over an LDS array of n floats for the whole wave (ties: the lowest index; -inf never wins)
    auto argmax = [&](const float *v, int n, float &best, int &besti) {
        best = -INFINITY;
        besti = 0x7fffffff;
        for (int e = lane; e < n; e += 64) {
            if (v[e] > best) {
                best = v[e];
                besti = e;
            }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const float ob = __shfl_xor(best, m, 64);
            const int oi = __shfl_xor(besti, m, 64);
            if (ob > best || (ob == best && oi < besti)) {
                best = ob;
                besti = oi;
            }
        }
    };
    if (count > 1 && keep < count) {
        const int per = experts / count;
        for (int g = lane; g < count; g += 64) {    // a group's score: its two largest choice scores (one, in groups of one)
            float a = -INFINITY, b = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; ++e) {
                const float v = choice[e];
                if (v > a) {
                    b = a;
                    a = v;
                } else if (v > b) {
                    b = v;
                }
            }
            gscore[g] = per > 1 ? a + b : a;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        for (int g = lane; g < count; g += 64) gkeep[g] = 0.f;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        for (int j = 0; j < keep; ++j) {
            float best;
            int besti;
            argmax(gscore, count, best, besti);
            if (lane == 0 && besti < count) {
                gscore[besti] = -INFINITY;      // (taken)
                gkeep[besti] = 1.f;
            }
            __builtin_amdgcn_wave_barrier();
            __threadfence_block();
        }
        for (int e = lane; e < experts; e += 64)
            if (gkeep[e / per] == 0.f) choice[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    float denom = 0.f;
    for (int j = 0; j < top; ++j) {
        float best;
        int besti;
        argmax(choice, experts, best, besti);
        if (besti >= experts) besti = 0;        // (fewer eligible experts than `top`: cannot happen for keep * per >= top)
        const float sc = score[besti];
        denom += sc;
        if (lane == 0) {
            idx_out[t * top + j] = besti;
            w_out[t * top + j] = sc;
            choice[besti] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (lane == 0) {
        const float mult = 1.0f / (denom + 1e-20f);
        for (int j = 0; j < top; ++j) w_out[t * top + j] *= mult;
    }
}

// grid (assignments, ceil(ff / 64)): wave w of the workgroup computes ff rows f0 + w, f0 + w + 4, ...
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_gate_up_kernel(T *y, const T *h, const T *gate_up,
                                                                  const int32_t *expert_idx, int width, int ff, int top,
                                                                  float limit, int act) {
    extern __shared__ float lds[];
    float *hf = lds;    // [width]
    const int64_t a = blockIdx.x;           // assignment = token * top + j
    const int64_t t = a / top;
    const int e = expert_idx[a];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < width; i += kMoeThreads) hf[i] = to_f(h[t * width + i]);
    __syncthreads();
    const T *wg = gate_up + static_cast<int64_t>(e) * 2 * ff * width;
    const T *wu = wg + static_cast<int64_t>(ff) * width;
    const int f0 = blockIdx.y * 64;
    for (int f = f0 + wave; f < min(ff, f0 + 64); f += kMoeWaves) {
        const T *rg = wg + static_cast<int64_t>(f) * width, *ru = wu + static_cast<int64_t>(f) * width;
        float g = lane_dot(hf, rg, width, lane), u = lane_dot(hf, ru, width, lane);
        g = wave_allreduce_sum(g);
        u = wave_allreduce_sum(u);
        if (lane == 0) y[a * ff + f] = to_t<T>(gated_unit(g, u, limit, act));
    }
}

// Experts without a gate: y = relu(W_up h)^2 for every (token, chosen expert); up [experts, ff, width]. Same grid.
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_up_relu2_kernel(T *y, const T *h, const T *up, const int32_t *expert_idx,
                                                                   int width, int ff, int top) {
    extern __shared__ float lds[];
    float *hf = lds;    // [width]
    const int64_t a = blockIdx.x;
    const int64_t t = a / top;
    const int e = expert_idx[a];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < width; i += kMoeThreads) hf[i] = to_f(h[t * width + i]);
    __syncthreads();
    const T *wu = up + static_cast<int64_t>(e) * ff * width;
    const int f0 = blockIdx.y * 64;
    for (int f = f0 + wave; f < min(ff, f0 + 64); f += kMoeWaves) {
        float u = wave_allreduce_sum(lane_dot(hf, wu + static_cast<int64_t>(f) * width, width, lane));
        if (lane == 0) {
            u = fmaxf(u, 0.f);
            y[a * ff + f] = to_t<T>(u * u);
        }
    }
}

// y[r][f] = relu(z[r][f])^2 over rows of z that may be wider than ff (in_stride)
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void relu_sq_kernel(T *y, const T *z, int64_t total, int ff, int64_t in_stride) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kMoeThreads + threadIdx.x;
    if (i >= total) return;
    const int64_t r = i / ff;
    const float v = fmaxf(to_f(z[r * in_stride + (i - r * ff)]), 0.f);
    y[i] = to_t<T>(v * v);
}

// the same for 16-bit rows of a multiple of 8 elements on 16-byte boundaries: 8 elements (16 bytes) per lane
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void relu_sq_wide_kernel(T *y, const T *z, int64_t total8, int ff8,
                                                                   int64_t in_stride) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kMoeThreads + threadIdx.x;
    if (i >= total8) return;
    const int64_t r = i / ff8;
    const int c = static_cast<int>(i - r * ff8) * 8;
    const vec8_t<T> x = load8(z + r * in_stride + c);
    vec8_t<T> o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v = fmaxf(to_f(x[j]), 0.f);
        o[j] = to_t<T>(v * v);
    }
    store8(y + r * static_cast<int64_t>(ff8) * 8 + c, o);
}

// grid (tokens, ceil(width / 64)): wave w computes output columns c0 + w, c0 + w + 4, ...
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_down_combine_kernel(T *out, const T *y, const T *down,
                                                                       const int32_t *expert_idx, const float *expert_w,
                                                                       int width, int ff, int top) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c0 = blockIdx.y * 64;
    for (int c = c0 + wave; c < min(width, c0 + 64); c += kMoeWaves) {
        float total = 0.f;
        for (int j = 0; j < top; ++j) {
            const int e = expert_idx[t * top + j];
            const T *wr = down + (static_cast<int64_t>(e) * width + c) * ff;
            const T *yr = y + (t * top + j) * ff;
            float a = wave_allreduce_sum(lane_dot2(yr, wr, ff, lane));
            total += expert_w[t * top + j] * a;
        }
        if (lane == 0) out[t * width + c] = to_t<T>(total);
    }
}


// ---- expert-stationary products for decode-sized steps -----------------------------------------------------------------------
// out[a][n] = sum_k W[e][n][k] X[xrow(a)][k] for the assignments a of expert e, on the matrix core. A workgroup owns (expert,
// 64 outputs n), a wave 16 of them: per 16-wide k step it loads its weight fragment ONCE (A operand: row n, 8 bytes per lane)
// and multiplies it with the input fragments of up to four tiles of 16 assignments (B operand: the assignment's input row,
// read through the caches — the rows of a decode step are few and stay resident). An expert's weights are thus streamed once
// per step however many tokens chose it (the per-assignment kernels above stream them once per token). GLU: n indexes ff,
// the gate row n and the up row ff + n share the input fragments and meet in the clamped gated unit; X rows are tokens
// (a / top). Otherwise (down projection) X rows are assignments and the output is the plain product, rounded to T.
constexpr int kEsRows = 64;         // outputs per workgroup at most (16 per wave; fewer waves when the grid would be small)
constexpr int kEsTiles = 4;         // tiles of 16 assignments per pass over the weights
constexpr int kEsMaxAssign = 1024;  // assignments per step (the sorted library path serves larger steps)

template <typename T, int MODE>
__global__ __launch_bounds__(kMoeThreads, 2) void moe_expert_stationary_kernel(T *out, const T *x, const T *w,
                                                                            const int32_t *expert_idx, int assignments,
                                                                            int K, int N, int top, float limit, int ksplit) {
    // ksplit = 1: every wave of the workgroup owns 16 outputs and the whole reduction. ksplit = waves of the workgroup: all
    // waves own the SAME 16 outputs and a quarter (half) of the reduction each; their accumulators meet in LDS and wave 0
    // finishes (short reductions and few outputs would otherwise leave most of the chip idle in a decode step).
    // MODE 0: plain product, X rows are assignments; 1: clamped gated unit, X rows are tokens; 2: squared ReLU of the plain
    // product (experts without a gate), X rows are tokens
    constexpr bool GLU = MODE == 1 || MODE == 3;      // (3: the plain gated unit silu(g) u)
    __shared__ int mine[kEsMaxAssign];
    __shared__ int count;
    __shared__ float red[3][2 * kEsTiles][256];
    const int e = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const int li = lane & 15, lq = lane >> 4;
    if (threadIdx.x == 0) count = 0;
    __syncthreads();
    for (int a = threadIdx.x; a < assignments; a += blockDim.x)
        if (expert_idx[a] == e) mine[atomicAdd(&count, 1)] = a;
    __syncthreads();
    const int m = count;
    const int n0 = ksplit > 1 ? blockIdx.y * 16 : (blockIdx.y * nwaves + wave) * 16;
    if (m == 0 || (ksplit == 1 && n0 >= N)) return;
    const int kper = K / ksplit;                       // (ksplit > 1: a multiple of 32, checked on the host)
    const int kbeg = ksplit > 1 ? wave * kper : 0, kend = kbeg + kper;
    const int nrow = min(n0 + li, N - 1);       // (rows past N compute a duplicate that is never stored)
    // this lane's share of a 32-wide reduction step: elements 8 lq .. 8 lq + 7 (one 16-byte load), fed to the matrix core as
    // two 4-element halves — the same split on both operands, so the order inside a step does not matter
    const T *wg = w + (static_cast<int64_t>(e) * (GLU ? 2 : 1) * N + nrow) * K + 8 * lq;
    const T *wu = wg + static_cast<int64_t>(N) * K;
    const bool wide = (kper & 31) == 0 && ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15) == 0 && (K & 7) == 0;
    for (int pass = 0; pass < m; pass += 16 * kEsTiles) {
        const int ntile = min(kEsTiles, (m - pass + 15) / 16);
        int arow[kEsTiles];
        const T *xp[kEsTiles];
#pragma unroll
        for (int t = 0; t < kEsTiles; ++t) {
            const int i = pass + t * 16 + li;
            const int a = i < m ? mine[i] : -1;
            arow[t] = a;
            xp[t] = x + static_cast<int64_t>(a < 0 ? 0 : (MODE != 0 ? a / top : a)) * K + 8 * lq;
        }
        float4_t accg[kEsTiles], accu[kEsTiles];
#pragma unroll
        for (int t = 0; t < kEsTiles; ++t) accg[t] = accu[t] = float4_t{0.f, 0.f, 0.f, 0.f};
        if (wide) {
#pragma unroll 2
            for (int k0 = kbeg; k0 < kend; k0 += 32) {
                const vec8_t<T> ag = load8(wg + k0);
                vec8_t<T> au = vec8_t<T>{};
                if constexpr (GLU) au = load8(wu + k0);
#pragma unroll
                for (int t = 0; t < kEsTiles; ++t) {
                    if (t < ntile) {
                        vec8_t<T> b = vec8_t<T>{};
                        if (arow[t] >= 0) b = load8(xp[t] + k0);
                        const vec4_t<T> b0 = {b[0], b[1], b[2], b[3]}, b1 = {b[4], b[5], b[6], b[7]};
                        accg[t] = mfma16(vec4_t<T>{ag[0], ag[1], ag[2], ag[3]}, b0, accg[t]);
                        accg[t] = mfma16(vec4_t<T>{ag[4], ag[5], ag[6], ag[7]}, b1, accg[t]);
                        if constexpr (GLU) {
                            accu[t] = mfma16(vec4_t<T>{au[0], au[1], au[2], au[3]}, b0, accu[t]);
                            accu[t] = mfma16(vec4_t<T>{au[4], au[5], au[6], au[7]}, b1, accu[t]);
                        }
                    }
                }
            }
        } else {
            // 16-wide steps, 8-byte fragments (this lane: elements 4 lq .. 4 lq + 3 of the step)
            const T *wg4 = wg - 4 * lq, *wu4 = wu - 4 * lq;
#pragma unroll 4
            for (int k0 = kbeg; k0 < kend; k0 += 16) {
                vec4_t<T> ag, au;
                load4(ag, wg4 + k0);
                if constexpr (GLU) load4(au, wu4 + k0);
#pragma unroll
                for (int t = 0; t < kEsTiles; ++t) {
                    if (t < ntile) {
                        vec4_t<T> b = vec4_t<T>{};
                        if (arow[t] >= 0) load4(b, xp[t] - 4 * lq + k0);
                        accg[t] = mfma16(ag, b, accg[t]);
                        if constexpr (GLU) accu[t] = mfma16(au, b, accu[t]);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < kEsTiles; ++t) {
            mfma_results_tie(accg[t]);
            mfma_results_ready<4>(accu[t]);
        }
        if (ksplit > 1) {       // (workgroup-uniform) sum the waves' partial accumulators in wave 0
            __syncthreads();    // (the previous pass's partials have been read)
            if (wave > 0) {
#pragma unroll
                for (int t = 0; t < kEsTiles; ++t) {
                    if (t < ntile) {
                        *reinterpret_cast<float4_t *>(&red[wave - 1][2 * t][lane * 4]) = accg[t];
                        if constexpr (GLU) *reinterpret_cast<float4_t *>(&red[wave - 1][2 * t + 1][lane * 4]) = accu[t];
                    }
                }
            }
            __syncthreads();
            if (wave > 0) continue;
            for (int o = 0; o + 1 < nwaves; ++o) {
#pragma unroll
                for (int t = 0; t < kEsTiles; ++t) {
                    if (t < ntile) {
                        accg[t] += *reinterpret_cast<const float4_t *>(&red[o][2 * t][lane * 4]);
                        if constexpr (GLU) accu[t] += *reinterpret_cast<const float4_t *>(&red[o][2 * t + 1][lane * 4]);
                    }
                }
            }
        }
        // accumulator r of lane (li, lq): output row n0 + 4 lq + r of the assignment in column li
#pragma unroll
        for (int t = 0; t < kEsTiles; ++t) {
            if (t < ntile && arow[t] >= 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + 4 * lq + r;
                    if (n < N) {
                        float v = accg[t][r];
                        if constexpr (GLU) v = gated_unit(v, accu[t][r], limit, MODE == 3 ? 1 : 0);
                        if constexpr (MODE == 2) {
                            v = fmaxf(v, 0.f);
                            v *= v;
                        }
                        out[static_cast<int64_t>(arow[t]) * N + n] = to_t<T>(v);
                    }
                }
            }
        }
    }
}

// y[r][f] = act(gu[r][f], gu[r][ff + f]) for rows of [gate | up] products that came from a library GEMM
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void glu_clamp_kernel(T *y, const T *gu, int64_t total, int ff, float limit,
                                                                int act) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kMoeThreads + threadIdx.x;
    if (i >= total) return;
    const int64_t r = i / ff;
    const int f = static_cast<int>(i - r * ff);
    y[i] = to_t<T>(gated_unit(to_f(gu[r * 2 * ff + f]), to_f(gu[r * 2 * ff + ff + f]), limit, act));
}

// out[t] = sum_j w[t][j] * rows[where[t * top + j]]  (fp32 sum in the order j = 0, 1, ...)
template <typename T>
__global__ __launch_bounds__(kMoeThreads) void moe_combine_kernel(T *out, const T *rows, const int64_t *where,
                                                                  const float *w, int width, int top) {
    const int64_t t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += kMoeThreads) {
        float a = 0.f;
        for (int j = 0; j < top; ++j) a += w[t * top + j] * to_f(rows[where[t * top + j] * width + c]);
        out[t * width + c] = to_t<T>(a);
    }
}

} // namespace swl

/* 1 when swl_moe_expert_stationary serves the shape: 16-bit, both reduction lengths multiples of 16, at most 1024
 * assignments. */
extern "C" int swl_moe_expert_stationary_supported(int64_t num_tokens, int32_t width, int32_t ff, int32_t top, int32_t dtype) {
    if (dtype != SWL_F16 && dtype != SWL_BF16) return 0;
    if (width <= 0 || ff <= 0 || (width & 15) || (ff & 15)) return 0;
    return num_tokens * top <= swl::kEsMaxAssign;
}

extern "C" int swl_moe_expert_stationary(void *out, const void *x, const void *w, const int32_t *expert_idx,
                                         int64_t num_tokens, int32_t experts, int32_t width, int32_t ff, int32_t top,
                                         int32_t glu, float limit, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || experts <= 0 || top <= 0) return SWL_ERR_BAD_ARG;
    if (!swl_moe_expert_stationary_supported(num_tokens, width, ff, top, dtype)) return SWL_ERR_UNSUPPORTED;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !x || !w || !expert_idx || !swl::aligned16(x) || !swl::aligned16(w)) return SWL_ERR_BAD_ARG;
    const int K = glu ? width : ff, N = glu ? ff : width;
    const int assignments = static_cast<int>(num_tokens * top);
    const size_t lds = 0;
    // Four waves per workgroup. With plenty of outputs each wave owns 16 of them; when that would launch under ~2048 waves
    // (a decode step must fill 256 CUs x 4 SIMDs, with latency to hide) the four waves share 16 outputs and split the reduction.
    const int nw = 4;
    const int64_t tiles16 = (N + 15) / 16;
    const int ksplit = (experts * tiles16 < 2048 && K % (32 * nw) == 0) ? nw : 1;
    const dim3 grid(static_cast<unsigned>(experts),
                    static_cast<unsigned>(ksplit > 1 ? tiles16 : (N + 16 * nw - 1) / (16 * nw)));
    if (grid.y > 65535) return SWL_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    SWL_DISPATCH_DTYPE(dtype, T, {
        if (glu == 1)
            hipLaunchKernelGGL((swl::moe_expert_stationary_kernel<T, 1>), grid, dim3(64 * nw), lds, s,
                               static_cast<T *>(out), static_cast<const T *>(x), static_cast<const T *>(w), expert_idx,
                               assignments, K, N, top, limit, ksplit);
        else if (glu == 2)
            hipLaunchKernelGGL((swl::moe_expert_stationary_kernel<T, 2>), grid, dim3(64 * nw), lds, s,
                               static_cast<T *>(out), static_cast<const T *>(x), static_cast<const T *>(w), expert_idx,
                               assignments, K, N, top, limit, ksplit);
        else if (glu == 3)
            hipLaunchKernelGGL((swl::moe_expert_stationary_kernel<T, 3>), grid, dim3(64 * nw), lds, s,
                               static_cast<T *>(out), static_cast<const T *>(x), static_cast<const T *>(w), expert_idx,
                               assignments, K, N, top, limit, ksplit);
        else
            hipLaunchKernelGGL((swl::moe_expert_stationary_kernel<T, 0>), grid, dim3(64 * nw), lds, s,
                               static_cast<T *>(out), static_cast<const T *>(x), static_cast<const T *>(w), expert_idx,
                               assignments, K, N, top, limit, ksplit);
    });
    return swl::check_launch();
}

extern "C" int swl_glu_clamp(void *y, const void *gate_up, int64_t num_rows, int32_t ff, float limit, int32_t act,
                             int32_t dtype, swl_stream_t stream) {
    if (num_rows < 0 || ff <= 0 || act < 0 || act > 1) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!y || !gate_up) return SWL_ERR_BAD_ARG;
    const int64_t total = num_rows * ff;
    const int64_t blocks = (total + swl::kMoeThreads - 1) / swl::kMoeThreads;
    if (blocks > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::glu_clamp_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(swl::kMoeThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(gate_up), total,
                           ff, limit, act);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_combine(void *out, const void *rows, const int64_t *where, const float *expert_w,
                               int64_t num_tokens, int32_t width, int32_t top, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || top <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !rows || !where || !expert_w) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_combine_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kMoeThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(out), static_cast<const T *>(rows), where,
                           expert_w, width, top);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_route(int32_t *idx_out, float *w_out, const void *h, const float *router, const float *bias,
                             int64_t num_tokens, int32_t width, int32_t experts, int32_t top, int32_t dtype,
                             swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || experts <= 0 || top <= 0 || top > experts) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!idx_out || !w_out || !h || !router || !bias) return SWL_ERR_BAD_ARG;
    const size_t lds = (static_cast<size_t>(width) + experts) * 4;
    if (num_tokens > 0x7fffffffLL || lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_route_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kMoeThreads),
                           lds, static_cast<hipStream_t>(stream), idx_out, w_out, static_cast<const T *>(h), router, bias,
                           width, experts, top, 0, 1.0f);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_route_scores(int32_t *idx_out, float *w_out, const void *h, const float *router, const float *bias,
                                    int64_t num_tokens, int32_t width, int32_t experts, int32_t top, float scale,
                                    int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || experts <= 0 || top <= 0 || top > experts) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!idx_out || !w_out || !h || !router) return SWL_ERR_BAD_ARG;
    const size_t lds = (static_cast<size_t>(width) + experts) * 4;
    if (num_tokens > 0x7fffffffLL || lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_route_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kMoeThreads),
                           lds, static_cast<hipStream_t>(stream), idx_out, w_out, static_cast<const T *>(h), router, bias,
                           width, experts, top, 1, scale);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_gate_up(void *y, const void *h, const void *gate_up, const int32_t *expert_idx,
                               int64_t num_tokens, int32_t width, int32_t ff, int32_t top, float limit, int32_t act,
                               int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || ff <= 0 || top <= 0 || act < 0 || act > 1) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!y || !h || !gate_up || !expert_idx) return SWL_ERR_BAD_ARG;
    const size_t lds = static_cast<size_t>(width) * 4;
    const int64_t assignments = num_tokens * top;
    if (assignments > 0x7fffffffLL || lds > 64 * 1024 || (ff + 63) / 64 > 65535) return SWL_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(assignments), static_cast<unsigned>((ff + 63) / 64));
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_gate_up_kernel<T>), grid, dim3(swl::kMoeThreads), lds,
                           static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(h),
                           static_cast<const T *>(gate_up), expert_idx, width, ff, top, limit, act);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_down_combine(void *out, const void *y, const void *down, const int32_t *expert_idx,
                                    const float *expert_w, int64_t num_tokens, int32_t width, int32_t ff, int32_t top,
                                    int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || ff <= 0 || top <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !y || !down || !expert_idx || !expert_w) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL || (width + 63) / 64 > 65535) return SWL_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(num_tokens), static_cast<unsigned>((width + 63) / 64));
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_down_combine_kernel<T>), grid, dim3(swl::kMoeThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(out), static_cast<const T *>(y),
                           static_cast<const T *>(down), expert_idx, expert_w, width, ff, top);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_up_relu2(void *y, const void *h, const void *up, const int32_t *expert_idx, int64_t num_tokens,
                                int32_t width, int32_t ff, int32_t top, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || ff <= 0 || top <= 0) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!y || !h || !up || !expert_idx) return SWL_ERR_BAD_ARG;
    const size_t lds = static_cast<size_t>(width) * 4;
    const int64_t assignments = num_tokens * top;
    if (assignments > 0x7fffffffLL || lds > 64 * 1024 || (ff + 63) / 64 > 65535) return SWL_ERR_UNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(assignments), static_cast<unsigned>((ff + 63) / 64));
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_up_relu2_kernel<T>), grid, dim3(swl::kMoeThreads), lds,
                           static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(h),
                           static_cast<const T *>(up), expert_idx, width, ff, top);
    });
    return swl::check_launch();
}

extern "C" int swl_relu_sq(void *y, const void *z, int64_t num_rows, int32_t ff, int64_t in_stride, int32_t dtype,
                           swl_stream_t stream) {
    if (num_rows < 0 || ff <= 0 || in_stride < ff) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!y || !z) return SWL_ERR_BAD_ARG;
    const int64_t total = num_rows * ff;
    if (dtype != SWL_F32 && ff % 8 == 0 && in_stride % 8 == 0 && swl::aligned16(y) && swl::aligned16(z)) {
        const int64_t total8 = total / 8, blocks8 = (total8 + swl::kMoeThreads - 1) / swl::kMoeThreads;
        SWL_DISPATCH_DTYPE(dtype, T, {
            hipLaunchKernelGGL((swl::relu_sq_wide_kernel<T>), dim3(static_cast<unsigned>(blocks8)), dim3(swl::kMoeThreads),
                               0, static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(z), total8,
                               ff / 8, in_stride);
        });
        return swl::check_launch();
    }
    const int64_t blocks = (total + swl::kMoeThreads - 1) / swl::kMoeThreads;
    if (blocks > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::relu_sq_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(swl::kMoeThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(y), static_cast<const T *>(z), total, ff,
                           in_stride);
    });
    return swl::check_launch();
}

extern "C" int swl_moe_route_grouped(int32_t *idx_out, float *w_out, const void *h, const float *router,
                                     const float *correction, int64_t num_tokens, int32_t width, int32_t experts, int32_t top,
                                     int32_t group_count, int32_t group_keep, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || width <= 0 || experts <= 0 || top <= 0 || top > experts) return SWL_ERR_BAD_ARG;
    if (group_count < 1 || group_keep < 1 || group_keep > group_count || experts % group_count) return SWL_ERR_BAD_ARG;
    if (static_cast<int64_t>(group_keep) * (experts / group_count) < top) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!idx_out || !w_out || !h || !router) return SWL_ERR_BAD_ARG;
    const size_t lds = (static_cast<size_t>(width) + 2 * experts + 2 * group_count) * 4;
    if (num_tokens > 0x7fffffffLL || lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::moe_route_grouped_kernel<T>), dim3(static_cast<unsigned>(num_tokens)),
                           dim3(swl::kMoeThreads), lds, static_cast<hipStream_t>(stream), idx_out, w_out,
                           static_cast<const T *>(h), router, correction, width, experts, top, group_count, group_keep);
    });
    return swl::check_launch();
}
