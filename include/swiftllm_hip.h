/*
 * swiftllm_hip.h — C ABI of libswiftllm_hip.so
 *
 * The drop-in boundary for swiftLLM's data plane (LlamaModel.forward) on MI355X / gfx950.
 * Every entry point replaces one operator of the reference's Python/Triton operator layer
 * (the modules under swiftllm/worker/kernels) or its one native function (csrc/src/block_swapping.cpp).
 * The reference file:line each entry replaces is cited above its declaration.
 *
 * Conventions
 *   - plain `extern "C"`, device pointers as void*, sizes as int32/int64, no torch types;
 *   - `dtype`: SWL_F16 (the reference's hard-coded precision) or SWL_BF16 (headline precision);
 *   - `stream` is a hipStream_t passed as void*; NOTHING is ever launched on the null stream
 *     unless the caller passes NULL explicitly. No allocation, no synchronisation, no global
 *     state: every call is re-entrant and may be captured into a hipGraph;
 *   - returns SWL_OK (0) or a negative SWL_ERR_* code; the Python shim maps non-zero to
 *     RuntimeError (the reference surfaces failures as AssertionError/RuntimeError);
 *   - zero-size batches are legal everywhere and return SWL_OK without launching
 *     (the reference's idle engine spins on empty forwards: server/engine.py:115-171);
 *   - all offsets into the KV pools are 64-bit (288 GB pools exceed 2^31 elements).
 *
 * KV pool layout (reference model.py:138-148): [num_blocks, num_layers, num_kv_heads, block_size, head_dim],
 * contiguous, one pool for K and one for V.
 */
#ifndef SWIFTLLM_HIP_H
#define SWIFTLLM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SWL_ABI_VERSION 1

#define SWL_F16 0
#define SWL_BF16 1
#define SWL_F32 2 /* only the operators that say so accept it */

#define SWL_OK 0
#define SWL_ERR_BAD_ARG (-1)     /* null pointer, negative size, misaligned pointer/stride          */
#define SWL_ERR_UNSUPPORTED (-2) /* shape outside what the kernels are specialised for              */
#define SWL_ERR_LAUNCH (-3)      /* hipGetLastError() != hipSuccess after the launch                */
#define SWL_ERR_RUNTIME (-4)     /* a HIP runtime call (memcpy) failed                              */

typedef void *swl_stream_t; /* hipStream_t */

int swl_abi_version(void);
/* Human-readable name for an SWL_ERR_* code. */
const char *swl_strerror(int code);

/* ---- RMSNorm ------------------------------------------------------------------------------
 * reference: rmsnorm.py:5-37 (_fwd_rmsnorm / rmsnorm_inplace)
 * x[T, hidden] <- x * rsqrt(mean(x^2) + eps) * w      (fp32 math, one rounding to dtype)
 * hidden % 8 == 0, hidden <= 16384; rows contiguous (row stride == hidden). */
int swl_rmsnorm(void *x, const void *w, float eps, int64_t num_tokens, int32_t hidden,
                int32_t dtype, swl_stream_t stream);

/* reference: rmsnorm.py:39-89 (_fwd_fused_add_rmsnorm / fused_add_rmsnorm_inplace)
 * residual <- x + residual (rounded to dtype and stored); x <- rmsnorm(residual) * w. */
int swl_fused_add_rmsnorm(void *x, void *residual, const void *w, float eps, int64_t num_tokens,
                          int32_t hidden, int32_t dtype, swl_stream_t stream);

/* ---- Rotary embedding ---------------------------------------------------------------------
 * reference: rotary_emb.py:7-58 (_fwd_rotary_embedding / rotary_embedding_inplace)
 * rotate-half RoPE in place on q[T, H, D] and k[T, KVH, D]; every multiply/add is rounded to
 * dtype as in the reference. cos/sin are [rows, D/2] in dtype. If pos_idx != NULL the row used
 * for token t is pos_idx[t] (tables = the model's full rope cache, model.py:224-225); if NULL
 * the row is t (tables already gathered: model.py:350-351).
 * q_tok_stride / k_tok_stride: elements between consecutive tokens (>= H*D / KVH*D; lets q,k be
 * column slices of one fused qkv GEMM output). D in {32, 64, 128, 256}. */
int swl_rotary(void *q, void *k, const void *cos_table, const void *sin_table,
               const int32_t *pos_idx, int64_t num_tokens, int32_t num_q_heads,
               int32_t num_kv_heads, int32_t head_dim, int64_t q_tok_stride, int64_t k_tok_stride,
               int32_t dtype, swl_stream_t stream);

/* ---- KV-cache store -----------------------------------------------------------------------
 * reference: kvcache_mgmt.py:10-48 (_fwd_kvcache_mgmt_prefill_kernel), launcher :81-109
 * For prefill seq s (id seq_ids[s], tokens [start_locs[s], +seq_lens[s]) of k/v), logical block j:
 * pool[block_table[seq_id, j], layer, kvh, t % bs, :] = k[start + j*bs + t, kvh, :]   (bit-exact). */
int swl_store_kv_prefill(void *k_cache, void *v_cache, const void *k, const void *v,
                         const int32_t *block_table, const int32_t *seq_ids,
                         const int32_t *start_locs, const int32_t *seq_lens,
                         int32_t num_prefill_seqs, int32_t max_prefill_len, int32_t cur_layer,
                         int32_t num_layers, int32_t num_kv_heads, int32_t block_size,
                         int32_t head_dim, int32_t max_blocks_per_seq, int64_t k_tok_stride,
                         int64_t v_tok_stride, int32_t dtype, swl_stream_t stream);

/* Prefill fusion: swl_rotary on the prefill tokens' q and k (rotary_emb.py:7-42) + swl_store_kv_prefill
 * (kvcache_mgmt.py:10-48) in ONE pass over k — transformer_layer.py:62-77 for the prefill sequences of a forward. q and k
 * are rotated in place (k is also what the prefill attention reads), the rotated k and v go into the pools. pos_idx: rope
 * table row per token (NULL: the token's index inside its sequence). Bit-identical to the two calls it replaces. */
int swl_rotary_store_kv_prefill(void *q, void *k, const void *v, const void *cos_table, const void *sin_table,
                                const int32_t *pos_idx, void *k_cache, void *v_cache, const int32_t *block_table,
                                const int32_t *seq_ids, const int32_t *start_locs, const int32_t *seq_lens,
                                int32_t num_prefill_seqs, int32_t max_prefill_len, int32_t cur_layer, int32_t num_layers,
                                int32_t num_q_heads, int32_t num_kv_heads, int32_t block_size, int32_t head_dim,
                                int32_t max_blocks_per_seq, int64_t q_tok_stride, int64_t k_tok_stride,
                                int64_t v_tok_stride, int32_t dtype, swl_stream_t stream);
/* reference: kvcache_mgmt.py:50-79 (_fwd_kvcache_mgmt_decoding_kernel), launcher :111-122
 * For decoding seq i (length len_i INCLUDING the new token): token i of k/v goes to slot
 * (block_table[seq_id, (len-1)/bs], (len-1)%bs). */
int swl_store_kv_decode(void *k_cache, void *v_cache, const void *k, const void *v,
                        const int32_t *block_table, const int32_t *seq_ids,
                        const int32_t *seq_lens, int32_t num_decoding_seqs, int32_t cur_layer,
                        int32_t num_layers, int32_t num_kv_heads, int32_t block_size,
                        int32_t head_dim, int32_t max_blocks_per_seq, int64_t k_tok_stride,
                        int64_t v_tok_stride, int32_t dtype, swl_stream_t stream);

/* ---- SiLU-gate ----------------------------------------------------------------------------
 * reference: silu_and_mul.py:5-34 (_fwd_silu_and_mul / silu_and_mul_inplace)
 * x[T, 2*I]: x[:, :I] <- x[:, :I] * round(silu_fp32(x[:, I:]))   (up = first half, gate = second,
 * weight.py:133).  I % 8 == 0 (the reference needs I % 256 == 0). */
int swl_silu_mul(void *x, int64_t num_tokens, int32_t ffn_inter_dim, int32_t dtype,
                 swl_stream_t stream);

/* Decode attention fed directly by the split-K slabs of the fused qkv projection (swl_gemm_skinny_partial,
 * k_splits >= 1): the rotary embedding and the KV-cache store of the new token (reference rotary_emb.py:7-42 +
 * kvcache_mgmt.py:50-79, separate launches at transformer_layer.py:62-77) run in the attention kernel's
 * prologue; results are bit-identical to swl_splitk_rotary_store_kv_decode + swl_paged_attn_decode.
 * qkv_slabs: [k_splits][Bd][(H + 2*KVH) * D] fp32. Other arguments as swl_paged_attn_decode. */
int swl_paged_attn_decode_qkv(void *o, const float *qkv_slabs, int32_t k_splits, const void *cos_table,
                              const void *sin_table, const int32_t *pos_idx, void *k_cache, void *v_cache,
                              const int32_t *block_table, const int32_t *seq_ids, const int32_t *seq_lens,
                              void *scratch, float softmax_scale, int32_t num_decoding_seqs,
                              int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t num_layers,
                              int32_t block_size, int32_t cur_layer, int32_t max_blocks_per_seq,
                              int32_t seq_block_size, int32_t num_seq_blocks, int64_t o_tok_stride,
                              int32_t dtype, swl_stream_t stream);

/* ---- Greedy sampling --------------------------------------------------------------------------
 * reference: post_layer.py:40 (`torch.argmax(logits, dim=1)`)
 * out[r] = argmax_j x[r, j] (int64), ties -> lowest j, NaNs never selected. n % 8 == 0.
 * scratch: swl_argmax_scratch_bytes(num_rows) bytes, 16-byte aligned. */
size_t swl_argmax_scratch_bytes(int64_t num_rows);
int swl_argmax(int64_t *out, const void *x, void *scratch, size_t scratch_bytes, int64_t num_rows, int32_t n,
               int64_t row_stride, int32_t dtype, swl_stream_t stream);

/* ---- Paged attention, decode (flash-decoding, "paged attention v2") --------------------------
 * reference: paged_attn.py:9-108 (phase 1), :111-149 (phase 2), launcher :152-222
 * q[Bd, H, D] (token stride q_tok_stride), o[Bd, H, D] (token stride o_tok_stride).
 * Phase 1 writes per (seq, q-head, seq-block) a normalised partial mid_o (fp32) and the base-2
 * log-sum-exp mid_lse (fp32), phase 2 merges them; with num_seq_blocks == 1 phase 1 writes o
 * directly. Scratch: mid_o [Bd, H, num_seq_blocks, D] fp32 followed by mid_lse [Bd, H, num_seq_blocks]
 * fp32 — the same shapes the reference allocates at paged_attn.py:170-180.
 * One workgroup serves ALL G = H/KVH q-heads of a kv-head, so every KV byte is fetched once.
 * seq_block_size % block_size == 0; block_size == 16; D in {32, 64, 128}; G in {1, 2, 4, 8}. */
size_t swl_paged_attn_scratch_bytes(int32_t num_decoding_seqs, int32_t num_q_heads,
                                    int32_t head_dim, int32_t num_seq_blocks);

int swl_paged_attn_decode(void *o, const void *q, const void *k_cache, const void *v_cache,
                          const int32_t *block_table, const int32_t *seq_ids,
                          const int32_t *seq_lens, void *scratch, float softmax_scale,
                          int32_t num_decoding_seqs, int32_t num_q_heads, int32_t num_kv_heads,
                          int32_t head_dim, int32_t num_layers, int32_t block_size,
                          int32_t cur_layer, int32_t max_blocks_per_seq, int32_t seq_block_size,
                          int32_t num_seq_blocks, int64_t q_tok_stride, int64_t o_tok_stride,
                          int32_t dtype, swl_stream_t stream);

/* Phase 1 / phase 2 separately (parity tests compare mid_o / mid_lse with the reference's). */
int swl_paged_attn_phase1(void *o_direct, const void *q, const void *k_cache, const void *v_cache,
                          const int32_t *block_table, const int32_t *seq_ids,
                          const int32_t *seq_lens, float *mid_o, float *mid_lse,
                          float softmax_scale, int32_t num_decoding_seqs, int32_t num_q_heads,
                          int32_t num_kv_heads, int32_t head_dim, int32_t num_layers,
                          int32_t block_size, int32_t cur_layer, int32_t max_blocks_per_seq,
                          int32_t seq_block_size, int32_t num_seq_blocks, int64_t q_tok_stride,
                          int64_t o_tok_stride, int32_t dtype, swl_stream_t stream);
int swl_paged_attn_phase2(void *o, const float *mid_o, const float *mid_lse,
                          const int32_t *seq_lens, int32_t num_decoding_seqs, int32_t num_q_heads,
                          int32_t head_dim, int32_t seq_block_size, int32_t num_seq_blocks,
                          int64_t o_tok_stride, int32_t dtype, swl_stream_t stream);

/* ---- Prefill attention (varlen causal flash attention, GQA) -------------------------------------
 * reference: the call at transformer_layer.py:83-96 (vllm_flash_attn.flash_attn_varlen_func) and its
 * in-repo equivalent prefill_attn.py:9-139 (_fwd_prefill_attention / prefill_attention).
 * q[P, H, D], k/v[P, KVH, D] are the FRESH projections (the paged pool is not read), cu_seqlens is
 * prefill_seq_start_locs_with_end (int32 [Bp+1]); o[P, H, D]. MFMA 32x32x16, fp32 softmax.
 * D in {32, 64, 128}; all four tensors 16-byte aligned with token strides that are multiples of 8 elements. */
int swl_prefill_attn_varlen(void *o, const void *q, const void *k, const void *v,
                            const int32_t *cu_seqlens, int32_t num_prefill_seqs,
                            int32_t max_prefill_len, int32_t num_q_heads, int32_t num_kv_heads,
                            int32_t head_dim, float softmax_scale, int64_t q_tok_stride,
                            int64_t k_tok_stride, int64_t v_tok_stride, int64_t o_tok_stride,
                            int32_t dtype, swl_stream_t stream);

/* ---- Block-table maintenance ------------------------------------------------------------------
 * reference: block_mgmt.py:5-46 (set), :49-80 (unset), :83-127 (gather + unset)
 * block_table int32 [max_seqs, max_blocks_per_seq]; num_seq_allocated_blocks int32 [max_seqs];
 * is_block_free uint8(bool) [num_blocks].
 * set: for batch entry i (seq s): block_table[s, n_s : n_s + need_i] = candidates[off_i : off_i + need_i],
 *      n_s += need_i, where off = exclusive cumsum(block_needed) (passed in by the caller).
 *      If is_block_free != NULL the candidates are also marked used (is_block_free[c] = 0), which
 *      fuses the reference's separate scatter at block_manager.py:52. */
int swl_block_table_set(int32_t *num_seq_allocated_blocks, int32_t *block_table,
                        const int32_t *candidate_blocks, const int32_t *seq_ids,
                        const int32_t *block_needed, const int32_t *block_needed_excl_cumsum,
                        uint8_t *is_block_free, int32_t batch_size, int32_t max_blocks_per_seq,
                        swl_stream_t stream);
/* unset: is_block_free[block_table[s, 0:n_s]] = 1; n_s = 0. */
int swl_block_table_unset(int32_t *num_seq_allocated_blocks, const int32_t *block_table,
                          const int32_t *seq_ids, uint8_t *is_block_free, int32_t batch_size,
                          int32_t max_blocks_per_seq, swl_stream_t stream);
/* gather: out[off_i : off_i + n_s] = block_table[s, 0:n_s]; then unset. */
int swl_block_table_gather(int32_t *num_seq_allocated_blocks, const int32_t *block_table,
                           const int32_t *seq_ids, uint8_t *is_block_free,
                           const int32_t *out_excl_cumsum, int32_t *gathered_block_ids,
                           int32_t batch_size, int32_t max_blocks_per_seq, swl_stream_t stream);

/* ---- Block swapping (host code) ---------------------------------------------------------------
 * reference: csrc/src/block_swapping.cpp:22-85 (swap_blocks), binding csrc/src/entrypoints.cpp:5-7
 * Copies block src_ids[i] -> dst_ids[i] for K and V between the GPU pools and the host swap pools,
 * run-length-coalescing consecutive (src, dst) pairs into one hipMemcpyAsync each, on `stream`.
 * src_ids/dst_ids are HOST arrays. block_bytes = bytes of one block in one pool. */
int swl_swap_blocks(const int64_t *src_ids, const int64_t *dst_ids, int64_t num_blocks_to_swap,
                    int32_t is_swap_in, void *k_cache, void *v_cache, void *k_swap, void *v_swap,
                    int64_t block_bytes, swl_stream_t stream);

/* ---- Fused hot-path helpers (no reference twin; result-identical compositions) ------------------
 * Decode-only: rotary on q,k followed by the decode KV store of the rotated k and of v, in one launch
 * (= swl_rotary(pos_idx) + swl_store_kv_decode). */
int swl_rotary_store_kv_decode(void *q, void *k, const void *v, const void *cos_table,
                               const void *sin_table, const int32_t *pos_idx, void *k_cache,
                               void *v_cache, const int32_t *block_table, const int32_t *seq_ids,
                               const int32_t *seq_lens, int32_t num_decoding_seqs,
                               int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                               int32_t cur_layer, int32_t num_layers, int32_t block_size,
                               int32_t max_blocks_per_seq, int64_t q_tok_stride,
                               int64_t k_tok_stride, int64_t v_tok_stride, int32_t dtype,
                               swl_stream_t stream);

/* ---- Skinny GEMM for decode batches -----------------------------------------------------------------
 * reference: kernels/linear.py:3-12 (F.linear), call sites transformer_layer.py:54-56,117,126,128 and
 * post_layer.py:38. out[M, N] = x[M, K] . W[N, K]^T with fp32 accumulation and one rounding, for
 * M <= 32 tokens: a weight-streaming MFMA kernel (every byte of W read once, in full lines). When N/32
 * tiles cannot fill the chip, K is split across workgroups into fp32 partial slabs in `workspace` and
 * reduced in a fixed order by a second kernel. N % 32 == 0, K % 128 == 0; x/out rows may be strided
 * (elements). k_splits: 0 = choose, or a power of two <= 16. Larger M: use the BLAS.
 * workspace: >= swl_gemm_skinny_workspace_bytes(M, N, K) bytes (0 = none needed). */
size_t swl_gemm_skinny_workspace_bytes(int32_t M, int32_t N, int32_t K);
int swl_gemm_skinny(void *out, const void *x, const void *w, void *workspace, size_t workspace_bytes,
                    int32_t M, int32_t N, int32_t K, int64_t x_row_stride, int64_t out_row_stride,
                    int32_t k_splits, int32_t dtype, swl_stream_t stream);

/* FFN up/gate projection with the SiLU-gate fused into the epilogue (reference: transformer_layer.py:126-127
 * = linear + silu_and_mul_inplace): out[M, I] = (x . W[0:I]^T) * silu(x . W[I:2I]^T), W = [up ; gate]
 * (weight.py:133). Bit-identical to swl_gemm_skinny(k_splits = 1) + swl_silu_mul. I % 32 == 0,
 * K % 128 == 0, M <= 32. */
int swl_gemm_skinny_silu_gate(void *out, const void *x, const void *w_up_gate, int32_t M, int32_t I,
                              int32_t K, int64_t x_row_stride, int64_t out_row_stride, int32_t dtype,
                              swl_stream_t stream);

/* ---- Pre-packed weights -----------------------------------------------------------------------------------------
 * swl_gemm_pack_weight repacks W[N, K] once (load time) into MFMA-fragment order [N/32][K/16][64 lanes][8 elements]:
 * the A operand of a 32x32x16 MFMA becomes one contiguous KiB and a wave's K range for its 32 rows one sequential
 * run, so the decode GEMMs read W with long DRAM bursts and without an LDS transpose (6.0-6.3 instead of 5.3-5.8
 * TB/s). The *_packed entry points take the packed copy and otherwise behave exactly like their row-major twins
 * (same arguments, same bits). N % 32 == 0, K % 128 == 0 (pack: K % 16 == 0), M <= 32. */
int swl_gemm_pack_weight(void *dst, const void *src, int32_t N, int32_t K, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed(void *out, const void *x, const void *w_packed, void *workspace, size_t workspace_bytes,
                           int32_t M, int32_t N, int32_t K, int64_t x_row_stride, int64_t out_row_stride,
                           int32_t k_splits, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_partial(float *slabs, size_t slabs_bytes, const void *x, const void *w_packed, int32_t M,
                                   int32_t N, int32_t K, int64_t x_row_stride, int32_t k_splits, int32_t dtype,
                                   swl_stream_t stream);
int swl_gemm_skinny_packed_silu_gate(void *out, const void *x, const void *w_up_gate_packed, int32_t M, int32_t I,
                                     int32_t K, int64_t x_row_stride, int64_t out_row_stride, int32_t dtype,
                                     swl_stream_t stream);
/* Medium batches on a packed weight: out[M, N] = x . W^T for 32 < M <= 64 tokens (valid for any M <= 64); 2 blocks of
 * 32 tokens share every weight fragment (65..256 tokens: swl_gemm_packed_wide below). workspace >= k_splits * M * N * 4 bytes when K is split
 * (k_splits = 0: library's choice; 16 * M * N * 4 bytes cover any). */
int swl_gemm_packed_mid(void *out, const void *x, const void *w_packed, void *workspace, size_t workspace_bytes,
                        int32_t M, int32_t N, int32_t K, int64_t x_row_stride, int64_t out_row_stride,
                        int32_t k_splits, int32_t dtype, swl_stream_t stream);
int swl_gemm_packed_mid_choose_splits(int32_t M, int32_t N, int32_t K); /* its choice for k_splits = 0 */
/* ... with the SiLU-gate of the FFN in its epilogue: out[M, I] = up * silu(gate), W = [up ; gate] packed */
int swl_gemm_packed_mid_silu_gate(void *out, const void *x, const void *w_up_gate_packed, int32_t M, int32_t I,
                                  int32_t K, int64_t x_row_stride, int64_t out_row_stride, int32_t dtype,
                                  swl_stream_t stream);
/* Large decode batches on a packed weight (csrc/gemm_wide.hip): out[M, N] = x . W^T for up to 256 tokens — the projections
 * of reference kernels/linear.py:3-12 (transformer_layer.py:54-56,117,126,128) at the batch sizes a 264 GB KV pool holds;
 * every weight fragment feeds ceil(M/32) <= 8 MFMAs, x^T shared by the workgroup through LDS. N % 32 == 0, K % 64 == 0.
 * waves_per_group: 0 = library's choice, 4 or 8; k_splits: 0 = library's choice, else a power of two <= 16 with
 * K % (64 * k_splits) == 0; workspace >= k_splits * M * N * 4 bytes when K is split. */
int swl_gemm_packed_wide(void *out, const void *x, const void *w_packed, void *workspace, size_t workspace_bytes,
                         int32_t M, int32_t N, int32_t K, int64_t x_row_stride, int64_t out_row_stride,
                         int32_t waves_per_group, int32_t k_splits, int32_t dtype, swl_stream_t stream);
size_t swl_gemm_packed_wide_workspace_bytes(int32_t M, int32_t N, int32_t K); /* for the library's own plan */
int swl_gemm_packed_wide_choose_splits(int32_t M, int32_t N, int32_t K);       /* its choice for k_splits = 0 */
/* ... stopping at the fp32 partial slabs [k_splits][M][N] (k_splits >= 1) for the split-K consumers */
int swl_gemm_packed_wide_partial(float *slabs, size_t slabs_bytes, const void *x, const void *w_packed, int32_t M,
                                 int32_t N, int32_t K, int64_t x_row_stride, int32_t waves_per_group, int32_t k_splits,
                                 int32_t dtype, swl_stream_t stream);
/* ... with the SiLU-gate of the FFN (reference kernels/silu_and_mul.py:5-34) in its epilogue: out[M, I] = up * silu(gate) */
int swl_gemm_packed_wide_silu_gate(void *out, const void *x, const void *w_up_gate_packed, int32_t M, int32_t I,
                                   int32_t K, int64_t x_row_stride, int64_t out_row_stride, int32_t waves_per_group,
                                   int32_t dtype, swl_stream_t stream);
/* ... stopping at the fp32 partial slabs [k_splits][M][N] (k_splits >= 1) for the split-K consumers */
int swl_gemm_packed_mid_partial(float *slabs, size_t slabs_bytes, const void *x, const void *w_packed, int32_t M,
                                int32_t N, int32_t K, int64_t x_row_stride, int32_t k_splits, int32_t dtype,
                                swl_stream_t stream);

/* Split-K without the reduce launch: the GEMM stops at its fp32 partial slabs [k_splits][M][N] and a FUSED
 * CONSUMER adds them (slab order, one rounding — bit-identical to swl_gemm_skinny's own reduce):
 *   o_proj / down_proj  -> swl_splitk_fused_add_rmsnorm      (reference: rmsnorm.py:39-89)
 *   fused qkv           -> swl_splitk_rotary_store_kv_decode (reference: rotary_emb.py + kvcache_mgmt.py:50-79)
 *   anything else       -> swl_splitk_reduce */
int swl_gemm_skinny_choose_splits(int32_t N, int32_t K);
/* ... on a packed weight (swl_gemm_skinny_packed*, k_splits = 0): splits may differ by one 128-column tile when K has no
 * power-of-two split of whole tiles that fills the chip (Llama-2-7B down_proj: K = 11008 -> 8 splits of 10-11 tiles). */
int swl_gemm_skinny_packed_choose_splits(int32_t N, int32_t K); /* 0 = shape unsupported, 1 = no split */
int swl_gemm_skinny_partial(float *slabs, size_t slabs_bytes, const void *x, const void *w, int32_t M,
                            int32_t N, int32_t K, int64_t x_row_stride, int32_t k_splits,
                            int32_t dtype, swl_stream_t stream);
int swl_splitk_reduce(void *out, const float *slabs, int32_t k_splits, int32_t M, int32_t N,
                      int64_t out_row_stride, int32_t dtype, swl_stream_t stream);
/* residual <- round(sum slabs) + residual ; x_out <- rmsnorm(residual) * w   (slabs: [k_splits][T][hidden]) */
int swl_splitk_fused_add_rmsnorm(void *x_out, void *residual, const void *w, float eps,
                                 const float *slabs, int32_t k_splits, int64_t num_tokens,
                                 int32_t hidden, int32_t dtype, swl_stream_t stream);
/* qkv_slabs: [k_splits][Bd][(H+2*KVH)*D]. Writes rotated q, rotated k and v to the (output) buffers
 * q_out/k_out/v_out and rotated k, v into the paged pools — swl_rotary_store_kv_decode on reduced inputs. */
int swl_splitk_rotary_store_kv_decode(void *q_out, void *k_out, void *v_out, const float *qkv_slabs,
                                      int32_t k_splits, const void *cos_table, const void *sin_table,
                                      const int32_t *pos_idx, void *k_cache, void *v_cache,
                                      const int32_t *block_table, const int32_t *seq_ids,
                                      const int32_t *seq_lens, int32_t num_decoding_seqs,
                                      int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                      int32_t cur_layer, int32_t num_layers, int32_t block_size,
                                      int32_t max_blocks_per_seq, int64_t q_tok_stride,
                                      int64_t k_tok_stride, int64_t v_tok_stride, int32_t dtype,
                                      swl_stream_t stream);

/* Per-step decode metadata derived on the device (so a captured hipGraph can be replayed):
 * pos_idx[i] = seq_lens[i] - 1. */
int swl_decode_positions(int32_t *pos_idx, const int32_t *seq_lens, int32_t num_decoding_seqs,
                         swl_stream_t stream);

/* ---- deferred RMSNorm on the decode fast path ---------------------------------------------------------------------
 * fused_add_rmsnorm (reference rmsnorm.py:67-89, called at transformer_layer.py:46,120) needs a whole token row before it
 * can write anything, so as a split-K consumer it runs one workgroup per token (32 workgroups on 256 CUs). The 1/rms is
 * a per-row scalar that commutes with the projection that follows, so the element-wise part runs fully parallel here and
 * the consumers below apply the scale in fp32 before their one rounding:
 *   swl_splitk_add_scale: residual[t, :] += round(sum_k slabs[k][t, :]) (stored, rounded to the storage dtype, as the
 *     reference stores it); x_scaled = round(residual * w); ssq_out[hidden / 1024][num_tokens] = per-1024-column sums of
 *     squares of the updated residual rows. hidden % 1024 == 0.
 *   swl_gemm_skinny_packed_silu_gate_rs: swl_gemm_skinny_packed_silu_gate of rstd[m] * (x_scaled . [up ; gate]^T),
 *     rstd[m] = 1/sqrt(sum_p row_ssq[p][m] / K + eps). Replaces transformer_layer.py:120-127 for decode batches.
 *   swl_paged_attn_decode_qkv_rs: swl_paged_attn_decode_qkv whose fused-qkv slab sums are scaled the same way before they
 *     are rounded, rotated and stored (transformer_layer.py:46-77 + paged_attn.py:152-222). k_splits in {1, 2, 4}.
 * ssq_parts <= 8 everywhere. */
int swl_splitk_add_scale(void *x_scaled, void *residual, const void *w, const float *slabs, int32_t k_splits,
                         float *ssq_out, int64_t num_tokens, int32_t hidden, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_silu_gate_rs(void *out, const void *x, const void *w_up_gate_packed, const float *row_ssq,
                                        int32_t ssq_parts, float eps, int32_t M, int32_t I, int32_t K,
                                        int64_t x_row_stride, int64_t out_row_stride, int32_t dtype, swl_stream_t stream);
int swl_paged_attn_decode_qkv_rs(void *o, const float *qkv_slabs, int32_t k_splits, const float *row_ssq,
                                 int32_t ssq_parts, int32_t hidden, float eps, const void *cos_table,
                                 const void *sin_table, const int32_t *pos_idx, void *k_cache, void *v_cache,
                                 const int32_t *block_table, const int32_t *seq_ids, const int32_t *seq_lens,
                                 void *scratch, float softmax_scale, int32_t num_decoding_seqs, int32_t num_q_heads,
                                 int32_t num_kv_heads, int32_t head_dim, int32_t num_layers, int32_t block_size,
                                 int32_t cur_layer, int32_t max_blocks_per_seq, int32_t seq_block_size,
                                 int32_t num_seq_blocks, int64_t o_tok_stride, int32_t dtype, swl_stream_t stream);

/* ---- decode projections for very small batches that consume the previous projection's slabs (csrc/gemm_tiny.hip) ----
 * M <= swl_gemm_tiny_max_tokens() (4). At batch 1 the two split-K consumers of a decode layer (swl_splitk_add_scale:
 * reference rmsnorm.py:67-89 at transformer_layer.py:46,120) are 10 % of the layer and run on four workgroups; here the
 * NEXT projection rebuilds its activations itself while its first weight tiles are in flight — residual_out = round(sum
 * slabs_in) + residual_in (stored by the workgroups with blockIdx.x == 0; residual_out != residual_in, the others still
 * read the old rows), x = round(residual_out * norm_w) kept in LDS for the whole K loop — and carries the sums of squares
 * to where the deferred 1/rms is applied. Packed weights (swl_gemm_pack_weight), K % 128 == 0, K / k_splits_out <= 4096.
 *   swl_gemm_tiny_partial_from_splitk: the fused qkv projection (transformer_layer.py:46-56): slabs_out[k_splits_out][M][N]
 *     fp32 = x . W^T per K-chunk (the bits of swl_splitk_add_scale + swl_gemm_skinny_packed_partial), ssq_out[k_splits_out]
 *     [M] = sums of squares of the residual rows per K-chunk — what swl_paged_attn_decode_qkv_rs takes as row_ssq
 *     (ssq_parts = k_splits_out). slabs_out != slabs_in.
 *   swl_gemm_tiny_silu_gate_from_splitk: the FFN up/gate projection + SiLU-gate (transformer_layer.py:120-127):
 *     out[M, I] = up * silu(gate) of rstd[m] * (x . [up ; gate]^T), rstd from the same rows. I % 64 == 0, K <= 4096. */
/*   swl_paged_attn_decode_qkv_rs_partials: swl_paged_attn_decode_qkv_rs stopped after phase 1 when num_seq_blocks > 1 — the
 *     flash-decoding partials stay in `scratch` (mid_o fp32 [Bd][H][nsb][D], then mid_lse fp32 [Bd][H][nsb]; reference
 *     paged_attn.py:106-108), `o` may be NULL; with num_seq_blocks == 1 it is swl_paged_attn_decode_qkv_rs.
 *   swl_gemm_tiny_partial_from_attn: o_proj (transformer_layer.py:117) on those partials — every workgroup merges the
 *     partials of its K-chunk of heads itself (phase 2's LSE-weighted sum, paged_attn.py:108-150, rounded to the storage
 *     dtype as phase 2 stores it) and writes slabs_out[k_splits_out][M][N]; K = num_q_heads * head_dim. Replaces the
 *     phase-2 launch of a batch of <= 4 sequences. */
int swl_paged_attn_decode_qkv_rs_partials(void *o, const float *qkv_slabs, int32_t k_splits, const float *row_ssq,
                                          int32_t ssq_parts, int32_t hidden, float eps, const void *cos_table,
                                          const void *sin_table, const int32_t *pos_idx, void *k_cache, void *v_cache,
                                          const int32_t *block_table, const int32_t *seq_ids, const int32_t *seq_lens,
                                          void *scratch, float softmax_scale, int32_t num_decoding_seqs,
                                          int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                          int32_t num_layers, int32_t block_size, int32_t cur_layer,
                                          int32_t max_blocks_per_seq, int32_t seq_block_size, int32_t num_seq_blocks,
                                          int64_t o_tok_stride, int32_t dtype, swl_stream_t stream);
int swl_gemm_tiny_partial_from_attn(float *slabs_out, size_t slabs_out_bytes, int32_t k_splits_out,
                                    const float *attn_scratch, const int32_t *seq_lens, int32_t num_q_heads,
                                    int32_t head_dim, int32_t seq_block_size, int32_t num_seq_blocks,
                                    const void *w_packed, int32_t M, int32_t N, int32_t dtype, swl_stream_t stream);
int swl_gemm_tiny_max_tokens(void);
int swl_gemm_tiny_partial_from_splitk(float *slabs_out, size_t slabs_out_bytes, int32_t k_splits_out, float *ssq_out,
                                      const float *slabs_in, int32_t k_splits_in, const void *residual_in,
                                      void *residual_out, const void *norm_w, const void *w_packed, int32_t M, int32_t N,
                                      int32_t K, int32_t dtype, swl_stream_t stream);
int swl_gemm_tiny_silu_gate_from_splitk(void *out, const float *slabs_in, int32_t k_splits_in, const void *residual_in,
                                        void *residual_out, const void *norm_w, float eps, const void *w_up_gate_packed,
                                        int32_t M, int32_t I, int32_t K, int64_t out_row_stride, int32_t dtype,
                                        swl_stream_t stream);

/* ---- hidden-wide projections of a decode layer with K split INSIDE the workgroup (csrc/gemm_rows.hip) ----------------------
 * o_proj / down_proj (reference kernels/linear.py:3-12 at layers/transformer_layer.py:117,128) and the residual add that
 * follows them (rmsnorm.py:54-57 at transformer_layer.py:120 and the next layer's :46) in ONE launch, M <= 32 tokens, packed
 * weight (swl_gemm_pack_weight), K % 1024 == 0, N % 32 == 0. A workgroup owns 16 rows of W for all of K (8 waves x K/8,
 * summed through LDS in K order): no slabs, no consumer launch.
 *   swl_gemm_rows_supported: 1 when (M, N, K) is a shape the kernel takes.
 *   swl_gemm_rows_add: residual[t, :] += round(x[t, :] . W^T) (stored rounded to the storage dtype, as the reference stores
 *     it) and nothing else. The norm weight and the sums of squares are left to the consumer, which sees every row anyway:
 *   swl_gemm_skinny_packed_partial_nf ("norm on the fly"): swl_gemm_skinny_packed_partial on x = round(r * norm_w) built
 *     while the raw rows r[M, K] are staged, + ssq_out[k_splits][M] = sum r^2 per K-chunk — the row_ssq of
 *     swl_paged_attn_decode_qkv_rs (ssq_parts = k_splits). Even splits only. The fused qkv projection, :46-56.
 *   swl_gemm_skinny_packed_silu_gate_nf: swl_gemm_skinny_packed_silu_gate_rs with rstd from its own sums (:120-127).
 * Together: a decode layer of <= 8 sequences in 5 launches (qkv, attention, o, up/gate, down), 6 up to 32 (down_proj stays
 * split-K + one consumer there). */
int swl_gemm_rows_supported(int32_t M, int32_t N, int32_t K);
int swl_gemm_rows_add(void *residual, const void *x, const void *w_packed, int32_t M, int32_t N, int32_t K,
                      int64_t x_row_stride, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_partial_nf(float *slabs, size_t slabs_bytes, float *ssq_out, const void *x, const void *norm_w,
                                      const void *w_packed, int32_t M, int32_t N, int32_t K, int64_t x_row_stride,
                                      int32_t k_splits, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_silu_gate_nf(void *out, const void *x, const void *norm_w, float eps,
                                        const void *w_up_gate_packed, int32_t M, int32_t I, int32_t K,
                                        int64_t x_row_stride, int64_t out_row_stride, int32_t dtype, swl_stream_t stream);

/* ---- the same path with the reference's rounding points (r06c: float16 AND bfloat16) -----------------------------------------
 * The deferred norm of the `_nf` entries rounds round(r * w) and applies the 1/rms after the projection — bfloat16 only
 * (DESIGN.md section 4.5). Here the norm is EXACT: fused_add_rmsnorm's arithmetic (reference rmsnorm.py:54-64 at
 * layers/transformer_layer.py:46,120: the sum rounded and stored, the sums of squares and the 1/rms in fp32, ONE rounding of
 * r * rstd * w), split over the two launches that are there anyway:
 *   swl_gemm_rows_add_ssq: swl_gemm_rows_add + ssq_out[M][N / 16] (fp32) = per (token, 16-column tile) sums of squares of the
 *     updated residual rows (the workgroup that finishes a tile has its values in registers);
 *   swl_gemm_skinny_packed_silu_gate_nx / swl_gemm_skinny_packed_partial_nx: the consuming projections add the ssq_parts
 *     (= hidden / 16, % 64 == 0) partials of every row in a fixed order before their first tile and stage
 *     round(r * rstd * norm_w); outputs as swl_gemm_skinny_packed_silu_gate / swl_gemm_skinny_packed_partial (nothing
 *     pending: the slabs go to swl_paged_attn_decode_qkv as they are). */
int swl_gemm_rows_add_ssq(void *residual, float *ssq_out, const void *x, const void *w_packed, int32_t M, int32_t N, int32_t K,
                          int64_t x_row_stride, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_silu_gate_nx(void *out, const void *x, const void *norm_w, float eps, const float *ssq_in,
                                        int32_t ssq_parts, const void *w_up_gate_packed, int32_t M, int32_t I, int32_t K,
                                        int64_t x_row_stride, int64_t out_row_stride, int32_t dtype, swl_stream_t stream);
int swl_gemm_skinny_packed_partial_nx(float *slabs, size_t slabs_bytes, const void *x, const void *norm_w, float eps,
                                      const float *ssq_in, int32_t ssq_parts, const void *w_packed, int32_t M, int32_t N,
                                      int32_t K, int64_t x_row_stride, int32_t k_splits, int32_t dtype, swl_stream_t stream);

/* ---- the transformer stack of a one-sequence decode step as ONE persistent launch (csrc/decode_engine.hip) ----------------
 * reference: the layer loop of LlamaModel._forward (swiftllm/worker/model.py:228-249) over
 * LlamaTransformerLayer.forward (swiftllm/worker/layers/transformer_layer.py:31-130) for ONE decoding sequence: embedding row
 * (pre_layer.py:15-20), and per layer fused add + RMSNorm (rmsnorm.py:39-89), q/k/v projections (linear.py:3-12), rotary
 * (rotary_emb.py:7-58), KV store of the new token (kvcache_mgmt.py:50-79), paged attention phase 1 + 2
 * (paged_attn.py:9-149), o projection, fused add + RMSNorm, up/gate projection, SiLU-gate (silu_and_mul.py:5-34), down
 * projection — with the reference's rounding points in BOTH dtypes. 256 workgroups (one per CU): a loader wave streams a
 * per-CU weight stream by LDS-DMA through a 7 x 16 KiB ring, three consumer waves do the arithmetic; operator boundaries
 * are all-to-all hand-offs of 8-byte {tag, payload} granules inside the launch; every wait is bounded.
 *   swl_decode_engine_supported: 1 when the model shape and the device (num_cus == 256, head_dim == 128, H*D == hidden,
 *     H/KVH in {1, 2, 4}, hidden and ffn_inter_dim multiples of 2048 ...) are what the kernel is laid out for.
 *   swl_decode_engine_slots_per_layer: 16 KiB slots one CU streams per layer (0: unsupported). The weight stream is
 *     [num_layers][256][slots][8192 elements]: per CU and layer qkv | o | up,gate | down; an operator's slots are ordered
 *     (row group of 8, k-chunk of 1024); inside a slot piece p (1 KiB), lane l holds W[row 8g + l/8][1024j + 64p + 8(l%8) ..+8]
 *     (swiftllm_amd/worker/decode_engine.py: pack_engine_layer). CU c owns rows [c*N/256, (c+1)*N/256) of every projection
 *     (up rows and the matching gate rows for the FFN).
 *   swl_decode_engine_workspace_bytes / swl_decode_engine_reset: the hand-off workspace (state words + granule regions);
 *     reset zeroes it and starts the epoch counter (synchronises the stream). Call once after allocation and after any
 *     step that reported an error.
 *   swl_decode_engine_step: resid_out[hidden] = the residual stream after the last layer for the sequence described by
 *     input_ids[0] / seq_ids[0] / seq_lens[0] (length INCLUDING the token being decoded, model.py:296); writes the new
 *     token's K/V into the pools. err_out (may be NULL) receives 0, or the code of a timed-out wait (the workspace then stays
 *     poisoned until reset: later steps return at once with the same code). debug_stamps (may be NULL): [7][num_layers][16]
 *     100 MHz timestamps of the phases of CUs 0, 37, ... 222. flags: bit 0 = the loader keeps one fill in flight instead of
 *     three to four while a consumer wave of its CU sweeps granules (pass 1 unless measuring). Must not run concurrently
 *     with another kernel on the device (one workgroup per CU, all 256 resident). */
int swl_decode_engine_supported(int32_t hidden, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                int32_t ffn_inter_dim, int32_t num_cus);
int swl_decode_engine_slots_per_layer(int32_t hidden, int32_t num_q_heads, int32_t num_kv_heads, int32_t ffn_inter_dim);
size_t swl_decode_engine_workspace_bytes(int32_t hidden, int32_t num_q_heads, int32_t num_kv_heads,
                                         int32_t ffn_inter_dim);
int swl_decode_engine_reset(void *workspace, size_t workspace_bytes, swl_stream_t stream);
int swl_decode_engine_step(void *resid_out, const void *w_stream, const void *norms, const void *wte, void *k_cache,
                           void *v_cache, const int32_t *block_table, const int32_t *input_ids, const int32_t *seq_ids,
                           const int32_t *seq_lens, const void *cos_table, const void *sin_table, void *workspace,
                           size_t workspace_bytes, int64_t *err_out, uint64_t *debug_stamps, int32_t num_layers,
                           int32_t hidden, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                           int32_t ffn_inter_dim, int32_t max_blocks_per_seq, float eps, float softmax_scale,
                           int32_t flags, int32_t dtype, swl_stream_t stream);

/* ---- fp32 residual stream: embedding with learned positions, LayerNorm, fused sandwich-norm step ------------------
 * (no counterpart in the reference, which serves LLaMA only; used by the Kekapel model.) dtype may be SWL_F32.
 * swl_embed_pos:     x[t] = embed[tokens[t]] * scale + pos[positions[t]] in fp32; x0 (may be NULL) gets a copy; pos NULL:
 *                    a model without learned positions (x[t] = embed[tokens[t]] * scale).
 * swl_layernorm:     out[r] = (x[i] - mean) / sqrt(var + eps) * w + b of row i = row_idx ? row_idx[r] : r (fp32 stats,
 *                    var = mean of squared deviations); out in dtype, x / w / b fp32.
 * swl_add_layernorm: x += mult * LN(y; w1, b1) (if y) + x0 (if x0) + step (if step, a [width] vector);
 *                    out = LN(x; w2, b2) (if out). y / out in dtype. */
int swl_embed_pos(float *x, float *x0, const void *embed, const void *pos, const int32_t *tokens,
                  const int32_t *positions, float scale, int64_t num_tokens, int32_t width, int32_t dtype,
                  swl_stream_t stream);
int swl_layernorm(void *out, const float *x, const int32_t *row_idx, const float *w, const float *b, float eps,
                  int64_t num_rows, int32_t width, int32_t dtype, swl_stream_t stream);
int swl_add_layernorm(float *x, const void *y, float mult, const float *w1, const float *b1, const float *x0,
                      const float *step, void *out, const float *w2, const float *b2, float eps, int64_t num_tokens,
                      int32_t width, int32_t dtype, swl_stream_t stream);

/* ---- per-head q/k RMS norm + paged KV store ---------------------------------------------------------------------------
 * qkv[T, tok_stride] = [q heads | k heads | v heads] of one fused projection. q heads are normalised in place (weight q_w
 * [dim], shared by the heads); k heads are normalised (k_w) into the K pool (block b = [kv_heads, 16, dim] at k_cache + b * block_stride
 * elements); v heads are copied into the V pool (block b = [kv_heads, vdim, 16], TRANSPOSED, at v_cache + b * block_stride), block
 * block_table[tok_seq[t]][tok_pos[t] / 16], slot tok_pos[t] % 16.
 * k_cache == NULL: only the query norm (memory-profiling runs). dtype may be SWL_F32. */
int swl_qknorm_store_kv(void *qkv, const float *q_w, const float *k_w, void *k_cache, void *v_cache,
                        const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos, int64_t num_tokens,
                        int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t tok_stride,
                        int32_t max_blocks_per_seq, int64_t block_stride, float eps, int32_t dtype, swl_stream_t stream);

/* ---- sliding-window attention with soft-capping and pre-softmax head mixing over the paged pool -----------------------
 * out[T, H * vdim]; token t attends keys [max(0, p - window + 1), p] of its sequence (window 0: all), p = tok_pos[t];
 * score = softcap * tanh(q.k * scale / softcap) (softcap 0: none), mixed over heads by talk[H, H] (fp32), softmax, values.
 * H <= 32, H * vdim <= 8192. dtype may be SWL_F32. */
/* talk may be NULL (no head mixing). rel (may be NULL): fp32 [num_q_heads, rel_len], a bias added to the (mixed) score of
 * head h at distance query position - key position (distances beyond rel_len - 1 take the last entry). */
int swl_window_attn(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                    const int32_t *tok_seq, const int32_t *tok_pos, const float *talk, const float *rel, int32_t rel_len, int64_t num_tokens,
                    int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride,
                    int32_t window, float scale, float softcap, int32_t max_blocks_per_seq, int64_t block_stride,
                    int32_t dtype, swl_stream_t stream);

/* The matrix-core form for 16-bit dtypes and head sizes 64 / 128: the step's tokens come as tiles of up to 16 consecutive
 * tokens of one sequence (tile_row0[i] = first token row, tile_cnt[i] = tokens; a decoded token is a tile of one). Same
 * arithmetic as swl_window_attn up to rounding (fp32 scores and weights; weights enter the value product as hi + lo 16-bit
 * terms). key_splits > 1 (few tiles, long windows: decode batches): each tile's pages are shared out over that many
 * workgroups, whose partial results (scratch: key_splits * num_tokens * H * (vdim + 2) floats, 16-byte aligned) a second launch
 * combines. swl_window_attn_tiles_supported: 1 when it serves the shape. */
int swl_window_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int32_t dtype);
int swl_window_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                          const int32_t *tok_seq, const int32_t *tok_pos, const int32_t *tile_row0,
                          const int32_t *tile_cnt, const float *talk, const float *rel, int32_t rel_len, int32_t num_tiles, int32_t num_q_heads,
                          int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride, int32_t window,
                          float scale, float softcap, int32_t max_blocks_per_seq, int64_t block_stride,
                          int32_t key_splits, float *scratch, int64_t num_tokens, int32_t dtype, swl_stream_t stream);

/* ---- the same attention loops with the masks and denominators of other designs --------------------------------------------
 * swl_masked_attn / swl_masked_attn_tiles are swl_window_attn / swl_window_attn_tiles with
 *   mask_kind     0: sliding window (keys [p - window + 1, p]); 1: chunks (keys [floor(p / window) * window, p], chunks
 *                 counted from position 0). window 0: every earlier key, whatever the kind.
 *   sink          NULL, or fp32 [num_q_heads]: a logit per head that is added to the softmax denominator only.
 *   num_v_heads   value heads in a page (divides num_kv_heads); key head g reads value head g % num_v_heads. Several score
 *                 maps over the same values: lay the maps out map-major, [map][head].
 *   out_f32       1: out is fp32 whatever dtype says of the operands.
 *   heads_per_group (tiles only; 0: all) heads handled by one workgroup when the heads are not mixed: the heads of a tile
 *                 are shared out over ceil(H / heads_per_group) workgroups. -1: the rows of a matrix-core tile are sixteen
 *                 HEADS of one token instead of sixteen tokens (requires num_tiles == num_tokens, i.e. every tile is one
 *                 token, num_kv_heads == 1, no talk, no rel): the form for decode steps of heads that share one key head.
 * The tiles form serves more (dim, vdim) pairs without a mixing matrix than with one: ask swl_masked_attn_tiles_supported. */
int swl_masked_attn(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                    const int32_t *tok_seq, const int32_t *tok_pos, const float *talk, const float *rel, int32_t rel_len,
                    int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim,
                    int64_t q_tok_stride, int32_t window, float scale, float softcap, int32_t max_blocks_per_seq,
                    int64_t block_stride, int32_t mask_kind, const float *sink, int32_t num_v_heads, int32_t out_f32,
                    int32_t dtype, swl_stream_t stream);
int swl_masked_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t num_v_heads, int32_t dim,
                                    int32_t vdim, int32_t dtype);
int swl_masked_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                          const int32_t *tok_seq, const int32_t *tok_pos, const int32_t *tile_row0,
                          const int32_t *tile_cnt, const float *talk, const float *rel, int32_t rel_len, int32_t num_tiles,
                          int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride,
                          int32_t window, float scale, float softcap, int32_t max_blocks_per_seq, int64_t block_stride,
                          int32_t key_splits, float *scratch, int64_t num_tokens, int32_t mask_kind, const float *sink,
                          int32_t num_v_heads, int32_t out_f32, int32_t heads_per_group, int32_t dtype,
                          swl_stream_t stream);

/* ---- rotary positions on interleaved pairs fused with the paged KV store; gated / combined heads ---------------------------
 * Rotation: dimension 2i of a head is paired with 2i + 1, i < rot_dims / 2; (u, v) at position p becomes
 * (u cos a - v sin a, v cos a + u sin a), a = p * freq[i] (freq: float64 [rot_dims / 2] on the device; angles are evaluated
 * in float64). dtype may be SWL_F32. Pages: keys [heads, 16, dim], values transposed [heads, vdim, 16].
 * swl_rope_store_kv: rows [q: num_q_heads x dim | k: num_k_heads x dim | v: num_v_heads x vdim]; q rotated in place, k
 *   rotated into the K pool, v into the V pool. k_cache NULL: queries only.
 * swl_latent_rope_store_kv: rows hold num_heads query heads [dim | rot_dim] and, at column dkv_col (< 0: none), the
 *   compressed row [kv_rank | rot_dim]. qa[t][h][kv_rank : kv_rank + rot_dim] = rotated query part; the RMS-normed latent
 *   (weight c_norm, eps) and the rotated shared key part are stored as one key head of kv_rank + rot_dim and the latent
 *   again, transposed, as one value head of kv_rank.
 * swl_diff_head_combine: maps fp32 [T, 2, H, vdim] -> out[T, H, vdim] = unit_rms(a1 - lambda a2; eps) * mult *
 *   sigmoid(gate[t * gate_stride + h]) (gate NULL: no gate).
 * swl_head_gate: y[T, H, vdim] *= sigmoid(gate[t * gate_stride + h]) in place. */
int swl_rope_store_kv(void *qkv, const double *freq, void *k_cache, void *v_cache, const int32_t *block_table,
                      const int32_t *tok_seq, const int32_t *tok_pos, int64_t num_tokens, int32_t num_q_heads,
                      int32_t num_k_heads, int32_t num_v_heads, int32_t dim, int32_t vdim, int32_t rot_dims,
                      int64_t tok_stride, int32_t max_blocks_per_seq, int64_t block_stride, int32_t dtype,
                      swl_stream_t stream);
int swl_latent_rope_store_kv(const void *proj, void *qa, const double *freq, const float *c_norm, void *k_cache,
                             void *v_cache, const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                             int64_t num_tokens, int32_t num_heads, int32_t dim, int32_t rot_dim, int32_t kv_rank,
                             int64_t proj_stride, int64_t dkv_col, int64_t qa_stride, int32_t max_blocks_per_seq,
                             int64_t block_stride, float eps, int32_t dtype, swl_stream_t stream);
int swl_diff_head_combine(void *out, const float *maps, const void *gate, int64_t gate_stride, float lambda, float mult,
                          float eps, int64_t num_tokens, int32_t num_heads, int32_t vdim, int32_t dtype,
                          swl_stream_t stream);
int swl_head_gate(void *y, const void *gate, int64_t gate_stride, int64_t num_tokens, int32_t num_heads, int32_t vdim,
                  int32_t dtype, swl_stream_t stream);

/* ---- PolyNorm activation: out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row ---------- */
int swl_polynorm(void *out, const void *z, float a, float b, float c, float e, float eps, int64_t num_rows, int32_t ff,
                 int32_t dtype, swl_stream_t stream);

/* ---- mixture of experts ---------------------------------------------------------------------------------------------------
 * swl_moe_route: idx_out[T, top] / w_out[T, top] = the top experts of fp32 logits router[experts, width] h + bias and the
 * softmax over the chosen logits. swl_moe_gate_up: y[T * top, ff] = clamped gated unit of expert idx[a] on token a / top;
 * gate_up [experts, 2 ff, width] = gate rows then up rows. swl_moe_down_combine: out[T, width] = sum_j w[t][j] down[e_j] y.
 * dtype may be SWL_F32. */
int swl_moe_route(int32_t *idx_out, float *w_out, const void *h, const float *router, const float *bias,
                  int64_t num_tokens, int32_t width, int32_t experts, int32_t top, int32_t dtype, swl_stream_t stream);
int swl_moe_gate_up(void *y, const void *h, const void *gate_up, const int32_t *expert_idx, int64_t num_tokens,
                    int32_t width, int32_t ff, int32_t top, float limit, int32_t act, int32_t dtype, swl_stream_t stream);
/* Large steps (prompt portions): assignments are sorted by expert and every expert's rows go through the library GEMM;
 * swl_glu_clamp: y[r][f] = act of [gate | up] product rows gate_up[r][2 ff]; swl_moe_combine: out[t] = sum_j w[t][j] *
 * rows[where[t * top + j]] (fp32, fixed order). dtype may be SWL_F32. */
/* Decode-sized steps, 16-bit, on the matrix core: a workgroup per (expert, 64 outputs) loads every weight fragment once and
 * multiplies it with all assignments of the expert (an expert's weights are streamed once per step). glu = 1: out = y[T * top, ff] from x = h[T, width]
 * and w = gate_up; glu = 0: out = rows[T * top, width] (plain products, for swl_moe_combine) from x = y and w = down.
 * act (swl_moe_gate_up, swl_glu_clamp): 0 the clamped unit min(g, limit) sigmoid(1.702 g) (clamp(u) + 1), 1 the plain gated
 * unit silu(g) u (limit unused); swl_moe_expert_stationary takes the latter as glu = 3. */
int swl_moe_expert_stationary_supported(int64_t num_tokens, int32_t width, int32_t ff, int32_t top, int32_t dtype);
int swl_moe_expert_stationary(void *out, const void *x, const void *w, const int32_t *expert_idx, int64_t num_tokens,
                              int32_t experts, int32_t width, int32_t ff, int32_t top, int32_t glu, float limit,
                              int32_t dtype, swl_stream_t stream);
int swl_glu_clamp(void *y, const void *gate_up, int64_t num_rows, int32_t ff, float limit, int32_t act, int32_t dtype,
                  swl_stream_t stream);
int swl_moe_combine(void *out, const void *rows, const int64_t *where, const float *expert_w, int64_t num_tokens,
                    int32_t width, int32_t top, int32_t dtype, swl_stream_t stream);
int swl_moe_down_combine(void *out, const void *y, const void *down, const int32_t *expert_idx, const float *expert_w,
                         int64_t num_tokens, int32_t width, int32_t ff, int32_t top, int32_t dtype, swl_stream_t stream);

/* Squared-ReLU experts and routers that weigh by the softmax over ALL experts. swl_moe_route_scores: the `top` experts with
 * the largest fp32 logits router h (+ bias, may be NULL); weights = scale * softmax(all logits)[chosen], not renormalised.
 * swl_moe_up_relu2: y[T * top, ff] = relu(up[e] h)^2, up [experts, ff, width]. swl_moe_expert_stationary with glu = 2 is its
 * matrix-core form. swl_relu_sq: y[r][f] = relu(z[r * in_stride + f])^2. dtype may be SWL_F32. */
int swl_moe_route_scores(int32_t *idx_out, float *w_out, const void *h, const float *router, const float *bias,
                         int64_t num_tokens, int32_t width, int32_t experts, int32_t top, float scale, int32_t dtype,
                         swl_stream_t stream);
int swl_moe_up_relu2(void *y, const void *h, const void *up, const int32_t *expert_idx, int64_t num_tokens, int32_t width,
                     int32_t ff, int32_t top, int32_t dtype, swl_stream_t stream);
int swl_relu_sq(void *y, const void *z, int64_t num_rows, int32_t ff, int64_t in_stride, int32_t dtype, swl_stream_t stream);

/* ---- q/k RMS norm over the whole projection + KV store (pool layout of swl_qknorm_store_kv) -------------------------------
 * q <- q / rms(q over all heads) * q_w[heads * dim] * (1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1)); keys likewise
 * (no multiplier) into the pool, values copied. k_cache NULL: the row holds queries only. dtype may be SWL_F32. */
int swl_qknorm_full_store_kv(void *qkv, const float *q_w, const float *k_w, void *k_cache, void *v_cache,
                             const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                             int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim,
                             int64_t tok_stride, int32_t max_blocks_per_seq, int64_t block_stride, float eps,
                             float temp_coef, int32_t temp_every, int32_t dtype, swl_stream_t stream);

/* ---- fp32 stream with RMS norms, gated sublayer results and causal input convolutions (csrc/rms_stream.hip) --------------
 * swl_gated_add_rmsnorm: y = m (+ sigmoid(m2_gate[t]) * m2); y *= sigmoid(r + r_bias); x += y / rms(y) * w1; out = x / rms(x)
 * * w2. m NULL: only the output norm, of rows row_idx when given. Per-sequence state: `state` is the base of the state slots
 * (fp32, slot_stride floats apart); tok_state[t] = slot * 2 + parity, tok_start[t] = position of the first token of t's
 * portion. swl_causal_conv_state: out = (h if add_input) + causal convolution of h over time with w [taps, channels] (fp32),
 * the carried inputs at tail_off inside the slot ([2][taps - 1][channels] floats). dtype may be SWL_F32. */
int swl_gated_add_rmsnorm(float *x, const void *m, const void *m2, const void *m2_gate, int64_t m2_gate_stride,
                          const void *r, int64_t r_stride, const float *r_bias, const float *w1, void *out, const float *w2,
                          const int32_t *row_idx, float eps, int64_t num_rows, int32_t width, int32_t dtype,
                          swl_stream_t stream);
int swl_causal_conv_state(void *out, int64_t out_stride, const void *h, int64_t h_stride, const float *w, float *state,
                          int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos, const int32_t *tok_start,
                          const int32_t *tok_state, const int32_t *tok_seq, int64_t num_tokens, int32_t channels,
                          int32_t taps, int32_t add_input, int32_t dtype, swl_stream_t stream);

/* ---- gated delta rule (csrc/delta_rule.hip) --------------------------------------------------------------------------------
 * swl_delta_prep: proj rows [q | k | v | gate | b | a] -> qn, kn [T, qk heads * dim], kq [T, qk heads] (their dot
 * products), vv [T, heads * vdim], beta, decay
 * [T, heads], all fp32 (convolution + SiLU with conv_w tap-major [taps, q | k | v channels], unit norms, sigmoid,
 * exp(-exp(A_log) softplus(a + dt_bias))).
 * swl_delta_rule: o[T, heads * vdim] (fp32) and the states [heads, dim, vdim] at s_off inside the slots, one portion per
 * (seq_row0, seq_cnt) entry. swl_gated_head_rmsnorm: out = o / rms(o over vdim) * w[vdim] * silu(gate). */
int swl_delta_prep(float *qn, float *kn, float *kq, float *vv, float *beta, float *decay, const void *proj, int64_t proj_stride,
                   const float *conv_w, const float *a_log, const float *dt_bias, float *state, int64_t slot_stride,
                   int64_t tail_off, const int32_t *tok_pos, const int32_t *tok_start, const int32_t *tok_state,
                   const int32_t *tok_seq, int64_t num_tokens, int32_t num_heads, int32_t num_qk_heads, int32_t dim,
                   int32_t vdim, int32_t taps, int32_t dtype, swl_stream_t stream);
int swl_delta_rule(float *o, const float *qn, const float *kn, const float *kq, const float *vv, const float *beta, const float *decay,
                   float *state, int64_t slot_stride, int64_t s_off, const int32_t *seq_row0, const int32_t *seq_cnt,
                   const int32_t *tok_pos, const int32_t *tok_state, int32_t num_seqs, int32_t num_heads,
                   int32_t num_qk_heads, int32_t dim, int32_t vdim, swl_stream_t stream);
int swl_gated_head_rmsnorm(void *out, const float *o, const void *gate, int64_t gate_stride, const float *w, float eps,
                           int64_t num_tokens, int32_t num_heads, int32_t vdim, int32_t dtype, swl_stream_t stream);

/* ---- sigmoid router with group-limited choice (csrc/moe.hip) ---------------------------------------------------------------
 * s = sigmoid(router[experts, width] h) in fp32. Experts are chosen by s + correction (NULL: by s): the experts form
 * group_count equal groups of neighbours, a group's score is the sum of its two largest choice scores, only experts of the
 * group_keep best groups are eligible (group_keep = group_count: all), of these the `top` largest. w_out = the chosen
 * experts' s divided by their sum (+ 1e-20). dtype may be SWL_F32. */
int swl_moe_route_grouped(int32_t *idx_out, float *w_out, const void *h, const float *router, const float *correction,
                          int64_t num_tokens, int32_t width, int32_t experts, int32_t top, int32_t group_count,
                          int32_t group_keep, int32_t dtype, swl_stream_t stream);

/* ---- projections with biases: per-head q/k RMS norm + value blend + KV store (pool layout of swl_qknorm_store_kv) -----------
 * q_h <- (q_h + q_b) / rms * q_w (in place; q_w[dim] shared by the heads, NULL: no weight), keys likewise into the pool,
 * v <- v + v_b, then v <- (1 - mix) v + mix v_other[t] when v_other is given; v is written back into the row and into the
 * pool. Biases fp32 (NULL: none). k_cache NULL: nothing is stored. dtype may be SWL_F32. */
int swl_qkv_bias_norm_store(void *qkv, const float *q_b, const float *k_b, const float *v_b, const float *q_w,
                            const float *k_w, const void *v_other, int64_t v_other_stride, float mix, void *k_cache,
                            void *v_cache, const int32_t *block_table, const int32_t *tok_seq, const int32_t *tok_pos,
                            int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim,
                            int64_t tok_stride, int32_t max_blocks_per_seq, int64_t block_stride, float eps, int32_t dtype,
                            swl_stream_t stream);

/* ---- sigmoid attention over the pool (csrc/sigmoid_attn.hip) ----------------------------------------------------------------
 * a[g] = sigmoid(scale q_g . k - r1[g] ln(1 + r2[g] (i - j)) + pb[g]) for every key j <= i (inside `window` when > 0), no
 * normalisation over keys; a'[h] = sum_g talk[h][g] a[g] (talk NULL: a' = a); out[t][h] = sum_j a'[h] v_j[kv head of h].
 * r1 / r2 (both or neither), pb, talk: fp32, may be NULL. dtype may be SWL_F32. */
int swl_sigmoid_attn(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                     const int32_t *tok_seq, const int32_t *tok_pos, const float *talk, const float *r1, const float *r2,
                     const float *pb, int64_t num_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t dim,
                     int32_t vdim, int64_t q_tok_stride, int32_t window, float scale, int32_t max_blocks_per_seq,
                     int64_t block_stride, int32_t dtype, swl_stream_t stream);
/* The matrix-core form (16-bit storage): tiles of up to 16 consecutive queries of one sequence (tile_row0, tile_cnt) against
 * 16-key pages; key_splits > 1: every tile's pages are shared out over that many workgroups, whose fp32 partial sums
 * (scratch: key_splits * num_tokens * heads * vdim floats) a second launch adds up. */
int swl_sigmoid_attn_tiles_supported(int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int32_t dtype);
int swl_sigmoid_attn_tiles(void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *block_table,
                           const int32_t *tok_seq, const int32_t *tok_pos, const int32_t *tile_row0, const int32_t *tile_cnt,
                           const float *talk, const float *r1, const float *r2, const float *pb, int32_t num_tiles,
                           int32_t num_q_heads, int32_t num_kv_heads, int32_t dim, int32_t vdim, int64_t q_tok_stride,
                           int32_t window, float scale, int32_t max_blocks_per_seq, int64_t block_stride, int32_t key_splits,
                           float *scratch, int64_t num_tokens, int32_t dtype, swl_stream_t stream);

/* ---- state-space recurrence with a scalar decay per head (csrc/ssd.hip) -----------------------------------------------------
 * swl_ssd_prep: proj rows [z | x | B | C | dt] (z, x: heads * vdim; B, C: groups * state; dt: heads) -> xbc [T, x | B | C]
 * fp32 after the causal convolution (conv_w tap-major [taps, channels], bias conv_b) and SiLU; dt [T, heads] =
 * softplus(raw + dt_bias); decay = exp(-exp(A_log) dt). swl_ssd_scan: y [T, heads * vdim] fp32 and the states
 * [heads, state, vdim] at s_off inside the slots: S <- decay S + dt B x^T, y = S^T C + dskip x, one portion per
 * (seq_row0, seq_cnt) entry. swl_gated_group_rmsnorm: g = y * silu(gate); out = g / rms(g over each of `groups` equal
 * parts of the row) * w[cols]. dtype (prep, norm) may be SWL_F32. */
int swl_ssd_prep(float *xbc, float *dt, float *decay, const void *proj, int64_t proj_stride, const float *conv_w,
                 const float *conv_b, const float *a_log, const float *dt_bias, float *state, int64_t slot_stride,
                 int64_t tail_off, const int32_t *tok_pos, const int32_t *tok_start, const int32_t *tok_state,
                 const int32_t *tok_seq, int64_t num_tokens, int32_t num_heads, int32_t vdim, int32_t state_dim,
                 int32_t groups, int32_t taps, int32_t dtype, swl_stream_t stream);
int swl_ssd_scan(float *y, const float *xbc, const float *dt, const float *decay, const float *dskip, float *state,
                 int64_t slot_stride, int64_t s_off, const int32_t *seq_row0, const int32_t *seq_cnt, const int32_t *tok_pos,
                 const int32_t *tok_state, int32_t num_seqs, int32_t num_heads, int32_t vdim, int32_t state_dim,
                 int32_t groups, swl_stream_t stream);
int swl_gated_group_rmsnorm(void *out, const float *y, const void *gate, int64_t gate_stride, const float *w, float eps,
                            int64_t num_tokens, int32_t cols, int32_t groups, int32_t dtype, swl_stream_t stream);

/* ---- fp32 stream of models that norm a sublayer's RESULT only (csrc/rms_stream.hip) -----------------------------------------
 * y = coef * (a' + b'), a' = a / rms(a) * wa (wa NULL: a itself), b' likewise (b NULL: none); x += y / rms(y) * w1;
 * out (may be NULL) = x in the compute dtype, or x / rms(x) * w2 when w2 is given. dtype may be SWL_F32. */
int swl_post_norm_add(float *x, const void *a, const float *wa, const void *b, const float *wb, float coef, const float *w1,
                      void *out, const float *w2, float eps, int64_t num_rows, int32_t width, int32_t dtype,
                      swl_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SWIFTLLM_HIP_H */
