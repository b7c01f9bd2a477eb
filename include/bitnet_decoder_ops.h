/*
 * Caller-side glue of the BitNet decoder around the BitLinear calls, exported
 * from the same shared library as include/bitlinear_hip.h.  Plain C; device
 * pointers owned by the caller; no allocation, no synchronisation, launches on
 * the given stream (hipStream_t as void*), legal under graph capture.
 */
#ifndef BITNET_DECODER_OPS_H
#define BITNET_DECODER_OPS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * One decode step of the attention block between wqkv and wo
 * (Attention.forward, gpu/model.py:128-157, which calls xformers' rope_padded
 * and flash attention on a padded KV cache): for every sequence b
 *   - rotate q and k of the new token by the angles of position positions[b]
 *     (adjacent pairs (2i, 2i+1), fp32, results rounded to bf16),
 *   - write k, v into the cache at that position,
 *   - out[b, h, :] = softmax(q_h . K[0..pos] / sqrt(head_dim)) V[0..pos] for the
 *     n_heads query heads, head h using kv head h / (n_heads / n_kv_heads).
 *   qkv      bf16 [B, (n_heads + 2 n_kv_heads) * head_dim]  (q | k | v)
 *   cache_k/v bf16 [B, S, n_kv_heads, head_dim]
 *   positions int64 [B], 0 <= positions[b] < S (a value outside is clamped
 *            into that range by the kernel: no access leaves the buffers)
 *   cos/sin  fp32 [S, head_dim / 2]
 *   out      bf16 [B, n_heads * head_dim]
 *   workspace float [bitnet_attn_decode_workspace_floats(B, n_heads, n_kv_heads, n_splits)], 8-byte
 *            aligned and zero before the first call that uses it (the calls keep it consistent: every
 *            split's record carries the tag of the call that wrote it, and the tag advances per call)
 *   counters  int [B * n_kv_heads]: kept in the signature for callers written against earlier versions; the
 *             kernel does not use it (must be non-NULL when n_splits > 1)
 *   n_splits  1..16 workgroups share the cache rows of one (sequence, kv head): blocks of 32 rows dealt
 *             round-robin, so the rows up to the position are spread over all splits whatever the capacity
 *             S is; with 1, workspace and counters may be NULL.  Calls that share a workspace must not
 *             overlap in time.  Fastest when B * n_kv_heads * n_splits <= 256 (one workgroup per CU: the
 *             kernel then runs eight waves per workgroup for long caches).
 * head_dim must be 128, g = n_heads / n_kv_heads one of 1, 2, 4, 8.  Returns 0, or 1 (shape), 2 (null
 * pointer), 3 (launch failed).  Scores and outputs on the bf16 matrix pipe with fp32 accumulation, the
 * probabilities rounded to bf16 in between; results agree with an fp32 evaluation of the same formula to
 * about 1e-2 relative on bf16 outputs.
 */
int bitnet_attn_decode(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v,
                       const int64_t* positions, const float* cos_table,
                       const float* sin_table, uint16_t* out, float* workspace,
                       int* counters, int n_splits, int B, int S, int n_heads,
                       int n_kv_heads, int head_dim, void* stream);

/*
 * Start of a decode step: h_out[b, :] = emb[tokens[b], :] (tok_embeddings, gpu/model.py:272) and
 * rope_rows[b, :] = cos_table[positions[b], :] | sin_table[positions[b], :] (64 + 64 floats), one
 * launch.  The rows let the step's attention kernels rotate without first loading the position
 * (bitnet_attn_decode_rows).  tokens / positions int64 [B] (clamped into [0, V) / [0, S) by the
 * kernel); emb bf16 [V, dim], dim % 8 == 0, emb and h_out 16-byte aligned; cos/sin fp32
 * [S, head_dim / 2]; head_dim must be 128.  Returns 0, 1 (shape / alignment), 2 (null), 3 (launch).
 */
int bitnet_decode_step_begin(const int64_t* tokens, const int64_t* positions, const uint16_t* emb,
                             const float* cos_table, const float* sin_table, uint16_t* h_out,
                             float* rope_rows, int B, int V, int dim, int S, int head_dim,
                             void* stream);

/*
 * bitnet_attn_decode with the rotation values of every sequence's position handed over as ready
 * rows (rope_rows float [B, head_dim], as bitnet_decode_step_begin writes them; they must be the
 * tables' rows at positions[b]): results are identical, the kernel saves the memory round trip of
 * the table lookup behind the position.
 */
int bitnet_attn_decode_rows(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v,
                            const int64_t* positions, const float* cos_table,
                            const float* sin_table, const float* rope_rows, uint16_t* out,
                            float* workspace, int* counters, int n_splits, int B, int S,
                            int n_heads, int n_kv_heads, int head_dim, void* stream);

/*
 * Rotary embedding and KV-cache write for a block of T new tokens per sequence (the prompt
 * pass of Attention.forward, gpu/model.py:128-157, where the reference calls xformers'
 * rope_padded): for token (b, t) at position positions[b * T + t]
 *   - q heads rotated (adjacent pairs, fp32, rounded to bf16) into q_out[b, t, h, :],
 *   - k heads rotated and v heads copied into cache_k/v[b, position, kvh, :].
 * The arithmetic is that of bitnet_attn_decode, so both leave identical cache rows.
 *   qkv bf16 [B * T, (n_heads + 2 n_kv_heads) * head_dim]; positions int64 [B * T] (clamped into
 *   [0, S) by the kernel); cos/sin fp32 [S, head_dim / 2]; q_out bf16 [B, T, n_heads, head_dim].
 * head_dim must be 128.  Returns 0, 1 (shape), 2 (null pointer), 3 (launch failed).
 */
int bitnet_rope_cache_tokens(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v,
                             const int64_t* positions, const float* cos_table,
                             const float* sin_table, uint16_t* q_out, int B, int T, int S,
                             int n_heads, int n_kv_heads, int head_dim, void* stream);

/*
 * Causal grouped-query attention of a block of T new tokens per sequence over the cache rows
 * 0 .. start + t (the prompt pass of Attention.forward, gpu/model.py:147-155, where the reference
 * calls xformers' flash attention): token t of sequence b sits at position start + t, its rotated
 * q in q[b, t, h, :] and the k / v of positions 0 .. start + T - 1 already in the cache (written by
 * bitnet_rope_cache_tokens, and by earlier calls for positions below start):
 *   out[b * T + t, h, :] = softmax(q . K[0 .. start + t] / sqrt(head_dim)) V[0 .. start + t]
 *   q bf16 [B, T, n_heads, head_dim]; cache_k/v bf16 [B, S, n_kv_heads, head_dim];
 *   out bf16 [B * T, n_heads * head_dim]; start >= 0, start + T <= S.
 * Scores and outputs on the bf16 matrix pipe with fp32 accumulation, probabilities rounded to
 * bf16 in between; an online softmax over steps of 32 positions.  head_dim must be 128,
 * n_heads / n_kv_heads one of 1, 2, 4, 8, all pointers 16-byte aligned.
 * Returns 0, 1 (shape / alignment), 2 (null pointer), 3 (launch failed).
 */
int bitnet_attn_prefill(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v,
                        uint16_t* out, int B, int T, int S, int start, int n_heads,
                        int n_kv_heads, int head_dim, void* stream);

/* Tuning override for tests and measurements: threads per workgroup of the attention kernel
 * (256 or 512; 0 restores the built-in choice).  Results do not depend on it beyond the
 * order of fp32 additions.  Returns 0, or 1 for another value. */
int bitnet_attn_decode_set_threads(int threads);

/* Number of floats bitnet_attn_decode needs as workspace; -1 for bad arguments. */
int bitnet_attn_decode_workspace_floats(int B, int n_heads, int n_kv_heads, int n_splits);

/*
 * Index (in floats) of the workspace's error word, an int that is zero in a healthy workspace.
 * With more than one split, the workgroup that merges the splits' records polls for them a bounded
 * number of times.  If a poll ever runs out (a workspace that was not zero before its first use, or
 * splits that did not start in the order the kernel counts on), the affected heads' output rows are
 * written as NaN and this word is set to 1; it stays set until the host clears the workspace.  No
 * entry point reads it back (none synchronises): the caller copies the word to the host when it
 * next synchronises anyway, e.g. at the end of a generation.  -1 for bad arguments.
 */
int bitnet_attn_decode_error_index(int B, int n_heads, int n_kv_heads, int n_splits);

/* Test hook: bound of that poll (< 0 restores the built-in bound of 65536 rounds; 0 makes every
 * merge of more than one split give up at once -- every kernel still runs to its end -- which is
 * how the failure path above is tested).  Returns 0. */
int bitnet_attn_decode_set_spin_limit(int polls);

/*
 * The tail of a greedy decode step (Transformer.forward's `self.output(self.norm(h))`,
 * gpu/model.py:280-281, and the argmax of the generation loop, gpu/generate.py:264-288):
 *   y      = RMSNorm(h) with norm_weight (same rounding points as bitlinear_norm_forward_bf16)
 *   logits = bf16(y . emb[v, :]) with fp32 accumulation, for the V rows of the (tied) embedding
 *   token_out[b] = the lowest v with the largest logits[b, v]
 *   h bf16 [B, K]; norm_weight bf16 [K]; emb bf16 [V, K] row-major; y_ws bf16 [B, K] scratch;
 *   logits fp32 [B, V] or NULL (not written then); token_out int64 [B];
 *   part_val float / part_idx int [bitnet_lm_head_workgroups(V) * 16] scratch.
 * B <= 16, K % 64 == 0, B * (2 K + 32) <= 96 KiB; h, norm_weight, emb, y_ws, part_val, part_idx
 * 16-byte aligned.
 * Three launches (norm; product with a best row per workgroup; reduction of those).
 * Returns 0, 1 (shape / alignment), 2 (null), 3 (launch).
 * Calls that share the scratch buffers must not overlap in time.
 */
int bitnet_lm_head_greedy(const uint16_t* h, const uint16_t* norm_weight, float eps,
                          const uint16_t* emb, uint16_t* y_ws, float* logits,
                          int64_t* token_out, float* part_val, int* part_idx,
                          int B, int V, int K, void* stream);

/*
 * The same call with the bookkeeping of a greedy decode loop (gpu/generate.py:264-288: the new
 * token is appended and fed back, the position advances) done by its last kernel instead of by
 * separate launches: next_input[b] = token, positions[b] += 1, history[step_idx[0] * B + b] = token,
 * step_idx[0] += 1.  Each of next_input / positions may be NULL (not done); history and step_idx
 * are given together or not at all (2 otherwise).  All int64, device memory.
 */
int bitnet_lm_head_greedy_step(const uint16_t* h, const uint16_t* norm_weight, float eps,
                               const uint16_t* emb, uint16_t* y_ws, float* logits,
                               int64_t* token_out, float* part_val, int* part_idx,
                               int64_t* next_input, int64_t* positions, int64_t* history,
                               int64_t* step_idx, int B, int V, int K, void* stream);

/* Upper bound of the workgroups bitnet_lm_head_greedy launches for V rows (sizes its scratch);
 * -1 for V < 1. */
int bitnet_lm_head_workgroups(int V);

/* Tuning override for tests and measurements: 0 = built-in choice (up to 8 tokens and K % 512 == 0:
 * a streaming kernel with fp32 multiply-adds on the vector pipe; otherwise a bf16 MFMA kernel), 1 = MFMA kernel always,
 * 2 = same as 0.  Results differ only in the order of fp32 additions.  Returns 0, or 1. */
int bitnet_lm_head_set_kernel(int which);

#ifdef __cplusplus
}
#endif
#endif /* BITNET_DECODER_OPS_H */
