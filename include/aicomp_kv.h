/*
 * aicomp_kv.h - C ABI of the MI355X (gfx950) paged KV-cache attention library.
 *
 * This is the whole drop-in boundary: plain pointers, sizes and a HIP stream
 * handle.  Every pointer except `stream` is DEVICE memory owned by the caller
 * and borrowed for the duration of the call; nothing is allocated, freed or
 * synchronised inside the library.  All work is enqueued on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream).
 *
 * The operator being replaced is the reference's
 *   CachedScaledDotProductAttention.forward     opt_prime/opt_prime/kv_cache.py:340-415
 *   KVCacheManager.update                       opt_prime/opt_prime/kv_cache.py:112-170
 * which run, per transformer layer and per step, (1) a slice-assign append of
 * the new K/V rows, (2) a .contiguous() copy of the whole prefix and (3)
 * torch's scaled_dot_product_attention.  The entry points below are those
 * three steps on a paged pool, with (2) removed.
 *
 * Pool layout (both pools):  [num_blocks, num_kv_heads, block_size, head_dim],
 * contiguous.  Token t of sequence s lives at slot
 *   block_table[s][t / block_size] * block_size + t % block_size.
 * Heads in the pool are KV heads; query head h reads KV head h / (Hq / Hkv),
 * the order HF Llama's repeat_kv produces (compiler_fx/modeling_llama.py:268-277).
 *
 * Return value: 0 on success, otherwise one of the AICOMP_KV_E* codes; the
 * message of the last failure on the calling thread is aicomp_kv_last_error().
 */
#ifndef AICOMP_KV_H
#define AICOMP_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AICOMP_KV_OK            0
#define AICOMP_KV_EINVAL        1   /* bad shape / dtype / null pointer / size   */
#define AICOMP_KV_EUNSUPPORTED  2   /* valid request the kernels do not cover    */
#define AICOMP_KV_EHIP          3   /* a HIP runtime call failed                 */
#define AICOMP_KV_EWORKSPACE    4   /* workspace missing or too small            */

/* element types */
#define AICOMP_KV_F32       0
#define AICOMP_KV_BF16      1
#define AICOMP_KV_FP8_E4M3  2       /* OCP e4m3 ("e4m3fn"), max finite 448       */
#define AICOMP_KV_F16       3       /* IEEE binary16                             */

/* Library version (major*10000 + minor*100 + patch).  200 = 0.2.0: added
 * aicomp_kv_set_small_decode_tokens, aicomp_paged_prefill_attn_items and
 * aicomp_paged_prefill_tile_positions; every 0.1 entry point is unchanged. */
int aicomp_kv_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* aicomp_kv_last_error(void);

/*
 * Routing threshold of automatic decode calls (partition_size 0), in tokens: a call with
 * batch * max_blocks_per_seq * block_size at or below it takes the grid schedule (see
 * aicomp_paged_decode_attn), a larger one the balanced schedule; 0 sends every supported shape
 * to the balanced schedule.  Process-wide; the initial value is 32768, or the value of the
 * environment variable AICOMP_KV_SMALL_DECODE_TOKENS at the library's first use of it (the
 * environment is read once, never per call).  Stores `tokens` and returns the previous value; a
 * negative `tokens` only queries.  aicomp_paged_decode_workspace_bytes and
 * aicomp_paged_decode_partition_size answer for the value current at their call, so a caller
 * that changes the threshold asks them again before reusing a cached size.  No counterpart in
 * the reference (which has a single torch call per step, kv_cache.py:397-403); it exists so
 * that a host can pin the schedule without touching the environment.
 */
long long aicomp_kv_set_small_decode_tokens(long long tokens);

/*
 * KV append: scatter T new rows into the pools by slot_mapping.
 * Replaces  key_cache[:, :, position:end_position, :] = new_k   (kv_cache.py:159-160)
 * and       self.cache_k[:, :, self.cache_pos:end_pos, :] = key (kv_cache.py:387-388).
 *
 *   key, value     [T, Hkv, D] of in_dtype; element (t,h,d) is at
 *                  t*kv_token_stride + h*kv_head_stride + d  (strides in elements)
 *   k_pool, v_pool pools of pool_dtype
 *   slot_mapping   [T] int64; slots must be distinct.  A row whose slot is negative (padding)
 *                  or >= num_blocks * block_size (outside the pool) is skipped without an error:
 *                  the library cannot report a per-row fault from a kernel, so a planner that
 *                  wants to hear about such rows checks its slots on the host
 *   in_dtype == pool_dtype                  raw copy, bit-exact (F32, BF16, F16, FP8_E4M3)
 *   in_dtype f32/bf16/f16, pool FP8_E4M3    code = e4m3_rne(clamp(x / scale[h], +-448)),
 *                                           k_scale / v_scale [Hkv] float, required
 */
int aicomp_kv_append(const void* key, const void* value,
                     int64_t kv_token_stride, int64_t kv_head_stride,
                     void* k_pool, void* v_pool, const int64_t* slot_mapping,
                     int64_t num_tokens, int num_kv_heads, int head_dim,
                     int block_size, int64_t num_blocks,
                     int in_dtype, int pool_dtype,
                     const float* k_scale, const float* v_scale,
                     void* stream);

/*
 * Paged decode attention: one query token per sequence, no mask.
 * Replaces the decode branch  F.scaled_dot_product_attention(query, full_key,
 * full_value, attn_mask=None, is_causal=False)   (kv_cache.py:397-403)
 * including the .contiguous() prefix copies it is fed from (kv_cache.py:391-392).
 *
 *   out, query      [B, Hq, D] of q_dtype (F32, BF16 or F16), contiguous; the pools hold
 *                   kv_dtype == q_dtype, or FP8_E4M3 under BF16 / F16 queries
 *   block_table     [B, max_blocks_per_seq] int32, row stride block_table_stride.  Entries are
 *                   trusted to lie in [0, num_blocks); one that does not is clamped into the
 *                   pool (no fault, and no error: the row then attends over another block)
 *   context_lens    [B] int32, tokens to attend to (0 -> the output row is zero); a length
 *                   beyond max_blocks_per_seq * block_size is cut to that
 *   scale           softmax scale (the reference's default is 1/sqrt(D))
 *   kv_dtype FP8    k_scale / v_scale [Hkv] float dequantisation factors, fused
 *                   into the loads.  Accuracy: against attention over the dequantised
 *                   codes the result meets the bf16 tolerance (1e-2 abs or 2e-2 rel);
 *                   against attention over the values BEFORE quantisation (unit-variance
 *                   K and V, absmax scales) the error per output element is at most
 *                   6e-2 abs or 1e-1 rel for rows attending to >= 1024 keys, and at most
 *                   1e-2 + min(0.3, 1.6 / sqrt(n)) for a row of n keys (the format's
 *                   3 mantissa bits; averaging over n keys shrinks it).  The same holds
 *                   for aicomp_paged_prefill_attn over an fp8 pool.
 *   partition_size  split-K (flash-decoding) tokens per partition; 0 = choose
 *                   from the shape (balanced schedule: every wave gets the same
 *                   number of 32-token tiles); a multiple of block_size otherwise.
 *                   Split work is merged by a second kernel from partial
 *                   (max, sum, output) triples.  With 0, a call over few short rows
 *                   (batch * max_blocks_per_seq * block_size at or below the process-wide
 *                   threshold of aicomp_kv_set_small_decode_tokens(), default 32768) runs one workgroup per (row, KV head,
 *                   256-token partition) instead, and no merge kernel at all when
 *                   max_blocks_per_seq * block_size <= 640: such a call is bound by
 *                   launch and memory latency, not by bandwidth.  The result is the
 *                   same to within the tolerance between split sizes (2e-3).
 *   workspace       device scratch of at least
 *                   aicomp_paged_decode_workspace_bytes(...) bytes (may be NULL
 *                   when that returns 0), 16-byte aligned.  Its contents need
 *                   no initialisation (every partial a call merges was written
 *                   by that call) and nothing is kept in it between calls, so
 *                   one allocation serves any number of calls.  Two calls that
 *                   may overlap (different streams) need separate workspaces.
 */
int aicomp_paged_decode_attn(void* out, const void* query,
                             const void* k_pool, const void* v_pool,
                             const int32_t* block_table, int64_t block_table_stride,
                             const int32_t* context_lens,
                             int batch, int num_q_heads, int num_kv_heads, int head_dim,
                             int block_size, int max_blocks_per_seq, int64_t num_blocks,
                             float scale, int q_dtype, int kv_dtype,
                             const float* k_scale, const float* v_scale,
                             int partition_size,
                             void* workspace, size_t workspace_bytes,
                             void* stream);

/*
 * Append of one new token per sequence fused with decode attention: what one decode-step
 * call of the reference operator does (kv_cache.py:383-403: store the new K/V row at the
 * write position, then attend over the whole prefix), in a single main kernel.
 *
 *   new_key, new_value  [B, Hkv, D] of q_dtype, element (b,h,d) at
 *                       b*kv_token_stride + h*kv_head_stride + d; row b becomes token
 *                       context_lens[b] - 1 of sequence b (its slot comes from the block
 *                       table), quantised with k_scale / v_scale for an fp8 pool
 *   context_lens        lengths INCLUDING the new token
 * Everything else as aicomp_paged_decode_attn.  The result equals aicomp_kv_append of those
 * rows followed by aicomp_paged_decode_attn: the pool contents are bit-identical.
 * Row b is stored only if 1 <= context_lens[b] <= max_blocks_per_seq * block_size and its
 * table entry lies in [0, num_blocks); otherwise the pools are left as they are for that
 * sequence (whichever kernel does the append), and its output row is computed from the pool
 * contents under the clamping rules above.
 */
int aicomp_paged_decode_attn_append(void* out, const void* query,
                                    const void* new_key, const void* new_value,
                                    int64_t kv_token_stride, int64_t kv_head_stride,
                                    void* k_pool, void* v_pool,
                                    const int32_t* block_table, int64_t block_table_stride,
                                    const int32_t* context_lens,
                                    int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                    int block_size, int max_blocks_per_seq, int64_t num_blocks,
                                    float scale, int q_dtype, int kv_dtype,
                                    const float* k_scale, const float* v_scale,
                                    int partition_size,
                                    void* workspace, size_t workspace_bytes,
                                    void* stream);

/*
 * aicomp_paged_decode_attn_append for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, results and bit patterns as
 * aicomp_paged_decode_attn_append, without the workspace pair: the split-K partials go to a
 * scratch array of AICOMP_KV_STATIC_SCRATCH_BYTES that is part of the loaded library (every GPU
 * the library runs on holds its own copy until the process ends).  The call allocates, frees and
 * clears nothing (no partial is read that the same call did not write, so nothing has to start
 * at zero).  The first call on a device looks the array's address up (hipGetSymbolAddress); make
 * that call outside graph capture, with the device of the pointers current.
 *
 * A shape whose aicomp_paged_decode_workspace_bytes() exceeds AICOMP_KV_STATIC_SCRATCH_BYTES is
 * refused with AICOMP_KV_EWORKSPACE (32 MiB covers batch 128 at 64 / 8 heads, head_dim 128).
 * All calls on one GPU share that GPU's array: calls that may overlap in time (different
 * streams, or several host threads on one device) race on the partials; serialise them or use
 * aicomp_paged_decode_attn_append with one workspace per stream.
 */
#define AICOMP_KV_STATIC_SCRATCH_BYTES (32u << 20)
int aicomp_paged_decode_attn_append_static(void* out, const void* query,
                                           const void* new_key, const void* new_value,
                                           int64_t kv_token_stride, int64_t kv_head_stride,
                                           void* k_pool, void* v_pool,
                                           const int32_t* block_table, int64_t block_table_stride,
                                           const int32_t* context_lens,
                                           int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                           int block_size, int max_blocks_per_seq, int64_t num_blocks,
                                           float scale, int q_dtype, int kv_dtype,
                                           const float* k_scale, const float* v_scale,
                                           int partition_size, void* stream);

size_t aicomp_paged_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads,
                                           int head_dim, int block_size,
                                           int max_blocks_per_seq, int q_dtype, int kv_dtype,
                                           int partition_size);

/* The partition size the library would pick for partition_size == 0. */
int aicomp_paged_decode_partition_size(int batch, int num_q_heads, int num_kv_heads,
                                       int head_dim, int block_size,
                                       int max_blocks_per_seq, int q_dtype, int kv_dtype);

/*
 * Chunked-prefill causal attention over the paged pool (matrix cores for bf16 and fp16).
 * Replaces the prefill branch  F.scaled_dot_product_attention(query, full_key,
 * full_value, attn_mask=None, is_causal=True)   (kv_cache.py:404-415).
 * The chunk's own K/V rows must already be in the pool (append first).
 *
 *   out, query     [T, Hq, D] of q_dtype, rows of sequence s are cu_q_lens[s]..cu_q_lens[s+1]
 *   context_lens   [S] int32: prior context + chunk length; a sequence whose length is
 *                  smaller than its chunk gets zero output rows (no error)
 *   cu_q_lens      [S+1] int32 prefix sums of the chunk lengths
 *   max_q_len      host-side upper bound of the chunk lengths (sizes the grid)
 * Mask: query i of a chunk with prior context P sees keys j <= P + i
 * (bottom-right aligned; P == 0 is the reference's is_causal=True, a chunk of
 * one token is the reference's decode).
 */
int aicomp_paged_prefill_attn(void* out, const void* query,
                              const void* k_pool, const void* v_pool,
                              const int32_t* block_table, int64_t block_table_stride,
                              const int32_t* context_lens, const int32_t* cu_q_lens,
                              int num_seqs, int64_t total_q, int max_q_len,
                              int num_q_heads, int num_kv_heads, int head_dim,
                              int block_size, int max_blocks_per_seq, int64_t num_blocks,
                              float scale, int q_dtype, int kv_dtype,
                              const float* k_scale, const float* v_scale,
                              void* stream);

/*
 * The same call with the order of the work given by the caller.  A prefill launch is one
 * workgroup row per (sequence, query tile); tiles differ several-fold in cost (a tile costs as many
 * steps as its last row has keys), and a host that plans the step knows every length, which the
 * library, holding device pointers only, does not.  `items` is a DEVICE array of num_items
 * (sequence, query tile) int32 pairs: workgroup row i takes pair i, so the list should name every
 * tile that has rows exactly once (a tile that is left out is not computed; a pair that names no
 * sequence or a tile beyond its chunk is skipped), most expensive first.  A query tile is
 * aicomp_paged_prefill_tile_positions(...) consecutive positions of a chunk (tile q of a chunk
 * holds its positions q * that .. ); when that returns 0 for the shapes at hand no kernel takes a
 * list and the call behaves like aicomp_paged_prefill_attn (also with a list longer than 65535).
 * Measured on ragged batches (32 chunks of 8 to 512 tokens over prior contexts up to 2048): 135 us
 * against 237 us in grid order.  No counterpart in the reference, which issues one prefill per
 * call (kv_cache.py:404-415); it is for step planners (continuous batching).
 */
int aicomp_paged_prefill_attn_items(void* out, const void* query,
                                    const void* k_pool, const void* v_pool,
                                    const int32_t* block_table, int64_t block_table_stride,
                                    const int32_t* context_lens, const int32_t* cu_q_lens,
                                    int num_seqs, int64_t total_q, int max_q_len,
                                    int num_q_heads, int num_kv_heads, int head_dim,
                                    int block_size, int max_blocks_per_seq, int64_t num_blocks,
                                    float scale, int q_dtype, int kv_dtype,
                                    const float* k_scale, const float* v_scale,
                                    const int32_t* items, int num_items, void* stream);

/* Positions per query tile of the kernel a prefill call with these shapes runs on (0: none that takes an item list). */
int aicomp_paged_prefill_tile_positions(int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                                        int q_dtype, int kv_dtype, int max_q_len);

/*
 * Rotary position embedding of Q and K fused with the KV append: one launch for
 *   q_embed = (q * cos) + (rotate_half(q) * sin)
 *   k_embed = (k * cos) + (rotate_half(k) * sin)   (compiler_fx/modeling_llama.py:200-231,
 *                                                   call site :582)
 * and the append of k_embed / value                (kv_cache.py:387-388), with the KV heads
 * stored once instead of repeat_kv's G copies      (modeling_llama.py:268-277, :589-590).
 *
 *   q_in, q_out     [T, Hq, D] of in_dtype (F32, BF16 or F16); element (t,h,d) at
 *                   t*token_stride + h*head_stride + d of the respective stride pair;
 *                   q_out may be q_in (in place)
 *   key, value      [T, Hkv, D] of in_dtype, strides as in aicomp_kv_append (the three inputs
 *                   may be slices of one fused QKV projection output)
 *   cos, sin        tables of in_dtype, row r at r*table_stride, D columns each (the
 *                   reference's cos/sin, cast to the tensor type: modeling_llama.py:150-168)
 *   positions       [T] int64 table row of each token, or NULL: token t uses row t (the
 *                   per-call cos/sin the reference passes as position_embeddings)
 *   table_rows      rows in the tables; a token whose position is outside is left alone
 *   slot_mapping    [T] int64 as in aicomp_kv_append (slot < 0: Q is still rotated, K/V of
 *                   that token are not stored)
 *   pool_dtype      in_dtype (K rotated, V copied raw) or FP8_E4M3 (both quantised like
 *                   aicomp_kv_append, K after the rotation)
 * Every product and the sum are rounded to in_dtype one after the other, without fused
 * multiply-add: bit-identical to the reference's eager evaluation.  D % 16 == 0; pointers
 * and strides 16-byte aligned.
 */
int aicomp_rope_kv_append(const void* q_in, void* q_out,
                          int64_t q_token_stride, int64_t q_head_stride,
                          int64_t qo_token_stride, int64_t qo_head_stride,
                          const void* key, const void* value,
                          int64_t kv_token_stride, int64_t kv_head_stride,
                          const void* cos, const void* sin, int64_t table_stride,
                          int64_t table_rows, const int64_t* positions,
                          void* k_pool, void* v_pool, const int64_t* slot_mapping,
                          int64_t num_tokens, int num_q_heads, int num_kv_heads, int head_dim,
                          int block_size, int64_t num_blocks, int in_dtype, int pool_dtype,
                          const float* k_scale, const float* v_scale, void* stream);

/*
 * Token sampling, one launch per batch of rows.  Replaces _sample_token
 * (opt_prime/opt_prime/inference.py:786-843): greedy argmax (:806-808), or
 * logits / temperature (:811-812), top-k (:815-818: entries below the k-th largest value are
 * removed, ties at that value stay), top-p (:821-837: in descending order an entry stays while
 * the mass before it is <= top_p; the first always stays; mass = softmax of what top-k left),
 * then a draw from the softmax of what is left (:840-841).
 *
 *   out           [B] int64 token ids
 *   logits        [B, V] F32, BF16 or F16, row b at b*row_stride elements; not modified
 *   uniforms      [B] float in [0, 1): the draw is the inverse CDF in index order at
 *                 uniforms[b] (the reference draws with torch.multinomial; the distribution is
 *                 the same, the random stream is the caller's).  Not read when greedy.
 *   probs_out     optional [B, V] float: the distribution the draw is made from
 *   temperature   > 0 (ignored when greedy);  top_k <= 0 or >= V: off;  top_p >= 1: off
 *   greedy        non-zero: argmax, lowest index among equal maxima
 * Ties at the nucleus threshold are kept in index order.  Probability mass is summed exactly
 * in 2^-40 fixed point, so a call is reproducible bit for bit.
 */
int aicomp_sample_tokens(int64_t* out, const void* logits, int64_t row_stride,
                         float* probs_out, const float* uniforms,
                         int batch, int vocab, float temperature, int top_k, float top_p,
                         int greedy, int logits_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AICOMP_KV_H */
