/*
 * xlite_hip.h — C ABI of the MI355X (gfx950) attention hot path.
 *
 * Every entry point replaces one host launcher of the Xlite runtime
 * (xlite/csrc/op.h) together with the device kernel it starts. Arguments are
 * plain device pointers and scalars: no framework types cross this boundary.
 *
 * Conventions
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream). Work
 *     is enqueued on it and the call returns without synchronising.
 *   - Every function returns XLITE_HIP_OK (0) or a negative XLITE_HIP_E* code;
 *     xlite_hip_last_error() then holds a message for the calling thread.
 *   - All tensors are dense row-major ("contiguous"); index tensors are int32
 *     except `position`, which is int64 (xlite/csrc/kernels/rope_and_cache.h:452).
 *   - `dtype` selects the 16-bit element type of activations and caches.
 */
#ifndef XLITE_HIP_H_
#define XLITE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XLITE_HIP_OK 0
#define XLITE_HIP_EINVAL (-1)   /* bad argument / unsupported combination */
#define XLITE_HIP_ERUNTIME (-2) /* HIP runtime reported an error */
#define XLITE_HIP_ENOSPC (-3)   /* workspace too small */

/* element types (same order as xlite/csrc/base.h XDtype FP16/BF16) */
#define XLITE_HIP_FP16 0
#define XLITE_HIP_BF16 1
/* KV cache element types: the activation dtype, or int8 / fp8 (OCP e4m3) with fp32 scales */
#define XLITE_HIP_KV_SAME 0
#define XLITE_HIP_KV_INT8 1
#define XLITE_HIP_KV_FP8 2

/* Message of the last failed call on this thread ("" if none). */
const char *xlite_hip_last_error(void);

/* Library / device probe: returns the ABI version, fills optional outputs. */
int xlite_hip_version(void);
int xlite_hip_device_info(int device, int *num_cu, int *lds_bytes_per_cu, char *arch, size_t arch_len);

/* ------------------------------------------------------------------------
 * rope_and_cache — replaces XliteOpRopeCache (xlite/csrc/op.cpp:905-943) +
 * kernel rope_and_cache<Dtype> (xlite/csrc/kernels/rope_and_cache.h:206-610).
 *
 * inout      [num_tokens, (n_heads + 2*n_kv_heads) * head_dim]  q | k | v, updated in place
 * k_cache    [num_blocks, block_size, n_kv_heads, head_dim]
 * v_cache    same shape
 * position   [num_tokens] int64, or [3, num_tokens] when an mrope mask is non-zero
 * cosin      [max_pos, rot_dim]  row = cos(rot_dim/2) | sin(rot_dim/2), in `dtype`
 * slot_mapping [num_tokens] int32, slot = block * block_size + offset (used unsigned)
 * NeoX (half-split) rotation only; q is additionally scaled by 1/sqrt(head_dim).
 * ---------------------------------------------------------------------- */
int xlite_hip_rope_and_cache(void *stream, void *inout, void *k_cache, void *v_cache,
                             const int64_t *position, const void *cosin,
                             const int32_t *slot_mapping, uint32_t num_tokens, uint32_t n_heads,
                             uint32_t n_kv_heads, uint32_t head_dim, uint32_t rot_dim,
                             uint32_t block_size, int is_neox, uint64_t mrope_mask_h,
                             uint64_t mrope_mask_w, int dtype);

/* ------------------------------------------------------------------------
 * attention — replaces XliteOpAttention and XliteOpFlashAttention
 * (xlite/csrc/op.cpp:945-993) + kernels attention.h / flash_attention.h.
 *
 * qkv         [total_tokens, (n_heads + 2*n_kv_heads) * head_dim]; only q is read,
 *             already rotated and scaled by rope_and_cache
 * k_cache/v_cache  paged caches as above; when kv_dtype is XLITE_HIP_KV_INT8 or
 *             XLITE_HIP_KV_FP8 they hold one byte per element and k_scale/v_scale
 *             [num_blocks, block_size, n_kv_heads] fp32 hold the per-token-per-head scales
 *             (x = q * scale). Decode batches of the streaming kernel's shapes (at most 16
 *             query heads per kv head, block size a multiple of 16) read the bytes directly,
 *             and so do multi-row batches of head_dim 128 (block size a multiple of 8) whose
 *             chunks are short (up to 2048 query rows x heads of the group per sequence on
 *             average) or whose workspace is too small for what follows;
 *             every other batch over a quantised cache (long prefill chunks, other decode
 *             shapes, head_dim 64) first copies the blocks it can see into a 16-bit
 *             cache in the workspace, which xlite_hip_attention_workspace_bytes_kv() sizes:
 *             2 tensors x batch x max_num_block x block_size x n_kv_heads x head_dim x 2 bytes
 *             (every block the tables can name, whatever the sequences' lengths: keep
 *             max_num_block close to what the batch needs). Same results either way.
 * output      [total_tokens, n_heads * head_dim]
 * query_start_loc, lens, cached_lens  [batch] int32
 * block_tables [batch * max_num_block] int32
 * Row r of sequence i attends to cache positions 0 .. cached_lens[i] + r.
 * No softmax scale is applied here (q arrives pre-scaled).
 * head_dim 64, 128 or 256 (the reference kernel is generic over headSize,
 * xlite/csrc/kernels/attention.h:39-74; 256 is its Qwen3.5 shape); quantised caches: 64 or 128.
 *
 * workspace   device scratch of at least xlite_hip_attention_workspace_bytes()
 *             (or ..._bytes_kv() for a quantised cache; split-KV partial results;
 *             contents need no initialisation and are not preserved). Decode batches
 *             need all of it, and so do batches over a quantised cache that go through
 *             the 16-bit copy and have no other way (XLITE_HIP_ENOSPC otherwise); a
 *             prefill batch given less, or NULL, still works but does not split the KV
 *             axis (head_dim 128 over a quantised cache included: it is then read directly).
 * ---------------------------------------------------------------------- */

size_t xlite_hip_attention_workspace_bytes(uint32_t total_tokens, uint32_t n_heads,
                                           uint32_t n_kv_heads, uint32_t head_dim,
                                           uint32_t block_size, uint32_t batch,
                                           uint32_t max_num_block);
/* the same for a given cache element type (the call above is kv_dtype = XLITE_HIP_KV_SAME) */
size_t xlite_hip_attention_workspace_bytes_kv(uint32_t total_tokens, uint32_t n_heads,
                                              uint32_t n_kv_heads, uint32_t head_dim,
                                              uint32_t block_size, uint32_t batch,
                                              uint32_t max_num_block, int kv_dtype);

int xlite_hip_attention(void *stream, const void *qkv, const void *k_cache, const void *v_cache,
                        void *output, const int32_t *query_start_loc, const int32_t *lens,
                        const int32_t *cached_lens, const int32_t *block_tables,
                        uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                        uint32_t head_dim, uint32_t block_size, uint32_t batch,
                        uint32_t max_num_block, int dtype, int kv_dtype, const float *k_scale,
                        const float *v_scale, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Instrumentation (no counterpart in the reference). device_words: four 64-bit words in
 * device memory, or NULL (off, the default). While set, workgroup 0 of every launch of the
 * streaming MLA kernel and of the streaming prefill kernel stores
 *   { shader clock counter at entry, 100 MHz wall clock at entry,
 *     shader clock counter behind its loop, 100 MHz wall clock there }
 * so that (w[2] - w[0]) / ((w[3] - w[1]) * 10 ns) is the clock the kernel ran at: the part is
 * power-managed, and the matrix peak is quoted at a clock these kernels do not hold.
 * Process-wide; the buffer must stay valid until the probe is set to NULL again.
 * ---------------------------------------------------------------------- */
int xlite_hip_set_clock_probe(void *device_words);

/* ------------------------------------------------------------------------
 * decode_step — the attention block of one layer as the reference's model loop runs it
 * (xlite/csrc/model.cpp:544-571: XliteOpRopeCache, then XliteOpAttention or
 * XliteOpFlashAttention over the same qkv rows and caches), enqueued from one call:
 * xlite_hip_rope_and_cache followed by xlite_hip_attention with the arguments of the
 * two (16-bit caches), same results bit for bit. For serving loops whose small batches
 * are bound by the cost of a call, not of the kernels. Any batch the two accept, not
 * only decode rows. A decode batch whose contexts are short by the width of its block
 * tables (the batches the decode kernel serves a whole row per workgroup, without a merge
 * launch) is a single kernel launch: the workgroup of a sequence rotates and stores the
 * sequence's rows, then walks them.
 * ---------------------------------------------------------------------- */
int xlite_hip_decode_step(void *stream, void *qkv, void *k_cache, void *v_cache, void *output,
                          const int64_t *position, const void *cosin, const int32_t *slot_mapping,
                          const int32_t *query_start_loc, const int32_t *lens,
                          const int32_t *cached_lens, const int32_t *block_tables,
                          uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                          uint32_t head_dim, uint32_t rot_dim, uint32_t block_size, uint32_t batch,
                          uint32_t max_num_block, int is_neox, uint64_t mrope_mask_h,
                          uint64_t mrope_mask_w, int dtype, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * mla_attention — replaces XliteOpMLAV2 / XliteOpFlashMLAV2
 * (xlite/csrc/op.cpp:995-1058) + kernels mla_v2.h / flash_mla_v2.h: the absorbed
 * MLA attention between the two einsums of the mla_v2 operator.
 *
 * q_absorb  [total_tokens, n_heads, kv_lora_rank]
 * qr        [total_tokens, n_heads, rope_head_dim]
 * k_cache   [num_blocks, block_size, kv_lora_rank]   (latent)
 * pe_cache  [num_blocks, block_size, rope_head_dim]  (rotated key slice)
 * o_absorb  [total_tokens, n_heads, kv_lora_rank]
 * scores = (q_absorb . k + qr . pe) * scale, causal as in attention.
 * topk_indices [total_tokens, top_k] int32 (top_k == 0: dense, pointer unused):
 * when top_k > 0 a row whose causal range is longer than top_k attends only to the
 * listed positions (ascending; entries outside the range, negative ones and repeats of
 * the predecessor are ignored); shorter rows see their whole range
 * (xlite/csrc/kernels/mla_v2.h:697-699). The workspace size depends on top_k: pass the
 * call's value to xlite_hip_mla_workspace_bytes. bf16 only (xlite/csrc/op.cpp:1014).
 * Any block size (kv_lora_rank 512 with rope_head_dim 64: the streaming kernel; other
 * sizes: a plain kernel).
 * workspace: at least xlite_hip_mla_workspace_bytes() for the same shape (required:
 * XLITE_HIP_ENOSPC otherwise; split-KV partials, no initialisation needed).
 * ---------------------------------------------------------------------- */
size_t xlite_hip_mla_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t kv_lora_rank,
                                     uint32_t rope_head_dim, uint32_t block_size, uint32_t batch,
                                     uint32_t max_num_blocks, uint32_t top_k);

int xlite_hip_mla_attention(void *stream, const void *q_absorb, const void *qr,
                            const void *k_cache, const void *pe_cache, void *o_absorb,
                            const int32_t *query_start_loc, const int32_t *lens,
                            const int32_t *cached_lens, const int32_t *block_tables,
                            uint32_t total_tokens, uint32_t n_heads, uint32_t rope_head_dim,
                            uint32_t kv_lora_rank, uint32_t block_size, uint32_t batch,
                            uint32_t max_num_blocks, float scale, const int32_t *topk_indices,
                            uint32_t top_k, int dtype, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * mla_v3 — replaces XliteOpMLAV3 (xlite/csrc/op.cpp:1086-1104) + kernel mla_v3.h:
 * absorbed MLA attention over a contiguous per-sequence cache
 * k_dense [batch, index_topk, kv_lora_rank], pe_dense [batch, index_topk, rope_head_dim];
 * every query row of sequence i attends to the first
 * min(cached_lens[i] + lens[i], index_topk) entries, no causal structure.
 * ---------------------------------------------------------------------- */
int xlite_hip_mla_v3(void *stream, const void *q_absorb, const void *qr, const void *k_dense,
                     const void *pe_dense, void *o_absorb, const int32_t *query_start_loc,
                     const int32_t *lens, const int32_t *cached_lens, uint32_t total_tokens,
                     uint32_t n_heads, uint32_t rope_head_dim, uint32_t kv_lora_rank,
                     uint32_t batch, uint32_t index_topk, float scale, int dtype, void *workspace,
                     size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * qk_rms_norm — replaces XliteOpQkRmsNorm (xlite/csrc/op.cpp:1177-1203) + kernel
 * qk_rms_norm.h:32-54 in its normalising mode without pre-reduced variances (the
 * call of xlite/csrc/model.cpp:516-519): for every row of `in` [num_tokens, row_elems],
 * RMSNorm of q_cnt_per_token vectors of q_norm_dim elements from column 0 with weight
 * q_norm [q_norm_dim] (+ q_norm_bias or NULL), and of k_cnt_per_token vectors of
 * k_norm_dim elements from column k_start_offset with k_norm (+ k_norm_bias or NULL):
 * y = x * rsqrt(mean(x^2) + eps) * w + b in fp32. Results go to the same columns of
 * `out` (same row pitch; may be `in`); other columns are not written.
 * ---------------------------------------------------------------------- */
int xlite_hip_qk_rms_norm(void *stream, const void *in, void *out, const void *q_norm,
                          const void *q_norm_bias, const void *k_norm, const void *k_norm_bias,
                          uint32_t num_tokens, uint32_t row_elems, uint32_t q_norm_dim,
                          uint32_t q_cnt_per_token, uint32_t k_norm_dim, uint32_t k_cnt_per_token,
                          uint32_t k_start_offset, float norm_eps, int dtype);

/* ------------------------------------------------------------------------
 * layernorm — replaces XliteOpLayerNorm (xlite/csrc/op.cpp:607-628) as bound by
 * `layernorm` (xlite/csrc/_C.cpp:1122-1133): LayerNorm with weight and bias over the
 * first norm_dim columns of every row, fp32 arithmetic, biased variance, one rounding;
 * rows of `in` are in_stride elements apart, rows of `out` out_stride (`out` may be `in`).
 * In the MLA layer it normalises the index key (xlite/csrc/model.cpp:291-292).
 * ---------------------------------------------------------------------- */
int xlite_hip_layernorm(void *stream, const void *in, const void *norm, const void *norm_bias, void *out,
                        uint32_t num_rows, uint32_t in_stride, uint32_t out_stride, uint32_t norm_dim,
                        float norm_eps, int dtype);

/* ------------------------------------------------------------------------
 * muls — replaces XliteOpMuls (xlite/csrc/op.cpp:1644-1680), bound as `muls`
 * (xlite/csrc/_C.cpp:1660-1667): output[r][calc_offset + i] = input[r][calc_offset + i] * scale
 * for i < calc_num (clipped to the row), fp32 product rounded once; other columns are not
 * written. The MLA layer scales the indexer's head weights with it (xlite/csrc/model.cpp:316).
 * ---------------------------------------------------------------------- */
int xlite_hip_muls(void *stream, const void *input, void *output, uint32_t num_rows, uint32_t row_len,
                   uint32_t calc_offset, uint32_t calc_num, float scale, int dtype);

/* ------------------------------------------------------------------------
 * rope_complex_and_cache — the general form of the interleaved-pair rope kernel
 * (xlite/csrc/kernels/rope_complex_and_cache.h:12-241) behind XliteOpRopeComplex
 * (xlite/csrc/op.cpp:1106-1126) and XliteOpRopeComplexAndCache (:1128-1150).
 * Of every head's step_dim columns the rope_dim columns from `offset` are rotated by
 * freqs[position[t]] (fp32 cos, sin pairs) and leave de-interleaved [re... | im...].
 *  cache == NULL: written to output[t][head * out_step_dim + out_offset ...]; `output`
 *    may be `input` (the in-place call on the indexer's query, xlite/csrc/model.cpp:311-313);
 *  cache != NULL (one head, block_size > 0): the vdim columns from `offset` - the rotated
 *    ones, then the rest unchanged - go to cache[slot / block_size][slot % block_size]
 *    ([num_blocks, block_size, vdim]) and nothing else is written (the index key cache,
 *    xlite/csrc/model.cpp:295-297).
 * xlite_hip_rope_complex is the case offset = step_dim - rope_dim, out_step_dim = rope_dim.
 * ---------------------------------------------------------------------- */
int xlite_hip_rope_complex_and_cache(void *stream, uint32_t num_tokens, uint32_t n_local_heads,
                                     uint32_t step_dim, uint32_t rope_dim, uint32_t offset, uint32_t vdim,
                                     const void *input, void *output, uint32_t out_step_dim,
                                     uint32_t out_offset, const float *freqs, const int64_t *position,
                                     uint32_t block_size, void *cache, const int32_t *slot_mapping, int dtype);

/* ------------------------------------------------------------------------
 * gather_sparse_kv_cache — replaces XliteOpGatherSparseKVCache
 * (xlite/csrc/op.cpp:1060-1084) + kernel gather_sparse_kv_cache.h:15-134.
 * dense[b, i] = paged[block_tables[b*max_num_blocks + tok / block_size], tok % block_size]
 * with tok = topk_indices[b, i], for i < min(query_lens[b] + cached_lens[b], index_topk).
 * Other dense slots are left untouched. kv_heads must be 1.
 * ---------------------------------------------------------------------- */
int xlite_hip_gather_sparse_kv_cache(void *stream, const void *k_cache, const void *pe_cache,
                                     const int32_t *block_tables, const int32_t *topk_indices,
                                     const int32_t *query_lens, const int32_t *cached_lens,
                                     void *k_dense, void *pe_dense, uint32_t batch,
                                     uint32_t index_topk, uint32_t block_size,
                                     uint32_t max_num_blocks, uint32_t kv_lora_rank,
                                     uint32_t rope_head_dim, uint32_t kv_heads, int dtype);

/* ------------------------------------------------------------------------
 * rope_complex — replaces XliteOpRopeComplex (xlite/csrc/op.cpp:1106-1126) +
 * kernel rope_complex_and_cache.h:12-241 in its "no cache" mode.
 * input  [num_tokens, n_local_heads, step_dim]; the last rope_dim elements of each
 *        head are interleaved (re, im) pairs
 * freqs  [max_pos, rope_dim/2] complex64 == interleaved fp32 (cos, sin)
 * output [num_tokens, n_local_heads, rope_dim] = [re... | im...] of x * freqs[position]
 * ---------------------------------------------------------------------- */
int xlite_hip_rope_complex(void *stream, uint32_t num_tokens, uint32_t n_local_heads,
                           uint32_t step_dim, uint32_t rope_dim, const void *input,
                           const float *freqs, const int64_t *position, void *output, int dtype);

/* ------------------------------------------------------------------------
 * mla_prepare — replaces XliteOpMlaPrepare (xlite/csrc/op.cpp:1151-1175) +
 * kernel mla_prepare.h:14-39 (two RMSNorms + rope_complex_and_cache).
 * attn_qkvc [num_tokens, q_lora_rank + kv_lora_rank + rope_head_dim]; the rope slice
 * is rotated in place. attn_norm_qc / attn_norm_kvc receive rms(x)*w + b of the first
 * two slices; the latter is also written to k_cache[slot], the rotated slice to
 * pe_cache[slot]. block_size == 0 disables both cache writes.
 * ---------------------------------------------------------------------- */
int xlite_hip_mla_prepare(void *stream, void *attn_qkvc, const void *q_norm,
                          const void *q_norm_bias, void *attn_norm_qc, const void *kv_norm,
                          const void *kv_norm_bias, void *attn_norm_kvc, const float *freqs,
                          const int64_t *position, uint32_t num_tokens, uint32_t q_lora_rank,
                          uint32_t kv_lora_rank, uint32_t rope_head_dim, uint32_t block_size,
                          void *k_cache, void *pe_cache, const int32_t *slot_mapping,
                          float norm_eps, int dtype);

/* ------------------------------------------------------------------------
 * einsum_mht_htd_mhd / einsum_mht_hdt_mhd — replace XliteOpEinsumMhtHtdMhd /
 * XliteOpEinsumMhtHdtMhd (xlite/csrc/op.cpp:1872-1918).
 * mhd[m, h, :d] = sum_t mht[m, h, t] * w[h, t, d]   (w_is_hdt == 0, w = [h, t, d])
 *                                   * w[h, d, t]   (w_is_hdt != 0, w = [h, d, t])
 * `t_stride` is the distance in elements between consecutive heads of mht
 * (>= t; the mla_v2 operator reads the first `nope` of each [nope + rope] head).
 * ---------------------------------------------------------------------- */
int xlite_hip_einsum_mht_mhd(void *stream, const void *mht, const void *w, void *mhd, uint32_t m,
                             uint32_t h, uint32_t t, uint32_t d, uint32_t t_stride, int w_is_hdt,
                             int dtype);

/* ------------------------------------------------------------------------
 * get_tile_size_of_cached_kv — replaces GetTileSizeOfCachedKV
 * (xlite/csrc/auto_tuner.cpp:163-210). Host-only, same integer results.
 * Returns the tile size, or a negative error code.
 * ---------------------------------------------------------------------- */
int xlite_hip_get_tile_size_of_cached_kv(const uint32_t *cached_lens, const uint32_t *query_lens,
                                         uint32_t batch, uint32_t head_num_in_group,
                                         uint32_t n_kv_heads, uint32_t block_size,
                                         uint32_t aic_num);

/* ------------------------------------------------------------------------
 * prepare_attn — replaces the host part of XRuntime::PrepareAttn
 * (xlite/csrc/runtime.cpp:404-550): from per-sequence lens / cached_lens and a
 * ragged block table (block_table_rows[i] points at row_lens[i] int32 entries)
 * fill query_start_loc[batch], position[sum lens], slot_mapping[sum lens] and the
 * dense block table [batch, *max_num_blocks]. Host memory only. Outputs must be
 * large enough (dense_tables: batch * ceil(max(lens+cached)/block_size)).
 * `is_decode` is set to 1 when every len == 1.
 * ---------------------------------------------------------------------- */
int xlite_hip_prepare_attn(const uint32_t *lens, const uint32_t *cached_lens, uint32_t batch,
                           const int32_t *const *block_table_rows, const uint32_t *row_lens,
                           uint32_t block_size, int32_t *query_start_loc, int64_t *position,
                           int32_t *slot_mapping, int32_t *dense_tables, size_t dense_capacity,
                           uint32_t *max_num_blocks, uint32_t *batched_tokens, int *is_decode);

/* ------------------------------------------------------------------------
 * indexer_scores — replaces XliteOpIndexerScores and kernel
 * xlite/csrc/kernels/indexer_scores.h:14-290 (API xlite/_C.pyi:1946-1983).
 * q       [total_tokens, n_heads, head_dim]
 * k_cache [num_blocks, block_size, head_dim] (one key head)
 * weight  [total_tokens, head_dim + n_heads]; the last n_heads columns weigh the heads
 * scores  [total_tokens, max_num_block * block_size]; row t gets
 *         scores[t][j] = sum_h weight[t][head_dim + h] * round16(q[t][h] . k[j])
 *         for j < cached_lens[i] + lens[i] of the sequence i that owns row t (no causal limit
 *         inside the sequence); the rest of the row is left untouched.
 * head_dim must be 128, n_heads 16, 32, 64 or 128.
 * ---------------------------------------------------------------------- */
int xlite_hip_indexer_scores(void *stream, const void *q, const void *k_cache, const void *weight,
                             void *scores, const int32_t *query_start_loc, const int32_t *lens,
                             const int32_t *cached_lens, const int32_t *block_tables,
                             uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                             uint32_t block_size, uint32_t batch, uint32_t max_num_block, int dtype);

/* ------------------------------------------------------------------------
 * indexer_topk — replaces XliteOpIndexerTopk and kernel
 * xlite/csrc/kernels/indexer_topk.h:14-660 (API xlite/_C.pyi:1985-2040): the scores
 * above, then for every row the top_k positions by score.
 * indices      [max_num_block * block_size] int32, the value reported for each position
 *              (the caller fills it with 0, 1, 2, ...)
 * topk_indices [total_tokens, top_k] int32: the first min(top_k, cached + query length)
 *              entries of a row are written, in ascending position order (the reference
 *              leaves the order unspecified; its test compares sets); ties at the k-th
 *              score go to the lower positions. top_k <= 2048.
 * workspace: xlite_hip_indexer_topk_workspace_bytes (the 16-bit score rows).
 * ---------------------------------------------------------------------- */
size_t xlite_hip_indexer_topk_workspace_bytes(uint32_t total_tokens, uint32_t block_size,
                                              uint32_t max_num_block);
int xlite_hip_indexer_topk(void *stream, const void *q, const void *k_cache, const void *weight,
                           const int32_t *indices, int32_t *topk_indices,
                           const int32_t *query_start_loc, const int32_t *lens,
                           const int32_t *cached_lens, const int32_t *block_tables,
                           uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                           uint32_t block_size, uint32_t batch, uint32_t max_num_block,
                           uint32_t top_k, int dtype, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Quantised KV caches (no counterpart in the reference, whose caches are always the
 * activation dtype). One fp32 scale per (token, kv head) row of head_dim elements:
 *   XLITE_HIP_KV_INT8: scale = absmax / 127, q = clamp(rint(x / scale), -127, 127)
 *   XLITE_HIP_KV_FP8:  scale = absmax / 448, q = e4m3(x / scale), OCP e4m3, round to nearest even
 * and x = q * scale. A row of zeros gets scale 0.
 * quantize_kv: rows of `src` [rows, head_dim] (16-bit) into `dst` (one byte per element) and
 * `scales` [rows]. quantize_kv_int8 is the same with kv_dtype = XLITE_HIP_KV_INT8.
 * ---------------------------------------------------------------------- */
int xlite_hip_quantize_kv(void *stream, const void *src, void *dst, float *scales, uint64_t rows,
                          uint32_t head_dim, int dtype, int kv_dtype);
int xlite_hip_quantize_kv_int8(void *stream, const void *src, int8_t *dst, float *scales,
                               uint64_t rows, uint32_t head_dim, int dtype);

/* ------------------------------------------------------------------------
 * rope_and_cache with quantise-on-write (no counterpart in the reference; the write it extends
 * is xlite/csrc/kernels/rope_and_cache.h:486-501, :563-564): the same rotation and q scaling as
 * xlite_hip_rope_and_cache, in place; the rotated K rows and the V rows go to
 * k_cache / v_cache [num_blocks, block_size, n_kv_heads, head_dim] (one byte per element) as the
 * quantisation above of the 16-bit rows, with k_scale / v_scale [num_blocks, block_size,
 * n_kv_heads] fp32, at the tokens' slots. One kernel launch for heads of at most 16 items
 * (head_dim / 8 - rot_dim / 16 <= 16); wider heads take a second, quantising launch.
 * rope_and_cache_int8 is the same with kv_dtype = XLITE_HIP_KV_INT8.
 * ---------------------------------------------------------------------- */
int xlite_hip_rope_and_cache_quant(void *stream, void *inout, void *k_cache, void *v_cache,
                                   float *k_scale, float *v_scale, const int64_t *position,
                                   const void *cosin, const int32_t *slot_mapping, uint32_t num_tokens,
                                   uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                   uint32_t rot_dim, uint32_t block_size, int is_neox,
                                   uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype, int kv_dtype);
int xlite_hip_rope_and_cache_int8(void *stream, void *inout, int8_t *k_cache, int8_t *v_cache,
                                  float *k_scale, float *v_scale, const int64_t *position,
                                  const void *cosin, const int32_t *slot_mapping, uint32_t num_tokens,
                                  uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                  uint32_t rot_dim, uint32_t block_size, int is_neox,
                                  uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype);

/* ------------------------------------------------------------------------
 * attention_noalloc - xlite_hip_attention for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid it). It has no
 * counterpart in the reference, whose operators draw scratch from the Runtime's tensor pool.
 * Same arguments and results as xlite_hip_attention without the workspace: the split-KV
 * partial results go to a buffer of XLITE_HIP_NOALLOC_SCRATCH_BYTES that is part of the
 * library's device image (one copy per GPU, held until the process ends). The call
 * allocates and frees nothing. A shape whose xlite_hip_attention_workspace_bytes() exceeds
 * the buffer is refused with XLITE_HIP_ENOSPC. Every call on a GPU shares that GPU's
 * buffer: calls that overlap on one GPU (two streams, two threads) race on it.
 * ---------------------------------------------------------------------- */
#define XLITE_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t xlite_hip_attention_noalloc_scratch_bytes(void);
int xlite_hip_attention_noalloc(void *stream, const void *qkv, const void *k_cache, const void *v_cache,
                                void *output, const int32_t *query_start_loc, const int32_t *lens,
                                const int32_t *cached_lens, const int32_t *block_tables,
                                uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                                uint32_t head_dim, uint32_t block_size, uint32_t batch,
                                uint32_t max_num_block, int dtype, int kv_dtype, const float *k_scale,
                                const float *v_scale);

#ifdef __cplusplus
}
#endif
#endif /* XLITE_HIP_H_ */
