// Argument bundles and launcher declarations shared by the attention entry points.
#pragma once

#include "common.h"

namespace xlite {

struct AttentionArgs {
    const void *qkv;
    const void *k_cache;
    const void *v_cache;
    void *output;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;
    uint32_t total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block;
    int dtype, kv_dtype;
    const float *k_scale;
    const float *v_scale;
    void *workspace;
    size_t workspace_bytes;
    // a batch served by two kernels: kOnlySingle = only the sequences with exactly one query row (the decode
    // kernels), kSkipSingle = all the others (the prefill kernel, the dequantising copy)
    int rows_mode;
    // a bf16 model over the fp16 copy of a quantised cache, on a kernel that converts at its edges: dtype says
    // FP16 (the products), qkv and output are bf16
    bool io_bf16;
};
enum { kAllRows = 0, kOnlySingle = 1, kSkipSingle = 2 };

struct MlaArgs {
    const void *q_absorb;
    const void *qr;
    const void *k_cache;     // paged [blocks, block_size, kv_lora_rank] or dense [batch, index_topk, ...]
    const void *pe_cache;
    void *o_absorb;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;   // nullptr: dense per-sequence cache (mla_v3)
    uint32_t total_tokens, n_heads, rope_head_dim, kv_lora_rank, block_size, batch, max_num_blocks;
    uint32_t dense_len;            // mla_v3: entries per sequence, attention is not causal
    float scale;
    const int32_t *topk_indices;
    uint32_t top_k;
    int dtype;
    void *workspace;
    size_t workspace_bytes;
};

// merge.hip: scratch for split-KV partial results and their merge.
// Layout of the workspace: cnt[rows * n_heads] int32 (number of partials of a (row, head); 0 = the
// producer stored the final value itself), then acc[rows * n_heads][max_slots][dv] and
// ml[rows * n_heads][max_slots][2] (running maximum in the log2 domain, sum) in fp32.
struct PartialBuffers {
    int32_t *cnt;
    float *acc;
    float *ml;
};
size_t partial_bytes(uint32_t rows, uint32_t n_heads, uint32_t dv, uint32_t max_slots);
PartialBuffers carve_partials(void *workspace, uint32_t rows, uint32_t n_heads, uint32_t dv, uint32_t max_slots);
int launch_merge(hipStream_t stream, int dtype, void *out, const PartialBuffers &b, uint32_t rows,
                 uint32_t n_heads, uint32_t dv, uint32_t max_slots);
// Partials of the MLA decode kernel: a row's s-th segment sits in slot 2 c0 + (1 - first flag) for s = 0 and
// 2 (c0 + s) after that (meta = segments, c0, first flag per row); acc holds O / l in the 16-bit activation type.
int launch_merge_mla(hipStream_t stream, int dtype, void *out, const uint16_t *acc, const float *ml, const int32_t *meta,
                     uint32_t rows, uint32_t n_heads, uint32_t dv);
// The same slot scheme with fp32 partials (O, maximum in the log2 domain, normaliser), [slot][head][dv].
int launch_merge_meta(hipStream_t stream, int dtype, void *out, const float *acc, const float *ml, const int32_t *meta,
                      uint32_t rows, uint32_t n_heads, uint32_t dv);

// decode_attention.hip
bool decode_supported(uint32_t head_dim);
void decode_geometry(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t *g_kernel,
                     uint32_t *head_chunks, uint32_t *nkv_wg, uint32_t *zdim);
uint32_t decode_pick_tile(uint32_t batch, uint32_t n_kv_heads, uint32_t block_size,
                          uint32_t max_num_block, uint32_t zdim);
size_t decode_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                              uint32_t max_tiles);
int launch_decode(hipStream_t stream, const AttentionArgs &a, uint32_t tile_tokens);

// decode_mfma.hip
bool decode_dma256_supported(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size, int kv_dtype);
bool decode_mfma_supported(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size,
                           uint32_t total_tokens);
struct DecodeSplitPlan {
    uint32_t max_chunks;   // bound on the number of chunks, hence of partial slots (two per chunk)
    size_t meta_bytes, ml_bytes, acc_bytes;
};
size_t decode_mfma_workspace_bytes(uint32_t batch, uint32_t n_heads, uint32_t head_dim, uint32_t block_size,
                                   uint32_t max_num_block);
// `rope`: the batch's rope_and_cache arguments, for a batch that decode_mfma_whole_rows accepts: the kernel then
// rotates and stores the rows itself
struct RopeArgs;
bool decode_mfma_whole_rows(const AttentionArgs &a);
int launch_decode_mfma(hipStream_t stream, const AttentionArgs &a, const RopeArgs *rope = nullptr);
uint32_t decode_mfma_slice_units();   // units (rows, sequences) one launch of the decode kernels can split

// mla_decode.hip
struct MlaDecodeParams {
    const uint16_t *q_absorb;
    const uint16_t *qr;
    const uint16_t *k_cache;
    const uint16_t *pe_cache;
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;   // nullptr: dense cache, dense_len rows per sequence, no causality
    int32_t *part_meta;   // [total_rows][4]: segments of the row (0: stored directly), first chunk, first-in-chunk flag
    float *part_acc;      // [2 * chunks][n_heads][512] 16-bit, O / l of a partial slot
    float *part_ml;       // [2 * chunks][n_heads][2]: running maximum (log2 domain), sum
    uint32_t n_heads;
    uint32_t batch;
    uint32_t total_rows;
    uint32_t block_size;
    uint32_t max_num_blocks;
    uint32_t dense_len;
    uint32_t chunk_min_steps;
    float scale_log2e;
    const int32_t *topk_indices;   // [total_rows][top_k] position lists (top_k == 0: none)
    uint32_t top_k;
    unsigned long long *clock_probe;   // nullptr, or where workgroup 0 leaves its shader-clock and wall-clock stamps
    uint32_t by_pos;      // 1: block sizes that are not a multiple of 32 - every row walks a list of positions, its own
                          // (0, 1, 2, ...) unless topk_indices gives it one
};
bool mla_decode_supported(const MlaArgs &a);
size_t mla_decode_workspace_bytes(const MlaArgs &a);
int launch_mla_decode(hipStream_t stream, const MlaArgs &a);

// prefill_mfma.hip
bool prefill_mfma_supported(const AttentionArgs &a);
bool prefill_kv8_supported(const AttentionArgs &a);
int launch_prefill_mfma(hipStream_t stream, const AttentionArgs &a);
size_t prefill_mfma_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                    uint32_t batch, uint32_t max_ctx);

// kv_dequant.hip: the 16-bit copy of a quantised cache's visible blocks, at the front of the workspace
size_t kv_dequant_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size, uint32_t batch, uint32_t max_num_block);
int launch_kv_dequant(hipStream_t stream, AttentionArgs *a);
// bf16 models run over the fp16 copy in fp16: converted queries and an fp16 result buffer in the workspace
size_t kv_dequant_f16_io_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim);
int launch_kv_dequant_f16_begin(hipStream_t stream, AttentionArgs *a, void **real_out);
int launch_kv_dequant_f16_finish(hipStream_t stream, const AttentionArgs &a, void *real_out);

// mla_topk.hip
size_t mla_topk_scratch_bytes(uint32_t total_tokens, uint32_t kv_lora_rank, uint32_t rope_head_dim, uint32_t top_k);
int launch_mla_topk(hipStream_t stream, const MlaArgs &a);

// mfma_attention.hip
bool mfma_gqa_supported(uint32_t head_dim);
size_t mfma_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t dv, uint32_t splits);
uint32_t mfma_pick_splits(uint32_t total_tokens, uint32_t rows_per_token, uint32_t batch,
                          uint32_t parallel_heads, uint32_t max_ctx, uint32_t tile);
int launch_mfma_gqa(hipStream_t stream, const AttentionArgs &a);
int launch_mfma_mla(hipStream_t stream, const MlaArgs &a);
// mla_generic.hip: any latent / rotary size, no matrix instructions
int launch_mla_generic(hipStream_t stream, const MlaArgs &a);

}  // namespace xlite
