// C entry points of the attention operators: argument checks and kernel selection.
#include "attention_common.h"
#include "rope_item.h"

using namespace xlite;

namespace {

// As many query rows as sequences: a decode step in all but contrived batches (the lengths live in
// device memory, so the host cannot look). The decode kernels work row by row and do not rely on it: a
// batch such as lens = [2, 0] is served correctly, only without sharing the cache reads of a
// sequence's rows. Reference: decode iff every length is 1 (xlite/csrc/runtime.cpp:466-470).
bool is_decode_batch(uint32_t total_tokens, uint32_t batch)
{
    return total_tokens == batch;
}

}  // namespace

namespace {

// scratch of a batch over 16-bit caches
size_t workspace_bytes_16(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                          uint32_t block_size, uint32_t batch, uint32_t max_num_block)
{
    const uint32_t max_ctx = max_num_block * block_size;
    if (is_decode_batch(total_tokens, batch) &&
        decode_dma256_supported(n_heads, n_kv_heads, head_dim, block_size, XLITE_HIP_KV_SAME)) {
        return decode_mfma_workspace_bytes(batch, n_heads, head_dim, block_size, max_num_block);
    }
    if (is_decode_batch(total_tokens, batch) && decode_supported(head_dim)) {
        if (decode_mfma_supported(n_heads, n_kv_heads, head_dim, block_size, total_tokens)) {
            return decode_mfma_workspace_bytes(batch, n_heads, head_dim, block_size, max_num_block);
        }
        uint32_t g_kernel, head_chunks, nkv_wg, zdim;
        decode_geometry(n_heads, n_kv_heads, head_dim, &g_kernel, &head_chunks, &nkv_wg, &zdim);
        const uint32_t tile = decode_pick_tile(batch, n_kv_heads, block_size, max_num_block, zdim);
        return std::max(decode_workspace_bytes(total_tokens, n_heads, head_dim, ceil_div(max_ctx, tile)),
                        prefill_mfma_workspace_bytes(total_tokens, n_heads, n_kv_heads, head_dim, batch, max_ctx));
    }
    const uint32_t splits =
        mfma_pick_splits(total_tokens, n_heads / n_kv_heads, batch, n_kv_heads, max_ctx, 64);
    // whichever prefill kernel serves the shape
    return std::max(mfma_workspace_bytes(total_tokens, n_heads, head_dim, splits + 1),
                    prefill_mfma_workspace_bytes(total_tokens, n_heads, n_kv_heads, head_dim, batch, max_ctx));
}

// A batch that is mostly decode rows with prefills among them (what a continuous-batching scheduler issues: the
// reference's decode flag is per batch, xlite/csrc/runtime.cpp:466-470) is served by two kernels: the
// sequences with one query row by the streaming decode kernel, the others by the streaming prefill kernel.
// Decided from the shape alone (the lengths live in device memory): at least 16 sequences and fewer than 4
// rows per sequence on average.
bool mixed_split(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size,
                 uint32_t batch)
{
    return !is_decode_batch(total_tokens, batch) && batch >= 16 && batch <= decode_mfma_slice_units() &&
           total_tokens > batch && total_tokens < 4 * batch &&
           decode_mfma_supported(n_heads, n_kv_heads, head_dim, block_size, batch);
}

// M rows (query rows x query heads of a kv head) per sequence, on average, up to which a multi-row batch over a
// quantised cache is read on the fly by the prefill kernel instead of through a 16-bit copy. Measured, int8, by copy /
// on the fly: Llama-3-8B 32 x 64 tokens 0.030 / 0.022 ms, 128 after 16384 cached 0.095 / 0.082, 8 x 256 after 4096
// 0.231 / 0.211, 8 x 512 after 4096 0.354 / 0.356 (the break-even: 2048 M rows), 8 x 2048 after 4096 1.45 / 1.60.
constexpr uint64_t kKv8DirectRows = 2048;

// A quantised cache is read directly by the streaming decode kernel (and, int8 only, by the vector decode
// kernel); every other batch goes through a 16-bit copy of its blocks.
bool quantised_direct(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size,
                      uint32_t batch, int kv_dtype)
{
    if (!is_decode_batch(total_tokens, batch)) {
        return false;
    }
    return decode_mfma_supported(n_heads, n_kv_heads, head_dim, block_size, total_tokens) ||
           (kv_dtype == XLITE_HIP_KV_INT8 && decode_supported(head_dim));
}

}  // namespace

static int run_16bit(hipStream_t s, AttentionArgs &a);

extern "C" size_t xlite_hip_attention_workspace_bytes_kv(uint32_t total_tokens, uint32_t n_heads,
                                                         uint32_t n_kv_heads, uint32_t head_dim,
                                                         uint32_t block_size, uint32_t batch,
                                                         uint32_t max_num_block, int kv_dtype)
{
    if (total_tokens == 0 || batch == 0 || n_kv_heads == 0 || n_heads % n_kv_heads != 0 || head_dim < 8) {
        return 0;
    }
    size_t need = workspace_bytes_16(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block);
    if (mixed_split(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch)) {
        need += decode_mfma_workspace_bytes(total_tokens, n_heads, head_dim, block_size, max_num_block);
    }
    if (kv_dtype != XLITE_HIP_KV_SAME &&
        !quantised_direct(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, kv_dtype)) {
        need += kv_dequant_bytes(n_kv_heads, head_dim, block_size, batch, max_num_block);
        need += kv_dequant_f16_io_bytes(total_tokens, n_heads, n_kv_heads, head_dim);   // bf16 models (the size does not know)
    }
    return need;
}

extern "C" size_t xlite_hip_attention_workspace_bytes(uint32_t total_tokens, uint32_t n_heads,
                                                      uint32_t n_kv_heads, uint32_t head_dim,
                                                      uint32_t block_size, uint32_t batch,
                                                      uint32_t max_num_block)
{
    return xlite_hip_attention_workspace_bytes_kv(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch,
                                                  max_num_block, XLITE_HIP_KV_SAME);
}

extern "C" int xlite_hip_attention(void *stream, const void *qkv, const void *k_cache,
                                   const void *v_cache, void *output,
                                   const int32_t *query_start_loc, const int32_t *lens,
                                   const int32_t *cached_lens, const int32_t *block_tables,
                                   uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                                   uint32_t head_dim, uint32_t block_size, uint32_t batch,
                                   uint32_t max_num_block, int dtype, int kv_dtype,
                                   const float *k_scale, const float *v_scale, void *workspace,
                                   size_t workspace_bytes)
{
    XL_REQUIRE(dtype == XLITE_HIP_FP16 || dtype == XLITE_HIP_BF16, "qkv/kCache/vCache/output dtype unsupported!");
    XL_REQUIRE(kv_dtype == XLITE_HIP_KV_SAME || kv_dtype == XLITE_HIP_KV_INT8 || kv_dtype == XLITE_HIP_KV_FP8,
               "kv cache dtype unsupported!");
    if (batch == 0 || total_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(qkv && k_cache && v_cache && output && query_start_loc && lens && cached_lens && block_tables,
               "null tensor");
    XL_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "n_heads must be a positive multiple of n_kv_heads");
    XL_REQUIRE(block_size > 0 && max_num_block > 0, "block_size and max_num_block must be positive");
    XL_REQUIRE(kv_dtype == XLITE_HIP_KV_SAME || (k_scale && v_scale), "a quantised KV cache needs k_scale and v_scale");
    AttentionArgs a{qkv, k_cache, v_cache, output, query_start_loc, lens, cached_lens, block_tables,
                    total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block,
                    dtype, kv_dtype, k_scale, v_scale, workspace, workspace_bytes};
    hipStream_t s = as_stream(stream);
    AttentionArgs as16 = a;   // the shape as the 16-bit kernels will see it
    as16.kv_dtype = XLITE_HIP_KV_SAME;
    if (mixed_split(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch) && prefill_mfma_supported(as16)) {
        // the decode rows first, straight from the cache (quantised or not); its scratch is the front of the workspace
        const size_t dec = decode_mfma_workspace_bytes(total_tokens, n_heads, head_dim, block_size, max_num_block);
        AttentionArgs d = a;
        d.rows_mode = kOnlySingle;
        if (workspace != nullptr && workspace_bytes >= dec) {
            if (const int rc = launch_decode_mfma(s, d)) {
                return rc;
            }
            a.rows_mode = kSkipSingle;
            a.workspace = static_cast<char *>(workspace) + dec;
            a.workspace_bytes = workspace_bytes - dec;
        }   // (too little scratch: one kernel serves every row, as for any prefill batch)
    }
    if (kv_dtype != XLITE_HIP_KV_SAME &&
        !quantised_direct(total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, kv_dtype)) {
        XL_REQUIRE(decode_supported(head_dim), "quantised KV caches: head_dim must be 64 or 128");
        // Multi-row batches of head_dim 128: the prefill kernel reads the bytes itself when the chunks are short (the
        // copy below dequantises the whole visible cache of the batch, five bytes of traffic per cached element,
        // whatever the number of query rows; reading on the fly costs the kernel a tenth of its time on long chunks)
        // or when the workspace cannot hold the copy.
        if (!is_decode_batch(total_tokens, batch) && prefill_kv8_supported(a)) {
            const size_t copy_bytes = kv_dequant_bytes(n_kv_heads, head_dim, block_size, batch, max_num_block);
            const bool short_chunks = static_cast<uint64_t>(total_tokens) * (n_heads / n_kv_heads) <= kKv8DirectRows * static_cast<uint64_t>(batch);
            if (short_chunks || a.workspace == nullptr || a.workspace_bytes < copy_bytes) {
                return launch_prefill_mfma(s, a);
            }
        }
        if (const int rc = launch_kv_dequant(s, &a)) {   // from here on: fp16 caches in the workspace
            return rc;
        }
        if (dtype == XLITE_HIP_BF16) {
            // a bf16 model: this batch runs in fp16 over the fp16 copy. The streaming prefill kernel converts the
            // query rows as it loads them and stores bf16; the other kernels get converted queries and an fp16
            // result buffer in the workspace, converted back afterwards
            AttentionArgs f = a;
            f.dtype = XLITE_HIP_FP16;
            if (!is_decode_batch(total_tokens, batch) && prefill_mfma_supported(f)) {
                f.io_bf16 = true;
                return launch_prefill_mfma(s, f);
            }
            void *real_out = nullptr;
            if (const int rc = launch_kv_dequant_f16_begin(s, &a, &real_out)) {
                return rc;
            }
            if (const int rc = run_16bit(s, a)) {
                return rc;
            }
            return launch_kv_dequant_f16_finish(s, a, real_out);
        }
    }
    return run_16bit(s, a);
}

// a batch over 16-bit caches (or a decode batch of the streaming kernels' shapes over a quantised one)
static int run_16bit(hipStream_t s, AttentionArgs &a)
{
    const uint32_t total_tokens = a.total_tokens, n_heads = a.n_heads, n_kv_heads = a.n_kv_heads, head_dim = a.head_dim,
                   block_size = a.block_size, batch = a.batch, max_num_block = a.max_num_block;
    // head_dim 256 (the reference kernel is generic over headSize, xlite/csrc/kernels/attention.h:39-74, and ships
    // such models): decode batches of up to 16 query heads per kv head stream the cache like head_dim 128 does, a
    // head as two 256-byte units; the generic matrix-core kernel serves every other batch
    if (is_decode_batch(total_tokens, batch) &&
        decode_dma256_supported(n_heads, n_kv_heads, head_dim, block_size, a.kv_dtype)) {
        return launch_decode_mfma(s, a);
    }
    if (is_decode_batch(total_tokens, batch) && decode_supported(head_dim)) {
        if (decode_mfma_supported(n_heads, n_kv_heads, head_dim, block_size, total_tokens)) {
            return launch_decode_mfma(s, a);
        }
        // more than 16 query heads per kv head, or a block size that is not a multiple of 16: the prefill
        // kernel takes the rows of a sequence as one (ragged) M tile and splits the KV range
        if (a.kv_dtype == XLITE_HIP_KV_SAME && prefill_mfma_supported(a)) {
            return launch_prefill_mfma(s, a);
        }
        // head_dim 64 or block sizes that are not a multiple of 4 at such shapes, int8 caches with wide groups
        uint32_t g_kernel, head_chunks, nkv_wg, zdim;
        decode_geometry(n_heads, n_kv_heads, head_dim, &g_kernel, &head_chunks, &nkv_wg, &zdim);
        uint32_t tile = decode_pick_tile(batch, n_kv_heads, block_size, max_num_block, zdim);
        // shrink the split count to what the caller's workspace can hold
        const uint32_t max_ctx = max_num_block * block_size;
        while (ceil_div(max_ctx, tile) > 1 &&
               (a.workspace == nullptr ||
                decode_workspace_bytes(total_tokens, n_heads, head_dim, ceil_div(max_ctx, tile)) > a.workspace_bytes)) {
            tile *= 2;
        }
        int rc = launch_decode(s, a, tile);
        if (rc != XLITE_HIP_OK) {
            return rc;
        }
        XL_LAUNCH_CHECK();
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(mfma_gqa_supported(head_dim), "head_dim must be 64, 128 or 256");
    if (prefill_mfma_supported(a)) {
        return launch_prefill_mfma(s, a);
    }
    return launch_mfma_gqa(s, a);
}

extern "C" int xlite_hip_decode_step(void *stream, void *qkv, void *k_cache, void *v_cache, void *output,
                                     const int64_t *position, const void *cosin, const int32_t *slot_mapping,
                                     const int32_t *query_start_loc, const int32_t *lens,
                                     const int32_t *cached_lens, const int32_t *block_tables,
                                     uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                                     uint32_t head_dim, uint32_t rot_dim, uint32_t block_size, uint32_t batch,
                                     uint32_t max_num_block, int is_neox, uint64_t mrope_mask_h,
                                     uint64_t mrope_mask_w, int dtype, void *workspace, size_t workspace_bytes)
{
    // Decode batches that the decode kernel takes as whole rows (contexts that are short by the width of the block
    // tables: such a step is bound by its launches): one launch, the kernel rotates and stores the rows itself. The
    // arguments are checked as the two calls check them.
    if (total_tokens != 0 && batch != 0 && qkv && k_cache && v_cache && output && query_start_loc && lens && cached_lens &&
        block_tables && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && block_size > 0 && max_num_block > 0 &&
        (dtype == XLITE_HIP_FP16 || dtype == XLITE_HIP_BF16) && is_decode_batch(total_tokens, batch) &&
        decode_supported(head_dim) && decode_mfma_supported(n_heads, n_kv_heads, head_dim, block_size, total_tokens)) {
        AttentionArgs a{qkv, k_cache, v_cache, output, query_start_loc, lens, cached_lens, block_tables,
                        total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block,
                        dtype, XLITE_HIP_KV_SAME, nullptr, nullptr, workspace, workspace_bytes};
        if (decode_mfma_whole_rows(a)) {
            RopeArgs rope{};
            if (const int rc = rope_prepare(qkv, k_cache, v_cache, position, cosin, slot_mapping, total_tokens, n_heads,
                                            n_kv_heads, head_dim, rot_dim, block_size, is_neox, mrope_mask_h, mrope_mask_w,
                                            dtype, true, &rope)) {
                return rc;
            }
            return launch_decode_mfma(as_stream(stream), a, &rope);
        }
    }
    // otherwise the two calls of a layer's attention block, enqueued back to back on the caller's stream
    if (const int rc = xlite_hip_rope_and_cache(stream, qkv, k_cache, v_cache, position, cosin, slot_mapping, total_tokens,
                                                n_heads, n_kv_heads, head_dim, rot_dim, block_size, is_neox, mrope_mask_h,
                                                mrope_mask_w, dtype)) {
        return rc;
    }
    return xlite_hip_attention(stream, qkv, k_cache, v_cache, output, query_start_loc, lens, cached_lens, block_tables,
                               total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block, dtype,
                               XLITE_HIP_KV_SAME, nullptr, nullptr, workspace, workspace_bytes);
}

extern "C" size_t xlite_hip_mla_workspace_bytes(uint32_t total_tokens, uint32_t n_heads,
                                                uint32_t kv_lora_rank, uint32_t rope_head_dim,
                                                uint32_t block_size, uint32_t batch,
                                                uint32_t max_num_blocks, uint32_t top_k)
{
    if (top_k > 0) {
        MlaArgs a{};
        a.total_tokens = total_tokens;
        a.batch = batch;
        a.n_heads = n_heads;
        a.kv_lora_rank = kv_lora_rank;
        a.rope_head_dim = rope_head_dim;
        a.block_size = block_size;
        a.max_num_blocks = max_num_blocks;
        a.top_k = top_k;
        static const int32_t dummy = 0;
        a.block_tables = &dummy;
        if (mla_decode_supported(a)) {
            return mla_decode_workspace_bytes(a);   // the decode kernel reads the listed rows itself
        }
        // the gathered per-row caches, then the dense attention over them (every row a sequence)
        return mla_topk_scratch_bytes(total_tokens, kv_lora_rank, rope_head_dim, top_k) +
               xlite_hip_mla_workspace_bytes(total_tokens, n_heads, kv_lora_rank, rope_head_dim, 1, total_tokens, top_k, 0);
    }
    const uint32_t max_ctx = max_num_blocks * block_size;
    const uint32_t splits = mfma_pick_splits(total_tokens, n_heads, batch, 1, max_ctx, 32);
    size_t need = mfma_workspace_bytes(total_tokens, n_heads, kv_lora_rank, splits + 1);
    if (block_size > 0) {
        // the decode kernel plans its own work split; block_size == 1 describes a dense cache of
        // max_num_blocks rows per sequence
        MlaArgs a{};
        a.total_tokens = total_tokens;
        a.batch = batch;
        a.n_heads = n_heads;
        a.kv_lora_rank = kv_lora_rank;
        a.block_size = block_size;
        a.max_num_blocks = max_num_blocks;
        a.dense_len = max_num_blocks * block_size;
        static const int32_t dummy = 0;
        a.block_tables = &dummy;
        const size_t d = mla_decode_workspace_bytes(a);
        need = d > need ? d : need;
        a.block_tables = nullptr;
        const size_t d2 = mla_decode_workspace_bytes(a);
        need = d2 > need ? d2 : need;
    }
    return need;
}

extern "C" int xlite_hip_mla_attention(void *stream, const void *q_absorb, const void *qr,
                                       const void *k_cache, const void *pe_cache, void *o_absorb,
                                       const int32_t *query_start_loc, const int32_t *lens,
                                       const int32_t *cached_lens, const int32_t *block_tables,
                                       uint32_t total_tokens, uint32_t n_heads,
                                       uint32_t rope_head_dim, uint32_t kv_lora_rank,
                                       uint32_t block_size, uint32_t batch, uint32_t max_num_blocks,
                                       float scale, const int32_t *topk_indices, uint32_t top_k,
                                       int dtype, void *workspace, size_t workspace_bytes)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16, "qAbsorb/qr/kCache/peCache/oAbsorb dtype unsupported!");
    XL_REQUIRE(top_k <= 2048, "topK should be less than or equal to 2048");
    if (batch == 0 || total_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(q_absorb && qr && k_cache && pe_cache && o_absorb && query_start_loc && lens &&
                   cached_lens && block_tables,
               "null tensor");
    XL_REQUIRE(n_heads > 0 && block_size > 0 && max_num_blocks > 0, "zero head count or block geometry");
    MlaArgs a{q_absorb, qr, k_cache, pe_cache, o_absorb, query_start_loc, lens, cached_lens, block_tables,
              total_tokens, n_heads, rope_head_dim, kv_lora_rank, block_size, batch, max_num_blocks,
              0, scale, topk_indices, top_k, dtype, workspace, workspace_bytes};
    if (kv_lora_rank != 512 || rope_head_dim != 64) {
        return launch_mla_generic(as_stream(stream), a);  // sizes the matrix-core kernels are not built for
    }
    if (mla_decode_supported(a)) {
        return launch_mla_decode(as_stream(stream), a);   // with or without position lists
    }
    if (top_k > 0) {
        return launch_mla_topk(as_stream(stream), a);      // other shapes: gather the listed rows, then dense
    }
    return launch_mfma_mla(as_stream(stream), a);
}

extern "C" int xlite_hip_mla_v3(void *stream, const void *q_absorb, const void *qr,
                                const void *k_dense, const void *pe_dense, void *o_absorb,
                                const int32_t *query_start_loc, const int32_t *lens,
                                const int32_t *cached_lens, uint32_t total_tokens, uint32_t n_heads,
                                uint32_t rope_head_dim, uint32_t kv_lora_rank, uint32_t batch,
                                uint32_t index_topk, float scale, int dtype, void *workspace,
                                size_t workspace_bytes)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16, "qAbsorb/qr/kDenseCache/peDenseCache/oAbsorb dtype unsupported!");
    if (batch == 0 || total_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(q_absorb && qr && k_dense && pe_dense && o_absorb && query_start_loc && lens && cached_lens,
               "null tensor");
    XL_REQUIRE(n_heads > 0 && index_topk > 0, "zero head count or dense length");
    if (batch == 0 || total_tokens == 0) {
        return XLITE_HIP_OK;
    }
    MlaArgs a{q_absorb, qr, k_dense, pe_dense, o_absorb, query_start_loc, lens, cached_lens, nullptr,
              total_tokens, n_heads, rope_head_dim, kv_lora_rank, 1, batch, index_topk,
              index_topk, scale, nullptr, 0, dtype, workspace, workspace_bytes};
    if (kv_lora_rank != 512 || rope_head_dim != 64) {
        return launch_mla_generic(as_stream(stream), a);
    }
    if (mla_decode_supported(a)) {
        return launch_mla_decode(as_stream(stream), a);
    }
    return launch_mfma_mla(as_stream(stream), a);
}
