// Quantised KV caches outside the streaming decode kernels (prefill and chunked prefill, mixed batches, decode
// shapes those kernels do not take): the blocks the batch can see are dequantised once into a compact 16-bit
// paged cache in the workspace, addressed by a block table of its own, and the 16-bit kernels run on that.
// The copy reads one byte and writes two per cached element, which a prefill's matrix work dwarfs; decode
// batches of the common shapes never come here (decode_mfma.hip reads the bytes directly).
// The copy is always fp16: a dequantised value (7 or 4 significant bits times an fp32 scale) then carries a
// rounding of 2^-11 instead of the 2^-8 of bf16, which unscaled queries would amplify. bf16 models run these
// batches in fp16: the queries are converted into the workspace, the 16-bit kernels compute and store fp16, and
// the result rows are converted back (values beyond the fp16 range saturate at +-65504).
#include <algorithm>

#include "attention_common.h"
#include "kv8.h"

namespace xlite {

namespace {

// workgroup (x = block j of the sequence and a part of it, y = sequence, z = K | V): block j of sequence i lands at
// block i * max_num_block + j of the compact cache; blocks beyond the sequence's visible range are skipped. A part is
// kDequantPart 16-byte chunks: a thread takes four of them, 256 apart, with their loads (bytes and scales) all in
// flight before the first conversion.
constexpr uint32_t kDequantUnroll = 4;
constexpr uint32_t kDequantPart = 256 * kDequantUnroll;

template <typename T, int KVF>
__global__ void __launch_bounds__(256)
dequant_blocks_kernel(const unsigned char *__restrict__ k_cache, const unsigned char *__restrict__ v_cache,
                      const float *__restrict__ k_scale, const float *__restrict__ v_scale,
                      const int32_t *__restrict__ block_tables, const int32_t *__restrict__ lens,
                      const int32_t *__restrict__ cached_lens, uint16_t *__restrict__ k_out, uint16_t *__restrict__ v_out,
                      int32_t *__restrict__ table_out, uint32_t block_size, uint32_t max_num_block, uint32_t n_kv_heads,
                      uint32_t head_dim, uint32_t parts, uint32_t skip_single)
{
    const uint32_t j = blockIdx.x / parts, part = blockIdx.x % parts, i = blockIdx.y;
    const bool is_v = blockIdx.z != 0;
    const uint64_t out_block = static_cast<uint64_t>(i) * max_num_block + j;
    const int32_t n_rows = lens[i], n_cached = cached_lens[i];
    const uint64_t phys = static_cast<uint32_t>(block_tables[out_block]);
    if (!is_v && part == 0 && threadIdx.x == 0) {
        table_out[out_block] = static_cast<int32_t>(out_block);
    }
    // sequences without rows need nothing; with skip_single those with one row read the bytes themselves
    const int32_t visible = n_rows > 0 && !(skip_single && n_rows == 1) ? n_cached + n_rows : 0;
    if (static_cast<int64_t>(j) * block_size >= visible) {
        return;
    }
    const uint32_t rows_here = min(block_size, static_cast<uint32_t>(visible) - j * block_size);   // positions of the block
    const uint32_t cpr = head_dim / 16;                              // 16-element chunks per (position, kv head) row
    const uint32_t chunks = rows_here * n_kv_heads * cpr;            // (a block is well below 2^32 chunks)
    const uint32_t all_chunks = block_size * n_kv_heads * cpr;
    const unsigned char *src = (is_v ? v_cache : k_cache) + phys * block_size * n_kv_heads * head_dim;
    const float *sc = (is_v ? v_scale : k_scale) + phys * block_size * n_kv_heads;
    uint16_t *dst = (is_v ? v_out : k_out) + out_block * block_size * n_kv_heads * head_dim;
    const uint32_t c0 = part * kDequantPart + threadIdx.x;
    // (every load is issued, from a clamped address: a load under a condition is compiled into a branch with a wait
    // of its own)
    uint4 raw[kDequantUnroll];
    float scale[kDequantUnroll];
#pragma unroll
    for (uint32_t u = 0; u < kDequantUnroll; u++) {
        const uint32_t c = min(c0 + u * 256, chunks - 1);
        typedef uint32_t words_t __attribute__((ext_vector_type(4)));
        const words_t w = __builtin_nontemporal_load(reinterpret_cast<const words_t *>(src + static_cast<uint64_t>(c) * 16));
        raw[u] = make_uint4(w[0], w[1], w[2], w[3]);
        scale[u] = sc[c / cpr];
    }
#pragma unroll
    for (uint32_t u = 0; u < kDequantUnroll; u++) {
        const uint32_t c = c0 + u * 256;
        if (c < chunks) {
            *reinterpret_cast<uint4 *>(dst + static_cast<uint64_t>(c) * 16) = dequant8<T, KVF>(make_uint2(raw[u].x, raw[u].y), scale[u]);
            *reinterpret_cast<uint4 *>(dst + static_cast<uint64_t>(c) * 16 + 8) = dequant8<T, KVF>(make_uint2(raw[u].z, raw[u].w), scale[u]);
        } else if (c < all_chunks) {
            // the rest of a partly visible block: zeros (the 16-bit kernels may load whole tiles and give the positions
            // past the end probability zero, which stale workspace bits that read as NaN would turn into NaN)
            *reinterpret_cast<uint4 *>(dst + static_cast<uint64_t>(c) * 16) = make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4 *>(dst + static_cast<uint64_t>(c) * 16 + 8) = make_uint4(0, 0, 0, 0);
        }
    }
}

// q | k | v rows of a bf16 model as fp16 (the whole fused row: the kernels address q inside it)
__global__ void __launch_bounds__(256)
rows_bf16_to_f16_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, uint64_t n_oct)
{
    auto one = [](uint32_t w) { return FP16::pack(clamp_f16(BF16::lo(w)), clamp_f16(BF16::hi(w))); };
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n_oct; i += gridDim.x * 256ull) {
        const uint4 w = reinterpret_cast<const uint4 *>(src)[i];
        reinterpret_cast<uint4 *>(dst)[i] = make_uint4(one(w.x), one(w.y), one(w.z), one(w.w));
    }
}

// result rows back to bf16, sequence by sequence (x = row chunk, y = sequence); with skip_single the rows of
// sequences with exactly one query row belong to another kernel, which wrote them in the output's own type
__global__ void __launch_bounds__(256)
rows_f16_to_bf16_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, const int32_t *__restrict__ query_start_loc,
                        const int32_t *__restrict__ lens, uint32_t row_oct, uint32_t skip_single)
{
    const uint32_t i = blockIdx.y;
    const int32_t n = lens[i];
    if (n <= 0 || (skip_single && n == 1)) {
        return;
    }
    auto one = [](uint32_t w) { return BF16::pack(FP16::lo(w), FP16::hi(w)); };
    const uint64_t first = static_cast<uint64_t>(query_start_loc[i]) * row_oct, count = static_cast<uint64_t>(n) * row_oct;
    for (uint64_t j = blockIdx.x * 256ull + threadIdx.x; j < count; j += gridDim.x * 256ull) {
        const uint4 w = reinterpret_cast<const uint4 *>(src)[first + j];
        reinterpret_cast<uint4 *>(dst)[first + j] = make_uint4(one(w.x), one(w.y), one(w.z), one(w.w));
    }
}

struct DequantLayout {
    size_t cache_bytes;   // one 16-bit tensor
    size_t table_bytes;
    size_t total;
};

DequantLayout dequant_layout(uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size, uint32_t batch,
                             uint32_t max_num_block)
{
    DequantLayout l{};
    l.cache_bytes = static_cast<size_t>(batch) * max_num_block * block_size * n_kv_heads * head_dim * 2;
    l.cache_bytes = (l.cache_bytes + 255) / 256 * 256;
    l.table_bytes = (static_cast<size_t>(batch) * max_num_block * sizeof(int32_t) + 255) / 256 * 256;
    l.total = 2 * l.cache_bytes + l.table_bytes;
    return l;
}

}  // namespace

size_t kv_dequant_bytes(uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size, uint32_t batch, uint32_t max_num_block)
{
    return dequant_layout(n_kv_heads, head_dim, block_size, batch, max_num_block).total;
}

// Fills the front of a.workspace with the 16-bit copy and rewrites `a` to address it: 16-bit caches, the
// identity-like table, the rest of the workspace.
int launch_kv_dequant(hipStream_t stream, AttentionArgs *a)
{
    XL_REQUIRE(a->head_dim % 16 == 0, "head_dim must be a multiple of 16");
    const DequantLayout l = dequant_layout(a->n_kv_heads, a->head_dim, a->block_size, a->batch, a->max_num_block);
    if (a->workspace == nullptr || a->workspace_bytes < l.total) {
        return fail(XLITE_HIP_ENOSPC, __func__,
                    "workspace too small: this batch over a quantised cache needs " + std::to_string(l.total) +
                        " bytes for the 16-bit copy of its blocks (2 tensors x batch x max_num_block x block_size x "
                        "n_kv_heads x head_dim x 2 bytes, plus a table of batch x max_num_block entries: every block the "
                        "tables can name, whatever the sequences' lengths), have " + std::to_string(a->workspace_bytes));
    }
    char *ws = static_cast<char *>(a->workspace);
    uint16_t *k_out = reinterpret_cast<uint16_t *>(ws);
    uint16_t *v_out = reinterpret_cast<uint16_t *>(ws + l.cache_bytes);
    int32_t *table = reinterpret_cast<int32_t *>(ws + 2 * l.cache_bytes);
    const uint64_t block_chunks = static_cast<uint64_t>(a->block_size) * a->n_kv_heads * (a->head_dim / 16);
    XL_REQUIRE(block_chunks < (1ull << 31), "a cache block of more than 2^31 16-byte chunks");
    const uint32_t parts = static_cast<uint32_t>((block_chunks + kDequantPart - 1) / kDequantPart);
    XL_REQUIRE(static_cast<uint64_t>(a->max_num_block) * parts < (1ull << 31), "block tables too wide for the dequantising copy");
    const dim3 grid(a->max_num_block * parts, a->batch, 2);
    XL_REQUIRE(a->batch <= 65535, "more than 65535 sequences over a quantised cache outside the decode kernels");
    auto launch = [&](auto tag, auto kv) {
        using T = decltype(tag);
        dequant_blocks_kernel<T, decltype(kv)::value><<<grid, 256, 0, stream>>>(
            static_cast<const unsigned char *>(a->k_cache), static_cast<const unsigned char *>(a->v_cache), a->k_scale,
            a->v_scale, a->block_tables, a->lens, a->cached_lens, k_out, v_out, table, a->block_size, a->max_num_block,
            a->n_kv_heads, a->head_dim, parts, a->rows_mode == kSkipSingle ? 1u : 0u);
    };
    using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
    using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
    a->kv_dtype == XLITE_HIP_KV_INT8 ? launch(FP16{}, I8{}) : launch(FP16{}, F8{});
    XL_LAUNCH_CHECK();
    a->k_cache = k_out;
    a->v_cache = v_out;
    a->block_tables = table;
    a->kv_dtype = XLITE_HIP_KV_SAME;
    a->k_scale = nullptr;
    a->v_scale = nullptr;
    a->workspace = ws + l.total;
    a->workspace_bytes -= l.total;
    return XLITE_HIP_OK;
}

// bf16 models over the fp16 copy: fp16 queries and an fp16 result buffer behind the copy
size_t kv_dequant_f16_io_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim)
{
    const size_t q = (static_cast<size_t>(total_tokens) * (n_heads + 2 * n_kv_heads) * head_dim * 2 + 255) / 256 * 256;
    const size_t o = (static_cast<size_t>(total_tokens) * n_heads * head_dim * 2 + 255) / 256 * 256;
    return q + o;
}

// Rewrites `a` of a bf16 model to an fp16 problem: qkv converted into the workspace, output redirected to an fp16
// buffer there; *real_out keeps the caller's output for kv_dequant_f16_finish.
int launch_kv_dequant_f16_begin(hipStream_t stream, AttentionArgs *a, void **real_out)
{
    const size_t row = static_cast<size_t>(a->n_heads + 2 * a->n_kv_heads) * a->head_dim;
    const size_t q_bytes = (static_cast<size_t>(a->total_tokens) * row * 2 + 255) / 256 * 256;
    const size_t o_bytes = (static_cast<size_t>(a->total_tokens) * a->n_heads * a->head_dim * 2 + 255) / 256 * 256;
    if (a->workspace == nullptr || a->workspace_bytes < q_bytes + o_bytes) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small for the fp16 queries and results of a bf16 batch over a "
                                                "quantised cache: need " + std::to_string(q_bytes + o_bytes) + " more bytes");
    }
    char *ws = static_cast<char *>(a->workspace);
    const uint64_t octs = static_cast<uint64_t>(a->total_tokens) * row / 8;   // head_dim is a multiple of 16
    const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>((octs + 255) / 256, 4096));
    rows_bf16_to_f16_kernel<<<blocks, 256, 0, stream>>>(static_cast<const uint16_t *>(a->qkv), reinterpret_cast<uint16_t *>(ws), octs);
    XL_LAUNCH_CHECK();
    *real_out = a->output;
    a->qkv = ws;
    a->output = ws + q_bytes;
    a->dtype = XLITE_HIP_FP16;
    a->workspace = ws + q_bytes + o_bytes;
    a->workspace_bytes -= q_bytes + o_bytes;
    return XLITE_HIP_OK;
}

int launch_kv_dequant_f16_finish(hipStream_t stream, const AttentionArgs &a, void *real_out)
{
    XL_REQUIRE(a.batch <= 65535, "more than 65535 sequences over a quantised cache outside the decode kernels");
    const uint32_t row_pairs = a.n_heads * a.head_dim / 8;
    // enough workgroups per sequence for the longest chunk a batch of this size can hold
    const uint64_t per_seq = static_cast<uint64_t>(a.total_tokens) * row_pairs;
    const uint32_t bx = static_cast<uint32_t>(std::min<uint64_t>((per_seq + 255) / 256, 256));
    rows_f16_to_bf16_kernel<<<dim3(bx, a.batch, 1), 256, 0, stream>>>(static_cast<const uint16_t *>(a.output),
                                                                      static_cast<uint16_t *>(real_out), a.query_start_loc,
                                                                      a.lens, row_pairs, a.rows_mode == kSkipSingle ? 1u : 0u);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

}  // namespace xlite
