// Top-k index mask of the absorbed MLA attention, as a gather followed by the dense kernel.
//
// With top_k > 0 a query row whose causal range is longer than top_k attends only to the cache
// positions listed for it (xlite/csrc/kernels/mla_v2.h:697-699, softmax_attn_aiv.h:159-243; rows with a
// causal range of at most top_k positions ignore the list and see their whole range). The listed
// positions of every row are copied into a dense per-row cache [row][top_k][kv_lora_rank | rope] in the
// workspace, then the rows run through the dense (mla_v3-style) attention as sequences of one query
// each. Indices are expected ascending (the reference requires it); an index outside the causal range
// or equal to its predecessor is dropped.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr int kThreads = 256;
constexpr int kMaxTopk = 2048;
constexpr int kItems = kMaxTopk / kThreads;
constexpr uint32_t kRun = 128;   // dense positions copied by one workgroup

__global__ void __launch_bounds__(kThreads)
topk_gather_kernel(const uint4 *__restrict__ k_cache, const uint4 *__restrict__ pe_cache,
                   const int32_t *__restrict__ block_tables, const int32_t *__restrict__ topk,
                   const int32_t *__restrict__ query_start_loc, const int32_t *__restrict__ lens,
                   const int32_t *__restrict__ cached_lens, uint4 *__restrict__ k_dense,
                   uint4 *__restrict__ pe_dense, int32_t *__restrict__ meta, uint16_t *__restrict__ out,
                   uint32_t total_tokens, uint32_t batch, uint32_t top_k, uint32_t block_size,
                   uint32_t max_num_blocks, uint32_t k_vecs, uint32_t pe_vecs, uint32_t out_row_elems)
{
    __shared__ uint32_t sel[kMaxTopk];
    __shared__ uint32_t counts[kThreads];
    const uint32_t t = blockIdx.x;
    // the sequence that owns row t
    uint32_t seq = 0;
    int32_t r = 0;
    bool found = false;
    {
        // query_start_loc is a prefix sum: the owner is the last sequence that starts at or before t
        uint32_t lo = 0, hi = batch;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) / 2;
            if (query_start_loc[mid] <= static_cast<int32_t>(t)) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        if (lo > 0) {
            const int32_t s = query_start_loc[lo - 1], l = lens[lo - 1];
            if (static_cast<int32_t>(t) < s + l) {
                seq = lo - 1;
                r = static_cast<int32_t>(t) - s;
                found = true;
            }
        }
    }
    const uint32_t limit = found ? static_cast<uint32_t>(cached_lens[seq] + r + 1) : 0u;
    uint32_t count;
    if (limit <= top_k) {
        for (uint32_t j = threadIdx.x; j < limit; j += kThreads) {
            sel[j] = j;
        }
        count = limit;
    } else {
        // keep index j if it is inside the causal range and differs from its predecessor; compact
        const int32_t *row = topk + static_cast<uint64_t>(t) * top_k;
        const uint32_t j0 = threadIdx.x * kItems;
        uint32_t keep[kItems];
        uint32_t mine = 0;
#pragma unroll
        for (int e = 0; e < kItems; e++) {
            const uint32_t j = j0 + e;
            bool ok = false;
            uint32_t v = 0;
            if (j < top_k) {
                const int32_t x = row[j];
                v = static_cast<uint32_t>(x);
                ok = x >= 0 && v < limit && (j == 0 || row[j - 1] != x);
            }
            keep[e] = ok ? v : 0xffffffffu;
            mine += ok;
        }
        counts[threadIdx.x] = mine;
        __syncthreads();
        for (uint32_t d = 1; d < kThreads; d <<= 1) {   // inclusive scan
            const uint32_t add = threadIdx.x >= d ? counts[threadIdx.x - d] : 0u;
            __syncthreads();
            counts[threadIdx.x] += add;
            __syncthreads();
        }
        uint32_t pos = counts[threadIdx.x] - mine;
        count = counts[kThreads - 1];
#pragma unroll
        for (int e = 0; e < kItems; e++) {
            if (keep[e] != 0xffffffffu) {
                sel[pos++] = keep[e];
            }
        }
    }
    __syncthreads();
    // the dense rows: one 16-lane group per position
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const int32_t *table = block_tables + static_cast<uint64_t>(seq) * max_num_blocks;
    // the row's dense positions are dealt to gridDim.y workgroups in runs of kRun (every one of them has
    // compacted the list; a single workgroup per row copied 2.4 MB alone)
    const uint32_t run0 = blockIdx.y * kRun;
    for (uint32_t i = run0 + group; i < min(count, run0 + kRun); i += kThreads / 16) {
        const uint32_t tok = sel[i];
        const uint32_t phys = static_cast<uint32_t>(table[tok / block_size]);
        const uint64_t src = static_cast<uint64_t>(phys) * block_size + tok % block_size;
        const uint64_t dst = static_cast<uint64_t>(t) * top_k + i;
        for (uint32_t c = lane; c < k_vecs; c += 16) {
            k_dense[dst * k_vecs + c] = k_cache[src * k_vecs + c];
        }
        for (uint32_t c = lane; c < pe_vecs; c += 16) {
            pe_dense[dst * pe_vecs + c] = pe_cache[src * pe_vecs + c];
        }
    }
    // the row as a dense "sequence" of one query: [query_start_loc | lens | cached_lens]
    if (blockIdx.y != 0) {
        return;
    }
    if (threadIdx.x == 0) {
        meta[t] = static_cast<int32_t>(t);
        meta[total_tokens + t] = count > 0 ? 1 : 0;
        meta[2 * total_tokens + t] = count > 0 ? static_cast<int32_t>(count) - 1 : 0;
    }
    if (count == 0) {   // no visible key: the row's result is zero (the attention kernel skips it)
        for (uint32_t c = threadIdx.x; c < out_row_elems; c += kThreads) {
            out[static_cast<uint64_t>(t) * out_row_elems + c] = 0;
        }
    }
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

}  // namespace

size_t mla_topk_scratch_bytes(uint32_t total_tokens, uint32_t kv_lora_rank, uint32_t rope_head_dim, uint32_t top_k)
{
    if (top_k == 0) {
        return 0;
    }
    return align256(3 * static_cast<size_t>(total_tokens) * sizeof(int32_t)) +
           align256(static_cast<size_t>(total_tokens) * top_k * kv_lora_rank * 2) +
           align256(static_cast<size_t>(total_tokens) * top_k * rope_head_dim * 2);
}

int launch_mla_topk(hipStream_t stream, const MlaArgs &a)
{
    XL_REQUIRE(a.top_k <= kMaxTopk, "topK should be less than or equal to 2048");
    XL_REQUIRE(a.topk_indices != nullptr, "top_k > 0 needs topk_indices");
    XL_REQUIRE(a.kv_lora_rank % 8 == 0 && a.rope_head_dim % 8 == 0, "kv_lora_rank and rope_head_dim must be multiples of 8");
    const size_t scratch = mla_topk_scratch_bytes(a.total_tokens, a.kv_lora_rank, a.rope_head_dim, a.top_k);
    if (a.workspace == nullptr || a.workspace_bytes < scratch) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small for the top-k gather: need " + std::to_string(scratch) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    char *ws = static_cast<char *>(a.workspace);
    int32_t *meta = reinterpret_cast<int32_t *>(ws);
    char *k_dense = ws + align256(3 * static_cast<size_t>(a.total_tokens) * sizeof(int32_t));
    char *pe_dense = k_dense + align256(static_cast<size_t>(a.total_tokens) * a.top_k * a.kv_lora_rank * 2);

    topk_gather_kernel<<<dim3(a.total_tokens, ceil_div(a.top_k, kRun), 1), kThreads, 0, stream>>>(
        static_cast<const uint4 *>(a.k_cache), static_cast<const uint4 *>(a.pe_cache), a.block_tables, a.topk_indices,
        a.query_start_loc, a.lens, a.cached_lens, reinterpret_cast<uint4 *>(k_dense), reinterpret_cast<uint4 *>(pe_dense),
        meta, static_cast<uint16_t *>(a.o_absorb), a.total_tokens, a.batch, a.top_k, a.block_size, a.max_num_blocks,
        a.kv_lora_rank / 8, a.rope_head_dim / 8, a.n_heads * a.kv_lora_rank);
    XL_LAUNCH_CHECK();

    MlaArgs d = a;
    d.k_cache = k_dense;
    d.pe_cache = pe_dense;
    d.block_tables = nullptr;
    d.dense_len = a.top_k;
    d.batch = a.total_tokens;
    d.query_start_loc = meta;
    d.lens = meta + a.total_tokens;
    d.cached_lens = meta + 2 * a.total_tokens;
    d.block_size = 1;
    d.max_num_blocks = a.top_k;
    d.topk_indices = nullptr;
    d.top_k = 0;
    d.workspace = ws + scratch;
    d.workspace_bytes = a.workspace_bytes - scratch;
    if (mla_decode_supported(d)) {
        return launch_mla_decode(stream, d);
    }
    return launch_mfma_mla(stream, d);
}

}  // namespace xlite
