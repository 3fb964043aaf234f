// Quantised KV caches outside the streaming decode kernels (prefill and chunked prefill, mixed batches, decode
// shapes those kernels do not take): the blocks the batch can see are dequantised once into a compact 16-bit
// paged cache in the workspace, addressed by a block table of its own, and the 16-bit kernels run on that.
// The copy reads one byte and writes two per cached element, which a prefill's matrix work dwarfs; decode
// batches of the common shapes never come here (decode_mfma.hip reads the bytes directly).
#include "attention_common.h"

namespace xlite {

namespace {

template <typename T, int KVF>
__device__ __forceinline__ uint4 dequant8(const uint2 &raw, float scale)
{
    float x[8];
    if constexpr (KVF == XLITE_HIP_KV_INT8) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int32_t b = static_cast<int8_t>(((j < 4 ? raw.x : raw.y) >> (8 * (j % 4))) & 0xffu);
            x[j] = static_cast<float>(b) * scale;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int w = static_cast<int>(j < 4 ? raw.x : raw.y);
            float f;
            switch (j % 4) {
            case 0: f = __builtin_amdgcn_cvt_f32_fp8(w, 0); break;
            case 1: f = __builtin_amdgcn_cvt_f32_fp8(w, 1); break;
            case 2: f = __builtin_amdgcn_cvt_f32_fp8(w, 2); break;
            default: f = __builtin_amdgcn_cvt_f32_fp8(w, 3); break;
            }
            x[j] = f * scale;
        }
    }
    return make_uint4(T::pack(x[0], x[1]), T::pack(x[2], x[3]), T::pack(x[4], x[5]), T::pack(x[6], x[7]));
}

// workgroup (x = block j of the sequence, y = sequence, z = K | V): block j of sequence i lands at block
// i * max_num_block + j of the compact cache; blocks beyond the sequence's visible range are skipped.
template <typename T, int KVF>
__global__ void __launch_bounds__(256)
dequant_blocks_kernel(const unsigned char *__restrict__ k_cache, const unsigned char *__restrict__ v_cache,
                      const float *__restrict__ k_scale, const float *__restrict__ v_scale,
                      const int32_t *__restrict__ block_tables, const int32_t *__restrict__ lens,
                      const int32_t *__restrict__ cached_lens, uint16_t *__restrict__ k_out, uint16_t *__restrict__ v_out,
                      int32_t *__restrict__ table_out, uint32_t block_size, uint32_t max_num_block, uint32_t n_kv_heads,
                      uint32_t head_dim, uint32_t skip_single)
{
    const uint32_t j = blockIdx.x, i = blockIdx.y;
    const bool is_v = blockIdx.z != 0;
    const uint64_t out_block = static_cast<uint64_t>(i) * max_num_block + j;
    if (!is_v && threadIdx.x == 0) {
        table_out[out_block] = static_cast<int32_t>(out_block);
    }
    // sequences without rows need nothing; with skip_single those with one row read the bytes themselves
    const int32_t visible = lens[i] > 0 && !(skip_single && lens[i] == 1) ? cached_lens[i] + lens[i] : 0;
    if (static_cast<int64_t>(j) * block_size >= visible) {
        return;
    }
    const uint32_t rows_here = min(block_size, static_cast<uint32_t>(visible) - j * block_size);   // positions of the block
    const uint64_t phys = static_cast<uint32_t>(block_tables[out_block]);
    const uint32_t cpr = head_dim / 8;                               // 8-element chunks per (position, kv head) row
    const uint64_t chunks = static_cast<uint64_t>(rows_here) * n_kv_heads * cpr;
    const unsigned char *src = (is_v ? v_cache : k_cache) + phys * block_size * n_kv_heads * head_dim;
    const float *sc = (is_v ? v_scale : k_scale) + phys * block_size * n_kv_heads;
    uint16_t *dst = (is_v ? v_out : k_out) + out_block * block_size * n_kv_heads * head_dim;
    for (uint64_t c = threadIdx.x; c < chunks; c += blockDim.x) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(src + c * 8);
        *reinterpret_cast<uint4 *>(dst + c * 8) = dequant8<T, KVF>(raw, sc[c / cpr]);
    }
    // the rest of a partly visible block: zeros (the 16-bit kernels may load whole tiles and give the positions
    // past the end probability zero, which stale workspace bits that read as NaN would turn into NaN)
    const uint64_t all_chunks = static_cast<uint64_t>(block_size) * n_kv_heads * cpr;
    for (uint64_t c = chunks + threadIdx.x; c < all_chunks; c += blockDim.x) {
        *reinterpret_cast<uint4 *>(dst + c * 8) = make_uint4(0, 0, 0, 0);
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
    XL_REQUIRE(a->head_dim % 8 == 0, "head_dim must be a multiple of 8");
    const DequantLayout l = dequant_layout(a->n_kv_heads, a->head_dim, a->block_size, a->batch, a->max_num_block);
    if (a->workspace == nullptr || a->workspace_bytes < l.total) {
        return fail(XLITE_HIP_ENOSPC, __func__,
                    "workspace too small: this batch over a quantised cache needs " + std::to_string(l.total) +
                        " bytes for the 16-bit copy of its blocks, have " + std::to_string(a->workspace_bytes));
    }
    char *ws = static_cast<char *>(a->workspace);
    uint16_t *k_out = reinterpret_cast<uint16_t *>(ws);
    uint16_t *v_out = reinterpret_cast<uint16_t *>(ws + l.cache_bytes);
    int32_t *table = reinterpret_cast<int32_t *>(ws + 2 * l.cache_bytes);
    const dim3 grid(a->max_num_block, a->batch, 2);
    XL_REQUIRE(a->batch <= 65535, "more than 65535 sequences over a quantised cache outside the decode kernels");
    auto launch = [&](auto tag, auto kv) {
        using T = decltype(tag);
        dequant_blocks_kernel<T, decltype(kv)::value><<<grid, 256, 0, stream>>>(
            static_cast<const unsigned char *>(a->k_cache), static_cast<const unsigned char *>(a->v_cache), a->k_scale,
            a->v_scale, a->block_tables, a->lens, a->cached_lens, k_out, v_out, table, a->block_size, a->max_num_block,
            a->n_kv_heads, a->head_dim, a->rows_mode == kSkipSingle ? 1u : 0u);
    };
    using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
    using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
    if (a->dtype == XLITE_HIP_BF16) {
        a->kv_dtype == XLITE_HIP_KV_INT8 ? launch(BF16{}, I8{}) : launch(BF16{}, F8{});
    } else {
        a->kv_dtype == XLITE_HIP_KV_INT8 ? launch(FP16{}, I8{}) : launch(FP16{}, F8{});
    }
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

}  // namespace xlite
