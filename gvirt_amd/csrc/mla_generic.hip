// Absorbed MLA attention for latent / rotary sizes the matrix-core kernels are not built for (the reference's
// smallest test model has kv_lora_rank 16, xlite/tests/kernels/mla.py:54): one 64-lane wave per (query row, head),
// no matrix instructions. Per 64 positions every lane scores one position (fp32 dot products over the latent
// and rotary columns), the wave keeps the online softmax (xlite/csrc/kernels/softmax_attn_aiv.h:595-647), and
// the lanes then own latent columns lane, lane + 64, ... of the output, the probabilities reaching them by
// shuffles; everything between the 16-bit inputs and the 16-bit output stays in fp32. Paged or dense cache,
// causal rule and top-k lists as in the other kernels.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr int kMaxColsPerLane = 8;   // kv_lora_rank <= 512

__global__ void __launch_bounds__(256)
mla_generic_kernel(const uint16_t *__restrict__ q_absorb, const uint16_t *__restrict__ qr,
                   const uint16_t *__restrict__ k_cache, const uint16_t *__restrict__ pe_cache,
                   uint16_t *__restrict__ out, const int32_t *__restrict__ query_start_loc,
                   const int32_t *__restrict__ lens, const int32_t *__restrict__ cached_lens,
                   const int32_t *__restrict__ block_tables, const int32_t *__restrict__ topk_indices, uint32_t total_rows,
                   uint32_t n_heads, uint32_t C, uint32_t R, uint32_t block_size, uint32_t batch, uint32_t max_num_blocks,
                   uint32_t dense_len, uint32_t top_k, float scale)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t rh = static_cast<uint64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (rh >= static_cast<uint64_t>(total_rows) * n_heads) {
        return;
    }
    const uint32_t t = static_cast<uint32_t>(rh / n_heads);
    // the sequence that owns row t: query_start_loc is a prefix sum
    uint32_t lo = 0, hi = batch;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) / 2;
        if (query_start_loc[mid] <= static_cast<int32_t>(t)) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    uint16_t *o = out + rh * C;
    const bool owned = lo > 0 && static_cast<int32_t>(t) < query_start_loc[lo - 1] + lens[lo - 1];
    const uint32_t seq = owned ? lo - 1 : 0;
    const bool dense = block_tables == nullptr;
    uint32_t causal = 0;
    if (owned) {
        const uint32_t clen = static_cast<uint32_t>(cached_lens[seq]);
        causal = dense ? min(clen + static_cast<uint32_t>(lens[seq]), dense_len)
                       : clen + (t - static_cast<uint32_t>(query_start_loc[seq])) + 1;
    }
    const bool listed = top_k != 0 && causal > top_k;
    const uint32_t n = listed ? top_k : causal;
    const int32_t *list = listed ? topk_indices + static_cast<uint64_t>(t) * top_k : nullptr;
    const int32_t *table = dense ? nullptr : block_tables + static_cast<uint64_t>(seq) * max_num_blocks;
    const uint16_t *qa = q_absorb + rh * C, *qp = qr + rh * R;

    float acc[kMaxColsPerLane];
#pragma unroll
    for (int i = 0; i < kMaxColsPerLane; i++) {
        acc[i] = 0.f;
    }
    float m_run = -INFINITY, l_run = 0.f;
    for (uint32_t j0 = 0; j0 < n; j0 += 64) {
        const uint32_t j = j0 + lane;
        // this lane's position: its cache row, or none
        bool ok = j < n;
        uint32_t pos = ok ? j : 0;
        if (listed && ok) {
            const int32_t x = list[j];
            ok = x >= 0 && static_cast<uint32_t>(x) < causal && (j == 0 || list[j - 1] != x);
            pos = ok ? static_cast<uint32_t>(x) : 0;
        }
        const uint64_t row = dense ? static_cast<uint64_t>(seq) * dense_len + pos
                                   : static_cast<uint64_t>(table[pos / block_size]) * block_size + pos % block_size;
        float s = -INFINITY;
        if (ok) {
            const uint16_t *k = k_cache + row * C, *pe = pe_cache + row * R;
            float dot = 0.f;
            for (uint32_t c = 0; c < C; c++) {
                dot += BF16::to_f32(qa[c]) * BF16::to_f32(k[c]);
            }
            for (uint32_t c = 0; c < R; c++) {
                dot += BF16::to_f32(qp[c]) * BF16::to_f32(pe[c]);
            }
            s = dot * scale;
        }
        float mx = s;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mx = fmaxf(mx, __shfl_xor(mx, d));
        }
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __expf(m_run - m_safe);
        float pr = ok ? __expf(s - m_safe) : 0.f;
        float ps = pr;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            ps += __shfl_xor(ps, d);
        }
        l_run = l_run * alpha + ps;
        m_run = m_new;
        const uint64_t my_row = row;
#pragma unroll
        for (int i = 0; i < kMaxColsPerLane; i++) {
            acc[i] *= alpha;
        }
        const uint32_t cnt = min(64u, n - j0);
        for (uint32_t u = 0; u < cnt; u++) {
            const float w = __shfl(pr, static_cast<int>(u));
            const uint64_t r_u = (static_cast<uint64_t>(__shfl(static_cast<uint32_t>(my_row >> 32), static_cast<int>(u))) << 32) |
                                 __shfl(static_cast<uint32_t>(my_row), static_cast<int>(u));
            if (w != 0.f) {   // uniform
                const uint16_t *k = k_cache + r_u * C;
#pragma unroll
                for (int i = 0; i < kMaxColsPerLane; i++) {
                    const uint32_t c = lane + 64 * i;
                    if (c < C) {
                        acc[i] += w * BF16::to_f32(k[c]);
                    }
                }
            }
        }
    }
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
#pragma unroll
    for (int i = 0; i < kMaxColsPerLane; i++) {
        const uint32_t c = lane + 64 * i;
        if (c < C) {
            o[c] = BF16::from_f32(acc[i] * inv);
        }
    }
}

}  // namespace

int launch_mla_generic(hipStream_t stream, const MlaArgs &a)
{
    XL_REQUIRE(a.dtype == XLITE_HIP_BF16, "mla: bf16 only");
    XL_REQUIRE(a.kv_lora_rank > 0 && a.kv_lora_rank <= 64 * kMaxColsPerLane, "kv_lora_rank must be at most 512");
    XL_REQUIRE(a.top_k == 0 || a.topk_indices != nullptr, "top_k > 0 needs topk_indices");
    const uint64_t rh = static_cast<uint64_t>(a.total_tokens) * a.n_heads;
    const dim3 grid(static_cast<uint32_t>((rh + 3) / 4), 1, 1);
    mla_generic_kernel<<<grid, 256, 0, stream>>>(
        static_cast<const uint16_t *>(a.q_absorb), static_cast<const uint16_t *>(a.qr), static_cast<const uint16_t *>(a.k_cache),
        static_cast<const uint16_t *>(a.pe_cache), static_cast<uint16_t *>(a.o_absorb), a.query_start_loc, a.lens, a.cached_lens,
        a.block_tables, a.topk_indices, a.total_tokens, a.n_heads, a.kv_lora_rank, a.rope_head_dim,
        a.block_tables == nullptr ? 1 : a.block_size, a.batch, a.max_num_blocks, a.dense_len, a.top_k, a.scale);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

}  // namespace xlite
