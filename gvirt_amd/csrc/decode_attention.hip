// GQA flash-decode over a paged KV cache, split along the KV axis.
//
// Work item = (sequence, KV tile of `tile_tokens` positions, group of kv heads). A workgroup
// streams its tile once: every wave-wide load instruction fetches 1 KiB of consecutive cache
// rows with 16 bytes per lane; a row (token, kv head) is spread over LPR = head_dim/8 adjacent
// lanes, so the lanes of one row reduce the q.k partial sums with DPP butterflies and every
// lane keeps the softmax statistics of its rows plus 8 output columns for each of the G query
// heads that share the kv head. Dot products use v_dot2 (two 16-bit products + fp32 add per
// instruction): K against the packed query, and V against packed probabilities of two
// consecutive rows. Rows of different lane groups are merged through LDS at the end of the
// tile; tiles of one query row leave fp32 partials in the workspace, merged by a second small
// kernel (merge.hip).
//
// Replaces attention.h / flash_attention.h of the reference for batches in which every
// sequence contributes one query row (xlite/csrc/kernels/flash_attention.h:323-628).
#include "attention_common.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;

template <bool KV8>
struct KVec;
template <>
struct KVec<false> {
    typedef uint4 type;  // 8 x 16-bit
};
template <>
struct KVec<true> {
    typedef uint2 type;  // 8 x int8
};

// 8 cache elements -> 4 registers of packed 16-bit pairs (element 2j in the low half).
template <typename T>
__device__ __forceinline__ void unpack8(const uint4 &raw, uint32_t (&w)[4])
{
    w[0] = raw.x;
    w[1] = raw.y;
    w[2] = raw.z;
    w[3] = raw.w;
}
template <typename T>
__device__ __forceinline__ void unpack8(const uint2 &raw, uint32_t (&w)[4])
{
    // int8 -> float is exact, and so is float -> 16-bit for |x| <= 127
    const uint32_t src[2] = {raw.x, raw.y};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t word = src[j / 2];
        const int sh = (j % 2) * 16;
        const float a = static_cast<float>(static_cast<int8_t>((word >> sh) & 0xff));
        const float b = static_cast<float>(static_cast<int8_t>((word >> (sh + 8)) & 0xff));
        w[j] = T::pack(a, b);
    }
}

struct DecodeParams {
    const uint16_t *q;          // qkv rows
    const void *k_cache;
    const void *v_cache;
    const float *k_scale;
    const float *v_scale;
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;
    int32_t *part_cnt;          // [token][head] number of partial tiles (0: final value stored directly)
    float *part_acc;            // [token][head][tile][D]
    float *part_ml;             // [token][head][tile][2]
    uint32_t q_row_stride;      // elements between query rows
    uint32_t n_heads, n_kv_heads, group;  // group = n_heads / n_kv_heads
    uint32_t block_size;
    int32_t block_shift;        // log2(block_size) or -1
    uint32_t max_num_block;
    uint32_t tile_tokens;
    uint32_t max_tiles;
    uint32_t nkv_wg;            // kv heads handled by one workgroup
    uint32_t head_chunks;       // ceil(group / G)
};

template <typename T, int D, int G, int NW, int U, bool KV8>
__global__ void __launch_bounds__(NW * 64)
decode_kernel(const DecodeParams p)
{
    constexpr int LPR = D / 8;          // lanes per cache row
    constexpr int RPW = 64 / LPR;       // rows per wave-wide load
    constexpr int GPW = NW * RPW;       // lane groups per workgroup
    typedef typename KVec<KV8>::type kvec_t;

    extern __shared__ float smem[];

    const uint32_t tile = blockIdx.x;
    const uint32_t seq = blockIdx.y;
    const uint32_t zkv = blockIdx.z / p.head_chunks;
    const uint32_t hchunk = blockIdx.z % p.head_chunks;

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t sub = lane % LPR;
    const uint32_t gid = wave * RPW + lane / LPR;
    const uint32_t kvh_local = gid % p.nkv_wg;
    const uint32_t phase = gid / p.nkv_wg;
    const uint32_t tpi = GPW / p.nkv_wg;           // tokens per workgroup step
    const uint32_t kvh = zkv * p.nkv_wg + kvh_local;
    const uint32_t head0 = kvh * p.group + hchunk * G;  // first query head of this lane group
    const uint32_t g_valid = min(static_cast<uint32_t>(G), p.group - hchunk * G);

    const int32_t qlen = p.lens[seq];
    const int32_t clen = p.cached_lens[seq];
    const int32_t qstart = p.query_start_loc[seq];
    const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;

    const kvec_t *kc = static_cast<const kvec_t *>(p.k_cache);
    const kvec_t *vc = static_cast<const kvec_t *>(p.v_cache);

    for (int32_t r = 0; r < qlen; r++) {
        const uint32_t tok = static_cast<uint32_t>(qstart + r);
        const uint32_t limit = static_cast<uint32_t>(clen + r + 1);  // visible positions
        const uint32_t n_tiles = ceil_div(limit, p.tile_tokens);
        if (tile >= n_tiles) {
            continue;  // uniform for the whole workgroup: no thread skips a barrier alone
        }
        const uint32_t t0 = tile * p.tile_tokens;
        const uint32_t t1 = min(limit, t0 + p.tile_tokens);

        // ---- query: G heads x 8 elements, packed pairs ----------------------------------
        uint32_t q[G][4];
        {
            const uint16_t *qrow = p.q + static_cast<uint64_t>(tok) * p.q_row_stride;
#pragma unroll
            for (int h = 0; h < G; h++) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (static_cast<uint32_t>(h) < g_valid) {
                    v = *reinterpret_cast<const uint4 *>(qrow + static_cast<uint64_t>(head0 + h) * D + sub * 8);
                }
                q[h][0] = v.x;
                q[h][1] = v.y;
                q[h][2] = v.z;
                q[h][3] = v.w;
            }
        }

        float m[G], l[G], acc[G][8];
#pragma unroll
        for (int h = 0; h < G; h++) {
            m[h] = -INFINITY;
            l[h] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                acc[h][e] = 0.f;
            }
        }

        // ---- stream the tile -----------------------------------------------------------------
        const uint32_t my_first = t0 + phase;
        const uint32_t n_mine = my_first < t1 ? ceil_div(t1 - my_first, tpi) : 0u;
        // every lane group runs the same number of batches so that all waves reach the barriers
        const uint32_t n_batches = ceil_div(ceil_div(t1 - t0, tpi), U);

        auto row_index = [&](uint32_t n) -> uint64_t {
            // cache row (in units of one kv-head row) of this group's n-th token, clamped
            uint32_t t = my_first + n * tpi;
            t = t < t1 ? t : t1 - 1;
            const uint32_t b = p.block_shift >= 0 ? t >> p.block_shift : t / p.block_size;
            const uint32_t o = p.block_shift >= 0 ? t & (p.block_size - 1) : t % p.block_size;
            const uint64_t phys = static_cast<uint32_t>(table[b]);
            return (phys * p.block_size + o) * p.n_kv_heads + kvh;
        };

        kvec_t kreg[U], vreg[U];
        float ksc[U], vsc[U];
        auto issue = [&](uint32_t batch) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const uint64_t row = row_index(batch * U + u);
                kreg[u] = kc[row * LPR + sub];
                vreg[u] = vc[row * LPR + sub];
                if constexpr (KV8) {
                    ksc[u] = p.k_scale[row];
                    vsc[u] = p.v_scale[row];
                }
            }
        };

        if (n_batches > 0) {
            issue(0);
        }
        for (uint32_t b = 0; b < n_batches; b++) {
            uint32_t kw[U][4], vw[U][4];
            float kscale[U], vscale[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                unpack8<T>(kreg[u], kw[u]);
                unpack8<T>(vreg[u], vw[u]);
                if constexpr (KV8) {
                    kscale[u] = ksc[u];
                    vscale[u] = vsc[u];
                }
            }
            if (b + 1 < n_batches) {
                issue(b + 1);
            }

            float s[U][G];
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int h = 0; h < G; h++) {
                    float a = 0.f;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        a = T::dot2(kw[u][j], q[h][j], a);
                    }
                    s[u][h] = a;
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool valid = (b * U + u) < n_mine;
#pragma unroll
                for (int h = 0; h < G; h++) {
                    float v = group_sum<LPR>(s[u][h]);
                    if constexpr (KV8) {
                        v *= kscale[u];
                    }
                    s[u][h] = valid ? v * kLog2e : -INFINITY;
                }
            }

            float pr[U][G];
#pragma unroll
            for (int h = 0; h < G; h++) {
                float mb = s[0][h];
#pragma unroll
                for (int u = 1; u < U; u++) {
                    mb = fmaxf(mb, s[u][h]);
                }
                const float m_new = fmaxf(m[h], mb);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m[h] - m_safe);
                float psum = 0.f;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const float e = fast_exp2(s[u][h] - m_safe);
                    psum += e;
                    if constexpr (KV8) {
                        pr[u][h] = e * vscale[u];
                    } else {
                        pr[u][h] = e;
                    }
                }
                l[h] = l[h] * alpha + psum;
                m[h] = m_new;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    acc[h][e] *= alpha;
                }
            }

#pragma unroll
            for (int u = 0; u < U; u += 2) {
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t a = vw[u][j];
                    const uint32_t bq = (u + 1 < U) ? vw[u + 1][j] : 0u;
                    lo[j] = __builtin_amdgcn_perm(bq, a, 0x05040100u);  // (a.lo, b.lo)
                    hi[j] = __builtin_amdgcn_perm(bq, a, 0x07060302u);  // (a.hi, b.hi)
                }
#pragma unroll
                for (int h = 0; h < G; h++) {
                    const uint32_t pp = T::pack(pr[u][h], (u + 1 < U) ? pr[u + 1][h] : 0.f);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        acc[h][2 * j] = T::dot2(lo[j], pp, acc[h][2 * j]);
                        acc[h][2 * j + 1] = T::dot2(hi[j], pp, acc[h][2 * j + 1]);
                    }
                }
            }
        }

        // ---- merge the lane groups that share a kv head (binary tree through LDS) ------------
        constexpr int SLOT = G * (D + 2);  // floats per lane group: acc[G][D], m[G], l[G]
        for (uint32_t bit = tpi >> 1; bit >= 1; bit >>= 1) {
            const bool sender = (phase & bit) && phase < 2 * bit;
            if (sender) {
                float *slot = smem + static_cast<size_t>((phase - bit) * p.nkv_wg + kvh_local) * SLOT;
#pragma unroll
                for (int h = 0; h < G; h++) {
                    float4 *dst = reinterpret_cast<float4 *>(slot + h * D + sub * 8);
                    dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
                    dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
                    if (sub == 0) {
                        slot[G * D + h] = m[h];
                        slot[G * D + G + h] = l[h];
                    }
                }
            }
            __syncthreads();
            if (phase < bit) {
                const float *slot = smem + static_cast<size_t>(phase * p.nkv_wg + kvh_local) * SLOT;
#pragma unroll
                for (int h = 0; h < G; h++) {
                    const float m2 = slot[G * D + h];
                    const float l2 = slot[G * D + G + h];
                    const float m_new = fmaxf(m[h], m2);
                    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                    const float a1 = fast_exp2(m[h] - m_safe);
                    const float a2 = fast_exp2(m2 - m_safe);
                    const float4 *src = reinterpret_cast<const float4 *>(slot + h * D + sub * 8);
                    const float4 x0 = src[0], x1 = src[1];
                    acc[h][0] = acc[h][0] * a1 + x0.x * a2;
                    acc[h][1] = acc[h][1] * a1 + x0.y * a2;
                    acc[h][2] = acc[h][2] * a1 + x0.z * a2;
                    acc[h][3] = acc[h][3] * a1 + x0.w * a2;
                    acc[h][4] = acc[h][4] * a1 + x1.x * a2;
                    acc[h][5] = acc[h][5] * a1 + x1.y * a2;
                    acc[h][6] = acc[h][6] * a1 + x1.z * a2;
                    acc[h][7] = acc[h][7] * a1 + x1.w * a2;
                    l[h] = l[h] * a1 + l2 * a2;
                    m[h] = m_new;
                }
            }
            __syncthreads();
        }

        // ---- phase-0 groups own the tile result: final value, or a partial for the merge kernel -------
        if (phase == 0) {
#pragma unroll
            for (int h = 0; h < G; h++) {
                if (static_cast<uint32_t>(h) < g_valid) {
                    const uint64_t rh = static_cast<uint64_t>(tok) * p.n_heads + head0 + h;
                    if (n_tiles == 1) {
                        const float inv = l[h] > 0.f ? 1.0f / l[h] : 0.f;
                        uint4 o;
                        o.x = T::pack(acc[h][0] * inv, acc[h][1] * inv);
                        o.y = T::pack(acc[h][2] * inv, acc[h][3] * inv);
                        o.z = T::pack(acc[h][4] * inv, acc[h][5] * inv);
                        o.w = T::pack(acc[h][6] * inv, acc[h][7] * inv);
                        *reinterpret_cast<uint4 *>(p.out + rh * D + sub * 8) = o;
                    } else {
                        const uint64_t slot = rh * p.max_tiles + tile;
                        float4 *dst = reinterpret_cast<float4 *>(p.part_acc + slot * D + sub * 8);
                        dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
                        dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
                        if (sub == 0) {
                            *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m[h], l[h]);
                        }
                    }
                    if (sub == 0 && tile == 0 && p.part_cnt != nullptr) {
                        p.part_cnt[rh] = n_tiles == 1 ? 0 : static_cast<int32_t>(n_tiles);
                    }
                }
            }
        }
        __syncthreads();  // the LDS tree buffers are reused by the next query row
    }
}

template <typename T, int D, int G, bool KV8>
int launch_decode_g(hipStream_t stream, const DecodeParams &p, uint32_t batch, uint32_t zdim)
{
    constexpr int NW = 4;
    constexpr int U = 4;
    constexpr int LPR = D / 8, RPW = 64 / LPR, GPW = NW * RPW;
    const uint32_t tpi = GPW / p.nkv_wg;
    const size_t lds_tree = tpi > 1 ? static_cast<size_t>(GPW / 2) * G * (D + 2) * sizeof(float) : 0;
    const size_t lds = lds_tree < 16 ? 16 : lds_tree;
    dim3 grid(p.max_tiles, batch, zdim);
    decode_kernel<T, D, G, NW, U, KV8><<<grid, NW * 64, lds, stream>>>(p);
    return XLITE_HIP_OK;
}

template <typename T, int D, bool KV8>
int launch_decode_d(hipStream_t stream, const DecodeParams &p, uint32_t batch, uint32_t zdim, uint32_t g)
{
    switch (g) {
        case 1: return launch_decode_g<T, D, 1, KV8>(stream, p, batch, zdim);
        case 2: return launch_decode_g<T, D, 2, KV8>(stream, p, batch, zdim);
        case 3: return launch_decode_g<T, D, 3, KV8>(stream, p, batch, zdim);
        case 4: return launch_decode_g<T, D, 4, KV8>(stream, p, batch, zdim);
        case 5: return launch_decode_g<T, D, 5, KV8>(stream, p, batch, zdim);
        case 6: return launch_decode_g<T, D, 6, KV8>(stream, p, batch, zdim);
        case 7: return launch_decode_g<T, D, 7, KV8>(stream, p, batch, zdim);
        default: return launch_decode_g<T, D, 8, KV8>(stream, p, batch, zdim);
    }
}

}  // namespace

bool decode_supported(uint32_t head_dim) { return head_dim == 64 || head_dim == 128; }

uint32_t decode_pick_tile(uint32_t batch, uint32_t n_kv_heads, uint32_t block_size,
                          uint32_t max_num_block, uint32_t zdim)
{
    // Aim for about four resident workgroups per compute unit when every sequence is as long as
    // the block table allows; never go below 256 positions per tile so that the fp32 partials
    // stay a small fraction of the KV bytes.
    const uint64_t max_ctx = static_cast<uint64_t>(max_num_block) * block_size;
    const uint64_t target_wgs = 256ull * 4;
    uint64_t per_seq = target_wgs / (static_cast<uint64_t>(batch) * zdim);
    if (per_seq < 1) {
        per_seq = 1;
    }
    uint64_t tile = (max_ctx + per_seq - 1) / per_seq;
    tile = (tile + 127) / 128 * 128;
    if (tile < 256) {
        tile = 256;
    }
    if (tile > max_ctx) {
        tile = (max_ctx + 127) / 128 * 128;
    }
    return static_cast<uint32_t>(tile);
}

void decode_geometry(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t *g_kernel,
                     uint32_t *head_chunks, uint32_t *nkv_wg, uint32_t *zdim)
{
    const uint32_t group = n_heads / n_kv_heads;
    *g_kernel = group < 8 ? group : 8;
    *head_chunks = ceil_div(group, *g_kernel);
    const uint32_t gpw = 4 * (64 / (head_dim / 8));
    // all kv heads in one workgroup when they tile its lane groups evenly, else one per workgroup
    *nkv_wg = (n_kv_heads <= gpw && gpw % n_kv_heads == 0) ? n_kv_heads : 1;
    *zdim = (n_kv_heads / *nkv_wg) * *head_chunks;
}

size_t decode_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                              uint32_t max_tiles)
{
    return max_tiles > 1 ? partial_bytes(total_tokens, n_heads, head_dim, max_tiles) : 0;
}

int launch_decode(hipStream_t stream, const AttentionArgs &a, uint32_t tile_tokens)
{
    uint32_t g_kernel, head_chunks, nkv_wg, zdim;
    decode_geometry(a.n_heads, a.n_kv_heads, a.head_dim, &g_kernel, &head_chunks, &nkv_wg, &zdim);
    const uint32_t max_ctx = a.max_num_block * a.block_size;
    const uint32_t max_tiles = ceil_div(max_ctx, tile_tokens);
    const size_t need = decode_workspace_bytes(a.total_tokens, a.n_heads, a.head_dim, max_tiles);
    if (max_tiles > 1 && (a.workspace == nullptr || a.workspace_bytes < need)) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    const PartialBuffers pb = max_tiles > 1 ? carve_partials(a.workspace, a.total_tokens, a.n_heads, a.head_dim, max_tiles)
                                            : PartialBuffers{};

    DecodeParams p;
    p.q = static_cast<const uint16_t *>(a.qkv);
    p.k_cache = a.k_cache;
    p.v_cache = a.v_cache;
    p.k_scale = a.k_scale;
    p.v_scale = a.v_scale;
    p.out = static_cast<uint16_t *>(a.output);
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.part_cnt = pb.cnt;
    p.part_acc = pb.acc;
    p.part_ml = pb.ml;
    p.q_row_stride = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim;
    p.n_heads = a.n_heads;
    p.n_kv_heads = a.n_kv_heads;
    p.group = a.n_heads / a.n_kv_heads;
    p.block_size = a.block_size;
    p.block_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
    p.max_num_block = a.max_num_block;
    p.tile_tokens = tile_tokens;
    p.max_tiles = max_tiles;
    p.nkv_wg = nkv_wg;
    p.head_chunks = head_chunks;

    const bool kv8 = a.kv_dtype == XLITE_HIP_KV_INT8;
    const bool bf = a.dtype == XLITE_HIP_BF16;
    const uint32_t g = g_kernel;
    int rc;
    if (a.head_dim == 128) {
        if (bf) {
            rc = kv8 ? launch_decode_d<BF16, 128, true>(stream, p, a.batch, zdim, g)
                     : launch_decode_d<BF16, 128, false>(stream, p, a.batch, zdim, g);
        } else {
            rc = kv8 ? launch_decode_d<FP16, 128, true>(stream, p, a.batch, zdim, g)
                     : launch_decode_d<FP16, 128, false>(stream, p, a.batch, zdim, g);
        }
    } else if (bf) {
        rc = kv8 ? launch_decode_d<BF16, 64, true>(stream, p, a.batch, zdim, g)
                 : launch_decode_d<BF16, 64, false>(stream, p, a.batch, zdim, g);
    } else {
        rc = kv8 ? launch_decode_d<FP16, 64, true>(stream, p, a.batch, zdim, g)
                 : launch_decode_d<FP16, 64, false>(stream, p, a.batch, zdim, g);
    }
    if (rc != XLITE_HIP_OK || max_tiles == 1) {
        return rc;
    }
    XL_LAUNCH_CHECK();
    return launch_merge(stream, a.dtype, a.output, pb, a.total_tokens, a.n_heads, a.head_dim, max_tiles);
}

}  // namespace xlite
