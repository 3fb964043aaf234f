// GQA flash-decode on the matrix cores, split along the KV axis.
//
// Workgroup = 8 wavefronts = one (sequence, KV tile). Every wave streams the positions of its KV
// range for ONE kv head (waves loop over kv heads when there are more than 8; when there are fewer,
// the spare waves take sub-ranges of the tile) and never synchronises with the other waves while
// streaming:
//   global -> registers : 1 KiB of consecutive cache bytes per wave-wide load, 16 bytes per lane
//   registers -> LDS    : rows stored 16-bit, row major, 16-byte chunks XOR-swizzled so that both
//                         read patterns below are bank-conflict free
//   S^T[token][head]  = K . Q^T    v_mfma_f32_16x16x32 (A = K rows via ds_read_b128, B = Q regs)
//   O^T[d][head]     += V^T . P^T  v_mfma_f32_16x16x32 (A = V^T via ds_read_b64_tr_b16, B = P regs)
// The query heads that share the kv head are the 16 MFMA columns (unused columns carry zeros), so
// one lane column owns one head: the online softmax needs two cross-lane exchanges per 32
// positions, and P leaves the first product in the register layout the second one consumes.
// int8 caches are widened to 16 bit (exactly) on their way into LDS; their per-position scales are
// applied to the scores (K) and to the probabilities (V).
//
// Each wave leaves an fp32 partial (max, sum, O) per query head in the workspace; the last
// workgroup of a query row to finish (ticket counter) merges all partials of the row.
//
// Replaces the split-KV path of the reference (xlite/csrc/kernels/flash_attention.h:323-628) for
// batches in which every sequence contributes one query row.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWaves = 8;
constexpr int kStep = 32;  // positions per inner step (one k=32 PV product)

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

template <typename T>
struct Mfma16;
template <>
struct Mfma16<BF16> {
    static __device__ __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma16<FP16> {
    static __device__ __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

struct DecodeMfmaParams {
    const uint16_t *q;
    const void *k_cache;
    const void *v_cache;
    const float *k_scale;
    const float *v_scale;
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;
    int32_t *counters;
    float *part_acc;   // [token][head][slot][D]
    float *part_ml;    // [token][head][slot][2]
    uint32_t q_row_stride;
    uint32_t n_heads, n_kv_heads, group;
    uint32_t block_size;
    uint32_t max_num_block;
    uint32_t tile_tokens;  // multiple of kStep * n_sub
    uint32_t n_sub;        // sub-ranges of a tile handled by different waves (kv heads < 8)
    uint32_t max_slots;    // max tiles * n_sub
};

// 8 cache elements (uint4 = 16-bit, uint2 = int8) -> 8 x 16-bit in a uint4
template <typename T>
__device__ __forceinline__ uint4 widen(const uint4 &raw) { return raw; }
template <typename T>
__device__ __forceinline__ uint4 widen(const uint2 &raw)
{
    const uint32_t src[2] = {raw.x, raw.y};
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t word = src[j / 2];
        const int sh = (j % 2) * 16;
        const float a = static_cast<float>(static_cast<int8_t>((word >> sh) & 0xff));
        const float b = static_cast<float>(static_cast<int8_t>((word >> (sh + 8)) & 0xff));
        w[j] = T::pack(a, b);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename T, int D, bool KV8>
__global__ void __launch_bounds__(kWaves * 64)
decode_mfma_kernel(const DecodeMfmaParams p)
{
    constexpr int CH = D / 8;            // 16-byte chunks per LDS row
    constexpr int ROWB = D * 2;          // LDS bytes per row
    constexpr int R256 = 256 / ROWB;     // rows per 256-byte bank window (1 or 2)
    constexpr int RPI = 64 / CH;         // cache rows fetched by one wave-wide load
    constexpr int NLD = kStep / RPI;     // loads per tile and tensor
    constexpr int KS = D / 32;           // k-steps of the QK product
    constexpr int MT = D / 16;           // 16-row tiles of O^T
    constexpr int TILE_BYTES = kStep * ROWB;
    typedef typename std::conditional<KV8, uint2, uint4>::type gvec_t;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t tile = blockIdx.x;
    const uint32_t seq = blockIdx.y;
    unsigned char *k_lds = smem + wave * 2 * TILE_BYTES;
    unsigned char *v_lds = k_lds + TILE_BYTES;

    // ---- lane roles ------------------------------------------------------------------------------
    const uint32_t col = lane & 15;       // MFMA column = query head inside the group
    const uint32_t jq = lane >> 4;        // 16-lane group
    // loader: row lr (+ RPI per load), 16-byte chunk lc
    const uint32_t lr = lane / CH, lc = lane % CH;

    // LDS write offsets of the loader (K and V swizzles differ), one per load of the tile
    uint32_t kw_off[NLD], vw_off[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
        const uint32_t row = i * RPI + lr;
        kw_off[i] = row * ROWB + ((lc ^ ((row / R256) % CH)) << 4);
        vw_off[i] = row * ROWB + ((lc ^ (2 * ((row / R256) % (CH / 2)))) << 4);
    }
    // LDS read offsets: K rows as the A operand of the QK product (sub tile 1 is +16 rows)
    uint32_t kr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        kr_off[ks] = col * ROWB + (((4 * ks + jq) ^ ((col / R256) % CH)) << 4);
    }
    // V^T through the transposing read: inside a 16-lane group lane 4*j' + q points at the four
    // elements [16*mt + 4q, +4) of position 4*jq + j'; it receives positions 4*jq .. 4*jq + 3 of
    // column 16*mt + (lane % 16)
    uint32_t vr_off[MT];
    {
        const uint32_t pos = 4 * jq + (col >> 2);
        const uint32_t q4 = lane & 3;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const uint32_t chunk = 2 * mt + (q4 >> 1);
            vr_off[mt] = pos * ROWB + ((chunk ^ (2 * ((pos / R256) % (CH / 2)))) << 4) + ((q4 & 1) << 3);
        }
    }

    const int32_t qlen = p.lens[seq];
    const int32_t clen = p.cached_lens[seq];
    const int32_t qstart = p.query_start_loc[seq];
    const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;
    const gvec_t *kc = static_cast<const gvec_t *>(p.k_cache);
    const gvec_t *vc = static_cast<const gvec_t *>(p.v_cache);
    const uint32_t row_vecs = static_cast<uint32_t>(CH);  // gvec_t per (position, kv head) row
    const uint32_t g_valid = p.group < 16 ? p.group : 16;
    const uint32_t sub_len = p.tile_tokens / p.n_sub;

    for (int32_t r = 0; r < qlen; r++) {
        const uint32_t tok = static_cast<uint32_t>(qstart + r);
        const uint32_t limit = static_cast<uint32_t>(clen + r + 1);
        const uint32_t n_tiles = ceil_div(limit, p.tile_tokens);
        if (tile >= n_tiles) {
            continue;
        }
        const uint32_t t0 = tile * p.tile_tokens;
        const uint32_t t1 = min(limit, t0 + p.tile_tokens);
        const bool single = n_tiles == 1 && p.n_sub == 1;

        // (kv head, sub range) passes of this wave
        for (uint32_t pass = wave; pass < p.n_kv_heads * p.n_sub; pass += kWaves) {
            const uint32_t kvh = pass % p.n_kv_heads;
            const uint32_t sub = pass / p.n_kv_heads;
            const uint32_t ta = min(t1, t0 + sub * sub_len);
            const uint32_t tb = min(t1, ta + sub_len);
            const uint32_t head0 = kvh * p.group;

            // ---- Q^T as the B operand: column = head, 8 consecutive elements per k group ----------
            uint4 qreg[KS];
            {
                const uint16_t *qrow = p.q + static_cast<uint64_t>(tok) * p.q_row_stride + static_cast<uint64_t>(head0 + col) * D;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    qreg[ks] = col < g_valid ? *reinterpret_cast<const uint4 *>(qrow + ks * 32 + jq * 8)
                                             : make_uint4(0, 0, 0, 0);
                }
            }
            f32x4_t O[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                O[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
            float m_run = -INFINITY, l_run = 0.f;

            // ---- stream [ta, tb) in steps of 32 positions; ta is a multiple of 32 -------------------
            gvec_t kreg[NLD], vreg[NLD];
            float ksc[2][4], vsc[2][4];
            // all 32 positions of a step lie in one block (block_size is a multiple of 32); the block
            // index and the offset inside it advance with the steps, no division in the loop
            uint32_t nxt_blk = ta / p.block_size, nxt_off = ta % p.block_size;
            auto issue = [&]() {
                const uint64_t phys = static_cast<uint32_t>(table[nxt_blk]);
                const uint64_t row0 = (phys * p.block_size + nxt_off) * p.n_kv_heads + kvh;
#pragma unroll
                for (int i = 0; i < NLD; i++) {
                    const uint64_t row = row0 + static_cast<uint64_t>(i * RPI + lr) * p.n_kv_heads;
                    kreg[i] = kc[row * row_vecs + lc];
                    vreg[i] = vc[row * row_vecs + lc];
                }
                if constexpr (KV8) {
                    // scales of the positions this lane will hold after the QK product
#pragma unroll
                    for (int s = 0; s < 2; s++) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const uint64_t row = row0 + static_cast<uint64_t>(16 * s + 4 * jq + e) * p.n_kv_heads;
                            ksc[s][e] = p.k_scale[row];
                            vsc[s][e] = p.v_scale[row];
                        }
                    }
                }
                nxt_off += kStep;
                if (nxt_off >= p.block_size) {
                    nxt_off = 0;
                    nxt_blk++;
                }
            };

            if (ta < tb) {
                issue();
            }
            for (uint32_t t = ta; t < tb; t += kStep) {
                // ---- registers -> LDS (rows beyond the end of the range become zeros) ----------------
                const bool partial = t + kStep > tb;
#pragma unroll
                for (int i = 0; i < NLD; i++) {
                    uint4 kv = widen<T>(kreg[i]);
                    uint4 vv = widen<T>(vreg[i]);
                    if (partial && t + i * RPI + lr >= tb) {
                        kv = make_uint4(0, 0, 0, 0);
                        vv = make_uint4(0, 0, 0, 0);
                    }
                    *reinterpret_cast<uint4 *>(k_lds + kw_off[i]) = kv;
                    *reinterpret_cast<uint4 *>(v_lds + vw_off[i]) = vv;
                }
                float kscale[2][4], vscale[2][4];
                if constexpr (KV8) {
#pragma unroll
                    for (int s = 0; s < 2; s++) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            kscale[s][e] = ksc[s][e];
                            vscale[s][e] = vsc[s][e];
                        }
                    }
                }
                if (t + kStep < tb) {
                    issue();
                }

                // ---- S^T = K . Q^T for the two 16-position sub tiles ----------------------------------
                f32x4_t S[2];
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    S[s] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ks++) {
                        const uint4 a = *reinterpret_cast<const uint4 *>(k_lds + kr_off[ks] + s * 16 * ROWB);
                        S[s] = Mfma16<T>::run(a, qreg[ks], S[s]);
                    }
                }

                // ---- online softmax; lane holds positions t + 16 s + 4 jq + e of head `col` -------------
                float mx = -INFINITY;
#pragma unroll
                for (int s = 0; s < 2; s++) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float v = S[s][e] * kLog2e;
                        if constexpr (KV8) {
                            v *= kscale[s][e];
                        }
                        v = (t + 16 * s + 4 * jq + e) < tb ? v : -INFINITY;  // also drops NaN of padding rows
                        S[s][e] = v;
                        mx = fmaxf(mx, v);
                    }
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                const float m_new = fmaxf(m_run, mx);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                m_run = m_new;
                float pe[2][4];
                float psum = 0.f;
#pragma unroll
                for (int s = 0; s < 2; s++) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float x = fast_exp2(S[s][e] - m_safe);
                        psum += x;
                        if constexpr (KV8) {
                            // the scale of a padding row may be anything (even NaN): keep p at 0 there
                            pe[s][e] = (t + 16 * s + 4 * jq + e) < tb ? x * vscale[s][e] : 0.f;
                        } else {
                            pe[s][e] = x;
                        }
                    }
                }
                l_run = l_run * alpha + psum;
                const uint4 pb = make_uint4(T::pack(pe[0][0], pe[0][1]), T::pack(pe[0][2], pe[0][3]),
                                            T::pack(pe[1][0], pe[1][1]), T::pack(pe[1][2], pe[1][3]));
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    O[mt][0] *= alpha;
                    O[mt][1] *= alpha;
                    O[mt][2] *= alpha;
                    O[mt][3] *= alpha;
                }

                // ---- O^T += V^T . P^T ---------------------------------------------------------------------
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
                    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_tr_ptr)(v_lds + vr_off[mt]));
                    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_tr_ptr)(v_lds + vr_off[mt] + 16 * ROWB));
                    const uint2 lo2 = __builtin_bit_cast(uint2, lo);
                    const uint2 hi2 = __builtin_bit_cast(uint2, hi);
                    O[mt] = Mfma16<T>::run(make_uint4(lo2.x, lo2.y, hi2.x, hi2.y), pb, O[mt]);
                }
            }

            // ---- this wave's result for (kv head, sub range) -----------------------------------------------
            float l_tot = l_run + __shfl_xor(l_run, 16);
            l_tot += __shfl_xor(l_tot, 32);
            if (col < g_valid) {
                // O^T lane layout: column = head `col`, rows 16 mt + 4 jq + e
                if (single) {
                    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
                    uint16_t *dst = p.out + (static_cast<uint64_t>(tok) * p.n_heads + head0 + col) * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        uint2 o;
                        o.x = T::pack(O[mt][0] * inv, O[mt][1] * inv);
                        o.y = T::pack(O[mt][2] * inv, O[mt][3] * inv);
                        *reinterpret_cast<uint2 *>(dst + mt * 16 + jq * 4) = o;
                    }
                } else {
                    const uint64_t slot = (static_cast<uint64_t>(tok) * p.n_heads + head0 + col) * p.max_slots + tile * p.n_sub + sub;
                    float *dst = p.part_acc + slot * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0) {
                        *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run, l_tot);
                    }
                }
            }
        }
        if (single) {
            continue;
        }

        // ---- publish, take a ticket; the last workgroup of the row merges all partials ---------------------
        __threadfence();
        __syncthreads();
        int32_t *flag = reinterpret_cast<int32_t *>(smem);
        int32_t *counter = p.counters + tok;
        if (threadIdx.x == 0) {
            *flag = atomicAdd(counter, 1);
        }
        __syncthreads();
        const bool last = *flag == static_cast<int32_t>(n_tiles) - 1;
        __syncthreads();
        if (!last) {
            continue;
        }
        __threadfence();
        const uint32_t n_slots = n_tiles * p.n_sub;
        constexpr int C4 = D / 4;
        for (uint32_t it = threadIdx.x; it < p.n_heads * C4; it += kWaves * 64) {
            const uint32_t head = it / C4, c = it % C4;
            const uint64_t base = (static_cast<uint64_t>(tok) * p.n_heads + head) * p.max_slots;
            float mm = -INFINITY;
            for (uint32_t s = 0; s < n_slots; s++) {
                mm = fmaxf(mm, p.part_ml[(base + s) * 2]);
            }
            const float ms = mm == -INFINITY ? 0.f : mm;
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
            float lsum = 0.f;
            for (uint32_t s = 0; s < n_slots; s++) {
                const float2 ml = *reinterpret_cast<const float2 *>(p.part_ml + (base + s) * 2);
                const float w = fast_exp2(ml.x - ms);
                lsum += ml.y * w;
                const float4 x = *reinterpret_cast<const float4 *>(p.part_acc + (base + s) * D + c * 4);
                acc.x += x.x * w;
                acc.y += x.y * w;
                acc.z += x.z * w;
                acc.w += x.w * w;
            }
            const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
            uint2 o;
            o.x = T::pack(acc.x * inv, acc.y * inv);
            o.y = T::pack(acc.z * inv, acc.w * inv);
            *reinterpret_cast<uint2 *>(p.out + (static_cast<uint64_t>(tok) * p.n_heads + head) * D + c * 4) = o;
        }
        if (threadIdx.x == 0) {
            *counter = 0;
        }
        __syncthreads();
    }
}

template <typename T, int D, bool KV8>
int launch_one(hipStream_t stream, const DecodeMfmaParams &p, uint32_t batch)
{
    constexpr size_t lds = static_cast<size_t>(kWaves) * 2 * kStep * D * 2;
    auto kernel = decode_mfma_kernel<T, D, KV8>;
    if (lds > 64 * 1024) {
        static bool configured = false;
        if (!configured) {
            XL_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            configured = true;
        }
    }
    dim3 grid(ceil_div(p.max_slots, p.n_sub), batch, 1);
    kernel<<<grid, kWaves * 64, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

}  // namespace

bool decode_mfma_supported(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size,
                           uint32_t total_tokens)
{
    const uint32_t group = n_heads / n_kv_heads;
    return (head_dim == 64 || head_dim == 128) && block_size % kStep == 0 && group <= 16 &&
           static_cast<size_t>(total_tokens) * sizeof(int32_t) <= XLITE_HIP_WS_COUNTER_BYTES;
}

void decode_mfma_plan(uint32_t batch, uint32_t n_kv_heads, uint32_t block_size, uint32_t max_num_block,
                      uint32_t *tile_tokens, uint32_t *n_sub, uint32_t *max_slots)
{
    const uint32_t subs = n_kv_heads >= kWaves ? 1 : kWaves / n_kv_heads;
    const uint64_t max_ctx = static_cast<uint64_t>(max_num_block) * block_size;
    const uint64_t quantum = static_cast<uint64_t>(kStep) * subs;
    // about one workgroup per compute unit if every sequence were as long as its block table
    // allows, but never tiles above 1024 positions (ragged batches balance through many tiles)
    // nor below 256 (the fp32 partials must stay a small fraction of the KV bytes)
    uint64_t tile = max_ctx * batch / 256;
    tile = tile > 1024 ? 1024 : (tile < 256 ? 256 : tile);
    tile = (tile + quantum - 1) / quantum * quantum;
    *tile_tokens = static_cast<uint32_t>(tile);
    *n_sub = subs;
    *max_slots = static_cast<uint32_t>((max_ctx + tile - 1) / tile) * subs;
}

size_t decode_mfma_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim, uint32_t max_slots)
{
    return XLITE_HIP_WS_COUNTER_BYTES +
           static_cast<size_t>(total_tokens) * n_heads * max_slots * (head_dim + 2) * sizeof(float);
}

int launch_decode_mfma(hipStream_t stream, const AttentionArgs &a)
{
    uint32_t tile, n_sub, max_slots;
    decode_mfma_plan(a.batch, a.n_kv_heads, a.block_size, a.max_num_block, &tile, &n_sub, &max_slots);
    const size_t need = decode_mfma_workspace_bytes(a.total_tokens, a.n_heads, a.head_dim, max_slots);
    if (max_slots > 1 && (a.workspace == nullptr || a.workspace_bytes < need)) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    DecodeMfmaParams p{};
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
    char *ws = static_cast<char *>(a.workspace);
    p.counters = reinterpret_cast<int32_t *>(ws);
    p.part_acc = ws ? reinterpret_cast<float *>(ws + XLITE_HIP_WS_COUNTER_BYTES) : nullptr;
    p.part_ml = ws ? p.part_acc + static_cast<size_t>(a.total_tokens) * a.n_heads * max_slots * a.head_dim : nullptr;
    p.q_row_stride = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim;
    p.n_heads = a.n_heads;
    p.n_kv_heads = a.n_kv_heads;
    p.group = a.n_heads / a.n_kv_heads;
    p.block_size = a.block_size;
    p.max_num_block = a.max_num_block;
    p.tile_tokens = tile;
    p.n_sub = n_sub;
    p.max_slots = max_slots;

    const bool kv8 = a.kv_dtype == XLITE_HIP_KV_INT8;
    const bool bf = a.dtype == XLITE_HIP_BF16;
    if (a.head_dim == 128) {
        if (bf) {
            return kv8 ? launch_one<BF16, 128, true>(stream, p, a.batch) : launch_one<BF16, 128, false>(stream, p, a.batch);
        }
        return kv8 ? launch_one<FP16, 128, true>(stream, p, a.batch) : launch_one<FP16, 128, false>(stream, p, a.batch);
    }
    if (bf) {
        return kv8 ? launch_one<BF16, 64, true>(stream, p, a.batch) : launch_one<BF16, 64, false>(stream, p, a.batch);
    }
    return kv8 ? launch_one<FP16, 64, true>(stream, p, a.batch) : launch_one<FP16, 64, false>(stream, p, a.batch);
}

}  // namespace xlite
