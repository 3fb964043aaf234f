// Dense attention on the bf16/fp16 matrix cores: chunked causal prefill over the paged GQA cache
// and DeepSeek-style absorbed MLA (paged or dense latent cache).
//
// One workgroup = 4 wavefronts = 128 "M rows", an M row being one (query position, query head)
// pair of a kv head (GQA) or of the single latent head (MLA). Each wave owns 32 M rows and keeps
// their query vectors in registers as the B operand of v_mfma_f32_32x32x16; the workgroup walks
// the visible KV positions in tiles of BN tokens staged in LDS:
//     S^T[token][m]  = K[token][:] . Q[m][:]          (A = K rows from LDS, B = Q registers)
//     O^T[d][m]     += V^T[d][token] . P^T[token][m]   (A = transposed V from LDS, B = P registers)
// Computing the transposed products keeps one M row per lane column, so the online softmax needs
// a single cross-lane exchange per tile, and the probabilities leave the QK accumulators already
// in the register layout the PV product wants (the token order inside a 16-token group is
// permuted identically on the V^T side). Scores and outputs accumulate in fp32; P is rounded to
// the 16-bit storage type before the second product, as in the reference (softmax_attn_aiv.h:904-908).
//
// The KV range of an M tile can be split across workgroups (grid.x); their partial (max, sum, O)
// are merged by a second small kernel (merge.hip).
//
// Replaces attention.h / flash_attention.h for batches with multi-token queries
// (xlite/csrc/kernels/attention.h:308-492) and mla_v2.h / flash_mla_v2.h / mla_v3.h.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kMTile = kWaves * 32;

template <typename T>
struct Mfma;
template <>
struct Mfma<BF16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma<FP16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

struct MfmaParams {
    const uint16_t *q0;   // first DQ0 columns of a query row
    const uint16_t *q1;   // remaining DQ1 columns (MLA rope part)
    const uint16_t *k0;   // cache rows matching q0
    const uint16_t *k1;   // cache rows matching q1
    const uint16_t *v;    // separate value cache (GQA)
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;  // nullptr: dense cache of dense_len rows per sequence, no causality
    int32_t *part_cnt;   // [token][head] number of partial splits (0: final value stored directly)
    float *part_acc;
    float *part_ml;
    uint32_t q0_tok_stride, q0_head_stride, q1_tok_stride, q1_head_stride;
    uint32_t k0_tok_stride, k1_tok_stride;   // elements between consecutive cache rows
    uint32_t out_tok_stride;
    uint32_t rows_per_pos;       // G: query heads sharing the kv head
    uint32_t n_heads;
    uint32_t batch;
    uint32_t block_size;
    int32_t block_shift;
    uint32_t max_num_block;
    uint32_t dense_len;
    uint32_t split_len;
    uint32_t max_splits;
    float scale_log2e;
    uint32_t table_in_lds;   // 1: the launch reserved LDS for the sequence's block-table row (max_num_block words)
};

// position inside a 16-token group at which token offset o is stored in the transposed V tile, so
// that the eight tokens a lane's P registers hold are contiguous
__device__ __forceinline__ uint32_t vt_pos(uint32_t o)
{
    return (o & ~15u) | (((o >> 2) & 1u) << 3) | (((o >> 3) & 1u) << 2) | (o & 3u);
}

template <typename T, int DQ0, int DQ1, int DV, int BN, bool SEPARATE_V>
__global__ void __launch_bounds__(kThreads)
mfma_attention_kernel(const MfmaParams p)
{
    constexpr int DQK = DQ0 + DQ1;
    constexpr int KS = DQK / 16;             // k-steps of the QK product
    constexpr int NT = BN / 32;              // 32-token sub tiles
    constexpr int DT = DV / 32;              // 32-row tiles of O^T
    constexpr int KSTRIDE = DQK + 8;         // LDS row stride of the K tile, elements
    constexpr int VSTRIDE = BN + 8;          // LDS row stride of the V^T tile, elements
    constexpr int CPR = DQK / 8;             // 16-byte chunks per K row
    constexpr int CPR0 = DQ0 / 8;
    constexpr int VCPR = DV / 8;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t *Ks = reinterpret_cast<uint16_t *>(smem_raw);
    uint16_t *Vt = Ks + BN * KSTRIDE;
    uint64_t *rowidx = reinterpret_cast<uint64_t *>(Vt + DV * VSTRIDE);
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(rowidx + BN);

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t col = lane & 31;
    const uint32_t half = lane >> 5;
    const uint32_t split = blockIdx.x;
    const uint32_t kvh = blockIdx.z;
    const uint32_t G = p.rows_per_pos;

    // ---- locate the M tile. Sequence i owns the tile ids from floor(query_start_loc[i] * G / 128) + i up to
    // the next sequence's first one: at least its ceil(lens[i] * G / 128) tiles (the surplus ids are empty),
    // and a formula of the prefix sums the caller provides, so the owner is found by bisection.
    auto first_id = [&](uint32_t i) {
        return static_cast<uint32_t>((static_cast<uint64_t>(p.query_start_loc[i]) * G) / kMTile) + i;
    };
    uint32_t seq = 0;
    {
        uint32_t hi = p.batch;   // first_id(seq) <= blockIdx.y < first_id(hi); first_id(0) == 0
        while (hi - seq > 1) {
            const uint32_t mid = (seq + hi) >> 1;
            if (first_id(mid) <= blockIdx.y) {
                seq = mid;
            } else {
                hi = mid;
            }
        }
    }
    const uint32_t mt = blockIdx.y - first_id(seq);
    const int32_t qlen = p.lens[seq];
    if (qlen <= 0 || mt >= ceil_div(static_cast<uint32_t>(qlen) * G, kMTile)) {
        return;
    }
    const int32_t clen = p.cached_lens[seq];
    const int32_t qstart = p.query_start_loc[seq];
    const uint32_t m_rows = static_cast<uint32_t>(qlen) * G;
    const uint32_t m_first = mt * kMTile;
    const uint32_t m_last = min(m_rows, m_first + kMTile) - 1;
    const bool dense = p.block_tables == nullptr;
    const uint32_t total_kv = dense ? min(static_cast<uint32_t>(clen + qlen), p.dense_len)
                                    : static_cast<uint32_t>(clen + qlen);
    // keys visible to at least one row of the tile
    const uint32_t limit_max = dense ? total_kv : static_cast<uint32_t>(clen) + m_last / G + 1;
    const uint32_t n_splits = ceil_div(limit_max, p.split_len);
    if (split >= n_splits) {
        return;
    }
    const uint32_t range_begin = split * p.split_len;
    const uint32_t range_end = min(limit_max, range_begin + p.split_len);

    // ---- this lane's M row -----------------------------------------------------------------------
    const uint32_t m = m_first + wave * 32 + col;
    const bool m_valid = m < m_rows;
    const uint32_t qpos = m_valid ? m / G : 0;
    const uint32_t hh = m_valid ? m % G : 0;
    const uint32_t head = kvh * G + hh;
    const uint32_t tok = static_cast<uint32_t>(qstart) + qpos;
    const uint32_t vis = !m_valid ? 0u
                         : min(range_end, dense ? total_kv : static_cast<uint32_t>(clen) + qpos + 1);

    uint4 qreg[KS];
    {
        const uint16_t *src0 = p.q0 + static_cast<uint64_t>(tok) * p.q0_tok_stride + static_cast<uint64_t>(head) * p.q0_head_stride;
        const uint16_t *src1 = DQ1 ? p.q1 + static_cast<uint64_t>(tok) * p.q1_tok_stride + static_cast<uint64_t>(head) * p.q1_head_stride : nullptr;
        // (every lane loads: rows past the tile's end point at the sequence's first row and are cleared below; a load
        // under a condition is compiled into a branch with a wait of its own, one trip to memory per load)
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int c = ks * 16 + half * 8;
            qreg[ks] = (ks * 16 < DQ0) ? *reinterpret_cast<const uint4 *>(src0 + c)
                                       : *reinterpret_cast<const uint4 *>(src1 + (c - DQ0));
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
            qreg[ks] = m_valid ? qreg[ks] : make_uint4(0, 0, 0, 0);
        }
    }

    f32x16_t O[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            O[dt][k] = 0.f;
        }
    }
    float m_run = -INFINITY, l_run = 0.f;

    const int32_t *table = dense ? nullptr : p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;

    // ---- staging. The cache rows of a tile travel through registers: a thread's K chunks (and, for a separate value
    // cache, its V chunks: four consecutive positions of one 16-byte column group at a time, so that the transposed
    // tile is written four positions = 8 bytes per store) are requested one tile ahead, all loads unconditional from
    // clamped positions (rows at or beyond the end of the range repeat its last row: finite values whose
    // probabilities are zero), and go to LDS when the previous tile has been consumed.
    constexpr int K_ITEMS = BN * CPR;                       // 16-byte chunks of a K tile
    constexpr int K_IT = (K_ITEMS + kThreads - 1) / kThreads;
    constexpr int V_ITEMS = SEPARATE_V ? (BN / 4) * VCPR : 0;   // (four positions, chunk) items of a V tile
    constexpr int V_IT = (V_ITEMS + kThreads - 1) / kThreads;
    uint32_t kbuf[K_IT][4];                       // (plain words: the staging registers must not end up in scratch memory)
    uint32_t vbuf[V_IT > 0 ? V_IT : 1][4][4];
    auto cache_row = [&](uint32_t t) __attribute__((always_inline)) -> uint64_t {
        t = t < range_end ? t : range_end - 1;
        if (dense) {
            return static_cast<uint64_t>(seq) * p.dense_len + t;
        }
        const uint32_t b = p.block_shift >= 0 ? t >> p.block_shift : t / p.block_size;
        const uint32_t o = p.block_shift >= 0 ? t & (p.block_size - 1) : t % p.block_size;
        // (from LDS when the row was staged: a load from memory here sits between the two barriers of every tile)
        const uint32_t entry = p.table_in_lds ? tbl_lds[b] : static_cast<uint32_t>(table[b]);
        return static_cast<uint64_t>(entry) * p.block_size + o;
    };
    if (!dense && p.table_in_lds) {
        const uint32_t b_lo = (p.block_shift >= 0 ? range_begin >> p.block_shift : range_begin / p.block_size);
        const uint32_t b_hi = (p.block_shift >= 0 ? (range_end - 1) >> p.block_shift : (range_end - 1) / p.block_size);
        for (uint32_t b = b_lo + threadIdx.x; b <= b_hi; b += kThreads) {
            tbl_lds[b] = static_cast<uint32_t>(table[b]);
        }
        __syncthreads();
    }
    // the tile's rows are looked up by the first BN threads and shared through LDS (two barriers around the table)
    auto lookup = [&](uint32_t j0) __attribute__((always_inline)) {
        if (threadIdx.x < BN) {
            rowidx[threadIdx.x] = cache_row(j0 + threadIdx.x);
        }
    };
    auto request = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            const uint32_t c = min(threadIdx.x + it * kThreads, static_cast<uint32_t>(K_ITEMS - 1));
            const uint32_t r = c / CPR, cc = c % CPR;
            const uint64_t row = rowidx[r];
            const uint16_t *src = (DQ1 == 0 || cc < CPR0) ? p.k0 + row * p.k0_tok_stride + (SEPARATE_V ? kvh * DQ0 : 0) + cc * 8
                                                          : p.k1 + row * p.k1_tok_stride + (cc - CPR0) * 8;
            const uint4 x = *reinterpret_cast<const uint4 *>(src);
            kbuf[it][0] = x.x;
            kbuf[it][1] = x.y;
            kbuf[it][2] = x.z;
            kbuf[it][3] = x.w;
        }
        if constexpr (SEPARATE_V) {
#pragma unroll
            for (int it = 0; it < V_IT; it++) {
                const uint32_t c = min(threadIdx.x + it * kThreads, static_cast<uint32_t>(V_ITEMS - 1));
                const uint32_t g = c % (BN / 4), cc = c / (BN / 4);   // (position groups across the lanes: see `stage`)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint4 x = *reinterpret_cast<const uint4 *>(p.v + rowidx[4 * g + j] * p.k0_tok_stride + kvh * DV + cc * 8);
                    vbuf[it][j][0] = x.x;
                    vbuf[it][j][1] = x.y;
                    vbuf[it][j][2] = x.z;
                    vbuf[it][j][3] = x.w;
                }
            }
        }
    };
    auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < K_IT; it++) {
            const uint32_t c = threadIdx.x + it * kThreads;
            if (K_ITEMS % kThreads == 0 || c < K_ITEMS) {
                const uint32_t r = c / CPR, cc = c % CPR;
                *reinterpret_cast<uint4 *>(Ks + r * KSTRIDE + cc * 8) = make_uint4(kbuf[it][0], kbuf[it][1], kbuf[it][2], kbuf[it][3]);
                if constexpr (!SEPARATE_V) {   // the value is the first DV columns of the same row
                    if (cc < VCPR) {
                        const uint32_t pos = vt_pos(r);
#pragma unroll
                        for (int i = 0; i < 8; i++) {
                            Vt[(cc * 8 + i) * VSTRIDE + pos] = static_cast<uint16_t>(kbuf[it][i / 2] >> ((i & 1) * 16));
                        }
                    }
                }
            }
        }
        if constexpr (SEPARATE_V) {
#pragma unroll
            for (int it = 0; it < V_IT; it++) {
                const uint32_t c = threadIdx.x + it * kThreads;
                if (V_ITEMS % kThreads == 0 || c < V_ITEMS) {
                    const uint32_t g = c % (BN / 4), cc = c / (BN / 4);   // (position groups across the lanes: see `stage`)
                    // positions 4 g .. 4 g + 3 stay next to each other. A wave's lanes are the 16 position groups of four
                    // consecutive chunks: consecutive 8-byte words of a V^T row (with the chunk across the lanes, a
                    // row of 8 x 144 bytes apart, every store was a 32-way bank conflict: 4300 of a tile's 12600 cycles)
                    const uint32_t pos = vt_pos(4 * g);
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        // element i of the four positions
                        const int wi = i / 2, sh = (i & 1) * 16;
                        uint2 o;
                        o.x = ((vbuf[it][0][wi] >> sh) & 0xffffu) | ((vbuf[it][1][wi] >> sh) << 16);
                        o.y = ((vbuf[it][2][wi] >> sh) & 0xffffu) | ((vbuf[it][3][wi] >> sh) << 16);
                        *reinterpret_cast<uint2 *>(Vt + (cc * 8 + i) * VSTRIDE + pos) = o;
                    }
                }
            }
        }
    };
    // (the latent-cache instantiation has no registers to spare: it requests a tile when it needs it)
    constexpr bool AHEAD = SEPARATE_V;
    lookup(range_begin);
    __syncthreads();
    if constexpr (AHEAD) {
        request();
    }

    for (uint32_t j0 = range_begin; j0 < range_end; j0 += BN) {
        __syncthreads();  // previous tile fully consumed (and its row table read by every request)
        if constexpr (AHEAD) {
            stage();
        } else {
            // chunk by chunk, in a loop the compiler keeps rolled: one staging register set
#pragma unroll 1
            for (uint32_t c = threadIdx.x; c < K_ITEMS; c += kThreads) {
                const uint32_t r = c / CPR, cc = c % CPR;
                const uint64_t row = rowidx[r];
                const uint16_t *src = (DQ1 == 0 || cc < CPR0) ? p.k0 + row * p.k0_tok_stride + (SEPARATE_V ? kvh * DQ0 : 0) + cc * 8
                                                              : p.k1 + row * p.k1_tok_stride + (cc - CPR0) * 8;
                const uint4 val = *reinterpret_cast<const uint4 *>(src);
                *reinterpret_cast<uint4 *>(Ks + r * KSTRIDE + cc * 8) = val;
                if (cc < VCPR) {
                    const uint32_t pos = vt_pos(r);
                    const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        Vt[(cc * 8 + i) * VSTRIDE + pos] = static_cast<uint16_t>(w[i / 2] >> ((i & 1) * 16));
                    }
                }
            }
            __syncthreads();   // the row table has been read: the next tile's may be written
        }
        if (j0 + BN < range_end) {
            lookup(j0 + BN);
        }
        __syncthreads();
        if constexpr (AHEAD) {
            if (j0 + BN < range_end) {
                request();   // the next tile's rows are in flight during this tile's products
            }
        }

        // ---- S^T = K . Q^T ----------------------------------------------------------------------------
        // (k-steps outermost: the NT score tiles are independent accumulation chains whose products alternate, and the
        // operands of a k-step are read from LDS while the products of the one before run)
        f32x16_t S[NT];
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                S[nt][k] = 0.f;
            }
        }
        {
            uint4 a_cur[NT], a_nxt[NT];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                a_cur[nt] = *reinterpret_cast<const uint4 *>(Ks + (nt * 32 + col) * KSTRIDE + half * 8);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                if (ks + 1 < KS) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) {
                        a_nxt[nt] = *reinterpret_cast<const uint4 *>(Ks + (nt * 32 + col) * KSTRIDE + (ks + 1) * 16 + half * 8);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);   // (left alone the scheduler sinks the reads to just ahead of their products)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    S[nt] = Mfma<T>::run(a_cur[nt], qreg[ks], S[nt]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    a_cur[nt] = a_nxt[nt];
                }
            }
        }

        // ---- online softmax over the tile -----------------------------------------------------------------
        float mx = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const uint32_t t = j0 + nt * 32 + (k / 4) * 8 + half * 4 + (k % 4);
                const float s = t < vis ? S[nt][k] * p.scale_log2e : -INFINITY;
                S[nt][k] = s;
                mx = fmaxf(mx, s);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        m_run = m_new;
        uint4 pb[NT][2];
        float psum = 0.f;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            uint32_t w[8];
#pragma unroll
            for (int k = 0; k < 16; k += 2) {
                const float e0 = fast_exp2(S[nt][k] - m_safe);
                const float e1 = fast_exp2(S[nt][k + 1] - m_safe);
                psum += e0 + e1;
                w[k / 2] = T::pack(e0, e1);
            }
            pb[nt][0] = make_uint4(w[0], w[1], w[2], w[3]);
            pb[nt][1] = make_uint4(w[4], w[5], w[6], w[7]);
        }
        l_run = l_run * alpha + psum;
        if (!SEPARATE_V || __any(alpha != 1.0f)) {   // the running maximum rarely moves after the first tiles (the latent-cache
                                                     // instantiation, short of registers, keeps one path)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    O[dt][k] *= alpha;
                }
            }
        }

        // ---- O^T += V^T . P^T -------------------------------------------------------------------------------
        // (the position k-steps outermost: the DT accumulator tiles are independent, their products go back to back)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const uint4 a = *reinterpret_cast<const uint4 *>(Vt + (dt * 32 + col) * VSTRIDE + nt * 32 + kk * 16 + half * 8);
                    O[dt] = Mfma<T>::run(a, pb[nt][kk], O[dt]);
                }
            }
        }
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);

    if (m_valid) {
        const uint64_t rh = static_cast<uint64_t>(tok) * p.n_heads + head;
        if (n_splits == 1) {
            const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
            uint16_t *dst = p.out + static_cast<uint64_t>(tok) * p.out_tok_stride + static_cast<uint64_t>(head) * DV;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int kg = 0; kg < 4; kg++) {
                    uint2 o;
                    o.x = T::pack(O[dt][kg * 4] * inv, O[dt][kg * 4 + 1] * inv);
                    o.y = T::pack(O[dt][kg * 4 + 2] * inv, O[dt][kg * 4 + 3] * inv);
                    *reinterpret_cast<uint2 *>(dst + dt * 32 + kg * 8 + half * 4) = o;
                }
            }
        } else {
            // partial result of this split; a second kernel merges the splits of every row (merge.hip)
            const uint64_t slot = rh * p.max_splits + split;
            float *dst = p.part_acc + slot * DV;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int kg = 0; kg < 4; kg++) {
                    *reinterpret_cast<float4 *>(dst + dt * 32 + kg * 8 + half * 4) =
                        make_float4(O[dt][kg * 4], O[dt][kg * 4 + 1], O[dt][kg * 4 + 2], O[dt][kg * 4 + 3]);
                }
            }
            if (half == 0) {
                *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run, l_tot);
            }
        }
        if (half == 0 && split == 0 && p.part_cnt != nullptr) {
            p.part_cnt[rh] = n_splits == 1 ? 0 : static_cast<int32_t>(n_splits);
        }
    }
}

template <int DQK, int DV, int BN>
constexpr size_t lds_bytes()
{
    return static_cast<size_t>(BN) * (DQK + 8) * 2 + static_cast<size_t>(DV) * (BN + 8) * 2 + BN * 8;
}

template <typename T, int DQ0, int DQ1, int DV, int BN, bool SEPARATE_V>
int launch_kernel(hipStream_t stream, const MfmaParams &p_in, dim3 grid)
{
    MfmaParams p = p_in;
    size_t lds = lds_bytes<DQ0 + DQ1, DV, BN>();
    // the sequence's block-table row behind the tiles, when it fits
    p.table_in_lds = p.block_tables != nullptr && lds + static_cast<size_t>(p.max_num_block) * 4 <= 150 * 1024 ? 1u : 0u;
    if (p.table_in_lds) {
        lds += static_cast<size_t>(p.max_num_block) * 4;
    }
    auto kernel = mfma_attention_kernel<T, DQ0, DQ1, DV, BN, SEPARATE_V>;
    if (lds > 64 * 1024) {
        if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) {
            return rc;
        }
    }
    kernel<<<grid, kThreads, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

void fill_common(MfmaParams &p, const PartialBuffers &pb)
{
    p.part_cnt = pb.cnt;
    p.part_acc = pb.acc;
    p.part_ml = pb.ml;
}

}  // namespace

bool mfma_gqa_supported(uint32_t head_dim) { return head_dim == 64 || head_dim == 128 || head_dim == 256; }

size_t mfma_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t dv, uint32_t splits)
{
    return splits <= 1 ? 0 : partial_bytes(total_tokens, n_heads, dv, splits);
}

// Number of KV splits so that about two workgroups per compute unit exist; the split length is a
// multiple of `tile` tokens.
uint32_t mfma_pick_splits(uint32_t total_tokens, uint32_t rows_per_token, uint32_t batch,
                          uint32_t parallel_heads, uint32_t max_ctx, uint32_t tile)
{
    const uint64_t m_tiles = (static_cast<uint64_t>(total_tokens) * rows_per_token + kMTile - 1) / kMTile + batch;
    const uint64_t base = m_tiles * parallel_heads;
    const uint64_t want = 512;
    if (base >= want) {
        return 1;
    }
    uint64_t splits = (want + base - 1) / base;
    const uint64_t max_by_len = (max_ctx + 4 * tile - 1) / (4 * tile);  // at least four tiles each
    if (splits > max_by_len) {
        splits = max_by_len;
    }
    return static_cast<uint32_t>(splits < 1 ? 1 : splits);
}

int launch_mfma_gqa(hipStream_t stream, const AttentionArgs &a)
{
    constexpr int BN = 64;
    const uint32_t G = a.n_heads / a.n_kv_heads;
    const uint32_t max_ctx = a.max_num_block * a.block_size;
    uint32_t splits = mfma_pick_splits(a.total_tokens, G, a.batch, a.n_kv_heads, max_ctx, BN);
    const uint32_t m_tiles = ceil_div(a.total_tokens * G, kMTile) + a.batch;
    if (a.workspace == nullptr ||
        a.workspace_bytes < mfma_workspace_bytes(a.total_tokens, a.n_heads, a.head_dim, splits + 1)) {
        splits = 1;  // no scratch: every M tile walks its whole KV range
    }
    uint32_t split_len = ceil_div(ceil_div(max_ctx, splits), BN) * BN;
    if (split_len == 0) {
        split_len = BN;
    }
    const uint32_t max_splits = ceil_div(max_ctx, split_len);

    MfmaParams p{};
    const uint32_t row = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim;
    p.q0 = static_cast<const uint16_t *>(a.qkv);
    p.q0_tok_stride = row;
    p.q0_head_stride = a.head_dim;
    p.k0 = static_cast<const uint16_t *>(a.k_cache);
    p.v = static_cast<const uint16_t *>(a.v_cache);
    p.k0_tok_stride = a.n_kv_heads * a.head_dim;
    p.out = static_cast<uint16_t *>(a.output);
    p.out_tok_stride = a.n_heads * a.head_dim;
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.rows_per_pos = G;
    p.n_heads = a.n_heads;
    p.batch = a.batch;
    p.block_size = a.block_size;
    p.block_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
    p.max_num_block = a.max_num_block;
    p.dense_len = 0;
    p.split_len = split_len;
    p.max_splits = max_splits;
    p.scale_log2e = kLog2e;
    const PartialBuffers pb = max_splits > 1 ? carve_partials(a.workspace, a.total_tokens, a.n_heads, a.head_dim, max_splits)
                                             : PartialBuffers{};
    fill_common(p, pb);

    dim3 grid(max_splits, m_tiles, a.n_kv_heads);
    const bool bf = a.dtype == XLITE_HIP_BF16;
    int rc;
    if (a.head_dim == 256) {
        rc = bf ? launch_kernel<BF16, 256, 0, 256, BN, true>(stream, p, grid)
                : launch_kernel<FP16, 256, 0, 256, BN, true>(stream, p, grid);
    } else if (a.head_dim == 128) {
        rc = bf ? launch_kernel<BF16, 128, 0, 128, BN, true>(stream, p, grid)
                : launch_kernel<FP16, 128, 0, 128, BN, true>(stream, p, grid);
    } else {
        rc = bf ? launch_kernel<BF16, 64, 0, 64, BN, true>(stream, p, grid)
                : launch_kernel<FP16, 64, 0, 64, BN, true>(stream, p, grid);
    }
    if (rc != XLITE_HIP_OK || max_splits == 1) {
        return rc;
    }
    return launch_merge(stream, a.dtype, a.output, pb, a.total_tokens, a.n_heads, a.head_dim, max_splits);
}

int launch_mfma_mla(hipStream_t stream, const MlaArgs &a)
{
    constexpr int BN = 32;
    const bool dense = a.block_tables == nullptr;
    const uint32_t max_ctx = dense ? a.dense_len : a.max_num_blocks * a.block_size;
    uint32_t splits = mfma_pick_splits(a.total_tokens, a.n_heads, a.batch, 1, max_ctx, BN);
    const uint32_t m_tiles = ceil_div(a.total_tokens * a.n_heads, kMTile) + a.batch;
    if (a.workspace == nullptr ||
        a.workspace_bytes < mfma_workspace_bytes(a.total_tokens, a.n_heads, a.kv_lora_rank, splits + 1)) {
        splits = 1;
    }
    uint32_t split_len = ceil_div(ceil_div(max_ctx, splits), BN) * BN;
    if (split_len == 0) {
        split_len = BN;
    }
    const uint32_t max_splits = ceil_div(max_ctx, split_len);

    MfmaParams p{};
    p.q0 = static_cast<const uint16_t *>(a.q_absorb);
    p.q0_tok_stride = a.n_heads * a.kv_lora_rank;
    p.q0_head_stride = a.kv_lora_rank;
    p.q1 = static_cast<const uint16_t *>(a.qr);
    p.q1_tok_stride = a.n_heads * a.rope_head_dim;
    p.q1_head_stride = a.rope_head_dim;
    p.k0 = static_cast<const uint16_t *>(a.k_cache);
    p.k1 = static_cast<const uint16_t *>(a.pe_cache);
    p.v = nullptr;
    p.k0_tok_stride = a.kv_lora_rank;
    p.k1_tok_stride = a.rope_head_dim;
    p.out = static_cast<uint16_t *>(a.o_absorb);
    p.out_tok_stride = a.n_heads * a.kv_lora_rank;
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.rows_per_pos = a.n_heads;
    p.n_heads = a.n_heads;
    p.batch = a.batch;
    p.block_size = dense ? 1 : a.block_size;
    p.block_shift = dense ? 0 : ((a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1);
    p.max_num_block = a.max_num_blocks;
    p.dense_len = a.dense_len;
    p.split_len = split_len;
    p.max_splits = max_splits;
    p.scale_log2e = a.scale * kLog2e;
    const PartialBuffers pb = max_splits > 1 ? carve_partials(a.workspace, a.total_tokens, a.n_heads, a.kv_lora_rank, max_splits)
                                             : PartialBuffers{};
    fill_common(p, pb);

    dim3 grid(max_splits, m_tiles, 1);
    if (a.kv_lora_rank == 512 && a.rope_head_dim == 64) {
        const int rc = launch_kernel<BF16, 512, 64, 512, BN, false>(stream, p, grid);
        if (rc != XLITE_HIP_OK || max_splits == 1) {
            return rc;
        }
        return launch_merge(stream, a.dtype, a.o_absorb, pb, a.total_tokens, a.n_heads, a.kv_lora_rank, max_splits);
    }
    return fail(XLITE_HIP_EINVAL, __func__,
                "only kv_lora_rank 512 with rope_head_dim 64 is built for the matrix-core path");
}

}  // namespace xlite
