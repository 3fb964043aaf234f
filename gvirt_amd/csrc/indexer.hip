// DSA indexer: scores of every cached position for every query row, and the top-k positions per row.
//
//   scores[t][j] = sum_h weight[t][head_dim + h] * round16(q[t][h][:] . k[j][:])      j < cached + query length
// The per-head dot products are rounded to the 16-bit activation type before they are weighted, as in the
// reference (xlite/csrc/kernels/indexer_scores.h:176-243: scores -> L1 as Dtype, then a second product with
// the weights); there is no causal limit inside a sequence and no activation function. Golden:
// xlite/tests/kernels/indexer_scores.py:96-118.
//
// A wavefront owns one query row (and, in decode batches, a range of 256 positions; in batches with several rows per
// sequence eight such waves share the K rows of 1024 positions through LDS). Q sits in registers as the A operand of
// v_mfma_f32_16x16x32 (16 heads x 32 dims per tile), K rows are the B operand, loaded straight from the paged cache
// or read from the shared stage (a lane holds 8 dims of one position), so a result tile holds 16 heads x 16 positions
// with one position per lane column: rounded and packed, it is already the B operand of the second
// product, whose A operand carries the 16 weights in row 0.
//
// The top-k selection (xlite/csrc/kernels/indexer_topk.h, golden xlite/tests/kernels/indexer_topk.py:139-152)
// runs on the 16-bit scores: a two-pass radix select finds the k-th largest key, then one ordered pass
// writes the positions above it, and the lowest positions among its ties, in ascending order (the order the
// top-k mask of the MLA attention wants). Rows with at most k candidates list them all.
#include "attention_common.h"

namespace xlite {

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;
constexpr int kWavesPerWg = 4;
constexpr int kRange = 256;          // positions per wave
// the kernel for batches with several rows per sequence: 8 rows share the K rows of 1024 positions through LDS
constexpr int kShWaves = 8;
constexpr int kShRange = 1024;       // positions per workgroup
constexpr int kShStage = 64;         // positions per LDS stage (16 KiB)
constexpr int kShStages = 3;
constexpr int kSelThreads = 1024;
constexpr uint32_t kSelStage = 24576;   // scores of a row kept in LDS between the passes (48 KiB)

template <typename T>
struct Mma;
template <>
struct Mma<BF16> {
    static __device__ __forceinline__ f32x4_t k32(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t k16(const uint2 &a, const uint2 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a),
                                                         __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mma<FP16> {
    typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4_t;
    static __device__ __forceinline__ f32x4_t k32(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t k16(const uint2 &a, const uint2 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                     __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
};

// The sequence that owns query row t, and its number of candidate positions. query_start_loc is a prefix sum
// (non-decreasing): the owner is the last sequence that starts at or before t, if t lies inside it.
__device__ __forceinline__ bool find_row(uint32_t t, const int32_t *query_start_loc, const int32_t *lens,
                                         const int32_t *cached_lens, uint32_t batch, uint32_t *seq, uint32_t *total)
{
    if (t < batch) {
        // a decode batch (one row per sequence) answers with one round of loads: row t is sequence t
        const int32_t s = query_start_loc[t], l = lens[t], c = cached_lens[t];
        if (s == static_cast<int32_t>(t) && l == 1) {
            *seq = t;
            *total = static_cast<uint32_t>(c + 1);
            return true;
        }
    }
    uint32_t lo = 0, hi = batch;   // first index in [lo, hi) whose start is beyond t
    while (lo < hi) {
        const uint32_t mid = (lo + hi) / 2;
        if (query_start_loc[mid] <= static_cast<int32_t>(t)) {
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    if (lo == 0) {
        return false;
    }
    const uint32_t i = lo - 1;
    const int32_t s = query_start_loc[i], l = lens[i];
    if (static_cast<int32_t>(t) >= s + l) {
        return false;
    }
    *seq = i;
    *total = static_cast<uint32_t>(cached_lens[i] + l);
    return true;
}

// Scores of query row t (of sequence `seq`, `total` candidate positions) for the positions [p0, p1), by one wave,
// K rows straight from the cache. NT = n_heads / 16, head_dim = 128.
template <typename T, int NT, bool TBL_IN_REG>
__device__ __forceinline__ void indexer_row_range_impl(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k_cache,
                                                  const uint16_t *__restrict__ weight, uint16_t *__restrict__ scores,
                                                  const int32_t *__restrict__ block_tables, uint32_t t, uint32_t seq,
                                                  uint32_t total, uint32_t p0, uint32_t p1, uint32_t block_size,
                                                  uint32_t max_num_block, uint32_t ld_scores, uint32_t lane)
{
    constexpr int D = 128;
    constexpr int KS = D / 32;
    constexpr int H = NT * 16;
    const uint32_t col = lane & 15, kg = lane >> 4;

    // the block-table entries of the range sit in the lanes of one register (lane i: block p0 / bs + i), so that
    // a K load does not wait for a table load first; ranges of more than 64 blocks look the table up directly.
    // Requested ahead of the query rows: the first K loads wait for these entries only, and travel with the queries.
    const int32_t *table = block_tables + static_cast<uint64_t>(seq) * max_num_block;
    const uint32_t blk0 = p0 / block_size;
    const uint32_t nblk = (p1 - 1) / block_size - blk0 + 1;
    // (TBL_IN_REG is a template parameter, not a run-time choice inside load_k: a load that may or may not be issued
    // is awaited at the join, and that wait covers every K load in flight)
    const int32_t tbl_reg = table[blk0 + min(lane, nblk - 1)];   // (every lane loads: no branch, no wait of its own)

    // A operands: Q of head 16 nt + col, dims 32 ks + 8 kg .. +8; weights of heads 16 nt + 4 kg .. +4 in the
    // lanes of row 0 only
    uint4 qa[NT][KS];
    uint2 wa[NT];
    const uint16_t *qrow = q + static_cast<uint64_t>(t) * H * D;
    const uint16_t *wrow = weight + static_cast<uint64_t>(t) * (D + H) + D;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            qa[nt][ks] = *reinterpret_cast<const uint4 *>(qrow + (16 * nt + col) * D + 32 * ks + 8 * kg);
        }
        // (every row of the operand carries the weights: only row 0 of the product is read, and a load under a
        // per-lane condition is compiled into a branch with a wait of its own, which here would also wait for every
        // query load before it)
        const uint16_t *wp = wrow + 16 * nt + 4 * kg;   // 2-byte aligned only: the row pitch may be odd pairs
        const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2], w3 = wp[3];
        wa[nt] = make_uint2(w0 | (w1 << 16), w2 | (w3 << 16));
    }

    auto load_k = [&](uint32_t pos0, uint4 (&kb)[KS]) {
        const uint32_t pos = min(pos0 + col, total - 1);   // positions past the end repeat the last one
        const uint32_t blk = pos / block_size;
        const uint32_t phys = static_cast<uint32_t>(TBL_IN_REG ? __shfl(tbl_reg, static_cast<int>(min(blk - blk0, 63u)))
                                                               : table[blk]);
        const uint16_t *row = k_cache + (static_cast<uint64_t>(phys) * block_size + pos % block_size) * D + 8 * kg;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            kb[ks] = *reinterpret_cast<const uint4 *>(row + 32 * ks);
        }
    };
    constexpr int kPre = 5;   // K tiles in registers: four are in flight while one is consumed (16 KiB per wave: with
                              // four waves on a compute unit, what its share of the memory system's latency needs)
    uint4 kb[kPre][KS];
#pragma unroll
    for (int i = 0; i < kPre - 1; i++) {
        if (p0 + 16 * i < p1) {
            load_k(p0 + 16 * i, kb[i]);
        }
    }
    uint16_t *out = scores + static_cast<uint64_t>(t) * ld_scores;
    auto tile = [&](uint32_t pos0, const uint4 (&kt)[KS], uint4 (&knext)[KS]) {
        if (pos0 + 16 * (kPre - 1) < p1) {
            load_k(pos0 + 16 * (kPre - 1), knext);
        }
        f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            f32x4_t s = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                s = Mma<T>::k32(qa[nt][ks], kt[ks], s);
            }
            // lane: position `col`, heads 16 nt + 4 kg + r: the B operand of the weighting product
            const uint2 sb = make_uint2(T::pack(s[0], s[1]), T::pack(s[2], s[3]));
            acc = Mma<T>::k16(wa[nt], sb, acc);
        }
        // row 0 of the result: lanes 0 .. 15, register 0
        if (kg == 0 && pos0 + col < p1) {
            out[pos0 + col] = T::from_f32(acc[0]);
        }
    };
    // the ring of register tiles, unrolled so that every index is a constant
    for (uint32_t pos0 = p0; pos0 < p1; pos0 += 16 * kPre) {
#pragma unroll
        for (int i = 0; i < kPre; i++) {
            if (pos0 + 16 * i < p1) {
                tile(pos0 + 16 * i, kb[i], kb[(i + kPre - 1) % kPre]);
            }
        }
    }
}

template <typename T, int NT>
__device__ __forceinline__ void indexer_row_range(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k_cache,
                                                  const uint16_t *__restrict__ weight, uint16_t *__restrict__ scores,
                                                  const int32_t *__restrict__ block_tables, uint32_t t, uint32_t seq,
                                                  uint32_t total, uint32_t p0, uint32_t p1, uint32_t block_size,
                                                  uint32_t max_num_block, uint32_t ld_scores, uint32_t lane)
{
    if ((p1 - 1) / block_size - p0 / block_size + 1 <= 64) {   // the same in every lane
        indexer_row_range_impl<T, NT, true>(q, k_cache, weight, scores, block_tables, t, seq, total, p0, p1, block_size,
                                            max_num_block, ld_scores, lane);
    } else {
        indexer_row_range_impl<T, NT, false>(q, k_cache, weight, scores, block_tables, t, seq, total, p0, p1, block_size,
                                             max_num_block, ld_scores, lane);
    }
}

// One wavefront per (query row, range of 256 positions): decode batches, where no two rows share a sequence.
template <typename T, int NT>
__global__ void __launch_bounds__(kWavesPerWg * 64)
indexer_scores_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k_cache,
                      const uint16_t *__restrict__ weight, uint16_t *__restrict__ scores,
                      const int32_t *__restrict__ query_start_loc, const int32_t *__restrict__ lens,
                      const int32_t *__restrict__ cached_lens, const int32_t *__restrict__ block_tables,
                      uint32_t total_tokens, uint32_t batch, uint32_t block_size, uint32_t max_num_block,
                      uint32_t ld_scores)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t t = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    if (t >= total_tokens) {
        return;
    }
    uint32_t seq = 0, total = 0;
    if (!find_row(t, query_start_loc, lens, cached_lens, batch, &seq, &total)) {
        return;
    }
    const uint32_t p0 = blockIdx.y * kRange;
    if (p0 >= total) {
        return;
    }
    indexer_row_range<T, NT>(q, k_cache, weight, scores, block_tables, t, seq, total, p0, min(total, p0 + kRange),
                             block_size, max_num_block, ld_scores, lane);
}

// XOR pattern of the 16-byte chunk index of LDS row `row` (256 bytes = one bank window): the rows that one pass of a
// ds_read_b128 touches (not 16 consecutive lanes: lanes 0-3, 12-15, 20-23, 24-27 go together) get different slots
__device__ __forceinline__ uint32_t idx_swz(uint32_t row)
{
    const uint32_t hi = (row >> 3) & 1;
    return (((row & 7) ^ (hi << 2)) << 1) | hi;
}
// one wave-wide copy of 64 x 16 bytes from per-lane global addresses into 1 KiB of LDS at `lds_addr` + 16 * lane
__device__ __forceinline__ void idx_dma_1k(uint32_t lds_addr, const void *lane_ptr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\t"
                 :: "s"(lds_addr), "v"(lane_ptr) : "memory", "m0");
}

// Batches with several rows per sequence (prefill): the 8 waves of a workgroup take 8 consecutive query rows and,
// when these belong to one sequence, share its K rows: 64 positions at a time are copied straight into LDS (a ring
// of three 16 KiB stages, chunks XOR-swizzled by the copy's per-lane addresses) and every wave reads them from
// there as its B operands, so a K row crosses the L2 once per 8 query rows instead of once per row. A wave's
// scores of the range collect in LDS and leave 16 bytes per lane at the end. Workgroups whose rows do not all
// belong to one sequence (its first or last rows, a decode row among them) run the per-row code above.
template <typename T, int NT>
__global__ void __launch_bounds__(kShWaves * 64, NT <= 4 ? 4 : 2)
indexer_scores_shared_kernel(const uint16_t *__restrict__ q, const uint16_t *__restrict__ k_cache,
                             const uint16_t *__restrict__ weight, uint16_t *__restrict__ scores,
                             const int32_t *__restrict__ query_start_loc, const int32_t *__restrict__ lens,
                             const int32_t *__restrict__ cached_lens, const int32_t *__restrict__ block_tables,
                             uint32_t total_tokens, uint32_t batch, uint32_t block_size, uint32_t max_num_block,
                             uint32_t ld_scores)
{
    constexpr int D = 128;
    constexpr int KS = D / 32;
    constexpr int H = NT * 16;
    constexpr int ROWB = D * 2;
    constexpr int STAGEB = kShStage * ROWB;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint16_t *out_lds = reinterpret_cast<uint16_t *>(smem + kShStages * STAGEB);          // [wave][kShRange]
    int32_t *row_seq = reinterpret_cast<int32_t *>(smem + kShStages * STAGEB + kShWaves * kShRange * 2);
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6)));
    const uint32_t t = blockIdx.x * kShWaves + wave;
    uint32_t seq = 0, total = 0;
    const bool valid = t < total_tokens && find_row(t, query_start_loc, lens, cached_lens, batch, &seq, &total);
    if (lane == 0) {
        row_seq[wave] = valid ? static_cast<int32_t>(seq) : -1 - static_cast<int32_t>(wave);
    }
    __syncthreads();
    bool same = row_seq[0] >= 0;
#pragma unroll
    for (int w = 1; w < kShWaves; w++) {
        same = same && row_seq[w] == row_seq[0];
    }
    const uint32_t p0 = blockIdx.y * kShRange;
    const uint32_t blk0 = p0 / block_size;
    // (the block-table entries of the range sit in the lanes of one register: at most 64 of them)
    const bool shared = __builtin_amdgcn_readfirstlane(
        same && p0 < total && (min(total, p0 + kShRange) - 1) / block_size - blk0 + 1 <= 64 ? 1 : 0);
    if (!shared) {
        if (valid && p0 < total) {
            indexer_row_range<T, NT>(q, k_cache, weight, scores, block_tables, t, seq, total, p0,
                                     min(total, p0 + kShRange), block_size, max_num_block, ld_scores, lane);
        }
        return;
    }
    const uint32_t p1 = min(total, p0 + kShRange);
    const uint32_t col = lane & 15, kg = lane >> 4;

    // A operands and weights, as in the per-row code
    uint4 qa[NT][KS];
    uint2 wa[NT];
    const uint16_t *qrow = q + static_cast<uint64_t>(t) * H * D;
    const uint16_t *wrow = weight + static_cast<uint64_t>(t) * (D + H) + D;
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            qa[nt][ks] = *reinterpret_cast<const uint4 *>(qrow + (16 * nt + col) * D + 32 * ks + 8 * kg);
        }
        uint2 w = make_uint2(0u, 0u);
        if (col == 0) {
            const uint16_t *wp = wrow + 16 * nt + 4 * kg;
            w.x = static_cast<uint32_t>(wp[0]) | (static_cast<uint32_t>(wp[1]) << 16);
            w.y = static_cast<uint32_t>(wp[2]) | (static_cast<uint32_t>(wp[3]) << 16);
        }
        wa[nt] = w;
    }
    const int32_t *table = block_tables + static_cast<uint64_t>(seq) * max_num_block;
    const uint32_t nblk = (p1 - 1) / block_size - blk0 + 1;
    const int32_t tbl_reg = lane < nblk ? table[blk0 + lane] : 0;
    // complete these loads before any copy is issued: the copies' completion is counted, and memory operations finish
    // in order
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            asm volatile("" : "+v"(qa[nt][ks].x), "+v"(qa[nt][ks].y), "+v"(qa[nt][ks].z), "+v"(qa[nt][ks].w));
        }
        asm volatile("" : "+v"(wa[nt].x), "+v"(wa[nt].y));
    }
    int32_t tbl_pinned = tbl_reg;
    asm volatile("" : "+v"(tbl_pinned));

    // copy role: wave w moves rows 8 w .. 8 w + 7 of a stage as two copies of four rows; lane = (row of the four, chunk
    // slot), and the slot receives the chunk the row's pattern assigns to it. Positions beyond the end repeat the last.
    auto issue = [&](uint32_t s) {
        const uint32_t st = smem_addr + (s % kShStages) * STAGEB;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t r = 8 * wave + 4 * i + (lane >> 4);
            const uint32_t pos = min(p0 + s * kShStage + r, total - 1);
            const uint32_t blk = pos / block_size;
            const uint32_t phys = static_cast<uint32_t>(__shfl(tbl_pinned, static_cast<int>(blk - blk0)));
            const unsigned char *src = reinterpret_cast<const unsigned char *>(k_cache) +
                                       (static_cast<uint64_t>(phys) * block_size + pos % block_size) * ROWB +
                                       (((lane & 15u) ^ idx_swz(r)) << 4);
            idx_dma_1k(st + (8 * wave + 4 * i) * ROWB, src);
        }
    };
    // read role: position 16 tile + col of the stage, dims 32 ks + 8 kg .. + 8
    uint32_t rd_off[4][KS];
#pragma unroll
    for (int tl = 0; tl < 4; tl++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            rd_off[tl][ks] = (16 * tl + col) * ROWB + (((4 * ks + kg) ^ idx_swz(16 * tl + col)) << 4);
        }
    }
    uint16_t *my_out = out_lds + wave * kShRange;
    const uint32_t n_st = ceil_div(p1 - p0, static_cast<uint32_t>(kShStage));
    issue(0);
    if (n_st > 1) {
        issue(1);
    }
    for (uint32_t s = 0; s < n_st; s++) {
        // every copy of this wave so far has landed (those of stage s + 1 were issued a stage's arithmetic ago) ...
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // ... and everybody else's; stage s - 1 is free
        if (s + 2 < n_st) {
            issue(s + 2);
        }
        const unsigned char *stage = smem + (s % kShStages) * STAGEB;
#pragma unroll
        for (int tl = 0; tl < 4; tl++) {
            const uint32_t pos0 = p0 + s * kShStage + 16 * tl;
            if (pos0 < p1) {
                f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
                uint4 kt[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    kt[ks] = *reinterpret_cast<const uint4 *>(stage + rd_off[tl][ks]);
                }
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    f32x4_t sc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ks++) {
                        sc = Mma<T>::k32(qa[nt][ks], kt[ks], sc);
                    }
                    const uint2 sb = make_uint2(T::pack(sc[0], sc[1]), T::pack(sc[2], sc[3]));
                    acc = Mma<T>::k16(wa[nt], sb, acc);
                }
                if (kg == 0) {
                    my_out[pos0 - p0 + col] = T::from_f32(acc[0]);
                }
            }
        }
    }
    // the wave's scores of [p0, p1) leave LDS (written and read by this wave only: the compiler's LDS counter waits
    // order them): 16 bytes per lane where the row pitch allows, 2-byte pieces for the rest
    uint16_t *out = scores + static_cast<uint64_t>(t) * ld_scores + p0;
    const uint32_t n = p1 - p0;
    const uint32_t n8 = (ld_scores % 8 == 0 && (reinterpret_cast<uint64_t>(scores) & 15u) == 0) ? n & ~7u : 0u;
    for (uint32_t j = lane * 8; j < n8; j += 64 * 8) {
        *reinterpret_cast<uint4 *>(out + j) = *reinterpret_cast<const uint4 *>(my_out + j);
    }
    for (uint32_t j = n8 + lane; j < n; j += 64) {
        out[j] = my_out[j];
    }
}

// 16-bit float bits -> unsigned key with the same order
__device__ __forceinline__ uint32_t order_key(uint16_t bits)
{
    return (bits & 0x8000u) ? (~static_cast<uint32_t>(bits) & 0xffffu) : (static_cast<uint32_t>(bits) | 0x8000u);
}

// One workgroup per query row. The row is read from memory once: its first kSelStage scores stay in LDS for
// the three passes (a longer row's remainder is re-read).
__global__ void __launch_bounds__(kSelThreads)
indexer_select_kernel(const uint16_t *__restrict__ scores, const int32_t *__restrict__ indices,
                      int32_t *__restrict__ topk_indices, const int32_t *__restrict__ query_start_loc,
                      const int32_t *__restrict__ lens, const int32_t *__restrict__ cached_lens,
                      uint32_t batch, uint32_t top_k, uint32_t ld_scores)
{
    __shared__ uint32_t hist[256];
    // 32 private copies of the histogram, copy c of bin b at [b][c]: a wave's lanes count into the copies of their
    // lane index modulo 32, which lie in 32 different banks. (Scores of one row share their sign and most of their
    // exponent: counted into one histogram, the high bytes of a wave's 64 keys fall into a handful of bins, and
    // atomic additions to one address are carried out one lane at a time.)
    __shared__ __attribute__((aligned(16))) uint32_t hist_priv[256 * 32];
    __shared__ uint32_t wave_cnt[2][kSelThreads / 64];
    __shared__ __attribute__((aligned(16))) uint16_t staged[kSelStage];
    __shared__ uint32_t sel[4];
    const uint32_t t = blockIdx.x;
    uint32_t seq = 0, n = 0;
    if (!find_row(t, query_start_loc, lens, cached_lens, batch, &seq, &n)) {
        return;
    }
    const uint16_t *row = scores + static_cast<uint64_t>(t) * ld_scores;
    int32_t *out = topk_indices + static_cast<uint64_t>(t) * top_k;
    if (n <= top_k) {
        for (uint32_t j = threadIdx.x; j < n; j += kSelThreads) {
            out[j] = indices[j];
        }
        return;
    }
    // ---- the k-th largest key: high byte, then low byte. Threads read eight keys (16 bytes) at a time.
    const uint32_t n8 = ld_scores % 8 == 0 ? n & ~7u : 0u;   // vector loads need 16-byte aligned rows
    const uint32_t n_st = min(n8, kSelStage);                // scores [0, n_st) are served from LDS
    for (uint32_t j = threadIdx.x * 8; j < n_st; j += kSelThreads * 8) {
        *reinterpret_cast<uint4 *>(staged + j) = *reinterpret_cast<const uint4 *>(row + j);
    }
    // (the first pass's barrier orders these stores before any read)
    uint32_t prefix = 0, above = 0;   // keys whose high byte equals `prefix` are the candidates of pass 2
    for (int pass = 0; pass < 2; pass++) {
#pragma unroll
        for (int i = 0; i < 256 * 32 / (kSelThreads * 4); i++) {
            reinterpret_cast<uint4 *>(hist_priv)[threadIdx.x + i * kSelThreads] = make_uint4(0u, 0u, 0u, 0u);
        }
        __syncthreads();
        const uint32_t my_copy = threadIdx.x & 31u;
        auto count = [&](uint32_t key) {
            if (pass == 0) {
                atomicAdd(&hist_priv[(key >> 8) * 32 + my_copy], 1u);
            } else if ((key >> 8) == prefix) {
                atomicAdd(&hist_priv[(key & 0xffu) * 32 + my_copy], 1u);
            }
        };
        for (uint32_t j = threadIdx.x * 8; j < n8; j += kSelThreads * 8) {
            const uint4 v = j < n_st ? *reinterpret_cast<const uint4 *>(staged + j) : *reinterpret_cast<const uint4 *>(row + j);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                count(order_key(static_cast<uint16_t>(w[e] & 0xffffu)));
                count(order_key(static_cast<uint16_t>(w[e] >> 16)));
            }
        }
        for (uint32_t j = n8 + threadIdx.x; j < n; j += kSelThreads) {
            count(order_key(row[j]));
        }
        __syncthreads();
        {
            // the bins' totals: thread = (bin, quarter of its copies)
            const uint32_t b = threadIdx.x >> 2, part = threadIdx.x & 3u;
            const uint4 x = *reinterpret_cast<const uint4 *>(hist_priv + b * 32 + part * 8);
            const uint4 y = *reinterpret_cast<const uint4 *>(hist_priv + b * 32 + part * 8 + 4);
            uint32_t sum = x.x + x.y + x.z + x.w + y.x + y.y + y.z + y.w;
            sum += __shfl_xor(sum, 1);
            sum += __shfl_xor(sum, 2);
            if (part == 0) {
                hist[b] = sum;
            }
        }
        __syncthreads();
        // the bin that holds the k-th key, counted from the top: a suffix sum over the 256 bins by one wave
        if (threadIdx.x < 64) {
            const uint32_t b0 = 255 - 4 * threadIdx.x;   // this lane's four bins, highest first
            const uint32_t c0 = hist[b0], c1 = hist[b0 - 1], c2 = hist[b0 - 2], c3 = hist[b0 - 3];
            uint32_t incl = c0 + c1 + c2 + c3;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d);
                incl += threadIdx.x >= static_cast<uint32_t>(d) ? up : 0;
            }
            uint32_t cum = above + incl - (c0 + c1 + c2 + c3);   // keys in the bins above this lane's
            const uint32_t cs[4] = {c0, c1, c2, c3};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (cum < top_k && cum + cs[e] >= top_k) {
                    sel[0] = b0 - e;
                    sel[1] = cum;
                }
                cum += cs[e];
            }
        }
        __syncthreads();
        prefix = pass == 0 ? sel[0] : ((prefix << 8) | sel[0]);
        above = sel[1];
        __syncthreads();
    }
    const uint32_t thr = prefix;            // the k-th largest key
    const uint32_t need = top_k - above;    // ties of it to take, lowest positions first
    // ---- ordered output: 1024 positions per round, four consecutive ones per thread
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t done = 0, ties = 0;   // running totals, the same in every thread
    for (uint32_t base = 0; base < n; base += kSelThreads * 4) {
        const uint32_t j0 = base + threadIdx.x * 4;
        uint32_t key[4];
        if (j0 + 4 <= n8) {
            const uint2 v = j0 < n_st ? *reinterpret_cast<const uint2 *>(staged + j0) : *reinterpret_cast<const uint2 *>(row + j0);
            key[0] = order_key(static_cast<uint16_t>(v.x & 0xffffu));
            key[1] = order_key(static_cast<uint16_t>(v.x >> 16));
            key[2] = order_key(static_cast<uint16_t>(v.y & 0xffffu));
            key[3] = order_key(static_cast<uint16_t>(v.y >> 16));
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                key[e] = j0 + e < n ? order_key(row[j0 + e]) : 0u;   // key 0 is below every threshold reached here
            }
        }
        uint32_t n_eq = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            n_eq += (j0 + e < n && key[e] == thr) ? 1u : 0u;
        }
        // ties before this thread: wave prefix, then the waves before
        uint32_t eq_incl = n_eq;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(eq_incl, d);
            eq_incl += lane >= static_cast<uint32_t>(d) ? up : 0;
        }
        if (lane == 63) {
            wave_cnt[0][wave] = eq_incl;
        }
        __syncthreads();
        uint32_t eq_rank = ties + eq_incl - n_eq, eq_total = 0;
#pragma unroll
        for (uint32_t w = 0; w < kSelThreads / 64; w++) {
            const uint32_t c = wave_cnt[0][w];
            eq_rank += w < wave ? c : 0;
            eq_total += c;
        }
        bool take[4];
        uint32_t n_tk = 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const bool in = j0 + e < n;
            const bool eq = in && key[e] == thr;
            take[e] = in && (key[e] > thr || (eq && eq_rank < need));
            eq_rank += eq ? 1u : 0u;
            n_tk += take[e] ? 1u : 0u;
        }
        uint32_t tk_incl = n_tk;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(tk_incl, d);
            tk_incl += lane >= static_cast<uint32_t>(d) ? up : 0;
        }
        if (lane == 63) {
            wave_cnt[1][wave] = tk_incl;
        }
        __syncthreads();
        uint32_t o = done + tk_incl - n_tk, tk_total = 0;
#pragma unroll
        for (uint32_t w = 0; w < kSelThreads / 64; w++) {
            const uint32_t c = wave_cnt[1][w];
            o += w < wave ? c : 0;
            tk_total += c;
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (take[e] && o < top_k) {
                out[o++] = indices[j0 + e];
            }
        }
        done += tk_total;
        ties += eq_total;
    }
}

template <typename T>
int launch_scores(hipStream_t stream, const void *q, const void *k_cache, const void *weight, void *scores,
                  const int32_t *query_start_loc, const int32_t *lens, const int32_t *cached_lens,
                  const int32_t *block_tables, uint32_t total_tokens, uint32_t n_heads, uint32_t block_size,
                  uint32_t batch, uint32_t max_num_block, uint32_t ld_scores)
{
    // eight or more rows per sequence on average: the kernel whose workgroups share K rows through LDS. (Its workgroups
    // take 1024 positions; with fewer rows per sequence most of them would span sequences and run the per-row code over
    // ranges four times as long as the per-row kernel's, on a quarter of its waves.)
    const bool shared = total_tokens >= 8 * static_cast<uint64_t>(batch);
    const dim3 grid(ceil_div(total_tokens, kWavesPerWg), ceil_div(max_num_block * block_size, kRange), 1);
    const dim3 grid_sh(ceil_div(total_tokens, kShWaves), ceil_div(max_num_block * block_size, kShRange), 1);
    const size_t lds_sh = static_cast<size_t>(kShStages) * kShStage * 256 + kShWaves * kShRange * 2 + kShWaves * 4;
#define XL_IDX_ARGS                                                                                                   \
    static_cast<const uint16_t *>(q), static_cast<const uint16_t *>(k_cache), static_cast<const uint16_t *>(weight), \
        static_cast<uint16_t *>(scores), query_start_loc, lens, cached_lens, block_tables, total_tokens, batch,      \
        block_size, max_num_block, ld_scores
#define XL_IDX(NT) indexer_scores_kernel<T, NT><<<grid, kWavesPerWg * 64, 0, stream>>>(XL_IDX_ARGS)
#define XL_IDX_SH(NT)                                                                                                 \
    do {                                                                                                              \
        auto kernel = indexer_scores_shared_kernel<T, NT>;                                                            \
        if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds_sh)) {                      \
            return rc;                                                                                                \
        }                                                                                                             \
        kernel<<<grid_sh, kShWaves * 64, lds_sh, stream>>>(XL_IDX_ARGS);                                              \
    } while (0)
    switch (n_heads / 16) {
    case 1: if (shared) { XL_IDX_SH(1); } else { XL_IDX(1); } break;
    case 2: if (shared) { XL_IDX_SH(2); } else { XL_IDX(2); } break;
    case 4: if (shared) { XL_IDX_SH(4); } else { XL_IDX(4); } break;
    case 8: if (shared) { XL_IDX_SH(8); } else { XL_IDX(8); } break;
    default: return fail(XLITE_HIP_EINVAL, __func__, "n_heads must be 16, 32, 64 or 128");
    }
#undef XL_IDX
#undef XL_IDX_SH
#undef XL_IDX_ARGS
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

int check_common(const void *q, const void *k_cache, const void *weight, const int32_t *query_start_loc,
                 const int32_t *lens, const int32_t *cached_lens, const int32_t *block_tables, uint32_t n_heads,
                 uint32_t head_dim, uint32_t block_size, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    XL_REQUIRE(q && k_cache && weight && query_start_loc && lens && cached_lens && block_tables, "null tensor");
    XL_REQUIRE(head_dim == 128, "head_dim must be 128");
    XL_REQUIRE(n_heads == 16 || n_heads == 32 || n_heads == 64 || n_heads == 128, "n_heads must be 16, 32, 64 or 128");
    XL_REQUIRE(block_size > 0, "block_size must be positive");
    return XLITE_HIP_OK;
}

}  // namespace

}  // namespace xlite

using namespace xlite;

extern "C" int xlite_hip_indexer_scores(void *stream, const void *q, const void *k_cache, const void *weight,
                                        void *scores, const int32_t *query_start_loc, const int32_t *lens,
                                        const int32_t *cached_lens, const int32_t *block_tables,
                                        uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                                        uint32_t block_size, uint32_t batch, uint32_t max_num_block, int dtype)
{
    if (total_tokens == 0 || batch == 0 || max_num_block == 0) {
        return XLITE_HIP_OK;
    }
    const int rc = check_common(q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables, n_heads,
                                head_dim, block_size, dtype);
    if (rc != XLITE_HIP_OK) {
        return rc;
    }
    XL_REQUIRE(scores != nullptr, "null tensor");
    const uint32_t ld = max_num_block * block_size;
    return dtype == XLITE_HIP_BF16
               ? launch_scores<BF16>(as_stream(stream), q, k_cache, weight, scores, query_start_loc, lens, cached_lens,
                                     block_tables, total_tokens, n_heads, block_size, batch, max_num_block, ld)
               : launch_scores<FP16>(as_stream(stream), q, k_cache, weight, scores, query_start_loc, lens, cached_lens,
                                     block_tables, total_tokens, n_heads, block_size, batch, max_num_block, ld);
}

extern "C" size_t xlite_hip_indexer_topk_workspace_bytes(uint32_t total_tokens, uint32_t block_size,
                                                         uint32_t max_num_block)
{
    return static_cast<size_t>(total_tokens) * max_num_block * block_size * sizeof(uint16_t);
}

extern "C" int xlite_hip_indexer_topk(void *stream, const void *q, const void *k_cache, const void *weight,
                                      const int32_t *indices, int32_t *topk_indices,
                                      const int32_t *query_start_loc, const int32_t *lens,
                                      const int32_t *cached_lens, const int32_t *block_tables,
                                      uint32_t total_tokens, uint32_t n_heads, uint32_t head_dim,
                                      uint32_t block_size, uint32_t batch, uint32_t max_num_block, uint32_t top_k,
                                      int dtype, void *workspace, size_t workspace_bytes)
{
    if (total_tokens == 0 || batch == 0 || max_num_block == 0 || top_k == 0) {
        return XLITE_HIP_OK;
    }
    const int rc = check_common(q, k_cache, weight, query_start_loc, lens, cached_lens, block_tables, n_heads,
                                head_dim, block_size, dtype);
    if (rc != XLITE_HIP_OK) {
        return rc;
    }
    XL_REQUIRE(indices != nullptr && topk_indices != nullptr, "null tensor");
    XL_REQUIRE(top_k <= 2048, "topK should be less than or equal to 2048");
    const size_t need = xlite_hip_indexer_topk_workspace_bytes(total_tokens, block_size, max_num_block);
    if (workspace == nullptr || workspace_bytes < need) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) + " bytes, have " +
                                                    std::to_string(workspace_bytes));
    }
    const uint32_t ld = max_num_block * block_size;
    const int rc2 =
        dtype == XLITE_HIP_BF16
            ? launch_scores<BF16>(as_stream(stream), q, k_cache, weight, workspace, query_start_loc, lens, cached_lens,
                                  block_tables, total_tokens, n_heads, block_size, batch, max_num_block, ld)
            : launch_scores<FP16>(as_stream(stream), q, k_cache, weight, workspace, query_start_loc, lens, cached_lens,
                                  block_tables, total_tokens, n_heads, block_size, batch, max_num_block, ld);
    if (rc2 != XLITE_HIP_OK) {
        return rc2;
    }
    indexer_select_kernel<<<total_tokens, kSelThreads, 0, as_stream(stream)>>>(
        static_cast<const uint16_t *>(workspace), indices, topk_indices, query_start_loc, lens, cached_lens, batch,
        top_k, ld);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}
