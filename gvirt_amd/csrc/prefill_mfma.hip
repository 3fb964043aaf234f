// Chunked causal prefill over the paged GQA cache on the matrix cores (head_dim 128 or 64, 16-bit cache).
//
// Workgroup = 8 wavefronts (two per SIMD: while one waits for LDS or does its softmax on the vector
// ALU, the other keeps the matrix pipe busy) = 256 "M rows" of one kv head, an M row being one
// (query position, query head of the group) pair. Each wave owns 32 M rows and keeps their query
// vectors in registers as the B operand; the visible KV positions are walked in tiles of 64:
//     S^T[pos][m]  = K[pos][:] . Q[m][:]           16 x v_mfma_f32_32x32x16 (A = K rows, ds_read_b128)
//     O^T[d][m]   += V^T[d][pos] . P^T[pos][m]     16 x v_mfma_f32_32x32x16 (A = V^T, ds_read_b64_tr_b16)
// K and V tiles are copied straight from the cache into LDS (global_load_lds_dwordx4, one instruction
// = four consecutive positions of the kv head = 1 KiB of LDS) into a ring of four 32 KiB stages; V
// stays row major and is transposed on the way out of LDS, so no transposing stores are needed. The
// 16-byte chunks of a row are XOR-swizzled by the position (the lane chooses which global chunk lands
// in its LDS slot) so that both read shapes are bank-conflict free. With head_dim 64 a 256-byte bank
// window holds two positions, a copy instruction eight, and the pattern is a function of the window.
// M tiles are numbered sequence by sequence and launched last-first: the tiles with the longest
// visible range start first. When there are fewer M tiles than compute units (a short chunk after a
// long cached context, decode rows mixed into the batch), grid.y splits every tile's visible range into
// equal runs of KV tiles; the runs leave fp32 partials (O, reference maximum, normaliser) that the merge
// kernel combines.
//
// Replaces attention.h / flash_attention.h for batches with multi-token queries
// (xlite/csrc/kernels/attention.h:308-492, causal rule softmax_attn_aiv.h:739-741).
#include <type_traits>

#include "attention_common.h"
#include "kv8.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kRescaleSlack = 2.0f / kLog2e;   // raw score units: a factor of 4
constexpr int kWaves = 8;
constexpr int kXcds = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kMTile = kWaves * 32;
constexpr int BN = 64;                    // positions per KV tile
constexpr int kStages = 4;
constexpr size_t kLdsLimit = 160 * 1024;   // LDS of a compute unit: the stages plus the staged block-table row must fit
constexpr uint32_t kMinSplitTiles = 8;          // a KV split walks at least 512 positions

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

template <typename T>
struct Mfma32;
template <>
struct Mfma32<BF16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma32<FP16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

struct PrefillParams {
    const uint16_t *q;
    const uint16_t *k_cache;
    const uint16_t *v_cache;
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;
    uint32_t q_tok_stride;     // elements
    uint32_t out_tok_stride;
    uint32_t group;            // query heads per kv head
    uint32_t n_kv_heads;
    uint32_t batch;
    uint32_t block_size;       // a multiple of 4
    uint32_t block_magic;      // floor(2^32 / block_size) + 1: position / block_size == mulhi(position, magic)
    uint32_t max_num_block;
    uint32_t n_mtiles;         // grid.x
    uint32_t max_splits;       // grid.y: KV splits per M tile (1: none, results are final)
    uint32_t n_heads;
    uint32_t skip_single;      // 1: sequences with exactly one query row are another kernel's
    int32_t *part_cnt;         // [token][head] number of partials to merge (0: the value is final)
    float *part_acc;           // [token][head][max_splits][D]
    float *part_ml;            // [token][head][max_splits][2]: reference maximum (log2 domain), normaliser
    unsigned long long *clock_probe;   // nullptr, or where workgroup 0 leaves its shader-clock and wall-clock stamps
    const float *k_scale;      // 8-bit caches read by the kernel itself: [slot][kv head] fp32
    const float *v_scale;
};

// XOR pattern of the 16-byte chunk index of LDS row `row` (rows are 256 bytes = one bank window). The
// 16 rows that one ds_read_b128 pass touches get 16 different chunk slots, and the 4 rows that one
// transposing pass touches get 4 different 64-byte groups.
__device__ __forceinline__ uint32_t swz(uint32_t row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
// head_dim 64: pattern of bank window `win` (two positions of 128 bytes; the upper half of the 16 chunk slots
// belongs to the odd position, so only the low three bits move). Eight consecutive windows get eight
// different values, neighbours differ in bit 2 (the 64-byte group a transposing pass reads).
__device__ __forceinline__ uint32_t swz64(uint32_t win) { return ((win & 1) << 2) | ((win >> 1) & 3); }
// byte offset inside a K or V tile of 16-byte chunk `chunk` of position `pos`
template <int D>
__device__ __forceinline__ uint32_t tile_off(uint32_t pos, uint32_t chunk)
{
    if constexpr (D == 128) {
        return pos * 256 + ((chunk ^ swz(pos)) << 4);
    } else {
        return (pos >> 1) * 256 + (((((pos & 1) << 3) | chunk) ^ swz64(pos >> 1)) << 4);
    }
}

// One wave-wide copy of 1 KiB from global memory into LDS at `lds_addr` + 16 * lane. The compiler sees
// neither the LDS write nor the memory counter: completion is awaited with dma_wait.
__device__ __forceinline__ void dma_1k(uint32_t lds_addr, uint32_t voff, const void *base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                 :: "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait()
{
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// eight 16-bit values of storage type FROM as type TO
template <typename FROM, typename TO>
__device__ __forceinline__ uint4 convert8(const uint4 &x)
{
    if constexpr (std::is_same<FROM, TO>::value) {
        return x;
    } else {
        auto one = [](uint32_t w) {
            return TO::pack(fminf(fmaxf(FROM::lo(w), -65504.f), 65504.f), fminf(fmaxf(FROM::hi(w), -65504.f), 65504.f));
        };
        return make_uint4(one(x.x), one(x.y), one(x.z), one(x.w));
    }
}

// T: the type of the caches and of the products; TIO: the type of the query rows and of the output (the same, or
// bf16 over fp16 caches: a bf16 model over the fp16 copy of a quantised cache)
// KVF: the cache is 16-bit (copied straight into LDS), or int8 / fp8 bytes with one fp32 scale per (position, kv head):
// then a wave loads the bytes and scales of its eight positions of a tile into registers, two tiles ahead, and writes
// them to the tile's stage as fp16 (value x scale, the arithmetic of the dequantising copy in kv_dequant.hip: same
// bits) one iteration later; everything behind the stages is the 16-bit kernel. head_dim 128, T = FP16.
template <typename T, int D, typename TIO = T, int KVF = XLITE_HIP_KV_SAME>
__global__ void __launch_bounds__(kThreads, 1)
prefill_kernel(const PrefillParams p)
{
    constexpr bool KV8 = KVF != XLITE_HIP_KV_SAME;
    static_assert(!KV8 || (D == 128 && std::is_same<T, FP16>::value), "8-bit caches: head_dim 128, fp16 products");
    constexpr int ROWB = D * 2;               // bytes of one (position, kv head) row in LDS
    constexpr int KBYTES = BN * ROWB;         // 16 KiB (8 KiB for head_dim 64)
    constexpr int STAGE = 2 * KBYTES;         // K tile, then V tile
    constexpr int KS = D / 16;                // k-steps of the QK product
    constexpr int DT = D / 32;                // 32-row tiles of O^T
    constexpr int PPC = 1024 / ROWB;          // positions per copy instruction (4 or 8)
    constexpr int CPT = BN / PPC / kWaves;    // copies per wave, tile and tensor (2 or 1)
    constexpr int PER_WAVE = 2 * CPT;         // copies per wave and tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t col = lane & 31;
    const uint32_t half = lane >> 5;
    const uint32_t G = p.group;

    // ---- which (kv head, M tile). Workgroups are dealt round-robin to the 8 XCDs, each with its own L2;
    // the M tiles of a kv head stream the same K/V, so a kv head's tiles are kept on one XCD (or on
    // 8 / n_kv_heads of them, interleaved), where the tiles running at the same time share the L2 lines.
    uint32_t kvh, mt_fwd;
    {
        const uint32_t xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
        if (p.n_kv_heads % kXcds == 0) {
            kvh = (slot / p.n_mtiles) * kXcds + xcd;
            mt_fwd = slot % p.n_mtiles;
        } else if (kXcds % p.n_kv_heads == 0) {
            const uint32_t r = kXcds / p.n_kv_heads;
            kvh = xcd % p.n_kv_heads;
            mt_fwd = slot * r + xcd / p.n_kv_heads;
        } else {
            kvh = blockIdx.x / p.n_mtiles;
            mt_fwd = blockIdx.x % p.n_mtiles;
        }
        if (kvh >= p.n_kv_heads || mt_fwd >= p.n_mtiles) {
            return;
        }
    }
    // ---- locate the M tile; the grid runs the tile ids backwards. Sequence i owns the ids from
    // floor(query_start_loc[i] * G / 256) + i up to the next sequence's first one: at least its
    // ceil(lens[i] * G / 256) tiles (the surplus ids are empty), and a formula of the prefix sums the caller
    // provides, so the owner of an id is found by bisection, not by a walk over the batch.
    const uint32_t tid = p.n_mtiles - 1 - mt_fwd;
    auto first_id = [&](uint32_t i) {
        return static_cast<uint32_t>((static_cast<uint64_t>(p.query_start_loc[i]) * G) / kMTile) + i;
    };
    uint32_t seq = 0;
    int32_t qlen, clen, qstart;
    uint32_t mt;
    // (the condition goes through readfirstlane: left to itself the compiler folds it into the per-lane `lane < batch`
    // below and then treats everything behind the join as divergent)
    if (__builtin_amdgcn_readfirstlane(p.batch <= 64 ? 1 : 0)) {
        // one round of loads instead of a chain of them: lane i fetches what the batch says about sequence i. The ids
        // are nondecreasing, so the sequences that start at or before `tid` are a prefix of the batch, and the owner
        // is its last one; its lengths are then read from the owner's lane.
        const bool in_batch = lane < p.batch;
        const int32_t my_start = in_batch ? p.query_start_loc[lane] : 0;
        const int32_t my_len = in_batch ? p.lens[lane] : 0;
        const int32_t my_cached = in_batch ? p.cached_lens[lane] : 0;
        const uint32_t fid = in_batch ? static_cast<uint32_t>((static_cast<uint64_t>(my_start) * G) / kMTile) + lane : 0xffffffffu;
        const uint64_t started = __ballot(fid <= tid);
        seq = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(__builtin_popcountll(started))) - 1;
        qstart = __builtin_amdgcn_readlane(my_start, static_cast<int>(seq));
        qlen = __builtin_amdgcn_readlane(my_len, static_cast<int>(seq));
        clen = __builtin_amdgcn_readlane(my_cached, static_cast<int>(seq));
        mt = tid - static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(fid), static_cast<int>(seq)));
    } else if (__builtin_amdgcn_readfirstlane(p.batch <= 16 * kThreads ? 1 : 0)) {
        // up to 8192 sequences: the whole workgroup counts the sequences that start at or before `tid`, every thread a
        // few of them with independent loads - one trip to memory, where the bisection below is a chain of a dozen (a
        // mixed batch of a thousand decode rows pays that chain in every one of its thousands of empty workgroups)
        uint32_t mine = 0;
        for (uint32_t i = threadIdx.x; i < p.batch; i += kThreads) {
            mine += first_id(i) <= tid ? 1u : 0u;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mine += __shfl_xor(mine, d);
        }
        uint32_t *cnt_lds = reinterpret_cast<uint32_t *>(smem);   // (the stages are not in use yet)
        if (lane == 0) {
            cnt_lds[wave] = mine;
        }
        __syncthreads();
        uint32_t started = 0;
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            started += cnt_lds[w];
        }
        __syncthreads();   // the words are free again before anything else is written there
        seq = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(started))) - 1;   // first_id(0) == 0: at least one
        mt = tid - first_id(seq);
        qlen = p.lens[seq];
        clen = p.cached_lens[seq];
        qstart = p.query_start_loc[seq];
    } else {
        uint32_t hi = p.batch;   // first_id(seq) <= tid < first_id(hi); first_id(0) == 0
        while (hi - seq > 1) {
            const uint32_t mid = (seq + hi) >> 1;
            if (first_id(mid) <= tid) {
                seq = mid;
            } else {
                hi = mid;
            }
        }
        seq = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(seq)));   // the same in every lane, said so
        mt = tid - first_id(seq);
        qlen = p.lens[seq];
        clen = p.cached_lens[seq];
        qstart = p.query_start_loc[seq];
    }
    if (p.skip_single && qlen == 1) {
        // the decode kernel writes this row; the merge of this kernel's partials must leave it alone
        if (p.part_cnt != nullptr && mt == 0 && blockIdx.y == 0 && threadIdx.x < G) {
            p.part_cnt[static_cast<uint64_t>(qstart) * p.n_heads + kvh * G + threadIdx.x] = 0;
        }
        return;
    }
    if (qlen <= 0 || mt >= ceil_div(static_cast<uint32_t>(qlen) * G, static_cast<uint32_t>(kMTile))) {
        return;
    }
    // Instrumentation, off unless a probe buffer was set: the workgroup of the first sequence's first tile leaves the
    // shader clock counter and the 100 MHz wall clock here and behind its tile loop, whose ratio is the clock the
    // kernel ran at.
    const bool probe = p.clock_probe != nullptr && seq == 0 && mt == 0 && kvh == 0 && blockIdx.y == 0 && threadIdx.x == 0;
    if (probe) {
        p.clock_probe[0] = clock64();
        p.clock_probe[1] = wall_clock64();
    }
    const uint32_t m_rows = static_cast<uint32_t>(qlen) * G;
    const uint32_t m_first = mt * kMTile;
    const uint32_t m_last = min(m_rows, m_first + kMTile) - 1;
    // keys visible to at least one row of the tile
    const uint32_t range_end = static_cast<uint32_t>(clen) + m_last / G + 1;
    // ---- this workgroup's run of KV tiles [first_tile, n_tiles): the whole range, or one of n_splits equal
    // runs of at least kMinSplitTiles tiles
    uint32_t n_tiles = ceil_div(range_end, static_cast<uint32_t>(BN));
    uint32_t first_tile = 0, n_splits = 1;
    const uint32_t split = blockIdx.y;
    if (p.max_splits > 1) {
        const uint32_t want = min(p.max_splits, max(1u, n_tiles / kMinSplitTiles));
        const uint32_t per = ceil_div(n_tiles, want);
        n_splits = ceil_div(n_tiles, per);
        if (split >= n_splits) {
            return;
        }
        first_tile = split * per;
        n_tiles = min(n_tiles, first_tile + per);
    }
    const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;
    const uint32_t row_bytes = p.n_kv_heads * (KV8 ? D : ROWB);   // of a position in the cache
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(smem + kStages * STAGE);

    // ---- this lane's M row ---------------------------------------------------------------------------
    const uint32_t m = m_first + wave * 32 + col;
    const bool m_valid = m < m_rows;
    const uint32_t qpos = m_valid ? m / G : 0;
    const uint32_t head = kvh * G + (m_valid ? m % G : 0);
    const uint32_t tok = static_cast<uint32_t>(qstart) + qpos;
    const uint32_t vis = m_valid ? static_cast<uint32_t>(clen) + qpos + 1 : 0u;   // causal: keys [0, vis)
    // tiles wholly below every row's limit need no mask; first tile that does (uniform per wave)
    const uint32_t wave_min_vis = static_cast<uint32_t>(clen) + min(m_first + wave * 32, m_rows - 1) / G + 1;

    uint4 qreg[KS];   // the lane's query row as the B operand of the first product; loaded by the set-up below
    f32x16_t O[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            O[dt][k] = 0.f;
        }
    }
    float m_run = -INFINITY, l_run = 0.f;

    // ---- read roles ------------------------------------------------------------------------------------
    // K rows as the A operand: row = position nt * 32 + col, chunk 2 ks + half. The pattern of position
    // col + 32 is that of col, so one XOR term serves both sub tiles.
    const uint32_t kx = D == 128 ? (half ^ swz(col)) << 4 : ((((col & 1) << 3) | half) ^ swz64(col >> 1)) << 4;
    const uint32_t k_row = D == 128 ? col * 256 : (col >> 1) * 256;
    // transposed V: 16-lane group g covers columns 16 (g % 2) .. +16 of a 32-column tile for the
    // positions of half g / 2; lane 4 j' + q points at elements [4 q, +4) of position 4 half + j' (+8 for
    // the second read of a 16-position k-step)
    uint32_t vr_off;
    {
        const uint32_t g = lane >> 4, jp = (lane & 15) >> 2, q = lane & 3;
        const uint32_t y = 2 * (g & 1) + (q >> 1);
        const uint32_t pos = 4 * (g >> 1) + jp;
        vr_off = KBYTES + tile_off<D>(pos, y) + ((q & 1) << 3);
    }
    // ---- copy role: wave w moves positions 8w .. 8w+7 of the tile, for K and for V: two copies of four
    // positions (head_dim 128) or one of eight. A copy fills 1 KiB of LDS, lane l the 16 bytes at 16 l: bank
    // window l / 16 of the copy, chunk slot l % 16; the slot receives the (position, chunk) whose pattern
    // maps there. copy_src: that position (relative to the copy's first) and its chunk.
    auto copy_src = [&](uint32_t first_pos, uint32_t *rel, uint32_t *chunk) {
        if constexpr (D == 128) {
            *rel = lane >> 4;
            *chunk = (lane & 15u) ^ swz(first_pos + (lane >> 4));
        } else {
            const uint32_t c16 = (lane & 15u) ^ swz64((first_pos >> 1) + (lane >> 4));
            *rel = 2 * (lane >> 4) + (c16 >> 3);
            *chunk = c16 & 7u;
        }
    };
    uint32_t c_voff[CPT];
#pragma unroll
    for (int i = 0; i < CPT; i++) {
        uint32_t rel, chunk;
        copy_src(PPC * (CPT * wave + i), &rel, &chunk);
        c_voff[i] = rel * row_bytes + (chunk << 4);
    }

    // copies of KV tile `tile` into stage tile % 4. The positions of a copy share one block (block_size a
    // multiple of the four or eight). Positions at or beyond the end of the range re-read the last valid one
    // (finite values; their probabilities are masked to zero).
    // (head_dim 128, blocks of a multiple of 8 positions: the wave's two copies of a tensor lie in one block, four
    // rows apart, so one lookup and one base address serve both: a third of the loop's scalar instructions)
    const bool one_lookup = CPT == 2 && (p.block_size & 7u) == 0;
    const uint32_t c_voff_second = c_voff[CPT - 1] + PPC * row_bytes;
    auto issue = [&](uint32_t tile) {
        const uint32_t st = smem_addr + (tile % kStages) * STAGE;
        if (one_lookup && tile * BN + PPC * CPT * (wave + 1) - 1 < range_end) {
            const uint32_t pos = PPC * CPT * wave;
            const uint32_t t = tile * BN + pos;
            const uint32_t blk = __umulhi(t, p.block_magic), off = t - blk * p.block_size;
            const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk]);
            const uint64_t row0 = static_cast<uint64_t>(phys) * p.block_size + off;
            const char *kb = reinterpret_cast<const char *>(p.k_cache) + row0 * row_bytes + kvh * ROWB;
            const char *vb = reinterpret_cast<const char *>(p.v_cache) + row0 * row_bytes + kvh * ROWB;
            dma_1k(st + pos * ROWB, c_voff[0], kb);
            dma_1k(st + KBYTES + pos * ROWB, c_voff[0], vb);
            dma_1k(st + (pos + PPC) * ROWB, c_voff_second, kb);
            dma_1k(st + KBYTES + (pos + PPC) * ROWB, c_voff_second, vb);
            return;
        }
#pragma unroll
        for (int i = 0; i < CPT; i++) {
            const uint32_t pos = PPC * (CPT * wave + i);
            uint32_t t = tile * BN + pos;
            uint32_t voff = c_voff[i];
            if (t + PPC - 1 >= range_end) {   // uniform; only the last tile
                const uint32_t lim = range_end - 1;
                uint32_t rel, chunk;
                copy_src(pos, &rel, &chunk);
                const uint32_t tl = min(t + rel, lim);
                t = min(t, lim) & ~static_cast<uint32_t>(PPC - 1);
                voff = (tl - t) * row_bytes + (chunk << 4);
            }
            // block-table entries come from LDS (copied there once): a vector load here would have to be
            // awaited together with every copy issued before it
            const uint32_t blk = __umulhi(t, p.block_magic), off = t - blk * p.block_size;
            const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk]);
            const uint64_t row0 = static_cast<uint64_t>(phys) * p.block_size + off;
            const char *kb = reinterpret_cast<const char *>(p.k_cache) + row0 * row_bytes + kvh * ROWB;
            const char *vb = reinterpret_cast<const char *>(p.v_cache) + row0 * row_bytes + kvh * ROWB;
            dma_1k(st + pos * ROWB, voff, kb);
            dma_1k(st + KBYTES + pos * ROWB, voff, vb);
        }
    };

    // 8-bit caches: lane l of wave w holds bytes 16 (l % 8) .. + 15 of position 8 w + l / 8 of the tile (K and V) and
    // the position's two scales. The eight positions share a block (block sizes are multiples of 8); positions at or
    // beyond the end of the range re-read the last valid one.
    uint4 kraw = make_uint4(0, 0, 0, 0), vraw = make_uint4(0, 0, 0, 0);
    float ksc = 0.f, vsc = 0.f;
    auto fetch8 = [&](uint32_t tile) {
        const uint32_t lim = range_end - 1;
        const uint32_t t_raw = tile * BN + 8 * wave;
        const uint32_t t = min(t_raw, lim) & ~7u;
        const uint32_t rel = min(t_raw + (lane >> 3), lim) - t;
        const uint32_t blk = __umulhi(t, p.block_magic), off = t - blk * p.block_size;
        const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk]);
        const uint64_t row = static_cast<uint64_t>(phys) * p.block_size + off + rel;
        const uint64_t at = (row * p.n_kv_heads + kvh) * D + (lane & 7u) * 16;
        kraw = *reinterpret_cast<const uint4 *>(reinterpret_cast<const unsigned char *>(p.k_cache) + at);
        vraw = *reinterpret_cast<const uint4 *>(reinterpret_cast<const unsigned char *>(p.v_cache) + at);
        ksc = p.k_scale[row * p.n_kv_heads + kvh];
        vsc = p.v_scale[row * p.n_kv_heads + kvh];
    };
    auto store8 = [&](uint32_t tile) {
        unsigned char *st = smem + (tile % kStages) * STAGE;
        const uint32_t pos = 8 * wave + (lane >> 3), c = 2 * (lane & 7u);
        *reinterpret_cast<uint4 *>(st + tile_off<D>(pos, c)) = dequant8<FP16, KVF>(make_uint2(kraw.x, kraw.y), ksc);
        *reinterpret_cast<uint4 *>(st + tile_off<D>(pos, c + 1)) = dequant8<FP16, KVF>(make_uint2(kraw.z, kraw.w), ksc);
        *reinterpret_cast<uint4 *>(st + KBYTES + tile_off<D>(pos, c)) = dequant8<FP16, KVF>(make_uint2(vraw.x, vraw.y), vsc);
        *reinterpret_cast<uint4 *>(st + KBYTES + tile_off<D>(pos, c + 1)) = dequant8<FP16, KVF>(make_uint2(vraw.z, vraw.w), vsc);
    };

    // A wave issues in order, so its own softmax does not overlap its own products; what the wave itself can
    // hide is LDS latency: a step's K operands are fetched during the previous step's second product, its V^T
    // operands during its own softmax. (The SIMD's other wave overlaps the rest: its products run while this
    // wave's vector instructions issue.)
    uint4 kop[KS];
    auto fetch_k = [&](uint32_t stage_off, int h) {
        const unsigned char *base = smem + stage_off + h * 32 * ROWB + k_row;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            kop[ks] = *reinterpret_cast<const uint4 *>(base + ((((2 * ks) & 15) << 4) ^ kx));
        }
    };

    // ---- one step of 32 positions. Register k of S holds position j0 + 8 (k / 4) + 4 half + k % 4. The
    // running maximum is kept in raw score units; q arrives scaled by head_dim^-0.5 (rope_and_cache), so the
    // only factor is log2(e), folded into the exponent's multiply-add.
    auto step = [&](uint32_t stage_off, int h, uint32_t j0, uint32_t next_stage_off, int next_h, auto mask_tag) {
        constexpr bool MASK = decltype(mask_tag)::value;
        // ---- S^T = K . Q^T (one accumulation chain: the SIMD's other wave fills the issue gaps between
        // dependent products, and a second chain would cost 16 more vector instructions of this wave's issue time)
        f32x16_t S;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            S[k] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            S = Mfma32<T>::run(kop[ks], qreg[ks], S);
        }
        // V^T operands of this step: in flight during the softmax
        typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
        unsigned char *vbase = smem + stage_off + h * 32 * ROWB;
        uint2 vop[2][DT][2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                vop[kk][dt][0] = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_tr_ptr)(vbase + kk * 16 * ROWB + (vr_off ^ ((dt & 3) << 6)))));
                // second read: 8 positions further; the pattern of position p + 8 is that of p XOR 2
                vop[kk][dt][1] = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_tr_ptr)(vbase + kk * 16 * ROWB + 8 * ROWB + (vr_off ^ (((dt & 3) << 6) | (1 << 5))))));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // the softmax runs at a raised wave priority: the SIMD's other wave is then mostly in its products, whose
        // issue slots are sparse, and this wave's vector instructions go first (1 % on the chunked-prefill step;
        // raising the priority around the products instead costs 4 %)
        __builtin_amdgcn_s_setprio(2);
        if constexpr (MASK) {
            const uint32_t rem = vis > j0 + half * 4 ? vis - (j0 + half * 4) : 0u;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const uint32_t o = (k / 4) * 8 + (k % 4);
                S[k] = rem > o ? S[k] : -INFINITY;
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            mx = fmaxf(mx, S[k]);
        }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        // The reference maximum only moves when the step maximum exceeds it by more than a factor of 4:
        // probabilities then stay below 4, the normaliser shares the reference, and the accumulators are
        // rescaled rarely. (A larger slack costs accuracy on peaked rows: with an exact reference the
        // dominant probability is exactly 1, with a stale one it is rounded to 16 bits like the others.)
        const float m_new = mx > m_run + kRescaleSlack ? mx : m_run;
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = fast_exp2((m_run - m_safe) * kLog2e);
        const float neg_m = -m_safe * kLog2e;
        m_run = m_new;
        uint32_t w[8];
        float psum = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k += 2) {
            const float e0 = fast_exp2(__builtin_fmaf(S[k], kLog2e, neg_m));
            const float e1 = fast_exp2(__builtin_fmaf(S[k + 1], kLog2e, neg_m));
            psum += e0 + e1;
            w[k / 2] = T::pack(e0, e1);
        }
        const uint4 pb[2] = {make_uint4(w[0], w[1], w[2], w[3]), make_uint4(w[4], w[5], w[6], w[7])};
        l_run = l_run * alpha + psum;
        if (__any(alpha != 1.0f)) {
            // in place (an opaque multiply keeps the accumulators in the same registers on both paths)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    asm volatile("v_mul_f32 %0, %1, %0" : "+v"(O[dt][k]) : "v"(alpha));
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        // K operands of the next step: in flight during the second product
        fetch_k(next_stage_off, next_h);
        // ---- O^T += V^T . P^T: four tiles of 32 columns x two k-steps of 16 positions. The k-step order
        // inside a lane's registers is positions 8 (e / 4) + 4 half + e % 4, on both operands.
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                O[dt] = Mfma32<T>::run(make_uint4(vop[kk][dt][0].x, vop[kk][dt][0].y, vop[kk][dt][1].x, vop[kk][dt][1].y),
                                       pb[kk], O[dt]);
            }
        }
    };

    // ---- pipeline: copies run two tiles ahead of the tile being consumed (three right after they are
    // issued); one barrier per tile of 64 positions, between its two steps, because the second step already
    // fetches the next tile's first K operands. Every copy is unconditional (tiles past the end copy the last
    // tile again into a stage nobody reads any more), so the wait counts are exact.
    const uint32_t last = n_tiles - 1;
    // Set-up in two trips to memory: the block-table entries of this workgroup's range are requested first and the
    // query rows right behind them; the entries go to LDS as soon as they are there (the wait leaves the query
    // loads in flight), the first three tiles' copies are issued, and only then are the query rows awaited
    // (memory operations finish in order: that wait covers the copies too, which were going to be awaited anyway).
    {
        const uint32_t i_lo = __umulhi(first_tile * BN, p.block_magic);
        const uint32_t i_hi = __umulhi(min(n_tiles * BN, range_end) - 1, p.block_magic);
        const uint32_t i_mine = i_lo + threadIdx.x;
        const uint32_t entry = i_mine <= i_hi ? static_cast<uint32_t>(table[i_mine]) : 0u;
        const uint16_t *src = p.q + static_cast<uint64_t>(tok) * p.q_tok_stride + static_cast<uint64_t>(head) * D;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            // (every lane loads: rows past the tile's end point at the sequence's first row and are cleared below; a
            // load under a condition is compiled into a branch with a wait of its own, eight trips to memory in a row)
            qreg[ks] = *reinterpret_cast<const uint4 *>(src + ks * 16 + half * 8);
        }
        if (i_mine <= i_hi) {
            tbl_lds[i_mine] = entry;
        }
        for (uint32_t i = i_mine + kThreads; i <= i_hi; i += kThreads) {   // (ranges of more than 512 blocks)
            tbl_lds[i] = static_cast<uint32_t>(table[i]);
        }
        __syncthreads();
    }
    if constexpr (KV8) {
        // the first two tiles go to their stages now, the third stays in registers: iteration `tile` writes tile + 2
        // (its stage was last read two iterations ago, a barrier has passed) and requests tile + 3
        fetch8(first_tile);
        store8(first_tile);
        fetch8(min(first_tile + 1, last));
        store8(first_tile + 1);
        fetch8(min(first_tile + 2, last));
    } else {
        issue(first_tile);
        issue(min(first_tile + 1, last));
        issue(min(first_tile + 2, last));
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
        qreg[ks] = m_valid ? convert8<TIO, T>(qreg[ks]) : make_uint4(0, 0, 0, 0);
    }
    if constexpr (!KV8) {
        dma_wait<2 * PER_WAVE>();
    }
    __syncthreads();
    fetch_k((first_tile % kStages) * STAGE, 0);
    using MaskOn = std::integral_constant<bool, true>;
    using MaskOff = std::integral_constant<bool, false>;
    auto tile_iter = [&](uint32_t tile, auto mask_tag) {
        const uint32_t so = (tile % kStages) * STAGE;
        const uint32_t so_next = (min(tile + 1, last) % kStages) * STAGE;
        const uint32_t j0 = tile * BN;
        step(so, 0, j0, so, 1, mask_tag);
        if constexpr (KV8) {
            store8(tile + 2);
            __syncthreads();
            fetch8(min(tile + 3, last));
        } else {
            dma_wait<PER_WAVE>();   // this wave's share of tile + 1 has landed
            __syncthreads();        // ... and everybody else's; stage (tile - 1) % 4 is free
            issue(min(tile + 3, last));
        }
        step(so, 1, j0 + 32, so_next, 0, mask_tag);
    };
    // Tiles wholly below the causal limit of every row of the wave need no mask. Two loops rather than a
    // branch in one: each loop body exists once, so the accumulators keep their registers. Every wave runs
    // n_tiles iterations in total (one barrier each), wherever its own boundary between the loops lies.
    const uint32_t first_masked = min(n_tiles, wave_min_vis / BN);
    uint32_t tile = first_tile;
    if (m_first + wave * 32 < m_rows) {
        for (; tile < first_masked; tile++) {
            tile_iter(tile, MaskOff{});
        }
        for (; tile < n_tiles; tile++) {
            tile_iter(tile, MaskOn{});
        }
    } else {
        // none of the wave's 32 rows exists (the last M tile of a sequence; a decode row in a mixed batch
        // fills 4 of 256): the wave only keeps copying its share and meeting the others at the barrier
        for (; tile < n_tiles; tile++) {
            if constexpr (KV8) {
                store8(tile + 2);
                __syncthreads();
                fetch8(min(tile + 3, last));
            } else {
                dma_wait<PER_WAVE>();
                __syncthreads();
                issue(min(tile + 3, last));
            }
        }
    }
    dma_wait<0>();
    if (probe) {
        p.clock_probe[2] = clock64();
        p.clock_probe[3] = wall_clock64();
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);
    // O^T lane layout: column = M row, register k of tile dt = element 32 dt + 8 (k / 4) + 4 half + k % 4
    if (n_splits == 1) {
        // Final values leave through LDS (stored straight from this layout a lane writes 8 bytes of its own row per
        // instruction, 64 scattered pieces: 4 us per workgroup): every wave lays its 32 rows out row-major in its
        // own part of the stage memory and stores them 16 bytes per lane, a row by consecutive lanes.
        constexpr int PITCH = ROWB + 8;     // rows 8 bytes apart in the bank window: the 32 lanes of a write pass differ
        constexpr int LPR = ROWB / 16;      // lanes per row of the store
        constexpr int RPI = 64 / LPR;       // rows per store instruction
        __syncthreads();   // every wave has left the loop and nothing is in flight: the stages are free
        unsigned char *mine = smem + wave * (32 * PITCH);
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
#pragma unroll
            for (int kg = 0; kg < 4; kg++) {
                uint2 o;
                o.x = TIO::pack(O[dt][kg * 4] * inv, O[dt][kg * 4 + 1] * inv);
                o.y = TIO::pack(O[dt][kg * 4 + 2] * inv, O[dt][kg * 4 + 3] * inv);
                *reinterpret_cast<uint2 *>(mine + col * PITCH + (dt * 32 + kg * 8 + half * 4) * 2) = o;
            }
        }
        // lane `col` knows where row `col` goes (0: the row does not exist)
        const uint64_t my_dst = m_valid ? reinterpret_cast<uint64_t>(p.out + static_cast<uint64_t>(tok) * p.out_tok_stride +
                                                                     static_cast<uint64_t>(head) * D)
                                        : 0;
#pragma unroll
        for (int i = 0; i < 32 / RPI; i++) {
            const uint32_t r = lane / LPR + RPI * i;
            const uint64_t dst = __shfl(my_dst, static_cast<int>(r));
            const unsigned char *src = mine + r * PITCH + (lane % LPR) * 16;
            const uint2 lo = *reinterpret_cast<const uint2 *>(src), hi = *reinterpret_cast<const uint2 *>(src + 8);
            if (dst != 0) {
                *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(dst) + (lane % LPR) * 16) = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
        }
    }
    if (m_valid) {
        const uint64_t rh = static_cast<uint64_t>(tok) * p.n_heads + head;
        if (n_splits > 1) {
            // this run's partial: a row that sees none of the run's positions leaves (-inf, 0, zeros)
            const uint64_t slot = rh * p.max_splits + split;
            float *dst = p.part_acc + slot * D;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                for (int kg = 0; kg < 4; kg++) {
                    *reinterpret_cast<float4 *>(dst + dt * 32 + kg * 8 + half * 4) =
                        make_float4(O[dt][kg * 4], O[dt][kg * 4 + 1], O[dt][kg * 4 + 2], O[dt][kg * 4 + 3]);
                }
            }
            if (half == 0) {
                *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run * kLog2e, l_tot);
            }
        }
        if (half == 0 && split == 0 && p.part_cnt != nullptr) {
            p.part_cnt[rh] = n_splits == 1 ? 0 : static_cast<int32_t>(n_splits);
        }
    }
}

}  // namespace

bool prefill_mfma_supported(const AttentionArgs &a)
{
    // the division by the block size is a multiply-high, exact while position * block_size < 2^32
    // the positions of one copy instruction (1 KiB: four rows of head_dim 128, eight of head_dim 64) share a block
    const uint32_t per_copy = a.head_dim == 128 ? 4 : 8;
    // the sequence's block-table row is staged in LDS behind the KV stages
    const size_t lds = static_cast<size_t>(kStages) * 2 * BN * a.head_dim * 2 +
                       (static_cast<size_t>(a.max_num_block) + 1) * sizeof(uint32_t);
    return (a.head_dim == 128 || a.head_dim == 64) && a.kv_dtype == XLITE_HIP_KV_SAME && a.block_size % per_copy == 0 &&
           lds <= kLdsLimit &&
           static_cast<uint64_t>(a.max_num_block) * a.block_size * a.block_size < (1ull << 32) &&
           a.n_heads % a.n_kv_heads == 0;
}

// 8-bit caches read by the kernel itself: head_dim 128, block sizes that are multiples of 8 (a wave's eight positions of
// a tile share a block)
bool prefill_kv8_supported(const AttentionArgs &a)
{
    const size_t lds = static_cast<size_t>(kStages) * 2 * BN * a.head_dim * 2 +
                       (static_cast<size_t>(a.max_num_block) + 1) * sizeof(uint32_t);
    return a.head_dim == 128 && (a.kv_dtype == XLITE_HIP_KV_INT8 || a.kv_dtype == XLITE_HIP_KV_FP8) &&
           a.k_scale != nullptr && a.v_scale != nullptr && a.block_size % 8 == 0 && lds <= kLdsLimit &&
           static_cast<uint64_t>(a.max_num_block) * a.block_size * a.block_size < (1ull << 32) &&
           a.n_heads % a.n_kv_heads == 0;
}

// KV splits per M tile. The cost of s splits, in units of one workgroup walking the longest possible context:
//     (rounds of workgroups over the chip) x (1 / s of the walk + a workgroup's set-up and drain, about four KV
//     tiles' time) + s x (the partials' trip through memory: fp32 O per row and head, written and read back)
// With fewer workgroups than compute units that is the old rule (rounds / s); it also cuts the last round of a
// batch that fills the chip once and a bit (a chunk's tail: 292 workgroups on 256 compute units run two rounds,
// three splits run four rounds of a third each). Each split keeps at least kMinSplitTiles tiles of the longest context.
uint32_t prefill_mfma_pick_splits(uint32_t total_tokens, uint32_t group, uint32_t batch, uint32_t n_kv_heads,
                                  uint32_t max_ctx, uint32_t head_dim)
{
    const uint64_t base = (static_cast<uint64_t>(ceil_div(total_tokens * group, static_cast<uint32_t>(kMTile))) + batch) *
                          n_kv_heads;
    const uint64_t n_cu = 256;
    const uint32_t cap = min(64u, max_ctx / (kMinSplitTiles * BN));
    if (cap <= 1) {
        return 1;
    }
    constexpr double kTileUs = 2.2;         // one KV tile of 64 positions, measured on the chunked-prefill shape
    constexpr double kPartialGBs = 4000.0;  // what the partials' round trip sustains
    const double walk_us = static_cast<double>(max_ctx) / BN * kTileUs;
    const double setup = 4.0 * kTileUs / walk_us;
    const double part = static_cast<double>(total_tokens) * group * n_kv_heads * head_dim * 8.0 / (kPartialGBs * 1e3) / walk_us;
    auto cost = [&](uint32_t n) {
        const double rounds = static_cast<double>((base * n + n_cu - 1) / n_cu);
        return rounds * (1.0 / n + setup) + (n > 1 ? part * n : 0.0);
    };
    uint32_t best = 1;
    double best_cost = cost(1);
    for (uint32_t n = 2; n <= cap; n++) {
        const double c = cost(n);
        if (c < best_cost * (best == 1 ? 0.95 : 1.0)) {   // splitting at all has to pay clearly
            best = n;
            best_cost = c;
        }
    }
    return best;
}

size_t prefill_mfma_workspace_bytes(uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                    uint32_t batch, uint32_t max_ctx)
{
    const uint32_t splits = prefill_mfma_pick_splits(total_tokens, n_heads / n_kv_heads, batch, n_kv_heads, max_ctx, head_dim);
    return splits <= 1 ? 0 : partial_bytes(total_tokens, n_heads, head_dim, splits);
}

int launch_prefill_mfma(hipStream_t stream, const AttentionArgs &a)
{
    const uint32_t G = a.n_heads / a.n_kv_heads;
    PrefillParams p{};
    p.clock_probe = clock_probe();
    p.q = static_cast<const uint16_t *>(a.qkv);
    p.k_cache = static_cast<const uint16_t *>(a.k_cache);
    p.v_cache = static_cast<const uint16_t *>(a.v_cache);
    p.out = static_cast<uint16_t *>(a.output);
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.q_tok_stride = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim;
    p.out_tok_stride = a.n_heads * a.head_dim;
    p.group = G;
    p.n_kv_heads = a.n_kv_heads;
    p.batch = a.batch;
    p.block_size = a.block_size;
    p.block_magic = static_cast<uint32_t>((1ull << 32) / a.block_size) + 1;
    p.max_num_block = a.max_num_block;
    // tile ids: every sequence may end with a ragged tile (see the kernel's numbering)
    p.n_mtiles = ceil_div(a.total_tokens * G, static_cast<uint32_t>(kMTile)) + a.batch;
    p.n_heads = a.n_heads;
    p.skip_single = a.rows_mode == kSkipSingle ? 1u : 0u;
    p.k_scale = a.k_scale;
    p.v_scale = a.v_scale;
    const bool kv8 = a.kv_dtype != XLITE_HIP_KV_SAME;
    XL_REQUIRE(!kv8 || prefill_kv8_supported(a), "8-bit caches: shape not served by the prefill kernel");
    uint32_t splits = prefill_mfma_pick_splits(a.total_tokens, G, a.batch, a.n_kv_heads, a.max_num_block * a.block_size, a.head_dim);
    if (a.workspace == nullptr || a.workspace_bytes < partial_bytes(a.total_tokens, a.n_heads, a.head_dim, splits)) {
        splits = 1;   // no scratch: every M tile walks its whole KV range
    }
    p.max_splits = splits;
    const PartialBuffers pb = splits > 1 ? carve_partials(a.workspace, a.total_tokens, a.n_heads, a.head_dim, splits)
                                         : PartialBuffers{};
    p.part_cnt = pb.cnt;
    p.part_acc = pb.acc;
    p.part_ml = pb.ml;

    const size_t lds = static_cast<size_t>(kStages) * 2 * BN * a.head_dim * 2 +
                       (static_cast<size_t>(a.max_num_block) + 1) * sizeof(uint32_t);
    const bool bf = a.dtype == XLITE_HIP_BF16;
    XL_REQUIRE(lds <= kLdsLimit, "block table too long for the prefill kernel");
    XL_REQUIRE(!a.io_bf16 || a.dtype == XLITE_HIP_FP16, "bf16 rows over fp16 caches: the products are fp16");
    // (T, D, TIO, KVF) of the launch
    auto with_kernel = [&](auto &&f) {
        using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
        using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
        using SAME = std::integral_constant<int, XLITE_HIP_KV_SAME>;
        using D128 = std::integral_constant<int, 128>;
        using D64 = std::integral_constant<int, 64>;
        if (kv8) {   // fp16 products, rows and results in the model's type
            if (a.kv_dtype == XLITE_HIP_KV_INT8) {
                return bf ? f(FP16{}, D128{}, BF16{}, I8{}) : f(FP16{}, D128{}, FP16{}, I8{});
            }
            return bf ? f(FP16{}, D128{}, BF16{}, F8{}) : f(FP16{}, D128{}, FP16{}, F8{});
        }
        if (a.io_bf16) {
            return a.head_dim == 128 ? f(FP16{}, D128{}, BF16{}, SAME{}) : f(FP16{}, D64{}, BF16{}, SAME{});
        }
        if (a.head_dim == 128) {
            return bf ? f(BF16{}, D128{}, BF16{}, SAME{}) : f(FP16{}, D128{}, FP16{}, SAME{});
        }
        return bf ? f(BF16{}, D64{}, BF16{}, SAME{}) : f(FP16{}, D64{}, FP16{}, SAME{});
    };
    uint32_t n_wg;
    if (a.n_kv_heads % kXcds == 0) {
        n_wg = a.n_kv_heads * p.n_mtiles;
    } else if (kXcds % a.n_kv_heads == 0) {
        n_wg = kXcds * ceil_div(p.n_mtiles, kXcds / a.n_kv_heads);
    } else {
        n_wg = a.n_kv_heads * p.n_mtiles;
    }
    const dim3 grid(n_wg, splits, 1);
    const int rc_launch = with_kernel([&](auto t, auto d, auto tio, auto kvf) -> int {
        auto kernel = prefill_kernel<decltype(t), decltype(d)::value, decltype(tio), decltype(kvf)::value>;
        if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) {
            return rc;
        }
        kernel<<<grid, kThreads, lds, stream>>>(p);
        return XLITE_HIP_OK;
    });
    if (rc_launch != XLITE_HIP_OK) {
        return rc_launch;
    }
    XL_LAUNCH_CHECK();
    if (splits == 1) {
        return XLITE_HIP_OK;
    }
    return launch_merge(stream, a.io_bf16 ? XLITE_HIP_BF16 : a.dtype, a.output, pb, a.total_tokens, a.n_heads, a.head_dim, splits);
}

}  // namespace xlite
