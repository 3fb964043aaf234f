// GQA flash-decode on the matrix cores, split along the KV axis.
//
// Workgroup = 8 wavefronts = one (sequence, KV tile). The tile is walked in steps of 16 positions.
// All 512 threads fetch a step's cache bytes in address order (HBM streams best when every
// wave-wide load covers 1 KiB of consecutive memory; 256-byte rows at a 2 KiB stride reach only
// ~60 % of that), then every wave computes ONE kv head of the step (passes over groups of 8 kv
// heads when there are more; when there are fewer, the spare waves take sub ranges of the tile):
//   global -> registers : 16 bytes per lane; two steps are always in flight (a single batch per
//                         wave leaves HBM idle for one round trip between batches)
//   registers -> LDS    : two stages (one barrier per step); rows stored 16-bit, row major, 16-byte
//                         chunks XOR-swizzled so that both read patterns below are conflict free
//   S^T[token][head]  = K . Q^T    v_mfma_f32_16x16x32 (A = K rows via ds_read_b128, B = Q regs)
//   O^T[d][head]     += V^T . P^T  v_mfma_f32_16x16x16 (A = V^T via ds_read_b64_tr_b16, B = P regs)
// The query heads that share the kv head are the 16 MFMA columns (unused columns carry zeros), so
// one lane column owns one head: the online softmax needs two cross-lane exchanges per step, and P leaves the first product in the register layout the second one consumes.
// int8 caches are widened to 16 bit (exactly) on their way into LDS; their per-position scales are
// applied to the scores (K) and to the probabilities (V).
//
// Each wave leaves an fp32 partial (max, sum, O) per query head in the workspace; a small second
// kernel merges the partials of every query row (merge.hip).
//
// Replaces the split-KV path of the reference (xlite/csrc/kernels/flash_attention.h:323-628) for
// batches with as many query rows as sequences. The unit of work is the query row: in the usual decode
// step every sequence has one, but sequences without rows and sequences with several (row r sees
// cached + r + 1 positions) are served alike.
#include "attention_common.h"
#include "rope_item.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWaves = 8;
constexpr int kStep = 16;  // positions per inner step

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
    // k = 16: four 16-bit elements per lane
    static __device__ __forceinline__ f32x4_t run16(const s16x4_t &a, const uint2 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mfma16<FP16> {
    static __device__ __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t run16(const s16x4_t &a, const uint2 &b, f32x4_t c)
    {
        typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4_t;
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                     __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
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
    int32_t *part_meta;    // [token] int4: segments to merge (0: final), first chunk, first-segment flag
    float *part_acc;       // [slot][head][D]; chunk c of the work split owns slots 2c and 2c + 1
    float *part_ml;        // [slot][head][2]: maximum (log2 domain), normaliser
    uint32_t q_row_stride;
    uint32_t n_heads, n_kv_heads, group;
    uint32_t block_size;
    uint32_t max_num_block;
    uint32_t n_sub;        // sub ranges of a segment handled by different waves (kv heads < 8)
    uint32_t batch;
    uint32_t total_rows;   // query rows of the batch (one per sequence in a plain decode step)
    uint32_t only_single;  // 1: the units of the split are the sequences, and only those with one query row take part
    uint32_t unit0, n_units;   // this launch's slice of the units (rows or sequences): unit0 .. unit0 + n_units - 1
    uint32_t step_mult;    // steps (of 16 positions) the kernel takes at a time: chunks are multiples of it
    uint32_t block_magic;  // floor(2^32 / block_size) + 1: position / block_size == mulhi(position, magic) for positions
                           // below 2^32 / block_size; 0 when a table reaches further (then the kernels divide)
    uint32_t kv_per_wg;    // whole rows: kv heads of a workgroup (all of them, or 4, 2, 1 with n_sub = 8 / kv_per_wg); blockIdx.y
                           // counts the groups
    RopeArgs rope;         // the whole-row kernel that rotates and stores the step's rows itself: that call's arguments
};

// block and offset inside it of position t (a division by a run-time block size is some twenty instructions)
__device__ __forceinline__ uint32_t block_of(const DecodeMfmaParams &p, uint32_t t, uint32_t *off)
{
    const uint32_t blk = p.block_magic != 0 ? __umulhi(t, p.block_magic) : t / p.block_size;
    *off = t - blk * p.block_size;
    return blk;
}

// A cache row is read once per decode step: the non-temporal hint keeps it from displacing other lines
// on its way through the caches. Measured on batch 64 x 4096 positions: the LDS copies of the streaming
// kernels gain a tenth (5.7 -> 6.4 TB/s), 16-byte register loads 4 %, 8-byte ones lose 1 % and stay plain.
template <typename V>
__device__ __forceinline__ V ld_stream(const void *src)
{
    if constexpr (sizeof(V) == 16) {
        typedef uint32_t words_t __attribute__((ext_vector_type(4)));
        const words_t w = __builtin_nontemporal_load(static_cast<const words_t *>(src));
        V out;
        __builtin_memcpy(&out, &w, sizeof(V));
        return out;
    } else {
        return *static_cast<const V *>(src);
    }
}

// 8 cache elements (uint4 = 16-bit, uint2 = int8) -> 8 x 16-bit in a uint4
template <typename T>
__device__ __forceinline__ uint4 widen(const uint4 &raw) { return raw; }
// int8 -> fp16, exactly, in five vector instructions per four values: byte b ^ 0x80 = b + 128 as an
// unsigned byte u; the half-precision bit pattern 0x6400 | u is 1024 + u; minus 1152 leaves b. (The
// int8 path therefore runs its matrix products in fp16 whatever the activation type: every int8 value
// and every probability is exact or as precise in fp16 as in bf16.)
template <typename T>
__device__ __forceinline__ uint4 widen(const uint2 &raw)
{
    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
    const h2_t bias = {static_cast<_Float16>(-1152.0f), static_cast<_Float16>(-1152.0f)};
    const uint32_t src[2] = {raw.x ^ 0x80808080u, raw.y ^ 0x80808080u};
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t spread = __builtin_amdgcn_perm(0x64646464u, src[j / 2], (j % 2) ? 0x04030402u : 0x04010400u);
        const h2_t v = __builtin_bit_cast(h2_t, spread) + bias;
        w[j] = __builtin_bit_cast(uint32_t, v);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// fp8 (OCP e4m3) -> fp16 scaled by 2^-8, exactly, in three vector instructions per two values: the byte's
// exponent and mantissa fields, shifted to the top of fp16's, read as that format give the value times 2^-8
// (biases 7 and 15), for normal and subnormal bytes alike; the sign bit moves to bit 15. The factor 2^8 is
// applied to the scores and to the output. (NaN bytes, which a quantiser never writes, would read as finite.)
struct Fp8Tag {};
template <typename T>
__device__ __forceinline__ uint4 widen(const uint2 &raw, Fp8Tag)
{
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        // bytes (2 (j % 2), 2 (j % 2) + 1) of word j / 2 to the high bytes of the two halves
        const uint32_t x = __builtin_amdgcn_perm(0u, (&raw.x)[j / 2], (j % 2) ? 0x030c020cu : 0x010c000cu);
        w[j] = ((x >> 1) & 0x3f803f80u) | (x & 0x80008000u);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// XOR pattern applied to the 16-byte chunk index of LDS row `row`. One pattern serves both read shapes of a
// step's 16 rows. K as the MFMA A operand (ds_read_b128, lane = 16 j + row reads chunk 4 ks + j of its row): the
// hardware serves the instruction in four passes of 16 lanes, and a pass is lanes 0-3, 12-15, 20-23 and 24-27, then
// 4-11, 16-19 and 28-31 (the upper half of the wave likewise) - rows 0-3 and 12-15 of one chunk next to rows 4-11
// of its neighbour -, so those two row sets must own complete pairs of slots (2k, 2k + 1) of the 256-byte bank
// window. (Measured: with a pattern that only gives 16 consecutive lanes 16 different slots every such read took 8
// cycles instead of 4.) The transposing V read (ds_read_b64_tr_b16, passes of 32 lanes = 8 consecutive rows read as
// 32-byte pieces) needs those 8 rows in 8 different 32-byte slots. head_dim 64: two rows share a bank window and the
// pattern has three bits.
template <int D>
__device__ __forceinline__ uint32_t swizzle(uint32_t row)
{
    if constexpr (D == 128) {
        const uint32_t hi = (row >> 3) & 1;
        return (((row & 7) ^ (hi << 2)) << 1) | hi;
    } else {
        static_assert(D == 64, "patterns exist for head_dim 128 and 64");
        return row & 6;
    }
}

// ---------------------------------------------------------------------------------------------------
// Work split of the decode kernels: every query row owns ceil(limit / 16) steps, limit its visible range;
// the rows' steps laid end to end are cut into equal chunks, one per workgroup (the lengths live in
// device memory, so every workgroup computes the prefix sums itself), so that ragged batches keep every
// compute unit equally busy. A chunk that crosses a row boundary runs as several segments. Only a
// chunk's first and last segment can be parts of rows that continue in other chunks: chunk c owns the
// partial slots 2c (its first segment) and 2c + 1 (its last, when that is another one); a row cut into
// n segments that starts in chunk c0 finds them at 2 c0 (+ 1 unless it is that chunk's first segment),
// 2 (c0 + 1), ... and its meta entry (n, c0, first flag) tells the merge kernel so. Rows inside one
// chunk are final.
// ---------------------------------------------------------------------------------------------------
constexpr uint32_t kSplitTblCap = 1024;         // block-table entries staged per segment
constexpr uint32_t kSplitSeqCap = 4096;         // query rows whose prefix sums fit in LDS (with 2^28 steps in all)
constexpr uint32_t kSplitMinChunk = 4;          // steps: no chunk below 64 positions
constexpr uint32_t kSplitMaxWorkgroups = 512;   // grid bound the partial slots are sized for (one workgroup per compute unit)
constexpr uint32_t kSplitLdsWords = kSplitTblCap + kWaves;   // + rows + 1

// what is the same in every lane, said so: scalar address arithmetic follows
__device__ __forceinline__ uint32_t uni(uint32_t x)
{
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(x)));
}

// WHOLE: no split - workgroup i walks the whole range of the rows i, i + grid, ...: nothing to merge (a template
// parameter, so that each kernel has one call site for its segment body: a second copy of that body, or the extra live
// values of a run-time choice, cost the streaming kernels 4 %)
// ROPE (with WHOLE): the units are the sequences; `before.rows(first row, rows, ...)` runs ahead of a sequence's rows.
template <bool WHOLE = false, bool ROPE = false>
struct DecodeSplit {
    const DecodeMfmaParams &p;
    uint32_t *wave_tot, *pref;   // LDS: kWaves words, units + 1 words
    uint32_t lane, wave, R;      // R: units of the split - the batch's query rows, or its sequences (only_single)
    bool in_lanes;
    uint32_t ln_pref = 0, ln_steps = 0, ln_limit = 0, ln_seq = 0, ln_tok = 0, total = 0, chunk = 0, n_chunks = 0;

    // `lanes_ok`: a kernel short of registers keeps the sums in LDS whatever the batch
    __device__ __forceinline__ DecodeSplit(const DecodeMfmaParams &params, uint32_t *lds, uint32_t lane_, uint32_t wave_,
                                           bool lanes_ok = true)
        : p(params), wave_tot(lds), pref(lds + kWaves), lane(lane_), wave(wave_),
          R(params.n_units), in_lanes(lanes_ok && params.n_units <= 64)
    {
    }
    // The sequence that owns query row t. A batch of one row per sequence answers at once; otherwise (some
    // sequences without rows, others with several) the last sequence that starts at or before t: a
    // sequence without rows shares its start with its successor, so the last one is the owner.
    __device__ __forceinline__ uint32_t seq_of_row(uint32_t t) const
    {
        if (t < p.batch && p.query_start_loc[t] == static_cast<int32_t>(t) && p.lens[t] == 1) {
            return t;
        }
        uint32_t lo = 0, hi = p.batch;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (p.query_start_loc[mid] <= static_cast<int32_t>(t)) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        return lo;
    }
    // Steps of unit u; *limit = its visible range (row r of a sequence sees cached + r + 1 positions), *seq and
    // *tok its sequence and query row. With only_single the unit is sequence u, which takes part when it has
    // exactly one row; the rows of the others are marked "nothing to merge" (`mark`, first workgroup only): another
    // kernel writes them.
    __device__ __forceinline__ uint32_t steps_of(uint32_t u, uint32_t *limit, uint32_t *seq, uint32_t *tok, bool mark) const
    {
        u += p.unit0;   // units are numbered inside the launch's slice
        if (p.only_single) {
            const int32_t ql = p.lens[u], start = p.query_start_loc[u], cached = p.cached_lens[u];   // one trip for the three
            *seq = u;
            *tok = static_cast<uint32_t>(start);
            if (ql != 1) {
                if (mark && blockIdx.x == 0) {
                    for (int32_t r = 0; r < ql; r++) {
                        reinterpret_cast<int4 *>(p.part_meta)[start + r] = make_int4(0, 0, 0, 0);
                    }
                }
                *limit = 0;
                return 0;
            }
            const int32_t lim = cached + 1;
            *limit = static_cast<uint32_t>(lim > 1 ? lim : 1);
            return ceil_div(*limit, static_cast<uint32_t>(kStep));
        }
        // A decode batch (one row per sequence) answers at once, and its cached length is requested together with
        // the two loads that say so: one trip to memory instead of two.
        int32_t lim;
        uint32_t s = u;
        if (u < p.batch) {
            const int32_t start = p.query_start_loc[u], ql = p.lens[u], cached = p.cached_lens[u];
            if (start == static_cast<int32_t>(u) && ql == 1) {
                lim = cached + 1;
            } else {
                s = seq_of_row(u);
                lim = p.cached_lens[s] + (static_cast<int32_t>(u) - p.query_start_loc[s]) + 1;
            }
        } else {
            s = seq_of_row(u);
            lim = p.cached_lens[s] + (static_cast<int32_t>(u) - p.query_start_loc[s]) + 1;
        }
        *limit = static_cast<uint32_t>(lim > 1 ? lim : 1);
        *seq = s;
        *tok = u;
        return ceil_div(*limit, static_cast<uint32_t>(kStep));
    }
    // Exclusive prefix sums of the step counts. Up to 64 rows: every wave keeps them in its lanes
    // (lane = row), nothing goes through LDS. More: thread t owns `ipt` consecutive rows and the
    // sums land in LDS, each entry packed with its row's (limit - 1) % 16. Contains barriers in the
    // second case: every thread of the workgroup calls it.
    __device__ __forceinline__ void scan()
    {
        if constexpr (WHOLE) {   // (the rows are looked up one by one in for_each_segment)
            total = 1;
            return;
        }
        if (in_lanes) {
            if (lane < R) {
                ln_steps = steps_of(lane, &ln_limit, &ln_seq, &ln_tok, true);
            }
            uint32_t incl = ln_steps;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d);
                incl += lane >= static_cast<uint32_t>(d) ? up : 0u;
            }
            ln_pref = incl - ln_steps;
            total = uni(__shfl(incl, 63));
        } else {
            const uint32_t ipt = ceil_div(R, static_cast<uint32_t>(kWaves * 64));
            const uint32_t i0 = min(R, threadIdx.x * ipt), i1 = min(R, i0 + ipt);
            uint32_t mine = 0, limit, seq, tok;
            for (uint32_t i = i0; i < i1; i++) {
                mine += steps_of(i, &limit, &seq, &tok, true);
            }
            uint32_t incl = mine;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d);
                incl += lane >= static_cast<uint32_t>(d) ? up : 0u;
            }
            if (lane == 63) {
                wave_tot[wave] = incl;
            }
            __syncthreads();
            uint32_t before = 0;
            for (uint32_t w = 0; w < wave; w++) {
                before += wave_tot[w];
            }
            uint32_t run = before + incl - mine;
            for (uint32_t i = i0; i < i1; i++) {
                const uint32_t n = steps_of(i, &limit, &seq, &tok, false);
                pref[i] = (run << 4) | ((limit - 1) & 15u);
                run += n;
            }
            if (threadIdx.x == kWaves * 64 - 1) {
                pref[R] = (before + incl) << 4;
            }
            __syncthreads();
            total = uni(pref[R]) >> 4;
        }
        if (total != 0) {
            chunk = max(ceil_div(total, gridDim.x), kSplitMinChunk);
            chunk = ceil_div(chunk, p.step_mult) * p.step_mult;
            chunk = min(chunk, (kSplitTblCap - 2) * p.block_size / kStep / p.step_mult * p.step_mult);
            n_chunks = ceil_div(total, chunk);
        }
    }
    // first step, step count and visible range of unit i (*limit is meaningless when the unit has no steps)
    __device__ __forceinline__ void row_info(uint32_t i, uint32_t *first, uint32_t *n, uint32_t *limit) const
    {
        if (in_lanes) {
            *first = uni(__shfl(ln_pref, static_cast<int>(i)));
            *n = uni(__shfl(ln_steps, static_cast<int>(i)));
            *limit = uni(__shfl(ln_limit, static_cast<int>(i)));
        } else {
            const uint32_t a = uni(pref[i]), b = uni(pref[i + 1]);
            *first = a >> 4;
            *n = (b >> 4) - *first;
            *limit = (*n - 1) * kStep + (a & 15u) + 1;
        }
    }
    // the row that holds step `start`: the last one whose prefix is <= start
    __device__ __forceinline__ uint32_t row_of_step(uint32_t start) const
    {
        if (in_lanes) {
            const uint64_t mask = __ballot(lane < R && ln_pref <= start);
            return static_cast<uint32_t>(__builtin_popcountll(mask)) - 1;
        }
        uint32_t lo = 0, hi = R;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uni(pref[mid]) >> 4) <= start) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        return lo;
    }
    __device__ __forceinline__ uint32_t seq_of(uint32_t unit) const
    {
        if (p.only_single) {
            return uni(unit + p.unit0);
        }
        return in_lanes ? uni(__shfl(ln_seq, static_cast<int>(unit))) : uni(seq_of_row(uni(unit + p.unit0)));
    }
    __device__ __forceinline__ uint32_t tok_of(uint32_t unit) const
    {
        if (!p.only_single) {
            return uni(unit + p.unit0);
        }
        return in_lanes ? uni(__shfl(ln_tok, static_cast<int>(unit))) : uni(static_cast<uint32_t>(p.query_start_loc[uni(unit + p.unit0)]));
    }
    // segment(seq, row, t0, t1, whole, partial slot, first piece of its row, meta of the row)
    struct NoPrologue {
        __device__ __forceinline__ int guess(uint32_t) const { return 0; }
        __device__ __forceinline__ void together(int &, int32_t &, int32_t &, int32_t &) const {}
        __device__ __forceinline__ void rows(uint32_t, uint32_t, uint32_t, int) const {}
    };
    template <typename F, typename G = NoPrologue>
    __device__ __forceinline__ void for_each_segment(F &&segment, G &&before = G()) const
    {
        if constexpr (WHOLE && ROPE) {
            // by sequence: the rows of a sequence see each other's new cache rows, so one workgroup writes them all
            // before it walks any. A plain decode step has one row per sequence, row s for sequence s: what the
            // prologue needs of that row is requested (`guess`) together with the three words that say whether the
            // guess holds.
            for (uint32_t s = blockIdx.x; s < p.batch; s += gridDim.x) {
                auto guessed = before.guess(s);
                int32_t start = p.query_start_loc[s], ql = p.lens[s], cached = p.cached_lens[s];
                before.together(guessed, start, ql, cached);
                if (ql <= 0) {
                    continue;
                }
                before.rows(uni(static_cast<uint32_t>(start)), uni(static_cast<uint32_t>(ql)), s, guessed);
                for (int32_t r = 0; r < ql; r++) {
                    const int32_t lim = cached + r + 1;
                    segment(uni(s), uni(static_cast<uint32_t>(start + r)), 0u, uni(static_cast<uint32_t>(lim > 1 ? lim : 1)), true,
                            0u, false, make_int4(0, 0, 0, 0));
                }
            }
        } else if constexpr (WHOLE) {
            // batches whose contexts are short by the width of their block tables: a row is one segment, stored
            // directly, and there is no second launch to merge anything (a step of such a batch is bound by its
            // launches, not by its bytes)
            for (uint32_t row = blockIdx.x; row < R; row += gridDim.x) {
                uint32_t limit, seq, tok;
                const uint32_t n = steps_of(row, &limit, &seq, &tok, false);
                if (n != 0) {
                    segment(uni(seq), uni(tok), 0u, uni(limit), true, 0u, false, make_int4(0, 0, 0, 0));
                }
            }
        } else {
            for (uint32_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
                const uint32_t start = c * chunk, end = min(total, start + chunk);
                uint32_t row = row_of_step(start), pos = start;
                while (pos < end) {
                    uint32_t first, n, limit;
                    row_info(row, &first, &n, &limit);
                    if (n == 0) {   // a unit that takes no part (units without steps share their prefix with the next one)
                        row++;
                        continue;
                    }
                    const uint32_t a = pos - first, b = min(n, a + (end - pos));
                    const bool whole = a == 0 && b == n;
                    const bool first_seg = pos == start;
                    const uint32_t n_slots = whole ? 0u : (first + n - 1) / chunk - c + 1;
                    const int4 meta = make_int4(static_cast<int>(n_slots), static_cast<int>(c), first_seg ? 1 : 0, 0);
                    segment(seq_of(row), tok_of(row), uni(a * kStep), uni(min(limit, b * kStep)), whole,
                            uni(2 * c + (first_seg ? 0u : 1u)), a == 0, meta);
                    pos += b - a;
                    row++;
                }
            }
        }
    }
};

// ROPE (whole rows over a 16-bit cache): the kernel is a layer's rope_and_cache and attention in one launch. The
// workgroup of a sequence rotates the sequence's new rows in place and stores their k and v in the cache (the items of
// rope_and_cache, spread over its 512 threads), and walks the rows behind a barrier: a workgroup sees its own stores.
template <typename T, int D, int KVF, bool MULTI_SUB, bool WHOLE = false, bool ROPE = false>
__global__ void __launch_bounds__(kWaves * 64)
decode_mfma_kernel(const DecodeMfmaParams p)
{
    constexpr bool KV8 = KVF != XLITE_HIP_KV_SAME;                  // a cache of bytes with per-position scales
    constexpr float kKvMul = KVF == XLITE_HIP_KV_FP8 ? 256.f : 1.f;  // fp8 bytes are widened to value * 2^-8
    constexpr int CH = D / 8;            // 16-byte chunks per LDS row
    constexpr int ROWB = D * 2;          // LDS bytes per row
    constexpr int KS = D / 32;           // k-steps of the QK product
    constexpr int MT = D / 16;           // 16-row tiles of O^T
    constexpr int TILE_BYTES = kStep * ROWB;
    constexpr int NT = kWaves * 64;
    constexpr int NV = kWaves * kStep * CH / NT;  // 16-byte vectors per thread, step and tensor
    constexpr int STAGE_BYTES = kWaves * 2 * TILE_BYTES;
    typedef typename std::conditional<KV8, uint2, uint4>::type gvec_t;
    typedef typename std::conditional<KV8, FP16, T>::type TM;   // element type of the matrix products

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    // LDS: two stages; in a stage one region per (kv head, sub range) pair of the pass = per
    // computing wave, K tile then V tile. int8 caches: behind the stages, the scales of the two
    // stages [stage][K | V][region][16 positions]
    const uint32_t my_lds = wave * 2 * TILE_BYTES;
    float *sc_lds = reinterpret_cast<float *>(smem + 2 * STAGE_BYTES);
    // block-table entries of the tile, copied once per query row: a lookup inside the streaming
    // loop must not be a vector memory load, whose completion can only be awaited together with
    // every cache load issued before it (that would drain the prefetch pipeline at every step)
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(smem + 2 * STAGE_BYTES + (KV8 ? 2 * 2 * kWaves * kStep * 4 : 0));

    // ---- compute roles -------------------------------------------------------------------------------
    const uint32_t col = lane & 15;       // MFMA column = query head inside the group
    const uint32_t jq = lane >> 4;        // 16-lane group
    uint32_t kr_off[KS];                  // K rows as the A operand of the QK product
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        kr_off[ks] = my_lds + col * ROWB + (((4 * ks + jq) ^ swizzle<D>(col)) << 4);
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
            vr_off[mt] = my_lds + TILE_BYTES + pos * ROWB + (((2 * mt + (q4 >> 1)) ^ swizzle<D>(pos)) << 4) + ((q4 & 1) << 3);
        }
    }

    // ---- loader roles: the 512 threads fetch the step's cache bytes in address order, so that every
    // wave-wide load covers 1 KiB of consecutive memory. Vector v = tid + 512 i of a step:
    // chunk = v % CH, kv head (inside the pass) = (v / CH) % KVW, position = (v / (CH KVW)) % 16,
    // sub range = v / (CH KVW 16). KVW = kv heads per pass (a power of two), KVW * n_sub = 8.
    const uint32_t kvw = kWaves / p.n_sub;
    const uint32_t kvw_shift = __builtin_ctz(kvw);
    const uint32_t lc = threadIdx.x % CH;
    auto vec_kvl = [&](int i) { return ((threadIdx.x + NT * i) / CH) & (kvw - 1); };
    auto vec_pos = [&](int i) { return ((threadIdx.x + NT * i) / CH >> kvw_shift) & (kStep - 1); };
    auto vec_sub = [&](int i) { return MULTI_SUB ? ((threadIdx.x + NT * i) / (CH * kStep)) >> kvw_shift : 0u; };
    uint32_t w_off[NV];   // LDS offset of the K vector; its V twin sits TILE_BYTES further
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const uint32_t region = vec_sub(i) * kvw + vec_kvl(i);   // the wave that consumes this vector
        w_off[i] = region * 2 * TILE_BYTES + vec_pos(i) * ROWB + ((lc ^ swizzle<D>(vec_pos(i))) << 4);
    }
    // scale loader (int8 caches): threads 0..127 fetch the K scales of the step, 128..255 the V scales
    const uint32_t sj = threadIdx.x & 127;
    const bool s_active = KV8 && threadIdx.x < 256;
    const uint32_t s_kvl = sj & (kvw - 1), s_pos = (sj >> kvw_shift) & (kStep - 1);
    const uint32_t s_sub = MULTI_SUB ? sj >> (kvw_shift + 4) : 0u;
    const float *s_src = threadIdx.x < 128 ? p.k_scale : p.v_scale;
    const uint32_t s_dst = (threadIdx.x < 128 ? 0 : kWaves * kStep) + (s_sub * kvw + s_kvl) * kStep + s_pos;

    const gvec_t *kc = static_cast<const gvec_t *>(p.k_cache);
    const gvec_t *vc = static_cast<const gvec_t *>(p.v_cache);
    const uint32_t g_valid = p.group < 16 ? p.group : 16;
    const uint32_t my_kvl = wave & (kvw - 1), my_sub = wave >> kvw_shift;
    // the workgroup's kv heads: all of them, or (whole rows of a batch that leaves compute units idle) one group of
    // kv_per_wg per workgroup - heads are independent, so rows cut this way still need no merge
    uint32_t kv_begin = 0, kv_end = p.n_kv_heads;
    if constexpr (WHOLE) {
        kv_begin = blockIdx.y * p.kv_per_wg;
        kv_end = min(p.n_kv_heads, kv_begin + p.kv_per_wg);
    }

    // one segment: positions [t0, t1) of the row `tok` of sequence `seq`. `single`: the result is final;
    // otherwise it goes to partial slot `pslot`. With fewer than 8 kv heads the waves of a kv head take equal
    // sub ranges of the segment and combine their results through LDS at its end.
    auto run_segment = [&](uint32_t seq, uint32_t tok, uint32_t t0, uint32_t t1, bool single, uint32_t pslot, bool write_meta,
                           int4 meta) {
        const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;
        const uint32_t sub_len = ceil_div(ceil_div(t1 - t0, static_cast<uint32_t>(kStep)), p.n_sub) * kStep;
        // every sub range runs the same number of steps (the first one is never shorter than the others)
        const uint32_t n_steps = ceil_div(min(t1 - t0, sub_len), kStep);
        const uint32_t ta = min(t1, t0 + my_sub * sub_len);   // this wave's range
        const uint32_t tb = min(t1, ta + sub_len);
        const uint32_t blk0 = t0 / p.block_size;
        // ---- Q^T as the B operand: column = head, 8 consecutive elements per k group. The first pass's rows are
        // requested ahead of the block-table entries: one trip to memory for the two.
        uint4 qreg[KS];
        auto request_q = [&](uint32_t kv0) {
            // Every lane loads: columns past the group's heads (and waves past the last kv head) repeat the last valid
            // head, and their results are never stored. (A load under a per-lane condition is compiled into a branch
            // with a wait of its own: one trip to memory per load instead of one for all.)
            const uint32_t kvh = min(kv0 + my_kvl, p.n_kv_heads - 1);
            const uint16_t *qrow = p.q + static_cast<uint64_t>(tok) * p.q_row_stride +
                                   static_cast<uint64_t>(kvh * p.group + min(col, g_valid - 1)) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                qreg[ks] = *reinterpret_cast<const uint4 *>(qrow + ks * 32 + jq * 8);
            }
        };
        request_q(kv_begin);
        {
            const uint32_t nblk = (t1 - 1) / p.block_size - blk0 + 1;
            for (uint32_t i = threadIdx.x; i < nblk; i += NT) {
                tbl_lds[i] = static_cast<uint32_t>(table[blk0 + i]);
            }
            if (write_meta && threadIdx.x == 0) {
                reinterpret_cast<int4 *>(p.part_meta)[tok] = meta;
            }
            __syncthreads();
        }

        // passes over groups of `kvw` kv heads
        for (uint32_t kv0 = kv_begin; kv0 < kv_end; kv0 += kvw) {
            const uint32_t kvh = kv0 + my_kvl;
            const bool kv_ok = kvh < kv_end;
            const uint32_t head0 = kvh * p.group;

            {
                if (kv0 != kv_begin) {
                    request_q(kv0);
                }
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    if constexpr (KV8 && !std::is_same<T, TM>::value) {   // bf16 activations: q as fp16
                        uint32_t *w = reinterpret_cast<uint32_t *>(&qreg[ks]);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            w[j] = TM::pack(T::to_f32(static_cast<uint16_t>(w[j] & 0xffff)), T::to_f32(static_cast<uint16_t>(w[j] >> 16)));
                        }
                    }
                }
                // Consume the query registers here, before any cache load is issued: their first real
                // use is inside the streaming loop, where waiting for them would mean waiting for
                // every prefetched cache load issued since (memory loads complete in order).
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
                }
            }
            f32x4_t O[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                O[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
            float m_run = -INFINITY, l_run = 0.f;

            // byte offset of this thread's i-th vector from the first cache row of its sub range's
            // step; kv heads past the last one (a pass may be ragged) re-read the last head.
            // Positions at or beyond the end of a range (last step only) re-read the last valid
            // position instead: their probabilities are forced to zero, and a finite value times
            // zero cannot poison the products the way stale cache bytes (NaN) could.
            constexpr uint32_t VB = sizeof(gvec_t);
            const uint32_t row_bytes = p.n_kv_heads * CH * VB;
            uint32_t g_off[NV];
#pragma unroll
            for (int i = 0; i < NV; i++) {
                g_off[i] = vec_pos(i) * row_bytes + (min(kv0 + vec_kvl(i), p.n_kv_heads - 1) * CH + lc) * VB;
            }
            const uint32_t s_off = s_pos * p.n_kv_heads + min(kv0 + s_kvl, p.n_kv_heads - 1);

            // two register sets: two steps are in flight at any time, so that the memory system always
            // has queued work when a step's data has arrived
            gvec_t kreg[2][NV], vreg[2][NV];
            float sreg[2] = {0.f, 0.f};
            // first position of a step of sub range `sub`: its 16 positions share one block
            // (block_size % 16 == 0 and every range starts at a multiple of 16)
            auto step_start = [&](uint32_t sub, uint32_t step) -> uint32_t {
                const uint32_t t = t0 + sub * sub_len + step * kStep;
                return t < t1 ? t : t0;   // exhausted sub range: any valid rows, nobody consumes them
            };
            auto row_of = [&](uint32_t t) -> uint64_t {
                uint32_t off;
                const uint32_t blk = block_of(p, t, &off);
                return (static_cast<uint64_t>(tbl_lds[blk - blk0]) * p.block_size + off) * p.n_kv_heads;
            };
            auto sub_end = [&](uint32_t sub) { return min(t1, t0 + (sub + 1) * sub_len); };
            // `raw_step` may lie beyond the last step (the pipeline's loads are unconditional): then every lane reads
            // the first 16 bytes of the last step, one cache line per instruction (the same rows again would be fetched
            // from memory again under the non-temporal hint)
            auto issue = [&](uint32_t raw_step, auto slot_tag) {
                constexpr int SL = decltype(slot_tag)::value;
                const uint32_t step = min(raw_step, n_steps - 1);
                const bool last_step = step + 1 == n_steps;
                const uint32_t keep = raw_step >= n_steps ? 0u : ~0u;
                if constexpr (!MULTI_SUB) {
                    const uint32_t ts = step_start(0, step);
                    const uint64_t row0 = row_of(ts);   // uniform: scalar address arithmetic
                    const char *kb = reinterpret_cast<const char *>(kc) + row0 * CH * VB;
                    const char *vb = reinterpret_cast<const char *>(vc) + row0 * CH * VB;
                    if (!last_step) {
#pragma unroll
                        for (int i = 0; i < NV; i++) {
                            kreg[SL][i] = ld_stream<gvec_t>(kb + g_off[i]);
                            vreg[SL][i] = ld_stream<gvec_t>(vb + g_off[i]);
                        }
                        if constexpr (KV8) {
                            if (s_active) {
                                sreg[SL] = s_src[row0 + s_off];
                            }
                        }
                    } else {
                        const uint32_t last_pos = t1 - 1 - ts;   // >= 0: the first range is never empty
#pragma unroll
                        for (int i = 0; i < NV; i++) {
                            const uint32_t back = vec_pos(i) > last_pos ? (vec_pos(i) - last_pos) * row_bytes : 0u;
                            kreg[SL][i] = ld_stream<gvec_t>(kb + ((g_off[i] - back) & keep));
                            vreg[SL][i] = ld_stream<gvec_t>(vb + ((g_off[i] - back) & keep));
                        }
                        if constexpr (KV8) {
                            if (s_active) {
                                const uint32_t back = s_pos > last_pos ? (s_pos - last_pos) * p.n_kv_heads : 0u;
                                sreg[SL] = s_src[row0 + ((s_off - back) & keep)];
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NV; i++) {
                        const uint32_t ts = step_start(vec_sub(i), step);
                        const uint32_t end = max(sub_end(vec_sub(i)), ts + 1);
                        const uint32_t last_pos = min(end - 1 - ts, static_cast<uint32_t>(kStep - 1));
                        const uint32_t back = vec_pos(i) > last_pos ? (vec_pos(i) - last_pos) * row_bytes : 0u;
                        const uint64_t row0 = row_of(ts);
                        kreg[SL][i] = ld_stream<gvec_t>(reinterpret_cast<const char *>(kc) + row0 * CH * VB + ((g_off[i] - back) & keep));
                        vreg[SL][i] = ld_stream<gvec_t>(reinterpret_cast<const char *>(vc) + row0 * CH * VB + ((g_off[i] - back) & keep));
                    }
                    if constexpr (KV8) {
                        if (s_active) {
                            const uint32_t ts = step_start(s_sub, step);
                            const uint32_t end = max(sub_end(s_sub), ts + 1);
                            const uint32_t last_pos = min(end - 1 - ts, static_cast<uint32_t>(kStep - 1));
                            const uint32_t back = s_pos > last_pos ? (s_pos - last_pos) * p.n_kv_heads : 0u;
                            sreg[SL] = s_src[row_of(ts) + s_off - back];
                        }
                    }
                }
            };
            // registers of set SL -> LDS stage SL (step s uses set and stage s % 2)
            auto stage_write = [&](auto slot_tag) {
                constexpr int SL = decltype(slot_tag)::value;
#pragma unroll
                for (int i = 0; i < NV; i++) {
                    if constexpr (KVF == XLITE_HIP_KV_FP8) {
                        *reinterpret_cast<uint4 *>(smem + SL * STAGE_BYTES + w_off[i]) = widen<T>(kreg[SL][i], Fp8Tag{});
                        *reinterpret_cast<uint4 *>(smem + SL * STAGE_BYTES + w_off[i] + TILE_BYTES) = widen<T>(vreg[SL][i], Fp8Tag{});
                    } else {
                        *reinterpret_cast<uint4 *>(smem + SL * STAGE_BYTES + w_off[i]) = widen<T>(kreg[SL][i]);
                        *reinterpret_cast<uint4 *>(smem + SL * STAGE_BYTES + w_off[i] + TILE_BYTES) = widen<T>(vreg[SL][i]);
                    }
                }
                if constexpr (KV8) {
                    if (s_active) {
                        sc_lds[SL * 2 * kWaves * kStep + s_dst] = sreg[SL];
                    }
                }
            };
            auto compute = [&](uint32_t step, auto slot_tag) {
                constexpr int SL = decltype(slot_tag)::value;
                const uint32_t t = ta + step * kStep;
                if (t >= tb) {
                    return;
                }
                const unsigned char *stage = smem + SL * STAGE_BYTES;
                // ---- S^T = K . Q^T: 16 positions x 16 heads ---------------------------------------------------
                f32x4_t S = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    const uint4 a = *reinterpret_cast<const uint4 *>(stage + kr_off[ks]);
                    S = Mfma16<TM>::run(a, qreg[ks], S);
                }
                // V^T operands do not depend on the softmax: fetch them now
                s16x4_t vt[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
                    vt[mt] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(const_cast<unsigned char *>(stage) + vr_off[mt]));
                }
                float4 kscale, vscale;
                if constexpr (KV8) {
                    const float *sc = sc_lds + SL * 2 * kWaves * kStep;
                    kscale = *reinterpret_cast<const float4 *>(sc + wave * kStep + 4 * jq);
                    vscale = *reinterpret_cast<const float4 *>(sc + (kWaves + wave) * kStep + 4 * jq);
                }
                // ---- online softmax; lane holds positions t + 4 jq + e of head `col` ----------------------------
                float mx = -INFINITY;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float v = S[e] * (kLog2e * kKvMul);
                    if constexpr (KV8) {
                        v *= reinterpret_cast<const float *>(&kscale)[e];
                    }
                    v = (t + 4 * jq + e) < tb ? v : -INFINITY;   // padding positions (also drops their NaN)
                    S[e] = v;
                    mx = fmaxf(mx, v);
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                const float m_new = fmaxf(m_run, mx);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                m_run = m_new;
                float pe[4];
                float psum = 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float x = fast_exp2(S[e] - m_safe);
                    psum += x;
                    if constexpr (KV8) {
                        pe[e] = (t + 4 * jq + e) < tb ? x * reinterpret_cast<const float *>(&vscale)[e] : 0.f;
                    } else {
                        pe[e] = x;
                    }
                }
                l_run = l_run * alpha + psum;
                const uint2 pb = make_uint2(TM::pack(pe[0], pe[1]), TM::pack(pe[2], pe[3]));
                // the running maximum rarely moves after the first steps: skip the rescale then
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        O[mt][0] *= alpha;
                        O[mt][1] *= alpha;
                        O[mt][2] *= alpha;
                        O[mt][3] *= alpha;
                    }
                }
                // ---- O^T += V^T . P^T (k = the 16 positions) ------------------------------------------------------
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    O[mt] = Mfma16<TM>::run16(vt[mt], pb, O[mt]);
                }
            };

            using S0 = std::integral_constant<int, 0>;
            using S1 = std::integral_constant<int, 1>;
            // Software pipeline: registers hold steps n+1 and n+2 while step n is computed from LDS.
            // Every load and LDS write below is unconditional (steps past the end read one line of the last
            // step and land in a stage nobody consumes): a conditional prefetch would force the
            // wait for the older batch to assume that the newer one was never issued, i.e. to wait
            // for everything in flight. (n_steps >= 1: the tile is not empty.)
            issue(0, S0{});
            issue(1u, S1{});
            stage_write(S0{});
            issue(2u, S0{});
            __syncthreads();
            for (uint32_t step = 0; step < n_steps; step += 2) {
                compute(step, S0{});
                stage_write(S1{});
                issue(step + 3, S1{});
                __syncthreads();
                compute(step + 1, S1{});
                stage_write(S0{});
                issue(step + 4, S0{});
                __syncthreads();
            }

            // ---- this wave's result for (kv head, sub range) -----------------------------------------------
            float l_tot = l_run + __shfl_xor(l_run, 16);
            l_tot += __shfl_xor(l_tot, 32);
            if constexpr (MULTI_SUB) {
                // the sub ranges of a kv head meet in its first wave: (m, l, O) of the others through the stage
                // memory, which nobody reads any more (every wave has passed the loop's last barrier)
                constexpr int XS = D + 4;   // floats per (wave, column): O, then m and l
                float *xch = reinterpret_cast<float *>(smem);
                if (my_sub != 0) {
                    float *dst = xch + (wave * 16 + col) * XS;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0) {
                        dst[D] = m_run;
                        dst[D + 1] = l_tot;
                    }
                }
                __syncthreads();
                if (my_sub == 0) {
                    for (uint32_t sub = 1; sub < p.n_sub; sub++) {
                        const float *src = xch + ((sub * kvw + my_kvl) * 16 + col) * XS;
                        const float m2 = src[D], l2 = src[D + 1];
                        const float m_new = fmaxf(m_run, m2);
                        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                        const float a1 = fast_exp2(m_run - m_safe), a2 = fast_exp2(m2 - m_safe);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++) {
                            const float4 o2 = *reinterpret_cast<const float4 *>(src + mt * 16 + jq * 4);
                            O[mt][0] = O[mt][0] * a1 + o2.x * a2;
                            O[mt][1] = O[mt][1] * a1 + o2.y * a2;
                            O[mt][2] = O[mt][2] * a1 + o2.z * a2;
                            O[mt][3] = O[mt][3] * a1 + o2.w * a2;
                        }
                        l_tot = l_tot * a1 + l2 * a2;
                        m_run = m_new;
                    }
                }
                __syncthreads();   // the next pass refills the stages
            }
            if (kv_ok && col < g_valid && my_sub == 0) {
                // O^T lane layout: column = head `col`, rows 16 mt + 4 jq + e
                // (fp8 cache: O carries the factor 2^-8 of the widened values; it leaves through the normaliser)
                if (single) {
                    const float inv = l_tot > 0.f ? kKvMul / l_tot : 0.f;
                    uint16_t *dst = p.out + (static_cast<uint64_t>(tok) * p.n_heads + head0 + col) * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        uint2 o;
                        o.x = T::pack(O[mt][0] * inv, O[mt][1] * inv);
                        o.y = T::pack(O[mt][2] * inv, O[mt][3] * inv);
                        *reinterpret_cast<uint2 *>(dst + mt * 16 + jq * 4) = o;
                    }
                } else {
                    const uint64_t slot = static_cast<uint64_t>(pslot) * p.n_heads + head0 + col;
                    float *dst = p.part_acc + slot * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0) {
                        *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run, l_tot * (1.0f / kKvMul));
                    }
                }
            }
        }
        __syncthreads();   // tbl_lds and the stages are rewritten by the next segment
    };

    DecodeSplit<WHOLE, ROPE> split(p, tbl_lds + kSplitTblCap, lane, wave, !(MULTI_SUB && D == 128));
    split.scan();
    if (split.total == 0) {
        return;
    }
    if constexpr (ROPE) {
        static_assert(WHOLE && !KV8, "the kernel rotates rows only when it takes them whole, over a 16-bit cache");
        // the head slots of the workgroup's kv heads: their query heads, then their k rows, then their v rows
        const uint32_t per_head = p.rope.head_dim / 8 - p.rope.rot_dim / 16;
        const uint32_t kvn = kv_end - kv_begin, nq = kvn * p.group;
        const uint32_t per_row = (nq + 2 * kvn) * per_head;
        auto slot_of = [&](uint32_t j) {
            const uint32_t jh = j / per_head;
            const uint32_t hs = jh < nq ? kv_begin * p.group + jh
                                        : (jh < nq + kvn ? p.n_heads + kv_begin + (jh - nq)
                                                         : p.n_heads + p.n_kv_heads + kv_begin + (jh - nq - kvn));
            return hs * per_head + j % per_head;
        };
        struct Prologue {
            const DecodeMfmaParams &p;
            decltype(slot_of) &slot_of;
            uint32_t per_row;
            // the thread's first item of row s, should that be the sequence's only row
            __device__ __forceinline__ RopeItemRegs guess(uint32_t s) const
            {
                return rope_item_load(p.rope, min(s, p.rope.num_tokens - 1), slot_of(min(threadIdx.x, per_row - 1)));
            }
            // One wait for all of it: left alone the compiler orders the loads by their first use, a trip to memory
            // for the row count, one for the other two words, one for the row.
            __device__ __forceinline__ void together(RopeItemRegs &x, int32_t &start, int32_t &ql, int32_t &cached) const
            {
                asm volatile("" : "+v"(x.a.v.x), "+v"(x.a.v.y), "+v"(x.a.v.z), "+v"(x.a.v.w), "+v"(x.b.v.x), "+v"(x.b.v.y),
                                  "+v"(x.b.v.z), "+v"(x.b.v.w), "+v"(x.pos_t), "+v"(x.slot), "+v"(start), "+v"(ql), "+v"(cached));
            }
            __device__ __forceinline__ void rows(uint32_t row0, uint32_t n, uint32_t s, const RopeItemRegs &guessed) const
            {
                uint32_t i = threadIdx.x;
                if (row0 == s && n == 1) {
                    if (i < per_row) {
                        rope_item_finish<T>(p.rope, row0, slot_of(i), guessed);
                    }
                    i += NT;
                }
                for (; i < n * per_row; i += NT) {
                    rope_item<T>(p.rope, row0 + i / per_row, slot_of(i % per_row));
                }
                __syncthreads();   // the rotated queries and the new cache rows are in memory before anyone reads them
            }
        };
        split.for_each_segment(run_segment, Prologue{p, slot_of, per_row});
    } else {
        split.for_each_segment(run_segment);
    }
}

// ---------------------------------------------------------------------------------------------------
// The same computation for the common shape (head_dim 128, 16-bit cache, kv heads a multiple of 8)
// with the cache copied straight from global memory into LDS (global_load_lds_dwordx4): no staging
// registers, no LDS store instructions, and a deeper queue of outstanding memory requests. A copy
// instruction moves 1 KiB of consecutive cache bytes (one position, four kv heads) to 1 KiB of
// consecutive LDS, so a stage is position major: [K | V][16 positions][8 kv heads][256 bytes]. The
// 16-byte chunks of a row are XOR-swizzled by the position (the lane picks which global chunk lands
// in its LDS slot), which keeps both read shapes conflict free exactly as in the kernel above.
// Two stages of 64 KiB; a step's copies are issued as soon as every wave has finished with the stage.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ void dma_1k(uint32_t lds_addr, uint32_t voff, const void *base)
{
    // the compiler sees neither the LDS write nor the memory counter: completion is awaited by dma_wait.
    // nt: the bytes are used once (see ld_stream)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\t"
                 :: "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait()
{
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// NKV: kv heads of a pass. 8, or all of a model's 4, 2 or 1: then 8 / NKV waves share a kv head, a step is
// 16 positions for each of them (wave w: kv head w % NKV, positions 16 (w / NKV) .. + 15 of the step), and
// their results meet in the head's first wave at the end of the segment.
// HD = 2: head_dim 256. A head is then two adjacent 256-byte units of a cache row, NKV counts units (8, 4 or 2: a
// model's 4 kv heads per pass, or all of its 2 or 1), and the stage layout and the copies are those of a head_dim-128
// model with twice the kv heads. The two waves of a head both form its scores over all 256 elements (K rows of both
// units; the kernel waits for memory, not for the matrix pipe) and each takes the 128 output columns of its own unit.
template <typename T, int NKV, int HD = 1>
__global__ void __launch_bounds__(kWaves * 64)
decode_dma_kernel(const DecodeMfmaParams p)
{
    constexpr int D = 128;                       // elements of a unit
    constexpr int DT = D * HD;                   // elements of a head
    constexpr int KS = DT / 32, MT = D / 16;
    constexpr int HEADB = D * 2;                 // bytes of one (position, kv head) row
    constexpr int NSUB = kWaves / NKV;           // 16-position groups of a step
    constexpr int POSB = NKV * HEADB;            // LDS bytes of one position: the kv heads of the pass
    constexpr int WSTEP = kStep * NSUB;          // positions of a step
    constexpr int KBYTES = WSTEP * POSB;         // 32 KiB: the K half of a stage
    constexpr int STAGE = 2 * KBYTES;
    constexpr int PER_WAVE = 8;                  // copies per wave and step
    constexpr int XS = D + 16;                   // floats of one head's (O, m, l) on its way to the head's first wave

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(smem + 2 * STAGE);
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t col = lane & 15;
    const uint32_t jq = lane >> 4;

    // read roles: this wave's kv head inside the pass and its group of 16 positions inside the step
    const uint32_t kvl = wave % NKV, sub = wave / NKV;   // (kvl: the wave's unit inside the pass)
    const uint32_t hsel = kvl / HD, hh = kvl % HD;       // its head inside the pass, and which unit of the head
    uint32_t kr_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        kr_off[ks] = (16 * sub + col) * POSB + (hsel * HD + ks / 4) * HEADB + (((4 * (ks % 4) + jq) ^ swizzle<D>(col)) << 4);
    }
    uint32_t vr_off[MT];
    {
        const uint32_t pos = 4 * jq + (col >> 2);
        const uint32_t q4 = lane & 3;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            vr_off[mt] = KBYTES + (16 * sub + pos) * POSB + kvl * HEADB + (((2 * mt + (q4 >> 1)) ^ swizzle<D>(pos)) << 4) + ((q4 & 1) << 3);
        }
    }
    // copy roles: wave w fills bytes 4096 w .. + 4095 of the K and of the V half of a stage with four copies each:
    // 8 kv heads: two positions, each as two copies of four kv heads; 4: four positions; 2: eight; 1: sixteen.
    // They are positions of the wave's own group. Lane = (256-byte row inside the KiB) * 16 + chunk slot; the slot
    // receives chunk slot ^ pattern(position). c_rel: the lane's position inside the group, c_voff: its offset
    // inside the position's cache row.
    uint32_t c_rel[4], c_voff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t byte = (4 * wave + i) * 1024 + 16 * lane;
        c_rel[i] = (byte / POSB) & 15u;
        c_voff[i] = ((byte % POSB) & ~255u) + (((lane & 15u) ^ swizzle<D>(c_rel[i])) << 4);
        if constexpr (NKV >= 4) {
            c_rel[i] = uni(c_rel[i]);   // a copy is one position
        }
    }

    const uint32_t g_valid = p.group < 16 ? p.group : 16;
    const uint32_t row_bytes = p.n_kv_heads * HD * HEADB;

    DecodeSplit<> split(p, tbl_lds + kSplitTblCap, lane, wave);
    split.scan();
    if (split.total == 0) {
        return;
    }

    // one segment: positions [t0, t1) of sequence `seq`
    auto run_segment = [&](uint32_t seq, uint32_t tok, uint32_t t0, uint32_t t1, bool whole, uint32_t pslot, bool first_piece,
                           int4 meta) {
        const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;
        const uint32_t n_steps = ceil_div(t1 - t0, static_cast<uint32_t>(WSTEP));
        const uint32_t blk0 = t0 / p.block_size;
        // the query rows of the first pass travel together with the block-table entries
        uint4 qreg[KS];
        auto load_q = [&](uint32_t kv0) {
            // (every lane loads: columns past the group's heads repeat its last head and are never stored; a load under
            // a per-lane condition is compiled into a branch with a wait of its own, one trip to memory per load)
            const uint16_t *qrow = p.q + static_cast<uint64_t>(tok) * p.q_row_stride +
                                   static_cast<uint64_t>((kv0 / HD + hsel) * p.group + min(col, g_valid - 1)) * DT;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                qreg[ks] = *reinterpret_cast<const uint4 *>(qrow + ks * 32 + jq * 8);
            }
        };
        load_q(0);
        {
            const uint32_t nblk = (t1 - 1) / p.block_size - blk0 + 1;
            for (uint32_t i = threadIdx.x; i < nblk; i += kWaves * 64) {
                tbl_lds[i] = static_cast<uint32_t>(table[blk0 + i]);
            }
            if (first_piece && threadIdx.x == 0) {
                reinterpret_cast<int4 *>(p.part_meta)[tok] = meta;
            }
            __syncthreads();
        }

        for (uint32_t kv0 = 0; kv0 < p.n_kv_heads * HD; kv0 += NKV) {   // (kv0 counts units)
            const uint32_t kvh = kv0 / HD + hsel;
            const uint32_t head0 = kvh * p.group;

            if (kv0 > 0) {
                load_q(kv0);
            }
            // complete these loads before any copy is issued: memory operations finish in order
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
            }
            f32x4_t O[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                O[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
            float m_run = -INFINITY, l_run = 0.f;

            // copies of one step into stage step % 2. The 16 positions of a group share one block
            // (block_size % 16 == 0, segments start at multiples of 16). Positions at or beyond the end re-read
            // the last valid one, a group beyond the end the last valid group.
            auto issue = [&](uint32_t step) {
                const uint32_t ts = t0 + step * WSTEP;
                const uint32_t gs = NSUB == 1 ? ts : min(ts + 16 * sub, (t1 - 1) & ~15u);
                uint32_t off;
                const uint32_t blk = block_of(p, gs, &off);
                const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk - blk0]);
                const uint64_t row0 = static_cast<uint64_t>(phys) * p.block_size + off;
                const uint32_t last_rel = min(t1 - 1 - gs, 15u);
                const uint32_t st = smem_addr + (step & 1) * STAGE + wave * 4096;
                const char *kb = static_cast<const char *>(p.k_cache) + row0 * row_bytes + kv0 * HEADB;
                const char *vb = static_cast<const char *>(p.v_cache) + row0 * row_bytes + kv0 * HEADB;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if constexpr (NKV >= 4) {
                        const uint32_t src = uni(min(c_rel[i], last_rel) * row_bytes);
                        dma_1k(st + i * 1024, c_voff[i], kb + src);
                        dma_1k(st + KBYTES + i * 1024, c_voff[i], vb + src);
                    } else {
                        const uint32_t voff = min(c_rel[i], last_rel) * POSB + c_voff[i];   // the cache row is the pass
                        dma_1k(st + i * 1024, voff, kb);
                        dma_1k(st + KBYTES + i * 1024, voff, vb);
                    }
                }
            };
            auto compute = [&](uint32_t step) {
                const uint32_t t = t0 + step * WSTEP + 16 * sub;
                const unsigned char *stage = smem + (step & 1) * STAGE;
                f32x4_t S = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    const uint4 a = *reinterpret_cast<const uint4 *>(stage + kr_off[ks]);
                    S = Mfma16<T>::run(a, qreg[ks], S);
                }
                s16x4_t vt[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
                    vt[mt] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(const_cast<unsigned char *>(stage) + vr_off[mt]));
                }
                float mx = -INFINITY;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float v = S[e] * kLog2e;
                    v = (t + 4 * jq + e) < t1 ? v : -INFINITY;
                    S[e] = v;
                    mx = fmaxf(mx, v);
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                const float m_new = fmaxf(m_run, mx);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                m_run = m_new;
                float pe[4];
                float psum = 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    pe[e] = fast_exp2(S[e] - m_safe);
                    psum += pe[e];
                }
                l_run = l_run * alpha + psum;
                const uint2 pb = make_uint2(T::pack(pe[0], pe[1]), T::pack(pe[2], pe[3]));
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        O[mt][0] *= alpha;
                        O[mt][1] *= alpha;
                        O[mt][2] *= alpha;
                        O[mt][3] *= alpha;
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    O[mt] = Mfma16<T>::run16(vt[mt], pb, O[mt]);
                }
            };

            // Two steps in flight. No copy is issued twice (the hint above sends a repeated one to memory
            // again: two of a segment's 66 steps), so the wait before the last step is for everything.
            const uint32_t last = n_steps - 1;
            issue(0);
            if (last >= 1) {
                issue(1);
            }
            for (uint32_t step = 0; step < n_steps; step++) {
                if (step < last) {
                    dma_wait<PER_WAVE>();   // this wave's share of `step` has landed: only the next step's is out
                } else {
                    dma_wait<0>();
                }
                __syncthreads();        // ... and everybody else's
                compute(step);
                __syncthreads();        // the stage is free again
                if (step + 2 <= last) {
                    issue(step + 2);
                }
            }

            float l_tot = l_run + __shfl_xor(l_run, 16);
            l_tot += __shfl_xor(l_tot, 32);
            if constexpr (NSUB > 1) {
                // the groups of a kv head meet in its first wave: (O, m, l) of the others through the stage memory,
                // which nobody reads any more (every wave has passed the loop's last barrier)
                float *xch = reinterpret_cast<float *>(smem);
                if (sub != 0) {
                    float *dst = xch + (wave * 16 + col) * XS;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0) {
                        dst[D] = m_run;
                        dst[D + 1] = l_tot;
                    }
                }
                __syncthreads();
                if (sub == 0) {
#pragma unroll
                    for (int s2 = 1; s2 < NSUB; s2++) {
                        const float *src = xch + ((s2 * NKV + kvl) * 16 + col) * XS;
                        const float m2 = src[D], l2 = src[D + 1];
                        const float m_new = fmaxf(m_run, m2);
                        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                        const float a1 = fast_exp2(m_run - m_safe), a2 = fast_exp2(m2 - m_safe);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++) {
                            const float4 o2 = *reinterpret_cast<const float4 *>(src + mt * 16 + jq * 4);
                            O[mt][0] = O[mt][0] * a1 + o2.x * a2;
                            O[mt][1] = O[mt][1] * a1 + o2.y * a2;
                            O[mt][2] = O[mt][2] * a1 + o2.z * a2;
                            O[mt][3] = O[mt][3] * a1 + o2.w * a2;
                        }
                        l_tot = l_tot * a1 + l2 * a2;
                        m_run = m_new;
                    }
                }
                __syncthreads();   // the next segment refills the stages
            }
            if (col < g_valid && sub == 0) {
                if (whole) {
                    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
                    uint16_t *dst = p.out + (static_cast<uint64_t>(tok) * p.n_heads + head0 + col) * DT + hh * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        uint2 o;
                        o.x = T::pack(O[mt][0] * inv, O[mt][1] * inv);
                        o.y = T::pack(O[mt][2] * inv, O[mt][3] * inv);
                        *reinterpret_cast<uint2 *>(dst + mt * 16 + jq * 4) = o;
                    }
                } else {
                    const uint64_t slot = static_cast<uint64_t>(pslot) * p.n_heads + head0 + col;
                    float *dst = p.part_acc + slot * DT + hh * D;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0 && hh == 0) {
                        *reinterpret_cast<float2 *>(p.part_ml + slot * 2) = make_float2(m_run, l_tot);
                    }
                }
            }
        }
    };

    split.for_each_segment(run_segment);
}

template <typename T, int NKV, int HD = 1>
int launch_dma_nkv(hipStream_t stream, const DecodeMfmaParams &p, uint32_t n_workgroups)
{
    const size_t lds = 2 * static_cast<size_t>(2 * kStep * kWaves * 128 * 2) +
                       (kSplitLdsWords + p.n_units + 1) * sizeof(uint32_t);
    auto kernel = decode_dma_kernel<T, NKV, HD>;
    if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) {
        return rc;
    }
    dim3 grid(n_workgroups, 1, 1);
    kernel<<<grid, kWaves * 64, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}
// head_dim 256: the units of a cache row are twice the kv heads
template <typename T>
int launch_dma256(hipStream_t stream, const DecodeMfmaParams &p, uint32_t n_workgroups)
{
    switch (p.n_kv_heads) {
    case 1: return launch_dma_nkv<T, 2, 2>(stream, p, n_workgroups);
    case 2: return launch_dma_nkv<T, 4, 2>(stream, p, n_workgroups);
    default: return launch_dma_nkv<T, 8, 2>(stream, p, n_workgroups);
    }
}
template <typename T>
int launch_dma(hipStream_t stream, const DecodeMfmaParams &p, uint32_t n_workgroups)
{
    switch (p.n_kv_heads) {
    case 1: return launch_dma_nkv<T, 1>(stream, p, n_workgroups);
    case 2: return launch_dma_nkv<T, 2>(stream, p, n_workgroups);
    case 4: return launch_dma_nkv<T, 4>(stream, p, n_workgroups);
    default: return launch_dma_nkv<T, 8>(stream, p, n_workgroups);
    }
}

// ---------------------------------------------------------------------------------------------------
// The direct-to-LDS kernel for 8-bit caches (head_dim 128, kv heads a multiple of 8). The cache bytes
// travel as they are: one copy instruction moves 1 KiB = one position of the pass's 8 kv heads, and the
// per-position scales follow by 4-byte copies. Bytes become fp16 (exactly) between the LDS read and the
// matrix product, so a wave reads half the LDS bytes of the 16-bit kernel and writes none.
// A step is 32 positions = two score tiles of 16. Stage: [K | V][32 positions][8 kv heads][128 bytes], then
// the scales in one 256-byte block per copying wave, [16-position half][pair of kv heads][K | V][head of the pair][16
// positions], so that a lane reads its eight scales of a tensor with two ds_read_b128. The 256-byte bank window of LDS holds two kv heads' rows of a
// position, so the XOR pattern of a position covers the 16-byte chunk (3 bits) and the kv head's low bit;
// it is chosen so that the 16 positions of a score tile (K rows as the A operand, ds_read_b128) and the
// 16 positions one half of the wave gathers for the second product (ds_read_b64_tr_b8) both land in 16
// different 16-byte slots.
//   K: lane (position = lane % 16, j = lane / 16) reads chunks j and j + 4 of its row; the 16 bytes of a
//      chunk feed two k steps, and the query registers hold the head's elements in that same order.
//   V: ds_read_b64_tr_b8 hands lane (column = lane % 16, j) the bytes of eight positions of one column:
//      rows 0-3 = positions 4j .. 4j+3 of the first tile, rows 4-7 = the same of the second, which is the
//      order in which the lane holds the probabilities after the first product (k = 32 positions).
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ void dma_4b(uint32_t lds_addr, const void *src)
{
    // no non-temporal hint: four waves take 8 bytes each of a position's 32 bytes of scales, and with the hint the
    // line comes from memory for each of them (counters: 1.019 x the algorithmic bytes instead of 1.005)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off\n\t"
                 :: "s"(lds_addr), "v"(src) : "memory", "m0");
}

// four cache bytes -> four fp16 values (two registers), exactly. fp8: the values themselves. int8: the values plus
// kInt8Bias: byte b ^ 0x80 = b + 128 as an unsigned byte u, and 0x6400 | u reads as 1024 + u in fp16. The constant does
// not have to be subtracted element by element (two packed subtractions per four values, a sixth of the kernel's
// vector instructions): a product over biased operands is the product wanted plus the constant times the sum of the
// other operand, which the caller takes off once - sum_d (k_d + c) q_d = sum_d k_d q_d + c sum_d q_d. Everything
// stays exact: 1024 + u and its products with an fp16 value fit fp32.
constexpr float kInt8Bias = 1152.0f;
template <int KVF>
__device__ __forceinline__ void widen4(uint32_t w, uint32_t *lo, uint32_t *hi)
{
    if constexpr (KVF == XLITE_HIP_KV_FP8) {
        *lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(static_cast<int>(w), 1.0f, false));
        *hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(static_cast<int>(w), 1.0f, true));
    } else {
        const uint32_t x = w ^ 0x80808080u;
        *lo = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
        *hi = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
    }
}

// NKV: kv heads of a pass. 8, or all of a model's 4 or 2: then 8 / NKV waves share a kv head, a step is 32 positions
// for each of them (wave w: kv head w % NKV, positions 32 (w / NKV) .. + 31 of the step), and their results meet in
// the head's first wave at the end of the segment.
template <typename T, int KVF, int NKV>
__global__ void __launch_bounds__(kWaves * 64)
decode_dma8_kernel(const DecodeMfmaParams p)
{
    constexpr int D = 128;
    constexpr int MT = D / 16;
    constexpr int STEP = 32;                     // positions per step and wave
    constexpr int NSUB = kWaves / NKV;           // 32-position groups of a step
    constexpr int WSTEP = STEP * NSUB;           // positions per step
    constexpr int HEADB = D;                     // bytes of one (position, kv head) row
    constexpr int POSB = NKV * HEADB;            // LDS bytes of one position: the kv heads of the pass
    constexpr int KBYTES = WSTEP * POSB;         // 32 KiB: the K half of a stage
    constexpr int SCALEB = kWaves * STEP * 4;    // 1 KiB: half of a stage's scale area (eight blocks of 256 bytes in all)
    constexpr int XS = D + 16;                   // floats of one head's (O, m, l) on its way to the head's first wave
    constexpr int STAGE = 2 * KBYTES + 2 * SCALEB;
    constexpr int PER_WAVE = 9;                  // copies per wave and step: 4 K rows, 4 V rows, 64 scales

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(smem + 2 * STAGE);
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t col = lane & 15;
    const uint32_t jq = lane >> 4;

    // XOR pattern of position `pos` of a wave's 32: chunk bits, kv-head bit
    auto pat_chunk = [](uint32_t pos) { return pos & 7u; };
    auto pat_head = [](uint32_t pos) { return ((pos >> 3) ^ (pos >> 4)) & 1u; };
    auto slot_off = [&](uint32_t pos, uint32_t head, uint32_t chunk) {   // pos: inside the whole step
        return pos * POSB + head / 2 * 256 + ((((head & 1u) ^ pat_head(pos & 31u)) << 3 | (chunk ^ pat_chunk(pos & 31u))) << 4);
    };
    // read roles: this wave's kv head inside the pass and its group of 32 positions inside the step
    const uint32_t kvl = wave % NKV, sub = wave / NKV;
    uint32_t kr_off[2][2];
#pragma unroll
    for (int tl = 0; tl < 2; tl++) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            kr_off[tl][r] = slot_off(STEP * sub + 16 * tl + col, kvl, jq + 4 * r);
        }
    }
    uint32_t vr_off[MT];
    {
        const uint32_t row = col >> 1;   // row of the 8 x 16 byte block this lane points at
        const uint32_t pos = row < 4 ? 4 * jq + row : 16 + 4 * jq + (row - 4);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            vr_off[mt] = KBYTES + slot_off(STEP * sub + pos, kvl, mt) + ((lane & 1) << 3);
        }
    }
    // scales of this wave's kv head: block (group, half, head pair) of the scale area, then [K | V][head of the pair][16]
    const uint32_t sc_off = 2 * KBYTES + (sub * NKV + kvl / 2) * 256 + (kvl & 1u) * 64 + 4 * jq * 4;   // K, first tile
    constexpr uint32_t kScHalf = (NKV / 2) * 256;   // the second tile's block
    // copy roles: wave w fills bytes 4096 w .. + 4095 of the K and of the V half of a stage with four copies each:
    // 8 kv heads: four positions; 4: eight; 2: sixteen. They are positions of one 16-position half of the wave's own
    // group. Lane = slot (position inside the KiB, kv head, chunk); the slot receives the (kv head, chunk) the
    // position's pattern assigns to it. c_rel: the lane's position inside the half, c_voff: its offset inside the
    // position's cache row.
    const uint32_t row_bytes = p.n_kv_heads * HEADB;
    uint32_t c_rel[4], c_voff[4], c_full[4];   // c_full: the lane's offset from the half's first row when no row is clamped
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t byte = (4 * wave + i) * 1024 + 16 * lane;
        const uint32_t pos = (byte / POSB) & 31u, in_pos = byte % POSB;
        c_rel[i] = pos & 15u;
        c_voff[i] = (in_pos / 256 * 2 + (((in_pos >> 7) & 1u) ^ pat_head(pos))) * HEADB + (((lane & 7u) ^ pat_chunk(pos)) << 4);
        c_full[i] = c_rel[i] * row_bytes + c_voff[i];
    }
    const uint32_t c_half = ((4 * wave * 1024 / POSB) >> 4) & 1u;   // the half of the group this wave's copies lie in
    // scale copies: every wave moves the scales it can address with the block lookup of its own half: those of the
    // half's 16 positions for two kv heads of its group, K and V. Lane = (tensor, head of the pair, position); the 256
    // bytes land in the wave's own block of the scale area, [tensor][head of the pair][16 positions].
    const uint32_t sc_pair = (wave % NKV) % (NKV / 2);           // which two kv heads of the group
    const uint32_t sc_head = 2 * sc_pair + ((lane >> 4) & 1u);
    const uint32_t sc_pos = lane & 15;
    const float *sc_src = (lane >> 5) ? p.v_scale : p.k_scale;
    const uint32_t sc_dst = 2 * KBYTES + wave * 256;

    const uint32_t g_valid = p.group < 16 ? p.group : 16;

    DecodeSplit<> split(p, tbl_lds + kSplitTblCap, lane, wave);
    split.scan();
    if (split.total == 0) {
        return;
    }

    auto run_segment = [&](uint32_t seq, uint32_t tok, uint32_t t0, uint32_t t1, bool whole, uint32_t pslot, bool first_piece,
                           int4 meta) {
        const int32_t *table = p.block_tables + static_cast<uint64_t>(seq) * p.max_num_block;
        const uint32_t n_steps = ceil_div(t1 - t0, static_cast<uint32_t>(WSTEP));
        const uint32_t blk0 = t0 / p.block_size;
        // Q^T as the B operand, as fp16: k step 2r + h of the first product covers the elements
        // [16 (j + 4r) + 8h, + 8) of the head
        uint4 qreg[4];
        auto load_q = [&](uint32_t kv0) {
            // (every lane loads: columns past the group's heads repeat its last head and are never stored)
            const uint16_t *qrow = p.q + static_cast<uint64_t>(tok) * p.q_row_stride +
                                   static_cast<uint64_t>((kv0 + kvl) * p.group + min(col, g_valid - 1)) * D;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                qreg[ks] = *reinterpret_cast<const uint4 *>(qrow + 16 * (jq + 4 * (ks >> 1)) + 8 * (ks & 1));
            }
        };
        auto q_to_fp16 = [&]() {
            if constexpr (!std::is_same<T, FP16>::value) {
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    uint32_t *w = reinterpret_cast<uint32_t *>(&qreg[ks]);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        w[j] = FP16::pack(T::to_f32(static_cast<uint16_t>(w[j] & 0xffff)), T::to_f32(static_cast<uint16_t>(w[j] >> 16)));
                    }
                }
            }
        };
        load_q(0);
        {
            const uint32_t nblk = (t1 - 1) / p.block_size - blk0 + 1;
            for (uint32_t i = threadIdx.x; i < nblk; i += kWaves * 64) {
                tbl_lds[i] = static_cast<uint32_t>(table[blk0 + i]);
            }
            if (first_piece && threadIdx.x == 0) {
                reinterpret_cast<int4 *>(p.part_meta)[tok] = meta;
            }
            __syncthreads();
        }

        for (uint32_t kv0 = 0; kv0 < p.n_kv_heads; kv0 += NKV) {
            const uint32_t kvh = kv0 + kvl;
            const uint32_t head0 = kvh * p.group;

            if (kv0 > 0) {
                load_q(kv0);
            }
            // complete these loads before any copy is issued: memory operations finish in order
            q_to_fp16();
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
            }
            f32x4_t O[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                O[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
            float m_run = -INFINITY, l_run = 0.f;
            // int8: what the bias of the K operand adds to every score of head `col` (the score accumulators start from
            // its negative), and the running sum of the probabilities as the second product sees them, for the bias
            // of the V operand
            float s_init = 0.f, pv_run = 0.f;
            if constexpr (KVF == XLITE_HIP_KV_INT8) {
                float qs = 0.f;
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    qs = FP16::dot2(qreg[ks].x, 0x3c003c00u, qs);
                    qs = FP16::dot2(qreg[ks].y, 0x3c003c00u, qs);
                    qs = FP16::dot2(qreg[ks].z, 0x3c003c00u, qs);
                    qs = FP16::dot2(qreg[ks].w, 0x3c003c00u, qs);
                }
                qs += __shfl_xor(qs, 16);
                qs += __shfl_xor(qs, 32);
                s_init = -kInt8Bias * qs;
            }

            // copies of one step into stage step % 2. Each half of a step (16 positions from a multiple of 16)
            // lies in one block (block_size % 16 == 0). Positions at or beyond the end re-read the last valid one.
            auto issue = [&](uint32_t step) {
                const uint32_t ts = t0 + step * WSTEP + STEP * sub;   // this wave's group; beyond the end: see below
                const uint32_t tl = t1 - 1;
                const uint32_t st = smem_addr + (step & 1) * STAGE;
                // one block lookup: everything this wave copies lies in its half of its group
                const uint32_t hs0 = ts + 16 * c_half;
                const uint32_t hs = min(hs0, tl);
                uint32_t off;
                const uint32_t blk = block_of(p, hs, &off);
                const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk - blk0]);
                const uint64_t my_row0 = static_cast<uint64_t>(phys) * p.block_size + off;
                const uint32_t my_max = hs0 > tl ? 0u : min(tl - hs0, 15u);
                const char *kb = static_cast<const char *>(p.k_cache) + my_row0 * row_bytes + kv0 * HEADB;
                const char *vb = static_cast<const char *>(p.v_cache) + my_row0 * row_bytes + kv0 * HEADB;
                if (my_max == 15) {
                    // every row of the half exists: the rows' offsets are part of the lanes' precomputed ones
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        dma_1k(st + (4 * wave + i) * 1024, c_full[i], kb);
                        dma_1k(st + KBYTES + (4 * wave + i) * 1024, c_full[i], vb);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t voff = min(c_rel[i], my_max) * row_bytes + c_voff[i];
                        dma_1k(st + (4 * wave + i) * 1024, voff, kb);
                        dma_1k(st + KBYTES + (4 * wave + i) * 1024, voff, vb);
                    }
                }
                dma_4b(st + sc_dst, sc_src + (my_row0 + min(sc_pos, my_max)) * p.n_kv_heads + kv0 + sc_head);
            };
            auto compute = [&](uint32_t step) {
                const uint32_t t = t0 + step * WSTEP + STEP * sub;
                const unsigned char *stage = smem + (step & 1) * STAGE;
                // ---- S^T = K . Q^T: two tiles of 16 positions x 16 heads ------------------------------------
                f32x4_t S[2];
#pragma unroll
                for (int tl = 0; tl < 2; tl++) {
                    S[tl] = f32x4_t{s_init, s_init, s_init, s_init};
#pragma unroll
                    for (int r = 0; r < 2; r++) {
                        const uint4 raw = *reinterpret_cast<const uint4 *>(stage + kr_off[tl][r]);
                        uint4 a0, a1;
                        widen4<KVF>(raw.x, &a0.x, &a0.y);
                        widen4<KVF>(raw.y, &a0.z, &a0.w);
                        widen4<KVF>(raw.z, &a1.x, &a1.y);
                        widen4<KVF>(raw.w, &a1.z, &a1.w);
                        S[tl] = Mfma16<FP16>::run(a0, qreg[2 * r], S[tl]);
                        S[tl] = Mfma16<FP16>::run(a1, qreg[2 * r + 1], S[tl]);
                    }
                }
                // V^T bytes do not depend on the softmax: fetch them now
                typedef int v2i_t __attribute__((ext_vector_type(2)));
                v2i_t vraw[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    typedef v2i_t __attribute__((address_space(3))) * lds_tr_ptr;
                    vraw[mt] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_tr_ptr)(const_cast<unsigned char *>(stage) + vr_off[mt]));
                }
                float ksc[8], vsc[8];
                {
                    const float4 k0 = *reinterpret_cast<const float4 *>(stage + sc_off);
                    const float4 k1 = *reinterpret_cast<const float4 *>(stage + sc_off + kScHalf);
                    const float4 v0 = *reinterpret_cast<const float4 *>(stage + sc_off + 128);
                    const float4 v1 = *reinterpret_cast<const float4 *>(stage + sc_off + kScHalf + 128);
                    ksc[0] = k0.x, ksc[1] = k0.y, ksc[2] = k0.z, ksc[3] = k0.w;
                    ksc[4] = k1.x, ksc[5] = k1.y, ksc[6] = k1.z, ksc[7] = k1.w;
                    vsc[0] = v0.x, vsc[1] = v0.y, vsc[2] = v0.z, vsc[3] = v0.w;
                    vsc[4] = v1.x, vsc[5] = v1.y, vsc[6] = v1.z, vsc[7] = v1.w;
                }
                // ---- online softmax; lane holds positions t + 16 tl + 4 jq + e of head `col` ------------------
                float sv[8];
                bool ok[8];
                float mx = -INFINITY;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    ok[i] = (t + 16 * (i >> 2) + 4 * jq + (i & 3)) < t1;
                    const float v = ok[i] ? S[i >> 2][i & 3] * kLog2e * ksc[i] : -INFINITY;   // also drops the padding's NaN
                    sv[i] = v;
                    mx = fmaxf(mx, v);
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                const float m_new = fmaxf(m_run, mx);
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                m_run = m_new;
                float pe[8];
                float psum = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float x = fast_exp2(sv[i] - m_safe);
                    psum += x;
                    pe[i] = ok[i] ? x * vsc[i] : 0.f;
                }
                l_run = l_run * alpha + psum;
                const uint4 pb = make_uint4(FP16::pack(pe[0], pe[1]), FP16::pack(pe[2], pe[3]),
                                            FP16::pack(pe[4], pe[5]), FP16::pack(pe[6], pe[7]));
                if constexpr (KVF == XLITE_HIP_KV_INT8) {
                    float ps = FP16::dot2(pb.x, 0x3c003c00u, 0.f);
                    ps = FP16::dot2(pb.y, 0x3c003c00u, ps);
                    ps = FP16::dot2(pb.z, 0x3c003c00u, ps);
                    ps = FP16::dot2(pb.w, 0x3c003c00u, ps);
                    pv_run = pv_run * alpha + ps;
                }
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        O[mt][0] *= alpha;
                        O[mt][1] *= alpha;
                        O[mt][2] *= alpha;
                        O[mt][3] *= alpha;
                    }
                }
                // ---- O^T += V^T . P^T (k = the 32 positions) -------------------------------------------------
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    uint4 a;
                    widen4<KVF>(static_cast<uint32_t>(vraw[mt].x), &a.x, &a.y);
                    widen4<KVF>(static_cast<uint32_t>(vraw[mt].y), &a.z, &a.w);
                    O[mt] = Mfma16<FP16>::run(a, pb, O[mt]);
                }
            };

            // Two steps in flight. No copy is issued twice (the hint above sends a repeated one to memory
            // again: two of a segment's 66 steps), so the wait before the last step is for everything.
            const uint32_t last = n_steps - 1;
            issue(0);
            if (last >= 1) {
                issue(1);
            }
            for (uint32_t step = 0; step < n_steps; step++) {
                if (step < last) {
                    dma_wait<PER_WAVE>();   // this wave's share of `step` has landed: only the next step's is out
                } else {
                    dma_wait<0>();
                }
                __syncthreads();        // ... and everybody else's
                compute(step);
                __syncthreads();        // the stage is free again
                if (step + 2 <= last) {
                    issue(step + 2);
                }
            }

            float l_tot = l_run + __shfl_xor(l_run, 16);
            l_tot += __shfl_xor(l_tot, 32);
            if constexpr (KVF == XLITE_HIP_KV_INT8) {
                // O^T of head `col` carries the bias of V times the probabilities summed over every position
                float pv_tot = pv_run + __shfl_xor(pv_run, 16);
                pv_tot += __shfl_xor(pv_tot, 32);
                const float corr = kInt8Bias * pv_tot;
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    O[mt][0] -= corr;
                    O[mt][1] -= corr;
                    O[mt][2] -= corr;
                    O[mt][3] -= corr;
                }
            }
            if constexpr (NSUB > 1) {
                // the groups of a kv head meet in its first wave: (O, m, l) of the others through the stage memory,
                // which nobody reads any more (every wave has passed the loop's last barrier)
                float *xch = reinterpret_cast<float *>(smem);
                if (sub != 0) {
                    float *dst = xch + (wave * 16 + col) * XS;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        *reinterpret_cast<float4 *>(dst + mt * 16 + jq * 4) = make_float4(O[mt][0], O[mt][1], O[mt][2], O[mt][3]);
                    }
                    if (jq == 0) {
                        dst[D] = m_run;
                        dst[D + 1] = l_tot;
                    }
                }
                __syncthreads();
                if (sub == 0) {
#pragma unroll
                    for (int s2 = 1; s2 < NSUB; s2++) {
                        const float *src = xch + ((s2 * NKV + kvl) * 16 + col) * XS;
                        const float m2 = src[D], l2 = src[D + 1];
                        const float m_new = fmaxf(m_run, m2);
                        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                        const float a1 = fast_exp2(m_run - m_safe), a2 = fast_exp2(m2 - m_safe);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++) {
                            const float4 o2 = *reinterpret_cast<const float4 *>(src + mt * 16 + jq * 4);
                            O[mt][0] = O[mt][0] * a1 + o2.x * a2;
                            O[mt][1] = O[mt][1] * a1 + o2.y * a2;
                            O[mt][2] = O[mt][2] * a1 + o2.z * a2;
                            O[mt][3] = O[mt][3] * a1 + o2.w * a2;
                        }
                        l_tot = l_tot * a1 + l2 * a2;
                        m_run = m_new;
                    }
                }
                __syncthreads();   // the next segment refills the stages
            }
            if (col < g_valid && sub == 0) {
                if (whole) {
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
                    const uint64_t slot = static_cast<uint64_t>(pslot) * p.n_heads + head0 + col;
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
    };

    split.for_each_segment(run_segment);
}

template <typename T, int KVF, int NKV>
int launch_dma8_nkv(hipStream_t stream, const DecodeMfmaParams &p, uint32_t n_workgroups)
{
    const size_t lds = 2 * static_cast<size_t>(2 * 32 * kWaves * 128 + 2 * kWaves * 32 * 4) +
                       (kSplitLdsWords + p.n_units + 1) * sizeof(uint32_t);
    auto kernel = decode_dma8_kernel<T, KVF, NKV>;
    if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) {
        return rc;
    }
    dim3 grid(n_workgroups, 1, 1);
    kernel<<<grid, kWaves * 64, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}
template <typename T, int KVF>
int launch_dma8(hipStream_t stream, const DecodeMfmaParams &p, uint32_t n_workgroups)
{
    switch (p.n_kv_heads) {
    case 2: return launch_dma8_nkv<T, KVF, 2>(stream, p, n_workgroups);
    case 4: return launch_dma8_nkv<T, KVF, 4>(stream, p, n_workgroups);
    default: return launch_dma8_nkv<T, KVF, 8>(stream, p, n_workgroups);
    }
}

template <typename T, int D, int KVF, bool MULTI_SUB, bool WHOLE = false, bool ROPE = false>
int launch_inst(hipStream_t stream, const DecodeMfmaParams &p, uint32_t grid_x)
{
    constexpr bool KV8 = KVF != XLITE_HIP_KV_SAME;
    const size_t lds = 2 * static_cast<size_t>(kWaves) * 2 * kStep * D * 2 + (KV8 ? 2 * 2 * kWaves * kStep * 4 : 0) +
                       (kSplitLdsWords + p.n_units + 1) * sizeof(uint32_t);
    auto kernel = decode_mfma_kernel<T, D, KVF, MULTI_SUB, WHOLE, ROPE>;
    if (lds > 64 * 1024) {
        if (const int rc = ensure_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) {
            return rc;
        }
    }
    dim3 grid(grid_x, WHOLE ? ceil_div(p.n_kv_heads, p.kv_per_wg) : 1u, 1);
    kernel<<<grid, kWaves * 64, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

template <typename T, int D, int KVF>
int launch_one(hipStream_t stream, const DecodeMfmaParams &p, uint32_t grid_x)
{
    return p.n_sub > 1 ? launch_inst<T, D, KVF, true>(stream, p, grid_x)
                       : launch_inst<T, D, KVF, false>(stream, p, grid_x);
}

// the whole-row instantiations (16-bit caches)
template <typename T, int D>
int launch_whole(hipStream_t stream, const DecodeMfmaParams &p, uint32_t grid_x)
{
    return p.n_sub > 1 ? launch_inst<T, D, XLITE_HIP_KV_SAME, true, true>(stream, p, grid_x)
                       : launch_inst<T, D, XLITE_HIP_KV_SAME, false, true>(stream, p, grid_x);
}

// ... that rotate and store the rows themselves
template <typename T, int D>
int launch_whole_rope(hipStream_t stream, const DecodeMfmaParams &p, uint32_t grid_x)
{
    return p.n_sub > 1 ? launch_inst<T, D, XLITE_HIP_KV_SAME, true, true, true>(stream, p, grid_x)
                       : launch_inst<T, D, XLITE_HIP_KV_SAME, false, true, true>(stream, p, grid_x);
}

template <typename T, int D>
int launch_fmt(hipStream_t stream, const DecodeMfmaParams &p, uint32_t grid_x, int kv_dtype)
{
    switch (kv_dtype) {
    case XLITE_HIP_KV_INT8:
        return launch_one<T, D, XLITE_HIP_KV_INT8>(stream, p, grid_x);
    case XLITE_HIP_KV_FP8:
        return launch_one<T, D, XLITE_HIP_KV_FP8>(stream, p, grid_x);
    default:
        return launch_one<T, D, XLITE_HIP_KV_SAME>(stream, p, grid_x);
    }
}

}  // namespace

// head_dim 256 over a 16-bit cache: the direct-to-LDS kernel with two units per head (4 kv heads per pass, or a
// model's 2 or 1)
bool decode_dma256_supported(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size, int kv_dtype)
{
    return head_dim == 256 && kv_dtype == XLITE_HIP_KV_SAME && block_size % kStep == 0 && n_kv_heads > 0 &&
           n_heads / n_kv_heads <= 16 && (n_kv_heads % 4 == 0 || n_kv_heads == 2 || n_kv_heads == 1);
}

bool decode_mfma_supported(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t block_size,
                           uint32_t total_tokens)
{
    const uint32_t group = n_heads / n_kv_heads;
    // (any number of rows: the work split keeps the prefix sums of up to kSplitSeqCap rows in LDS, larger batches
    // run as several launches)
    (void)n_kv_heads;
    (void)total_tokens;
    return (head_dim == 64 || head_dim == 128) && block_size % kStep == 0 && group <= 16;
}

uint32_t decode_mfma_slice_units() { return kSplitSeqCap; }

// decode_dma_kernel: head_dim 128, 16-bit cache, kv heads a multiple of 8, or 4, 2 or 1 of them
bool decode_dma_supported(uint32_t n_kv_heads, uint32_t head_dim, int kv_dtype)
{
    return head_dim == 128 && kv_dtype == XLITE_HIP_KV_SAME &&
           (n_kv_heads % kWaves == 0 || n_kv_heads == 4 || n_kv_heads == 2 || n_kv_heads == 1);
}

// decode_dma8_kernel: head_dim 128, 8-bit cache, kv heads a multiple of 8, or 4 or 2 of them
bool decode_dma8_supported(uint32_t n_kv_heads, uint32_t head_dim, int kv_dtype)
{
    return head_dim == 128 && kv_dtype != XLITE_HIP_KV_SAME &&
           (n_kv_heads % kWaves == 0 || n_kv_heads == 4 || n_kv_heads == 2);
}

// The chunk the kernel really uses is the batch's total step count over the number of workgroups, which the
// host cannot know (the lengths live in device memory); it is never below kSplitMinChunk steps nor above what
// the block-table staging holds, which bounds the number of chunks and hence of partial slots (two per chunk).
void decode_split_plan(uint32_t batch, uint32_t n_heads, uint32_t head_dim, uint32_t block_size, uint32_t max_num_block,
                       DecodeSplitPlan *pl)
{
    const uint64_t max_steps = ceil_div(max_num_block * block_size, static_cast<uint32_t>(kStep));
    // (the kernels round the cap down to a multiple of the steps they take at a time, at most 16: the bound uses 16)
    const uint64_t chunk_cap = static_cast<uint64_t>(kSplitTblCap - 2) * block_size / kStep / 16 * 16;
    const uint64_t by_cap = (static_cast<uint64_t>(batch) * max_steps + chunk_cap - 1) / chunk_cap;
    pl->max_chunks = static_cast<uint32_t>(by_cap > kSplitMaxWorkgroups ? by_cap : kSplitMaxWorkgroups);
    pl->meta_bytes = ((static_cast<size_t>(batch) * sizeof(int4) + 255) / 256) * 256;
    pl->ml_bytes = static_cast<size_t>(2) * pl->max_chunks * n_heads * 2 * sizeof(float);
    pl->acc_bytes = static_cast<size_t>(2) * pl->max_chunks * n_heads * head_dim * sizeof(float);
}

size_t decode_mfma_workspace_bytes(uint32_t batch, uint32_t n_heads, uint32_t head_dim, uint32_t block_size,
                                   uint32_t max_num_block)
{
    DecodeSplitPlan pl{};
    decode_split_plan(batch, n_heads, head_dim, block_size, max_num_block, &pl);
    return pl.meta_bytes + pl.ml_bytes + pl.acc_bytes;
}

// Contexts that are short by the width of the block tables (at most 16 steps per wave: the waves of a kv head
// share a row when there are fewer than 8 kv heads): no split, one workgroup per row, no merge launch. Such a
// step is bound by its launches: Qwen2-0.5B, 4 sequences of up to 512 positions, 12.7 us + 3.9 us of merge -> one
// kernel.
bool decode_mfma_whole_rows(const AttentionArgs &a)
{
    const uint32_t waves_per_kv = a.n_kv_heads >= kWaves ? 1u : kWaves / a.n_kv_heads;
    return a.rows_mode != kOnlySingle && a.kv_dtype == XLITE_HIP_KV_SAME && a.head_dim != 256 &&
           ceil_div(static_cast<uint64_t>(a.max_num_block) * a.block_size, static_cast<uint64_t>(kStep)) <= 16ull * waves_per_kv &&
           a.max_num_block <= kSplitTblCap - 2;
}

int launch_decode_mfma(hipStream_t stream, const AttentionArgs &a, const RopeArgs *rope)
{
    const bool bf = a.dtype == XLITE_HIP_BF16;
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
    p.q_row_stride = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim;
    p.n_heads = a.n_heads;
    p.n_kv_heads = a.n_kv_heads;
    p.group = a.n_heads / a.n_kv_heads;
    p.block_size = a.block_size;
    p.max_num_block = a.max_num_block;
    p.batch = a.batch;
    p.total_rows = a.total_tokens;
    p.only_single = a.rows_mode == kOnlySingle ? 1u : 0u;
    DecodeSplitPlan pl{};
    decode_split_plan(a.total_tokens, a.n_heads, a.head_dim, a.block_size, a.max_num_block, &pl);
    const size_t need = pl.meta_bytes + pl.ml_bytes + pl.acc_bytes;
    if (a.workspace == nullptr || a.workspace_bytes < need) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    thread_local int cu_dev = -1, n_cu = 0;   // the compute-unit count of the device this thread last used
    int dev = 0;
    XL_HIP(hipGetDevice(&dev));
    if (dev != cu_dev) {
        XL_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
        cu_dev = dev;
    }
    const uint32_t grid_x = min(static_cast<uint32_t>(n_cu), kSplitMaxWorkgroups);
    char *ws = static_cast<char *>(a.workspace);
    p.part_meta = reinterpret_cast<int32_t *>(ws);
    p.part_ml = reinterpret_cast<float *>(ws + pl.meta_bytes);
    p.part_acc = reinterpret_cast<float *>(ws + pl.meta_bytes + pl.ml_bytes);
    p.n_sub = a.n_kv_heads >= kWaves ? 1 : kWaves / a.n_kv_heads;

    // slices of at most kSplitSeqCap units, each with its own merge: the partial slots are reused from slice to
    // slice. (Sequences' rows lie anywhere among the batch's rows, so a batch served by two kernels is one slice.)
    const uint32_t units = p.only_single ? a.batch : a.total_tokens;
    XL_REQUIRE(!p.only_single || units <= kSplitSeqCap, "too many sequences for a batch served by two kernels");
    const bool whole_rows = decode_mfma_whole_rows(a);
    if (whole_rows) {
        // Rows that would leave compute units idle: a workgroup takes a group of 1, 2 or 4 of a row's kv heads instead
        // of all of them (the finest cut whose workgroups still run all at once: a second round of workgroups costs
        // more than it brings), its waves sharing each head's range - heads are independent, so this still needs no
        // merge. With nothing in the caches one compute unit takes in about 50 GB/s: Qwen2-0.5B, 4 rows of up to 512
        // positions, 248 KB each, 15.1 -> 13.0 us; Llama-3-8B, 64 rows of 256 positions, 1 MB each, 34.6 -> 27.6 us.
        const uint32_t rows = rope != nullptr ? a.batch : a.total_tokens;
        p.kv_per_wg = a.n_kv_heads;
        for (uint32_t c = 1; c < a.n_kv_heads && c < kWaves; c *= 2) {
            if (static_cast<uint64_t>(rows) * ceil_div(a.n_kv_heads, c) <= grid_x) {
                p.kv_per_wg = c;
                p.n_sub = kWaves / c;
                break;
            }
        }
    }
    if (rope != nullptr) {
        // one launch for the layer's rope_and_cache and attention: by sequence, whatever the batch size
        XL_REQUIRE(whole_rows && rope->num_tokens == a.total_tokens && rope->n_heads == a.n_heads &&
                       rope->n_kv_heads == a.n_kv_heads && rope->head_dim == a.head_dim && rope->k_cache != nullptr,
                   "the decode kernel rotates rows only for batches it takes whole");
        p.rope = *rope;
        p.unit0 = 0;
        p.n_units = 1;   // (sizes the prefix sums in LDS, which this mode does not keep)
        p.step_mult = 1;
        p.block_magic = static_cast<uint64_t>(a.max_num_block) * a.block_size * a.block_size < (1ull << 32)
                            ? static_cast<uint32_t>((1ull << 32) / a.block_size) + 1
                            : 0u;
        const uint32_t gx = min(grid_x, a.batch);
        return a.head_dim == 128 ? (bf ? launch_whole_rope<BF16, 128>(stream, p, gx) : launch_whole_rope<FP16, 128>(stream, p, gx))
                                 : (bf ? launch_whole_rope<BF16, 64>(stream, p, gx) : launch_whole_rope<FP16, 64>(stream, p, gx));
    }
    for (uint32_t u0 = 0; u0 < units; u0 += kSplitSeqCap) {
        p.unit0 = u0;
        p.n_units = min(kSplitSeqCap, units - u0);
        int rc;
        p.step_mult = 1;
        p.block_magic = static_cast<uint64_t>(a.max_num_block) * a.block_size * a.block_size < (1ull << 32)
                            ? static_cast<uint32_t>((1ull << 32) / a.block_size) + 1
                            : 0u;
        const uint32_t gx = whole_rows ? min(grid_x, p.n_units) : grid_x;   // (whole rows: no workgroups without a row)
        if (whole_rows) {   // (the register-staged kernel, whatever the shape: these contexts are a few steps long)
            rc = a.head_dim == 128 ? (bf ? launch_whole<BF16, 128>(stream, p, gx) : launch_whole<FP16, 128>(stream, p, gx))
                                   : (bf ? launch_whole<BF16, 64>(stream, p, gx) : launch_whole<FP16, 64>(stream, p, gx));
        } else if (a.head_dim == 256) {
            XL_REQUIRE(decode_dma256_supported(a.n_heads, a.n_kv_heads, a.head_dim, a.block_size, a.kv_dtype),
                       "head_dim 256: shape not served by the streaming decode kernel");
            p.step_mult = 2 * a.n_kv_heads < kWaves ? kWaves / (2 * a.n_kv_heads) : 1;
            rc = bf ? launch_dma256<BF16>(stream, p, gx) : launch_dma256<FP16>(stream, p, gx);
        } else if (decode_dma_supported(a.n_kv_heads, a.head_dim, a.kv_dtype)) {
            p.step_mult = a.n_kv_heads < kWaves ? kWaves / a.n_kv_heads : 1;
            rc = bf ? launch_dma<BF16>(stream, p, gx) : launch_dma<FP16>(stream, p, gx);
        } else if (decode_dma8_supported(a.n_kv_heads, a.head_dim, a.kv_dtype)) {
            p.step_mult = 2 * (a.n_kv_heads < kWaves ? kWaves / a.n_kv_heads : 1);   // a wave takes 32 positions at a time
            if (a.kv_dtype == XLITE_HIP_KV_FP8) {
                rc = bf ? launch_dma8<BF16, XLITE_HIP_KV_FP8>(stream, p, gx) : launch_dma8<FP16, XLITE_HIP_KV_FP8>(stream, p, gx);
            } else {
                rc = bf ? launch_dma8<BF16, XLITE_HIP_KV_INT8>(stream, p, gx) : launch_dma8<FP16, XLITE_HIP_KV_INT8>(stream, p, gx);
            }
        } else if (a.head_dim == 128) {
            rc = bf ? launch_fmt<BF16, 128>(stream, p, gx, a.kv_dtype) : launch_fmt<FP16, 128>(stream, p, gx, a.kv_dtype);
        } else {
            rc = bf ? launch_fmt<BF16, 64>(stream, p, gx, a.kv_dtype) : launch_fmt<FP16, 64>(stream, p, gx, a.kv_dtype);
        }
        if (rc != XLITE_HIP_OK) {
            return rc;
        }
        if (whole_rows) {
            continue;   // every row was stored directly
        }
        if (!p.only_single) {
            // the slice's rows are u0 .. u0 + n_units - 1
            rc = launch_merge_meta(stream, a.dtype, static_cast<uint16_t *>(a.output) + static_cast<size_t>(u0) * a.n_heads * a.head_dim,
                                   p.part_acc, p.part_ml, p.part_meta + static_cast<size_t>(u0) * 4, p.n_units, a.n_heads, a.head_dim);
        } else {
            rc = launch_merge_meta(stream, a.dtype, a.output, p.part_acc, p.part_ml, p.part_meta, a.total_tokens, a.n_heads, a.head_dim);
        }
        if (rc != XLITE_HIP_OK) {
            return rc;
        }
    }
    return XLITE_HIP_OK;
}

}  // namespace xlite
