// DeepSeek-style absorbed MLA decode on the matrix cores, split along the KV axis.
//
// One latent "kv head" is shared by all query heads. A workgroup of eight wavefronts (two per SIMD, 256 registers
// each, all of them ordinary vector registers) covers up to 128 heads; a row's positions are walked in steps of 32:
//   S^T[pos][head]  = [kc | pe][pos][:] . [q_absorb | qr][head][:]   2 x 18 v_mfma_f32_16x16x32_bf16
//   O^T[c][head]   += kc^T[c][pos] . P^T[pos][head]                   16 x v_mfma_f32_32x32x16_bf16
// The two products split the work differently. Scores by heads: wave w owns heads 16 w .. 16 w + 15 (Q in 72
// registers per lane, the online softmax state of its heads). The second product by latent columns: wave w owns
// columns 64 w .. 64 w + 63 of O^T for ALL heads (128 accumulators per lane): it reads only its own eighth of the
// transposed latent from LDS, once for the 128 heads, and takes the probabilities of the other waves' heads from
// LDS, where every wave leaves the 1 KiB of its heads after the softmax (with the factor by which the reference
// maximum moved). Per step that is 16 + 16 LDS operand reads and products of 32 x 32 heads instead of 64 reads and
// 32 products per wave. The probabilities of step i are consumed one step later (behind the barrier of step i + 1,
// which the copies need anyway), so there is still one barrier per step.
// The cache never passes through registers: every wave copies its share of a step straight from global memory
// into LDS (global_load_lds_dwordx4, 1 KiB of consecutive cache bytes per instruction) into a ring of three 36 KiB
// stages (the step whose scores are being formed, the one before it whose second product is running, the one after
// it in flight). K rows are read from LDS as MFMA A operands with ds_read_b128; the latent is read again,
// transposed, with ds_read_b64_tr_b16, so the same LDS bytes serve both products. The 16-byte chunks of a
// row are XOR-swizzled (by choosing which global chunk a lane copies) so that both read shapes are
// bank-conflict free.
// Work is balanced over the compute units on the device: the rows' steps, laid end to end, are cut into
// equal chunks, one per workgroup. Every segment (a row's part inside a chunk) leaves a partial (max and
// sum in fp32, O / sum in bf16: half the bytes of fp32, one more rounding of the same size as the final
// one) that a second kernel merges (merge.hip); rows that fit one segment are stored directly.
//
// Replaces mla_v2.h / flash_mla_v2.h (paged cache, xlite/csrc/kernels/flash_mla_v2.h:537-847) and
// mla_v3.h (dense per-sequence cache) of the reference for batches with one query row per sequence.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kRescaleSlack = 8.0f;
constexpr int kWaves = 8;
constexpr int kNT = kWaves * 64;
constexpr int kStep = 32;
constexpr int kStages = 3;
constexpr int kAhead = 4;               // operand fetches in flight ahead of the matrix instruction using them
constexpr int C = 512;                 // kv_lora_rank
constexpr int R = 64;                  // rope_head_dim
constexpr int KS_C = C / 32;           // k-steps over the latent part
constexpr int KS_R = R / 32;           // k-steps over the rotary part
constexpr int kHeads = 16 * kWaves;    // heads of one pass
constexpr int HG = kHeads / 32;        // 32-head groups of the second product
constexpr int WC = C / kWaves;         // latent columns a wave owns in the second product
constexpr int CT = WC / 32;            // its 32-column tiles
constexpr int KC_ROWB = C * 2;         // 1024: LDS bytes of a latent row
constexpr int PE_ROWB = R * 2;         // 128
constexpr int KC_BYTES = kStep * KC_ROWB;             // 32 KiB
constexpr int STAGE_BYTES = KC_BYTES + kStep * PE_ROWB;  // 36 KiB: latent rows, then rotary rows
constexpr int PE_WAVES = kStep * PE_ROWB / 1024;      // waves that also copy 1 KiB of rotary rows
constexpr int P_ROWB = kStep * 2;      // a head's probabilities of one step
constexpr int P_BYTES = kHeads * P_ROWB;   // 8 KiB: two such buffers, used in turn
constexpr int F_BYTES = kHeads * 4;    // one fp32 per head: two buffers of rescale factors, one of final normalisers
constexpr int TR_ROWB = WC * 2 + 16;   // row pitch of the output transposition (a head's 64 columns of one wave)
constexpr uint32_t kTblCap = 3000;     // block-table entries of a segment staged in LDS

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

// XOR patterns for the 16-byte chunk index inside a row.
// Latent rows (1024 bytes, every row starts at bank 0): the pattern is even (a chunk pair stays a pair). The
// hardware serves a ds_read_b128 in four passes of 16 lanes, and a pass is not 16 consecutive lanes: lanes 0-3, 12-15,
// 20-23 and 24-27 go together, then 4-11, 16-19 and 28-31 (the upper half of the wave likewise). With lane = 16 j + row
// (j picks one of four consecutive chunks) a pass is rows 0-3 and 12-15 of one chunk next to rows 4-11 of its odd
// neighbour: half the pattern must be a bijection onto 0..7 on either row set. The transposing reads of the second
// product touch four consecutive rows 4 t .. 4 t + 3 per pass (32 lanes, 64 bytes of each row): their patterns differ
// in the two upper bits, so they land in four different 64-byte groups.
__device__ __forceinline__ uint32_t swz_kc(uint32_t row) { return ((row & 3) << 2) | (((row >> 2) & 1) << 1); }
// Rotary rows (128 bytes, two per bank window): low three chunk bits; rows of equal parity differ.
__device__ __forceinline__ uint32_t swz_pe(uint32_t row) { return (row >> 1) & 7; }

__device__ __forceinline__ void dma_1k(uint32_t lds_addr, uint32_t voff, const void *base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                 :: "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
// Four copies whose LDS and global addresses advance by 1 KiB each: the instruction's immediate offset is
// added to both, so one M0 value and one base serve the four.
__device__ __forceinline__ void dma_4x1k(uint32_t lds_addr, uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3,
                                         const void *base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %5\n\t"
                 "global_load_lds_dwordx4 %2, %5 offset:1024\n\t"
                 "global_load_lds_dwordx4 %3, %5 offset:2048\n\t"
                 "global_load_lds_dwordx4 %4, %5 offset:3072\n\t"
                 :: "s"(lds_addr), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(base) : "memory", "m0");
}
// the same copy with a 64-bit address per lane (rows gathered from anywhere in a cache of any size)
__device__ __forceinline__ void dma_1k_ptr(uint32_t lds_addr, const void *lane_ptr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\t"
                 :: "s"(lds_addr), "v"(lane_ptr) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void dma_wait()
{
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// LISTS: rows may come with position lists (p.top_k != 0); a separate instantiation, so that the plain kernel
// keeps its register allocation.
template <bool LISTS, int HGN>
__global__ void __launch_bounds__(kNT)
mla_decode_kernel(const MlaDecodeParams p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *p_lds = smem + kStages * STAGE_BYTES;                        // probabilities: 2 x [head][32 positions]
    float *f_lds = reinterpret_cast<float *>(p_lds + 2 * P_BYTES);              // 2 x rescale factors, then normalisers
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(p_lds + 2 * P_BYTES + 3 * F_BYTES);
    uint32_t *mask_lds = tbl_lds + kTblCap;   // kTblCap / kStep + 2 words: valid positions of a listed row's steps
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));

    const uint32_t lane = threadIdx.x & 63;
    // Instrumentation, off unless a probe buffer was set: workgroup 0 leaves the shader clock counter and the 100 MHz
    // wall clock at entry and after its last segment, whose ratio is the clock the kernel ran at.
    if (p.clock_probe != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
        p.clock_probe[0] = clock64();
        p.clock_probe[1] = wall_clock64();
    }
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t col = lane & 15;    // head inside the wave's 16 (column of every product)
    const uint32_t gi = lane >> 4;     // which 8 of a k-step's 32 elements / which 4 rows of a result tile
    const bool dense = p.block_tables == nullptr;

    // ---- per-lane address roles, recomputed from the lane index at every step (a dozen vector
    // instructions) instead of living in registers for the whole kernel.
    // Copy roles: wave w moves latent rows 4w .. 4w+3 (lane = chunk slot; a slot holds chunk
    // slot ^ pattern(row), and the pattern of row 4w + i is (i << 2) | ((w & 1) << 1)) and, for w < 4, rotary
    // rows 8w .. 8w+7 (lane / 8 = row, lane % 8 = chunk slot).
    // Score product: K rows as the A operand (row = position 16 mt + col, chunk 4 ks + gi).
    // Second product (32 x 32 x 16, lane = 32 half + n): n is a latent column of the tile (A) and a head of the
    // group (B, D), `half` picks 8 of a k-step's 16 positions. Transposed latent: the 16-lane group (half, cg)
    // covers positions 8 half .. + 3 (+4 for the second read) of a k-step and columns 16 cg .. + 15 of the tile;
    // lane 4 j' + q of the group points at elements [4 q, +4) of position 8 half + j'.
    uint32_t kc_voff, pe_voff, pe_row, kx, px, k_row, p_row, gi4, vt0, vt1, pr_off;
    auto set_roles = [&](uint32_t ln) {
        const uint32_t c4 = ln & 15, g = ln >> 4;
        gi4 = g * 4;
        kc_voff = ((ln & ~15u) | ((ln & 15u) ^ swz_kc(4 * wave))) << 4;   // (row 4 wave + i: this ^ (i << 6))
        pe_row = (wave & (PE_WAVES - 1)) * 8 + (ln >> 3);
        pe_voff = ((ln & 7u) ^ swz_pe(pe_row)) << 4;
        kx = (g ^ swz_kc(c4)) << 4;
        px = (g ^ swz_pe(c4)) << 4;
        k_row = c4 * KC_ROWB;
        p_row = KC_BYTES + c4 * PE_ROWB;
        const uint32_t hf = ln >> 5, cg = (ln >> 4) & 1, jp = (ln & 15) >> 2, q = ln & 3, n = ln & 31;
        // the wave's columns start at chunk 8 w; tile ct adds 4 chunks (XOR of bit 6 of the byte offset)
        const uint32_t chunk = 8 * (wave & 1) + 2 * cg + (q >> 1);
        vt0 = (8 * hf + jp) * KC_ROWB + (wave >> 1) * 256 + ((chunk ^ ((jp << 2) | 0u)) << 4) + ((q & 1) << 3);
        vt1 = (8 * hf + 4 + jp) * KC_ROWB + (wave >> 1) * 256 + ((chunk ^ ((jp << 2) | 2u)) << 4) + ((q & 1) << 3);
        // probabilities of head n of a 32-head group: 16 bytes = the 8 positions of this half of a k-step
        pr_off = n * P_ROWB + ((hf ^ ((n >> 2) & 3)) << 4);
    };
    set_roles(lane);

    // ---- one (sequence, query row, range of steps) at a time
    // `n_slots`: segments the row is cut into; `pslot`: where this segment's partial goes when there are several;
    // `meta`: what the merge needs to find the row's partials (written with the row's first segment).
    // `limit`: the row's length in positions - its causal range, or top_k entries of its position list when
    // the range (`causal`) is longer than that (`listed`): then position j of the row is list entry j.
    auto run_segment = [&](uint32_t seq, uint32_t tok, uint32_t limit, uint32_t causal, uint32_t step_a, uint32_t step_b,
                           uint32_t n_slots, uint32_t pslot, int4 meta) {
        const int32_t *table = dense ? nullptr : p.block_tables + static_cast<uint64_t>(seq) * p.max_num_blocks;
        const uint32_t t0 = step_a * kStep;
        const uint32_t t1 = min(limit, step_b * kStep);
        const uint32_t n_steps = step_b - step_a;
        const bool single = n_slots == 1;
        // (by_pos: a block size that is not a multiple of 32 - a step's positions do not share a block, so every row
        // is walked position by position through the same staging of cache rows; rows without a list of their own
        // walk 0, 1, 2, ...)
        const bool by_list = LISTS && p.top_k != 0 && causal > p.top_k;
        const bool listed = LISTS && (by_list || p.by_pos != 0);
        const uint32_t blk0 = dense || listed ? 0 : t0 / p.block_size;
        // ---- [q_absorb | qr] of the lane's head: 16 bytes of every 64-byte k-step. Heads past the end repeat
        // the last one; their results are never stored. The first pass's loads are issued here, ahead of the
        // block-table lookups, so that both travel together.
        uint4 qreg[KS_C + KS_R];
        auto load_q = [&](uint32_t h0) {
            const uint32_t head = h0 + wave * 16 + col;
            const uint64_t rh = static_cast<uint64_t>(tok) * p.n_heads + min(head, p.n_heads - 1);
            const uint4 *qa = reinterpret_cast<const uint4 *>(p.q_absorb + rh * C) + gi;
            const uint4 *qq = reinterpret_cast<const uint4 *>(p.qr + rh * R) + gi;
#pragma unroll
            for (int ks = 0; ks < KS_C; ks++) {
                qreg[ks] = qa[4 * ks];
            }
#pragma unroll
            for (int ks = 0; ks < KS_R; ks++) {
                qreg[KS_C + ks] = qq[4 * ks];
            }
        };
        // The block-table entries of the segment are requested before the query rows (memory operations finish in
        // order: behind the 147 KB of queries the first copies would start five microseconds later) ...
        const uint32_t nblk_seg = dense || listed ? 0 : (t1 - 1) / p.block_size - blk0 + 1;
        uint32_t tbl_first = 0;
        if (threadIdx.x < nblk_seg) {
            tbl_first = static_cast<uint32_t>(table[blk0 + threadIdx.x]);
        }
        load_q(0);
        if (listed) {
            // cache row of every list entry of the segment (tbl_lds[i] for entry t0 + i) and, per step, the mask
            // of its usable entries: inside the causal range, not a repeat of its predecessor. The others point
            // at the row of position 0 and get probability zero.
            const int32_t *list = p.topk_indices + static_cast<uint64_t>(tok) * p.top_k;
            for (uint32_t base = 0; base < n_steps * kStep; base += kNT) {
                const uint32_t i = base + threadIdx.x, j = t0 + i;
                int32_t x = -1;
                bool ok = false;
                if (i < n_steps * kStep && j < t1) {
                    if (by_list) {
                        x = list[j];
                        ok = x >= 0 && static_cast<uint32_t>(x) < causal && (j == 0 || list[j - 1] != x);
                    } else {   // the row's own positions
                        x = static_cast<int32_t>(j);
                        ok = true;
                    }
                }
                const uint32_t pos = ok ? static_cast<uint32_t>(x) : 0u;
                if (i < n_steps * kStep) {
                    tbl_lds[i] = static_cast<uint32_t>(table[pos / p.block_size]) * p.block_size + pos % p.block_size;
                }
                const uint64_t m = __ballot(ok);
                if (lane == 0 && base + wave * 64 < n_steps * kStep + 32) {
                    mask_lds[(base >> 5) + 2 * wave] = static_cast<uint32_t>(m);
                    mask_lds[(base >> 5) + 2 * wave + 1] = static_cast<uint32_t>(m >> 32);
                }
            }
        } else if (!dense) {
            // block-table entries of the tile (lookups in the loop then cost an LDS read only)
            // ... and stored here, with the query loads still in flight (segments of more than 512 blocks: the rest)
            if (threadIdx.x < nblk_seg) {
                tbl_lds[threadIdx.x] = tbl_first;
            }
            for (uint32_t i = threadIdx.x + kNT; i < nblk_seg; i += kNT) {
                tbl_lds[i] = static_cast<uint32_t>(table[blk0 + i]);
            }
        }
        __syncthreads();

        // passes over groups of 128 heads
        for (uint32_t h0 = 0; h0 < p.n_heads; h0 += 16 * kWaves) {
            if (h0 != 0) {
                load_q(h0);
            }
            // O^T of the wave's 64 columns for all heads of the pass: tile (ct, hg) is columns 32 ct .. + 31 by heads
            // 32 hg .. + 31; lane = 32 half + n holds head n, register v column 8 (v / 4) + 4 half + v % 4 of the tile
            f32x16_t O[CT][HG];
#pragma unroll
            for (int ct = 0; ct < CT; ct++) {
#pragma unroll
                for (int hg = 0; hg < HG; hg++) {
#pragma unroll
                    for (int k = 0; k < 16; k++) {
                        O[ct][hg][k] = 0.f;
                    }
                }
            }
            float m_run = -INFINITY, l_run = 0.f;   // of the lane's own head (the score side)

            // ---- cache copies of one step: scalars first, then four or five 1 KiB copies per wave ---------
            struct StepCopy {
                const char *kb, *pb;
                uint32_t stage, last_pos;
            };
            auto plan = [&](uint32_t step) {
                const uint32_t ts = t0 + step * kStep;
                uint64_t row0;   // first cache row: the 32 positions share one block (block_size % 32 == 0)
                if (dense) {
                    row0 = static_cast<uint64_t>(seq) * p.dense_len + ts;
                } else {
                    const uint32_t blk = ts / p.block_size, off = ts % p.block_size;
                    const uint32_t phys = __builtin_amdgcn_readfirstlane(tbl_lds[blk - blk0]);
                    row0 = static_cast<uint64_t>(phys) * p.block_size + off;
                }
                StepCopy c;
                // positions at or beyond the end re-read the last valid one: finite values whose
                // probabilities are forced to zero
                c.last_pos = min(t1 - 1 - ts, static_cast<uint32_t>(kStep - 1));
                c.stage = smem_addr + (step % kStages) * STAGE_BYTES;
                c.kb = reinterpret_cast<const char *>(p.k_cache) + row0 * KC_ROWB;
                c.pb = reinterpret_cast<const char *>(p.pe_cache) + row0 * PE_ROWB;
                return c;
            };
            auto issue = [&](uint32_t step) {
                const uint32_t r0 = 4 * wave;
                if (listed) {
                    const uint32_t stage = smem_addr + (step % kStages) * STAGE_BYTES;
                    const uint32_t e0 = step * kStep;
                    // the wave's four entries in one LDS read (a lookup is awaited with every operand read pending)
                    const uint4 rows = *reinterpret_cast<const uint4 *>(tbl_lds + e0 + r0);
                    const uint32_t row_of[4] = {rows.x, rows.y, rows.z, rows.w};
#pragma unroll
                    for (uint32_t i = 0; i < 4; i++) {
                        const uint64_t phys = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row_of[i])));
                        dma_1k(stage + (r0 + i) * KC_ROWB, kc_voff ^ (i << 6),
                               reinterpret_cast<const char *>(p.k_cache) + phys * KC_ROWB);
                    }
                    if (wave < PE_WAVES) {
                        const uint64_t phys = tbl_lds[e0 + pe_row];   // per lane: eight rotary rows per copy
                        dma_1k_ptr(stage + KC_BYTES + wave * 1024,
                                   reinterpret_cast<const char *>(p.pe_cache) + phys * PE_ROWB + pe_voff);
                    }
                    return;
                }
                const StepCopy c = plan(step);
                if (c.last_pos == kStep - 1) {
                    dma_4x1k(c.stage + r0 * KC_ROWB, kc_voff, kc_voff ^ (1u << 6), kc_voff ^ (2u << 6),
                             kc_voff ^ (3u << 6), c.kb + r0 * KC_ROWB);
                    if (wave < PE_WAVES) {
                        dma_1k(c.stage + KC_BYTES + wave * 1024, pe_row * PE_ROWB + pe_voff, c.pb);
                    }
                } else {
#pragma unroll
                    for (uint32_t i = 0; i < 4; i++) {
                        const uint32_t src = min(r0 + i, c.last_pos);   // uniform
                        dma_1k(c.stage + (r0 + i) * KC_ROWB, kc_voff ^ (i << 6), c.kb + src * KC_ROWB);
                    }
                    if (wave < PE_WAVES) {
                        const uint32_t prow = min(pe_row, c.last_pos);
                        dma_1k(c.stage + KC_BYTES + wave * 1024, prow * PE_ROWB + pe_voff, c.pb);
                    }
                }
            };

            // ---- S^T = K . Q^T of one step: two tiles of 16 positions x 16 heads, 18 k-steps of 32 elements.
            // The two accumulation chains alternate; operands are fetched kAhead products ahead.
            // The first kAhead operands are fetched by `qk_fetch`, which the loop calls right behind the step's barrier:
            // their latency then overlaps the address arithmetic of the copies issued in between.
            // The operand reads of a step go through six per-lane base offsets (the four XOR variants of the latent
            // rows, the two of the rotary rows), formed once per step and made opaque to the compiler; everything else
            // of a read's address is a constant that fits the instruction's offset field. (Left to itself the compiler
            // forms biased bases and adds a negative constant per read: 35 vector additions per step.)
            uint32_t kbase[4], pbase[2];
            auto set_bases = [&](uint32_t step) {
                const uint32_t soff = (step % kStages) * STAGE_BYTES;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    kbase[j] = soff + k_row + ((j << 6) ^ kx);
                    asm volatile("" : "+v"(kbase[j]));
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    pbase[j] = soff + p_row + ((j << 6) ^ px);
                    asm volatile("" : "+v"(pbase[j]));
                }
            };
            auto rd_k = [&](int i) {
                const int ks = i >> 1, mt = i & 1;
                return ks < KS_C ? *reinterpret_cast<const uint4 *>(smem + kbase[ks & 3] + (((ks >> 2) << 8) + mt * 16 * KC_ROWB))
                                 : *reinterpret_cast<const uint4 *>(smem + pbase[ks - KS_C] + mt * 16 * PE_ROWB);
            };
            auto qk_fetch = [&](uint32_t step, uint4 (&a)[kAhead]) {
                set_bases(step);
#pragma unroll
                for (int i = 0; i < kAhead; i++) {
                    a[i] = rd_k(i);
                }
            };
            auto qk = [&](uint32_t step, f32x4_t (&S)[2], uint4 (&a)[kAhead]) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    S[0][k] = 0.f;
                    S[1][k] = 0.f;
                }
#pragma unroll
                for (int i = 0; i < 2 * (KS_C + KS_R); i++) {
                    S[i & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[i % kAhead]),
                                                                     __builtin_bit_cast(bf16x8_t, qreg[i >> 1]),
                                                                     S[i & 1], 0, 0, 0);
                    if (i + kAhead < 2 * (KS_C + KS_R)) {
                        a[i % kAhead] = rd_k(i + kAhead);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            };

            // ---- online softmax of one step. Register k of score tile mt holds position t + 16 mt + 4 gi + k. The
            // reference maximum only moves when the step maximum exceeds it by more than 2^8: probabilities then
            // stay below 2^8 (the same relative precision in bf16, and the normaliser shares the reference), and the
            // accumulators are rescaled rarely. The probabilities of the lane's head go to LDS, [head][position] in
            // 16-bit, 16-byte chunk c of head h in slot c ^ ((h >> 2) & 3) (the reads of the second product, 32 heads
            // a pass, then touch every bank once), and with them the factor by which the head's reference moved.
            auto softmax = [&](uint32_t step, f32x4_t (&S)[2]) {
                const uint32_t t = t0 + step * kStep;
                const uint32_t lane_pos = t + gi4;
                float mx = -INFINITY;
                // the softmax runs at a raised wave priority: its vector instructions go ahead of the products of
                // the SIMD's other wave
                __builtin_amdgcn_s_setprio(2);
#pragma unroll
                for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        S[mt][k] *= p.scale_log2e;
                    }
                }
                if (listed) {
                    const uint32_t valid = __builtin_amdgcn_readfirstlane(mask_lds[step]) >> gi4;
                    if (static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(mask_lds[step])) != 0xffffffffu) {
#pragma unroll
                        for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                            for (int k = 0; k < 4; k++) {
                                S[mt][k] = ((valid >> (mt * 16 + k)) & 1u) ? S[mt][k] : -INFINITY;
                            }
                        }
                    }
                } else if (t + kStep > t1) {   // uniform: only a tile's last step has positions to mask
#pragma unroll
                    for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            const uint32_t pos = lane_pos + mt * 16 + k;
                            S[mt][k] = pos < t1 ? S[mt][k] : -INFINITY;
                        }
                    }
                }
#pragma unroll
                for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        mx = fmaxf(mx, S[mt][k]);
                    }
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16));
                {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
                    mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                const float m_new = mx > m_run + kRescaleSlack ? mx : m_run;
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                // (nothing accumulated yet: no rescale)
                const float alpha = m_run == -INFINITY ? 1.0f : fast_exp2(m_run - m_safe);
                m_run = m_new;
                uint32_t pw[4];
                float psum = 0.f;
#pragma unroll
                for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                    for (int k = 0; k < 4; k += 2) {
                        const float e0 = fast_exp2(S[mt][k] - m_safe);
                        const float e1 = fast_exp2(S[mt][k + 1] - m_safe);
                        psum += e0 + e1;
                        pw[mt * 2 + k / 2] = BF16::pack(e0, e1);
                    }
                }
                l_run = l_run * alpha + psum;
                // positions 16 mt + 4 gi .. + 3 of head 16 wave + col: chunk 2 mt + gi / 2, its half gi % 2
                {
                    uint32_t ln;
                    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
                    const uint32_t h = wave * 16 + (ln & 15), g = ln >> 4;
                    unsigned char *row = p_lds + (step & 1) * P_BYTES + h * P_ROWB + ((g & 1) << 3);
                    const uint32_t f = (h >> 2) & 3;
                    *reinterpret_cast<uint2 *>(row + (((g >> 1) ^ f) << 4)) = make_uint2(pw[0], pw[1]);
                    *reinterpret_cast<uint2 *>(row + (((2 + (g >> 1)) ^ f) << 4)) = make_uint2(pw[2], pw[3]);
                    if (g == 0) {
                        f_lds[(step & 1) * kHeads + h] = alpha;
                    }
                }
                __builtin_amdgcn_s_setprio(0);
            };

            // ---- O^T += kc^T . P^T of step `step`, whose probabilities every wave left in LDS before the barrier
            // this call follows: the wave's two 32-column tiles by four 32-head groups, two k-steps of 16 positions.
            // Four transposed latent operands (two reads each) and eight probability operands per step.
            auto pv = [&](uint32_t step) {
                const uint32_t soff = (step % kStages) * STAGE_BYTES;
                typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
                // the heads' rescale factors (rarely other than 1)
                {
                    float al[HG];
                    bool any = false;
#pragma unroll
                    for (int hg = 0; hg < HGN; hg++) {
                        al[hg] = f_lds[(step & 1) * kHeads + hg * 32 + (pr_off / P_ROWB)];
                        any = any || al[hg] != 1.0f;
                    }
                    if (__any(any)) {
#pragma unroll
                        for (int ct = 0; ct < CT; ct++) {
#pragma unroll
                            for (int hg = 0; hg < HGN; hg++) {
#pragma unroll
                                for (int k = 0; k < 16; k++) {
                                    O[ct][hg][k] *= al[hg];
                                }
                            }
                        }
                    }
                }
                // (per-lane base offsets formed once per step and opaque to the compiler, the rest of an address a
                // constant in the instruction's offset field: see the first product)
                uint32_t vbase[2][CT], prbase[2];
#pragma unroll
                for (int ct = 0; ct < CT; ct++) {
                    vbase[0][ct] = soff + (vt0 ^ (ct << 6));
                    vbase[1][ct] = soff + (vt1 ^ (ct << 6));
                    asm volatile("" : "+v"(vbase[0][ct]), "+v"(vbase[1][ct]));
                }
#pragma unroll
                for (int ks2 = 0; ks2 < 2; ks2++) {
                    prbase[ks2] = (step & 1) * P_BYTES + (pr_off ^ (ks2 << 5));
                    asm volatile("" : "+v"(prbase[ks2]));
                }
                auto rd_v = [&](int ks2, int ct) {
                    const uint2 lo = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(smem + vbase[0][ct] + ks2 * 16 * KC_ROWB)));
                    const uint2 hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(smem + vbase[1][ct] + ks2 * 16 * KC_ROWB)));
                    return make_uint4(lo.x, lo.y, hi.x, hi.y);
                };
                auto rd_p = [&](int ks2, int hg) {
                    return *reinterpret_cast<const uint4 *>(p_lds + prbase[ks2] + hg * 32 * P_ROWB);
                };
                // (operands of one k-step at a time: 24 registers; the SIMD's other wave covers their latency)
#pragma unroll
                for (int ks2 = 0; ks2 < 2; ks2++) {
                    uint4 va[CT], pb[HG];
#pragma unroll
                    for (int ct = 0; ct < CT; ct++) {
                        va[ct] = rd_v(ks2, ct);
                    }
#pragma unroll
                    for (int hg = 0; hg < HG; hg++) {
                        pb[hg] = rd_p(ks2, hg);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ct = 0; ct < CT; ct++) {
#pragma unroll
                        for (int hg = 0; hg < HG; hg++) {
                            // (head groups beyond the model's heads hold nothing: HGN = 1 for models of at most 32 heads,
                            // which run a quarter of the products)
                            if (hg < HGN) {
                                O[ct][hg] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, va[ct]),
                                                                                   __builtin_bit_cast(bf16x8_t, pb[hg]),
                                                                                   O[ct][hg], 0, 0, 0);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            };

            // ---- pipeline. Iteration `it` follows a barrier behind which step it's copies (issued one iteration
            // earlier) have landed for everybody, every wave has left the probabilities of step it - 1 in LDS and
            // nobody reads the stage of step it - 2 any more: it issues the copies of step it + 1 into that stage,
            // forms the scores of step it, runs their softmax and then the second product of step it - 1. Every copy
            // is unconditional (steps past the end copy the last step again, same bytes to the same place), so the
            // wait counts are exact.
            const uint32_t last = n_steps - 1;
            __syncthreads();   // the previous pass has left the stages
            issue(0);
            // The query loads were issued before this copy and complete before it (memory operations finish in
            // order); their latency overlaps the copy's. They must have landed before the loop: a wait for them
            // inside it would also wait for the cache copies in flight. The wait the compiler places here counts
            // the copies too (it does not know of them).
#pragma unroll
            for (int ks = 0; ks < KS_C + KS_R; ks++) {
                asm volatile("" : "+v"(qreg[ks].x), "+v"(qreg[ks].y), "+v"(qreg[ks].z), "+v"(qreg[ks].w));
            }
            f32x4_t S[2];
            for (uint32_t it = 0; it < n_steps; it++) {
                {
                    // the lane index from the hardware, opaque to the compiler: nothing derived from it can be
                    // hoisted out of the loop (and end up in a spill slot, whose reload would wait for every copy)
                    uint32_t ln;
                    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
                    set_roles(ln);
                }
                dma_wait<0>();              // this wave's share of step `it` has landed ...
                __syncthreads();            // ... and everybody else's; see above
                uint4 a[kAhead];
                qk_fetch(it, a);
                __builtin_amdgcn_sched_barrier(0);
                issue(min(it + 1, last));
                qk(it, S, a);
                softmax(it, S);
                if (it > 0) {
                    pv(it - 1);
                }
            }
            dma_wait<0>();
            __syncthreads();   // the last step's probabilities are in LDS
            {
                uint32_t ln;
                asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
                set_roles(ln);
            }
            pv(last);

            // ---- results. The normaliser of a head lives with the wave that formed its scores: it goes through LDS
            // to the eight waves that hold the head's columns.
            // (lane roles from the hardware once more: nothing derived from threadIdx stays live across the loop,
            // where its register would be spilled and reloaded every step)
            uint32_t ln_e;
            asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln_e));
            const uint32_t col_e = ln_e & 15, gi_e = ln_e >> 4;
            float l_tot = l_run + __shfl_xor(l_run, 16);
            l_tot += __shfl_xor(l_tot, 32);
            const float inv_own = l_tot > 0.f ? 1.0f / l_tot : 0.f;
            const uint32_t head = h0 + wave * 16 + col_e;
            const bool h_ok = head < p.n_heads;
            if (gi_e == 0) {
                f_lds[2 * kHeads + wave * 16 + col_e] = inv_own;
            }
            if (h_ok && gi_e == 0 && !single) {
                *reinterpret_cast<float2 *>(p.part_ml + (static_cast<uint64_t>(pslot) * p.n_heads + head) * 2) =
                    make_float2(m_run, l_tot);
            }
            __syncthreads();   // normalisers visible; every wave is past its last product: the stages are free
            // O^T lane layout: lane = 32 half + n holds head 32 hg + n, register v of tile (ct, hg) = column
            // 64 wave + 32 ct + 8 (v / 4) + 4 half + v % 4. Normalised, rounded and transposed through a wave-private
            // LDS region (64 heads x 64 columns at a time) so that a store instruction writes 128 contiguous bytes of
            // each of eight heads' rows.
            {
                const uint32_t n = ln_e & 31, hf = ln_e >> 5;
                unsigned char *my_tr = smem + wave * (64 * TR_ROWB);
                uint16_t *dst_base = single ? p.out + static_cast<uint64_t>(tok) * p.n_heads * C
                                            : reinterpret_cast<uint16_t *>(p.part_acc) + static_cast<uint64_t>(pslot) * p.n_heads * C;
#pragma unroll
                for (int half_pass = 0; half_pass < (HGN + 1) / 2; half_pass++) {
#pragma unroll
                    for (int hh = 0; hh < (HGN < 2 ? HGN : 2); hh++) {
                        const int hg = 2 * half_pass + hh;
                        const float inv = f_lds[2 * kHeads + hg * 32 + n];
#pragma unroll
                        for (int ct = 0; ct < CT; ct++) {
#pragma unroll
                            for (int g4 = 0; g4 < 4; g4++) {
                                uint2 o;
                                o.x = BF16::pack(O[ct][hg][4 * g4 + 0] * inv, O[ct][hg][4 * g4 + 1] * inv);
                                o.y = BF16::pack(O[ct][hg][4 * g4 + 2] * inv, O[ct][hg][4 * g4 + 3] * inv);
                                *reinterpret_cast<uint2 *>(my_tr + (hh * 32 + n) * TR_ROWB + (32 * ct + 8 * g4 + 4 * hf) * 2) = o;
                            }
                        }
                    }
                    // wave-private region: the LDS counter wait the compiler inserts is all the ordering needed.
                    // Lane l stores 16 bytes: head 8 i + l / 8 of the 64, chunk l % 8 of its 128 bytes.
#pragma unroll
                    for (int i = 0; i < (HGN < 2 ? 4 : 8); i++) {
                        const uint32_t hl = 8 * i + (ln_e >> 3);
                        const uint32_t hd = h0 + 64 * half_pass + hl;
                        const uint4 x = *reinterpret_cast<const uint4 *>(my_tr + hl * TR_ROWB + (ln_e & 7) * 16);
                        if (hd < p.n_heads) {
                            *reinterpret_cast<uint4 *>(dst_base + static_cast<uint64_t>(hd) * C + wave * WC + (ln_e & 7) * 8) = x;
                        }
                    }
                }
            }
            if (step_a == 0 && h0 == 0 && wave == 0 && ln_e == 0) {
                reinterpret_cast<int4 *>(p.part_meta)[tok] = meta;
            }
        }
        __syncthreads();   // tbl_lds and the stages are rewritten by the next segment
        if (p.clock_probe != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
            p.clock_probe[2] = clock64();
            p.clock_probe[3] = wall_clock64();
        }
    };

    // ---- the work list. Every query row owns ceil(limit / 32) steps.
    // Few rows (at most 64: a decode batch with several workgroups per row): every row is cut into chunks of its
    // own, so that no workgroup pays the set-up of a segment (query load, pipeline fill, partial store) twice.
    // With G workgroups the chunk bound is the smallest L for which sum ceil(n_t / L) <= G; row t then gets
    // ceil(n_t / L) chunks of equal length. Everything lives in the lanes of a wave (lane = row), every wave
    // computing the same.
    // Many rows: the rows' steps, laid end to end, are cut into chunks of equal length, one chunk per workgroup
    // (more when a chunk would not fit the block table staging); a chunk that crosses a row boundary is
    // processed as several segments.
    // Either way only a chunk's first and last segment can be parts of rows that continue in other chunks:
    // chunk c owns the partial slots 2c (its first segment) and 2c + 1 (its last, when that is another one), and
    // a row cut into n segments starting in chunk c0 finds them at 2 c0 (+ 1 unless it is that chunk's first
    // segment), 2 (c0 + 1), 2 (c0 + 2), ...
    __shared__ uint32_t scan_ws[kWaves];
    __shared__ uint32_t found[4];
    const uint32_t B = p.batch, T = p.total_rows;
    // Workgroups are dealt round-robin to the 8 XCDs, each with an L2 of its own; consecutive chunks are parts of
    // one row and read the same 147 KB of queries, so chunk numbers follow the XCD first: XCD x takes the chunks
    // x G / 8 .. (x + 1) G / 8 - 1, and a row's query block is fetched from memory once, not once per chunk.
    const uint32_t wg = gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
    // the sequence that owns query row t (query_start_loc is a prefix sum), or B. A batch of one row per
    // sequence answers with one round of loads.
    auto seq_of = [&](uint32_t t) {
        if (t < B && p.query_start_loc[t] == static_cast<int32_t>(t) && p.lens[t] == 1) {
            return t;
        }
        uint32_t lo = 0, hi = B;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) / 2;
            if (p.query_start_loc[mid] <= static_cast<int32_t>(t)) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        if (lo == 0) {
            return B;
        }
        return static_cast<int32_t>(t) < p.query_start_loc[lo - 1] + p.lens[lo - 1] ? lo - 1 : B;
    };
    // first sequence at or after `seq` that contains row t (rows are in sequence order), or B
    auto advance = [&](uint32_t seq, uint32_t t) {
        while (seq < B && static_cast<int32_t>(t) >= p.query_start_loc[seq] + p.lens[seq]) {
            seq++;
        }
        return seq < B && static_cast<int32_t>(t) >= p.query_start_loc[seq] ? seq : B;
    };
    auto row_causal = [&](uint32_t t, uint32_t seq) -> uint32_t {
        if (seq >= B) {
            return 0;   // a row outside every sequence
        }
        const uint32_t clen = static_cast<uint32_t>(p.cached_lens[seq]);
        return dense ? min(clen + static_cast<uint32_t>(p.lens[seq]), p.dense_len)
                     : clen + (t - static_cast<uint32_t>(p.query_start_loc[seq])) + 1;
    };
    // positions the row walks: its causal range, or its list of top_k entries when the range is longer
    auto row_limit = [&](uint32_t t, uint32_t seq) -> uint32_t {
        const uint32_t causal = row_causal(t, seq);
        return LISTS && p.top_k != 0 && causal > p.top_k ? p.top_k : causal;
    };
    uint32_t chunk_cap = (kTblCap - 2) * p.block_size / kStep;
    if (LISTS) {
        chunk_cap = min(chunk_cap, static_cast<uint32_t>(kTblCap / kStep));   // a listed row stages one entry per position
    }

    if (T <= 64) {
        uint32_t my_seq = B, my_causal = 0, my_limit = 0, my_n = 0;
        if (lane < T) {
            // a decode batch has row t in sequence t: that sequence's cached length is fetched in the same round of
            // loads as the answer to "which sequence" (one memory round trip instead of two)
            // (three unconditional loads from a clamped index: written as a chain of && the compiler issues and
            // awaits them one after the other)
            const uint32_t li = min(lane, B - 1);
            const int32_t g_cached = p.cached_lens[li], g_start = p.query_start_loc[li], g_len = p.lens[li];
            const uint32_t guess = static_cast<uint32_t>(g_cached);
            const bool own = (lane < B) & (g_start == static_cast<int32_t>(lane)) & (g_len == 1);
            my_seq = own ? lane : seq_of(lane);
            my_causal = own && !dense ? guess + 1 : row_causal(lane, my_seq);
            my_limit = LISTS && p.top_k != 0 && my_causal > p.top_k ? p.top_k : my_causal;
            my_n = ceil_div(my_limit, static_cast<uint32_t>(kStep));
            if (my_n == 0 && blockIdx.x == 0 && wave == 0) {
                reinterpret_cast<int4 *>(p.part_meta)[lane] = make_int4(0, 0, 0, 0);   // a row without keys: nothing to merge
            }
        }
        auto wave_sum = [&](uint32_t v) {
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                v += __shfl_xor(v, d);
            }
            return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
        };
        const uint32_t total = wave_sum(my_n);
        if (total == 0) {
            return;
        }
        // the smallest chunk bound that needs no more chunks than there are workgroups
        uint32_t bound = max(ceil_div(total, gridDim.x), p.chunk_min_steps);
        uint32_t my_k = 0, n_chunks = 0;
        bool fits = false;
        for (uint32_t tries = 0; tries < 24 && bound <= chunk_cap; tries++, bound++) {
            my_k = ceil_div(my_n, bound);
            n_chunks = wave_sum(my_k);
            if (n_chunks <= gridDim.x) {
                fits = true;
                break;
            }
        }
        if (fits) {
            const uint32_t c = wg;
            if (c >= n_chunks) {
                return;
            }
            uint32_t incl = my_k;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d);
                incl += lane >= static_cast<uint32_t>(d) ? up : 0u;
            }
            const uint32_t my_base = incl - my_k;   // first chunk of the lane's row
            const uint32_t row = static_cast<uint32_t>(__builtin_popcountll(__ballot(my_base <= c && lane < T))) - 1;
            // rows without steps share their base with the next row: the last row whose base is <= c owns the
            // chunk only if it has chunks, and a row with steps after such rows has the larger lane index
            const uint32_t r_seq = __builtin_amdgcn_readfirstlane(__shfl(my_seq, static_cast<int>(row)));
            const uint32_t r_causal = __builtin_amdgcn_readfirstlane(__shfl(my_causal, static_cast<int>(row)));
            const uint32_t r_limit = __builtin_amdgcn_readfirstlane(__shfl(my_limit, static_cast<int>(row)));
            const uint32_t r_n = __builtin_amdgcn_readfirstlane(__shfl(my_n, static_cast<int>(row)));
            const uint32_t r_k = __builtin_amdgcn_readfirstlane(__shfl(my_k, static_cast<int>(row)));
            const uint32_t r_base = __builtin_amdgcn_readfirstlane(__shfl(my_base, static_cast<int>(row)));
            const uint32_t len = ceil_div(r_n, r_k);          // equal chunks inside the row, none above the bound
            const uint32_t n_slots = ceil_div(r_n, len);      // the chunks that are not empty
            const uint32_t j = c - r_base;
            if (j >= n_slots) {
                return;
            }
            const int4 meta = make_int4(n_slots > 1 ? static_cast<int>(n_slots) : 0, static_cast<int>(r_base), 1, 0);
            run_segment(r_seq, row, r_limit, r_causal, j * len, min(r_n, (j + 1) * len), n_slots, 2 * c, meta);
            return;
        }
        // no bound within reach (rows far longer than the staging allows): the general split below
    }

    for (uint32_t c = wg;; c += gridDim.x) {
        // block-wide prefix sums of the rows' step counts (redone for every chunk: nothing of it stays in
        // registers while a segment runs)
        const uint32_t per = ceil_div(T, kNT);
        const uint32_t i_lo = min(T, threadIdx.x * per), i_hi = min(T, i_lo + per);
        uint32_t local = 0;
        {
            uint32_t seq = i_lo < i_hi ? seq_of(i_lo) : B;
            for (uint32_t t = i_lo; t < i_hi; t++) {
                if (t > i_lo) {
                    seq = advance(seq < B ? seq : 0, t);
                }
                const uint32_t n = ceil_div(row_limit(t, seq), kStep);
                local += n;
                if (n == 0 && blockIdx.x == 0 && c == 0) {
                    reinterpret_cast<int4 *>(p.part_meta)[t] = make_int4(0, 0, 0, 0);   // a row without keys: nothing to merge
                }
            }
        }
        uint32_t incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d);
            incl += lane >= static_cast<uint32_t>(d) ? up : 0;
        }
        __syncthreads();   // the previous chunk's readers of scan_ws and found are done
        if (lane == 63) {
            scan_ws[wave] = incl;
        }
        __syncthreads();
        uint32_t excl = incl - local, total = 0;
#pragma unroll
        for (uint32_t w = 0; w < kWaves; w++) {
            const uint32_t ws = scan_ws[w];
            excl += w < wave ? ws : 0;
            total += ws;
        }
        total = __builtin_amdgcn_readfirstlane(total);
        uint32_t chunk = max(ceil_div(total, gridDim.x), p.chunk_min_steps);
        chunk = min(chunk, chunk_cap);
        if (c >= ceil_div(total, chunk)) {
            return;
        }
        const uint32_t start = c * chunk;
        uint32_t remaining = min(total, start + chunk) - start;
        // the thread whose rows contain flat step `start` finds the row, its sequence and its first flat step
        if (excl <= start && start < excl + local) {
            uint32_t t = i_lo, first = excl, seq = seq_of(i_lo);
            for (;;) {
                const uint32_t n = ceil_div(row_limit(t, seq), kStep);
                if (start < first + n) {
                    break;
                }
                first += n;
                t++;
                seq = advance(seq < B ? seq : 0, t);
            }
            found[0] = t;
            found[1] = first;
            found[2] = seq;
        }
        __syncthreads();
        uint32_t row = __builtin_amdgcn_readfirstlane(found[0]);
        uint32_t first = __builtin_amdgcn_readfirstlane(found[1]);
        uint32_t seq = __builtin_amdgcn_readfirstlane(found[2]);
        uint32_t a = start - first;
        bool first_seg = true;
        for (;;) {
            const uint32_t limit = row_limit(row, seq);
            const uint32_t n = ceil_div(limit, kStep);
            if (n > 0) {
                const uint32_t b = min(n, a + remaining);
                const uint32_t c0 = first / chunk;
                const uint32_t n_slots = (first + n - 1) / chunk - c0 + 1;
                // written with the row's first segment (a == 0): then c0 == c
                const int4 meta = make_int4(n_slots > 1 ? static_cast<int>(n_slots) : 0, static_cast<int>(c),
                                            first_seg ? 1 : 0, 0);
                run_segment(seq, row, limit, row_causal(row, seq), a, b, n_slots, 2 * c + (first_seg ? 0 : 1), meta);
                remaining -= b - a;
                first_seg = false;
            }
            if (remaining == 0) {
                break;
            }
            first += n;
            row++;
            a = 0;
            seq = advance(seq < B ? seq : 0, row);
        }
        if (c + gridDim.x >= ceil_div(total, chunk)) {
            return;   // the usual case: one chunk per workgroup, no second scan
        }
    }
}

}  // namespace

bool mla_decode_supported(const MlaArgs &a)
{
    const bool dense = a.block_tables == nullptr;
    // position lists (top_k) go with the paged cache only
    // (a paged cache of any block size: those that are not a multiple of 32 are walked position by position)
    return a.kv_lora_rank == C && a.rope_head_dim == R && (dense ? a.top_k == 0 : a.block_size > 0) && a.top_k <= 2048;
}

namespace {

struct MlaPlan {
    uint32_t chunk_min_steps;   // smallest chunk a workgroup takes
    uint32_t n_workgroups;      // one per compute unit (the LDS ring allows no more)
    uint32_t max_chunks;        // bound on the number of chunks, hence of partial slots (two per chunk)
    size_t meta_bytes, ml_bytes, acc_bytes;
};

// The chunk the kernel really uses is the batch's total step count over the number of workgroups, which the
// host cannot know (the lengths live in device memory); it is never smaller than chunk_min_steps nor larger
// than what the block-table staging holds.
int mla_decode_plan(const MlaArgs &a, MlaPlan *pl)
{
    const bool dense = a.block_tables == nullptr;
    const uint64_t max_ctx = dense ? a.dense_len : static_cast<uint64_t>(a.max_num_blocks) * a.block_size;
    int dev = 0;
    XL_HIP(hipGetDevice(&dev));
    thread_local int cu_dev = -1, n_cu = 0;   // the compute-unit count of the device this thread last used
    if (cu_dev != dev) {
        XL_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
        cu_dev = dev;
    }
    // half of what one workgroup per compute unit would get if every row were as long as allowed, between 128
    // and 512 positions
    // with position lists no row walks more than top_k positions, and a chunk stages one entry per position
    const uint64_t max_len = a.top_k != 0 && a.top_k < max_ctx ? a.top_k : max_ctx;
    uint64_t tok = max_len * a.total_tokens / static_cast<uint64_t>(n_cu) / 2;
    tok = tok > 512 ? 512 : (tok < 128 ? 128 : tok);
    pl->chunk_min_steps = static_cast<uint32_t>(tok / kStep);
    pl->n_workgroups = static_cast<uint32_t>(n_cu);
    const uint64_t max_steps = (max_len + kStep - 1) / kStep;
    uint64_t chunk_cap = static_cast<uint64_t>(kTblCap - 2) * (dense ? kStep : a.block_size) / kStep;
    const bool by_pos = !dense && a.block_size % kStep != 0;
    if ((a.top_k != 0 || by_pos) && chunk_cap > kTblCap / kStep) {
        chunk_cap = kTblCap / kStep;
    }
    const uint64_t by_cap = (static_cast<uint64_t>(a.total_tokens) * max_steps + chunk_cap - 1) / chunk_cap;
    pl->max_chunks = static_cast<uint32_t>(by_cap > pl->n_workgroups ? by_cap : pl->n_workgroups);
    pl->meta_bytes = ((static_cast<size_t>(a.total_tokens) * sizeof(int4) + 255) / 256) * 256;
    pl->ml_bytes = static_cast<size_t>(2) * pl->max_chunks * a.n_heads * 2 * sizeof(float);
    pl->acc_bytes = static_cast<size_t>(2) * pl->max_chunks * a.n_heads * C * sizeof(uint16_t);
    return XLITE_HIP_OK;
}

}  // namespace

size_t mla_decode_workspace_bytes(const MlaArgs &a)
{
    MlaPlan pl{};
    if (mla_decode_plan(a, &pl) != XLITE_HIP_OK) {
        return 0;
    }
    return pl.meta_bytes + pl.ml_bytes + pl.acc_bytes;
}

int launch_mla_decode(hipStream_t stream, const MlaArgs &a)
{
    MlaPlan pl{};
    if (const int rc = mla_decode_plan(a, &pl)) {
        return rc;
    }
    const size_t need = pl.meta_bytes + pl.ml_bytes + pl.acc_bytes;
    if (a.workspace == nullptr || a.workspace_bytes < need) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    char *ws = static_cast<char *>(a.workspace);
    MlaDecodeParams p{};
    p.clock_probe = clock_probe();
    p.q_absorb = static_cast<const uint16_t *>(a.q_absorb);
    p.qr = static_cast<const uint16_t *>(a.qr);
    p.k_cache = static_cast<const uint16_t *>(a.k_cache);
    p.pe_cache = static_cast<const uint16_t *>(a.pe_cache);
    p.out = static_cast<uint16_t *>(a.o_absorb);
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.part_meta = reinterpret_cast<int32_t *>(ws);
    p.part_ml = reinterpret_cast<float *>(ws + pl.meta_bytes);
    p.part_acc = reinterpret_cast<float *>(ws + pl.meta_bytes + pl.ml_bytes);
    p.n_heads = a.n_heads;
    p.batch = a.batch;
    p.total_rows = a.total_tokens;
    p.block_size = a.block_tables == nullptr ? kStep : a.block_size;
    p.max_num_blocks = a.max_num_blocks;
    p.dense_len = a.dense_len;
    p.chunk_min_steps = pl.chunk_min_steps;
    p.scale_log2e = a.scale * kLog2e;
    p.topk_indices = a.topk_indices;
    p.top_k = a.top_k;
    XL_REQUIRE(a.top_k == 0 || a.topk_indices != nullptr, "top_k > 0 needs topk_indices");

    const size_t lds = static_cast<size_t>(kStages) * STAGE_BYTES + 2 * P_BYTES + 3 * F_BYTES +
                       (kTblCap + kTblCap / kStep + 2) * sizeof(uint32_t);
    // the kernel also has a few words of static LDS: ask for exactly the dynamic part
    p.by_pos = a.block_tables != nullptr && a.block_size % kStep != 0 ? 1u : 0u;
    const bool lists = a.top_k != 0 || p.by_pos != 0;
    const bool few = a.n_heads <= 32;
    const void *kernel = lists ? (few ? reinterpret_cast<const void *>(mla_decode_kernel<true, 1>)
                                      : reinterpret_cast<const void *>(mla_decode_kernel<true, 4>))
                               : (few ? reinterpret_cast<const void *>(mla_decode_kernel<false, 1>)
                                      : reinterpret_cast<const void *>(mla_decode_kernel<false, 4>));
    if (const int rc = ensure_dynamic_lds(kernel, lds)) {
        return rc;
    }
    const dim3 grid(pl.n_workgroups, 1, 1);
    if (lists) {
        if (few) {
            mla_decode_kernel<true, 1><<<grid, kNT, lds, stream>>>(p);
        } else {
            mla_decode_kernel<true, 4><<<grid, kNT, lds, stream>>>(p);
        }
    } else if (few) {
        mla_decode_kernel<false, 1><<<grid, kNT, lds, stream>>>(p);
    } else {
        mla_decode_kernel<false, 4><<<grid, kNT, lds, stream>>>(p);
    }
    XL_LAUNCH_CHECK();
    // rows that ended up in a single segment were stored directly
    return launch_merge_mla(stream, a.dtype, a.o_absorb, reinterpret_cast<const uint16_t *>(p.part_acc), p.part_ml,
                            p.part_meta, a.total_tokens, a.n_heads, C);
}

}  // namespace xlite
