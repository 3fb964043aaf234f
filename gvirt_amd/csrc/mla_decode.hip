// DeepSeek-style absorbed MLA decode on the matrix cores, split along the KV axis.
//
// One latent "kv head" is shared by all query heads, so the heads are the MFMA columns: a
// workgroup of 4 wavefronts (one per SIMD, each with the full 512-register budget) covers up to
// 128 heads, 32 per wave, of one (sequence, KV tile). The tile is walked in steps of 32 positions:
//   S^T[pos][head]  = [kc | pe][pos][:] . [q_absorb | qr][head][:]   36 x v_mfma_f32_32x32x16_bf16
//   O^T[c][head]   += kc^T[c][pos] . P^T[pos][head]                   32 x v_mfma_f32_32x32x16_bf16
// Register plan per lane: Q (B operand of the first product) 144, O^T accumulators 256, the rest
// for S, P and operands in flight. The cache never passes through registers: every wave copies its
// share of a step straight from global memory into LDS (global_load_lds_dwordx4, 1 KiB of
// consecutive cache bytes per instruction) into a ring of four 36 KiB stages, three steps in
// flight while the fourth is consumed, one barrier per step. K rows are read from LDS as MFMA A
// operands with ds_read_b128; the latent is read again, transposed, with ds_read_b64_tr_b16, so the
// same LDS bytes serve both products. The 16-byte chunks of a row are XOR-swizzled (by choosing
// which global chunk a lane copies) so that both read shapes are bank-conflict free.
// Every workgroup leaves a partial (max and sum in fp32, O / sum in bf16: half the bytes of fp32, one more
// rounding of the same size as the final one) that a second kernel merges (merge.hip).
//
// Replaces mla_v2.h / flash_mla_v2.h (paged cache, xlite/csrc/kernels/flash_mla_v2.h:537-847) and
// mla_v3.h (dense per-sequence cache) of the reference for batches with one query row per sequence.
#include "attention_common.h"

namespace xlite {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kRescaleSlack = 8.0f;
constexpr int kWaves = 4;
constexpr int kNT = kWaves * 64;
constexpr int kStep = 32;
constexpr int kStages = 4;
constexpr int kAhead = 2;               // operand fetches in flight ahead of the matrix instruction using them
constexpr int C = 512;                 // kv_lora_rank
constexpr int R = 64;                  // rope_head_dim
constexpr int KS_C = C / 16;           // k-steps over the latent part
constexpr int KS_R = R / 16;           // k-steps over the rotary part
constexpr int DT = C / 32;             // 32-row tiles of O^T
constexpr int KC_ROWB = C * 2;         // 1024: LDS bytes of a latent row
constexpr int PE_ROWB = R * 2;         // 128
constexpr int KC_BYTES = kStep * KC_ROWB;             // 32 KiB
constexpr int STAGE_BYTES = KC_BYTES + kStep * PE_ROWB;  // 36 KiB: latent rows, then rotary rows
constexpr int DMA_PER_WAVE = (kStep + kStep * PE_ROWB / 1024) / kWaves;  // 8 latent rows + 1 rotary block

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

struct MlaDecodeParams {
    const uint16_t *q_absorb;
    const uint16_t *qr;
    const uint16_t *k_cache;
    const uint16_t *pe_cache;
    uint16_t *out;
    const int32_t *query_start_loc;
    const int32_t *lens;
    const int32_t *cached_lens;
    const int32_t *block_tables;   // nullptr: dense cache, dense_len rows per sequence, no causality
    int32_t *part_cnt;
    float *part_acc;
    float *part_ml;
    uint32_t n_heads;
    uint32_t block_size;
    uint32_t max_num_blocks;
    uint32_t dense_len;
    uint32_t tile_tokens;
    uint32_t max_slots;
    float scale_log2e;
};

// XOR patterns for the 16-byte chunk index inside a row.
// Latent rows (1024 bytes, every row starts at bank 0): low four chunk bits. The 16 rows that one
// ds_read_b128 pass touches get 16 different chunk slots, and the 4 rows that one transposing pass
// touches get 4 different 64-byte groups.
__device__ __forceinline__ uint32_t swz_kc(uint32_t row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
// Rotary rows (128 bytes, two per bank window): low three chunk bits; rows of equal parity differ.
__device__ __forceinline__ uint32_t swz_pe(uint32_t row) { return (row >> 1) & 7; }

// One wave-wide copy of 1 KiB from global memory into LDS at `lds_addr` + 16 * lane. The compiler
// does not see the LDS write nor the vmcnt increment: completion is awaited with dma_wait below.
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
template <int N>
__device__ __forceinline__ void dma_wait()
{
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

__global__ void __launch_bounds__(kNT)
mla_decode_kernel(const MlaDecodeParams p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint32_t *tbl_lds = reinterpret_cast<uint32_t *>(smem + kStages * STAGE_BYTES);
    const uint32_t smem_addr = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(
        static_cast<uint32_t>((size_t)((__attribute__((address_space(3))) unsigned char *)smem)))));

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tile = blockIdx.x;
    const uint32_t seq = blockIdx.y;
    const uint32_t col = lane & 31;
    const uint32_t half = lane >> 5;
    const bool dense = p.block_tables == nullptr;

    // ---- per-lane address roles. They are recomputed from the lane index at every step (a dozen vector
    // instructions) instead of living in a dozen registers for the whole kernel: there are none to spare.
    // Copy roles: wave w moves latent rows 8w .. 8w+7 (lane = chunk slot) and rotary rows 8w .. 8w+7
    // (lane / 8 = row, lane % 8 = chunk slot); a slot holds chunk (slot ^ pattern(row)). The pattern of row
    // 8w + i is 4 (i % 4) | (2w % 4 + i / 4): one lane offset, XORed with a constant per copy.
    // Read roles: K rows as the A operand (row = position `col`, chunk 2 ks + half, chunk' = 2 ks ^ x);
    // transposed latent: 16-lane group g = lane / 16 covers columns 16 (g % 2) .. +16 of a 32-column tile
    // for the positions of half g / 2; lane 4 j' + q points at elements [4 q, +4) of position 4 half + j'
    // (+8 for the second read, +16 for the second k-step). The offsets of tile a = dt % 4 and of the second
    // read differ from vr_off by XOR constants (64 a, and 32 plus 8 rows); a tile's 256-byte group and the
    // second k-step are immediates.
    uint32_t kc_voff, pe_voff, pe_row, kx, px, k_row, p_row, vr_off, half4;
    auto set_roles = [&](uint32_t ln) {
        const uint32_t c5 = ln & 31, hf = ln >> 5;
        half4 = hf * 4;
        kc_voff = ((ln & ~15u) | ((ln & 15u) ^ ((2 * wave) & 3))) << 4;
        pe_row = wave * 8 + (ln >> 3);
        pe_voff = ((ln & 7u) ^ swz_pe(pe_row)) << 4;
        kx = (hf ^ swz_kc(c5)) << 4;
        px = (hf ^ swz_pe(c5)) << 4;
        k_row = c5 * KC_ROWB;
        p_row = KC_BYTES + c5 * PE_ROWB;
        const uint32_t g = ln >> 4, jp = (ln & 15) >> 2, q = ln & 3;
        const uint32_t y = 2 * (g & 1) + (q >> 1);
        const uint32_t pos = 4 * (g >> 1) + jp;
        vr_off = pos * KC_ROWB + ((y ^ swz_kc(pos)) << 4) + ((q & 1) << 3);
    };
    set_roles(lane);

    const int32_t qlen = p.lens[seq];
    const int32_t clen = p.cached_lens[seq];
    const int32_t qstart = p.query_start_loc[seq];
    const int32_t *table = dense ? nullptr : p.block_tables + static_cast<uint64_t>(seq) * p.max_num_blocks;

    for (int32_t r = 0; r < qlen; r++) {
        const uint32_t tok = static_cast<uint32_t>(qstart + r);
        const uint32_t limit = dense ? min(static_cast<uint32_t>(clen + qlen), p.dense_len)
                                     : static_cast<uint32_t>(clen + r + 1);
        const uint32_t n_tiles = ceil_div(limit, p.tile_tokens);
        if (tile >= n_tiles) {
            continue;
        }
        const uint32_t t0 = tile * p.tile_tokens;
        const uint32_t t1 = min(limit, t0 + p.tile_tokens);
        const uint32_t n_steps = ceil_div(t1 - t0, kStep);
        const bool single = n_tiles == 1;
        const uint32_t blk0 = dense ? 0 : t0 / p.block_size;
        if (!dense) {
            // block-table entries of the tile (lookups in the loop then cost an LDS read only)
            const uint32_t nblk = (t1 - 1) / p.block_size - blk0 + 1;
            for (uint32_t i = threadIdx.x; i < nblk; i += kNT) {
                tbl_lds[i] = static_cast<uint32_t>(table[blk0 + i]);
            }
        }
        __syncthreads();

        // passes over groups of 128 heads
        for (uint32_t h0 = 0; h0 < p.n_heads; h0 += 32 * kWaves) {
            const uint32_t head = h0 + wave * 32 + col;
            const bool h_ok = head < p.n_heads;
            unsigned char *my_stage = smem + wave * STAGE_BYTES;   // private to the wave outside the loop

            // ---- [q_absorb | qr] of this wave's 32 heads: copied into the wave's stage with the layout of
            // a cache step (head = row), then read as the B operand (column = head, 8 elements per half).
            // Heads past the end repeat the last one; their results are never stored.
            uint4 qreg[KS_C + KS_R];
            {
                const uint32_t st = smem_addr + wave * STAGE_BYTES;
                const uint32_t h_last = p.n_heads - 1;
                const char *qa = reinterpret_cast<const char *>(p.q_absorb) + static_cast<uint64_t>(tok) * p.n_heads * KC_ROWB;
                const char *qq = reinterpret_cast<const char *>(p.qr) + static_cast<uint64_t>(tok) * p.n_heads * PE_ROWB;
                const uint32_t hw = h0 + wave * 32;
                if (hw + 32 <= p.n_heads) {
                    // 32 consecutive heads: 32 KiB and 4 KiB of consecutive memory, four copies per M0 value
                    const uint32_t lv = lane << 4;
#pragma unroll
                    for (int g = 0; g < 8; g++) {
                        dma_4x1k(st + g * 4 * KC_ROWB, lv ^ (swz_kc(4 * g) << 4), lv ^ (swz_kc(4 * g + 1) << 4),
                                 lv ^ (swz_kc(4 * g + 2) << 4), lv ^ (swz_kc(4 * g + 3) << 4),
                                 qa + static_cast<uint64_t>(hw + 4 * g) * KC_ROWB);
                    }
                    // rotary rows 8 i + lane / 8: pattern (4 i + lane / 16) % 8, i.e. the lane's own XOR 4 (i % 2)
                    const uint32_t pv = ((lane >> 3) * PE_ROWB) + (((lane & 7u) ^ ((lane >> 4) & 7u)) << 4);
                    dma_4x1k(st + KC_BYTES, pv, pv ^ (4u << 4), pv, pv ^ (4u << 4), qq + static_cast<uint64_t>(hw) * PE_ROWB);
                } else {
#pragma unroll
                    for (uint32_t row = 0; row < 32; row++) {
                        const uint32_t hr = min(hw + row, h_last);
                        dma_1k(st + row * KC_ROWB, ((lane & ~15u) | ((lane & 15u) ^ swz_kc(row))) << 4, qa + static_cast<uint64_t>(hr) * KC_ROWB);
                    }
#pragma unroll
                    for (uint32_t i = 0; i < 4; i++) {
                        const uint32_t row = i * 8 + (lane >> 3);
                        const uint32_t hr = min(hw + row, h_last);
                        dma_1k(st + KC_BYTES + i * 1024, hr * PE_ROWB + (((lane & 7u) ^ swz_pe(row)) << 4), qq);
                    }
                }
                dma_wait<0>();
#pragma unroll
                for (int ks = 0; ks < KS_C; ks++) {
                    qreg[ks] = *reinterpret_cast<const uint4 *>(my_stage + k_row + ((ks >> 3) << 8) + ((((2 * ks) & 15) << 4) ^ kx));
                }
#pragma unroll
                for (int ks = 0; ks < KS_R; ks++) {
                    qreg[KS_C + ks] = *reinterpret_cast<const uint4 *>(my_stage + p_row + ((((2 * ks) & 7) << 4) ^ px));
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
            __syncthreads();   // every wave holds its Q: the stages may be overwritten

            // ---- cache copies of one step: scalars first, then nine 1 KiB copies per wave ----------------
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
            auto row_xor = [](int i) { return static_cast<uint32_t>(((i & 3) << 6) | ((i >> 2) << 4)); };
            // piece 0, 1: four latent rows each; piece 2: the rotary rows. A step that ends inside the
            // tile's last positions takes the general path (piece 0 issues all nine copies).
            auto copy_piece = [&](const StepCopy &c, int piece) {
                const bool full = c.last_pos == kStep - 1;
                if (full) {
                    if (piece < 2) {
                        const uint32_t r0 = 8 * wave + 4 * piece;
                        dma_4x1k(c.stage + r0 * KC_ROWB, kc_voff ^ row_xor(4 * piece), kc_voff ^ row_xor(4 * piece + 1),
                                 kc_voff ^ row_xor(4 * piece + 2), kc_voff ^ row_xor(4 * piece + 3), c.kb + r0 * KC_ROWB);
                    } else {
                        dma_1k(c.stage + KC_BYTES + wave * 1024, pe_row * PE_ROWB + pe_voff, c.pb);
                    }
                } else if (piece == 0) {
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const uint32_t row = 8 * wave + i;
                        const uint32_t src = min(row, c.last_pos);   // uniform
                        dma_1k(c.stage + row * KC_ROWB, kc_voff ^ row_xor(i), c.kb + src * KC_ROWB);
                    }
                    const uint32_t prow = min(pe_row, c.last_pos);
                    dma_1k(c.stage + KC_BYTES + wave * 1024, prow * PE_ROWB + pe_voff, c.pb);
                }
            };
            auto issue = [&](uint32_t step) {
                const StepCopy c = plan(step);
#pragma unroll
                for (int i = 0; i < 3; i++) {
                    copy_piece(c, i);
                }
            };

            // ---- S^T = K . Q^T of one step: 32 positions x 32 heads; operands are fetched three ahead -----
            // One accumulation chain (a product that accumulates onto the previous result issues every ~44
            // cycles instead of 32) with the operand fetches kAhead products ahead: kAhead x 44 cycles cover
            // the LDS latency, and a second accumulator would cost 16 registers that are not there.
            // ---- S^T = K . Q^T of one step: 32 positions x 32 heads. One accumulation chain (a product that
            // accumulates onto the previous result issues every ~44 cycles instead of 32) with the operand
            // fetches kAhead products ahead.
            auto qk = [&](uint32_t step) {
                // addresses of the latent part: 8 registers (the chunk index of k-step ks is 2 ks ^ x; its low
                // bits select the register, the rest is an immediate)
                const uint32_t soff = (step % kStages) * STAGE_BYTES;
                uint32_t xk[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    xk[j] = soff + k_row + ((j << 5) ^ kx);
                }
                auto rd_k = [&](int ks) {
                    return ks < KS_C ? *reinterpret_cast<const uint4 *>(smem + xk[ks & 7] + ((ks >> 3) << 8))
                                     : *reinterpret_cast<const uint4 *>(smem + soff + p_row + ((((ks - KS_C) & 3) << 5) ^ px));
                };
                f32x16_t S;
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    S[k] = 0.f;
                }
                uint4 a[kAhead];
#pragma unroll
                for (int i = 0; i < kAhead; i++) {
                    a[i] = rd_k(i);
                }
#pragma unroll
                for (int ks = 0; ks < KS_C + KS_R; ks++) {
                    S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[ks % kAhead]),
                                                                __builtin_bit_cast(bf16x8_t, qreg[ks]), S, 0, 0, 0);
                    if (ks + kAhead < KS_C + KS_R) {
                        a[ks % kAhead] = rd_k(ks + kAhead);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                return S;
            };

            // ---- pipeline: copies run three steps ahead of the step being consumed. Every copy is
            // unconditional (steps past the end copy the last step again, same bytes to the same place), so
            // the wait counts are exact.
            const uint32_t last = n_steps - 1;
            issue(0);
            issue(min(1u, last));
            issue(min(2u, last));
            for (uint32_t step = 0; step < n_steps; step++) {
                const uint32_t t = t0 + step * kStep;
                {
                    // the lane index from the hardware, opaque to the compiler: nothing derived from it can be
                    // hoisted out of the loop (and end up in a spill slot, whose reload would wait for every copy)
                    uint32_t ln;
                    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
                    set_roles(ln);
                }
                dma_wait<2 * DMA_PER_WAVE>();   // this wave's share of `step` has landed
                __syncthreads();            // ... and everybody else's; stage (step - 1) % 4 is free

                // ---- scores, then the online softmax. Register k holds position t + 8 (k / 4) + 4 half +
                // k % 4. The reference maximum only moves when the step maximum exceeds it by more than
                // 2^8: probabilities then stay below 2^8 (the same relative precision in bf16, and the
                // normaliser shares the reference), and the accumulators are rescaled rarely.
                f32x16_t S = qk(step);
                const uint32_t lane_pos = t + half4;
                float mx = -INFINITY;
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    S[k] *= p.scale_log2e;
                }
                if (t + kStep > t1) {   // uniform: only a tile's last step has positions to mask
#pragma unroll
                    for (int k = 0; k < 16; k++) {
                        const uint32_t pos = lane_pos + (k / 4) * 8 + (k % 4);
                        S[k] = pos < t1 ? S[k] : -INFINITY;
                    }
                }
#pragma unroll
                for (int k = 0; k < 16; k++) {
                    mx = fmaxf(mx, S[k]);
                }
                {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
                    mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                const float m_new = mx > m_run + kRescaleSlack ? mx : m_run;
                const float m_safe = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m_run - m_safe);
                m_run = m_new;
                uint32_t pw[8];
                float psum = 0.f;
#pragma unroll
                for (int k = 0; k < 16; k += 2) {
                    const float e0 = fast_exp2(S[k] - m_safe);
                    const float e1 = fast_exp2(S[k + 1] - m_safe);
                    psum += e0 + e1;
                    pw[k / 2] = BF16::pack(e0, e1);
                }
                l_run = l_run * alpha + psum;

                if (__any(alpha != 1.0f)) {
                    // the accumulators live in the accumulation registers, which the vector ALU cannot
                    // multiply in place: one element at a time through a temporary. The waits cover the
                    // distance the hardware wants between a matrix instruction and a read of its result
                    // (and between the write-back and the next matrix instruction).
                    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" ::: "memory");
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
#pragma unroll
                        for (int k = 0; k < 16; k++) {
                            float tmp;
                            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                                         : "+a"(O[dt][k]), "=&v"(tmp) : "v"(alpha));
                        }
                    }
                    asm volatile("s_nop 7" ::: "memory");
                }

                // ---- O^T += kc^T . P^T: 16 tiles of 32 latent columns, two k-steps of 16 positions; the
                // transposed operands of the next tile are fetched before this tile's products, and the
                // copies of step + 3 are issued in between
                {
                    const StepCopy c = plan(min(step + 3, last));
                    const uint4 pb0 = make_uint4(pw[0], pw[1], pw[2], pw[3]);
                    const uint4 pb1 = make_uint4(pw[4], pw[5], pw[6], pw[7]);
                    typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
                    uint32_t xv[4][2];
                    {
                        const uint32_t soff = (step % kStages) * STAGE_BYTES;
#pragma unroll
                        for (int a = 0; a < 4; a++) {
#pragma unroll
                            for (int rd = 0; rd < 2; rd++) {
                                xv[a][rd] = soff + (vr_off ^ ((a << 6) | (rd << 5)));
                            }
                        }
                    }
                    auto rd_v = [&](int dt, int kk, int rd) {
                        unsigned char *ptr = smem + xv[dt & 3][rd] + ((dt >> 2) << 8) + kk * 16 * KC_ROWB + rd * 8 * KC_ROWB;
                        return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)ptr));
                    };
                    constexpr int VB = 3;   // operand buffers: the fetches run two tiles ahead of the products
                    uint2 v[VB][4];
#pragma unroll
                    for (int d = 0; d < VB - 1; d++) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            v[d][j] = rd_v(d, j >> 1, j & 1);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    uint2 carry[2];
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        if (dt + VB - 1 < DT) {
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                v[(dt + VB - 1) % VB][j] = rd_v(dt + VB - 1, j >> 1, j & 1);
                            }
                        }
                        const uint2 *x = v[dt % VB];
                        O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(bf16x8_t, make_uint4(x[0].x, x[0].y, x[1].x, x[1].y)),
                            __builtin_bit_cast(bf16x8_t, pb0), O[dt], 0, 0, 0);
                        if (dt > 0) {
                            O[dt - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(bf16x8_t, make_uint4(carry[0].x, carry[0].y, carry[1].x, carry[1].y)),
                                __builtin_bit_cast(bf16x8_t, pb1), O[dt - 1], 0, 0, 0);
                        }
                        carry[0] = x[2];
                        carry[1] = x[3];
                        if (dt % 5 == 0 && dt < 15) {
                            copy_piece(c, dt / 5);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    O[DT - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8_t, make_uint4(carry[0].x, carry[0].y, carry[1].x, carry[1].y)),
                        __builtin_bit_cast(bf16x8_t, pb1), O[DT - 1], 0, 0, 0);
                }
            }
            dma_wait<0>();
            __syncthreads();   // nothing in flight, nobody reading: the ring can be reused

            // ---- results: O^T lane layout is column = head, register k of tile dt = latent
            // 32 dt + 8 (k / 4) + 4 half + k % 4. Transposed through the wave's stage, 256 latent columns at a
            // time, so that every store instruction writes one head's contiguous row segment.
            const float l_tot = l_run + __shfl_xor(l_run, 32);
            const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
            constexpr int TR_ROWB = 256 * 4 + 16;
            const uint32_t heads_here = min(32u, p.n_heads > h0 + wave * 32 ? p.n_heads - (h0 + wave * 32) : 0u);
            const uint64_t rh0 = static_cast<uint64_t>(tok) * p.n_heads + h0 + wave * 32;
#pragma unroll
            for (int ch = 0; ch < 2; ch++) {
#pragma unroll
                for (int d8 = 0; d8 < 8; d8++) {
                    const int dt = ch * 8 + d8;
#pragma unroll
                    for (int kg = 0; kg < 4; kg++) {
                        const float sc = inv;   // partials are stored normalised too
                        *reinterpret_cast<float4 *>(my_stage + col * TR_ROWB + (d8 * 32 + kg * 8 + half * 4) * 4) =
                            make_float4(O[dt][kg * 4] * sc, O[dt][kg * 4 + 1] * sc, O[dt][kg * 4 + 2] * sc, O[dt][kg * 4 + 3] * sc);
                    }
                }
                // wave-private region: the LDS counter wait the compiler inserts is all the ordering needed
                for (uint32_t hr = 0; hr < heads_here; hr++) {
                    const float4 x = *reinterpret_cast<const float4 *>(my_stage + hr * TR_ROWB + lane * 16);
                    uint2 o;
                    o.x = BF16::pack(x.x, x.y);
                    o.y = BF16::pack(x.z, x.w);
                    uint16_t *dst = single ? p.out + (rh0 + hr) * C
                                           : reinterpret_cast<uint16_t *>(p.part_acc) + ((rh0 + hr) * p.max_slots + tile) * C;
                    *reinterpret_cast<uint2 *>(dst + ch * 256 + lane * 4) = o;
                }
            }
            if (h_ok && half == 0) {
                const uint64_t rh = rh0 + col;
                if (!single) {
                    *reinterpret_cast<float2 *>(p.part_ml + (rh * p.max_slots + tile) * 2) = make_float2(m_run, l_tot);
                }
                if (tile == 0 && p.part_cnt != nullptr) {
                    p.part_cnt[rh] = single ? 0 : static_cast<int32_t>(n_tiles);
                }
            }
            __syncthreads();   // the stages are reused by the next pass
        }
    }
}

}  // namespace

bool mla_decode_supported(const MlaArgs &a)
{
    const bool dense = a.block_tables == nullptr;
    return a.total_tokens == a.batch && a.kv_lora_rank == C && a.rope_head_dim == R && a.top_k == 0 &&
           (dense || a.block_size % kStep == 0);
}

void mla_decode_plan(const MlaArgs &a, uint32_t *tile_tokens, uint32_t *max_slots)
{
    const bool dense = a.block_tables == nullptr;
    const uint64_t max_ctx = dense ? a.dense_len : static_cast<uint64_t>(a.max_num_blocks) * a.block_size;
    // about one workgroup per compute unit if every sequence were as long as allowed; tiles between
    // 256 and 1024 positions
    uint64_t tile = max_ctx * a.batch / 256;
    tile = tile > 1024 ? 1024 : (tile < 256 ? 256 : tile);
    tile = (tile + kStep - 1) / kStep * kStep;
    *tile_tokens = static_cast<uint32_t>(tile);
    *max_slots = static_cast<uint32_t>((max_ctx + tile - 1) / tile);
}

size_t mla_decode_workspace_bytes(const MlaArgs &a)
{
    uint32_t tile, max_slots;
    mla_decode_plan(a, &tile, &max_slots);
    return max_slots > 1 ? partial_bytes(a.total_tokens, a.n_heads, C, max_slots) : 0;
}

int launch_mla_decode(hipStream_t stream, const MlaArgs &a)
{
    uint32_t tile, max_slots;
    mla_decode_plan(a, &tile, &max_slots);
    const size_t need = mla_decode_workspace_bytes(a);
    if (max_slots > 1 && (a.workspace == nullptr || a.workspace_bytes < need)) {
        return fail(XLITE_HIP_ENOSPC, __func__, "workspace too small: need " + std::to_string(need) +
                                                    " bytes, have " + std::to_string(a.workspace_bytes));
    }
    const PartialBuffers pb = max_slots > 1 ? carve_partials(a.workspace, a.total_tokens, a.n_heads, C, max_slots)
                                            : PartialBuffers{};
    MlaDecodeParams p{};
    p.q_absorb = static_cast<const uint16_t *>(a.q_absorb);
    p.qr = static_cast<const uint16_t *>(a.qr);
    p.k_cache = static_cast<const uint16_t *>(a.k_cache);
    p.pe_cache = static_cast<const uint16_t *>(a.pe_cache);
    p.out = static_cast<uint16_t *>(a.o_absorb);
    p.query_start_loc = a.query_start_loc;
    p.lens = a.lens;
    p.cached_lens = a.cached_lens;
    p.block_tables = a.block_tables;
    p.part_cnt = pb.cnt;
    p.part_acc = pb.acc;
    p.part_ml = pb.ml;
    p.n_heads = a.n_heads;
    p.block_size = a.block_size;
    p.max_num_blocks = a.max_num_blocks;
    p.dense_len = a.dense_len;
    p.tile_tokens = tile;
    p.max_slots = max_slots;
    p.scale_log2e = a.scale * kLog2e;

    const size_t lds = static_cast<size_t>(kStages) * STAGE_BYTES + (tile / 16 + 2) * sizeof(uint32_t);
    static bool configured = false;
    if (!configured) {
        XL_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(mla_decode_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        configured = true;
    }
    dim3 grid(max_slots, a.batch, 1);
    mla_decode_kernel<<<grid, kNT, lds, stream>>>(p);
    XL_LAUNCH_CHECK();
    if (max_slots == 1) {
        return XLITE_HIP_OK;
    }
    return launch_merge_norm16(stream, a.dtype, a.o_absorb, pb, a.total_tokens, a.n_heads, C, max_slots);
}

}  // namespace xlite
