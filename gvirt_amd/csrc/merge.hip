// Merge of split-KV partial results: out[row][head] = sum_s w_s O_s / sum_s w_s l_s with
// w_s = 2^(m_s - max_s m_s) (maxima are kept in the log2 domain). A separate launch instead of a
// "last workgroup to finish merges" scheme: the device-scope fences the latter needs write back
// and invalidate the L2 of every XCD once per workgroup, which costs far more than this kernel.
// The algebra is the online-softmax update of the reference
// (xlite/csrc/kernels/softmax_attn_aiv.h:595-647), applied once over fp32 partials.
#include "attention_common.h"

namespace xlite {

namespace {

// A wave owns one (row, head): lane s computes the weight and the weighted sum of slot s, then the slots'
// rows (four columns per lane) are read four at a time so that several loads are in flight per lane.
template <typename T>
__global__ void __launch_bounds__(256)
merge_kernel(uint16_t *__restrict__ out, const float *__restrict__ part_acc,
             const float *__restrict__ part_ml, const int32_t *__restrict__ part_cnt, uint32_t total_rh,
             uint32_t dv, uint32_t max_slots)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t rh = static_cast<uint64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (rh >= total_rh) {
        return;
    }
    const uint64_t base = rh * max_slots;
    // the count, the first maxima and the first rows are fetched together (one round trip to memory instead
    // of three); what lies beyond the count is discarded unseen
    const float2 ml_first = *reinterpret_cast<const float2 *>(part_ml + (base + min(lane, max_slots - 1)) * 2);
    const uint32_t n = static_cast<uint32_t>(part_cnt[rh]);
    if (n == 0) {
        return;  // the producer wrote the final value itself
    }
    float mm = lane < n ? ml_first.x : -INFINITY;
    for (uint32_t s = lane + 64; s < n; s += 64) {
        mm = fmaxf(mm, part_ml[(base + s) * 2]);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        mm = fmaxf(mm, __shfl_xor(mm, d));
    }
    const float ms = mm == -INFINITY ? 0.f : mm;
    for (uint32_t c0 = 0; c0 < dv / 4; c0 += 64) {
        const uint32_t c = c0 + lane;
        const bool c_ok = c < dv / 4;   // idle lanes still take part in the exchanges
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        float lsum = 0.f;
        for (uint32_t s0 = 0; s0 < n; s0 += 64) {
            const uint32_t cnt = min(64u, n - s0);
            float w_lane = 0.f, l_lane = 0.f;
            if (lane < cnt) {
                const float2 ml = s0 == 0 ? ml_first : *reinterpret_cast<const float2 *>(part_ml + (base + s0 + lane) * 2);
                w_lane = fast_exp2(ml.x - ms);
                l_lane = ml.y * w_lane;
            }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                l_lane += __shfl_xor(l_lane, d);
            }
            lsum += l_lane;
            for (uint32_t j = 0; j < cnt; j += 4) {
                float4 x[4];
                float w[4];
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    const uint32_t idx = min(j + u, cnt - 1);
                    x[u] = c_ok ? *reinterpret_cast<const float4 *>(part_acc + (base + s0 + idx) * dv + c * 4)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
                    w[u] = j + u < cnt ? __shfl(w_lane, static_cast<int>(j + u)) : 0.f;
                }
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    acc.x += x[u].x * w[u];
                    acc.y += x[u].y * w[u];
                    acc.z += x[u].z * w[u];
                    acc.w += x[u].w * w[u];
                }
            }
        }
        if (c_ok) {
            const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
            uint2 o;
            o.x = T::pack(acc.x * inv, acc.y * inv);
            o.y = T::pack(acc.z * inv, acc.w * inv);
            *reinterpret_cast<uint2 *>(out + rh * dv + c * 4) = o;
        }
    }
}

constexpr uint64_t kMergeWideBelow = 512;   // (row, head)s up to which four waves share one

// The merge of the MLA decode kernel's partials: O is stored normalised (O_s / l_s) in 16 bits,
// out = sum_s (w_s l_s) Ohat_s / sum_s (w_s l_s). A row's segments sit in per-chunk slots: meta[row] =
// (segments n, first chunk c0, first-in-chunk flag f); segment 0 is slot 2 c0 + (1 - f), segment s slot
// 2 (c0 + s). A wave owns one (row, head): lane s computes the weight of segment s, then the segments' rows
// (eight columns per lane) are read four at a time so that several loads are in flight per lane.
// With few (row, head)s WPR = 4 waves share one, each summing every fourth segment, and add up through LDS.
template <typename T, int WPR>
__global__ void __launch_bounds__(256)
merge_mla_kernel(uint16_t *__restrict__ out, const uint16_t *__restrict__ part_acc, const float *__restrict__ part_ml,
                 const int4 *__restrict__ meta, uint32_t rows, uint32_t n_heads, uint32_t dv)
{
    __shared__ float xch[WPR > 1 ? (WPR - 1) * 9 * 64 : 1];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t stream = wave % WPR;
    const uint64_t rh = static_cast<uint64_t>(blockIdx.x) * (4 / WPR) + wave / WPR;
    if (rh >= static_cast<uint64_t>(rows) * n_heads) {
        return;   // WPR is 1 (no barrier below) or 4 (the whole workgroup leaves together)
    }
    const uint32_t row = static_cast<uint32_t>(rh / n_heads), head = static_cast<uint32_t>(rh % n_heads);
    const int4 mt = meta[row];
    const uint32_t n = static_cast<uint32_t>(mt.x);
    if (n == 0) {
        return;  // the producer wrote the final value itself
    }
    const uint32_t c0 = static_cast<uint32_t>(mt.y), first_flag = static_cast<uint32_t>(mt.z);
    auto slot_of = [&](uint32_t s) -> uint64_t {
        const uint32_t ps = s == 0 ? 2 * c0 + (1 - first_flag) : 2 * (c0 + s);
        return static_cast<uint64_t>(ps) * n_heads + head;
    };
    if (n <= 64 && dv <= 512) {
        // The common case in one round trip after the meta entry: lane s fetches (maximum, sum) of segment s and, without
        // waiting for it, the first four segments' rows; the weights are worked out while those are on their way.
        // (The general loop below waits for the maxima, then for the sums, then for every round of rows in turn.)
        const uint32_t c = lane;
        const bool c_ok = c < dv / 8;
        auto load_round = [&](uint32_t j, uint4 (&x)[4]) {
#pragma unroll
            for (uint32_t u = 0; u < 4; u++) {
                const uint32_t idx = min(j + u * WPR + stream, n - 1);
                x[u] = c_ok ? *reinterpret_cast<const uint4 *>(part_acc + slot_of(idx) * dv + c * 8) : make_uint4(0, 0, 0, 0);
            }
        };
        const float2 ml = *reinterpret_cast<const float2 *>(part_ml + slot_of(min(lane, n - 1)) * 2);
        uint4 x[4];
        load_round(0, x);
        float mm = lane < n ? ml.x : -INFINITY;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mm = fmaxf(mm, __shfl_xor(mm, d));
        }
        const float ms = mm == -INFINITY ? 0.f : mm;
        const float w_lane = lane < n ? fast_exp2(ml.x - ms) * ml.y : 0.f;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float wsum = 0.f;
        for (uint32_t j = 0; j < n; j += 4 * WPR) {
            if (j > 0) {
                load_round(j, x);
            }
#pragma unroll
            for (uint32_t u = 0; u < 4; u++) {
                const uint32_t want = j + u * WPR + stream;
                float w = __shfl(w_lane, static_cast<int>(min(want, n - 1)));
                w = want < n ? w : 0.f;
                const uint32_t xs[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
                wsum += w;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    acc[2 * k] += T::lo(xs[k]) * w;
                    acc[2 * k + 1] += T::hi(xs[k]) * w;
                }
            }
        }
        if constexpr (WPR > 1) {
            if (wave != 0) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    xch[((wave - 1) * 9 + k) * 64 + lane] = acc[k];
                }
                xch[((wave - 1) * 9 + 8) * 64 + lane] = wsum;
            }
            __syncthreads();
            if (wave != 0) {
                return;
            }
            for (uint32_t w = 0; w + 1 < WPR; w++) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    acc[k] += xch[(w * 9 + k) * 64 + lane];
                }
                wsum += xch[(w * 9 + 8) * 64 + lane];
            }
        }
        const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
        if (c_ok) {
            uint4 o;
            o.x = T::pack(acc[0] * inv, acc[1] * inv);
            o.y = T::pack(acc[2] * inv, acc[3] * inv);
            o.z = T::pack(acc[4] * inv, acc[5] * inv);
            o.w = T::pack(acc[6] * inv, acc[7] * inv);
            *reinterpret_cast<uint4 *>(out + rh * dv + c * 8) = o;
        }
        return;
    }
    float mm = -INFINITY;
    for (uint32_t s = lane; s < n; s += 64) {
        mm = fmaxf(mm, part_ml[slot_of(s) * 2]);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        mm = fmaxf(mm, __shfl_xor(mm, d));
    }
    const float ms = mm == -INFINITY ? 0.f : mm;
    for (uint32_t cc = 0; cc < dv / 8; cc += 64) {
        const uint32_t c = cc + lane;
        const bool c_ok = c < dv / 8;   // idle lanes still take part in the exchanges
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float wsum = 0.f;
        for (uint32_t s0 = 0; s0 < n; s0 += 64) {
            const uint32_t cnt = min(64u, n - s0);
            float w_lane = 0.f;
            if (lane < cnt) {
                const float2 ml = *reinterpret_cast<const float2 *>(part_ml + slot_of(s0 + lane) * 2);
                w_lane = fast_exp2(ml.x - ms) * ml.y;
            }
            for (uint32_t j = 0; j < cnt; j += 4 * WPR) {
                uint4 x[4];
                float w[4];
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    const uint32_t want = j + u * WPR + stream;
                    const uint32_t idx = min(want, cnt - 1);
                    x[u] = c_ok ? *reinterpret_cast<const uint4 *>(part_acc + slot_of(s0 + idx) * dv + c * 8)
                                : make_uint4(0, 0, 0, 0);
                    w[u] = __shfl(w_lane, static_cast<int>(idx));
                    w[u] = want < cnt ? w[u] : 0.f;
                }
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    const uint32_t xs[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
                    wsum += w[u];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        acc[2 * k] += T::lo(xs[k]) * w[u];
                        acc[2 * k + 1] += T::hi(xs[k]) * w[u];
                    }
                }
            }
        }
        if constexpr (WPR > 1) {
            // one column pass at most: the waves of a (row, head) meet at the barrier the same number of times
            if (wave != 0) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    xch[((wave - 1) * 9 + k) * 64 + lane] = acc[k];
                }
                xch[((wave - 1) * 9 + 8) * 64 + lane] = wsum;
            }
            __syncthreads();
            if (wave != 0) {
                return;
            }
            for (uint32_t w = 0; w + 1 < WPR; w++) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    acc[k] += xch[(w * 9 + k) * 64 + lane];
                }
                wsum += xch[(w * 9 + 8) * 64 + lane];
            }
        }
        const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
        uint4 o;
        o.x = T::pack(acc[0] * inv, acc[1] * inv);
        o.y = T::pack(acc[2] * inv, acc[3] * inv);
        o.z = T::pack(acc[4] * inv, acc[5] * inv);
        o.w = T::pack(acc[6] * inv, acc[7] * inv);
        if (c_ok) {
            *reinterpret_cast<uint4 *>(out + rh * dv + c * 8) = o;
        }
    }
}

// The balanced GQA decode kernel's partials: fp32 (O, maximum in the log2 domain, normaliser) in the same
// per-chunk slots as above, [slot][head][dv]. A lane owns four columns, so a (row, head) needs dv / 4 lanes
// and a wave runs 64 / (dv / 4) slots side by side; WPR waves share a (row, head) when there are few of
// them and many slots each (a long sequence alone in its batch), and add their sums up through LDS.
template <typename T, int WPR>
__global__ void __launch_bounds__(256)
merge_meta_kernel(uint16_t *__restrict__ out, const float *__restrict__ part_acc, const float *__restrict__ part_ml,
                  const int4 *__restrict__ meta, uint32_t rows, uint32_t n_heads, uint32_t dv)
{
    __shared__ float4 xch[WPR > 1 ? (WPR - 1) * 64 : 1];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t rh = static_cast<uint64_t>(blockIdx.x) * (4 / WPR) + wave / WPR;
    if (rh >= static_cast<uint64_t>(rows) * n_heads) {
        return;   // WPR is 1 (no barrier below) or 4 (the whole workgroup leaves together)
    }
    const uint32_t row = static_cast<uint32_t>(rh / n_heads), head = static_cast<uint32_t>(rh % n_heads);
    const int4 mt = meta[row];
    const uint32_t n = static_cast<uint32_t>(mt.x);
    if (n == 0) {
        return;  // the producer wrote the final value itself
    }
    const uint32_t c0 = static_cast<uint32_t>(mt.y), first_flag = static_cast<uint32_t>(mt.z);
    auto slot_of = [&](uint32_t s) -> uint64_t {
        const uint32_t ps = s == 0 ? 2 * c0 + (1 - first_flag) : 2 * (c0 + s);
        return static_cast<uint64_t>(ps) * n_heads + head;
    };
    const uint32_t lanes_per = dv / 4;                 // 16, 32 or 64
    const uint32_t c = lane % lanes_per;
    const uint32_t streams = 64 / lanes_per * WPR;     // slots summed side by side
    const uint32_t stream = (wave % WPR) * (64 / lanes_per) + lane / lanes_per;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float lsum = 0.f;
    float ms = 0.f;
    if (n <= 64) {
        // The common case in one round trip after the meta entry: lane s fetches (maximum, normaliser) of slot s and,
        // without waiting for it, the first round of rows; the weights are worked out while those are on their way.
        auto load_round = [&](uint32_t j, float4 (&x)[4]) {
#pragma unroll
            for (uint32_t u = 0; u < 4; u++) {
                const uint32_t safe = min(j + u * streams + stream, n - 1);
                x[u] = *reinterpret_cast<const float4 *>(part_acc + slot_of(safe) * dv + c * 4);
            }
        };
        const float2 ml = *reinterpret_cast<const float2 *>(part_ml + slot_of(min(lane, n - 1)) * 2);
        float4 x[4];
        load_round(0, x);
        float mm = lane < n ? ml.x : -INFINITY;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mm = fmaxf(mm, __shfl_xor(mm, d));
        }
        ms = mm == -INFINITY ? 0.f : mm;
        const float w_lane = lane < n ? fast_exp2(ml.x - ms) : 0.f;
        float l_lane = lane < n ? ml.y * w_lane : 0.f;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            l_lane += __shfl_xor(l_lane, d);
        }
        lsum = l_lane;
        for (uint32_t j = 0; j < n; j += 4 * streams) {   // uniform trip count: every lane takes part in the exchanges
            if (j > 0) {
                load_round(j, x);
            }
#pragma unroll
            for (uint32_t u = 0; u < 4; u++) {
                const uint32_t idx = j + u * streams + stream;
                float w = __shfl(w_lane, static_cast<int>(min(idx, n - 1)));
                w = idx < n ? w : 0.f;
                acc.x += x[u].x * w;
                acc.y += x[u].y * w;
                acc.z += x[u].z * w;
                acc.w += x[u].w * w;
            }
        }
    } else {
        float mm = -INFINITY;
        for (uint32_t s = lane; s < n; s += 64) {
            mm = fmaxf(mm, part_ml[slot_of(s) * 2]);
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mm = fmaxf(mm, __shfl_xor(mm, d));
        }
        ms = mm == -INFINITY ? 0.f : mm;
        for (uint32_t s0 = 0; s0 < n; s0 += 64) {
            const uint32_t cnt = min(64u, n - s0);
            float w_lane = 0.f, l_lane = 0.f;
            if (lane < cnt) {
                const float2 ml = *reinterpret_cast<const float2 *>(part_ml + slot_of(s0 + lane) * 2);
                w_lane = fast_exp2(ml.x - ms);
                l_lane = ml.y * w_lane;
            }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                l_lane += __shfl_xor(l_lane, d);
            }
            lsum += l_lane;
            for (uint32_t j = 0; j < cnt; j += 4 * streams) {   // uniform trip count: every lane takes part in the exchanges
                float4 x[4];
                float w[4];
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    const uint32_t idx = j + u * streams + stream;
                    const uint32_t safe = min(idx, cnt - 1);
                    x[u] = *reinterpret_cast<const float4 *>(part_acc + slot_of(s0 + safe) * dv + c * 4);
                    w[u] = __shfl(w_lane, static_cast<int>(safe));
                    w[u] = idx < cnt ? w[u] : 0.f;
                }
#pragma unroll
                for (uint32_t u = 0; u < 4; u++) {
                    acc.x += x[u].x * w[u];
                    acc.y += x[u].y * w[u];
                    acc.z += x[u].z * w[u];
                    acc.w += x[u].w * w[u];
                }
            }
        }
    }
    for (uint32_t d = 32; d >= lanes_per; d >>= 1) {
        acc.x += __shfl_xor(acc.x, static_cast<int>(d));
        acc.y += __shfl_xor(acc.y, static_cast<int>(d));
        acc.z += __shfl_xor(acc.z, static_cast<int>(d));
        acc.w += __shfl_xor(acc.w, static_cast<int>(d));
    }
    if constexpr (WPR > 1) {
        if (wave != 0) {
            xch[(wave - 1) * 64 + lane] = acc;
        }
        __syncthreads();
        if (wave != 0) {
            return;
        }
        for (uint32_t w = 0; w + 1 < WPR; w++) {
            const float4 o = xch[w * 64 + lane];
            acc.x += o.x;
            acc.y += o.y;
            acc.z += o.z;
            acc.w += o.w;
        }
    }
    if (lane < lanes_per) {
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
        uint2 o;
        o.x = T::pack(acc.x * inv, acc.y * inv);
        o.y = T::pack(acc.z * inv, acc.w * inv);
        *reinterpret_cast<uint2 *>(out + rh * dv + c * 4) = o;
    }
}

}  // namespace

size_t partial_bytes(uint32_t rows, uint32_t n_heads, uint32_t dv, uint32_t max_slots)
{
    const size_t rh = static_cast<size_t>(rows) * n_heads;
    return ((rh * sizeof(int32_t) + 255) / 256) * 256 + rh * max_slots * (dv + 2) * sizeof(float);
}

PartialBuffers carve_partials(void *workspace, uint32_t rows, uint32_t n_heads, uint32_t dv, uint32_t max_slots)
{
    PartialBuffers b{};
    if (workspace == nullptr) {
        return b;
    }
    const size_t rh = static_cast<size_t>(rows) * n_heads;
    char *ws = static_cast<char *>(workspace);
    b.cnt = reinterpret_cast<int32_t *>(ws);
    b.acc = reinterpret_cast<float *>(ws + ((rh * sizeof(int32_t) + 255) / 256) * 256);
    b.ml = b.acc + rh * max_slots * dv;
    return b;
}

int launch_merge(hipStream_t stream, int dtype, void *out, const PartialBuffers &b, uint32_t rows,
                 uint32_t n_heads, uint32_t dv, uint32_t max_slots)
{
    if (rows == 0) {
        return XLITE_HIP_OK;
    }
    // one wave per (row, head), four per workgroup
    const uint32_t total_rh = rows * n_heads;
    const dim3 grid(ceil_div(total_rh, 4u), 1, 1);
    if (dtype == XLITE_HIP_BF16) {
        merge_kernel<BF16><<<grid, 256, 0, stream>>>(static_cast<uint16_t *>(out), b.acc, b.ml, b.cnt, total_rh, dv, max_slots);
    } else {
        merge_kernel<FP16><<<grid, 256, 0, stream>>>(static_cast<uint16_t *>(out), b.acc, b.ml, b.cnt, total_rh, dv, max_slots);
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

int launch_merge_mla(hipStream_t stream, int dtype, void *out, const uint16_t *acc, const float *ml, const int32_t *meta,
                     uint32_t rows, uint32_t n_heads, uint32_t dv)
{
    if (rows == 0) {
        return XLITE_HIP_OK;
    }
    const uint64_t total_rh = static_cast<uint64_t>(rows) * n_heads;
    const int4 *m4 = reinterpret_cast<const int4 *>(meta);
    uint16_t *o = static_cast<uint16_t *>(out);
    const bool bf = dtype == XLITE_HIP_BF16;
    if (total_rh <= kMergeWideBelow && dv <= 512) {   // few (row, head)s: a workgroup each
        const dim3 grid(static_cast<uint32_t>(total_rh), 1, 1);
        if (bf) {
            merge_mla_kernel<BF16, 4><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        } else {
            merge_mla_kernel<FP16, 4><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        }
    } else {
        const dim3 grid(static_cast<uint32_t>((total_rh + 3) / 4), 1, 1);
        if (bf) {
            merge_mla_kernel<BF16, 1><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        } else {
            merge_mla_kernel<FP16, 1><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        }
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

int launch_merge_meta(hipStream_t stream, int dtype, void *out, const float *acc, const float *ml, const int32_t *meta,
                      uint32_t rows, uint32_t n_heads, uint32_t dv)
{
    if (rows == 0) {
        return XLITE_HIP_OK;
    }
    if (dv != 64 && dv != 128 && dv != 256) {
        return fail(XLITE_HIP_EINVAL, __func__, "value width " + std::to_string(dv) + " is none of 64, 128, 256");
    }
    const uint64_t total_rh = static_cast<uint64_t>(rows) * n_heads;
    const int4 *m4 = reinterpret_cast<const int4 *>(meta);
    uint16_t *o = static_cast<uint16_t *>(out);
    const bool bf = dtype == XLITE_HIP_BF16;
    if (total_rh <= kMergeWideBelow) {   // few (row, head)s: a workgroup each
        const dim3 grid(static_cast<uint32_t>(total_rh), 1, 1);
        if (bf) {
            merge_meta_kernel<BF16, 4><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        } else {
            merge_meta_kernel<FP16, 4><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        }
    } else {
        const dim3 grid(static_cast<uint32_t>((total_rh + 3) / 4), 1, 1);
        if (bf) {
            merge_meta_kernel<BF16, 1><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        } else {
            merge_meta_kernel<FP16, 1><<<grid, 256, 0, stream>>>(o, acc, ml, m4, rows, n_heads, dv);
        }
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

}  // namespace xlite
