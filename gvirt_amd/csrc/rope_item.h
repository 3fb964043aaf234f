// One item of rope_and_cache, shared by the stand-alone kernel (cache_ops.hip) and by the decode kernel that
// rotates and stores a step's rows itself (decode_mfma.hip).
#pragma once

#include "common.h"

namespace xlite {

union Vec16 {
    uint4 v;
    uint16_t h[8];
    uint32_t w[4];
};

// One chunk pair of a q or k head: elements e0 .. e0+7 of the rotary span's first half (`a`) with their partners
// in the second half (`b`), rotated in place; q is then scaled. Rounding follows calc_cossin_cast
// (xlite/csrc/kernels/rope_and_cache.h:93-129): each product is rounded to the storage type, the difference /
// sum is formed in fp32 and rounded again; the q scale is applied in fp32 and rounded once more (:576-586).
template <typename T>
__device__ __forceinline__ void rotate_chunk_pair(Vec16 &a, Vec16 &b, uint32_t e0, uint32_t half, uint32_t t, int64_t pos_t,
                                                  uint32_t num_tokens, uint32_t rot_dim, const int64_t *position,
                                                  const uint16_t *cosin, uint64_t mask_h, uint64_t mask_w, bool is_q,
                                                  float q_scale)
{
    Vec16 c, s;
    if ((mask_h | mask_w) == 0) {
        const uint16_t *cs = cosin + static_cast<uint64_t>(pos_t) * rot_dim;
        c.v = *reinterpret_cast<const uint4 *>(cs + e0);
        s.v = *reinterpret_cast<const uint4 *>(cs + half + e0);
    } else {
        // lane j of the rotary half takes its angle from the height / width position
        // when bit j of the matching mask is set, else from the temporal position
        const uint16_t *cs_t = cosin + static_cast<uint64_t>(pos_t) * rot_dim;
        const uint16_t *cs_h = cosin + static_cast<uint64_t>(position[num_tokens + t]) * rot_dim;
        const uint16_t *cs_w = cosin + static_cast<uint64_t>(position[2ull * num_tokens + t]) * rot_dim;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t lane = e0 + j;
            const uint16_t *src = ((mask_h >> lane) & 1) ? cs_h : ((mask_w >> lane) & 1) ? cs_w : cs_t;
            c.h[j] = src[lane];
            s.h[j] = src[half + lane];
        }
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float x1 = T::to_f32(a.h[j]), x2 = T::to_f32(b.h[j]);
        const float cc = T::to_f32(c.h[j]), ss = T::to_f32(s.h[j]);
        const float p1 = T::to_f32(T::from_f32(x1 * cc));
        const float p2 = T::to_f32(T::from_f32(x2 * ss));
        const float p3 = T::to_f32(T::from_f32(x2 * cc));
        const float p4 = T::to_f32(T::from_f32(x1 * ss));
        uint16_t o1 = T::from_f32(p1 - p2);
        uint16_t o2 = T::from_f32(p3 + p4);
        if (is_q) {
            o1 = T::from_f32(T::to_f32(o1) * q_scale);
            o2 = T::from_f32(T::to_f32(o2) * q_scale);
        }
        a.h[j] = o1;
        b.h[j] = o2;
    }
}

// The tensors and sizes of a rope_and_cache call.
struct RopeArgs {
    uint16_t *inout;
    uint16_t *k_cache;             // nullptr: no 16-bit caches (the caller quantises the rows afterwards)
    uint16_t *v_cache;
    const int64_t *position;
    const uint16_t *cosin;
    const int32_t *slot_mapping;
    uint32_t num_tokens, n_heads, n_kv_heads, head_dim, rot_dim, block_size;
    float q_scale;
    uint64_t mask_h, mask_w;
};

// cache_ops.hip: checks the arguments of a rope_and_cache call (its errors are that call's) and gathers them
int rope_prepare(void *inout, void *k_cache, void *v_cache, const int64_t *position, const void *cosin,
                 const int32_t *slot_mapping, uint32_t num_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                 uint32_t head_dim, uint32_t rot_dim, uint32_t block_size, int is_neox, uint64_t mrope_mask_h,
                 uint64_t mrope_mask_w, int dtype, bool with_cache, RopeArgs *out);

// Items of a token: (head slot, chunk pair of the rotary span or pass-through chunk behind it).
__device__ __forceinline__ uint32_t rope_items_per_token(const RopeArgs &r)
{
    return (r.n_heads + 2 * r.n_kv_heads) * (r.head_dim / 8 - r.rot_dim / 16);
}

// Item `rem` of token `t`: a thread rotates 8 elements of the first half of the rotary span together with their 8
// partners in the second half (both are written in place, so one thread must own both), or copies / scales one
// pass-through chunk; k and v rows also go to the token's cache slot. In two parts, so that a caller can have the
// item's loads in flight while it finds out whether `t` is the token it wants.
struct RopeItemRegs {
    Vec16 a, b;        // the chunk (pair) of the row
    int64_t pos_t;     // the token's position and cache slot
    uint32_t slot;
};

__device__ __forceinline__ RopeItemRegs rope_item_load(const RopeArgs &r, uint32_t t, uint32_t rem)
{
    const uint32_t rot_pairs = r.rot_dim / 16;    // chunk pairs inside the rotary span
    const uint32_t items_per_head = r.head_dim / 8 - rot_pairs;
    const uint32_t hs = rem / items_per_head, item = rem % items_per_head;
    const uint16_t *row = r.inout + (static_cast<uint64_t>(t) * (r.n_heads + 2 * r.n_kv_heads) + hs) * r.head_dim;
    // the token's position and slot are requested together with its row (every thread loads both: under a
    // condition each would be a trip to memory of its own); only the cos / sin row waits for the position
    RopeItemRegs x;
    x.pos_t = r.position[t];
    x.slot = static_cast<uint32_t>(r.slot_mapping[t]);
    const uint32_t e_first = item < rot_pairs ? item * 8 : (item + rot_pairs) * 8;
    x.a.v = *reinterpret_cast<const uint4 *>(row + e_first);
    x.b.v = *reinterpret_cast<const uint4 *>(row + (item < rot_pairs ? e_first + r.rot_dim / 2 : e_first));
    return x;
}

template <typename T>
__device__ __forceinline__ void rope_item_finish(const RopeArgs &r, uint32_t t, uint32_t rem, const RopeItemRegs &x)
{
    uint16_t *const k_cache = r.k_cache, *const v_cache = r.v_cache;
    const uint32_t n_heads = r.n_heads, n_kv_heads = r.n_kv_heads, head_dim = r.head_dim, rot_dim = r.rot_dim,
                   block_size = r.block_size;
    const uint32_t rot_pairs = rot_dim / 16;
    const uint32_t items_per_head = head_dim / 8 - rot_pairs;
    const uint32_t half = rot_dim / 2;
    const uint32_t hs = rem / items_per_head;
    const uint32_t item = rem % items_per_head;
    uint16_t *row = r.inout + (static_cast<uint64_t>(t) * (n_heads + 2 * n_kv_heads) + hs) * head_dim;
    const bool is_q = hs < n_heads;
    const bool is_k = !is_q && hs < n_heads + n_kv_heads;
    Vec16 a = x.a, b = x.b;
    uint16_t *cache_row = nullptr;
    if (!is_q && k_cache != nullptr) {   // no 16-bit caches: the caller quantises the rows afterwards
        const uint32_t kvh = is_k ? hs - n_heads : hs - n_heads - n_kv_heads;
        const uint64_t off =
            ((static_cast<uint64_t>(x.slot / block_size) * block_size + x.slot % block_size) * n_kv_heads + kvh) * head_dim;
        cache_row = (is_k ? k_cache : v_cache) + off;
    }
    if (item < rot_pairs) {
        const uint32_t e0 = item * 8;  // first-half elements e0..e0+7, partners at +half
        if (is_q || is_k) {
            rotate_chunk_pair<T>(a, b, e0, half, t, x.pos_t, r.num_tokens, rot_dim, r.position, r.cosin, r.mask_h, r.mask_w, is_q,
                                 r.q_scale);
            *reinterpret_cast<uint4 *>(row + e0) = a.v;
            *reinterpret_cast<uint4 *>(row + e0 + half) = b.v;
        }
        if (cache_row) {
            *reinterpret_cast<uint4 *>(cache_row + e0) = a.v;
            *reinterpret_cast<uint4 *>(cache_row + e0 + half) = b.v;
        }
    } else {
        const uint32_t e0 = (item + rot_pairs) * 8;  // beyond the rotary span
        if (is_q) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                a.h[j] = T::from_f32(T::to_f32(a.h[j]) * r.q_scale);
            }
            *reinterpret_cast<uint4 *>(row + e0) = a.v;
        } else if (cache_row) {
            *reinterpret_cast<uint4 *>(cache_row + e0) = a.v;
        }
    }
}

template <typename T>
__device__ __forceinline__ void rope_item(const RopeArgs &r, uint32_t t, uint32_t rem)
{
    rope_item_finish<T>(r, t, rem, rope_item_load(r, t, rem));
}

}  // namespace xlite
